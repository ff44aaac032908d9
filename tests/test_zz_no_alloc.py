"""odsd_moe_forward_static (the whole block on the library's own static scratch array, no
allocation anywhere in the call) against odsd_moe_forward on a caller-provided workspace: same
kernels, so every output must be bit-identical.  Two calls in a row share the array; the second is
smaller, so it runs over what the first one left behind."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _layer(dev, T, H, E, K, I, seed):
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(seed)
    gate = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    bank = odsd.W4ExpertBank(E, H, I, dev)
    for e in range(E):
        bank.load_expert(e, torch.randn(I, H, generator=g) * 0.02, torch.randn(I, H, generator=g) * 0.02,
                         torch.randn(H, I, generator=g) * 0.02)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    norm = (1 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16).to(dev)
    return gate, bank, x, norm


def _run(lib, static, shape, x, norm, gate, table, dev):
    from on_device_sd_amd import _lib
    T, H, E, K = shape.T, shape.H, shape.E, shape.K
    o = dict(out_f32=torch.full((T, H), float("nan"), dtype=torch.float32, device=dev),
             out_act=torch.zeros(T, H, dtype=torch.bfloat16, device=dev),
             idx=torch.full((T, K), -7, dtype=torch.int32, device=dev),
             w=torch.zeros(T, K, dtype=torch.float32, device=dev),
             counts=torch.full((E,), -7, dtype=torch.int32, device=dev),
             offsets=torch.full((E + 1,), -7, dtype=torch.int32, device=dev),
             perm=torch.full((T * K,), -7, dtype=torch.int32, device=dev))
    st = torch.cuda.current_stream().cuda_stream
    head = (C.byref(shape), x.data_ptr(), norm.data_ptr(), 1e-6, gate.data_ptr(), table.data_ptr(), 1,
            o["out_f32"].data_ptr(), o["out_act"].data_ptr(), o["idx"].data_ptr(), o["w"].data_ptr(),
            o["counts"].data_ptr(), o["offsets"].data_ptr(), o["perm"].data_ptr(), None, None)
    if static:
        _lib.check(lib.odsd_moe_forward_static(*head, st), "odsd_moe_forward_static")
    else:
        need = lib.odsd_moe_workspace_bytes(C.byref(shape))
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        _lib.check(lib.odsd_moe_forward(*head, ws.data_ptr(), need, st), "odsd_moe_forward")
    torch.cuda.synchronize()
    return o


def test_static_scratch_matches_workspace_call(dev):
    from on_device_sd_amd import _lib
    lib = _lib.load()
    H, E, K, I = 512, 16, 4, 512
    for T, seed in ((96, 11), (20, 12)):          # the second call is the smaller one
        print("no-alloc entry point: T", T, flush=True)
        gate, bank, x, norm = _layer(dev, T, H, E, K, I, seed)
        shape = _lib.MoeShape(T, H, E, K, I, 1, _lib.DT_BF16, 0)
        assert lib.odsd_moe_workspace_bytes(C.byref(shape)) <= _lib.STATIC_SCRATCH_BYTES
        got = _run(lib, True, shape, x, norm, gate, bank.table(), dev)
        ref = _run(lib, False, shape, x, norm, gate, bank.table(), dev)
        for name in ref:
            assert torch.equal(got[name].view(torch.uint8), ref[name].view(torch.uint8)), \
                f"T={T}: {name} differs between the static-scratch call and the workspace call"
        assert int(ref["counts"].sum()) == T * K and torch.isfinite(ref["out_f32"]).all()


def test_static_scratch_call_at_the_one_launch_shape(dev):
    """The Qwen3-30B-A3B layer shape (one-launch expert kernel with the dispatch inside, 29 MiB of
    workspace) through the static array, then a smaller call over what it left behind."""
    from on_device_sd_amd import _lib
    lib = _lib.load()
    H, E, K, I = 2048, 128, 8, 768
    gate, bank, x, norm = _layer(dev, 256, H, E, K, I, 31)
    for T in (256, 136):
        print("no-alloc entry point, one-launch shape: T", T, flush=True)
        shape = _lib.MoeShape(T, H, E, K, I, 1, _lib.DT_BF16, 0)
        assert lib.odsd_experts_one_launch(C.byref(shape)) == 1
        assert lib.odsd_moe_workspace_bytes(C.byref(shape)) <= _lib.STATIC_SCRATCH_BYTES
        xt = x[:T].contiguous()
        got = _run(lib, True, shape, xt, norm, gate, bank.table(), dev)
        ref = _run(lib, False, shape, xt, norm, gate, bank.table(), dev)
        for name in ref:
            assert torch.equal(got[name].view(torch.uint8), ref[name].view(torch.uint8)), \
                f"T={T}: {name} differs between the static-scratch call and the workspace call"
        assert int(ref["counts"].sum()) == T * K and torch.isfinite(ref["out_f32"]).all()


def test_static_scratch_call_under_graph_capture(dev):
    """The use the entry point is offered for: after odsd_moe_static_init() the call is captured into
    a HIP graph (nothing may allocate or query the runtime there) and replayed several times, with
    eager work and synchronisations of the program's own between the replays; every replay must give
    the bits of the eager workspace call."""
    from on_device_sd_amd import _lib
    lib = _lib.load()
    T, H, E, K, I = 48, 512, 16, 4, 512
    print("no-alloc entry point under graph capture: T", T, flush=True)
    gate, bank, x, norm = _layer(dev, T, H, E, K, I, 21)
    table = bank.table()
    shape = _lib.MoeShape(T, H, E, K, I, 1, _lib.DT_BF16, 0)
    _lib.check(lib.odsd_moe_static_init(), "odsd_moe_static_init")
    ref = _run(lib, False, shape, x, norm, gate, table, dev)
    out_f32 = torch.zeros(T, H, dtype=torch.float32, device=dev)
    out_act = torch.zeros(T, H, dtype=torch.bfloat16, device=dev)
    idx = torch.zeros(T, K, dtype=torch.int32, device=dev)
    x_in = x.clone()

    def call():
        _lib.check(lib.odsd_moe_forward_static(
            C.byref(shape), x_in.data_ptr(), norm.data_ptr(), 1e-6, gate.data_ptr(), table.data_ptr(), 1,
            out_f32.data_ptr(), out_act.data_ptr(), idx.data_ptr(), None, None, None, None, None, None,
            torch.cuda.current_stream().cuda_stream), "odsd_moe_forward_static")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()                                   # warm-up on the capture stream, outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    # (a device allocation or a symbol look-up inside the capture would invalidate it and fail here;
    # torch's own allocator cannot be used as a witness: beginning a capture allocates its RNG state)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(4):
        out_f32.fill_(float("nan")); out_act.zero_(); idx.fill_(-1)
        if rep == 2:                             # other inputs through the same graph, then the first ones again
            x_in.copy_(torch.flip(x, dims=[0]))
        elif rep == 3:
            x_in.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        if rep == 2:
            assert torch.equal(idx, torch.flip(ref["idx"], dims=[0]))
            continue
        for name, got in (("out_f32", out_f32), ("out_act", out_act), ("idx", idx)):
            assert torch.equal(got.view(torch.uint8), ref[name].view(torch.uint8)), f"replay {rep}: {name} differs"
        # eager work of the program's own on the shared scratch between the replays
        _run(lib, True, _lib.MoeShape(20, H, E, K, I, 1, _lib.DT_BF16, 0), x[:20].contiguous(), norm, gate, table, dev)
