"""The C-ABI library loads without a GPU, exports every function the header declares, and
rejects bad arguments with status codes before touching the device (CPU only)."""
import ctypes as C
import os
import re

from on_device_sd_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "odsd_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(odsd_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 18
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_version_and_status_strings():
    lib = _lib.load()
    assert lib.odsd_version() == 115
    assert lib.odsd_status_string(0) == b"ok"
    for code in range(1, 9):
        assert len(lib.odsd_status_string(code)) > 3


def test_one_launch_plan_follows_shape_and_max_rows():
    """The whole-block experts calls take the one-launch kernel at the Qwen3-30B expert shape with
    8 to 20 rows per expert on average, unless the caller says that some expert has more rows than
    one pass of that kernel holds (the counts the reference engine reads on the host between
    route_experts and forward_moe, qwen3_runner.py:110-112)."""
    lib = _lib.load()
    q = lambda T, mr: lib.odsd_experts_one_launch(C.byref(_lib.MoeShape(T, 2048, 128, 8, 768, 1, _lib.DT_BF16, mr)))
    assert q(256, 0) == 1 and q(128, 0) == 1 and q(320, 0) == 1
    assert q(256, 32) == 1 and q(256, 33) == 0 and q(256, 70) == 0
    assert q(64, 0) == 0 and q(384, 0) == 0 and q(4096, 0) == 0          # too few / too many rows per expert
    assert lib.odsd_experts_one_launch(C.byref(_lib.MoeShape(160, 4096, 8, 2, 14336, 0, _lib.DT_BF16, 0))) == 0
    assert lib.odsd_experts_one_launch(C.byref(_lib.MoeShape(160, 4000, 8, 2, 14336, 0, _lib.DT_BF16, 0))) == -2
    # the workspace answer does not depend on the statement (one buffer serves either plan)
    ws = lambda mr: lib.odsd_experts_workspace_bytes(C.byref(_lib.MoeShape(256, 2048, 128, 8, 768, 1, _lib.DT_BF16, mr)))
    assert ws(0) == ws(40) > 0


def test_argument_checks_need_no_gpu():
    lib = _lib.load()
    ok = _lib.MoeShape(8, 256, 8, 2, 256, 1, _lib.DT_BF16, 0)
    assert lib.odsd_moe_workspace_bytes(C.byref(ok)) > 0
    assert lib.odsd_router_workspace_bytes(C.byref(ok)) > 0
    assert lib.odsd_experts_workspace_bytes(C.byref(ok)) > 0
    assert lib.odsd_w4_down_splits(C.byref(ok)) >= 1
    bad_h = _lib.MoeShape(8, 200, 8, 2, 256, 1, _lib.DT_BF16, 0)      # H % 128 != 0
    assert lib.odsd_moe_workspace_bytes(C.byref(bad_h)) == 0
    # shapes whose row offsets do not fit the kernels' 32-bit byte offsets are refused up front
    huge = _lib.MoeShape(70000, 4096, 8, 8, 4096, 1, _lib.DT_BF16, 0)   # P * I * 2 >= 2^32
    assert lib.odsd_experts_workspace_bytes(C.byref(huge)) == 0 and lib.odsd_moe_workspace_bytes(C.byref(huge)) == 0
    assert lib.odsd_w4_gate_up_silu(C.byref(huge), 1 << 20, 1 << 20, 1 << 20, 1 << 20, 1 << 20, 1 << 20, None) == 3
    long_t = _lib.MoeShape(100000, 1024, 8, 2, 512, 1, _lib.DT_BF16, 0)  # more than 65535 tokens is fine
    assert lib.odsd_experts_workspace_bytes(C.byref(long_t)) > 0
    big_e = _lib.MoeShape(8, 256, 1024, 2, 256, 1, _lib.DT_BF16, 0)   # E > 512
    assert lib.odsd_router_workspace_bytes(C.byref(big_e)) == 0
    k_gt_e = _lib.MoeShape(8, 256, 4, 8, 256, 1, _lib.DT_BF16, 0)
    assert lib.odsd_router_workspace_bytes(C.byref(k_gt_e)) == 0
    # NULL pointers and bad shapes come back as status codes, nothing is launched
    assert lib.odsd_w4_quantize(None, 0, 16, 128, None, None, None, None) == 1
    assert lib.odsd_w4_quantize(1 << 20, 0, 16, 100, 1 << 20, 1 << 20, 1 << 20, None) == 2
    assert lib.odsd_w4_quantize(1 << 20, 9, 16, 128, 1 << 20, 1 << 20, 1 << 20, None) == 7
    assert lib.odsd_w4_pack(None, None, None, 16, 128, 1, 0, None, None, None) == 1
    assert lib.odsd_w4_pack(1 << 20, 1 << 20, 1 << 20, 10, 128, 1, 0, 1 << 20, 1 << 20, None) == 2
    assert lib.odsd_rmsnorm(None, None, 1, 4, 128, 1e-6, None, None) == 1
    assert lib.odsd_add_rmsnorm(None, None, None, 1, 4, 128, 1e-6, None, None, None) == 1
    assert lib.odsd_add_rmsnorm(1 << 20, 1 << 20, 1 << 20, 7, 4, 128, 1e-6, 1 << 20, 1 << 20, None) == 7
    assert lib.odsd_router_topk(C.byref(ok), None, None, None, None, None, None, None, 0, None) == 1
    # the combined call needs all five dispatch arrays
    assert lib.odsd_route_dispatch(C.byref(ok), 1 << 20, 1 << 20, 1 << 20, 1 << 20, None, None, 1 << 20, None,
                                   1 << 20, 1 << 20, 1 << 20, 1 << 20, 1 << 30, None) == 1
    # the logits form needs its extra output
    assert lib.odsd_router_topk_logits(C.byref(ok), 1 << 20, 1 << 20, 1 << 20, 1 << 20, None, None, None,
                                       1 << 20, 1 << 30, None) == 1
    assert lib.odsd_router_topk(C.byref(ok), 1 << 20, 1 << 20, 1 << 20, 1 << 20, None, None, 1 << 20, 16, None) == 5
    assert lib.odsd_router_topk(C.byref(ok), (1 << 20) + 4, 1 << 20, 1 << 20, 1 << 20, None, None, 1 << 20, 1 << 30, None) == 4
    assert lib.odsd_dispatch(C.byref(ok), None, None, None, None, None, None, None) == 1
    assert lib.odsd_moe_forward(C.byref(bad_h), None, None, 1e-6, None, None, 0, None, None, None, None, None,
                                None, None, None, None, None, 0, None) == 2
    assert lib.odsd_moe_forward(C.byref(ok), 1 << 20, None, 1e-6, 1 << 20, 1 << 20, 0, None, None, None, None,
                                None, None, None, None, None, 1 << 20, 16, None) == 5
    assert lib.odsd_w4_packed_q_bytes(32, 256) == 32 * 256 // 2
    assert lib.odsd_w4_packed_sz_bytes(32, 256) == 32 * 2 * 4
    assert lib.odsd_w4_packed_q_bytes(30, 256) == 0
    # KV store: argument checks
    assert lib.odsd_kv_store(None, None, 64, 64, None, None, None, None, 4, 4, 64, 2, 16, None) == 1
    assert lib.odsd_kv_store(1 << 20, 1 << 20, 32, 64, 1 << 20, 1 << 20, 1 << 20, None, 4, 4, 64, 2, 16, None) == 2
    assert lib.odsd_kv_store(1 << 20, 1 << 20, 64, 64, 1 << 20, 1 << 20, 1 << 20, None, 4, 4, 64, 3, 16, None) == 7
    assert lib.odsd_kv_store(None, None, 64, 64, None, None, None, None, 0, 0, 64, 2, 16, None) == 0
    # paged attention: argument checks (q, k, v, tables, lens, q_lens, n_seqs, max_q_len, H, KVH, HD, block,
    # max_blocks, num_slots, scale, dtype, out, workspace, workspace_bytes, stream)
    P = 1 << 20
    att = lambda *a: lib.odsd_paged_attention(*a)
    assert att(P, P, P, P, P, None, 2, 8, 32, 4, 128, 256, 16, 8192, 0.1, _lib.DT_BF16, None, None, 0, None) == 1
    assert att(P, P, P, P, P, None, 2, 8, 32, 5, 128, 256, 16, 8192, 0.1, _lib.DT_BF16, P, None, 0, None) == 2
    assert att(P, P, P, P, P, None, 2, 8, 32, 4, 96, 256, 16, 8192, 0.1, _lib.DT_BF16, P, None, 0, None) == 3
    assert att(P, P, P, P, P, None, 2, 8, 32, 4, 128, 256, 16, 8192, 0.1, 9, P, None, 0, None) == 7
    assert att(None, None, None, None, None, None, 0, 8, 32, 4, 128, 256, 16, 8192, 0.1, _lib.DT_BF16, None, None, 0, None) == 0
    # few sequences with long tables share a sequence's keys between workgroups: workspace required
    need = lib.odsd_paged_attention_workspace_bytes(2, 8, 32, 4, 128, 256, 16)
    assert need > 256 and need % 256 == 0
    assert att(P, P, P, P, P, None, 2, 8, 32, 4, 128, 256, 16, 8192, 0.1, _lib.DT_BF16, P, None, 0, None) == 1
    assert att(P, P, P, P, P, None, 2, 8, 32, 4, 128, 256, 16, 8192, 0.1, _lib.DT_BF16, P, P, need - 1, None) == 5
    assert lib.odsd_paged_attention_workspace_bytes(2, 8, 32, 4, 96, 256, 16) == 0
    # more query rows per (sequence, KV head) than the launch grid holds: refused, not truncated
    assert att(P, P, P, P, P, None, 1, 600000, 32, 4, 128, 256, 16, 8192, 0.1, _lib.DT_BF16, P, P, 1 << 30, None) == 3
    assert lib.odsd_paged_attention_workspace_bytes(1, 600000, 32, 4, 128, 256, 16) == 0
    # many sequences: one workgroup per (sequence, KV head) walks all its keys, no partial results
    assert lib.odsd_paged_attention_workspace_bytes(512, 1, 32, 4, 128, 256, 16) == 256
    # variable-length (prefill) attention: q, k, v, cu_q, cu_k, n_seqs, max_q, max_k, H, KVH, HD, scale, dtype,
    # out, workspace, workspace_bytes, stream
    var = lambda *a: lib.odsd_varlen_attention(*a)
    assert var(P, P, P, P, P, 2, 64, 64, 32, 4, 128, 0.1, _lib.DT_BF16, None, None, 0, None) == 1
    assert var(P, P, P, P, P, 2, 64, 64, 32, 4, 128, 0.0, _lib.DT_BF16, P, None, 0, None) == 2
    assert var(P, P, P, P, P, 2, 64, 64, 32, 4, 80, 0.1, _lib.DT_BF16, P, None, 0, None) == 3
    assert var(P, P, P, P, P, 2, 64, 64, 32, 4, 128, 0.1, _lib.DT_F32, P, None, 0, None) == 7
    assert var(None, None, None, None, None, 0, 64, 64, 32, 4, 128, 0.1, _lib.DT_BF16, None, None, 0, None) == 0
    assert lib.odsd_varlen_attention_workspace_bytes(2, 64, 64, 32, 4, 128) == 256       # short: no key slicing
    assert lib.odsd_varlen_attention_workspace_bytes(1, 8, 8192, 32, 4, 128) > 256
    empty = _lib.MoeShape(0, 256, 8, 2, 256, 1, _lib.DT_BF16, 0)       # T == 0 is a no-op
    assert lib.odsd_dispatch(C.byref(empty), 1 << 20, 1 << 20, 1 << 20, 1 << 20, 1 << 20, 1 << 20, None) == 0


def test_static_scratch_call_refuses_what_does_not_fit():
    """odsd_moe_forward_static returns ODSD_ERR_SCRATCH, before touching the device, for a shape
    whose workspace is larger than the library's static array."""
    lib = _lib.load()
    big = _lib.MoeShape(4096, 4096, 128, 8, 1536, 1, _lib.DT_BF16, 0)
    assert lib.odsd_moe_workspace_bytes(C.byref(big)) > _lib.STATIC_SCRATCH_BYTES
    rc = lib.odsd_moe_forward_static(C.byref(big), 1 << 20, None, 1e-6, 1 << 20, 1 << 20, 0, 1 << 20, None,
                                     None, None, None, None, None, None, None, None)
    assert rc == 8
    assert b"scratch" in lib.odsd_status_string(rc)
    # the header's constant and the binding's agree
    text = open(os.path.join(ROOT, "include", "odsd_moe.h")).read()
    m = re.search(r"#define ODSD_STATIC_SCRATCH_BYTES \((\d+)u << (\d+)\)", text)
    assert m and int(m.group(1)) << int(m.group(2)) == _lib.STATIC_SCRATCH_BYTES
    # the events form needs its event array
    ok = _lib.MoeShape(8, 256, 8, 2, 256, 1, _lib.DT_BF16, 0)
    assert lib.odsd_moe_forward_events(C.byref(ok), 1 << 20, None, 1e-6, 1 << 20, 1 << 20, 0, 1 << 20, None,
                                       None, None, 1 << 20, 1 << 30, None, None, None) == 1
