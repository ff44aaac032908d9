"""Phase time-line of the one-launch expert kernel (`python -m on_device_sd_amd.timeline [T] [zipf_s]`).

Needs the timing-only build of the library (`make -C on_device_sd_amd/csrc timeline`), in which every
wavefront of `w4_expert_fused_kernel` stamps the GPU's 100 MHz real-time counter at eight points.  One
Qwen3-30B-A3B layer (H = 2048, E = 128, K = 8, I = 768) is run through the whole-block call on rotating
weight replicas, and the stamps of the 256 x 8 wavefronts are summarised relative to the launch's
first stamp.  A diagnostic, not part of the product path: the product library has no stamps.
"""
from __future__ import annotations

import ctypes as C
import os
import sys


def main(argv) -> int:
    import numpy as np
    import torch
    from . import _lib
    tl_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libodsd_moe_timeline.so")
    if not os.path.exists(tl_path):
        raise SystemExit(f"{tl_path} is missing: build it with `make -C on_device_sd_amd/csrc timeline`")
    _lib.LIB_PATH = tl_path                    # before the first load(): the whole package then runs on this build
    from . import W4ExpertBank, ops
    from .workloads import LayerInputs, MoEWorkload
    T = int(argv[0]) if argv else 256
    zipf = float(argv[1]) if len(argv) > 1 else None
    dev = torch.device("cuda:0")
    wl = MoEWorkload("stack_layer", T=T, H=2048, E=128, K=8, I=768, renorm=True, act_dtype=torch.bfloat16,
                     zipf_s=zipf)
    inp = LayerInputs(wl, dev, 0)
    gate = inp.gate_weight()
    bank = W4ExpertBank(wl.E, wl.H, wl.I, dev)
    for e, gw, uw, dw in inp.experts():
        bank.load_expert(e, gw, uw, dw)
    x = inp.x()
    banks = [bank] + [bank.clone() for _ in range(3)]
    tables = [b.table() for b in banks]
    plan = ops.MoeForwardPlan(wl.T, wl.H, wl.E, wl.K, wl.I, wl.renorm, wl.act_dtype, dev)
    lib = _lib.load()
    lib.odsd_debug_timeline.restype = C.c_int
    lib.odsd_debug_timeline.argtypes = [C.c_void_p]
    n_wg, waves = 2 * wl.E, 8
    buf = torch.zeros(n_wg * waves * 8, dtype=torch.int64, device=dev)
    if lib.odsd_debug_timeline(buf.data_ptr()) != 0:
        raise SystemExit("odsd_debug_timeline failed")
    names = ["own id scan done", "token rows in LDS", "x group sums done", "gate_up stream done", "h complete (barrier)",
             "h group sums done", "end (after overflow units)"]
    runs = []
    for it in range(12):
        plan.run(x, gate, tables[it % 4])
        torch.cuda.synchronize()
        if it < 4:
            continue
        t = buf.cpu().numpy().reshape(n_wg, waves, 8).astype(np.float64) * 0.01      # microseconds
        runs.append(t - t[:, :, 0].min())
    a = np.stack(runs)                          # [launch, workgroup, wavefront, stamp]
    counts = plan.counts.cpu().numpy()
    print(f"w4_expert_fused_kernel, T={T}, zipf_s={zipf}: rows per expert mean {counts.mean():.1f} max {counts.max()}, "
          f"experts beyond one 32-row pass: {(counts > 32).sum()}")
    print(f"microseconds from the launch's first stamp; mean over {a.shape[0]} launches of the "
          f"(min / mean / max) over the {n_wg * waves} wavefronts")
    print(f"  {'start':28s} {a[..., 0].min(axis=(1, 2)).mean():7.2f} {a[..., 0].mean():7.2f} {a[..., 0].max(axis=(1, 2)).mean():7.2f}")
    for k, nm in enumerate(names, start=1):
        v = a[..., k]
        print(f"  {nm:28s} {v.min(axis=(1, 2)).mean():7.2f} {v.mean():7.2f} {v.max(axis=(1, 2)).mean():7.2f}")
    d = np.diff(a, axis=-1)
    print("phase durations per wavefront (mean / mean of the launch's longest):")
    for k, nm in enumerate(names):
        print(f"  -> {nm:28s} {d[..., k].mean():7.2f} {d[..., k].max(axis=(1, 2)).mean():7.2f}")
    end = a[..., 7].max(axis=2).mean(axis=0)
    print("workgroup end times: min %.2f p10 %.2f median %.2f p90 %.2f max %.2f"
          % (end.min(), np.percentile(end, 10), np.median(end), np.percentile(end, 90), end.max()))
    rows = np.repeat(counts, 2)
    light, heavy = end[(rows > 0) & (rows <= 16)], end[rows > 16]
    if len(light) and len(heavy):
        print("  workgroups with 1..16 rows end at %.2f on average, with 17 or more at %.2f" % (light.mean(), heavy.mean()))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
