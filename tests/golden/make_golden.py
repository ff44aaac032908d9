#!/usr/bin/env python3
"""Writes tests/golden/tiny_moe.npz: inputs and expected results of the tiny configuration
(T=32, H=512, E=8, top-2 softmax routing without renormalisation, I=1024, fp32 activations,
seed 0), computed by the CPU oracle.  Expert weights are not stored (25 MB); the fixture
holds the SHA-256 of every expert's canonical W4 arrays instead, which a run regenerates
from the seed and checks.

Usage:  python tests/golden/make_golden.py
"""
import hashlib
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from on_device_sd_amd.workloads import CONFIGS, LayerInputs   # noqa: E402
from oracle import moe_oracle as orc                            # noqa: E402


def expert_digest(ex: orc.W4Expert) -> str:
    h = hashlib.sha256()
    for q, s, z in (ex.gate, ex.up, ex.down):
        h.update(np.ascontiguousarray(q).tobytes())
        h.update(np.ascontiguousarray(s).tobytes())
        h.update(np.ascontiguousarray(z).tobytes())
    return h.hexdigest()


def build():
    wl = CONFIGS["tiny"]
    inp = LayerInputs(wl, "cpu")
    gate = inp.gate_weight()
    experts = {e: orc.quantize_expert(g.numpy(), u.numpy(), d.numpy()) for e, g, u, d in inp.experts()}
    x = inp.x()
    logits = orc.router_logits(x, gate)
    idx, w = orc.route(logits, wl.K, wl.renorm)
    counts, offsets, perm, inv = orc.dispatch(idx, wl.E)
    out = orc.moe_forward(x, idx, w, experts)
    return dict(x=x.numpy(), gate_weight=gate.numpy(), indices=idx, weights=w, counts=counts,
                offsets=offsets, perm=perm, inv=inv, out=out.numpy(),
                expert_sha256=np.array([expert_digest(experts[e]) for e in range(wl.E)])), experts


if __name__ == "__main__":
    data, _ = build()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tiny_moe.npz")
    np.savez_compressed(path, **data)
    print("wrote", path, os.path.getsize(path), "bytes")
