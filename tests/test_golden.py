"""The CPU oracle reproduces the committed golden fixture of the tiny configuration."""
import os

import numpy as np

from tests.golden import make_golden

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_moe.npz")


def test_oracle_reproduces_golden_fixture():
    gold = np.load(GOLDEN, allow_pickle=False)
    data, _ = make_golden.build()
    for k in ("x", "gate_weight", "indices", "counts", "offsets", "perm", "inv"):
        assert np.array_equal(gold[k], data[k]), k
    assert list(gold["expert_sha256"]) == list(data["expert_sha256"])
    np.testing.assert_allclose(gold["weights"], data["weights"], rtol=1e-6)
    # the fp32 matmuls may be blocked differently on another host: compare to fp32 accuracy
    np.testing.assert_allclose(gold["out"], data["out"], rtol=1e-4, atol=1e-5)
    assert gold["indices"].shape == (32, 2) and gold["counts"].sum() == 64
    # no renormalisation in this configuration: the two weights do not sum to one
    assert (gold["weights"].sum(-1) < 0.999).all()
