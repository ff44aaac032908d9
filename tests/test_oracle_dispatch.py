"""Pins the oracle's dispatch against the reference's per-expert torch.where order (CPU only)."""
import numpy as np
import torch
from hypothesis import given, settings, strategies as st

from oracle import moe_oracle as orc


def _reference_order(idx: np.ndarray, E: int):
    """qwen3_runner.py:303-314: per expert, mask = (topk_indices == e); torch.where(mask)."""
    t = torch.from_numpy(idx.astype(np.int64))
    pairs, counts = [], []
    K = idx.shape[1]
    for e in range(E):
        tok, k = torch.where(t == e)
        counts.append(len(tok))
        pairs += (tok * K + k).tolist()
    return np.array(counts, dtype=np.int32), np.array(pairs, dtype=np.int32)


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 40), st.integers(1, 6), st.integers(1, 20), st.integers(0, 2 ** 31 - 1))
def test_dispatch_properties(T, K, E, seed):
    rng = np.random.default_rng(seed)
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)     # duplicates inside a token allowed
    counts, offsets, perm, inv = orc.dispatch(idx, E)
    P = T * K
    assert counts.sum() == P and offsets[0] == 0 and offsets[-1] == P
    assert np.array_equal(offsets[1:] - offsets[:-1], counts)
    assert np.array_equal(np.sort(perm), np.arange(P))            # bijection
    assert np.array_equal(inv[perm], np.arange(P))
    assert np.array_equal(counts, np.bincount(idx.reshape(-1), minlength=E))
    c_ref, order_ref = _reference_order(idx, E)
    assert np.array_equal(counts, c_ref) and np.array_equal(inv, order_ref)
    # stable: inside one expert the pair ids ascend
    for e in range(E):
        seg = inv[offsets[e]:offsets[e + 1]]
        assert (np.diff(seg) > 0).all()
        assert (idx.reshape(-1)[seg] == e).all()


def test_dispatch_matches_stable_argsort_and_out_of_range():
    idx = np.array([[0, 0], [3, 9], [-1, 2], [2, 2]], dtype=np.int32)
    counts, offsets, perm, inv = orc.dispatch(idx, 4)
    assert counts.tolist() == [2, 0, 3, 1] and offsets.tolist() == [0, 2, 2, 5, 6]
    assert perm.tolist() == [0, 1, 5, -1, -1, 2, 3, 4]
    assert inv.tolist() == [0, 1, 5, 6, 7, 2, -1, -1]


def test_layer_activations_cover_every_pair_once():
    """Pins oracle.layer_activations against a brute-force one-hot expansion: the (rank, expert,
    token) triples are exactly the nonzeros of onehot[t, k, e], ordered by rank then expert with
    ascending tokens, and the weights are those of the pair."""
    rng = np.random.default_rng(5)
    T, K, E = 23, 3, 7
    idx = rng.integers(0, E, size=(T, K))
    w = rng.random((T, K)).astype(np.float32)
    acts = orc.layer_activations(idx, w, E)
    onehot = np.zeros((T, K, E), dtype=bool)
    for t in range(T):
        for k in range(K):
            onehot[t, k, idx[t, k]] = True
    seen = np.zeros((T, K), dtype=int)
    last = (-1, -1)
    for k, e, tok, ww in acts:
        assert (k, e) > last
        last = (k, e)
        assert tok.size > 0 and np.all(np.diff(tok) > 0)
        assert np.array_equal(tok, np.nonzero(onehot[:, k, e])[0])
        assert np.array_equal(ww, w[tok, k])
        seen[tok, k] += 1
    assert np.all(seen == 1)
