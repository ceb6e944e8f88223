"""Pins oracle.index_build without retyping it: explicit loops, numpy.nonzero,
and the permutation invariants the reference guarantees."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

import oracle
from helpers import make_routing


def _check_invariants(mask, out, K=None):
    N, M = mask.shape
    sizes, cums, idx, which = out["sizes_N"], out["cumsums_N"], out["idx_Msum"], out["which_Msum"]
    assert sizes.dtype == np.int64 and cums.dtype == np.int32
    assert idx.dtype == np.int32 and which.dtype == np.int32
    assert cums[0] == 0 and cums[-1] == (mask != 0).sum()
    assert np.array_equal(np.diff(cums.astype(np.int64)), sizes)
    for i in range(N):
        rows = idx[cums[i]:cums[i + 1]]
        assert np.array_equal(rows, np.nonzero(mask[i])[0])  # ascending token ids of expert i
    # slots of each token are a permutation of 0..count-1
    for m in range(M):
        w = np.sort(which[idx == m])
        assert np.array_equal(w, np.arange(w.shape[0]))
    if K is not None:
        assert cums[-1] == M * K


@given(st.integers(1, 9), st.integers(1, 40), st.integers(0, 2 ** 31 - 1))
@settings(max_examples=60, deadline=None)
def test_matches_bruteforce_random_masks(N, M, seed):
    rng = np.random.default_rng(seed)
    mask = (rng.random((N, M)) < 0.4).astype(np.int32)
    a = oracle.index_build(mask)
    b = oracle.index_build_bruteforce(mask)
    for k in ("sizes_N", "cumsums_N", "idx_Msum", "which_Msum", "expert_of_row"):
        assert np.array_equal(a[k], b[k]), k
        assert a[k].dtype == b[k].dtype, k
    _check_invariants(mask, a)


@pytest.mark.parametrize("M,N,K,Ks", [(128, 8, 2, 0), (96, 12, 4, 2), (1, 4, 4, 0), (33, 5, 1, 0)])
def test_exactly_k_routing(M, N, K, Ks):
    mask, _ = make_routing(M, N, K, Ks, seed=3)
    out = oracle.index_build(mask)
    _check_invariants(mask.numpy(), out, K=K)
    inv = out["inv_MK"]
    assert inv.shape == (M, K)
    # inverse map: row inv[m,k] belongs to token m with slot k
    assert np.array_equal(out["idx_Msum"][inv], np.repeat(np.arange(M)[:, None], K, 1))
    assert np.array_equal(out["which_Msum"][inv], np.repeat(np.arange(K)[None, :], M, 0))


def test_hand_computed_case():
    mask = np.array([[1, 0, 1, 0],
                     [0, 1, 1, 0],
                     [0, 0, 0, 0],
                     [1, 1, 0, 0]], dtype=np.int32)
    out = oracle.index_build(mask)
    assert out["sizes_N"].tolist() == [2, 2, 0, 2]
    assert out["cumsums_N"].tolist() == [0, 2, 4, 4, 6]
    assert out["idx_Msum"].tolist() == [0, 2, 1, 2, 0, 1]
    assert out["which_Msum"].tolist() == [0, 0, 0, 1, 1, 1]


def test_empty_and_full():
    out = oracle.index_build(np.zeros((3, 5), dtype=np.int32))
    assert out["sizes_N"].tolist() == [0, 0, 0] and out["idx_Msum"].shape == (0,)
    out = oracle.index_build(np.ones((3, 5), dtype=np.int32))
    assert out["idx_Msum"].tolist() == [0, 1, 2, 3, 4] * 3
    assert out["which_Msum"].tolist() == [0] * 5 + [1] * 5 + [2] * 5


def test_strided_mask_view():
    mask, _ = make_routing(64, 8, 2, seed=5)
    t = mask.T.contiguous().T  # same values, strides (1, N)
    a, b = oracle.index_build(mask), oracle.index_build(t)
    for k in a:
        assert np.array_equal(a[k], b[k])
