"""Pins the CPU oracle (oracle/) before anything is compared with it.

Nothing here retypes the oracle's own formulas: the dense formulation is checked against torch's
library SDPA in float64, scipy's logsumexp/softmax, closed forms and the golden vectors (written
by torch); the two independent transcriptions of every mask (dense loops of verify.py vs per-row
kernel bounds) are checked against each other by brute force; the C restatement is checked
against the numpy one.
"""
import math

import numpy as np
import pytest
import scipy.special
import torch

from oracle import c_oracle
from oracle import spfa_oracle as so


def _rand(n, d, seed, n_k=None):
    rng = np.random.default_rng(seed)
    n_k = n if n_k is None else n_k
    return rng.standard_normal((n, d)), rng.standard_normal((n_k, d)), rng.standard_normal((n_k, d))


def _torch_sdpa(q, k, v, mask):
    out = torch.nn.functional.scaled_dot_product_attention(
        torch.tensor(q), torch.tensor(k), torch.tensor(v), attn_mask=torch.tensor(mask)).numpy()
    out[~mask.any(axis=1)] = np.nan
    return out


# ---------------------------------------------------------------- dense formulation
@pytest.mark.parametrize("seed,density", [(0, 0.05), (1, 0.3), (2, 1.0)])
def test_dense_matches_torch_sdpa_fp64(seed, density):
    n, d = 80, 16
    q, k, v = _rand(n, d, seed)
    rng = np.random.default_rng(100 + seed)
    mask = rng.random((n, n)) < density
    mask[7, :] = False  # a dead row
    out, m, l = so.dense_masked_attention(q, k, v, mask)
    ref = _torch_sdpa(q, k, v, mask)
    assert np.array_equal(np.isnan(out), np.isnan(ref))
    np.testing.assert_allclose(np.nan_to_num(out), np.nan_to_num(ref), rtol=0, atol=1e-13)


def test_dense_statistics_are_max_and_logsumexp():
    n, d = 50, 8
    q, k, v = _rand(n, d, 3)
    mask = np.random.default_rng(4).random((n, n)) < 0.2
    mask[np.arange(n), np.arange(n)] = True
    out, m, l = so.dense_masked_attention(q, k, v, mask)
    s = np.where(mask, q @ k.T / math.sqrt(d), -np.inf)
    np.testing.assert_allclose(m, s.max(axis=1), atol=0)
    np.testing.assert_allclose(m + np.log(l), scipy.special.logsumexp(s, axis=1), atol=1e-13)
    np.testing.assert_allclose(out, scipy.special.softmax(s, axis=1) @ v, atol=1e-13)


def test_dense_closed_forms():
    n, d = 40, 8
    q, k, v = _rand(n, d, 5)
    # identity mask: softmax of one element is 1 -> out == v (verify.py:158-177)
    out, m, l = so.dense_masked_attention(q, k, v, np.eye(n, dtype=bool))
    np.testing.assert_allclose(out, v, atol=0)
    np.testing.assert_allclose(l, 1.0, atol=0)
    # V == 1 -> every live row is exactly a convex combination of ones
    mask = np.random.default_rng(6).random((n, n)) < 0.3
    mask[:, 0] = True
    out, _, _ = so.dense_masked_attention(q, k, np.ones((n, d)), mask)
    np.testing.assert_allclose(out, 1.0, atol=1e-14)
    # q == 0 -> uniform weights -> out = mean of the live V rows
    out, _, _ = so.dense_masked_attention(np.zeros((n, d)), k, v, mask)
    expect = np.stack([v[mask[i]].mean(axis=0) for i in range(n)])
    np.testing.assert_allclose(out, expect, atol=1e-13)


# ---------------------------------------------------------------- gradients of the dense formulation
@pytest.mark.parametrize("seed,density", [(0, 0.1), (1, 0.5), (2, 1.0)])
def test_backward_matches_torch_autograd_fp64(seed, density):
    """Library autograd through the library's SDPA, float64, rows without a live column left out
    of the loss (torch gives NaN gradients there; the oracle gives them none)."""
    n, n_k, d = 48, 40, 16
    q, k, v = _rand(n, d, seed, n_k)
    rng = np.random.default_rng(200 + seed)
    mask = rng.random((n, n_k)) < density
    mask[5, :] = False
    mask[6, :] = False
    mask[6, 3] = True  # a single live column
    d_out = rng.standard_normal((n, d))
    tq, tk, tv = (torch.tensor(x, requires_grad=True) for x in (q, k, v))
    live = torch.tensor(mask.any(axis=1))
    out = torch.nn.functional.scaled_dot_product_attention(tq[live], tk, tv,
                                                           attn_mask=torch.tensor(mask)[live])
    (out * torch.tensor(d_out)[live]).sum().backward()
    d_q, d_k, d_v = so.dense_masked_attention_backward(q, k, v, mask, d_out)
    np.testing.assert_allclose(d_q, tq.grad.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(d_k, tk.grad.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(d_v, tv.grad.numpy(), rtol=0, atol=1e-12)
    assert not d_q[5].any()  # dead row
    np.testing.assert_allclose(d_q[6], 0, atol=1e-13)  # one live column: the softmax is constant


def test_backward_matches_finite_differences_of_the_forward_oracle():
    n, d = 12, 4
    q, k, v = _rand(n, d, 9)
    rng = np.random.default_rng(10)
    mask = rng.random((n, n)) < 0.4
    mask[np.arange(n), np.arange(n)] = True
    d_out = rng.standard_normal((n, d))
    loss = lambda a, b, c: float((so.dense_masked_attention(a, b, c, mask)[0] * d_out).sum())
    grads = so.dense_masked_attention_backward(q, k, v, mask, d_out)
    eps = 1e-6
    for which, g in enumerate(grads):
        num = np.zeros_like(g)
        for i in range(n):
            for e in range(d):
                args = [q.copy(), k.copy(), v.copy()]
                args[which][i, e] += eps
                up = loss(*args)
                args[which][i, e] -= 2 * eps
                num[i, e] = (up - loss(*args)) / (2 * eps)
        np.testing.assert_allclose(g, num, rtol=0, atol=1e-7)


def test_backward_closed_forms():
    n, d = 30, 8
    q, k, v = _rand(n, d, 11)
    d_out = np.random.default_rng(12).standard_normal((n, d))
    # window 0: out == v, so dv == d_out and nothing flows to q or k
    d_q, d_k, d_v = so.dense_masked_attention_backward(q, k, v, np.eye(n, dtype=bool), d_out)
    np.testing.assert_allclose(d_q, 0, atol=1e-13)
    np.testing.assert_allclose(d_k, 0, atol=1e-13)
    np.testing.assert_allclose(d_v, d_out, atol=1e-15)
    # V == 1 on a full mask: out == 1 whatever q and k are, so dq == dk == 0 and dv sums d_out
    full = np.ones((n, n), dtype=bool)
    d_q, d_k, d_v = so.dense_masked_attention_backward(q, k, np.ones_like(v), full, d_out)
    np.testing.assert_allclose(d_q, 0, atol=1e-13)
    np.testing.assert_allclose(d_k, 0, atol=1e-13)
    np.testing.assert_allclose(d_v.sum(axis=0), d_out.sum(axis=0), atol=1e-12)


def test_rowwise_query_gradient_matches_the_dense_backward():
    n, n_k, d = 60, 45, 8
    q, k, v = _rand(n, d, 13, n_k)
    rng = np.random.default_rng(14)
    mask = rng.random((n, n_k)) < 0.3
    mask[2] = False
    d_out = rng.standard_normal((n, d))
    ro, ci = so.csr_from_dense(mask)
    ref = so.dense_masked_attention_backward(q, k, v, mask, d_out)[0]
    np.testing.assert_allclose(so.rowwise_query_gradient(q, k, v, d_out, ro, ci), ref, rtol=0, atol=1e-13)


def test_scale_rule_is_one_over_sqrt_d():
    # one query, two keys with a known score gap: weights must be sigmoid(gap / sqrt(d))
    d = 16
    q = np.zeros((1, d)); q[0, 0] = 4.0
    k = np.zeros((2, d)); k[0, 0] = 1.0; k[1, 0] = -1.0
    v = np.zeros((2, d)); v[0, 0] = 1.0
    out, m, l = so.dense_masked_attention(q, k, v, np.ones((1, 2), dtype=bool))
    gap = (4.0 - (-4.0)) / math.sqrt(d)
    assert abs(out[0, 0] - 1.0 / (1.0 + math.exp(-gap))) < 1e-15
    assert m[0] == 4.0 / math.sqrt(d)


# ---------------------------------------------------------------- golden vectors
def _lse(m, l):
    with np.errstate(divide="ignore"):
        return m + np.log(l)


@pytest.mark.parametrize("kind", ["csr", "local", "d1", "d2", "glob"])
def test_oracle_matches_golden(golden, kind):
    q, k, v = golden["q"], golden["k"], golden["v"]
    n = q.shape[0]
    if kind == "csr":
        mask = golden["csr_mask"]
        ro, ci = so.csr_from_dense(mask)
        c_out, c_m, c_l = c_oracle.csr(q, k, v, ro, ci, use_nan=True, chunk=7)
    elif kind == "local":
        w = int(golden["local_w"])
        mask = so.mask_local_dense(n, w)
        c_out, c_m, c_l = c_oracle.local(q, k, v, w, chunk=4)
    elif kind == "d1":
        w, dil = int(golden["d1_w"]), int(golden["d1_dil"])
        mask = so.mask_local_1d_dilated_dense(n, w, dil)
        c_out, c_m, c_l = c_oracle.local_1d_dilated(q, k, v, w, dil, chunk=3)
    elif kind == "d2":
        b, dil = int(golden["d2_block"]), int(golden["d2_dil"])
        mask = so.mask_local_2d_dilated_dense(n, b, dil)
        c_out, c_m, c_l = c_oracle.local_2d_dilated(q, k, v, b, dil, use_nan=True, chunk=3)
    else:
        g, w = golden["glob_inds"], int(golden["glob_w"])
        mask = so.mask_global_no_local_dense(n, g, w)
        c_out, c_m, c_l = c_oracle.global_no_local(q, k, v, g, w, chunk=5)
    out, m, l = so.dense_masked_attention(q, k, v, mask)
    exp_out, exp_lse = golden[kind + "_out"], golden[kind + "_lse"]
    for o, mm, ll in ((out, m, l), (c_out, c_m, c_l)):
        if kind == "glob":
            # rows without a live column: golden holds NaN, the kernels leave such rows untouched
            dead = np.isnan(exp_out).any(axis=1)
            assert np.all(o[dead] == 0.0) or np.all(np.isnan(o[dead]))
            o = np.where(dead[:, None], np.nan, o)
        assert np.array_equal(np.isnan(o), np.isnan(exp_out))
        np.testing.assert_allclose(np.nan_to_num(o), np.nan_to_num(exp_out), atol=1e-12)
        live = np.isfinite(exp_lse)
        np.testing.assert_allclose(_lse(mm, ll)[live], exp_lse[live], atol=1e-12)


def test_chained_union_matches_golden(golden):
    """local -> global-minus-local -> CSR remainder on one (m, l, out) == union mask
    (verification/verify.py:337-355)."""
    q, k, v = golden["q"], golden["k"], golden["v"]
    g, w = golden["glob_inds"], int(golden["glob_w"])
    out, m, l = c_oracle.local(q, k, v, w, chunk=4)
    out, m, l = c_oracle.global_no_local(q, k, v, g, w, m=m, l=l, out=out, chunk=5)
    ro, ci = so.csr_from_dense(golden["union_rest_mask"])
    out, m, l = c_oracle.csr(q, k, v, ro, ci, m=m, l=l, out=out, use_nan=False, chunk=6)
    np.testing.assert_allclose(out, golden["union_out"], atol=1e-12)
    np.testing.assert_allclose(_lse(m, l), golden["union_lse"], atol=1e-12)
    # the numpy row-wise restatement, chained the same way
    r1, c1 = so.csr_from_live(q.shape[0], lambda i: so.live_local(q.shape[0], w, i))
    r2, c2 = so.csr_from_live(q.shape[0], lambda i: so.live_global_no_local(q.shape[0], g, w, i))
    o2, m2, l2 = so.rowwise_attention(q, k, v, r1, c1)
    o2, m2, l2 = so.rowwise_attention(q, k, v, r2, c2, m2, l2, o2)
    o2, m2, l2 = so.rowwise_attention(q, k, v, ro, ci, m2, l2, o2)
    np.testing.assert_allclose(o2, golden["union_out"], atol=1e-12)


# ---------------------------------------------------------------- mask definitions
@pytest.mark.parametrize("n", [1, 2, 7, 33])
def test_local_bounds_vs_dense_loops(n):
    for w in range(0, n):
        dense = so.mask_local_dense(n, w)
        for i in range(n):
            assert np.array_equal(np.nonzero(dense[i])[0], so.live_local(n, w, i))
        assert dense.sum() == so.nnz_local(n, w)
        # band definition
        i, j = np.indices((n, n))
        assert np.array_equal(dense, np.abs(i - j) <= w)


@pytest.mark.parametrize("n", [5, 16, 37])
def test_1d_dilated_bounds_vs_dense_loops(n):
    for w in range(0, min(n, 6)):
        for dil in range(0, 4):
            dense = so.mask_local_1d_dilated_dense(n, w, dil)
            for i in range(n):
                assert np.array_equal(np.nonzero(dense[i])[0], so.live_local_1d_dilated(n, w, dil, i))
            assert dense.sum() == so.nnz_local_1d_dilated(n, w, dil)
            i, j = np.indices((n, n))
            s = dil + 1
            assert np.array_equal(dense, ((i - j) % s == 0) & (np.abs(i - j) <= w * s))
            if dil == 0:
                assert np.array_equal(dense, so.mask_local_dense(n, w))


@pytest.mark.parametrize("n,block", [(16, 4), (48, 16), (30, 5), (12, 1)])
def test_2d_dilated_bounds_vs_dense_loops(n, block):
    for dil in range(0, block):
        dense = so.mask_local_2d_dilated_dense(n, block, dil)
        for i in range(n):
            assert np.array_equal(np.nonzero(dense[i])[0], so.live_local_2d_dilated(n, block, dil, i))
        assert dense.sum() == so.nnz_local_2d_dilated(n, block, dil)
        i, j = np.indices((n, n))
        s = dil + 1
        assert np.array_equal(dense, (i // block == j // block) & ((i % block) % s == 0) & ((j % block) % s == 0))


@pytest.mark.parametrize("n,globs,w", [(32, [0, 1, 10], 3), (32, [31], 0), (20, [5, 6, 7], 19),
                                       (40, [3, 39, 20, 21], 5), (9, list(range(9)), 2)])
def test_global_no_local_bounds_vs_dense_loops(n, globs, w):
    dense = so.mask_global_no_local_dense(n, globs, w)
    for i in range(n):
        assert np.array_equal(np.nonzero(dense[i])[0], np.sort(so.live_global_no_local(n, globs, w, i)))
    assert dense.sum() == so.nnz_global_no_local(n, globs, w)
    # local(w) and global-minus-local(w) are disjoint by construction
    assert not (dense & so.mask_local_dense(n, w)).any()


# ---------------------------------------------------------------- row-wise and C restatements
@pytest.mark.parametrize("chunk", [1, 3, 8, 46, 1000])
def test_c_and_rowwise_match_dense_random_csr(chunk):
    n, d = 70, 12
    q, k, v = _rand(n, d, 11)
    rng = np.random.default_rng(12)
    mask = rng.random((n, n)) < 0.2
    mask[4, :] = False
    mask[9, :] = True
    # rows whose length is an exact multiple of the chunk must not lose their last chunk
    mask[10, :] = False
    mask[10, : 2 * min(chunk, 30)] = True
    ro, ci = so.csr_from_dense(mask)
    out, m, l = so.dense_masked_attention(q, k, v, mask)
    for o2, m2, l2 in (so.rowwise_attention(q, k, v, ro, ci, use_nan=True),
                       c_oracle.csr(q, k, v, ro, ci, use_nan=True, chunk=chunk)):
        assert np.array_equal(np.isnan(o2), np.isnan(out))
        np.testing.assert_allclose(np.nan_to_num(o2), np.nan_to_num(out), atol=1e-12)
        live = l > 0
        np.testing.assert_allclose(m2[live], m[live], atol=1e-12)
        np.testing.assert_allclose(l2[live], l[live], rtol=1e-12)
        assert np.all(np.isneginf(m2[~live])) and np.all(l2[~live] == 0)


def test_empty_rows_nan_or_untouched_and_state_untouched():
    n, d = 20, 4
    q, k, v = _rand(n, d, 13)
    mask = np.zeros((n, n), dtype=bool)
    mask[::2, 1] = True
    ro, ci = so.csr_from_dense(mask)
    out0 = np.full((n, d), 7.0)
    m0 = np.full(n, -1.5)
    l0 = np.full(n, 2.5)
    for use_nan in (False, True):
        for o, m, l in (c_oracle.csr(q, k, v, ro, ci, m=m0, l=l0, out=out0, use_nan=use_nan),
                        so.rowwise_attention(q, k, v, ro, ci, m0, l0, out0, use_nan=use_nan)):
            dead = np.arange(n) % 2 == 1
            assert np.all(m[dead] == -1.5) and np.all(l[dead] == 2.5)
            if use_nan:
                assert np.isnan(o[dead]).all()
            else:
                assert np.all(o[dead] == 7.0)


def test_coo_is_order_independent_and_equals_csr():
    n, d = 60, 8
    q, k, v = _rand(n, d, 14)
    mask = np.random.default_rng(15).random((n, n)) < 0.15
    ro, ci = so.csr_from_dense(mask)
    r, c = so.coo_from_dense(mask)
    perm = np.random.default_rng(16).permutation(len(r))
    a = c_oracle.csr(q, k, v, ro, ci, use_nan=True)
    b = c_oracle.coo(q, k, v, r, c, use_nan=True)
    cc = c_oracle.coo(q, k, v, r[perm], c[perm], use_nan=True)
    for x, y in zip(a, b):
        np.testing.assert_allclose(np.nan_to_num(x), np.nan_to_num(y), atol=1e-13)
    for x, y in zip(a, cc):
        np.testing.assert_allclose(np.nan_to_num(x), np.nan_to_num(y), atol=1e-12)
    ro2, ci2 = so.csr_from_coo(r[perm], c[perm], n)
    assert np.array_equal(ro2, ro)
    assert np.array_equal(so.dense_from_csr(ro2, ci2, n, n), mask)


def test_split_and_chain_equals_single_call():
    n, d = 48, 8
    q, k, v = _rand(n, d, 17)
    rng = np.random.default_rng(18)
    mask = rng.random((n, n)) < 0.3
    part = rng.integers(0, 3, size=(n, n))
    full, mf, lf = so.dense_masked_attention(q, k, v, mask)
    out, m, l = None, None, None
    for p in range(3):
        ro, ci = so.csr_from_dense(mask & (part == p))
        out, m, l = c_oracle.csr(q, k, v, ro, ci, m=m, l=l, out=out, use_nan=False, chunk=5)
    live = mask.any(axis=1)
    np.testing.assert_allclose(out[live], full[live], atol=1e-12)
    np.testing.assert_allclose((m + np.log(l))[live], (mf + np.log(lf))[live], atol=1e-12)


def test_merge_state_identity_and_associativity():
    rng = np.random.default_rng(19)
    parts = [(rng.standard_normal(), rng.random() + 0.1, rng.standard_normal(4)) for _ in range(3)]
    fresh = (-np.inf, 0.0, np.zeros(4))
    a = so.merge_state(*fresh, *parts[0])
    assert a[0] == parts[0][0] and a[1] == parts[0][1] and np.allclose(a[2], parts[0][2], atol=0)
    left = so.merge_state(*so.merge_state(*parts[0], *parts[1]), *parts[2])
    right = so.merge_state(*parts[0], *so.merge_state(*parts[1], *parts[2]))
    for x, y in zip(left, right):
        np.testing.assert_allclose(x, y, atol=1e-14)


@pytest.mark.parametrize("kind", ["local", "d1", "d2", "glob"])
def test_c_implicit_masks_match_dense(kind):
    n, d = 96, 8
    q, k, v = _rand(n, d, 21)
    if kind == "local":
        cases = [(so.mask_local_dense(n, w), lambda w=w: c_oracle.local(q, k, v, w, chunk=7)) for w in (0, 1, 13, n - 1)]
    elif kind == "d1":
        cases = [(so.mask_local_1d_dilated_dense(n, w, dil),
                  lambda w=w, dil=dil: c_oracle.local_1d_dilated(q, k, v, w, dil, chunk=4))
                 for w, dil in ((3, 0), (10, 2), (40, 1), (n - 1, 5))]
    elif kind == "d2":
        cases = [(so.mask_local_2d_dilated_dense(n, b, dil),
                  lambda b=b, dil=dil: c_oracle.local_2d_dilated(q, k, v, b, dil, use_nan=True, chunk=4))
                 for b, dil in ((16, 0), (16, 1), (32, 2), (96, 7), (8, 7))]
    else:
        cases = [(so.mask_global_no_local_dense(n, g, w),
                  lambda g=g, w=w: c_oracle.global_no_local(q, k, v, g, w, chunk=9))
                 for g, w in (([0, 1, 10, 40], 10), ([95], 0), ([50, 3], 95), (list(range(0, 96, 5)), 2))]
    for mask, fn in cases:
        out, m, l = so.dense_masked_attention(q, k, v, mask)
        o2, m2, l2 = fn()
        live = mask.any(axis=1)
        np.testing.assert_allclose(o2[live], out[live], atol=1e-12)
        np.testing.assert_allclose(m2[live], m[live], atol=1e-12)
        np.testing.assert_allclose(l2[live], l[live], rtol=1e-12)
        if kind == "d2":
            assert np.isnan(o2[~live]).all()
        else:
            assert np.all(o2[~live] == 0)
        assert np.all(np.isneginf(m2[~live])) and np.all(l2[~live] == 0)


# ---------------------------------------------------------------- parameter checks
def test_parameter_checks_match_reference_texts():
    q, k, v = _rand(8, 4, 22)
    with pytest.raises(ValueError, match="local size specified"):
        c_oracle.local(q, k, v, 8)
    with pytest.raises(ValueError, match="local size specified"):
        c_oracle.local(q, k, v, -1)
    with pytest.raises(ValueError, match="dilation factor must be atleast 0"):
        c_oracle.local_1d_dilated(q, k, v, 2, -1)
    with pytest.raises(ValueError, match="must be a divisor"):
        c_oracle.local_2d_dilated(q, k, v, 3, 0)
    with pytest.raises(ValueError, match="dilation factor must be atleast 0"):
        c_oracle.local_2d_dilated(q, k, v, 4, -1)
    with pytest.raises(ValueError, match="less than the block/window size"):
        c_oracle.local_2d_dilated(q, k, v, 4, 4)
    with pytest.raises(ValueError, match="no global tokens"):
        c_oracle.global_no_local(q, k, v, [], 1)
    with pytest.raises(ValueError, match="no global tokens"):
        c_oracle.global_no_local(q, k, v, list(range(9)), 1)
    with pytest.raises(ValueError, match="local size specified"):
        c_oracle.global_no_local(q, k, v, [1], 8)
    for fn, args in ((so.check_local, (8, 8)), (so.check_local_1d_dilated, (8, 2, -1)),
                     (so.check_local_2d_dilated, (8, 3, 0)), (so.check_local_2d_dilated, (8, 4, 4)),
                     (so.check_global_no_local, (8, 0, 1))):
        with pytest.raises(ValueError):
            fn(*args)
