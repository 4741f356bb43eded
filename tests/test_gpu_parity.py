"""GPU parity tests: the six spfa_* modules (host wrapper -> C ABI -> HIP kernels) against the CPU
oracle on the same seeded inputs.  Bars: max-abs 1e-4 (fp32), 2e-2 (fp16 / bf16) on the output,
identical sets of computed rows, and m + log(l) equal to the oracle's log-sum-exp."""
import math

import numpy as np
import pytest
import torch

import spfa_synth as syn
from helpers import OUT_TOL, check, csr_rows_subset, np64, oracle_rows
from oracle import c_oracle
from oracle import spfa_oracle as so

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def sync():
    torch.cuda.synchronize()


def dev_qkv(n, d, dtype, seed, scale=1.0, n_k=None):
    q, k, v = syn.qkv(n, d, dtype=dtype, device="cpu", seed=seed, scale=scale, n_k=n_k)
    return q.to(DEV), k.to(DEV), v.to(DEV)


def state(n, d, dtype, state_dtype=None):
    return syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=state_dtype)


def csr_tensors(ro, ci, off_dtype=torch.uint64, col_dtype=torch.uint32):
    ro_t = torch.as_tensor(np.asarray(ro, dtype=np.int64)).to(off_dtype).to(DEV)
    ci_t = torch.as_tensor(np.asarray(ci, dtype=np.int64)).to(col_dtype).to(DEV)
    return ro_t, ci_t


def run_csr(mods, q, k, v, ro, ci, use_nan, st=None, off_dtype=torch.uint64, col_dtype=torch.uint32,
            state_dtype=None):
    n, d = q.shape
    m, l, o = st if st is not None else state(n, d, q.dtype, state_dtype)
    ro_t, ci_t = csr_tensors(ro, ci, off_dtype, col_dtype)
    val = torch.ones(ci_t.numel(), device=DEV, dtype=q.dtype)
    fresh = st is None
    ret = mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, use_nan)
    sync()
    assert ret.data_ptr() == o.data_ptr()
    if fresh and q.dim() == 2:
        # Small problems take a single-launch path in a plain call; a planned call always takes the
        # general one (work list, short / medium / segmented rows).  Both must agree.
        m2, l2, o2 = state(n, d, q.dtype, state_dtype)
        plan = mods["spfa_csr"].plan(ro_t, ci_t)
        mods["spfa_csr"].forward_planned(q, k, v, ro_t, ci_t, val, m2, l2, o2, use_nan, plan)
        sync()
        tol = 2e-5 if q.dtype in (torch.float32, torch.float64) else 2e-2
        assert torch.allclose(torch.nan_to_num(o).float(), torch.nan_to_num(o2).float(), atol=tol)
        assert torch.equal(torch.isnan(o), torch.isnan(o2))
        assert torch.allclose(lse_t(m, l), lse_t(m2, l2), atol=1e-3 if tol > 1e-3 else 1e-5, equal_nan=True)
    return o, m, l


def lse_t(m, l):
    with torch.no_grad():
        x = m.float() + torch.log(l.float())
    return torch.where(l.float() > 0, x, torch.zeros_like(x))


# ------------------------------------------------------------------ the reference's own checks
class TestVerifyScript:
    """Seeded re-statements of the eleven comparisons of verification/verify.py (N=256, d=32,
    fp32, uniform [0,1) inputs)."""
    N, D = 256, 32

    def setup_method(self, _):
        g = torch.Generator().manual_seed(1234)
        self.q, self.k, self.v = [torch.rand(self.N, self.D, generator=g).to(DEV) for _ in range(3)]
        self.qn, self.kn, self.vn = np64(self.q), np64(self.k), np64(self.v)

    def dense(self, mask):
        return so.dense_masked_attention(self.qn, self.kn, self.vn, mask)

    def test_csr_coo_local_full_agree_with_dense(self, mods):  # verify.py:42-152
        n, d = self.N, self.D
        mask = np.ones((n, n), dtype=bool)
        ref = self.dense(mask)
        ro, ci = so.csr_from_dense(mask)
        o1, m1, l1 = run_csr(mods, self.q, self.k, self.v, ro, ci, True)
        check(o1, m1, l1, *ref, torch.float32)
        r, c = so.coo_from_dense(mask)
        m, l, o2 = state(n, d, torch.float32)
        mods["spfa_coo"].forward(self.q, self.k, self.v, torch.as_tensor(r).to(torch.uint64).to(DEV),
                                 torch.as_tensor(c).to(torch.uint32).to(DEV),
                                 torch.ones(len(c), device=DEV), m, l, o2, True)
        sync()
        check(o2, m, l, *ref, torch.float32)
        m, l, o3 = state(n, d, torch.float32)
        mods["spfa_local"].forward(self.q, self.k, self.v, m, l, o3, n - 1)
        sync()
        check(o3, m, l, *ref, torch.float32)
        assert torch.allclose(o1, o2, atol=1e-5) and torch.allclose(o1, o3, atol=1e-5)

    def test_local_window_zero_returns_v(self, mods):  # verify.py:158-177
        m, l, o = state(self.N, self.D, torch.float32)
        mods["spfa_local"].forward(self.q, self.k, self.v, m, l, o, 0)
        sync()
        assert torch.equal(o, self.v)
        assert torch.all(l == 1.0)

    def test_global_no_local(self, mods):  # verify.py:183-229
        globs, w = [0, 1, 10, 40], 10
        ref = self.dense(so.mask_global_no_local_dense(self.N, globs, w))
        m, l, o = state(self.N, self.D, torch.float32)
        g = torch.tensor(globs, dtype=torch.int32, device=DEV)
        mods["spfa_global_no_local"].forward(self.q, self.k, self.v, m, l, o, g, w)
        sync()
        check(o, m, l, *ref, torch.float32)

    def _bigbird(self, seed):
        n = self.N
        rng = np.random.default_rng(seed)
        globs = np.sort(rng.choice(n, 5, replace=False))
        w = 10
        rnd = rng.random((n, n)) < 0.1
        fixed = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, globs, w)
        return globs, w, rnd, fixed

    def test_bigbird_as_one_csr(self, mods):  # verify.py:235-290
        globs, w, rnd, fixed = self._bigbird(7)
        mask = fixed | rnd
        ro, ci = so.csr_from_dense(mask)
        o, m, l = run_csr(mods, self.q, self.k, self.v, ro, ci, False)
        check(o, m, l, *self.dense(mask), torch.float32)

    def test_bigbird_chained_three_kernels(self, mods):  # verify.py:296-362
        globs, w, rnd, fixed = self._bigbird(8)
        m, l, o = state(self.N, self.D, torch.float32)
        mods["spfa_local"].forward(self.q, self.k, self.v, m, l, o, w)
        mods["spfa_global_no_local"].forward(self.q, self.k, self.v, m, l, o,
                                             torch.tensor(globs, dtype=torch.int32, device=DEV), w)
        ro, ci = so.csr_from_dense(rnd & ~fixed)
        o, m, l = run_csr(mods, self.q, self.k, self.v, ro, ci, False, st=(m, l, o))
        check(o, m, l, *self.dense(fixed | rnd), torch.float32)

    def test_local_1d_dilated(self, mods):  # verify.py:368-409
        w, dil = 10, 2
        m, l, o = state(self.N, self.D, torch.float32)
        mods["spfa_local_1d_dilated"].forward(self.q, self.k, self.v, m, l, o, w, dil)
        sync()
        check(o, m, l, *self.dense(so.mask_local_1d_dilated_dense(self.N, w, dil)), torch.float32)

    @pytest.mark.parametrize("dil", [0, 1])
    def test_local_2d_dilated(self, mods, dil):  # verify.py:415-505
        m, l, o = state(self.N, self.D, torch.float32)
        mods["spfa_local_2d_dilated"].forward(self.q, self.k, self.v, m, l, o, 16, dil, True)
        sync()
        check(o, m, l, *self.dense(so.mask_local_2d_dilated_dense(self.N, 16, dil)), torch.float32,
              dead_expect="nan")


# ------------------------------------------------------------------ golden vectors, every dtype
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["csr", "coo", "local", "d1", "d2", "glob", "union"])
def test_golden_vectors(mods, golden, kind, dtype):
    q, k, v = [torch.tensor(golden[x], dtype=dtype, device=DEV) for x in ("q", "k", "v")]
    n, d = q.shape
    m, l, o = state(n, d, dtype, torch.float32)
    dead_expect = None
    key = kind
    if kind in ("csr", "coo"):
        key = "csr"
        ro, ci = so.csr_from_dense(golden["csr_mask"])
        val = torch.ones(len(ci), device=DEV, dtype=dtype)
        if kind == "csr":
            ro_t, ci_t = csr_tensors(ro, ci)
            mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, True)
        else:
            r, c = so.coo_from_dense(golden["csr_mask"])
            perm = np.random.default_rng(5).permutation(len(r))
            mods["spfa_coo"].forward(q, k, v, torch.as_tensor(r[perm]).to(torch.uint64).to(DEV),
                                     torch.as_tensor(c[perm]).to(torch.uint32).to(DEV), val, m, l, o, True)
        dead_expect = "nan"
    elif kind == "local":
        mods["spfa_local"].forward(q, k, v, m, l, o, int(golden["local_w"]))
    elif kind == "d1":
        mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, int(golden["d1_w"]), int(golden["d1_dil"]))
    elif kind == "d2":
        mods["spfa_local_2d_dilated"].forward(q, k, v, m, l, o, int(golden["d2_block"]),
                                              int(golden["d2_dil"]), True)
        dead_expect = "nan"
    else:
        g = torch.tensor(golden["glob_inds"], dtype=torch.int32, device=DEV)
        w = int(golden["glob_w"])
        if kind == "union":
            mods["spfa_local"].forward(q, k, v, m, l, o, w)
        mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g, w)
        if kind == "union":
            ro, ci = so.csr_from_dense(golden["union_rest_mask"])
            ro_t, ci_t = csr_tensors(ro, ci)
            mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, torch.ones(len(ci), device=DEV, dtype=dtype),
                                     m, l, o, False)
    sync()
    exp_out, exp_lse = golden[key + "_out"], golden[key + "_lse"]
    live = np.isfinite(exp_lse)
    ref_l = np.where(live, 1.0, 0.0)
    ref_m = np.where(live, exp_lse, -np.inf)  # lse == m + log(1)
    check(o, m, l, np.nan_to_num(exp_out), ref_m, ref_l, dtype, state_dtype=torch.float32,
          dead_expect=dead_expect, check_m=False)
    if not live.all():
        assert torch.all(torch.isneginf(m[torch.tensor(~live, device=DEV)]))
        assert torch.all(l[torch.tensor(~live, device=DEV)] == 0)


# ------------------------------------------------------------------ CSR
def test_csr_bernoulli_n4096_d64_fp32(mods):
    """The CPU-runnable configuration: N=4096, d=64, fp32, 2% random mask plus diagonal, against the
    dense float64 formulation."""
    n, d = 4096, 64
    q, k, v = dev_qkv(n, d, torch.float32, 0)
    ro, ci = syn.bernoulli_csr(n, 0.02, seed=0)
    o, m, l = run_csr(mods, q, k, v, ro, ci, True)
    mask = so.dense_from_csr(ro.numpy(), ci.numpy(), n, n)
    check(o, m, l, *so.dense_masked_attention(np64(q), np64(k), np64(v), mask), torch.float32)


def _special_rows_csr(n, rng, lengths):
    """Mask whose first rows have the given lengths (the rest random short rows)."""
    cols, off = [], [0]
    for i in range(n):
        ln = lengths[i] if i < len(lengths) else int(rng.integers(0, 6))
        c = np.sort(rng.choice(n, ln, replace=False)) if ln else np.zeros(0, np.int64)
        cols.append(c)
        off.append(off[-1] + ln)
    return np.array(off, np.int64), np.concatenate(cols).astype(np.int64)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.float32, 32), (torch.float32, 128),
                                     (torch.bfloat16, 64), (torch.float16, 128), (torch.float32, 256)])
def test_csr_row_lengths_around_every_threshold(mods, dtype, d):
    """Rows of length 0, 1, the in-place limit and one more, one segment and one more, several
    segments exactly, and the longest possible row."""
    n = 2048
    rng = np.random.default_rng(3)
    lengths = [0, 1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 255, 256, 257, 511, 512, 513, 768, 1024, 2048, 0, 7]
    ro, ci = _special_rows_csr(n, rng, lengths)
    q, k, v = dev_qkv(n, d, dtype, 21)
    o, m, l = run_csr(mods, q, k, v, ro, ci, True, state_dtype=torch.float32)
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro, ci, use_nan=True)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32, dead_expect="nan")


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 128), (torch.float32, 200)])
def test_csr_small_problem_with_very_long_rows(mods, dtype, d):
    """Few rows, some of them longer than the single-launch path gives one wavefront: whole key range, repeated
    columns, lengths around the hand-over."""
    n_q, n_k = 37, 8192
    rng = np.random.default_rng(77)
    lengths = [8192, 0, 2048, 2049, 5000, 3, 12000, 1, 2047, 4097] + [int(x) for x in rng.integers(0, 40, n_q - 10)]
    cols, off = [], [0]
    for ln in lengths:
        cols.append(rng.integers(0, n_k, ln) if ln > n_k else rng.choice(n_k, ln, replace=False))
        off.append(off[-1] + ln)
    ro, ci = np.array(off, np.int64), np.concatenate(cols).astype(np.int64)
    q, k, v = dev_qkv(n_q, d, dtype, 78, n_k=n_k)
    o, m, l = run_csr(mods, q, k, v, ro, ci, True, state_dtype=torch.float32)
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro, ci, use_nan=True)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32, dead_expect="nan")


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 64), (torch.float32, 40)])
def test_csr_rows_of_more_segments_than_the_work_list_has_phases(mods, dtype, d):
    """More keys than the single-launch path takes, so the rows go through the work list: rows cut into up to 79
    segments of 512 (the list is handed out in 64 phases, so several segments of a row share one), rows of one
    and two segments, medium and short rows, empty rows."""
    n_q, n_k = 64, 40000
    rng = np.random.default_rng(91)
    lengths = [40000, 39999, 9000, 1025, 1024, 513, 512, 300, 257, 256, 129, 128, 33, 17, 16, 5, 0, 1] + \
        [int(x) for x in rng.integers(0, 400, n_q - 18)]
    cols, off = [], [0]
    for ln in lengths:
        cols.append(np.sort(rng.choice(n_k, ln, replace=False)))
        off.append(off[-1] + ln)
    ro, ci = np.array(off, np.int64), np.concatenate(cols).astype(np.int64)
    q, k, v = dev_qkv(n_q, d, dtype, 92, n_k=n_k)
    o, m, l = run_csr(mods, q, k, v, ro, ci, True, state_dtype=torch.float32)
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro, ci, use_nan=True)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32, dead_expect="nan")


@pytest.mark.parametrize("dtype", DTYPES)
def test_csr_power_law_rows(mods, dtype):
    """Zipf(1.5) degrees clipped to [1, 4096] at N=16384: short rows, single-segment rows and
    rows split over several segments in one call."""
    n, d = 16384, 64
    q, k, v = dev_qkv(n, d, dtype, 5)
    ro, ci = syn.zipf_csr(n, 1.5, 1, 4096, seed=5)
    o, m, l = run_csr(mods, q, k, v, ro, ci, False, state_dtype=torch.float32)
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy())
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)


@pytest.mark.parametrize("d", [1, 3, 40, 100, 200, 520])
def test_csr_any_embedding_size(mods, d):
    n = 300
    q, k, v = dev_qkv(n, d, torch.float32, 9)
    ro, ci = syn.zipf_csr(n, 1.3, 0, 300, seed=9)
    o, m, l = run_csr(mods, q, k, v, ro, ci, True)
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy(), use_nan=True)
    check(o, m, l, *ref, torch.float32, dead_expect="nan")


@pytest.mark.parametrize("off_dtype,col_dtype", [(torch.uint64, torch.uint32), (torch.int64, torch.int32),
                                                 (torch.int32, torch.int32), (torch.uint32, torch.uint32)])
def test_csr_index_dtypes(mods, off_dtype, col_dtype):
    n, d = 512, 64
    q, k, v = dev_qkv(n, d, torch.float32, 10)
    ro, ci = syn.zipf_csr(n, 1.5, 0, 512, seed=10)
    o, m, l = run_csr(mods, q, k, v, ro, ci, True, off_dtype=off_dtype, col_dtype=col_dtype)
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy(), use_nan=True)
    check(o, m, l, *ref, torch.float32, dead_expect="nan")


def test_csr_rectangular_k(mods):
    """K/V may have a different row count than Q: columns index K/V rows."""
    n, n_k, d = 256, 1000, 64
    q, k, v = dev_qkv(n, d, torch.float32, 12, n_k=n_k)
    g = torch.Generator().manual_seed(12)
    deg = torch.randint(0, 40, (n,), generator=g)
    ro, ci = syn.csr_from_degrees(deg, n_k, g, "cpu", force_diagonal=False)
    o, m, l = run_csr(mods, q, k, v, ro, ci, True)
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy(), use_nan=True)
    check(o, m, l, *ref, torch.float32, dead_expect="nan")


@pytest.mark.parametrize("use_nan", [False, True])
def test_csr_empty_rows_and_state_untouched(mods, use_nan):
    n, d = 128, 64
    q, k, v = dev_qkv(n, d, torch.float32, 13)
    mask = np.zeros((n, n), dtype=bool)
    mask[::2, 5] = True
    ro, ci = so.csr_from_dense(mask)
    m = torch.full((n,), -1.5, device=DEV)
    l = torch.full((n,), 2.5, device=DEV)
    o = torch.full((n, d), 7.0, device=DEV)
    m0, l0, o0 = m.clone(), l.clone(), o.clone()
    run_csr(mods, q, k, v, ro, ci, use_nan, st=(m, l, o))
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro, ci, m=np64(m0), l=np64(l0), out=np64(o0), use_nan=use_nan)
    dead = torch.arange(n, device=DEV) % 2 == 1
    assert torch.equal(m[dead], m0[dead]) and torch.equal(l[dead], l0[dead])
    if use_nan:
        assert torch.isnan(o[dead]).all()
    else:
        assert torch.equal(o[dead], o0[dead])
    live = ~dead
    assert np.abs(np64(o[live]) - ref[0][np64(live) > 0]).max() <= 1e-4
    assert np.abs(np64(m[live]) - ref[1][np64(live) > 0]).max() <= 1e-4
    assert np.abs(np64(l[live]) / ref[2][np64(live) > 0] - 1).max() <= 1e-4


def test_csr_split_and_chain_equals_single_call(mods):
    n, d = 1024, 64
    q, k, v = dev_qkv(n, d, torch.float32, 14)
    rng = np.random.default_rng(14)
    mask = rng.random((n, n)) < 0.08
    part = rng.integers(0, 3, size=(n, n))
    st = state(n, d, torch.float32)
    for p in range(3):
        ro, ci = so.csr_from_dense(mask & (part == p))
        o, m, l = run_csr(mods, q, k, v, ro, ci, False, st=st)
    check(o, m, l, *so.dense_masked_attention(np64(q), np64(k), np64(v), mask), torch.float32)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_csr_state_in_element_dtype(mods, dtype):
    """m and l in the element type, as the reference allocates them."""
    n, d = 512, 64
    q, k, v = dev_qkv(n, d, dtype, 15)
    ro, ci = syn.zipf_csr(n, 1.5, 1, 512, seed=15)
    o, m, l = run_csr(mods, q, k, v, ro, ci, False)
    assert m.dtype == dtype and l.dtype == dtype
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy())
    check(o, m, l, *ref, dtype)


# ------------------------------------------------------------------ batch x heads
def _stacked(n, d, dtype, shape, seed, n_k=None):
    """q, k, v with leading batch dimensions `shape`, and a fresh state."""
    b = int(np.prod(shape))
    qs, ks, vs = [], [], []
    for i in range(b):
        q, k, v = syn.qkv(n, d, dtype=dtype, device="cpu", seed=seed + i, n_k=n_k)
        qs.append(q), ks.append(k), vs.append(v)
    n_k = n if n_k is None else n_k
    q = torch.stack(qs).reshape(*shape, n, d).to(DEV)
    k = torch.stack(ks).reshape(*shape, n_k, d).to(DEV)
    v = torch.stack(vs).reshape(*shape, n_k, d).to(DEV)
    m = torch.full((*shape, n), -float("inf"), device=DEV, dtype=torch.float32)
    l = torch.zeros((*shape, n), device=DEV, dtype=torch.float32)
    o = torch.zeros((*shape, n, d), device=DEV, dtype=dtype)
    return q, k, v, m, l, o


def _check_heads(q, k, v, o, m, l, ref_fn, dtype, **kw):
    n, d = q.shape[-2:]
    qf, kf, vf = q.reshape(-1, n, d), k.reshape(-1, k.shape[-2], d), v.reshape(-1, v.shape[-2], d)
    of, mf, lf = o.reshape(-1, n, d), m.reshape(-1, n), l.reshape(-1, n)
    for b in range(qf.shape[0]):
        ref = ref_fn(np64(qf[b]), np64(kf[b]), np64(vf[b]))
        check(of[b], mf[b], lf[b], *ref, dtype, state_dtype=torch.float32, **kw)


@pytest.mark.parametrize("dtype,shape", [(torch.float32, (3,)), (torch.bfloat16, (2, 3)), (torch.float16, (5,))])
def test_csr_batch_of_heads_shares_the_mask(mods, dtype, shape):
    """[batch..., tokens, embedding] tensors: every problem of the batch against the oracle; long
    rows (segments + merge) and short rows, empty rows NaN."""
    n, d = 3000, 64
    ro, ci = syn.zipf_csr(n, 1.3, 0, 2500, seed=51)
    ro_t, ci_t = csr_tensors(ro, ci)
    q, k, v, m, l, o = _stacked(n, d, dtype, shape, 51)
    val = torch.ones(ci_t.numel(), device=DEV, dtype=dtype)
    ret = mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, True)
    sync()
    assert ret.data_ptr() == o.data_ptr()
    _check_heads(q, k, v, o, m, l,
                 lambda a, b, c: c_oracle.csr(a, b, c, ro.numpy(), ci.numpy(), use_nan=True), dtype,
                 dead_expect="nan")
    # the planned call takes the same plan for any batch
    plan = mods["spfa_csr"].plan(ro_t, ci_t)
    q, k, v, m2, l2, o2 = q, k, v, torch.full_like(m, -float("inf")), torch.zeros_like(l), torch.zeros_like(o)
    mods["spfa_csr"].forward_planned(q, k, v, ro_t, ci_t, val, m2, l2, o2, True, plan)
    sync()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(torch.nan_to_num(o).float(), torch.nan_to_num(o2).float(), atol=tol)


def test_coo_batch_rectangular_keys(mods):
    n, n_k, d = 1500, 2200, 64
    g = torch.Generator().manual_seed(52)
    deg = torch.randint(0, 90, (n,), generator=g)
    deg[17] = 1800
    ro, ci = syn.csr_from_degrees(deg, n_k, g, "cpu", force_diagonal=False)
    r, c = syn.coo_from_csr(ro, ci, shuffle_seed=52)
    q, k, v, m, l, o = _stacked(n, d, torch.float32, (4,), 52, n_k=n_k)
    mods["spfa_coo"].forward(q, k, v, r.to(torch.uint64).to(DEV), c.to(torch.uint32).to(DEV),
                             torch.ones(c.numel(), device=DEV), m, l, o, False)
    sync()
    _check_heads(q, k, v, o, m, l, lambda a, b, cc: c_oracle.csr(a, b, cc, ro.numpy(), ci.numpy()),
                 torch.float32)


@pytest.mark.parametrize("use_nan", [False, True])
@pytest.mark.parametrize("shape", [(), (3,)])
def test_csr_mostly_empty_rows(mods, shape, use_nan):
    """Seven rows in ten empty, the others short (1 - 25 columns) with a few medium and long ones:
    the short rows are then taken from a list instead of row by row (when empty rows are left
    untouched), one problem and a batch sharing the mask, plain and planned calls."""
    n, d = 40_000, 64
    g = torch.Generator().manual_seed(53)
    deg = torch.randint(1, 26, (n,), generator=g)
    deg[torch.rand(n, generator=g) < 0.7] = 0
    deg[torch.randperm(n, generator=g)[:60]] = 150
    deg[torch.randperm(n, generator=g)[:5]] = 3000
    ro, ci = syn.csr_from_degrees(deg, n, g, "cpu", force_diagonal=False)
    ro_t, ci_t = csr_tensors(ro, ci)
    q, k, v, m, l, o = _stacked(n, d, torch.float32, shape, 53)
    val = torch.ones(ci_t.numel(), device=DEV)
    mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, use_nan)
    sync()
    ref_fn = lambda a, b, c: c_oracle.csr(a, b, c, ro.numpy(), ci.numpy(), use_nan=use_nan)
    if shape:
        _check_heads(q, k, v, o, m, l, ref_fn, torch.float32, dead_expect="nan" if use_nan else "zero")
    else:
        check(o, m, l, *ref_fn(np64(q), np64(k), np64(v)), torch.float32, dead_expect="nan" if use_nan else "zero")
    plan = mods["spfa_csr"].plan(ro_t, ci_t)
    m2, l2, o2 = torch.full_like(m, -float("inf")), torch.zeros_like(l), torch.zeros_like(o)
    mods["spfa_csr"].forward_planned(q, k, v, ro_t, ci_t, val, m2, l2, o2, use_nan, plan)
    sync()
    assert torch.allclose(torch.nan_to_num(o), torch.nan_to_num(o2), atol=2e-6)
    assert torch.equal(m, m2) and torch.allclose(l, l2, rtol=1e-5)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 64), (torch.float32, 40)])
def test_implicit_masks_batch_of_heads(mods, dtype, d):
    """d = 64 runs the dense-tile kernels as they are, d = 40 those of d = 64 with zero-filled operands."""
    n = 1024
    shape = (2, 2)
    w, dil, blk = 40, 1, 64
    globs = [3, 500, 501, 900]
    cases = [
        ("spfa_local", (w,), so.mask_local_dense(n, w), None),
        ("spfa_local_1d_dilated", (w, dil), so.mask_local_1d_dilated_dense(n, w, dil), None),
        ("spfa_local_2d_dilated", (blk, dil, True), so.mask_local_2d_dilated_dense(n, blk, dil), "nan"),
    ]
    for name, args, dense, dead in cases:
        q, k, v, m, l, o = _stacked(n, d, dtype, shape, 53)
        mods[name].forward(q, k, v, m, l, o, *args)
        sync()
        _check_heads(q, k, v, o, m, l, lambda a, b, c: so.dense_masked_attention(a, b, c, dense), dtype,
                     dead_expect=dead)
    q, k, v, m, l, o = _stacked(n, d, dtype, shape, 54)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, torch.tensor(globs, dtype=torch.int32, device=DEV), w)
    sync()
    dense = so.mask_global_no_local_dense(n, globs, w)
    _check_heads(q, k, v, o, m, l, lambda a, b, c: so.dense_masked_attention(a, b, c, dense), dtype)


# ------------------------------------------------------------------ fp64
def _f64_problem(n, d, seed, n_k=None):
    g = torch.Generator().manual_seed(seed)
    n_k = n if n_k is None else n_k
    q = torch.randn(n, d, generator=g, dtype=torch.float64).to(DEV)
    k = torch.randn(n_k, d, generator=g, dtype=torch.float64).to(DEV)
    v = torch.randn(n_k, d, generator=g, dtype=torch.float64).to(DEV)
    m = torch.full((n,), -float("inf"), device=DEV, dtype=torch.float64)
    l = torch.zeros(n, device=DEV, dtype=torch.float64)
    o = torch.zeros(n, d, device=DEV, dtype=torch.float64)
    return q, k, v, m, l, o


@pytest.mark.parametrize("d", [64, 40, 200])
def test_fp64_every_mask_matches_the_oracle_to_rounding(mods, d):
    """double tensors (the reference dispatches double, sp_flatt_csr_kernel.cu:270): double
    arithmetic on the device, compared with the float64 oracle at 1e-11."""
    n = 700
    f64 = torch.float64
    # CSR with empty, short and long rows, rectangular K; then the same entries as shuffled COO
    n_k = 900
    g = torch.Generator().manual_seed(71)
    deg = torch.randint(0, 40, (n,), generator=g)
    deg[5] = 0
    deg[123] = 850
    ro, ci = syn.csr_from_degrees(deg, n_k, g, "cpu", force_diagonal=False)
    ro_t, ci_t = csr_tensors(ro, ci)
    q, k, v, m, l, o = _f64_problem(n, d, 71, n_k)
    val = torch.ones(ci_t.numel(), device=DEV, dtype=f64)
    mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, True)
    sync()
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy(), use_nan=True)
    check(o, m, l, *ref, f64, dead_expect="nan")
    r, c = syn.coo_from_csr(ro, ci, shuffle_seed=71)
    m2 = torch.full_like(m, -float("inf"))
    l2, o2 = torch.zeros_like(l), torch.zeros_like(o)
    mods["spfa_coo"].forward(q, k, v, r.to(torch.uint64).to(DEV), c.to(torch.uint32).to(DEV), val, m2, l2, o2, True)
    sync()
    check(o2, m2, l2, *ref, f64, dead_expect="nan")
    # implicit masks
    w, dil, blk = 30, 2, 70
    globs = [0, 350, 699]
    for name, args, dense, dead in [
            ("spfa_local", (w,), so.mask_local_dense(n, w), None),
            ("spfa_local_1d_dilated", (w, dil), so.mask_local_1d_dilated_dense(n, w, dil), None),
            ("spfa_local_2d_dilated", (blk, dil, True), so.mask_local_2d_dilated_dense(n, blk, dil), "nan")]:
        q, k, v, m, l, o = _f64_problem(n, d, 72)
        mods[name].forward(q, k, v, m, l, o, *args)
        sync()
        check(o, m, l, *so.dense_masked_attention(np64(q), np64(k), np64(v), dense), f64, dead_expect=dead)
    q, k, v, m, l, o = _f64_problem(n, d, 73)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, torch.tensor(globs, dtype=torch.int32, device=DEV), w)
    sync()
    dense = so.mask_global_no_local_dense(n, globs, w)
    check(o, m, l, *so.dense_masked_attention(np64(q), np64(k), np64(v), dense), f64)


def test_fp64_chained_calls_accumulate(mods):
    n, d, w = 512, 32, 12
    globs = [9, 200]
    q, k, v, m, l, o = _f64_problem(n, d, 74)
    mods["spfa_local"].forward(q, k, v, m, l, o, w)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, torch.tensor(globs, dtype=torch.int32, device=DEV), w)
    sync()
    dense = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, globs, w)
    check(o, m, l, *so.dense_masked_attention(np64(q), np64(k), np64(v), dense), torch.float64)


def test_heads_with_masks_of_their_own_in_one_call(mods):
    """spfa_masks.stack_csr_masks: heads whose masks differ run as one block-diagonal problem on the
    stacked tensors (the batched call is for heads that share a mask)."""
    import spfa_masks
    n, n_k, d, heads = 200, 260, 64, 3
    rng = np.random.default_rng(141)
    dense = [rng.random((n, n_k)) < p for p in (0.05, 0.3, 0.01)]
    parts = []
    for dm in dense:
        ro, ci = so.csr_from_dense(dm)
        parts.append(csr_tensors(ro, ci))
    ro_t, ci_t = spfa_masks.stack_csr_masks(parts, n_k)
    g = torch.Generator().manual_seed(142)
    q = torch.randn(heads, n, d, generator=g).to(DEV)
    k = torch.randn(heads, n_k, d, generator=g).to(DEV)
    v = torch.randn(heads, n_k, d, generator=g).to(DEV)
    m = torch.full((heads, n), -float("inf"), device=DEV)
    l = torch.zeros(heads, n, device=DEV)
    o = torch.zeros(heads, n, d, device=DEV)
    val = torch.empty(0, device=DEV)
    mods["spfa_csr"].forward(q.view(-1, d), k.view(-1, d), v.view(-1, d), ro_t, ci_t, val, m.view(-1), l.view(-1),
                             o.view(-1, d), False)
    sync()
    for h in range(heads):
        check(o[h], m[h], l[h], *so.dense_masked_attention(np64(q[h]), np64(k[h]), np64(v[h]), dense[h]),
              torch.float32)


# ------------------------------------------------------------------ window + global + CSR in one call
@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 64), (torch.float16, 128),
                                      (torch.float32, 40)])
@pytest.mark.parametrize("n,w,n_globs", [(1024, 10, 5), (2000, 64, 70), (1500, 0, 1)])
def test_bigbird_one_call_equals_dense_union(mods, dtype, d, n, w, n_globs):
    """spfa_bigbird.forward == dense attention over Local | Global-no-local | random (the chain of
    verification/verify.py:337-352 in one call)."""
    rng = np.random.default_rng(n + w)
    globs = np.sort(rng.choice(n, n_globs, replace=False))
    fixed = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, globs, w)
    rnd = (rng.random((n, n)) < 0.03) & ~fixed
    ro, ci = so.csr_from_dense(rnd)
    q, k, v = dev_qkv(n, d, dtype, 61)
    m, l, o = state(n, d, dtype, torch.float32)
    ro_t, ci_t = csr_tensors(ro, ci)
    ret = mods["spfa_bigbird"].forward(q, k, v, m, l, o, w, torch.tensor(globs, dtype=torch.int32, device=DEV),
                                       ro_t, ci_t, torch.ones(len(ci), device=DEV, dtype=dtype))
    sync()
    assert ret.data_ptr() == o.data_ptr()
    ref = so.dense_masked_attention(np64(q), np64(k), np64(v), fixed | rnd)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.float16, 128), (torch.bfloat16, 32),
                                     (torch.float16, 256), (torch.float32, 64), (torch.float32, 128)])
@pytest.mark.parametrize("n,w,kind", [(3000, 16, "one"), (3000, 100, "tile"), (2500, 40, "tile+1"),
                                      (4100, 64, "many"), (2048, 33, "repeats"), (1000, 999, "tile"),
                                      (3300, 48, "most"), (3300, 48, "most+1")])
def test_bigbird_window_and_listed_tokens_in_one_kernel(mods, dtype, d, n, w, kind):
    """Half types on the tile kernels: the band kernel takes the listed tokens as further keys.  Against
    the dense union mask where every token is listed once, and against the two chained calls (which
    count a token as often as it is listed and drop entries outside [0, n)) otherwise; three problems
    in one call, on top of a state left by an earlier call."""
    rng = np.random.default_rng(n + w)
    # ("most": the largest list the band kernel takes as further keys, "most+1": the first one that
    # runs as window call + global call)
    count = {"one": 1, "tile": 64, "tile+1": 65, "many": 200, "repeats": 40, "most": 256, "most+1": 257}[kind]
    globs = rng.choice(n, count, replace=False)
    if kind == "repeats":
        globs = np.concatenate([globs, globs[:7], [-3, n, n + 5]])
        rng.shuffle(globs)
    g_t = torch.tensor(globs, dtype=torch.int32, device=DEV)
    e_u64 = torch.zeros(0, dtype=torch.uint64, device=DEV)
    e_u32 = torch.zeros(0, dtype=torch.uint32, device=DEV)
    q, k, v, m, l, o = _stacked(n, d, dtype, (3,), 64)
    mods["spfa_bigbird"].forward(q, k, v, m, l, o, w, g_t, e_u64, e_u32, torch.zeros(0, device=DEV, dtype=dtype))
    sync()
    if kind != "repeats":
        dense = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, np.sort(globs), w)
        _check_heads(q, k, v, o, m, l, lambda a, b, c: so.dense_masked_attention(a, b, c, dense), dtype)
    m2, l2, o2 = torch.full_like(m, -float("inf")), torch.zeros_like(l), torch.zeros_like(o)
    mods["spfa_local"].forward(q, k, v, m2, l2, o2, w)
    mods["spfa_global_no_local"].forward(q, k, v, m2, l2, o2, g_t, w)
    sync()
    assert torch.allclose(o.float(), o2.float(), atol=2e-2)
    assert torch.allclose(m + torch.log(l), m2 + torch.log(l2), atol=2e-2)
    # a second call on the same state: every row has the same keys again
    l1, o1 = l.clone(), o.clone()
    mods["spfa_bigbird"].forward(q, k, v, m, l, o, w, g_t, e_u64, e_u32, torch.zeros(0, device=DEV, dtype=dtype))
    sync()
    assert torch.allclose(l, 2 * l1, rtol=2e-3)
    assert torch.allclose(o.float(), o1.float(), atol=2e-2)


def test_bigbird_parts_may_be_empty_and_batched(mods):
    n, d, w = 1024, 64, 16
    globs = [7, 300, 1000]
    q, k, v, m, l, o = _stacked(n, d, torch.float32, (3,), 62)
    e_i32 = torch.zeros(0, dtype=torch.int32, device=DEV)
    e_u64 = torch.zeros(0, dtype=torch.uint64, device=DEV)
    e_u32 = torch.zeros(0, dtype=torch.uint32, device=DEV)
    e_val = torch.zeros(0, device=DEV)
    # window + globals, no CSR part, three problems at once
    mods["spfa_bigbird"].forward(q, k, v, m, l, o, w, torch.tensor(globs, dtype=torch.int32, device=DEV),
                                 e_u64, e_u32, e_val)
    sync()
    dense = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, globs, w)
    _check_heads(q, k, v, o, m, l, lambda a, b, c: so.dense_masked_attention(a, b, c, dense), torch.float32)
    # window only
    q, k, v, m, l, o = _stacked(n, d, torch.float32, (1,), 63)
    mods["spfa_bigbird"].forward(q, k, v, m, l, o, w, e_i32, e_u64, e_u32, e_val)
    sync()
    dense = so.mask_local_dense(n, w)
    _check_heads(q, k, v, o, m, l, lambda a, b, c: so.dense_masked_attention(a, b, c, dense), torch.float32)


# ------------------------------------------------------------------ mask plans
@pytest.mark.parametrize("dtype", DTYPES)
def test_csr_plan_is_reused_across_calls_and_dtypes(mods, dtype):
    """One plan, built once from the mask alone, serves calls with different Q, K, V (and element
    types); each result matches the oracle and the plain call."""
    n, d = 8192, 64
    ro, ci = syn.zipf_csr(n, 1.4, 0, 3000, seed=41)
    ro_t, ci_t = csr_tensors(ro, ci)
    plan = mods["spfa_csr"].plan(ro_t, ci_t)
    plan_before = plan.clone()
    for seed in (41, 42):
        q, k, v = dev_qkv(n, d, dtype, seed)
        val = torch.ones(ci_t.numel(), device=DEV, dtype=dtype)
        m, l, o = state(n, d, dtype, torch.float32)
        ret = mods["spfa_csr"].forward_planned(q, k, v, ro_t, ci_t, val, m, l, o, True, plan)
        sync()
        assert ret.data_ptr() == o.data_ptr()
        ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy(), use_nan=True)
        check(o, m, l, *ref, dtype, state_dtype=torch.float32, dead_expect="nan")
        o2, m2, l2 = run_csr(mods, q, k, v, ro, ci, True, state_dtype=torch.float32)
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        assert torch.allclose(torch.nan_to_num(o).float(), torch.nan_to_num(o2).float(), atol=tol)
    assert torch.equal(plan, plan_before), "a planned call must not write to the plan"


def test_csr_plan_short_rows_only_and_chaining(mods):
    """A mask without long rows has an empty work list; chained planned calls accumulate."""
    n, d = 2048, 64
    q, k, v = dev_qkv(n, d, torch.float32, 43)
    ro, ci = syn.bernoulli_csr(n, 0.004, seed=43)
    half = len(ci) // 2
    # split every row's columns over two masks
    rows = np.repeat(np.arange(n), np.diff(ro.numpy()))
    first = np.arange(len(ci)) % 2 == 0
    ro1 = np.concatenate([[0], np.cumsum(np.bincount(rows[first], minlength=n))])
    ro2 = np.concatenate([[0], np.cumsum(np.bincount(rows[~first], minlength=n))])
    ci1, ci2 = ci.numpy()[first], ci.numpy()[~first]
    m, l, o = state(n, d, torch.float32)
    for ro_x, ci_x in ((ro1, ci1), (ro2, ci2)):
        ro_t, ci_t = csr_tensors(ro_x, ci_x)
        plan = mods["spfa_csr"].plan(ro_t, ci_t)
        mods["spfa_csr"].forward_planned(q, k, v, ro_t, ci_t, torch.ones(len(ci_x), device=DEV), m, l, o,
                                         False, plan)
    sync()
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy())
    check(o, m, l, *ref, torch.float32)
    assert half > 0


@pytest.mark.parametrize("shuffle", [True, False])
def test_coo_plan_sorted_and_unsorted(mods, shuffle):
    n, d = 4096, 64
    ro, ci = syn.zipf_csr(n, 1.4, 0, 2048, seed=44)
    r, c = syn.coo_from_csr(ro, ci, shuffle_seed=44 if shuffle else None)
    r_t, c_t = r.to(torch.uint64).to(DEV), c.to(torch.uint32).to(DEV)
    plan = mods["spfa_coo"].plan(r_t, c_t, n)
    plan_before = plan.clone()
    for seed, dtype in ((44, torch.float32), (45, torch.bfloat16)):
        q, k, v = dev_qkv(n, d, dtype, seed)
        m, l, o = state(n, d, dtype, torch.float32)
        mods["spfa_coo"].forward_planned(q, k, v, r_t, c_t, torch.ones(c.numel(), device=DEV, dtype=dtype),
                                         m, l, o, True, plan)
        sync()
        ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy(), use_nan=True)
        check(o, m, l, *ref, dtype, state_dtype=torch.float32, dead_expect="nan")
    assert torch.equal(plan, plan_before)


def test_plans_of_empty_masks(mods):
    n, d = 64, 64
    q, k, v = dev_qkv(n, d, torch.float32, 46)
    e64 = torch.zeros(0, dtype=torch.uint64, device=DEV)
    e32 = torch.zeros(0, dtype=torch.uint32, device=DEV)
    m, l, o = state(n, d, torch.float32)
    plan = mods["spfa_coo"].plan(e64, e32, n)
    mods["spfa_coo"].forward_planned(q, k, v, e64, e32, torch.zeros(0, device=DEV), m, l, o, True, plan)
    sync()
    assert torch.isnan(o).all() and torch.all(l == 0)
    ro_t = torch.zeros(n + 1, dtype=torch.uint64, device=DEV)
    m, l, o = state(n, d, torch.float32)
    plan = mods["spfa_csr"].plan(ro_t, e32)
    mods["spfa_csr"].forward_planned(q, k, v, ro_t, e32, torch.zeros(0, device=DEV), m, l, o, True, plan)
    sync()
    assert torch.isnan(o).all() and torch.all(l == 0)


# ------------------------------------------------------------------ COO
@pytest.mark.parametrize("row_dtype", [torch.uint64, torch.int64, torch.int32])
def test_coo_unsorted_equals_csr(mods, row_dtype):
    n, d = 4096, 64
    q, k, v = dev_qkv(n, d, torch.float32, 16)
    ro, ci = syn.zipf_csr(n, 1.4, 0, 2048, seed=16)
    r, c = syn.coo_from_csr(ro, ci, shuffle_seed=16)
    m, l, o = state(n, d, torch.float32)
    mods["spfa_coo"].forward(q, k, v, r.to(row_dtype).to(DEV), c.to(torch.uint32).to(DEV),
                             torch.ones(c.numel(), device=DEV), m, l, o, True)
    sync()
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy(), use_nan=True)
    check(o, m, l, *ref, torch.float32, dead_expect="nan")
    o2, m2, l2 = run_csr(mods, q, k, v, ro, ci, True)
    assert torch.allclose(torch.nan_to_num(o), torch.nan_to_num(o2), atol=2e-5)


@pytest.mark.parametrize("row_dtype", [torch.uint64, torch.int32])
def test_coo_sorted_by_row_takes_the_callers_columns(mods, row_dtype):
    """Row-sorted entries (the reference's contract), columns in any order inside a row, leading,
    inner and trailing empty rows."""
    n, d = 3000, 64
    q, k, v = dev_qkv(n, d, torch.float32, 19)
    g = torch.Generator().manual_seed(19)
    deg = torch.randint(0, 50, (n,), generator=g)
    deg[:7] = 0
    deg[100:300] = 0
    deg[-40:] = 0
    deg[1234] = 1500
    ro, ci = syn.csr_from_degrees(deg, n, g, "cpu", force_diagonal=False)
    r, c = syn.coo_from_csr(ro, ci)
    # shuffle the columns inside every row: still sorted by row
    key = r.double() + torch.rand(c.numel(), generator=g).double() * 0.5
    order = torch.argsort(key)
    r, c = r[order].contiguous(), c[order].contiguous()
    assert torch.all(r[1:] >= r[:-1])
    m, l, o = state(n, d, torch.float32)
    mods["spfa_coo"].forward(q, k, v, r.to(row_dtype).to(DEV), c.to(torch.uint32).to(DEV),
                             torch.ones(c.numel(), device=DEV), m, l, o, True)
    sync()
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy(), use_nan=True)
    check(o, m, l, *ref, torch.float32, dead_expect="nan")


def test_coo_power_law_with_many_empty_rows(mods):
    n, d = 65536, 64
    q, k, v = dev_qkv(n, d, torch.float32, 17)
    r, c = syn.zipf_coo(n, 600_000, 1.3, seed=17)
    m, l, o = state(n, d, torch.float32)
    mods["spfa_coo"].forward(q, k, v, r.to(torch.uint64).to(DEV), c.to(torch.uint32).to(DEV),
                             torch.ones(c.numel(), device=DEV), m, l, o, False)
    sync()
    ref = c_oracle.coo(np64(q), np64(k), np64(v), r.numpy(), c.numpy())
    check(o, m, l, *ref, torch.float32)


@pytest.mark.parametrize("case,n,n_k,nnz,d,dtype", [
    ("two_windows", 2048, 2048, 3_000_000, 64, torch.float32),       # 64 buckets of ~47 K entries
    ("beyond_registers", 2048, 2048, 8_000_000, 64, torch.float32),  # ~125 K entries per bucket
    ("direct", 256, 256, 6_000_000, 64, torch.float32),              # 16 buckets of ~375 K entries
    ("one_heavy_row", 2048, 2048, 3_000_000, 64, torch.float32),     # 60 % of the entries in one row
    # 1465 buckets of 2048 rows; row in bucket and column do not fit 32 bits together
    ("many_buckets_pairs", 3_000_000, 3_000_000, 2_000_000, 32, torch.bfloat16),
    # 1465 buckets of 1024 rows, 32-bit entries between the passes
    ("many_buckets_packed", 1_500_000, 65536, 2_000_000, 32, torch.bfloat16),
])
def test_coo_unsorted_bucket_shapes(mods, case, n, n_k, nnz, d, dtype):
    """Unsorted entries whose row buckets have the sizes that the bucketing pre-pass treats
    differently (one or several staged windows, entries beyond those kept in registers, buckets too
    large to stage, a bucket dominated by one row, the largest number of buckets), a number of
    entries that is no multiple of a tile, repeated entries: the attention result against the
    same mask sorted by torch and given as CSR, and to_csr against that sort entry by entry."""
    g = torch.Generator(device=DEV)
    g.manual_seed(61)
    nnz += 12345
    r = torch.randint(0, n, (nnz,), generator=g, device=DEV, dtype=torch.int64)
    c = torch.randint(0, n_k, (nnz,), generator=g, device=DEV, dtype=torch.int64)
    if case == "one_heavy_row":
        r[torch.rand(nnz, generator=g, device=DEV) < 0.6] = 5
    q, k, v = dev_qkv(n, d, dtype, 61, n_k=n_k)
    r_t, c_t = r.to(torch.uint64), c.to(torch.uint32)
    val = torch.ones(nnz, device=DEV, dtype=dtype)
    m, l, o = state(n, d, dtype, torch.float32)
    mods["spfa_coo"].forward(q, k, v, r_t, c_t, val, m, l, o, False)
    sync()
    order = torch.argsort(r, stable=True)
    deg = torch.bincount(r, minlength=n)
    ro = torch.zeros(n + 1, dtype=torch.int64, device=DEV)
    ro[1:] = torch.cumsum(deg, 0)
    m2, l2, o2 = state(n, d, dtype, torch.float32)
    mods["spfa_csr"].forward(q, k, v, ro.to(torch.uint64), c[order].to(torch.uint32).contiguous(), val, m2, l2, o2,
                             False)
    sync()
    assert torch.equal(m, m2)
    assert torch.allclose(l, l2, rtol=1e-4, atol=0)
    # (the order of a row's columns differs, and with it the rounding: one unit of a bf16 output)
    atol, rtol = (2e-5, 1e-3) if dtype == torch.float32 else (2e-3, 8e-3)
    assert torch.allclose(o.float(), o2.float(), atol=atol, rtol=rtol)
    ro3, ci3 = mods["spfa_coo"].to_csr(r_t, c_t, n)
    sync()
    assert torch.equal(ro3.to(torch.int64), ro)
    rows3 = torch.repeat_interleave(torch.arange(n, device=DEV), deg)
    assert torch.equal(torch.sort(rows3 * n_k + ci3.to(torch.int64))[0], torch.sort(r * n_k + c)[0])


def test_coo_empty_mask(mods):
    n, d = 64, 64
    q, k, v = dev_qkv(n, d, torch.float32, 18)
    m, l, o = state(n, d, torch.float32)
    e64 = torch.zeros(0, dtype=torch.uint64, device=DEV)
    e32 = torch.zeros(0, dtype=torch.uint32, device=DEV)
    mods["spfa_coo"].forward(q, k, v, e64, e32, torch.zeros(0, device=DEV), m, l, o, True)
    sync()
    assert torch.isnan(o).all() and torch.all(l == 0) and torch.all(torch.isneginf(m))


# ------------------------------------------------------------------ implicit masks
@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 64), (torch.float16, 32),
                                     (torch.bfloat16, 128), (torch.float32, 48), (torch.float32, 128),
                                     (torch.bfloat16, 32), (torch.bfloat16, 256), (torch.float16, 256),
                                     (torch.float32, 32), (torch.float32, 256), (torch.float32, 96),
                                     (torch.bfloat16, 96), (torch.float16, 160), (torch.float32, 160),
                                     (torch.bfloat16, 192), (torch.float32, 192), (torch.float16, 224),
                                     (torch.float32, 224)])
@pytest.mark.parametrize("n,w", [(1000, 0), (1000, 1), (1000, 128), (777, 776), (4096, 300), (130, 20)])
def test_local(mods, dtype, d, n, w):
    q, k, v = dev_qkv(n, d, dtype, 30)
    m, l, o = state(n, d, dtype, torch.float32)
    mods["spfa_local"].forward(q, k, v, m, l, o, w)
    sync()
    ref = c_oracle.local(np64(q), np64(k), np64(v), w)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 128), (torch.float16, 64),
                                     (torch.float32, 128), (torch.float16, 32), (torch.bfloat16, 256),
                                     (torch.float32, 32), (torch.float32, 96), (torch.bfloat16, 160),
                                     (torch.float16, 192), (torch.float32, 224)])
@pytest.mark.parametrize("n,w,dil", [(1000, 10, 2), (1000, 0, 3), (1000, 999, 0), (1001, 100, 1),
                                     (2048, 256, 2), (300, 299, 6), (5000, 40, 4)])
def test_local_1d_dilated(mods, dtype, d, n, w, dil):
    q, k, v = dev_qkv(n, d, dtype, 31, scale=0.5)
    m, l, o = state(n, d, dtype, torch.float32)
    mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, w, dil)
    sync()
    ref = c_oracle.local_1d_dilated(np64(q), np64(k), np64(v), w, dil)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 128), (torch.float16, 64),
                                     (torch.float32, 128), (torch.bfloat16, 32), (torch.float16, 256),
                                     (torch.float32, 32), (torch.bfloat16, 96), (torch.float32, 160),
                                     (torch.float32, 192), (torch.float16, 224)])
@pytest.mark.parametrize("n,block,dil", [(1024, 16, 0), (1024, 16, 1), (1024, 256, 2), (1000, 1000, 3),
                                         (1024, 1, 0), (960, 32, 31), (2048, 2048, 0), (1200, 300, 1)])
@pytest.mark.parametrize("use_nan", [True, False])
def test_local_2d_dilated(mods, dtype, d, n, block, dil, use_nan):
    q, k, v = dev_qkv(n, d, dtype, 32, scale=0.5)
    m, l, o = state(n, d, dtype, torch.float32)
    mods["spfa_local_2d_dilated"].forward(q, k, v, m, l, o, block, dil, use_nan)
    sync()
    ref = c_oracle.local_2d_dilated(np64(q), np64(k), np64(v), block, dil, use_nan=use_nan)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32, dead_expect="nan" if use_nan else None)


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.float16, 128), (torch.bfloat16, 32),
                                     (torch.float16, 256), (torch.bfloat16, 96), (torch.float32, 32),
                                     (torch.float32, 64), (torch.float32, 128), (torch.float32, 256),
                                     (torch.float32, 40)])
@pytest.mark.parametrize("w,dil", [(1, 0), (3, 0), (6, 0), (6, 2), (10, 1), (13, 0), (15, 3)])
def test_narrow_windows_in_calls_of_many_rows(mods, dtype, d, w, dil):
    """From 32768 rows on, windows of a few candidates per row already run on the tiles (from 7
    candidates for the half types, 13 - 27 for fp32 depending on d); below, on the row-gather
    engine.  Both sides of every limit against the oracle."""
    n = 33001
    q, k, v = dev_qkv(n, d, dtype, 40, scale=0.7)
    m, l, o = state(n, d, dtype, torch.float32)
    mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, w, dil)
    sync()
    ref = c_oracle.local_1d_dilated(np64(q), np64(k), np64(v), w, dil)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)
    if dil == 0:
        m, l, o = state(n, d, dtype, torch.float32)
        mods["spfa_local"].forward(q, k, v, m, l, o, w)
        sync()
        check(o, m, l, *ref, dtype, state_dtype=torch.float32)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 4), (torch.float32, 40), (torch.float32, 100),
                                     (torch.float32, 132), (torch.float32, 252), (torch.bfloat16, 8),
                                     (torch.bfloat16, 40), (torch.float16, 80), (torch.bfloat16, 104),
                                     (torch.float16, 136), (torch.bfloat16, 200), (torch.float16, 248)])
def test_band_masks_rows_that_are_no_multiple_of_32(mods, dtype, d):
    """Rows of whole 16-byte pieces (4 floats, 8 halves) run on the tiles of the next multiple of 32
    with zero-filled operands: every band mask, ragged last tiles, dead rows, and a chained call
    whose incoming state is set for some rows and empty for others."""
    for n, w in [(1000, 128), (777, 776), (130, 0)]:
        q, k, v = dev_qkv(n, d, dtype, 33)
        m, l, o = state(n, d, dtype, torch.float32)
        mods["spfa_local"].forward(q, k, v, m, l, o, w)
        sync()
        check(o, m, l, *c_oracle.local(np64(q), np64(k), np64(v), w), dtype, state_dtype=torch.float32)
    for n, w, dil in [(1001, 100, 1), (5000, 40, 4)]:
        q, k, v = dev_qkv(n, d, dtype, 34, scale=0.5)
        m, l, o = state(n, d, dtype, torch.float32)
        mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, w, dil)
        sync()
        check(o, m, l, *c_oracle.local_1d_dilated(np64(q), np64(k), np64(v), w, dil), dtype,
              state_dtype=torch.float32)
    for n, block, dil, use_nan in [(1200, 300, 1, True), (1024, 64, 1, False), (2048, 2048, 0, True)]:
        q, k, v = dev_qkv(n, d, dtype, 35, scale=0.5)
        m, l, o = state(n, d, dtype, torch.float32)
        mods["spfa_local_2d_dilated"].forward(q, k, v, m, l, o, block, dil, use_nan)
        sync()
        ref = c_oracle.local_2d_dilated(np64(q), np64(k), np64(v), block, dil, use_nan=use_nan)
        check(o, m, l, *ref, dtype, state_dtype=torch.float32, dead_expect="nan" if use_nan else None)
    # a random mask outside the window first (half of its rows empty), then the window on top
    n, w = 900, 60
    rng = np.random.default_rng(36)
    band = so.mask_local_dense(n, w)
    rand = (rng.random((n, n)) < 0.03) & ~band
    rand[rng.random(n) < 0.5] = False
    q, k, v = dev_qkv(n, d, dtype, 36)
    ro, ci = so.csr_from_dense(rand)
    o, m, l = run_csr(mods, q, k, v, ro, ci, False, st=state(n, d, dtype, torch.float32))
    mods["spfa_local"].forward(q, k, v, m, l, o, w)
    sync()
    check(o, m, l, *so.dense_masked_attention(np64(q), np64(k), np64(v), band | rand), dtype,
          state_dtype=torch.float32)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.float32, 128), (torch.bfloat16, 64),
                                     (torch.float16, 128), (torch.float16, 32), (torch.bfloat16, 256),
                                     (torch.float32, 32), (torch.float32, 96), (torch.bfloat16, 192)])
@pytest.mark.parametrize("kind,n,p1,p2", [("local", 20011, 33, 0), ("local", 20011, 0, 0), ("local", 17000, 700, 0),
                                          ("d1", 20011, 70, 2), ("d1", 20000, 1500, 1), ("d1", 33333, 129, 4),
                                          ("d2", 20480, 128, 1), ("d2", 42000, 300, 2), ("d2", 30000, 200, 0)])
def test_band_masks_with_a_few_hundred_tiles(mods, dtype, d, kind, n, p1, p2):
    """Band masks with 130 .. 500 query tiles: whole tiles only (the kernels whose loads write LDS directly),
    sequence ends inside a tile, windows narrower and wider than a tile; then a second call on top of the first."""
    q, k, v = dev_qkv(n, d, dtype, 41, scale=0.5)
    m, l, o = state(n, d, dtype, torch.float32)
    if kind == "local":
        call = lambda: mods["spfa_local"].forward(q, k, v, m, l, o, p1)
        ref = c_oracle.local(np64(q), np64(k), np64(v), p1)
    elif kind == "d1":
        call = lambda: mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, p1, p2)
        ref = c_oracle.local_1d_dilated(np64(q), np64(k), np64(v), p1, p2)
    else:
        call = lambda: mods["spfa_local_2d_dilated"].forward(q, k, v, m, l, o, p1, p2, False)
        ref = c_oracle.local_2d_dilated(np64(q), np64(k), np64(v), p1, p2, use_nan=False)
    call()
    sync()
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)
    l1, o1 = l.clone(), o.clone()
    call()
    sync()
    assert torch.allclose(l, 2 * l1, rtol=1e-5)
    assert torch.allclose(o.float(), o1.float(), atol=2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.float16, 128), (torch.float16, 32), (torch.float32, 64)])
@pytest.mark.parametrize("kind,n,p1,p2", [("local", 66098, 40, 0), ("local", 65700, 300, 0), ("d1", 131500, 70, 1),
                                          ("d1", 66000, 20, 2)])
def test_band_masks_with_a_few_tiles_beyond_a_full_round(mods, dtype, d, kind, n, p1, p2):
    """Query tiles a few more than the device holds at once (512 at two workgroups per CU of 256): the
    tiles of the last, sparsely filled round are shared out to four workgroups each, whose wavefronts
    deal the key tiles among themselves and fold their partial results.  The last tile of a
    subsequence is partly filled; then a second call on top of the first."""
    q, k, v = dev_qkv(n, d, dtype, 43, scale=0.5)
    m, l, o = state(n, d, dtype, torch.float32)
    if kind == "local":
        call = lambda: mods["spfa_local"].forward(q, k, v, m, l, o, p1)
        ref = c_oracle.local(np64(q), np64(k), np64(v), p1)
    else:
        call = lambda: mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, p1, p2)
        ref = c_oracle.local_1d_dilated(np64(q), np64(k), np64(v), p1, p2)
    call()
    sync()
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)
    l1, o1 = l.clone(), o.clone()
    call()
    sync()
    assert torch.allclose(l, 2 * l1, rtol=1e-5)
    assert torch.allclose(o.float(), o1.float(), atol=2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.float32, 128), (torch.bfloat16, 128)])
def test_band_masks_batch_with_a_few_hundred_tiles(mods, dtype, d):
    """Three heads of 9000 tokens in one call: 213 whole tiles over the stacked problems."""
    n, shape = 9000, (3,)
    cases = [("spfa_local", (50,), lambda a, b, c: c_oracle.local(a, b, c, 50)),
             ("spfa_local_1d_dilated", (200, 2), lambda a, b, c: c_oracle.local_1d_dilated(a, b, c, 200, 2)),
             ("spfa_local_2d_dilated", (250, 1, False), lambda a, b, c: c_oracle.local_2d_dilated(a, b, c, 250, 1, use_nan=False))]
    for name, args, ref_fn in cases:
        q, k, v, m, l, o = _stacked(n, d, dtype, shape, 57)
        mods[name].forward(q, k, v, m, l, o, *args)
        sync()
        _check_heads(q, k, v, o, m, l, ref_fn, dtype)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 64), (torch.float16, 128),
                                     (torch.float32, 128), (torch.float32, 32), (torch.bfloat16, 32),
                                     (torch.float16, 256), (torch.bfloat16, 256), (torch.float32, 256),
                                     (torch.float32, 96), (torch.bfloat16, 96), (torch.float16, 160),
                                     (torch.float32, 192), (torch.bfloat16, 224), (torch.float32, 224)])
@pytest.mark.parametrize("n,n_globs,w", [(1024, 4, 10), (1024, 1, 0), (1024, 64, 64), (1500, 100, 1499),
                                         (1024, 1024, 3), (8192, 16, 100), (3000, 200, 7)])
def test_global_no_local(mods, dtype, d, n, n_globs, w):
    q, k, v = dev_qkv(n, d, dtype, 33)
    g = syn.global_indices(n, n_globs, seed=33)
    m, l, o = state(n, d, dtype, torch.float32)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g.to(DEV), w)
    sync()
    ref = c_oracle.global_no_local(np64(q), np64(k), np64(v), g.numpy(), w)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)


@pytest.mark.parametrize("dtype,d", [(torch.float32, 4), (torch.float32, 40), (torch.float32, 100),
                                     (torch.float32, 200), (torch.float32, 252), (torch.bfloat16, 8),
                                     (torch.bfloat16, 40), (torch.float16, 80), (torch.bfloat16, 104),
                                     (torch.float16, 136), (torch.bfloat16, 200), (torch.float16, 248)])
def test_global_no_local_rows_that_are_no_multiple_of_32(mods, dtype, d):
    """Rows of whole 16-byte pieces on the tiles of the next multiple of 32 (zero-filled operands,
    partial results and merge at the real row length): one tile of listed tokens and several, a
    chained call on a state that the window call has set, a batch, and the one-call composite."""
    for n, n_globs, w in [(1024, 4, 10), (1500, 100, 1499), (3000, 200, 7), (8192, 16, 100)]:
        q, k, v = dev_qkv(n, d, dtype, 37)
        g = syn.global_indices(n, n_globs, seed=37)
        m, l, o = state(n, d, dtype, torch.float32)
        mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g.to(DEV), w)
        sync()
        check(o, m, l, *c_oracle.global_no_local(np64(q), np64(k), np64(v), g.numpy(), w), dtype,
              state_dtype=torch.float32)
    n, w, globs = 1100, 30, [5, 6, 400, 1099]
    g = torch.tensor(globs, dtype=torch.int32, device=DEV)
    union = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, globs, w)
    q, k, v = dev_qkv(n, d, dtype, 38)
    m, l, o = state(n, d, dtype, torch.float32)
    mods["spfa_local"].forward(q, k, v, m, l, o, w)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g, w)
    sync()
    ref = so.dense_masked_attention(np64(q), np64(k), np64(v), union)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)
    m2, l2, o2 = state(n, d, dtype, torch.float32)
    empty = torch.empty(0, device=DEV)
    mods["spfa_bigbird"].forward(q, k, v, m2, l2, o2, w, g, torch.zeros(0, dtype=torch.uint64, device=DEV),
                                 torch.zeros(0, dtype=torch.uint32, device=DEV), empty)
    sync()
    check(o2, m2, l2, *ref, dtype, state_dtype=torch.float32)
    q, k, v, m, l, o = _stacked(n, d, dtype, (3,), 39)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g, w)
    sync()
    dense = so.mask_global_no_local_dense(n, globs, w)
    _check_heads(q, k, v, o, m, l, lambda a, b, c: so.dense_masked_attention(a, b, c, dense), dtype)


def test_global_indices_need_not_be_sorted(mods):
    n, d, w = 512, 64, 7
    q, k, v = dev_qkv(n, d, torch.float32, 34)
    g = torch.tensor([400, 3, 77, 2, 300, 4], dtype=torch.int32)
    m, l, o = state(n, d, torch.float32)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g.to(DEV), w)
    sync()
    check(o, m, l, *so.dense_masked_attention(np64(q), np64(k), np64(v),
                                              so.mask_global_no_local_dense(n, g.numpy(), w)), torch.float32)


# ------------------------------------------------------------------ errors
def test_errors_keep_reference_types_and_texts(mods):
    n, d = 64, 64
    q, k, v = dev_qkv(n, d, torch.float32, 40)
    m, l, o = state(n, d, torch.float32)
    g = torch.tensor([1, 2], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match="local size specified"):
        mods["spfa_local"].forward(q, k, v, m, l, o, n)
    with pytest.raises(ValueError, match="local size specified"):
        mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, -1, 0)
    with pytest.raises(ValueError, match="atleast 0"):
        mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, 3, -1)
    with pytest.raises(ValueError, match="divisor"):
        mods["spfa_local_2d_dilated"].forward(q, k, v, m, l, o, 5, 0, True)
    with pytest.raises(ValueError, match="atleast 0"):
        mods["spfa_local_2d_dilated"].forward(q, k, v, m, l, o, 8, -1, True)
    with pytest.raises(ValueError, match="less than the block"):
        mods["spfa_local_2d_dilated"].forward(q, k, v, m, l, o, 8, 8, True)
    with pytest.raises(ValueError, match="no global tokens"):
        mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g[:0], 1)
    with pytest.raises(ValueError, match="local size specified"):
        mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g, n)
    with pytest.raises(RuntimeError, match="K must be contiguous"):
        mods["spfa_local"].forward(q, k.t().contiguous().t(), v, m, l, o, 1)
    with pytest.raises(RuntimeError, match="m must be a CUDA tensor"):
        mods["spfa_local"].forward(q, k, v, m.cpu(), l, o, 1)
    with pytest.raises(RuntimeError, match="unsupported element type"):
        mods["spfa_local"].forward(q.int(), k.int(), v.int(), m.int(), l.int(), o.int(), 1)
    with pytest.raises(RuntimeError, match="int32"):
        mods["spfa_global_no_local"].forward(q, k, v, m, l, o, g.long(), 1)
    # nothing above may have modified the state
    sync()
    assert torch.all(o == 0) and torch.all(l == 0)


def test_runs_on_a_side_stream(mods):
    n, d = 2048, 64
    q, k, v = dev_qkv(n, d, torch.float32, 41)
    ro, ci = syn.zipf_csr(n, 1.5, 1, 2048, seed=41)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        o, m, l = run_csr(mods, q, k, v, ro, ci, False)
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro.numpy(), ci.numpy())
    check(o, m, l, *ref, torch.float32)
