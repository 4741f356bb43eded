"""The benchmark configurations at their full sizes, on the GPU, checked through properties that do
not need a full-size CPU result: closed forms (window 0 => out == v, V == 1 => out == 1), the
statistics of a constant-score problem, chained == single call, COO == CSR, and the float64 oracle
on a random sample of rows."""
import math

import numpy as np
import pytest
import torch

import spfa_synth as syn
from helpers import OUT_TOL, np64
from oracle import c_oracle
from oracle import spfa_oracle as so

pytestmark = pytest.mark.gpu
DEV = "cuda"


def sample_check(q, k, v, out, m, l, rows, live_fn, dtype, expect_dead=None):
    """Oracle on the sampled rows only (live_fn(i) -> column list of row i)."""
    rows = np.asarray(rows, dtype=np.int64)
    cols = [np.asarray(live_fn(int(i)), dtype=np.int64) for i in rows]
    off = np.zeros(len(rows) + 1, dtype=np.int64)
    np.cumsum([len(c) for c in cols], out=off[1:])
    ci = np.concatenate(cols) if len(cols) else np.zeros(0, np.int64)
    sel = torch.as_tensor(rows).to(DEV)
    ref_o, ref_m, ref_l = c_oracle.csr(np64(q[sel]), np64(k), np64(v), off, ci)
    got_o, got_m, got_l = np64(out[sel]), np64(m[sel]), np64(l[sel])
    live = ref_l > 0
    assert live.any()
    err = np.abs(got_o[live] - ref_o[live]).max()
    assert err <= OUT_TOL[dtype], "max-abs %.3e" % err
    with np.errstate(divide="ignore", invalid="ignore"):
        lse_err = np.abs((got_m + np.log(got_l))[live] - (ref_m + np.log(ref_l))[live]).max()
    assert lse_err <= (1e-4 if dtype == torch.float32 else 2e-3)
    if (~live).any():
        if expect_dead == "nan":
            assert np.isnan(got_o[~live]).all()
        else:
            assert np.all(got_o[~live] == 0) and np.all(got_l[~live] == 0)


def rand_rows(n, count, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.sort(torch.randperm(n, generator=g)[:count])[0].numpy()


# ------------------------------------------------------------------ Local N=65536 d=64, fp32 / bf16
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_local_n65536(mods, dtype):
    n, d, w = 65536, 64, 128
    q, k, v = syn.qkv(n, d, dtype=dtype, device=DEV, seed=0)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local"].forward(q, k, v, m, l, o, w)
    rows = np.concatenate([[0, 1, 127, 128, 129, n - 130, n - 129, n - 128, n - 1], rand_rows(n, 150, 1)])
    sample_check(q, k, v, o, m, l, rows, lambda i: so.live_local(n, w, i), dtype)
    # closed forms at full size
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local"].forward(q, k, v, m, l, o, 0)
    assert torch.equal(o, v) and torch.all(l == 1)
    ones = torch.ones_like(v)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local"].forward(q, k, ones, m, l, o, w)
    assert torch.allclose(o.float(), torch.ones_like(o, dtype=torch.float32), atol=1e-2 if dtype != torch.float32 else 1e-5)
    # q == 0: every score is 0 -> m == 0 and l == number of live columns (closed form)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local"].forward(torch.zeros_like(q), k, v, m, l, o, w)
    i = torch.arange(n, device=DEV)
    cnt = (torch.clamp(i + w + 1, max=n) - torch.clamp(i - w, min=0)).float()
    assert torch.all(m == 0) and torch.equal(l, cnt)
    assert int(l.sum().item()) == so.nnz_local(n, w)


# ------------------------------------------------------------------ CSR N=131072 d=64 fp32, Zipf(1.5)
def test_csr_zipf_n131072(mods):
    n, d = 131072, 64
    q, k, v = syn.qkv(n, d, device=DEV, seed=0)
    ro, ci = syn.zipf_csr(n, 1.5, 1, 4096, device=DEV, seed=0)
    ro_t, ci_t = ro.to(torch.uint64), ci.to(torch.uint32)
    val = torch.empty(ci.numel(), device=DEV)
    m, l, o = syn.fresh_state(n, d, device=DEV)
    mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, False)
    ro_c, ci_c = ro.cpu().numpy(), ci.cpu().numpy()
    deg = ro_c[1:] - ro_c[:-1]
    assert deg.min() >= 1 and deg.max() == 4096
    # sample every length class: shortest, longest, around the in-place limit, random
    rows = np.concatenate([np.nonzero(deg == 1)[0][:20], np.nonzero(deg == 4096)[0][:20],
                           np.nonzero((deg >= 14) & (deg <= 18))[0][:20], np.nonzero((deg >= 30) & (deg <= 36))[0][:20],
                           np.nonzero((deg > 250) & (deg < 520))[0][:20], rand_rows(n, 100, 2)])
    sample_check(q, k, v, o, m, l, rows, lambda i: ci_c[ro_c[i]:ro_c[i + 1]], torch.float32)
    # q == 0 -> l == row length exactly, m == 0
    m2, l2, o2 = syn.fresh_state(n, d, device=DEV)
    mods["spfa_csr"].forward(torch.zeros_like(q), k, v, ro_t, ci_t, val, m2, l2, o2, False)
    assert torch.all(m2 == 0) and torch.equal(l2, (ro[1:] - ro[:-1]).float())
    # the same mask as shuffled COO gives the same result
    r, c = syn.coo_from_csr(ro, ci, shuffle_seed=3)
    m3, l3, o3 = syn.fresh_state(n, d, device=DEV)
    mods["spfa_coo"].forward(q, k, v, r.to(torch.uint64), c.to(torch.uint32), val, m3, l3, o3, False)
    assert torch.allclose(o3, o, atol=2e-5) and torch.allclose(m3, m, atol=1e-6)
    assert torch.allclose(l3, l, rtol=1e-5)
    # two disjoint halves chained == one call
    keep = torch.rand(ci.numel(), device=DEV, generator=torch.Generator(device=DEV).manual_seed(4)) < 0.5
    rows_of = torch.repeat_interleave(torch.arange(n, device=DEV), ro[1:] - ro[:-1])
    m4, l4, o4 = syn.fresh_state(n, d, device=DEV)
    for part in (keep, ~keep):
        cnt = torch.bincount(rows_of[part], minlength=n)
        off = torch.zeros(n + 1, dtype=torch.int64, device=DEV)
        off[1:] = torch.cumsum(cnt, 0)
        cp = ci[part].to(torch.uint32)
        mods["spfa_csr"].forward(q, k, v, off.to(torch.uint64), cp, torch.empty(cp.numel(), device=DEV), m4, l4, o4, False)
    assert torch.allclose(o4, o, atol=2e-5) and torch.allclose(m4, m, atol=1e-6)
    assert torch.allclose(l4, l, rtol=1e-5)


# ------------------------------------------------------------------ CSR with more than 2^31 entries
def test_csr_more_than_2_31_entries(mods):
    """64-bit row offsets that really need their upper half (the reference indexes its rows with
    size_t offsets, Sparse_FlashAttention_CSR/sp_flatt_csr_kernel.cu:29-30): 2^20 rows of 2048 to
    2176 distinct columns each, 2.2e9 entries, against 4096 keys at d = 16 in bf16.  q = 0 gives
    l == row length exactly and out == the mean of the row's V rows; sampled rows of a call with
    random q against the oracle, among them the rows whose entries straddle position 2^31."""
    n_q, n_k, d = 1 << 20, 4096, 16
    dtype = torch.bfloat16
    free = torch.cuda.mem_get_info()[0]
    if free < 40 * (1 << 30):
        pytest.skip("needs about 40 GiB of free device memory for the mask, has %.1f GiB" % (free / 2**30))
    rows = torch.arange(n_q, device=DEV, dtype=torch.int64)
    deg = 2048 + rows % 129
    ro = torch.zeros(n_q + 1, dtype=torch.int64, device=DEV)
    ro[1:] = torch.cumsum(deg, 0)
    nnz = int(ro[-1])
    assert nnz > (1 << 31)
    ci = torch.empty(nnz, dtype=torch.int32, device=DEV)
    step = 1 << 15
    for a in range(0, n_q, step):  # row i lists (17 i + j) mod n_k, j < deg[i]: distinct, unsorted
        b = min(n_q, a + step)
        r = torch.repeat_interleave(rows[a:b], deg[a:b])
        j = torch.arange(int(ro[a]), int(ro[b]), device=DEV, dtype=torch.int64) - ro[r]
        ci[int(ro[a]):int(ro[b])] = ((17 * r + j) % n_k).to(torch.int32)
        del r, j
    ro_t, ci_t = ro.to(torch.uint64), ci.view(torch.uint32)
    val = torch.empty(0, device=DEV, dtype=dtype)
    q, k, v = syn.qkv(n_q, d, dtype=dtype, device=DEV, seed=0, n_k=n_k)

    def live(i):
        return (17 * i + np.arange(2048 + i % 129)) % n_k

    # q == 0: m == 0, l == row length, out == mean of the listed V rows
    m, l, o = syn.fresh_state(n_q, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_csr"].forward(torch.zeros_like(q), k, v, ro_t, ci_t, val, m, l, o, False)
    assert torch.all(m == 0) and torch.equal(l, deg.float())
    ro_c = ro.cpu().numpy()
    cross = int(np.searchsorted(ro_c, 1 << 31, side="right")) - 1  # the row that holds entry 2^31
    sample = np.unique(np.concatenate([[0, 1, cross - 1, cross, cross + 1, n_q - 2, n_q - 1],
                                       rand_rows(n_q, 24, 5)]))
    vv = np64(v)
    for i in sample:
        want = vv[live(int(i))].mean(axis=0)
        assert np.abs(np64(o[int(i)]) - want).max() <= 2e-3, int(i)
    # random q: sampled rows against the oracle
    m, l, o = syn.fresh_state(n_q, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, False)
    sample_check(q, k, v, o, m, l, sample, live, dtype)


# ------------------------------------------------------------------ dilated masks N=262144 d=128 bf16
def test_local_1d_dilated_n262144(mods):
    n, d, w, dil = 262144, 128, 256, 2
    dtype = torch.bfloat16
    q, k, v = syn.qkv(n, d, dtype=dtype, device=DEV, seed=0, scale=0.5)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, w, dil)
    rows = np.concatenate([[0, 1, 2, 3, 767, 768, 769, n - 770, n - 3, n - 2, n - 1], rand_rows(n, 100, 5)])
    sample_check(q, k, v, o, m, l, rows, lambda i: so.live_local_1d_dilated(n, w, dil, i), dtype)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local_1d_dilated"].forward(torch.zeros_like(q), k, v, m, l, o, w, dil)
    assert torch.all(m == 0)
    assert int(l.double().sum().item()) == so.nnz_local_1d_dilated(n, w, dil)


@pytest.mark.parametrize("case", ["local_d64", "dilated_d128"])
def test_band_fp32_shared_tail_tiles(mods, case):
    """fp32 band masks whose tile count is a few over a multiple of the resident workgroups: the
    left-over tiles are shared by four workgroups each.  Rows of those tiles (the end of the last
    subsequence) and of ordinary ones, against the oracle."""
    dtype = torch.float32
    if case == "local_d64":
        n, d, w = 128 * 515 + 40, 64, 96
        call = lambda q, k, v, m, l, o: mods["spfa_local"].forward(q, k, v, m, l, o, w)
        live = lambda i: so.live_local(n, w, i)
        nnz = so.nnz_local(n, w)
    else:
        n, d, w, dil = 262144, 128, 256, 2
        call = lambda q, k, v, m, l, o: mods["spfa_local_1d_dilated"].forward(q, k, v, m, l, o, w, dil)
        live = lambda i: so.live_local_1d_dilated(n, w, dil, i)
        nnz = so.nnz_local_1d_dilated(n, w, dil)
    q, k, v = syn.qkv(n, d, dtype=dtype, device=DEV, seed=3, scale=0.5)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    call(q, k, v, m, l, o)
    rows = np.concatenate([np.arange(n - 600, n, 7), [0, 1, 2, n - 3, n - 2, n - 1], rand_rows(n, 60, 9)])
    sample_check(q, k, v, o, m, l, np.unique(rows), live, dtype)
    # a second call on top of the first doubles l and leaves out where it was
    m2, l2, o2 = m.clone(), l.clone(), o.clone()
    call(q, k, v, m2, l2, o2)
    assert torch.allclose(l2, 2 * l, rtol=1e-5) and torch.allclose(o2, o, atol=2e-5)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    call(torch.zeros_like(q), k, v, m, l, o)
    assert torch.all(m == 0) and int(l.double().sum().item()) == nnz


@pytest.mark.parametrize("use_nan", [True, False])
def test_local_2d_dilated_n262144(mods, use_nan):
    n, d, block, dil = 262144, 128, 256, 2
    dtype = torch.bfloat16
    q, k, v = syn.qkv(n, d, dtype=dtype, device=DEV, seed=0, scale=0.5)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local_2d_dilated"].forward(q, k, v, m, l, o, block, dil, use_nan)
    rows = np.concatenate([[0, 1, 3, 255, 256, n - 256, n - 1], rand_rows(n, 120, 6)])
    sample_check(q, k, v, o, m, l, rows, lambda i: so.live_local_2d_dilated(n, block, dil, i), dtype,
                 expect_dead="nan" if use_nan else None)
    live = ((torch.arange(n, device=DEV) % block) % (dil + 1)) == 0
    assert int(live.sum()) == 88064
    assert torch.all(l[~live] == 0) and torch.all(torch.isneginf(m[~live]))
    assert torch.isnan(o[~live]).all() if use_nan else torch.all(o[~live] == 0)
    assert torch.isfinite(o[live].float()).all()


# ------------------------------------------------------------------ N = 1,048,576 d=64 fp32
def test_global_no_local_n1m(mods):
    n, d, g, w = 1 << 20, 64, 64, 64
    q, k, v = syn.qkv(n, d, device=DEV, seed=0)
    globs = syn.global_indices(n, g, device=DEV, seed=0)
    m, l, o = syn.fresh_state(n, d, device=DEV)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, globs, w)
    gl = globs.cpu().numpy()
    near = np.clip(np.concatenate([gl[:8] - 1, gl[:8] + 1, gl[:4] - w, gl[:4] + w + 1]), 0, n - 1)
    rows = np.unique(np.concatenate([gl[:3], near, rand_rows(n, 60, 7)]))
    sample_check(q, k, v, o, m, l, rows, lambda i: so.live_global_no_local(n, gl, w, i), torch.float32)
    # q == 0: l counts the live columns; the total is the closed-form nnz
    m, l, o = syn.fresh_state(n, d, device=DEV)
    mods["spfa_global_no_local"].forward(torch.zeros_like(q), k, v, m, l, o, globs, w)
    assert int(l.double().sum().item()) == so.nnz_global_no_local(n, gl, w)


def test_coo_zipf_n1m_50m_entries(mods):
    n, d = 1 << 20, 64
    q, k, v = syn.qkv(n, d, device=DEV, seed=0)
    r, c = syn.zipf_coo(n, 50_000_000, 1.3, device=DEV, seed=0)
    nnz = c.numel()
    assert nnz == 50_000_000
    r_t, c_t = r.to(torch.uint64), c.to(torch.uint32)
    val = torch.empty(nnz, device=DEV)
    m, l, o = syn.fresh_state(n, d, device=DEV)
    mods["spfa_coo"].forward(q, k, v, r_t, c_t, val, m, l, o, False)
    deg = torch.bincount(r, minlength=n)
    # q == 0 -> l == degree of the row (also checks that no entry was lost or duplicated)
    m2, l2, o2 = syn.fresh_state(n, d, device=DEV)
    mods["spfa_coo"].forward(torch.zeros_like(q), k, v, r_t, c_t, val, m2, l2, o2, False)
    assert torch.equal(l2, deg.float())
    # the row-sorted copy of the same entries gives the same result (other code path)
    order = torch.argsort(r, stable=True)
    m3, l3, o3 = syn.fresh_state(n, d, device=DEV)
    mods["spfa_coo"].forward(q, k, v, r[order].to(torch.uint64), c[order].to(torch.uint32), val, m3, l3, o3, False)
    assert torch.allclose(o3, o, atol=2e-5) and torch.allclose(l3, l, rtol=1e-5)
    # oracle on sampled rows (heaviest rows, empty rows, random rows)
    heavy = torch.topk(deg, 4)[1].cpu().numpy()
    empty = torch.nonzero(deg == 0)[:4, 0].cpu().numpy()
    rows = np.unique(np.concatenate([heavy, empty, rand_rows(n, 40, 8)]))
    sample_check(q, k, v, o, m, l, rows, lambda i: c[r == i].cpu().numpy(), torch.float32)


# ------------------------------------------------------------------ gradients at the full sizes
def _grad_properties(q, k, v, d_out, l, dq, dk, dv, dtype):
    """Two identities that hold for any mask: every live row's weights sum to one, so the columns
    of dV add up to those of dO over the live rows; and sum_i q_i.dQ_i == sum_j k_j.dK_j (both are
    sum_ij dS_ij s_ij)."""
    live = (l > 0).double().unsqueeze(-1)
    want = (d_out.double() * live).sum(dim=-2)
    got = dv.double().sum(dim=-2)
    scale = float(d_out.double().abs().sum(dim=-2).max())
    tol = 1e-6 if dtype == torch.float32 else 3e-3
    assert float((got - want).abs().max()) <= tol * scale
    a = float((q.double() * dq.double()).sum())
    b = float((k.double() * dk.double()).sum())
    ref = float((q.double() * dq.double()).abs().sum())
    assert abs(a - b) <= (1e-5 if dtype == torch.float32 else 2e-2) * ref


def _dq_sample_check(q, k, v, d_out, dq, rows, live_fn, dtype):
    rows = np.asarray(rows, dtype=np.int64)
    cols = [np.asarray(live_fn(int(i)), dtype=np.int64) for i in rows]
    off = np.zeros(len(rows) + 1, dtype=np.int64)
    np.cumsum([len(c) for c in cols], out=off[1:])
    ci = np.concatenate(cols)
    sel = torch.as_tensor(rows).to(DEV)
    ref = so.rowwise_query_gradient(np64(q[sel]), np64(k), np64(v), np64(d_out[sel]), off, ci)
    err = np.abs(np64(dq[sel]) - ref).max()
    assert err <= (2e-4 if dtype == torch.float32 else 3e-2) * max(1.0, np.abs(ref).max()), err


def test_backward_csr_zipf_n131072(mods):
    n, d = 131072, 64
    q, k, v = syn.qkv(n, d, device=DEV, seed=0)
    ro, ci = syn.zipf_csr(n, 1.5, 1, 4096, device=DEV, seed=0)
    ro_t, ci_t = ro.to(torch.uint64), ci.to(torch.uint32)
    val = torch.empty(0, device=DEV)
    m, l, o = syn.fresh_state(n, d, device=DEV)
    mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, False)
    d_out = torch.randn(n, d, device=DEV, generator=torch.Generator(device=DEV).manual_seed(5))
    dq, dk, dv = (torch.zeros(n, d, device=DEV) for _ in range(3))
    mods["spfa_csr"].backward(q, k, v, ro_t, ci_t, val, m, l, o, d_out, dq, dk, dv)
    torch.cuda.synchronize()
    _grad_properties(q, k, v, d_out, l, dq, dk, dv, torch.float32)
    ro_c, ci_c = ro.cpu().numpy(), ci.cpu().numpy()
    deg = ro_c[1:] - ro_c[:-1]
    rows = np.concatenate([np.nonzero(deg == 1)[0][:10], np.nonzero(deg == 4096)[0][:6],
                           np.nonzero((deg > 1000) & (deg < 1100))[0][:6], rand_rows(n, 60, 6)])
    _dq_sample_check(q, k, v, d_out, dq, rows, lambda i: ci_c[ro_c[i]:ro_c[i + 1]], torch.float32)
    # key side on a sample of columns: the rows that attend column j, weighted with the forward
    # pass's own statistics, in float64
    rows_of = torch.repeat_interleave(torch.arange(n, device=DEV), ro[1:] - ro[:-1])
    lse = (m.double() + l.double().log())
    delta = (d_out.double() * o.double()).sum(dim=1)
    for j in rand_rows(n, 12, 7):
        att = rows_of[ci == int(j)]
        s = (q[att].double() @ k[j].double()) / math.sqrt(d)
        p = torch.exp(s - lse[att])
        ds = p * (d_out[att].double() @ v[j].double() - delta[att]) / math.sqrt(d)
        assert float((dv[j].double() - p @ d_out[att].double()).abs().max()) <= 2e-4
        assert float((dk[j].double() - ds @ q[att].double()).abs().max()) <= 2e-4
    # the mask transposed once and handed in gives the same gradients (up to summation order)
    t_ro, t_ci = mods["spfa_csr"].transpose(ro_t, ci_t, n)
    dq2, dk2, dv2 = (torch.zeros(n, d, device=DEV) for _ in range(3))
    mods["spfa_csr"].backward(q, k, v, ro_t, ci_t, val, m, l, o, d_out, dq2, dk2, dv2, t_ro, t_ci)
    # (rows longer than a segment are added up in whatever order their pieces finish)
    assert torch.allclose(dq2, dq, atol=1e-4)
    assert torch.allclose(dk2, dk, atol=1e-4) and torch.allclose(dv2, dv, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_backward_local_n65536(mods, dtype):
    n, d, w = 65536, 64, 128
    q, k, v = syn.qkv(n, d, dtype=dtype, device=DEV, seed=0)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local"].forward(q, k, v, m, l, o, w)
    d_out = torch.randn(n, d, device=DEV, generator=torch.Generator(device=DEV).manual_seed(8)).to(dtype)
    dq, dk, dv = (torch.zeros(n, d, device=DEV) for _ in range(3))
    mods["spfa_local"].backward(q, k, v, m, l, o, w, d_out, dq, dk, dv)
    torch.cuda.synchronize()
    _grad_properties(q, k, v, d_out, l, dq, dk, dv, dtype)
    rows = np.concatenate([[0, 1, w, n - 1, n - w - 1], rand_rows(n, 60, 9)])
    _dq_sample_check(q, k, v, d_out, dq, rows, lambda i: so.live_local(n, w, i), dtype)
    # the mask is symmetric: swapping the roles (q <-> k, d_out -> v's place) is not an identity,
    # but window 0 is a closed form: p == 1, so dV == dO and dQ == dK == 0
    m0, l0, o0 = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_local"].forward(q, k, v, m0, l0, o0, 0)
    dq0, dk0, dv0 = (torch.zeros(n, d, device=DEV) for _ in range(3))
    mods["spfa_local"].backward(q, k, v, m0, l0, o0, 0, d_out, dq0, dk0, dv0)
    assert torch.allclose(dv0, d_out.float(), atol=1e-5)
    assert float(dq0.abs().max()) <= (1e-4 if dtype == torch.float32 else 0.3) and float(dk0.abs().max()) <= (
        1e-4 if dtype == torch.float32 else 0.3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["d1", "d2"])
def test_backward_dilated_d128(mods, kind, dtype):
    """Gradient tiles at d = 128 (one workgroup per CU, accumulators beyond 256 registers) on a few hundred tiles:
    sampled dQ rows against the oracle, dK / dV of sampled columns from the forward pass's own statistics in float64
    (the masks are symmetric: the rows that attend column j are live(j)), and the two identities."""
    d = 128
    if kind == "d1":
        n, w, dil = 40000, 200, 2
        fwd = lambda *a: mods["spfa_local_1d_dilated"].forward(*a, w, dil)
        bwd = lambda q, k, v, m, l, o, *g: mods["spfa_local_1d_dilated"].backward(q, k, v, m, l, o, w, dil, *g)
        live = lambda i: so.live_local_1d_dilated(n, w, dil, i)
    else:
        n, block, dil = 40000, 400, 1
        fwd = lambda *a: mods["spfa_local_2d_dilated"].forward(*a, block, dil, False)
        bwd = lambda q, k, v, m, l, o, *g: mods["spfa_local_2d_dilated"].backward(q, k, v, m, l, o, block, dil, *g)
        live = lambda i: so.live_local_2d_dilated(n, block, dil, i)
    q, k, v = syn.qkv(n, d, dtype=dtype, device=DEV, seed=2, scale=0.5)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    fwd(q, k, v, m, l, o)
    d_out = torch.randn(n, d, device=DEV, generator=torch.Generator(device=DEV).manual_seed(12)).to(dtype)
    dq, dk, dv = (torch.zeros(n, d, device=DEV) for _ in range(3))
    bwd(q, k, v, m, l, o, d_out, dq, dk, dv)
    torch.cuda.synchronize()
    _grad_properties(q, k, v, d_out, l, dq, dk, dv, dtype)
    rows = np.concatenate([[0, 2, 3, n - 3, n - 1], rand_rows(n, 40, 13)])
    rows = np.asarray([i for i in rows if len(live(int(i)))])
    _dq_sample_check(q, k, v, d_out, dq, rows, live, dtype)
    lse = m.double() + l.double().log()
    delta = (d_out.double() * o.double()).sum(dim=1)
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    for j in rand_rows(n, 10, 14):
        att = torch.as_tensor(np.asarray(live(int(j)), dtype=np.int64)).to(DEV)
        if att.numel() == 0:
            assert float(dk[j].abs().max()) == 0 and float(dv[j].abs().max()) == 0
            continue
        sco = (q[att].double() @ k[j].double()) / math.sqrt(d)
        pw = torch.exp(sco - lse[att])
        ds = pw * (d_out[att].double() @ v[j].double() - delta[att]) / math.sqrt(d)
        want_v, want_k = pw @ d_out[att].double(), ds @ q[att].double()
        assert float((dv[j].double() - want_v).abs().max()) <= tol * max(1.0, float(want_v.abs().max()))
        assert float((dk[j].double() - want_k).abs().max()) <= tol * max(1.0, float(want_k.abs().max()))


def test_backward_global_no_local_n1m(mods):
    n, d, g, w = 1 << 20, 64, 64, 64
    q, k, v = syn.qkv(n, d, device=DEV, seed=0)
    globs = syn.global_indices(n, g, device=DEV, seed=0)
    m, l, o = syn.fresh_state(n, d, device=DEV)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, globs, w)
    d_out = torch.randn(n, d, device=DEV, generator=torch.Generator(device=DEV).manual_seed(10))
    dq, dk, dv = (torch.zeros(n, d, device=DEV) for _ in range(3))
    mods["spfa_global_no_local"].backward(q, k, v, m, l, o, globs, w, d_out, dq, dk, dv)
    torch.cuda.synchronize()
    _grad_properties(q, k, v, d_out, l, dq, dk, dv, torch.float32)
    gl = globs.cpu().tolist()
    rows = np.concatenate([np.asarray(gl[:3]), rand_rows(n, 40, 11)])
    _dq_sample_check(q, k, v, d_out, dq, rows, lambda i: so.live_global_no_local(n, gl, w, i), torch.float32)


def test_backward_coo_zipf_n1m_50m_entries(mods):
    """Unsorted COO at the bench size: two bucketing pre-passes (by row, by column); columns are
    uniform, rows are not, so the heaviest rows leave segment items behind."""
    n, d = 1 << 20, 64
    q, k, v = syn.qkv(n, d, device=DEV, seed=0)
    r, c = syn.zipf_coo(n, 50_000_000, 1.3, device=DEV, seed=0)
    r_t, c_t = r.to(torch.uint64), c.to(torch.uint32)
    val = torch.empty(0, device=DEV)
    m, l, o = syn.fresh_state(n, d, device=DEV)
    mods["spfa_coo"].forward(q, k, v, r_t, c_t, val, m, l, o, False)
    d_out = torch.randn(n, d, device=DEV, generator=torch.Generator(device=DEV).manual_seed(12))
    dq, dk, dv = (torch.zeros(n, d, device=DEV) for _ in range(3))
    mods["spfa_coo"].backward(q, k, v, r_t, c_t, val, m, l, o, d_out, dq, dk, dv)
    torch.cuda.synchronize()
    _grad_properties(q, k, v, d_out, l, dq, dk, dv, torch.float32)
    deg = torch.bincount(r, minlength=n)
    heavy = torch.topk(deg, 3)[1].cpu().numpy()
    empty = torch.nonzero(deg == 0)[:3, 0].cpu().numpy()
    rows = np.unique(np.concatenate([heavy, empty, rand_rows(n, 30, 13)]))
    _dq_sample_check(q, k, v, d_out, dq, rows, lambda i: c[r == i].cpu().numpy(), torch.float32)
    assert not dq[torch.as_tensor(empty).to(DEV)].any()
    # key side on a few columns, weighted with the forward pass's own statistics
    lse = m.double() + l.double().log()
    delta = (d_out.double() * o.double()).sum(dim=1)
    for j in rand_rows(n, 6, 14):
        att = r[c == int(j)]
        s = (q[att].double() @ k[j].double()) / math.sqrt(d)
        p = torch.exp(s - lse[att])
        ds = p * (d_out[att].double() @ v[j].double() - delta[att]) / math.sqrt(d)
        assert float((dv[j].double() - p @ d_out[att].double()).abs().max()) <= 2e-4
        assert float((dk[j].double() - ds @ q[att].double()).abs().max()) <= 2e-4
