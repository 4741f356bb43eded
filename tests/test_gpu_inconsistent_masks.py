"""What the library does with mask arrays that disagree with the sizes a call states.  The
reference launches on whatever it is given (sp_flatt_csr_kernel.cu:271-287); here such arrays can
neither send a load outside the tensors nor go unnoticed: rows are cut to the entries that exist,
out-of-range columns / listed tokens are masked, and the device's status word reports what the
kernels saw.  Every case is checked against the oracle on the mask that is left."""
import numpy as np
import pytest
import torch

import spfa_synth as syn
from helpers import check, np64
from oracle import c_oracle
from oracle import spfa_oracle as so

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _state(n, d):
    return syn.fresh_state(n, d, device=DEV)


def _qkv(n, d, seed, n_k=None):
    q, k, v = syn.qkv(n, d, device="cpu", seed=seed, n_k=n_k)
    return q.to(DEV), k.to(DEV), v.to(DEV)


def _csr_call(mods, q, k, v, ro, ci, use_nan=False):
    m, l, o = _state(*q.shape)
    ro_t = torch.as_tensor(np.asarray(ro, np.int64)).to(torch.uint64).to(DEV)
    ci_t = torch.as_tensor(np.asarray(ci, np.int64)).to(torch.uint32).to(DEV)
    val = torch.ones(ci_t.numel(), device=DEV)
    mods["spfa_csr"].forward(q, k, v, ro_t, ci_t, val, m, l, o, use_nan)
    torch.cuda.synchronize()
    return o, m, l


@pytest.mark.parametrize("n", [600, 40000])  # the single-launch path and the general path
def test_columns_beyond_the_key_count_are_masked(mods, n):
    d, n_k = 64, 500
    q, k, v = _qkv(n, d, 3, n_k=n_k)
    rng = np.random.default_rng(3)
    deg = rng.integers(0, 90, n)
    deg[5] = 700  # a long row
    ro = np.zeros(n + 1, np.int64)
    np.cumsum(deg, out=ro[1:])
    ci = rng.integers(0, n_k + 200, ro[-1])  # about 2 in 7 point past K and V
    mods["spfa_csr"].device_status(True)
    o, m, l = _csr_call(mods, q, k, v, ro, ci)
    lists = [ci[ro[i]:ro[i + 1]] for i in range(n)]
    lists = [x[x < n_k] for x in lists]
    ro2 = np.zeros(n + 1, np.int64)
    np.cumsum([len(x) for x in lists], out=ro2[1:])
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro2, np.concatenate(lists))
    check(o, m, l, *ref, torch.float32)
    assert mods["spfa_csr"].device_status(False) == 0  # (columns are masked silently)


@pytest.mark.parametrize("n", [600, 40000])
def test_row_offsets_beyond_nnz_are_cut_and_reported(mods, n):
    d = 64
    q, k, v = _qkv(n, d, 4)
    ro, ci = syn.zipf_csr(n, 1.5, 1, 512, seed=4)
    ro, ci = ro.numpy().copy(), ci.numpy()
    nnz = len(ci)
    # the last fifth of the rows claims entries past the end of the column array, one row's
    # offsets run backwards
    bad = ro.copy()
    first_bad = n - n // 5
    bad[first_bad + 1:] += 1000
    bad[100] = bad[101] + 7 if bad[101] + 7 <= nnz else bad[101]
    mods["spfa_csr"].device_status(True)
    o, m, l = _csr_call(mods, q, k, v, bad, ci)
    # what is left: every row's range cut to [0, nnz), a backwards range is empty
    a = np.minimum(bad[:-1], nnz)
    b = np.minimum(bad[1:], nnz)
    a = np.minimum(a, b)
    lists = [ci[a[i]:b[i]] for i in range(n)]
    ro2 = np.zeros(n + 1, np.int64)
    np.cumsum([len(x) for x in lists], out=ro2[1:])
    ref = c_oracle.csr(np64(q), np64(k), np64(v), ro2, np.concatenate(lists))
    check(o, m, l, *ref, torch.float32)
    bits = mods["spfa_csr"].device_status(True)
    assert bits & 2, bits
    assert mods["spfa_csr"].device_status(False) == 0


def test_more_long_row_entries_than_nnz_is_reported_and_leaves_long_rows_alone(mods):
    """Offsets that jump back and forth: every other row claims the whole column array (each such
    row is consistent in itself), the rows between run backwards.  Together the rows claim 20000
    times the entries that exist; the work list, sized from nnz, cannot hold them."""
    n, d, nnz = 40000, 64, 30000
    q, k, v = _qkv(n, d, 5)
    ci = np.random.default_rng(5).integers(0, n, nnz)
    ro = np.zeros(n + 1, np.int64)
    ro[1::2] = nnz
    mods["spfa_csr"].device_status(True)
    o, m, l = _csr_call(mods, q, k, v, ro, ci, use_nan=True)
    bits = mods["spfa_csr"].device_status(True)
    assert bits & 1, bits  # work list overflow
    assert bits & 2, bits  # rows whose offsets run backwards
    # no long row was computed; the rows whose range was cut to nothing count as empty rows
    assert (l == 0).all() and torch.isinf(m).all()
    on = np64(o)
    assert (on[0::2] == 0).all()
    assert np.isnan(on[1::2]).all()


def test_plan_refuses_offsets_that_do_not_end_at_nnz(mods):
    ro = torch.tensor([0, 2, 5], dtype=torch.int64).to(torch.uint64).to(DEV)
    ci = torch.tensor([0, 1, 0, 1], dtype=torch.int32).to(torch.uint32).to(DEV)
    with pytest.raises(RuntimeError, match="must end at the number of entries"):
        mods["spfa_csr"].plan(ro, ci)


@pytest.mark.parametrize("d,n,w", [(64, 4096, 5), (40, 700, 5)])  # dense tiles and the gather path
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_listed_tokens_outside_the_sequence_are_ignored(mods, dtype, d, n, w):
    q, k, v = [x.to(dtype) for x in _qkv(n, d, 6)]
    good = [7, n - 1, 300, 301, 40]
    listed = torch.tensor([good[0], -3, good[1], n, good[2], good[3], 2 ** 31 - 1, good[4], n + 5000],
                          dtype=torch.int32, device=DEV)
    m, l, o = syn.fresh_state(n, d, dtype=dtype, device=DEV, state_dtype=torch.float32)
    mods["spfa_global_no_local"].forward(q, k, v, m, l, o, listed, w)
    torch.cuda.synchronize()
    ref = c_oracle.global_no_local(np64(q), np64(k), np64(v), np.asarray(good, np.int32), w)
    check(o, m, l, *ref, dtype, state_dtype=torch.float32)
    # and the gradients (tile and gather passes) of the same call
    gen = torch.Generator(device=DEV).manual_seed(6)
    d_out = torch.randn(n, d, device=DEV, generator=gen).to(dtype)
    grads = [torch.zeros(n, d, device=DEV) for _ in range(3)]
    mods["spfa_global_no_local"].backward(q, k, v, m, l, o, listed, w, d_out, *grads)
    torch.cuda.synchronize()
    mask = so.mask_global_no_local_dense(n, good, w)
    refs = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), mask, np64(d_out))
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    for got, want in zip(grads, refs):
        assert np.abs(np64(got) - want).max() <= tol * max(1.0, np.abs(want).max())


def test_coo_rows_by_the_atomic_path_beyond_four_million_rows(mods):
    """More than 2^22 rows: the row-bucketing pre-pass of unsorted entries takes its histogram +
    scatter path instead of the partition in LDS.  to_csr exposes the result."""
    n_rows, nnz = 5_000_000, 120_000
    g = torch.Generator().manual_seed(9)
    rows = torch.randint(0, n_rows, (nnz,), generator=g, dtype=torch.int64)
    rows[:2000] = 4_999_999  # one long row at the very end
    rows[2000:2500] = 0
    cols = torch.randint(0, 1 << 20, (nnz,), generator=g, dtype=torch.int64)
    ro, ci = mods["spfa_coo"].to_csr(rows.to(torch.uint64).to(DEV), cols.to(torch.uint32).to(DEV), n_rows)
    torch.cuda.synchronize()
    ro, ci = ro.cpu().to(torch.int64), ci.cpu().to(torch.int64)
    counts = torch.bincount(rows, minlength=n_rows)
    assert torch.equal(ro[1:] - ro[:-1], counts)
    assert int(ro[0]) == 0 and int(ro[-1]) == nnz
    # the columns of every row, as multisets: sort (row, col) pairs on both sides
    got_rows = torch.repeat_interleave(torch.arange(n_rows), counts)
    got = torch.sort(got_rows * (1 << 20) + ci)[0]
    want = torch.sort(rows * (1 << 20) + cols)[0]
    assert torch.equal(got, want)


@pytest.mark.parametrize("n,nnz", [(3000, 40_000), (40_000, 900_000)])
def test_coo_entries_outside_the_mask_are_dropped(mods, n, nnz):
    """Unsorted COO entries whose row is not a query row (at or beyond n, or a 64-bit pattern far
    beyond) are dropped by the row-bucketing pre-pass, entries whose column is not a key are
    masked: the result is that of the entries left."""
    d, n_k = 64, n - 100
    q, k, v = _qkv(n, d, 12, n_k=n_k)
    rng = np.random.default_rng(12)
    rows = rng.integers(0, n, nnz).astype(np.uint64)
    cols = rng.integers(0, n_k + n_k // 5, nnz).astype(np.int64)  # one in six past the keys
    bad = rng.random(nnz) < 0.1
    rows[bad] = rng.choice(np.array([n, n + 7, 2 ** 31, 2 ** 40 + 3, 2 ** 63 + 5, 2 ** 64 - 1], dtype=np.uint64),
                           int(bad.sum()))
    m, l, o = _state(n, d)
    r_t = torch.as_tensor(rows.view(np.int64)).view(torch.uint64).to(DEV)
    c_t = torch.as_tensor(cols).to(torch.uint32).to(DEV)
    mods["spfa_coo"].forward(q, k, v, r_t, c_t, torch.ones(nnz, device=DEV), m, l, o, False)
    torch.cuda.synchronize()
    keep = ~bad & (cols < n_k)
    ref = c_oracle.coo(np64(q), np64(k), np64(v), rows[keep].astype(np.int64), cols[keep])
    check(o, m, l, *ref, torch.float32)
