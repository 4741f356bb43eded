"""GPU parity of the gradient entry points with the float64 oracle (dense masked attention
differentiated by hand, itself pinned against library autograd and finite differences on the CPU).

The reference has no backward pass, so there is no reference test to mirror; the bars are
rounding-level for float64, 2e-4 of the gradient's scale for float32 and 3e-2 of it for the half
types (their q, k, v, out and d_out are rounded to 8 / 11 bits)."""
import numpy as np
import pytest
import torch

import spfa_autograd
import spfa_synth as syn
from helpers import np64
from oracle import spfa_oracle as so

pytestmark = pytest.mark.gpu
DEV = "cuda"
GRAD_TOL = {torch.float64: 1e-10, torch.float32: 2e-4, torch.float16: 3e-2, torch.bfloat16: 3e-2}


def _problem(n, d, dtype, seed, n_k=None, lead=()):
    g = torch.Generator().manual_seed(seed)
    n_k = n if n_k is None else n_k
    mk = lambda rows: torch.randn(*lead, rows, d, generator=g, dtype=torch.float64).to(dtype).to(DEV)
    return mk(n), mk(n_k), mk(n_k), mk(n)  # q, k, v, d_out


def _check_grads(got, ref, dtype, what):
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        a = np64(a)
        scale = max(1.0, float(np.abs(b).max()))
        err = float(np.abs(a - b).max())
        assert np.isfinite(a).all(), "%s %s: non-finite gradient" % (what, name)
        assert err <= GRAD_TOL[dtype] * scale, "%s %s: max-abs error %.3e > %.1e * %.2f" % (
            what, name, err, GRAD_TOL[dtype], scale)


def _grads_of(q, k, v, d_out, parts):
    q, k, v = (x.clone().requires_grad_(True) for x in (q, k, v))
    out = spfa_autograd.attention(q, k, v, parts)
    out.backward(d_out)
    torch.cuda.synchronize()
    return out.detach(), (q.grad, k.grad, v.grad)


def _csr_part(dense):
    ro, ci = so.csr_from_dense(dense)
    return ("csr", torch.as_tensor(ro).to(torch.uint64).to(DEV), torch.as_tensor(ci).to(torch.uint32).to(DEV))


def _coo_part(dense, seed):
    r, c = so.coo_from_dense(dense)
    perm = np.random.default_rng(seed).permutation(len(r))
    return ("coo", torch.as_tensor(r[perm]).to(torch.uint64).to(DEV),
            torch.as_tensor(c[perm]).to(torch.uint32).to(DEV))


def _random_mask(n, n_k, seed):
    rng = np.random.default_rng(seed)
    dense = rng.random((n, n_k)) < 0.08
    dense[3] = False           # an empty row
    dense[4] = False
    dense[4, n_k // 2] = True  # one live column
    dense[10] = True           # a full row (several chunks of 64 candidates)
    return dense


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 40, 200])
def test_explicit_masks_match_the_oracle(mods, dtype, d):
    n, n_k = 300, 420
    q, k, v, d_out = _problem(n, d, dtype, 5, n_k)
    dense = _random_mask(n, n_k, 6)
    ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
    _, got = _grads_of(q, k, v, d_out, [_csr_part(dense)])
    _check_grads(got, ref, dtype, "csr")
    assert not np64(got[0])[3].any()  # the empty row carries nothing
    _, got = _grads_of(q, k, v, d_out, [_coo_part(dense, 7)])
    _check_grads(got, ref, dtype, "coo (shuffled)")


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32, torch.bfloat16])
def test_implicit_masks_match_the_oracle(mods, dtype):
    n, d = 480, 64
    w, dil, blk = 70, 2, 96
    globs = [0, 17, 200, 479]
    gl = torch.tensor(globs, dtype=torch.int32, device=DEV)
    cases = [
        ([("local", w)], so.mask_local_dense(n, w)),
        ([("local", 0)], so.mask_local_dense(n, 0)),
        ([("local_1d_dilated", w, dil)], so.mask_local_1d_dilated_dense(n, w, dil)),
        ([("local_2d_dilated", blk, dil)], so.mask_local_2d_dilated_dense(n, blk, dil)),
        ([("global_no_local", gl, 9)], so.mask_global_no_local_dense(n, globs, 9)),
    ]
    for parts, dense in cases:
        q, k, v, d_out = _problem(n, d, dtype, 11)
        ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
        _, got = _grads_of(q, k, v, d_out, parts)
        _check_grads(got, ref, dtype, parts[0][0])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128, 32, 96, 160, 192])
def test_band_masks_on_the_tile_path(mods, dtype, d):
    """Band, block and global masks at d = 32 / 64 / 96 / 128 (band and block masks of the half types
    also at 160 / 192) with rows of 32 and more live positions go to the dense-tile gradient kernels:
    windows below, at and above a tile, sequence ends inside a tile, dilation (several
    subsequences of unequal length), blocks with and without dilation, a stacked batch."""
    cases = [
        (517, [("local", 16)], lambda n: so.mask_local_dense(n, 16)),
        (700, [("local", 150)], lambda n: so.mask_local_dense(n, 150)),
        (300, [("local", 299)], lambda n: so.mask_local_dense(n, 299)),
        (1000, [("local_1d_dilated", 40, 2)], lambda n: so.mask_local_1d_dilated_dense(n, 40, 2)),
        (640, [("local_2d_dilated", 160, 0)], lambda n: so.mask_local_2d_dilated_dense(n, 160, 0)),
        (768, [("local_2d_dilated", 256, 1)], lambda n: so.mask_local_2d_dilated_dense(n, 256, 1)),
        (700, [("global_no_local", torch.tensor([3, 350, 699], dtype=torch.int32, device=DEV), 5)],
         lambda n: so.mask_global_no_local_dense(n, [3, 350, 699], 5)),
        # more listed tokens than one tile of owners (128) or of streamed rows (64)
        (900, [("global_no_local", torch.arange(2, 900, 6, dtype=torch.int32, device=DEV), 0)],
         lambda n: so.mask_global_no_local_dense(n, list(range(2, 900, 6)), 0)),
    ]
    for n, parts, mask_fn in cases:
        q, k, v, d_out = _problem(n, d, dtype, 91)
        dense = mask_fn(n)
        ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
        _, got = _grads_of(q, k, v, d_out, parts)
        _check_grads(got, ref, dtype, "%s n=%d" % (parts[0], n))
    # a batch of problems sharing the mask
    n, lead = 400, (3,)
    q, k, v, d_out = _problem(n, d, dtype, 92, lead=lead)
    gl = [7, 120, 399]
    for parts, dense in [([("local", 50)], so.mask_local_dense(n, 50)),
                         ([("global_no_local", torch.tensor(gl, dtype=torch.int32, device=DEV), 20)],
                          so.mask_global_no_local_dense(n, gl, 20))]:
        _, got = _grads_of(q, k, v, d_out, parts)
        for b in range(lead[0]):
            ref = so.dense_masked_attention_backward(np64(q[b]), np64(k[b]), np64(v[b]), dense, np64(d_out[b]))
            _check_grads([x[b] for x in got], ref, dtype, "%s batch %d" % (parts[0][0], b))


@pytest.mark.parametrize("dtype,d", [(torch.float32, 4), (torch.float32, 40), (torch.float32, 100),
                                     (torch.float32, 124), (torch.bfloat16, 8), (torch.bfloat16, 40),
                                     (torch.float16, 80), (torch.bfloat16, 104), (torch.float16, 136),
                                     (torch.bfloat16, 184), (torch.float16, 200)])
def test_band_masks_rows_that_are_no_multiple_of_32(mods, dtype, d):
    """Rows of whole 16-byte pieces on the gradient tiles of the next multiple of 32 that is built
    (zero-filled operands; d = 200 has none and takes the gather passes): window, dilation, blocks,
    sequence ends inside a tile, a stacked batch."""
    cases = [
        (517, [("local", 16)], lambda n: so.mask_local_dense(n, 16)),
        (700, [("local", 150)], lambda n: so.mask_local_dense(n, 150)),
        (1000, [("local_1d_dilated", 40, 2)], lambda n: so.mask_local_1d_dilated_dense(n, 40, 2)),
        (768, [("local_2d_dilated", 256, 1)], lambda n: so.mask_local_2d_dilated_dense(n, 256, 1)),
    ]
    for n, parts, mask_fn in cases:
        q, k, v, d_out = _problem(n, d, dtype, 94)
        ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), mask_fn(n), np64(d_out))
        _, got = _grads_of(q, k, v, d_out, parts)
        _check_grads(got, ref, dtype, "%s n=%d" % (parts[0], n))
    n, lead = 400, (3,)
    q, k, v, d_out = _problem(n, d, dtype, 95, lead=lead)
    dense = so.mask_local_dense(n, 50)
    _, got = _grads_of(q, k, v, d_out, [("local", 50)])
    for b in range(lead[0]):
        ref = so.dense_masked_attention_backward(np64(q[b]), np64(k[b]), np64(v[b]), dense, np64(d_out[b]))
        _check_grads([x[b] for x in got], ref, dtype, "batch %d" % b)
    # the global mask (its gradient tiles are built up to d = 128): a few listed tokens, more than a
    # tile of them with repeats, a batch
    for n, gl, w in [(700, [3, 350, 699], 5), (900, list(range(2, 900, 6)) + [8, 8, 14], 0)]:
        q, k, v, d_out = _problem(n, d, dtype, 96)
        dense_w = so.mask_global_no_local_dense(n, gl, w)
        ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense_w, np64(d_out)) \
            if len(set(gl)) == len(gl) else None
        _, got = _grads_of(q, k, v, d_out, [("global_no_local", torch.tensor(gl, dtype=torch.int32, device=DEV), w)])
        if ref is not None:
            _check_grads(got, ref, dtype, "global n=%d" % n)
        else:
            # repeats (an ordinary row counts a listed token once per occurrence): against the same
            # call at the next multiple of 32 with zero columns appended, q and k rescaled so that
            # q.k / sqrt(d) is unchanged
            dp = (d + 31) // 32 * 32
            pad = lambda x: torch.nn.functional.pad(x, (0, dp - d))
            _, got_p = _grads_of(pad(q) * (dp / d) ** 0.25, pad(k) * (dp / d) ** 0.25, pad(v), pad(d_out),
                                 [("global_no_local", torch.tensor(gl, dtype=torch.int32, device=DEV), w)])
            scale_back = (dp / d) ** 0.25
            ref_p = [np64(got_p[0])[:, :d] * scale_back, np64(got_p[1])[:, :d] * scale_back, np64(got_p[2])[:, :d]]
            _check_grads(got, ref_p, dtype, "global with repeats n=%d" % n)


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.float16, 128), (torch.bfloat16, 32),
                                     (torch.float32, 32), (torch.float32, 64), (torch.float32, 128)])
@pytest.mark.parametrize("w,dil", [(1, 0), (2, 1), (5, 0), (6, 0), (12, 2), (13, 0)])
def test_narrow_windows_in_calls_of_many_rows(mods, dtype, d, w, dil):
    """From 32768 rows on (16 problems of 2100 tokens here) the gradient of a window mask runs on
    the tiles from 3 candidates per row for the half types and fp32 at d = 32, from 13 / 27 for
    fp32 at d = 64 / 128; both sides of the limits against the oracle (first and last problem)."""
    n, lead = 2100, (16,)
    q, k, v, d_out = _problem(n, d, dtype, 93, lead=lead)
    dense = so.mask_local_1d_dilated_dense(n, w, dil)
    _, got = _grads_of(q, k, v, d_out, [("local_1d_dilated", w, dil)])
    for b in (0, lead[0] - 1):
        ref = so.dense_masked_attention_backward(np64(q[b]), np64(k[b]), np64(v[b]), dense, np64(d_out[b]))
        _check_grads([x[b] for x in got], ref, dtype, "w=%d dil=%d problem %d" % (w, dil, b))


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_chained_parts_are_differentiated_as_their_union(mods, dtype):
    """window + global + random, the chain of verification/verify.py:337-352: one backward call
    per part against the finished state equals the gradient of attention over the union."""
    n, d, w = 400, 32, 12
    globs = [5, 250]
    rng = np.random.default_rng(21)
    rand = rng.random((n, n)) < 0.03
    union = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, globs, w)
    rand &= ~union
    gl = torch.tensor(globs, dtype=torch.int32, device=DEV)
    q, k, v, d_out = _problem(n, d, dtype, 22)
    ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), union | rand, np64(d_out))
    out, got = _grads_of(q, k, v, d_out, [("local", w), ("global_no_local", gl, w), _csr_part(rand)])
    _check_grads(got, ref, dtype, "chain")
    ref_out = so.dense_masked_attention(np64(q), np64(k), np64(v), union | rand)[0]
    assert np.abs(np64(out) - ref_out).max() <= (1e-11 if dtype == torch.float64 else 1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rows_and_columns_longer_than_one_segment(mods, dtype):
    """Owners with many live positions are split over several wavefronts: a query row and a key
    column with ~2500 entries, rows and columns of 512 ... 2049 (explicit mask), a band of 1401, the
    rows and columns of listed global tokens."""
    n, d = 2600, 64
    rng = np.random.default_rng(61)
    dense = rng.random((n, n)) < 0.01
    dense[7, rng.permutation(n)[:2500]] = True
    dense[rng.permutation(n)[:2500], 11] = True
    # owners around the length from which a row goes on the work list, and around one segment
    for i, ln in enumerate([512, 513, 1024, 1025, 2049]):
        dense[20 + i, :] = False
        dense[20 + i, rng.permutation(n)[:ln]] = True
        dense[:, 40 + i] = False
        dense[rng.permutation(n)[:ln], 40 + i] = True
    q, k, v, d_out = _problem(n, d, dtype, 62)
    for parts, mask in [([_csr_part(dense)], dense), ([_coo_part(dense, 63)], dense),
                        ([("local", 700)], so.mask_local_dense(n, 700)),
                        ([("global_no_local", torch.tensor([3, 1300], dtype=torch.int32, device=DEV), 4)],
                         so.mask_global_no_local_dense(n, [3, 1300], 4))]:
        ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), mask, np64(d_out))
        _, got = _grads_of(q, k, v, d_out, parts)
        _check_grads(got, ref, dtype, parts[0][0])


@pytest.mark.parametrize("d", [32, 64])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_repeated_global_indices_count_as_often_as_in_the_forward_pass(mods, dtype, d):
    """A token listed twice is walked twice by every ordinary row
    (sp_flatt_global_no_local_kernel.cu:134-162 reads the list as given) and once by listed rows.
    The dense statement of that: one extra key/value column per repetition, live for the ordinary
    rows outside their window; the gradient of the repeated token is the sum over its copies."""
    n, w = 300, 6  # (d = 32: gather passes, d = 64: dense tiles)
    globs = [40, 200, 40, 7]
    q, k, v, d_out = _problem(n, d, dtype, 71)
    base = so.mask_global_no_local_dense(n, sorted(set(globs)), w)
    extra = np.zeros((n, 1), dtype=bool)
    for i in range(n):
        extra[i, 0] = (i not in globs) and abs(i - 40) > w
    mask = np.concatenate([base, extra], axis=1)
    k2 = np.concatenate([np64(k), np64(k)[40:41]])
    v2 = np.concatenate([np64(v), np64(v)[40:41]])
    dq, dk2, dv2 = so.dense_masked_attention_backward(np64(q), k2, v2, mask, np64(d_out))
    dk, dv = dk2[:n].copy(), dv2[:n].copy()
    dk[40] += dk2[n]
    dv[40] += dv2[n]
    out, got = _grads_of(q, k, v, d_out, [("global_no_local", torch.tensor(globs, dtype=torch.int32, device=DEV), w)])
    ref_out = so.dense_masked_attention(np64(q), k2, v2, mask)[0]
    assert np.abs(np64(out) - ref_out).max() <= (1e-11 if dtype == torch.float64 else 1e-4)
    _check_grads(got, (dq, dk, dv), dtype, "repeated globals")


def test_transposed_mask_is_exact_and_reusable(mods):
    """spfa_csr.transpose against a CPU transposition (bit-exact offsets, the rows of every column
    as a set), for a rectangular mask with empty rows and columns, both offset widths; and the
    gradients with the transposed mask handed in equal those that rebuild it."""
    n, n_k, d = 500, 700, 64
    rng = np.random.default_rng(81)
    dense = rng.random((n, n_k)) < 0.05
    dense[9] = False
    dense[:, 13] = False
    dense[20] = True
    ro, ci = so.csr_from_dense(dense)
    t_ro_ref, t_ci_ref = so.csr_from_dense(dense.T)
    for off_dtype in (torch.uint64, torch.int32):
        ro_t = torch.as_tensor(ro).to(off_dtype).to(DEV)
        ci_t = torch.as_tensor(ci).to(torch.uint32).to(DEV)
        t_ro, t_ci = mods["spfa_csr"].transpose(ro_t, ci_t, n_k)
        torch.cuda.synchronize()
        assert t_ro.dtype == torch.uint32 and t_ci.dtype == torch.uint32
        t_ro, t_ci = t_ro.cpu().numpy().astype(np.int64), t_ci.cpu().numpy().astype(np.int64)
        assert np.array_equal(t_ro, t_ro_ref)
        for j in range(n_k):
            assert np.array_equal(np.sort(t_ci[t_ro[j]:t_ro[j + 1]]), t_ci_ref[t_ro_ref[j]:t_ro_ref[j + 1]]), j
    q, k, v, d_out = _problem(n, d, torch.float32, 82, n_k)
    part = _csr_part(dense)
    ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
    _, got = _grads_of(q, k, v, d_out, [spfa_autograd.csr_part(part[1], part[2], n_k)])
    _check_grads(got, ref, torch.float32, "csr with transposed mask")
    # an empty mask transposes to empty columns
    z_ro, z_ci = mods["spfa_csr"].transpose(torch.zeros(5, dtype=torch.int64, device=DEV),
                                            torch.zeros(0, dtype=torch.int32, device=DEV), 6)
    torch.cuda.synchronize()
    assert z_ro.cpu().tolist() == [0] * 7 and z_ci.numel() == 0


def test_transposition_of_masks_with_runs_of_empty_and_of_one_entry_rows(mods):
    """The transposition walks the entries in fixed chunks and finds their rows from windows of 64
    row offsets: rows longer than a chunk, runs of more than 64 and more than 128 empty rows (also
    first and last), runs of rows of one entry, and a number of entries that is no multiple of the
    chunk, against a CPU transposition."""
    n_k = 5000
    rng = np.random.default_rng(83)
    deg = np.concatenate([
        np.zeros(70, np.int64), [3], np.ones(150, np.int64), [4100], np.zeros(200, np.int64),
        rng.integers(0, 3, 300), [2048, 2049, 1], np.zeros(64, np.int64), [5], np.zeros(63, np.int64),
        rng.integers(0, 40, 200), np.ones(1000, np.int64), [0, 0, 2500], np.zeros(130, np.int64)])
    n = len(deg)
    ro = np.concatenate([[0], np.cumsum(deg)])
    ci = np.concatenate([np.sort(rng.choice(n_k, int(g), replace=False)) for g in deg]).astype(np.int64)
    rows = np.repeat(np.arange(n), deg)
    order = np.lexsort((rows, ci))
    t_ro_ref = np.concatenate([[0], np.cumsum(np.bincount(ci, minlength=n_k))])
    t_ci_ref = rows[order]
    for off_dtype in (torch.int64, torch.int32):
        t_ro, t_ci = mods["spfa_csr"].transpose(torch.as_tensor(ro).to(off_dtype).to(DEV),
                                                torch.as_tensor(ci).to(torch.int32).to(DEV), n_k)
        torch.cuda.synchronize()
        t_ro, t_ci = t_ro.cpu().numpy().astype(np.int64), t_ci.cpu().numpy().astype(np.int64)
        assert np.array_equal(t_ro, t_ro_ref)
        # (the rows of a column come in no particular order)
        key = np.repeat(np.arange(n_k), np.diff(t_ro))
        assert np.array_equal(t_ci[np.lexsort((t_ci, key))], t_ci_ref)


def test_batch_of_heads_shares_the_mask(mods):
    n, d, lead = 200, 64, (2, 3)
    q, k, v, d_out = _problem(n, d, torch.float32, 31, lead=lead)
    dense = _random_mask(n, n, 32)
    _, got = _grads_of(q, k, v, d_out, [_csr_part(dense), ])
    for b in range(lead[0]):
        for h in range(lead[1]):
            ref = so.dense_masked_attention_backward(np64(q[b, h]), np64(k[b, h]), np64(v[b, h]), dense,
                                                     np64(d_out[b, h]))
            _check_grads([g[b, h] for g in got], ref, torch.float32, "head %d,%d" % (b, h))


def test_gradcheck_float64(mods):
    """torch's own numerical gradient check through the autograd function (float64; the atomics
    make two runs differ in the last bits, hence nondet_tol)."""
    n, d = 24, 8
    q, k, v, _ = _problem(n, d, torch.float64, 41)
    dense = np.random.default_rng(42).random((n, n)) < 0.3
    dense[np.arange(n), np.arange(n)] = False
    parts = [("local", 0), _csr_part(dense)]
    q, k, v = (x.requires_grad_(True) for x in (q, k, v))
    assert torch.autograd.gradcheck(lambda a, b, c: spfa_autograd.attention(a, b, c, parts), (q, k, v),
                                    eps=1e-6, atol=1e-7, rtol=1e-6, nondet_tol=1e-9)


def test_backward_adds_to_the_given_gradients_and_checks_parameters(mods):
    n, d = 64, 16
    q, k, v, d_out = _problem(n, d, torch.float32, 51)
    m = torch.full((n,), -float("inf"), device=DEV)
    l = torch.zeros(n, device=DEV)
    o = torch.zeros_like(q)
    mods["spfa_local"].forward(q, k, v, m, l, o, 3)
    base = torch.full((n, d), 2.0, device=DEV)
    dq, dk, dv = base.clone(), base.clone(), base.clone()
    ret = mods["spfa_local"].backward(q, k, v, m, l, o, 3, d_out, dq, dk, dv)
    torch.cuda.synchronize()
    assert ret[0].data_ptr() == dq.data_ptr()
    ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), so.mask_local_dense(n, 3), np64(d_out))
    _check_grads((dq - 2.0, dk - 2.0, dv - 2.0), ref, torch.float32, "accumulate")
    with pytest.raises(ValueError, match="local size"):
        mods["spfa_local"].backward(q, k, v, m, l, o, n, d_out, dq, dk, dv)
    with pytest.raises(RuntimeError, match="float32"):
        mods["spfa_local"].backward(q, k, v, m, l, o, 3, d_out, dq.half(), dk, dv)
    with pytest.raises(RuntimeError, match="dO must have the shape"):
        mods["spfa_local"].backward(q, k, v, m, l, o, 3, d_out[:-1].contiguous(), dq, dk, dv)


@pytest.mark.parametrize("d", [1, 3, 512, 1024])
def test_extreme_embedding_sizes(mods, d):
    """d = 1 .. 1024 (the limit the forward calls accept) through the general lane layouts."""
    n = 96
    q, k, v, d_out = _problem(n, d, torch.float32, 101)
    dense = np.random.default_rng(102).random((n, n)) < 0.2
    dense[np.arange(n), np.arange(n)] = True
    ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
    _, got = _grads_of(q, k, v, d_out, [_csr_part(dense)])
    _check_grads(got, ref, torch.float32, "csr d=%d" % d)
    ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), so.mask_local_dense(n, 40), np64(d_out))
    _, got = _grads_of(q, k, v, d_out, [("local", 40)])
    _check_grads(got, ref, torch.float32, "local d=%d" % d)


def test_empty_masks_and_dead_rows_leave_gradients_alone(mods):
    n, d = 50, 16
    q, k, v, d_out = _problem(n, d, torch.float32, 111)
    empty = np.zeros((n, n), dtype=bool)
    out, got = _grads_of(q, k, v, d_out, [_csr_part(empty)])
    assert not np64(out).any()
    for x in got:
        assert not np64(x).any()
    # use_nan forward leaves NaN rows in out; the backward call must not spread them
    dense = np.random.default_rng(112).random((n, n)) < 0.1
    dense[7] = False
    part = _csr_part(dense)
    m = torch.full((n,), -float("inf"), device=DEV)
    l = torch.zeros(n, device=DEV)
    o = torch.zeros(n, d, device=DEV)
    val = torch.empty(0, device=DEV)
    mods["spfa_csr"].forward(q, k, v, part[1], part[2], val, m, l, o, True)
    assert torch.isnan(o[7]).all()
    dq, dk, dv = (torch.zeros(n, d, device=DEV) for _ in range(3))
    mods["spfa_csr"].backward(q, k, v, part[1], part[2], val, m, l, o, d_out, dq, dk, dv)
    torch.cuda.synchronize()
    ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
    _check_grads((dq, dk, dv), ref, torch.float32, "NaN rows in out")


def test_composite_backward_equals_dense_union(mods):
    """spfa_bigbird.backward == gradients of dense attention over window | global | random, with
    and without the transposed CSR part handed in; parts may be empty."""
    n, d, w = 600, 64, 9
    globs = [4, 333]
    rng = np.random.default_rng(121)
    union = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, globs, w)
    rand = (rng.random((n, n)) < 0.02) & ~union
    ro, ci = so.csr_from_dense(rand)
    ro_t = torch.as_tensor(ro).to(torch.uint64).to(DEV)
    ci_t = torch.as_tensor(ci).to(torch.uint32).to(DEV)
    gl = torch.tensor(globs, dtype=torch.int32, device=DEV)
    q, k, v, d_out = _problem(n, d, torch.float32, 122)
    val = torch.empty(0, device=DEV)
    tr = mods["spfa_csr"].transpose(ro_t, ci_t, n)
    none_i = torch.zeros(0, dtype=torch.int32, device=DEV)
    none_o = torch.zeros(0, dtype=torch.int64, device=DEV)
    for gl_arg, csr_arg, dense, extra in [(gl, (ro_t, ci_t), union | rand, ()), (gl, (ro_t, ci_t), union | rand, tr),
                                          (none_i, (none_o, none_i), so.mask_local_dense(n, w), ())]:
        m = torch.full((n,), -float("inf"), device=DEV)
        l = torch.zeros(n, device=DEV)
        o = torch.zeros(n, d, device=DEV)
        mods["spfa_bigbird"].forward(q, k, v, m, l, o, w, gl_arg, csr_arg[0], csr_arg[1], val)
        dq, dk, dv = (torch.zeros(n, d, device=DEV) for _ in range(3))
        mods["spfa_bigbird"].backward(q, k, v, m, l, o, w, gl_arg, csr_arg[0], csr_arg[1], val, d_out, dq, dk, dv,
                                      *extra)
        torch.cuda.synchronize()
        ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
        _check_grads((dq, dk, dv), ref, torch.float32, "composite")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_statistics_stored_in_the_element_type(mods, dtype):
    """m and l in the element type (the reference's convention) instead of float32: the gradient
    calls read them the same way the forward calls wrote them.  m is then rounded to 8 / 11 bits,
    so the bar is the statistics' own (1e-1 on m + log l, as in the forward tests)."""
    n, d, w = 300, 64, 20
    q, k, v, d_out = _problem(n, d, dtype, 131)
    for name, args, dense in [("spfa_local", (w,), so.mask_local_dense(n, w)),
                              ("spfa_local_1d_dilated", (5, 1), so.mask_local_1d_dilated_dense(n, 5, 1))]:
        m = torch.full((n,), -float("inf"), device=DEV, dtype=dtype)
        l = torch.zeros(n, device=DEV, dtype=dtype)
        o = torch.zeros(n, d, device=DEV, dtype=dtype)
        mods[name].forward(q, k, v, m, l, o, *args)
        dq, dk, dv = (torch.zeros(n, d, device=DEV) for _ in range(3))
        mods[name].backward(q, k, v, m, l, o, *args, d_out, dq, dk, dv)
        torch.cuda.synchronize()
        ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
        for nm, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), ref):
            err = float(np.abs(np64(a) - b).max())
            assert err <= 0.15 * max(1.0, float(np.abs(b).max())), "%s %s: %.3e" % (name, nm, err)


def test_coo_entries_converted_once(mods):
    """spfa_coo.to_csr against a CPU conversion (exact offsets, every row's columns as a set, both
    row index widths, sorted and shuffled entries), and spfa_autograd.coo_part == the coo part."""
    n, n_k, d = 300, 410, 64
    rng = np.random.default_rng(151)
    dense = rng.random((n, n_k)) < 0.06
    dense[17] = False
    r, c = so.coo_from_dense(dense)
    ro_ref, ci_ref = so.csr_from_dense(dense)
    for perm, rdt in ((np.arange(len(r)), torch.uint64), (rng.permutation(len(r)), torch.int32)):
        r_t = torch.as_tensor(r[perm]).to(rdt).to(DEV)
        c_t = torch.as_tensor(c[perm]).to(torch.uint32).to(DEV)
        ro, ci = mods["spfa_coo"].to_csr(r_t, c_t, n)
        torch.cuda.synchronize()
        ro, ci = ro.cpu().numpy().astype(np.int64), ci.cpu().numpy().astype(np.int64)
        assert np.array_equal(ro, ro_ref)
        for i in range(n):
            assert np.array_equal(np.sort(ci[ro[i]:ro[i + 1]]), ci_ref[ro_ref[i]:ro_ref[i + 1]]), i
    q, k, v, d_out = _problem(n, d, torch.float32, 152, n_k)
    ref = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
    out, got = _grads_of(q, k, v, d_out, [spfa_autograd.coo_part(r_t, c_t, n, n_k)])
    _check_grads(got, ref, torch.float32, "coo_part")
    assert np.abs(np64(out) - np.nan_to_num(so.dense_masked_attention(np64(q), np64(k), np64(v), dense)[0])).max() <= 1e-4
