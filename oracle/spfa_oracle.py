"""CPU oracle for the six sparse-FlashAttention paths.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped product imports this module: it is the checker used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``.

The reference computes, for every query row ``i`` of a single head,

    O[i] = softmax_j( Q[i].K[j] / sqrt(d)  for j in live(i) ) @ V[live(i)]

where ``live(i)`` is the set of un-masked columns of row ``i``; the mask is either
explicit (CSR / COO arrays) or implied by a few integers.  Its own correctness
check is the dense formulation ``scaled_dot_product_attention(q, k, v, bool_mask)``
(verification/verify.py:61-63).  This file restates that formulation in float64
numpy, restates every mask definition twice (once from the dense constructions of
verification/verify.py, once from the per-row bounds of the kernels) and restates
the running-softmax state merge that makes chained calls work.

How each function is pinned (none of them is checked against itself):
  * dense_masked_attention   - torch CPU scaled_dot_product_attention in float64
                               (library routine), scipy logsumexp/softmax, the
                               closed forms "window 0 => out == v" and
                               "V == 1 => out == 1", and the committed golden
                               vectors under tests/golden/ (written by torch).
  * rowwise_attention        - dense_masked_attention on the same mask, row
                               permutation invariance, split-and-chain == one call.
  * mask_*_dense             - literal transcriptions of verify.py's loops;
    live_* (per-row bounds)  - transcriptions of the kernels' index arithmetic;
                               the two are compared by brute force for every
                               parameter combination at small N, and nnz closed
                               forms are compared with counted nnz.
  * merge_state              - associativity/identity properties and the
                               split-and-chain test.
  * dense_masked_attention_backward
                             - torch CPU autograd through the library's
                               scaled_dot_product_attention in float64, central
                               finite differences of dense_masked_attention, and
                               the closed forms "one live column => dq = dk = 0,
                               dv = d_out" and "sum_j dS_ij == 0".
  * rowwise_query_gradient   - dense_masked_attention_backward on the same mask.
"""
from __future__ import annotations

import math

import numpy as np

NEG_INF = -np.inf


# --------------------------------------------------------------------------
# dense formulation (verification/verify.py:61-63)
# --------------------------------------------------------------------------
def dense_masked_attention(q, k, v, mask):
    """float64 ``softmax(where(mask, q k^T / sqrt(d), -inf)) v``.

    Returns ``(out, m, l)`` with ``m[i]`` the largest un-masked score of row i and
    ``l[i] = sum_j exp(score_ij - m[i])`` - the two statistics every reference kernel
    leaves in its ``m`` / ``l`` arguments (sp_flatt_csr_kernel.cu:162-179, 208-212).
    Rows without a live column come back as NaN in ``out`` (what the dense library
    routine produces and what ``use_nan=True`` must reproduce,
    verification/verify.py:498), with ``m = -inf`` and ``l = 0``.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    mask = np.asarray(mask, dtype=bool)
    d = q.shape[1]
    # scale rule: divide the finished dot product by sqrt(d) (sp_flatt_csr_kernel.cu:137)
    s = (q @ k.T) / math.sqrt(float(d))
    s = np.where(mask, s, NEG_INF)
    m = s.max(axis=1)
    live = np.isfinite(m)
    m_safe = np.where(live, m, 0.0)
    p = np.exp(s - m_safe[:, None])
    p = np.where(mask, p, 0.0)
    l = p.sum(axis=1)
    with np.errstate(invalid="ignore", divide="ignore"):
        out = (p @ v) / l[:, None]
    out[~live] = np.nan
    return out, np.where(live, m, NEG_INF), l


# --------------------------------------------------------------------------
# running-softmax state (sp_flatt_csr_kernel.cu:79-92, 162-201, 208-218)
# --------------------------------------------------------------------------
def dense_masked_attention_backward(q, k, v, mask, d_out):
    """Gradients of ``dense_masked_attention`` with respect to q, k and v, float64.

    The reference has no backward pass; this is the textbook differentiation of the formulation
    its verification uses (verification/verify.py:61-63).  With P the masked softmax,
    ``dV = P^T dO``, ``dP = dO V^T``, ``dS = P * (dP - rowsum(dO * O))``,
    ``dQ = dS K / sqrt(d)``, ``dK = dS^T Q / sqrt(d)``.  Rows without a live column carry no
    gradient.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    d_out = np.asarray(d_out, dtype=np.float64)
    mask = np.asarray(mask, dtype=bool)
    scale = 1.0 / math.sqrt(float(q.shape[1]))
    s = np.where(mask, (q @ k.T) * scale, NEG_INF)
    mx = s.max(axis=1)
    live = np.isfinite(mx)
    p = np.where(mask, np.exp(s - np.where(live, mx, 0.0)[:, None]), 0.0)
    den = p.sum(axis=1)
    p = p / np.where(live, den, 1.0)[:, None]
    d_out = np.where(live[:, None], d_out, 0.0)
    out = p @ v
    d_v = p.T @ d_out
    d_p = d_out @ v.T
    d_s = p * (d_p - (d_out * out).sum(axis=1)[:, None])
    d_q = (d_s @ k) * scale
    d_k = (d_s.T @ q) * scale
    return d_q, d_k, d_v


def merge_state(m_a, l_a, o_a, m_b, l_b, o_b):
    """Merge two normalised partial results of the same row.

    ``m' = max(m_a, m_b)``; ``l' = l_a e^{m_a-m'} + l_b e^{m_b-m'}``;
    ``O' = (l_a O_a e^{m_a-m'} + l_b O_b e^{m_b-m'}) / l'``
    (sp_flatt_csr_kernel.cu:171-193).  A side with ``l == 0`` contributes nothing,
    whatever its ``O`` holds - the convention ``m=-inf, l=0, out=0`` of a fresh
    state (verification/verify.py:73-75).
    """
    m_new = max(m_a, m_b)
    if not np.isfinite(m_new):
        return m_new, 0.0, np.array(o_a, dtype=np.float64)
    wa = l_a * math.exp(m_a - m_new) if l_a != 0.0 else 0.0
    wb = l_b * math.exp(m_b - m_new) if l_b != 0.0 else 0.0
    l_new = wa + wb
    acc = np.zeros_like(np.asarray(o_b, dtype=np.float64))
    if wa != 0.0:
        acc = acc + wa * np.asarray(o_a, dtype=np.float64)
    if wb != 0.0:
        acc = acc + wb * np.asarray(o_b, dtype=np.float64)
    return m_new, l_new, acc / l_new


def rowwise_attention(q, k, v, row_off, col_ind, m=None, l=None, out=None, use_nan=False):
    """Row-by-row float64 attention over adjacency lists, merged into ``(m, l, out)``.

    Follows the reference kernel's per-row steps: row bounds
    (sp_flatt_csr_kernel.cu:29-33), empty row -> optional NaN fill, statistics
    untouched (:45-54), incoming state load (:79-92), scores (:130-138), softmax
    statistics and merge (:142-201), write-back (:208-218).  The chunking of the
    reference loop is an implementation detail with no effect on the mathematics
    and is not restated here.  Returns new arrays.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    n, d = q.shape
    row_off = np.asarray(row_off).astype(np.int64)
    col_ind = np.asarray(col_ind).astype(np.int64)
    m = np.full(n, NEG_INF) if m is None else np.array(m, dtype=np.float64)
    l = np.zeros(n) if l is None else np.array(l, dtype=np.float64)
    out = np.zeros((n, d)) if out is None else np.array(out, dtype=np.float64)
    inv = 1.0 / math.sqrt(float(d))
    for i in range(n):
        lo, hi = row_off[i], row_off[i + 1]
        if hi == lo:
            if use_nan:
                out[i, :] = np.nan
            continue
        cols = col_ind[lo:hi]
        s = (k[cols] @ q[i]) * inv
        mb = s.max()
        p = np.exp(s - mb)
        lb = p.sum()
        ob = (p @ v[cols]) / lb
        m[i], l[i], out[i] = merge_state(m[i], l[i], out[i], mb, lb, ob)
    return out, m, l


def rowwise_query_gradient(q, k, v, d_out, row_off, col_ind):
    """``dQ`` of attention over adjacency lists, row by row (each row only needs its own live
    columns, so a sample of rows of a large problem can be checked).  Same mathematics as
    ``dense_masked_attention_backward``; checked against it in the tests."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    d_out = np.asarray(d_out, dtype=np.float64)
    row_off = np.asarray(row_off).astype(np.int64)
    col_ind = np.asarray(col_ind).astype(np.int64)
    n, d = q.shape
    inv = 1.0 / math.sqrt(float(d))
    d_q = np.zeros((n, d))
    for i in range(n):
        cols = col_ind[row_off[i]:row_off[i + 1]]
        if len(cols) == 0:
            continue
        s = (k[cols] @ q[i]) * inv
        p = np.exp(s - s.max())
        p /= p.sum()
        d_p = v[cols] @ d_out[i]
        d_s = p * (d_p - p @ d_p)
        d_q[i] = (d_s @ k[cols]) * inv
    return d_q


# --------------------------------------------------------------------------
# explicit masks
# --------------------------------------------------------------------------
def csr_from_dense(mask):
    """(row_off[int64 N+1], col_ind[int64 nnz]) of a boolean matrix, columns ascending."""
    mask = np.asarray(mask, dtype=bool)
    counts = mask.sum(axis=1)
    row_off = np.zeros(mask.shape[0] + 1, dtype=np.int64)
    np.cumsum(counts, out=row_off[1:])
    col_ind = np.nonzero(mask)[1].astype(np.int64)
    return row_off, col_ind


def coo_from_dense(mask):
    """(row_ind, col_ind) of a boolean matrix in row-major order (row-sorted)."""
    r, c = np.nonzero(np.asarray(mask, dtype=bool))
    return r.astype(np.int64), c.astype(np.int64)


def dense_from_csr(row_off, col_ind, n_rows, n_cols):
    mask = np.zeros((n_rows, n_cols), dtype=bool)
    row_off = np.asarray(row_off).astype(np.int64)
    col_ind = np.asarray(col_ind).astype(np.int64)
    rows = np.repeat(np.arange(n_rows), np.diff(row_off))
    mask[rows, col_ind] = True
    return mask


def csr_from_coo(row_ind, col_ind, n_rows):
    """Bucket COO entries by row, keeping the entry order inside a row.

    The reference finds ``[low, up)`` of a row by scanning ``W_row_ind``
    (sp_flatt_coo_kernel.cu:47-79), i.e. it needs row-sorted input; as a set
    definition ``live(i) = {col[p] : row[p] == i}`` the order is irrelevant.
    """
    row_ind = np.asarray(row_ind).astype(np.int64)
    col_ind = np.asarray(col_ind).astype(np.int64)
    order = np.argsort(row_ind, kind="stable")
    counts = np.bincount(row_ind, minlength=n_rows)
    row_off = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(counts, out=row_off[1:])
    return row_off, col_ind[order]


# --------------------------------------------------------------------------
# implicit masks, dense constructions (transcribed from verification/verify.py)
# --------------------------------------------------------------------------
def mask_local_dense(n, w):
    """Band |i-j| <= w (verification/verify.py:253-256)."""
    mask = np.zeros((n, n), dtype=bool)
    for i in range(n):
        start = max(0, i - w)
        end = min(n, i + w + 1)
        mask[i, start:end] = True
    return mask


def mask_local_1d_dilated_dense(n, w, dil):
    """Strided band (verification/verify.py:376-382)."""
    mask = np.zeros((n, n), dtype=bool)
    for i in range(n):
        start = max(i - (w * (dil + 1)), i % (dil + 1))
        end = min(i + (w * (dil + 1)), n - 1)
        num_times = ((end - start) // (dil + 1)) + 1
        for j in range(num_times):
            mask[i][start + (j * (dil + 1))] = True
    return mask


def mask_local_2d_dilated_dense(n, block, dil):
    """Block-diagonal with 2-D dilation (verification/verify.py:423-431)."""
    mask = np.zeros((n, n), dtype=bool)
    for i in range(n):
        block_num = i // block
        start = block_num * block
        count = min(block, ((block - 1) // (dil + 1)) + 1)
        if (i - start) % (dil + 1) == 0:
            for j in range(count):
                mask[i][start + (j * (dil + 1))] = True
    return mask


def mask_global_no_local_dense(n, globs, w):
    """Global rows/columns with every row's own window cleared (verification/verify.py:194-205)."""
    mask = np.zeros((n, n), dtype=bool)
    for g in globs:
        mask[int(g), :] = True
        mask[:, int(g)] = True
    for i in range(n):
        left_bound = max(0, i - w)
        right_bound = min(n, i + w) + 1
        mask[i][left_bound:right_bound] = False
    return mask


# --------------------------------------------------------------------------
# implicit masks, per-row column lists (transcribed from the kernels' bounds)
# --------------------------------------------------------------------------
def live_local(n, w, i):
    """sp_flatt_local_kernel.cu:24-28, column rule :101."""
    low = max(0, i - w)
    up = min(n, i + w + 1)
    return np.arange(low, up, dtype=np.int64)


def live_local_1d_dilated(n, w, dil, i):
    """sp_flatt_local_1d_dilated_kernel.cu:25-29, column rule :102 (``t*s + low``)."""
    s = dil + 1
    low = max(i - w * s, i % s)
    up = min(i + w * s, n - 1)
    tot = (up - low) // s + 1
    return low + s * np.arange(tot, dtype=np.int64)


def live_local_2d_dilated(n, block, dil, i):
    """sp_flatt_local_2d_dilated_kernel.cu:26-39, column rule :123."""
    s = dil + 1
    low = (i // block) * block
    if (i - low) % s != 0:
        return np.zeros(0, dtype=np.int64)
    tot = min(block, (block - 1) // s + 1)
    return low + s * np.arange(tot, dtype=np.int64)


def live_global_no_local(n, globs, w, i):
    """sp_flatt_global_no_local_kernel.cu:38-64 (counts) and :134-162 (index map).

    Global row: every column outside ``[low, up)``; other rows: the global
    indices outside ``[low, up)``.
    """
    low = max(0, i - w)
    up = min(n, i + w + 1)
    globs = [int(g) for g in globs]
    if i in globs:
        return np.concatenate([np.arange(0, low), np.arange(up, n)]).astype(np.int64)
    return np.array([g for g in globs if g < low or g > up - 1], dtype=np.int64)


def csr_from_live(n, live_fn):
    """CSR arrays from a per-row column-list function."""
    cols = [np.asarray(live_fn(i), dtype=np.int64) for i in range(n)]
    row_off = np.zeros(n + 1, dtype=np.int64)
    np.cumsum([len(c) for c in cols], out=row_off[1:])
    col_ind = np.concatenate(cols) if cols else np.zeros(0, dtype=np.int64)
    return row_off, col_ind


# --------------------------------------------------------------------------
# nnz closed forms (used as independent checks of the builders above)
# --------------------------------------------------------------------------
def nnz_local(n, w):
    return n * (2 * w + 1) - w * (w + 1)


def nnz_local_2d_dilated(n, block, dil):
    s = dil + 1
    cnt = min(block, (block - 1) // s + 1)
    return (n // block) * cnt * cnt


def nnz_local_1d_dilated(n, w, dil):
    s = dil + 1
    i = np.arange(n, dtype=np.int64)
    low = np.maximum(i - w * s, i % s)
    up = np.minimum(i + w * s, n - 1)
    return int(((up - low) // s + 1).sum())


def nnz_global_no_local(n, globs, w):
    globs = np.unique(np.asarray(globs, dtype=np.int64))
    i = np.arange(n, dtype=np.int64)
    low = np.maximum(0, i - w)
    up = np.minimum(n, i + w + 1)
    win = up - low
    # number of globals inside each row's window
    gs = np.sort(globs)
    inside = np.searchsorted(gs, up, side="left") - np.searchsorted(gs, low, side="left")
    is_g = np.zeros(n, dtype=bool)
    is_g[globs] = True
    per_row = np.where(is_g, n - win, len(globs) - inside)
    return int(per_row.sum())


# --------------------------------------------------------------------------
# parameter validation (the dispatchers' checks, in their order)
# --------------------------------------------------------------------------
MSG_EMB = "The embedded dimension is too large for the amount of shared memory on your GPU."
MSG_LOCAL = "The local size specified is either negative or greater than/equal to (1 - Sequence Length)."
MSG_DIL = "The dilation factor must be atleast 0."
MSG_BLOCK_DIV = "The block/window size must be a divisor of the whole tensor's size."
MSG_BLOCK_DIL = "The dilation factor must be less than the block/window size."
MSG_GLOBS = "There are either no global tokens provided or there are more than the sequence length given."


def check_local(n, w):
    """sp_flatt_local_kernel.cu:252-254."""
    if w < 0 or w > n - 1:
        raise ValueError(MSG_LOCAL)


def check_local_1d_dilated(n, w, dil):
    """sp_flatt_local_1d_dilated_kernel.cu:254-261."""
    if w < 0 or w > n - 1:
        raise ValueError(MSG_LOCAL)
    if dil < 0:
        raise ValueError(MSG_DIL)


def check_local_2d_dilated(n, block, dil):
    """sp_flatt_local_2d_dilated_kernel.cu:274-286."""
    if n % block != 0:
        raise ValueError(MSG_BLOCK_DIV)
    if dil < 0:
        raise ValueError(MSG_DIL)
    if block // (dil + 1) < 1:
        raise ValueError(MSG_BLOCK_DIL)


def check_global_no_local(n, n_globs, w):
    """sp_flatt_global_no_local_kernel.cu:325-334."""
    if n_globs == 0 or n_globs > n:
        raise ValueError(MSG_GLOBS)
    if w < 0 or w > n - 1:
        raise ValueError(MSG_LOCAL)
