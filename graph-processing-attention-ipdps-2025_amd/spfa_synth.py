"""Seeded synthetic workloads for the sparse-attention paths (torch, any device).

Each generator returns plain tensors shaped like what the six ``spfa_*`` modules take.  Masks are
built so that a row never lists a column twice (the kernels, like the reference ones, would count
a repeated entry twice).  All randomness comes from a ``torch.Generator`` seeded by the caller;
streams differ between CPU and GPU generators, so parity checks always move the generated data,
never re-generate it.
"""
from __future__ import annotations

import math

import torch


def _gen(device, seed):
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    return g


def qkv(n, d, dtype=torch.float32, device="cpu", seed=0, scale=1.0, n_k=None):
    """Q [n, d], K and V [n_k, d], iid N(0, scale^2)."""
    g = _gen(device, seed)
    n_k = n if n_k is None else n_k
    q = torch.randn(n, d, generator=g, device=device, dtype=torch.float32) * scale
    k = torch.randn(n_k, d, generator=g, device=device, dtype=torch.float32) * scale
    v = torch.randn(n_k, d, generator=g, device=device, dtype=torch.float32) * scale
    return q.to(dtype), k.to(dtype), v.to(dtype)


def fresh_state(n, d, dtype=torch.float32, device="cpu", state_dtype=None):
    """(m, l, out) = (-inf, 0, 0), the state every first call starts from."""
    sd = dtype if state_dtype is None else state_dtype
    m = torch.full((n,), -float("inf"), device=device, dtype=sd)
    l = torch.zeros(n, device=device, dtype=sd)
    out = torch.zeros(n, d, device=device, dtype=dtype)
    return m, l, out


def zipf_clipped(n, a, kmin, kmax, generator, device):
    """n draws of Zipf(a) (pmf ~ k^-a, k >= 1) clipped to [kmin, kmax], by inverse transform."""
    from scipy.special import zeta

    k = torch.arange(1, kmax, device=device, dtype=torch.float64)
    cdf = torch.cumsum(k.pow(-a) / float(zeta(a, 1)), dim=0)  # P(X <= k), k = 1 .. kmax-1
    u = torch.rand(n, generator=generator, device=device, dtype=torch.float64)
    x = torch.searchsorted(cdf, u, right=True) + 1  # values in 1 .. kmax (the tail lands on kmax)
    return x.clamp_(min=kmin, max=kmax)


def csr_from_degrees(deg, n_cols, generator, device, force_diagonal=True):
    """Rows with exactly deg[i] distinct uniform columns (diagonal included), sorted per row.

    Returns (row_off int64 [n+1], col_ind int64 [nnz]).
    """
    n = deg.numel()
    deg = deg.to(torch.int64).clamp(max=n_cols)
    rows_all = torch.arange(n, device=device, dtype=torch.int64)
    keys = rows_all * n_cols + rows_all.clamp(max=n_cols - 1) if force_diagonal else \
        torch.zeros(0, device=device, dtype=torch.int64)
    need = deg - (1 if force_diagonal else 0)
    need = need.clamp(min=0)
    # draw with replacement, drop repeats, top up the rows that fell short
    for _ in range(64):
        tot = int(need.sum())
        if tot == 0:
            break
        r = torch.repeat_interleave(rows_all, need)
        c = torch.randint(0, n_cols, (tot,), generator=generator, device=device, dtype=torch.int64)
        keys = torch.unique(torch.cat([keys, r * n_cols + c]))
        have = torch.bincount(keys // n_cols, minlength=n)
        need = (deg - have).clamp(min=0)
        # a row can overshoot only through the forced diagonal, never through the draws
    keys, _ = torch.sort(keys)
    rows = keys // n_cols
    cols = keys - rows * n_cols
    counts = torch.bincount(rows, minlength=n)
    row_off = torch.zeros(n + 1, device=device, dtype=torch.int64)
    row_off[1:] = torch.cumsum(counts, 0)
    return row_off, cols


def bernoulli_csr(n, density, device="cpu", seed=0):
    """Random mask: each entry live with probability `density`, plus the diagonal."""
    g = _gen(device, seed)
    mask = torch.rand(n, n, generator=g, device=device) < density
    mask |= torch.eye(n, dtype=torch.bool, device=device)
    counts = mask.sum(dim=1)
    row_off = torch.zeros(n + 1, device=device, dtype=torch.int64)
    row_off[1:] = torch.cumsum(counts, 0)
    cols = mask.nonzero()[:, 1].contiguous()
    return row_off, cols


def zipf_csr(n, a=1.5, kmin=1, kmax=4096, device="cpu", seed=0):
    """Power-law row degrees ~ Zipf(a) clipped to [kmin, kmax], uniform distinct columns."""
    g = _gen(device, seed)
    deg = zipf_clipped(n, a, kmin, min(kmax, n), g, device)
    return csr_from_degrees(deg, n, g, device, force_diagonal=True)


def zipf_coo(n, nnz, a=1.3, device="cpu", seed=0, weight_cap=None):
    """About `nnz` distinct (row, col) pairs, unsorted: rows drawn with probability proportional
    to a Zipf(a) weight per row (capped), columns uniform.  Returns (row int64, col int64)."""
    g = _gen(device, seed)
    cap = weight_cap if weight_cap is not None else max(2, n // 64)
    w = zipf_clipped(n, a, 1, cap, g, device).to(torch.float64)
    cdf = torch.cumsum(w, 0)
    keys = torch.zeros(0, device=device, dtype=torch.int64)
    need = nnz
    for _ in range(16):
        if need <= 0:
            break
        u = torch.rand(need, generator=g, device=device, dtype=torch.float64) * cdf[-1]
        r = torch.searchsorted(cdf, u, right=True).clamp_(max=n - 1)
        c = torch.randint(0, n, (need,), generator=g, device=device, dtype=torch.int64)
        keys = torch.unique(torch.cat([keys, r * n + c]))
        need = nnz - keys.numel()
    perm = torch.randperm(keys.numel(), generator=g, device=device)
    keys = keys[perm]
    rows = keys // n
    return rows, keys - rows * n


def global_indices(n, count, device="cpu", seed=0):
    """`count` distinct global token indices, uniform, int32, ascending."""
    g = _gen(device, seed)
    idx = torch.randperm(n, generator=g, device=device)[:count]
    return torch.sort(idx)[0].to(torch.int32)


def coo_from_csr(row_off, cols, shuffle_seed=None):
    """COO arrays of a CSR mask; with a seed the entries are shuffled."""
    n = row_off.numel() - 1
    rows = torch.repeat_interleave(torch.arange(n, device=cols.device, dtype=torch.int64),
                                   row_off[1:] - row_off[:-1])
    if shuffle_seed is not None:
        g = _gen(cols.device, shuffle_seed)
        perm = torch.randperm(cols.numel(), generator=g, device=cols.device)
        return rows[perm].contiguous(), cols[perm].contiguous()
    return rows, cols


# ---------------------------------------------------------------------------------------------
# work accounting (what the throughput figures are counted on)
# ---------------------------------------------------------------------------------------------
def attention_flops(nnz, d):
    """2d for q.k plus 2d for p.v per live position."""
    return 4 * d * nnz


def explicit_mask_bytes(nnz, n, d, elem_bytes, off_bytes=8, col_bytes=4):
    """Algorithmic bytes of one explicit-mask call: every live position fetches one K row and one
    V row and one column index; every query row reads its offset, Q row, (m, l), and reads and
    writes its out row and writes (m, l)."""
    gathered = nnz * 2 * d * elem_bytes
    total = nnz * (2 * d * elem_bytes + col_bytes) + n * (off_bytes + 3 * d * elem_bytes + 4 * elem_bytes)
    return gathered, total


def implicit_mask_bytes(n, d, elem_bytes, live_rows=None):
    """Compulsory traffic of an implicit-mask call: Q, K, V once, out read + write, m and l."""
    rows = n if live_rows is None else live_rows
    return rows * d * elem_bytes * 5 + 4 * rows * elem_bytes


def local_nnz(n, w):
    return n * (2 * w + 1) - w * (w + 1)


def local_1d_dilated_nnz(n, w, dil):
    s = dil + 1
    i = torch.arange(n, dtype=torch.int64)
    low = torch.maximum(i - w * s, i % s)
    up = torch.clamp(i + w * s, max=n - 1)
    return int(((up - low) // s + 1).sum())


def local_2d_dilated_nnz(n, block, dil):
    s = dil + 1
    cnt = min(block, (block - 1) // s + 1)
    return (n // block) * cnt * cnt


def global_no_local_nnz(n, globs, w):
    g = torch.unique(globs.to(torch.int64).cpu())
    i = torch.arange(n, dtype=torch.int64)
    low = torch.clamp(i - w, min=0)
    up = torch.clamp(i + w + 1, max=n)
    inside = torch.searchsorted(g, up) - torch.searchsorted(g, low)
    is_g = torch.zeros(n, dtype=torch.bool)
    is_g[g] = True
    per_row = torch.where(is_g, n - (up - low), g.numel() - inside)
    return int(per_row.sum())
