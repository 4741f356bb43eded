"""Mask arrays of the explicit-mask modules from torch's sparse tensor classes.

The reference's callers build their masks as torch sparse tensors and pull the index arrays out by
hand (verification/verify.py:66-71 for CSR, 93-98 for COO).  These helpers do the same
conversions, with the index types the kernels read without a further cast, so that

    row_off, col_ind, val = spfa_masks.csr_arrays(mask.to_sparse_csr())
    plan = spfa_csr.plan(row_off, col_ind)
    spfa_csr.forward_planned(q, k, v, row_off, col_ind, val, m, l, out, use_nan, plan)

is the whole path from a dense boolean mask to repeated calls.
"""
import torch


def csr_arrays(sparse_csr, value_dtype=None):
    """(w_row_off uint64, w_col_ind uint32, w_val) of a 2-D torch.sparse_csr tensor
    (verification/verify.py:68-71).  w_val is only type-checked by forward(); value_dtype casts it
    to the element type of Q when the mask was built in another type."""
    if sparse_csr.layout != torch.sparse_csr or sparse_csr.dim() != 2:
        raise ValueError("expected a 2-D torch.sparse_csr tensor")
    w_row_off = sparse_csr.crow_indices().to(torch.uint64).contiguous()
    w_col_ind = sparse_csr.col_indices().to(torch.uint32).contiguous()
    w_val = sparse_csr.values()
    if value_dtype is not None:
        w_val = w_val.to(value_dtype)
    return w_row_off, w_col_ind, w_val.contiguous()


def coo_arrays(sparse_coo, value_dtype=None):
    """(w_row_ind uint64, w_col_ind uint32, w_val) of a 2-D torch.sparse_coo tensor
    (verification/verify.py:95-98).  Coalesced tensors come out sorted by row, the order the
    reference's kernel needs; this build accepts any order."""
    if sparse_coo.layout != torch.sparse_coo or sparse_coo.dim() != 2:
        raise ValueError("expected a 2-D torch.sparse_coo tensor")
    idx = sparse_coo.indices()
    w_row_ind = idx[0].to(torch.uint64).contiguous()
    w_col_ind = idx[1].to(torch.uint32).contiguous()
    w_val = sparse_coo.values()
    if value_dtype is not None:
        w_val = w_val.to(value_dtype)
    return w_row_ind, w_col_ind, w_val.contiguous()


def stack_csr_masks(masks, n_cols):
    """One CSR mask for several problems that each have a mask of their own (heads with different
    masks): problem b's rows and columns are shifted by b * n_rows and b * n_cols, so the masks
    form a block diagonal and

        row_off, col_ind = stack_csr_masks([(ro_0, ci_0), (ro_1, ci_1), ...], n_cols)
        spfa_csr.forward(q.reshape(-1, d), k.reshape(-1, d), v.reshape(-1, d), row_off, col_ind, w_val,
                         m.reshape(-1), l.reshape(-1), out.reshape(-1, d), use_nan)

    runs all of them in one call on the stacked [B * n, d] tensors (the batched call with leading
    dimensions is for problems that SHARE a mask).  masks: sequence of (w_row_off, w_col_ind), all
    with the same number of rows; returns (uint64 offsets, uint32 columns)."""
    masks = list(masks)
    if not masks:
        raise ValueError("no masks given")
    n_rows = masks[0][0].numel() - 1
    offs, cols = [], []
    base = 0
    for b, (ro, ci) in enumerate(masks):
        if ro.numel() - 1 != n_rows:
            raise ValueError("all masks must have the same number of rows")
        ro64 = ro.to(torch.int64)
        offs.append(ro64[:-1] + base if b + 1 < len(masks) else ro64 + base)
        cols.append(ci.to(torch.int64) + b * n_cols)
        base += int(ro64[-1])
    if len(masks) * n_cols >= 1 << 32:
        raise ValueError("stacked column indices do not fit 32 bits")
    return torch.cat(offs).to(torch.uint64).contiguous(), torch.cat(cols).to(torch.uint32).contiguous()
