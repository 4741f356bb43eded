"""Differentiable masked attention on top of the spfa_* modules.

The reference binds `forward` only (Sparse_FlashAttention_CSR/sp_flatt_csr.cpp:57-59) and its
callers chain calls on one (m, l, out) state to combine masks (verification/verify.py:337-352).
`attention` is that chain as one autograd function: the forward pass runs the parts in order on a
fresh state, the backward pass runs each part's `backward` against the finished state, all adding
into the same gradients.

    parts = [("local", 64), ("global_no_local", globs, 64), ("csr", row_off, col_ind)]
    out = spfa_autograd.attention(q, k, v, parts)
    out.sum().backward()

Parts (their masks must not overlap, as with chained forward calls):
    ("csr", w_row_off, w_col_ind[, t_row_off, t_col_ind])   - see csr_part()
    ("coo", w_row_ind, w_col_ind)
    ("local", w)                            ("local_1d_dilated", w, dilation)
    ("local_2d_dilated", block, dilation)   ("global_no_local", global_inds int32, w)
Rows that no part gives a live column come out as zeros and carry no gradient.
"""
import importlib

import torch

_KINDS = ("csr", "coo", "local", "local_1d_dilated", "local_2d_dilated", "global_no_local")


def _module(kind):
    if kind not in _KINDS:
        raise ValueError("unknown mask part %r (one of %s)" % (kind, ", ".join(_KINDS)))
    return importlib.import_module("spfa_" + kind)


def _run_forward(kind, args, q, k, v, m, l, out):
    mod = _module(kind)
    if kind in ("csr", "coo"):
        val = torch.empty(0, dtype=q.dtype, device=q.device)  # type-checked, never read
        mod.forward(q, k, v, args[0], args[1], val, m, l, out, False)
    elif kind == "local_2d_dilated":
        mod.forward(q, k, v, m, l, out, args[0], args[1], False)
    else:
        mod.forward(q, k, v, m, l, out, *args)


def _run_backward(kind, args, q, k, v, m, l, out, d_out, d_q, d_k, d_v):
    mod = _module(kind)
    if kind in ("csr", "coo"):
        val = torch.empty(0, dtype=q.dtype, device=q.device)
        mod.backward(q, k, v, args[0], args[1], val, m, l, out, d_out, d_q, d_k, d_v, *args[2:])
    else:
        mod.backward(q, k, v, m, l, out, *args, d_out, d_q, d_k, d_v)


class _MaskedAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, parts):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        state = torch.float64 if q.dtype == torch.float64 else torch.float32
        m = torch.full(q.shape[:-1], float("-inf"), dtype=state, device=q.device)
        l = torch.zeros(q.shape[:-1], dtype=state, device=q.device)
        out = torch.zeros_like(q)
        for part in parts:
            _run_forward(part[0], part[1:], q, k, v, m, l, out)
        ctx.parts = parts
        ctx.save_for_backward(q, k, v, m, l, out)
        ctx.mark_non_differentiable(m, l)
        return out, m, l

    @staticmethod
    def backward(ctx, d_out, _dm, _dl):
        q, k, v, m, l, out = ctx.saved_tensors
        acc = torch.float64 if q.dtype == torch.float64 else torch.float32
        d_q = torch.zeros(q.shape, dtype=acc, device=q.device)
        d_k = torch.zeros(k.shape, dtype=acc, device=q.device)
        d_v = torch.zeros(v.shape, dtype=acc, device=q.device)
        d_out = d_out.contiguous()
        for part in ctx.parts:
            _run_backward(part[0], part[1:], q, k, v, m, l, out, d_out, d_q, d_k, d_v)
        return d_q.to(q.dtype), d_k.to(k.dtype), d_v.to(v.dtype), None


def csr_part(w_row_off, w_col_ind, n_cols):
    """A "csr" part that carries the mask read by column as well, so that backward passes do not
    rebuild it: transpose once, reuse for every step that uses the mask."""
    t_row_off, t_col_ind = importlib.import_module("spfa_csr").transpose(w_row_off, w_col_ind, n_cols)
    return ("csr", w_row_off, w_col_ind, t_row_off, t_col_ind)


def coo_part(w_row_ind, w_col_ind, n_rows, n_cols):
    """COO entries (any order) as a "csr" part with the mask by column attached: converted and
    transposed once, so that no forward or backward pass buckets the entries again."""
    row_off, col_ind = importlib.import_module("spfa_coo").to_csr(w_row_ind, w_col_ind, n_rows)
    return csr_part(row_off, col_ind, n_cols)


def attention(q, k, v, parts, return_state=False):
    """Masked attention over the union of `parts` (see the module text), differentiable in q, k, v.

    q, k, v: [tokens, d] or with leading batch dimensions (the parts' masks are shared by every
    problem of the batch).  Returns out, or (out, m, l) with the softmax statistics when
    return_state is set."""
    parts = tuple(tuple(p) for p in parts)
    if not parts:
        raise ValueError("at least one mask part is needed")
    for p in parts:
        _module(p[0])
    out, m, l = _MaskedAttention.apply(q, k, v, parts)
    return (out, m, l) if return_state else out
