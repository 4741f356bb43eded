"""Seeded random sweep over mask parameters, sizes and element types: forward output, statistics
and gradients of every mask kind against the dense float64 oracle.  Sizes are drawn around the
tile sizes of the kernels (32, 64, 128) and the sequence ends, where index arithmetic goes wrong
first."""
import numpy as np
import pytest
import torch

import spfa_autograd
from helpers import np64
from oracle import spfa_oracle as so

pytestmark = pytest.mark.gpu
DEV = "cuda"
OUT_TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}
GRAD_TOL = {torch.float32: 2e-4, torch.bfloat16: 3e-2, torch.float16: 3e-2}


def _draw_case(rng):
    kind = rng.choice(["local", "local_1d_dilated", "local_2d_dilated", "global_no_local", "csr", "coo"])
    d = int(rng.choice([8, 40, 64, 64, 128]))
    dtype = [torch.float32, torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 4))]
    n = int(rng.choice([1, 2, 31, 33, 63, 64, 65, 127, 128, 129, 200, 257, 500]))
    if kind == "local":
        w = int(rng.integers(0, n))
        return kind, n, n, d, dtype, (w,), so.mask_local_dense(n, w)
    if kind == "local_1d_dilated":
        w, dil = int(rng.integers(0, n)), int(rng.integers(0, 5))
        return kind, n, n, d, dtype, (w, dil), so.mask_local_1d_dilated_dense(n, w, dil)
    if kind == "local_2d_dilated":
        divisors = [b for b in range(1, n + 1) if n % b == 0]
        block = int(rng.choice(divisors))
        dil = int(rng.integers(0, block))
        return kind, n, n, d, dtype, (block, dil), so.mask_local_2d_dilated_dense(n, block, dil)
    if kind == "global_no_local":
        g = int(rng.integers(1, min(n, 70) + 1))
        globs = sorted(rng.choice(n, size=g, replace=False).tolist())
        w = int(rng.integers(0, n))
        return kind, n, n, d, dtype, (globs, w), so.mask_global_no_local_dense(n, globs, w)
    n_k = int(rng.choice([1, 50, n, 300]))
    dense = rng.random((n, n_k)) < rng.choice([0.0, 0.02, 0.3, 1.0])
    return kind, n, n_k, d, dtype, (), dense


def _part(kind, args, dense, rng):
    if kind == "csr":
        ro, ci = so.csr_from_dense(dense)
        return ("csr", torch.as_tensor(ro).to(torch.uint64).to(DEV), torch.as_tensor(ci).to(torch.uint32).to(DEV))
    if kind == "coo":
        r, c = so.coo_from_dense(dense)
        perm = rng.permutation(len(r))
        return ("coo", torch.as_tensor(r[perm]).to(torch.uint64).to(DEV),
                torch.as_tensor(c[perm]).to(torch.uint32).to(DEV))
    if kind == "global_no_local":
        return (kind, torch.tensor(args[0], dtype=torch.int32, device=DEV), args[1])
    return (kind, *args)


@pytest.mark.parametrize("seed", range(60))
def test_random_configuration(mods, seed):
    rng = np.random.default_rng(1000 + seed)
    kind, n, n_k, d, dtype, args, dense = _draw_case(rng)
    g = torch.Generator().manual_seed(seed)
    mk = lambda rows: torch.randn(rows, d, generator=g, dtype=torch.float64).to(dtype).to(DEV)
    q, k, v, d_out = mk(n), mk(n_k), mk(n_k), mk(n)
    what = "%s n=%d n_k=%d d=%d %s args=%s" % (kind, n, n_k, d, dtype, args if kind != "global_no_local" else (len(args[0]), args[1]))
    qg, kg, vg = (x.clone().requires_grad_(True) for x in (q, k, v))
    out, m, l = spfa_autograd.attention(qg, kg, vg, [_part(kind, args, dense, rng)], return_state=True)
    out.backward(d_out)
    torch.cuda.synchronize()
    ref_out, ref_m, ref_l = so.dense_masked_attention(np64(q), np64(k), np64(v), dense)
    live = ref_l > 0
    o = np64(out)
    assert np.isfinite(o).all(), what
    if live.any():
        assert np.abs(o[live] - ref_out[live]).max() <= OUT_TOL[dtype], what
        with np.errstate(divide="ignore"):
            lse = np64(m) + np.log(np64(l))
        assert np.abs(lse[live] - (ref_m + np.log(np.where(live, ref_l, 1.0)))[live]).max() <= 2e-3, what
    assert not o[~live].any() and not np64(l)[~live].any(), what  # rows without a live column: untouched
    refs = so.dense_masked_attention_backward(np64(q), np64(k), np64(v), dense, np64(d_out))
    for name, got, want in zip(("dq", "dk", "dv"), (qg.grad, kg.grad, vg.grad), refs):
        got = np64(got)
        assert np.isfinite(got).all(), what + " " + name
        tol = GRAD_TOL[dtype] * max(1.0, float(np.abs(want).max()))
        if dtype != torch.float32:
            tol *= 2  # gradients come back rounded to the element type as well
        assert np.abs(got - want).max() <= tol, "%s %s: %.3e > %.3e" % (what, name, np.abs(got - want).max(), tol)
