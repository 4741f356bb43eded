"""Shared pieces of the GPU parity tests: tolerances, conversions, oracle calls on row samples."""
import numpy as np
import torch

from oracle import c_oracle
from oracle import spfa_oracle as so

# max-abs bars on the output: fp32 1e-4, half types 2e-2
OUT_TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2, torch.float64: 1e-11}
# bar on m + log(l): fp32 statistics 1e-4 / 2e-3 (fp16 inputs, fp32 state) / 3e-3 (bf16: where the
# tile kernels take the row sum off the matrix pipe, l is the sum of the weights as rounded to
# bf16 for the second product - the ones the numerator is built from - and a row that one weight
# dominates carries that weight's rounding, up to 2^-9 = 1.95e-3 relative); statistics stored in
# a half type carry that type's rounding of m (|m| up to ~10): 1e-1
LSE_TOL_F32_STATE = {torch.float32: 1e-4, torch.float16: 2e-3, torch.bfloat16: 3e-3}
LSE_TOL_F64 = 1e-11
LSE_TOL_HALF_STATE = 1e-1


def np64(t):
    if t.dtype == torch.float64:
        return t.detach().cpu().numpy()
    return t.detach().to(torch.float32).cpu().numpy().astype(np.float64)


def lse(m, l):
    with np.errstate(divide="ignore", invalid="ignore"):
        return m + np.log(l)


def check(out, m, l, ref_out, ref_m, ref_l, dtype, state_dtype=None, dead_expect=None, out0=None,
          check_m=True):
    """Compare a GPU result with the oracle's.

    Rows with ref_l == 0 saw no live column: their out must be NaN (dead_expect == "nan") or
    equal to what was there before (out0 rows, default zeros), and m, l must be untouched
    (the caller passes the incoming state as ref_m / ref_l for those rows).
    """
    o, mm, ll = np64(out), np64(m), np64(l)
    state_dtype = dtype if state_dtype is None else state_dtype
    live = np.asarray(ref_l) > 0
    assert np.isfinite(o[live]).all(), "non-finite values in live rows"
    err = np.abs(o[live] - ref_out[live]).max() if live.any() else 0.0
    assert err <= OUT_TOL[dtype], "out max-abs error %.3e > %.1e" % (err, OUT_TOL[dtype])
    if dtype == torch.float64:
        tol = LSE_TOL_F64
    else:
        tol = LSE_TOL_F32_STATE[dtype] if state_dtype == torch.float32 else LSE_TOL_HALF_STATE
    if live.any():
        lerr = np.abs(lse(mm, ll)[live] - lse(np.asarray(ref_m), np.asarray(ref_l))[live]).max()
        assert lerr <= tol, "m + log l error %.3e > %.1e" % (lerr, tol)
        if check_m and state_dtype == torch.float32 and dtype == torch.float32:
            assert np.abs(mm[live] - np.asarray(ref_m)[live]).max() <= 1e-4
    dead = ~live
    if dead.any():
        if dead_expect == "nan":
            assert np.isnan(o[dead]).all(), "dead rows must be NaN"
        else:
            expect = np.zeros_like(o[dead]) if out0 is None else np64(out0)[dead]
            assert np.array_equal(o[dead], expect), "dead rows must be untouched"
    return err


def csr_rows_subset(row_off, cols, rows):
    """CSR arrays (numpy int64) restricted to the listed rows."""
    ro = np.asarray(row_off.cpu() if torch.is_tensor(row_off) else row_off).astype(np.int64)
    ci = cols.cpu().numpy().astype(np.int64) if torch.is_tensor(cols) else np.asarray(cols, np.int64)
    lens = ro[rows + 1] - ro[rows]
    sub_off = np.zeros(len(rows) + 1, dtype=np.int64)
    np.cumsum(lens, out=sub_off[1:])
    sub_cols = np.concatenate([ci[ro[r]:ro[r + 1]] for r in rows]) if len(rows) else np.zeros(0, np.int64)
    return sub_off, sub_cols


def oracle_rows(q, k, v, rows, live_fn):
    """Oracle result for a sample of query rows, live columns given by live_fn(i)."""
    cols = [np.asarray(live_fn(int(i)), dtype=np.int64) for i in rows]
    off = np.zeros(len(rows) + 1, dtype=np.int64)
    np.cumsum([len(c) for c in cols], out=off[1:])
    ci = np.concatenate(cols) if cols else np.zeros(0, np.int64)
    return c_oracle.csr(np64(q)[rows], np64(k), np64(v), off, ci, use_nan=False)
