#!/usr/bin/env python3
"""Throughput of the sparse-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--dtype f32|f16|bf16]

Default workload: explicit CSR mask, N=131072, d=64, fp32, Zipf(1.5) row degrees clipped to
[1, 4096], uniform distinct sorted columns, diagonal included (seeded, generated on the device).
One step = one spfa_csr.forward call on a fresh (m, l, out) state with all inputs resident in HBM.

Prints ONE JSON line: nnz-counted GFLOP/s (4*d*nnz flops per step) as `value`, the HBM roofline of
the dominant kernel (algorithmic bytes / its launch time measured with HIP events on the launch
stream), and a CPU baseline timed on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "graph-processing-attention-ipdps-2025_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
FP32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix
HALF_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 / fp16 matrix

WORKLOADS = {
    "csr_zipf": "CSR N=131072 d=64 Zipf(1.5) degrees clipped [1,4096], uniform sorted columns + diagonal",
    "csr_zipf_hbm": "CSR N=4194304 d=64 Zipf(1.5) degrees clipped [1,4096], uniform sorted columns + diagonal "
                    "(the headline generator at a size whose K and V, 2 GiB, do not fit the 256 MiB memory-side cache)",
    "csr_bernoulli": "CSR N=4096 d=64 Bernoulli(2%) + diagonal",
    "coo_zipf": "COO N=1048576 d=64 ~50M unsorted entries, row weights Zipf(1.3), uniform columns",
    "coo_zipf_sorted": "COO N=1048576 d=64 ~50M entries sorted by row, row weights Zipf(1.3), uniform columns",
    "local": "Local N=65536 d=64 LOCAL_SIZE=128 (|i-j|<=128)",
    "local_1d": "Local-1D-dilated N=262144 d=128 LOCAL_SIZE=256 DILATE_FACTOR=2 (stride 3)",
    "local_2d": "Local-2D-dilated N=262144 d=128 BLOCK_SIZE=256 DILATE_FACTOR=2 (stride 3)",
    "global": "Global-no-local N=1048576 d=64 64 global tokens LOCAL_SIZE=64",
    "bigbird": "Window + global + random in one call: N=65536 d=64 LOCAL_SIZE=128, 64 global tokens, "
               "192 random columns per row (CSR)",
}


class HipEvents:
    """hipEvent pair created straight from the HIP runtime (torch.cuda.Event only sees torch's
    own record calls; these are recorded inside the library around one kernel)."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.start = ctypes.c_void_p()
        self.stop = ctypes.c_void_p()
        assert self.hip.hipEventCreate(ctypes.byref(self.start)) == 0
        assert self.hip.hipEventCreate(ctypes.byref(self.stop)) == 0

    def elapsed_ms(self):
        ms = ctypes.c_float()
        assert self.hip.hipEventSynchronize(self.stop) == 0
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), self.start, self.stop)
        assert rc == 0, "hipEventElapsedTime rc=%d" % rc
        return float(ms.value)


def load_library():
    lib_path = os.path.join(os.environ.get("SPFA_LIB_DIR", PKG), "libspfa_hip.so")
    if not os.path.exists(lib_path):
        raise RuntimeError("libspfa_hip.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
    lib = ctypes.CDLL(lib_path)
    lib.spfa_set_kernel_events.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    lib.spfa_set_kernel_events.restype = None
    lib.spfa_explicit_inline_row_limit.restype = ctypes.c_int64
    lib.spfa_explicit_long_rows_on_grid.restype = ctypes.c_int
    lib.spfa_explicit_one_launch_row_limit.restype = ctypes.c_int64
    lib.spfa_explicit_long_rows_on_grid.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
    return lib


def load_probe_library():
    """libspfa_probe.so: the gather without arithmetic (include/spfa_probe.h), a measurement aid kept
    apart from the attention library."""
    path = os.path.join(os.environ.get("SPFA_LIB_DIR", PKG), "libspfa_probe.so")
    if not os.path.exists(path):
        path = os.path.join(PKG, "libspfa_probe.so")
    if not os.path.exists(path):
        raise RuntimeError("libspfa_probe.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
    probe = ctypes.CDLL(path)
    probe.spfa_probe_gather.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    return probe


def make_workload(name, dtype, torch, syn, inline_limit=32, planned=False, heads=1, loop_heads=False, d_local=64,
                  tokens=None):
    """Returns dict(call=fn(state) -> None, n, d, nnz, bytes_total, bytes_gathered, sample=fn())."""
    dev = "cuda"
    es = torch.tensor([], dtype=dtype).element_size()
    w = {"name": name, "desc": WORKLOADS[name]}
    if name in ("csr_zipf", "csr_zipf_hbm", "csr_bernoulli", "coo_zipf", "coo_zipf_sorted"):
        if name in ("csr_zipf", "csr_zipf_hbm"):
            n, d = (131072 if name == "csr_zipf" else 1 << 22), 64
            if tokens is not None and name == "csr_zipf":  # the headline generator at another size
                n = tokens
                w["desc"] = w["desc"].replace("N=131072", "N=%d" % n)
            ro, ci = syn.zipf_csr(n, 1.5, 1, 4096, device=dev, seed=0)
        elif name == "csr_bernoulli":
            n, d = 4096, 64
            ro, ci = syn.bernoulli_csr(n, 0.02, device=dev, seed=0)
        else:
            n, d = 1 << 20, 64
            r, c = syn.zipf_coo(n, 50_000_000, 1.3, device=dev, seed=0)
            if name == "coo_zipf_sorted":
                order = torch.argsort(r, stable=True)
                r, c = r[order].contiguous(), c[order].contiguous()
        q, k, v = syn.qkv(n, d, dtype=dtype, device=dev, seed=0)
        if heads > 1:  # independent problems sharing the mask: [heads, n, d]
            q, k, v = [torch.stack([syn.qkv(n, d, dtype=dtype, device=dev, seed=h)[j] for h in range(heads)])
                       for j in range(3)]
        if name.startswith("coo"):
            import spfa_coo
            nnz = int(c.numel())
            r_t, c_t = r.to(torch.uint64), c.to(torch.uint32)
            val = torch.empty(nnz, device=dev, dtype=dtype)
            w["bwd"] = lambda st, do, g: spfa_coo.backward(q, k, v, r_t, c_t, val, st[0], st[1], st[2], do, *g)
            if planned:
                plan = spfa_coo.plan(r_t, c_t, n)  # mask pre-pass, outside the timed region
                w["call"] = lambda st: spfa_coo.forward_planned(q, k, v, r_t, c_t, val, st[0], st[1], st[2],
                                                                False, plan)
            else:
                w["call"] = lambda st: spfa_coo.forward(q, k, v, r_t, c_t, val, st[0], st[1], st[2], False)
            w["csr"] = None
            w["coo"] = (r, c)
            # the columns in the order the attention kernel walks them (row by row)
            w["probe_idx"] = c[torch.argsort(r, stable=True)].to(torch.int32).contiguous()
            w["probe_sorted_rows"] = True
            off_b = 8
        else:
            import spfa_csr
            nnz = int(ci.numel())
            ro_t, ci_t = ro.to(torch.uint64), ci.to(torch.uint32)
            val = torch.empty(nnz, device=dev, dtype=dtype)
            if planned:
                tr = spfa_csr.transpose(ro_t, ci_t, n)  # the mask by column, for the gradients
                w["bwd"] = lambda st, do, g: spfa_csr.backward(q, k, v, ro_t, ci_t, val, st[0], st[1], st[2],
                                                               do, *g, *tr)
            else:
                w["bwd"] = lambda st, do, g: spfa_csr.backward(q, k, v, ro_t, ci_t, val, st[0], st[1], st[2],
                                                               do, *g)
            if planned:
                plan = spfa_csr.plan(ro_t, ci_t)  # mask pre-pass, outside the timed region
                w["call"] = lambda st: spfa_csr.forward_planned(q, k, v, ro_t, ci_t, val, st[0], st[1], st[2],
                                                                False, plan)
            else:
                w["call"] = lambda st: spfa_csr.forward(q, k, v, ro_t, ci_t, val, st[0], st[1], st[2], False)
            if heads > 1 and loop_heads:  # the reference's way: one call per head
                def looped(st):
                    for h in range(heads):
                        spfa_csr.forward(q[h], k[h], v[h], ro_t, ci_t, val, st[0][h], st[1][h], st[2][h], False)
                w["call"] = looped
            w["csr"] = (ro, ci)
            w["probe_idx"] = ci.to(torch.int32).contiguous()
            off_b = 8
        gathered, total = syn.explicit_mask_bytes(nnz, n, d, es, off_bytes=off_b)
        if name.startswith("coo"):
            total += nnz * 8  # row index of every entry
            deg = torch.bincount(r, minlength=n)
        else:
            deg = ro[1:] - ro[:-1]
        # the dominant (segment) kernel owns the rows longer than the library's in-place limit
        long_rows = deg > inline_limit
        nnz_long, rows_long = int(deg[long_rows].sum()), int(long_rows.sum())
        if nnz_long > 0:  # the ceiling probe walks what the segment kernel walks: the long rows' columns
            w["probe_idx"] = handed_out_order(w["probe_idx"][torch.repeat_interleave(long_rows, deg)],
                                              deg[long_rows], torch)
        _, kernel_bytes = syn.explicit_mask_bytes(nnz_long, rows_long, d, es, off_bytes=off_b)
        w.update(n=n, d=d, nnz=nnz * heads, bytes_total=total * heads, bytes_gathered=gathered * heads,
                 bound="hbm", kernel_bytes=kernel_bytes * heads, kernel_nnz=nnz_long * heads,
                 kernel_rows=rows_long * heads)
    else:
        if name == "local":
            import spfa_local
            n, d, wsz = 65536, d_local, 128
            if d != 64:
                w["desc"] = "Local N=65536 d=%d LOCAL_SIZE=128 (|i-j|<=128)" % d
            if heads > 1:  # many heads of a short sequence instead of one long one
                n = 4096
                w["desc"] = "Local N=4096 d=%d LOCAL_SIZE=128 (|i-j|<=128)" % d
            q, k, v = syn.qkv(n, d, dtype=dtype, device=dev, seed=0)
            if heads > 1:
                q, k, v = [torch.stack([syn.qkv(n, d, dtype=dtype, device=dev, seed=h)[j] for h in range(heads)])
                           for j in range(3)]
            nnz = syn.local_nnz(n, wsz)
            w["call"] = lambda st: spfa_local.forward(q, k, v, st[0], st[1], st[2], wsz)
            w["bwd"] = lambda st, do, g: spfa_local.backward(q, k, v, st[0], st[1], st[2], wsz, do, *g)
            if heads > 1 and loop_heads:
                def looped(st):
                    for h in range(heads):
                        spfa_local.forward(q[h], k[h], v[h], st[0][h], st[1][h], st[2][h], wsz)
                w["call"] = looped
            w["params"] = {"LOCAL_SIZE": wsz}
            live = n
        elif name == "local_1d":
            import spfa_local_1d_dilated
            n, d, wsz, dil = 262144, 128, 256, 2
            q, k, v = syn.qkv(n, d, dtype=dtype, device=dev, seed=0, scale=0.5)
            nnz = syn.local_1d_dilated_nnz(n, wsz, dil)
            w["call"] = lambda st: spfa_local_1d_dilated.forward(q, k, v, st[0], st[1], st[2], wsz, dil)
            w["bwd"] = lambda st, do, g: spfa_local_1d_dilated.backward(q, k, v, st[0], st[1], st[2], wsz, dil,
                                                                        do, *g)
            w["params"] = {"LOCAL_SIZE": wsz, "DILATE_FACTOR": dil}
            live = n
        elif name == "local_2d":
            import spfa_local_2d_dilated
            n, d, blk, dil = 262144, 128, 256, 2
            q, k, v = syn.qkv(n, d, dtype=dtype, device=dev, seed=0, scale=0.5)
            nnz = syn.local_2d_dilated_nnz(n, blk, dil)
            w["call"] = lambda st: spfa_local_2d_dilated.forward(q, k, v, st[0], st[1], st[2], blk, dil, False)
            w["bwd"] = lambda st, do, g: spfa_local_2d_dilated.backward(q, k, v, st[0], st[1], st[2], blk, dil,
                                                                        do, *g)
            w["params"] = {"BLOCK_SIZE": blk, "DILATE_FACTOR": dil}
            live = (n // blk) * min(blk, (blk - 1) // (dil + 1) + 1)
        elif name == "bigbird":
            import spfa_bigbird
            import spfa_csr
            import spfa_global_no_local
            import spfa_local
            n, d, g, wsz, per_row = 65536, 64, 64, 128, 192
            q, k, v = syn.qkv(n, d, dtype=dtype, device=dev, seed=0)
            globs = syn.global_indices(n, g, device=dev, seed=0)
            # random part: per_row columns per row, none inside the window or among the globals
            gen = torch.Generator(device=dev).manual_seed(0)
            cols = torch.randint(0, n, (n, per_row), generator=gen, device=dev)
            rows = torch.arange(n, device=dev).unsqueeze(1)
            is_glob = torch.zeros(n, dtype=torch.bool, device=dev)
            is_glob[globs.long()] = True
            keep = ((cols - rows).abs() > wsz) & ~is_glob[cols] & ~is_glob[rows.expand_as(cols)]
            cols_sorted, _ = torch.sort(torch.where(keep, cols, torch.full_like(cols, n)), dim=1)
            dup = torch.zeros_like(keep)
            dup[:, 1:] = cols_sorted[:, 1:] == cols_sorted[:, :-1]
            keep = (cols_sorted < n) & ~dup
            ro = torch.zeros(n + 1, dtype=torch.int64, device=dev)
            ro[1:] = torch.cumsum(keep.sum(dim=1), 0)
            ci = cols_sorted[keep]
            ro_t, ci_t = ro.to(torch.uint64), ci.to(torch.uint32)
            val = torch.empty(ci.numel(), device=dev, dtype=dtype)
            nnz_csr = int(ci.numel())
            nnz = syn.local_nnz(n, wsz) + syn.global_no_local_nnz(n, globs, wsz) + nnz_csr
            if loop_heads:  # (re-used flag) the reference's way: three chained calls
                def chained(st):
                    spfa_local.forward(q, k, v, st[0], st[1], st[2], wsz)
                    spfa_global_no_local.forward(q, k, v, st[0], st[1], st[2], globs, wsz)
                    spfa_csr.forward(q, k, v, ro_t, ci_t, val, st[0], st[1], st[2], False)
                w["call"] = chained
            else:
                w["call"] = lambda st: spfa_bigbird.forward(q, k, v, st[0], st[1], st[2], wsz, globs, ro_t, ci_t, val)
            tr = spfa_csr.transpose(ro_t, ci_t, n) if planned else ()  # the random part by column
            w["bwd"] = lambda st, do, gr: spfa_bigbird.backward(q, k, v, st[0], st[1], st[2], wsz, globs, ro_t,
                                                                ci_t, val, do, *gr, *tr)
            w["params"] = {"n_globals": g, "LOCAL_SIZE": wsz, "csr_nnz": nnz_csr}
            w["globs"] = globs
            w["csr"] = (ro, ci)
            w["probe_idx"] = ci.to(torch.int32).contiguous()
            w["whole_call"] = True
            live = n
            w["extra_bytes"] = syn.explicit_mask_bytes(nnz_csr, n, d, es, off_bytes=8)[1]
        else:
            import spfa_global_no_local
            n, d, g, wsz = 1 << 20, 64, 64, 64
            q, k, v = syn.qkv(n, d, dtype=dtype, device=dev, seed=0)
            globs = syn.global_indices(n, g, device=dev, seed=0)
            nnz = syn.global_no_local_nnz(n, globs, wsz)
            w["call"] = lambda st: spfa_global_no_local.forward(q, k, v, st[0], st[1], st[2], globs, wsz)
            w["bwd"] = lambda st, do, gr: spfa_global_no_local.backward(q, k, v, st[0], st[1], st[2], globs, wsz,
                                                                        do, *gr)
            w["params"] = {"n_globals": g, "LOCAL_SIZE": wsz}
            w["globs"] = globs
            live = n
            # live positions of the global rows alone (what the event-timed kernel covers)
            w["n_global_rows_nnz"] = g * n - int(sum(min(n, int(x) + wsz + 1) - max(0, int(x) - wsz)
                                                      for x in globs.cpu().tolist()))
        total = syn.implicit_mask_bytes(n, d, es, live_rows=live) + w.get("extra_bytes", 0)
        w.update(n=n, d=d, nnz=nnz * heads, bytes_total=total * heads, bytes_gathered=nnz * 2 * d * es * heads,
                 bound="hbm", kernel_bytes=total * heads, kernel_nnz=nnz * heads, kernel_rows=live * heads)
    w.update(q=q, k=k, v=v, heads=heads)
    return w


def live_columns_fn(w, torch):
    """i -> numpy array of the live columns of query row i of the workload's mask."""
    import numpy as np
    from oracle import spfa_oracle as so
    n, name = w["n"], w["name"]
    if name.startswith("csr"):
        ro, ci = w["csr"]
        ro_c = ro.cpu().numpy()
        return lambda i: ci[ro_c[i]:ro_c[i + 1]].cpu().numpy()
    if name.startswith("coo"):
        # (the entries are bucketed by row once; a compare over all of them per sampled row would
        # take minutes for a block of the CPU baseline)
        r, c = w["coo"]
        order = torch.argsort(r, stable=True)
        c_sorted = c[order]
        off = torch.searchsorted(r[order].contiguous(), torch.arange(n + 1, device=r.device)).cpu().numpy()
        del order
        return lambda i: c_sorted[off[i]:off[i + 1]].cpu().numpy()
    if name == "local":
        return lambda i: so.live_local(n, w["params"]["LOCAL_SIZE"], int(i))
    if name == "local_1d":
        p = w["params"]
        return lambda i: so.live_local_1d_dilated(n, p["LOCAL_SIZE"], p["DILATE_FACTOR"], int(i))
    if name == "local_2d":
        p = w["params"]
        return lambda i: so.live_local_2d_dilated(n, p["BLOCK_SIZE"], p["DILATE_FACTOR"], int(i))
    gl = w["globs"].cpu().numpy()
    gset = set(int(x) for x in gl)
    wsz = w["params"]["LOCAL_SIZE"]
    if name == "bigbird":
        ro, ci = w["csr"]
        ro_c = ro.cpu().numpy()

        def live_bb(i):
            low, up = max(0, i - wsz), min(n, i + wsz + 1)
            if i in gset:
                return np.arange(0, n)
            outside = np.array([x for x in gl if x < low or x >= up], dtype=np.int64)
            return np.concatenate([np.arange(low, up), outside, ci[ro_c[i]:ro_c[i + 1]].cpu().numpy()])
        return live_bb

    def live_global(i):
        low, up = max(0, i - wsz), min(n, i + wsz + 1)
        if i in gset:
            return np.concatenate([np.arange(0, low), np.arange(up, n)])
        return np.array([x for x in gl if x < low or x >= up], dtype=np.int64)
    return live_global


def verify_sample(w, state, torch, rows=192, d_out=None, d_q=None):
    """Max-abs error of `rows` sampled output rows against the float64 CPU oracle; with d_out and
    d_q, of the sampled rows of the query gradient instead (relative to its largest entry)."""
    import numpy as np
    from oracle import c_oracle
    from oracle import spfa_oracle as so
    n = w["n"]
    if w.get("heads", 1) > 1:  # a batch of heads: the last one is checked
        w = dict(w, q=w["q"][-1], k=w["k"][-1], v=w["v"][-1])
        state = [x[-1] for x in state]
        if d_out is not None:
            d_out, d_q = d_out[-1], d_q[-1]
    g = torch.Generator().manual_seed(123)
    idx_np = torch.sort(torch.randperm(n, generator=g)[:rows])[0].numpy()
    name = w["name"]
    if name.startswith("coo"):
        idx_np = idx_np[:32]
    elif name in ("bigbird", "global"):
        # one global row is enough (each is an n-column row for the CPU)
        idx_np = np.concatenate([idx_np[:63], w["globs"].cpu().numpy()[:1].astype(np.int64)])
    qs = w["q"][torch.as_tensor(idx_np).to("cuda")].float().cpu().numpy().astype(np.float64)
    kk = w["k"].float().cpu().numpy().astype(np.float64)
    vv = w["v"].float().cpu().numpy().astype(np.float64)
    live = live_columns_fn(w, torch)
    lists = [live(int(i)) for i in idx_np]
    off = np.zeros(len(lists) + 1, dtype=np.int64)
    np.cumsum([len(x) for x in lists], out=off[1:])
    cols = np.concatenate(lists).astype(np.int64) if len(lists) else np.zeros(0, np.int64)
    sel = torch.as_tensor(idx_np).to("cuda")
    if d_out is not None:
        ref = so.rowwise_query_gradient(qs, kk, vv, d_out[sel].float().cpu().numpy().astype(np.float64), off, cols)
        got = d_q[sel].float().cpu().numpy().astype(np.float64)
        return float(np.abs(got - ref).max() / max(1.0, np.abs(ref).max())), len(idx_np)
    ref_out, ref_m, ref_l = c_oracle.csr(qs, kk, vv, off, cols)
    got = state[2][sel].float().cpu().numpy().astype(np.float64)
    live_rows = ref_l > 0
    err = float(np.abs(got[live_rows] - ref_out[live_rows]).max()) if live_rows.any() else 0.0
    return err, int(live_rows.sum())


def cpu_baseline(w, torch, target_s=12.0):
    """The reference's verification formulation on host cores: dense masked
    scaled_dot_product_attention in fp32 over blocks of query rows against all keys
    (verification/verify.py:61-63).  The dense formulation costs the same for every query row
    whatever its mask, so the whole job is the sampled blocks' time scaled to all n rows, and the
    nnz-counted rate credits it with the workload's live positions."""
    n, d = w["n"], w["d"]
    heads = w.get("heads", 1)
    if heads > 1:
        w = dict(w, q=w["q"][-1], k=w["k"][-1], v=w["v"][-1])
    k = w["k"].float().cpu()
    v = w["v"].float().cpu()
    q = w["q"].float().cpu()
    # scores of a block are block x n floats (twice, with the softmax) plus the boolean mask
    block = int(min(1024, n, max(64, (1 << 28) // n)))
    g = torch.Generator().manual_seed(7)
    live = live_columns_fn(w, torch)

    def one_block():
        rows = torch.sort(torch.randperm(n, generator=g)[:block])[0]
        mask = torch.zeros(block, n, dtype=torch.bool)
        for j, i in enumerate(rows.tolist()):
            cols = torch.as_tensor(live(i), dtype=torch.int64)
            mask[j, cols] = True
        qb = q[rows]
        t0 = time.perf_counter()
        torch.nn.functional.scaled_dot_product_attention(qb, k, v, attn_mask=mask)
        return time.perf_counter() - t0

    one_block()  # warm-up
    t_tot, blocks = 0.0, 0
    t_begin = time.perf_counter()
    while (time.perf_counter() - t_begin) < target_s and blocks < 64:
        t_tot += one_block()
        blocks += 1
    job_s = t_tot / blocks * (n / block)  # one head
    nnz_head = w["nnz"] / heads
    return {
        "value": 4.0 * d * nnz_head / job_s / 1e9, "unit": "GFLOP/s (nnz-counted)",
        "cores": torch.get_num_threads(), "kind": "port",
        "sample": "%d blocks of %d random query rows x all %d keys, torch CPU dense masked "
                  "scaled_dot_product_attention fp32 (the reference's verification formulation), "
                  "%.2f s of SDPA time; scaled to all %d rows (%.1f s for the whole mask) and "
                  "credited with its %d live positions" % (blocks, block, n, t_tot, n, job_s, nnz_head),
        "dense_gflops": 4.0 * d * block * blocks * n / t_tot / 1e9, "host_cpus": os.cpu_count(),
        "whole_job_s": job_s,
    }


def cpu_sparse_port(w, torch, rows=8192):
    """The row-wise C restatement (float64, OpenMP) on a sample of rows - the same sparse algorithm
    as the GPU path, for scale."""
    import numpy as np
    from oracle import c_oracle
    if not w["name"].startswith("csr"):
        return None
    n, d = w["n"], w["d"]
    ro, ci = w["csr"]
    ro_c, ci_c = ro.cpu().numpy(), ci.cpu().numpy()
    g = torch.Generator().manual_seed(11)
    idx = torch.sort(torch.randperm(n, generator=g)[:min(rows, n)])[0].numpy()
    lens = ro_c[idx + 1] - ro_c[idx]
    off = np.zeros(len(idx) + 1, dtype=np.int64)
    np.cumsum(lens, out=off[1:])
    cols = np.concatenate([ci_c[ro_c[i]:ro_c[i + 1]] for i in idx]).astype(np.int64)
    qs = w["q"].float().cpu().numpy().astype(np.float64)[idx]
    kk = w["k"].float().cpu().numpy().astype(np.float64)
    vv = w["v"].float().cpu().numpy().astype(np.float64)
    c_oracle.csr(qs[:64], kk, vv, off[:65], cols[:off[64]])
    t0 = time.perf_counter()
    c_oracle.csr(qs, kk, vv, off, cols)
    t = time.perf_counter() - t0
    return {"value": 4.0 * d * int(lens.sum()) / t / 1e9, "unit": "GFLOP/s (nnz-counted)",
            "cores": os.cpu_count(), "kind": "port",
            "sample": "%d random rows, row-wise sparse float64 C restatement with OpenMP, %.2f s" % (len(idx), t)}


def measured_traffic(workload, dtype_name):
    """HBM-side bytes per launch of the dominant kernel from the committed counter summary of this
    workload (profiles/<workload>..._pmc.md, line `traffic_bytes_per_launch = N`), else None."""
    import glob
    import re
    names = {"csr_zipf": "csr_zipf_n131072_d64", "coo_zipf": "coo_zipf_unsorted_n1048576_d64",
             "csr_zipf_hbm": "csr_zipf_hbm_n4194304_d64"}
    stem = names.get(workload)
    if stem is None:
        return None, None
    for path in glob.glob(os.path.join(ROOT, "profiles", "%s_%s_pmc.md" % (stem, {"f32": "f32"}.get(dtype_name, dtype_name)))):
        m = re.search(r"^traffic_bytes_per_launch\s*=\s*(\d+)", open(path).read(), re.M)
        if m:
            return int(m.group(1)), os.path.relpath(path, ROOT)
    return None, None


def bench_backward(a, w, st, dtype, torch, syn, lib):
    """--backward: one forward call builds the state, then K timed gradient calls (they add into
    the same dQ, dK, dV; the parity check afterwards starts from zeroed gradients)."""
    if a.loop_heads:
        sys.exit("bench.py: --backward times the batched / single call only")
    n, d, nnz = w["n"], w["d"], w["nnz"]
    es = torch.tensor([], dtype=dtype).element_size()
    w["call"](st)
    gen = torch.Generator(device="cuda").manual_seed(1)
    d_out = torch.randn(w["q"].shape, device="cuda", generator=gen).to(dtype)
    grads = tuple(torch.zeros(x.shape, device="cuda", dtype=torch.float32) for x in (w["q"], w["k"], w["v"]))
    for _ in range(a.warmup):
        w["bwd"](st, d_out, grads)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        w["bwd"](st, d_out, grads)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / a.steps * 1e3
    for g in grads:
        g.zero_()
    w["bwd"](st, d_out, grads)
    torch.cuda.synchronize()
    err, checked = verify_sample(w, st, torch, rows=64, d_out=d_out, d_q=grads[0])
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    # every live row's weights sum to one: the columns of dV add up to those of dO
    live = (st[1] > 0).double().unsqueeze(-1)
    col_err = float(((grads[2].double().sum(dim=-2) - (d_out.double() * live).sum(dim=-2)).abs().max()
                     / d_out.double().abs().sum(dim=-2).max()))
    # Algorithmic work: five products of length d per live position (scores, dO.V, dQ, dK, dV).
    # Bytes: the dense tensors once (q, k, v, out, dO read; dQ, dK, dV read and written in fp32);
    # a position that a GATHER pass processes also fetches K, V rows (query pass) and Q, dO rows
    # (key pass) and two index words; a position that a TILE kernel processes is matrix work on
    # streamed tiles and fetches nothing of its own.  The composite's window and listed-token
    # positions are tile work, only its random (CSR) part is gathered.
    heads = w.get("heads", 1)
    name = w["name"]
    explicit = name.startswith(("csr", "coo"))
    flops = 10.0 * d * nnz
    # (a 2-D dilated mask touches only the rows that have a live column)
    rows_touched = heads * n if (explicit or name == "bigbird") else w["kernel_rows"]
    dense = rows_touched * d * (5 * es + 6 * 4)
    nnz_gather = nnz if explicit else (w["params"]["csr_nnz"] if name == "bigbird" else 0)
    nnz_tiles = nnz - nnz_gather
    gathered = nnz_gather * 4 * d * es
    index = nnz_gather * 8
    total = dense + gathered + index
    t_s = ms_per_step * 1e-3
    mfma_peak = FP32_PEAK_TFLOPS if a.dtype == "f32" else HALF_PEAK_TFLOPS
    # What the gather passes can be served at: the published HBM rate when Q, K, V, dO together do
    # not fit the 256 MiB memory-side cache, else what the same gather without arithmetic sustains
    # on this device - for the query pass over K, V and the mask's entries in row order (as for
    # the forward call), for the key pass over Q, dO and the entries in column order (a mask with
    # a few very long rows makes that a gather from a small hot set of Q / dO rows, which the L2
    # serves: its ceiling is well above the query pass's).
    ws_bytes = 4 * w["k"].numel() * es
    gq = gk = None
    if nnz_gather and ws_bytes <= (256 << 20):
        gq = measured_gather_ceiling(lib, w, torch)
        if w.get("csr") is not None:
            ro_m, ci_m = w["csr"]
            rows_of = torch.repeat_interleave(torch.arange(ro_m.numel() - 1, device=ci_m.device), ro_m[1:] - ro_m[:-1])
            idx_t = rows_of[torch.argsort(ci_m, stable=True)].to(torch.int32).contiguous()
        else:
            r_m, c_m = w["coo"]
            idx_t = r_m[torch.argsort(c_m, stable=True)].to(torch.int32).contiguous()
        gk = measured_gather_ceiling(lib, w, torch, tensors=(w["q"], d_out), idx=idx_t)
        del idx_t
    if gq is None or gk is None:
        peak_q = peak_k = HBM_PEAK_GBS
        gather_src = "MI355X HBM3E, published"
        gather_bound = "hbm"
    else:
        peak_q, peak_k = gq["GBs"], gk["GBs"]
        gather_src = "measured on this device: the same gathers without arithmetic (spfa_probe_gather), " \
                     "query pass over K, V by row-ordered entries, key pass over Q, dO by column-ordered entries"
        gather_bound = "l2" if ws_bytes <= (4 << 20) else "infinity_cache"
    half_bytes = (gathered + index) / 2.0
    gather_ms = (half_bytes / (peak_q * 1e9) + half_bytes / (peak_k * 1e9)) * 1e3 if nnz_gather else 0.0
    gather_peak = (gathered + index) / (gather_ms * 1e-3) / 1e9 if nnz_gather else None
    tile_flops = 10.0 * d * nnz_tiles
    dense_ms = dense / (HBM_PEAK_GBS * 1e9) * 1e3
    mfma_ms = tile_flops / (mfma_peak * 1e12) * 1e3
    # the gather passes and the tile kernels run one after the other: the floor of the call is the
    # gather time plus the larger of the dense tensors' HBM time and the tiles' matrix time
    roof_ms = gather_ms + max(dense_ms, mfma_ms)
    half_band = a.dtype != "f32" and d in (64, 128) and name in ("local", "local_1d", "local_2d", "bigbird")
    tile_kernels = ("band_grad_dma_kernel (query pass, key pass%s)" % (" as dK and dV launches" if d == 128 else "")
                    if half_band else "tile_grad_kernel (query pass, key pass)")
    if name == "global" or name == "bigbird":
        tile_kernels += " + tile_grad_kernel / global_grad_merge_kernel for the listed tokens"
    gather_kernels = "grad_prologue_kernel, grad_rows_kernel (query pass, key pass), order_kernel, grad_segments_kernel" + \
                     (", mask transposition" if not a.planned and name.startswith(("csr", "bigbird")) else "") + \
                     (", two COO bucketing pre-passes" if name.startswith("coo") else "")
    if gather_ms >= max(dense_ms, mfma_ms):
        bound, unit = gather_bound, "GB/s"
        achieved, peak = total / t_s / 1e9, gather_peak
    elif dense_ms >= mfma_ms:
        bound, unit = "hbm", "GB/s"
        achieved, peak = total / t_s / 1e9, HBM_PEAK_GBS
    else:
        bound, unit = "mfma", "TFLOP/s"
        achieved, peak = flops / t_s / 1e12, mfma_peak
    roofline = {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit,
                "frac": roof_ms / ms_per_step, "frac_is": "roofline_time_ms / ms_per_step (the whole call; "
                "no single kernel dominates a gradient call, so no per-kernel time is taken)",
                "frac_above_one": bool(roof_ms > ms_per_step), "traffic": None,
                "kernel": "whole call: " + ", ".join(x for x in (gather_kernels if nnz_gather else None,
                                                                 tile_kernels if nnz_tiles else None) if x),
                "roofline_time_ms": roof_ms, "gather_time_ms": gather_ms, "hbm_time_ms": dense_ms,
                "mfma_time_ms": mfma_ms, "gather_peak_GBs": gather_peak,
                "gather_peak_query_pass_GBs": peak_q if nnz_gather else None,
                "gather_peak_key_pass_GBs": peak_k if nnz_gather else None,
                "gather_peak_source": gather_src if nnz_gather else None,
                "working_set_bytes": ws_bytes, "algorithmic_bytes": total, "gathered_bytes": gathered,
                "gathered_positions": nnz_gather, "tile_positions": nnz_tiles,
                "executed_over_counted_tile_flops": 1.4}
    if gq is not None and gk is not None:
        roofline["measured_gather_query_pass"] = gq["how"]
        roofline["measured_gather_key_pass"] = gk["how"]
    out = {
        "metric": "masked-attn backward GFLOP/s (10*d per live position) + algorithmic GB/s",
        "value": flops / (ms_per_step * 1e-3) / 1e9, "unit": "GFLOP/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": a.dtype, "data": "synthetic",
        "config": {"workload": w["desc"] + " (gradients)", "n": n, "d": d, "nnz": nnz, "seed": 0, "heads": heads,
                   "transposed_mask": ("reused (built outside the timed region)" if a.planned else
                                       "rebuilt every call") if w["name"].startswith(("csr", "bigbird")) else None},
        "algorithmic_GBs": total / (ms_per_step * 1e-3) / 1e9,
        "roofline": roofline,
        "parity": {"dq_rel_err": err, "rows_checked": checked, "tolerance": tol,
                   "dv_column_sum_rel_err": col_err, "ok": bool(err <= tol and col_err <= (1e-5 if es == 4 else 3e-3))},
    }
    print(json.dumps(out))
    if not out["parity"]["ok"]:
        sys.exit("parity check of the gradients failed")


def measured_copy_bandwidth(torch, mib=1024, reps=5):
    """Bytes read + written per second by a plain device-to-device copy of `mib` MiB on this box:
    what the memory system delivers to the simplest streaming kernel, beside the vendor's 8 TB/s."""
    src = torch.empty(mib * 1024 * 1024 // 4, dtype=torch.float32, device="cuda").normal_()
    dst = torch.empty_like(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    dst.copy_(src)
    best = float("inf")
    for _ in range(reps):
        e0.record()
        dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1))
    return 2.0 * src.numel() * 4 / (best * 1e-3) / 1e9


def handed_out_order(cols, deg, torch, seg=1024, phases=64):
    """The columns of the long rows (`cols`, row after row; `deg` entries each) in the order the
    library's segment kernel takes them: rows cut into segments of `seg`, the segments ordered by the
    place of their middle in the row (in `phases` steps), every segment filled up to `seg` list
    slots with entries the probe skips (top bit set), so that one chunk of the probe's list is one
    segment."""
    deg = deg.to(torch.int64)
    nseg = (deg + seg - 1) // seg
    row_of_seg = torch.repeat_interleave(torch.arange(deg.numel(), device=deg.device), nseg)
    first_seg = torch.cumsum(nseg, 0) - nseg
    j = torch.arange(int(nseg.sum()), device=deg.device) - first_seg[row_of_seg]
    phase = ((2 * j + 1) * phases) // (2 * nseg[row_of_seg])
    # (a row's last segment comes the later the shorter it is)
    last = j + 1 == nseg[row_of_seg]
    missing = nseg[row_of_seg] * seg - deg[row_of_seg]
    phase = torch.where(last, phase + (missing * (phases - phase)) // seg, phase).clamp_(max=phases - 1)
    place = torch.empty_like(j)
    place[torch.argsort(phase, stable=True)] = torch.arange(j.numel(), device=deg.device)
    # entry t of row r is entry t % seg of the row's segment t // seg
    row_of_entry = torch.repeat_interleave(torch.arange(deg.numel(), device=deg.device), deg)
    t = torch.arange(cols.numel(), device=deg.device) - (torch.cumsum(deg, 0) - deg)[row_of_entry]
    dest = place[first_seg[row_of_entry] + t // seg] * seg + t % seg
    out = torch.full((j.numel() * seg,), -1, dtype=torch.int32, device=cols.device)
    out[dest.to(cols.device)] = cols.to(torch.int32)
    return out.contiguous()


def measured_gather_ceiling(lib, w, torch, min_entries=8_000_000, reps=5, tensors=None, idx=None):
    """What the memory system delivers to the explicit-mask access pattern at this working set:
    spfa_probe_gather (the gather of segments_kernel without any arithmetic) over the workload's
    own K, V and column list (the list is repeated up to min_entries so that the launch is long
    enough to time); `tensors` / `idx`: another pair of row tensors and another list (the key
    pass of the gradients gathers Q and dO rows by the mask's entries in column order).  Best of
    a few launch shapes.  None when the row size has no probe."""
    k, v = tensors if tensors is not None else (w["k"], w["v"])
    if k.dim() != 2:
        k, v = k[-1], v[-1]
    row_bytes = k.shape[1] * k.element_size()
    idx = w.get("probe_idx") if idx is None else idx
    if idx is None or row_bytes not in (64, 128, 256, 512) or idx.numel() == 0:
        return None
    if idx.numel() < min_entries:
        idx = idx.repeat((min_entries + idx.numel() - 1) // idx.numel())
    n_live = int((idx >= 0).sum())  # (negative: a slot the probe skips)
    probe = load_probe_library()
    cursor = torch.zeros(64, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    # timed like the kernel it is compared with: the dispatch's own start and end stamps
    ev = HipEvents()
    best, best_shape = float("inf"), None
    # (workgroups per CU of a persistent grid, or 0: an ordinary grid of one wavefront per 1024 list entries)
    shapes = ((1, 8), (1, 16), (1, 32), (2, 8), (2, 16), (2, 32), (4, 4), (4, 8), (4, 16), (4, 32), (8, 4), (8, 8), (8, 16),
              (0, 4), (0, 8), (0, 16))
    for wg, fl in shapes:
        for _ in range(reps):
            rc = probe.spfa_probe_gather(k.data_ptr(), v.data_ptr(), k.shape[0], row_bytes, idx.data_ptr(),
                                         idx.numel(), 1024, wg, fl, cursor.data_ptr(), ev.start, ev.stop, stream)
            assert rc == 0, "spfa_probe_gather rc=%d" % rc
            torch.cuda.synchronize()
            ms = ev.elapsed_ms()
            if ms < best:
                best, best_shape = ms, (wg, fl)
    bytes_moved = n_live * (2 * row_bytes + 4)
    return {"GBs": bytes_moved / (best * 1e-3) / 1e9,
            "how": "%d list entries x (2 rows of %d B + 4 B index) in %.3f ms; best of %d launches each of "
                   "(workgroups per CU, rows in flight) %s: (%d,%d)"
                   % (n_live, row_bytes, best, reps, " ".join("(%d,%d)" % x for x in shapes), *best_shape)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 20; 200 for the workloads whose call takes less than 0.2 ms and 100 "
                         "for the gradient calls of all but the COO workloads, which 20 steps would time "
                         "while the clocks are still ramping up)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 3; 20; 10)")
    ap.add_argument("--workload", default="csr_zipf", choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default="f32", choices=["f32", "f16", "bf16"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--d", type=int, default=64, choices=[32, 64, 96, 128, 160, 192, 224, 256],
                    help="head dimension of the `local` workload (BASELINE config 2 has 64; the reference's own "
                         "check runs at 32)")
    ap.add_argument("--tokens", type=int, default=None,
                    help="csr_zipf only: the headline generator at N tokens instead of 131072 (2048 ... 1048576)")
    ap.add_argument("--heads", type=int, default=1,
                    help="csr_* and local workloads: this many independent problems sharing the mask, stacked "
                         "[heads, n, d] (local: of N=4096 tokens each)")
    ap.add_argument("--loop-heads", action="store_true",
                    help="with --heads: one call per head (the reference's only way) instead of one batched "
                         "call; with --workload bigbird: the three chained calls instead of spfa_bigbird")
    ap.add_argument("--planned", action="store_true",
                    help="explicit masks: build the mask plan once, outside the timed region, and time "
                         "forward_planned (a mask reused across calls)")
    ap.add_argument("--graph", action="store_true",
                    help="capture one step (state reset + the call) in a HIP graph and time K replays "
                         "(for the launch-bound small workloads)")
    ap.add_argument("--backward", action="store_true",
                    help="time the gradient call (dQ, dK, dV from a finished forward state) instead of the "
                         "forward call; with --planned the transposed CSR mask is built outside the timed region")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the timed region, run one plain 256 MiB device copy (a kernel of known "
                         "traffic that counter runs use to scale FETCH_SIZE / WRITE_SIZE)")
    a = ap.parse_args()
    short = a.workload in ("local", "local_2d", "local_1d", "csr_bernoulli", "global") and not a.backward
    short_bwd = a.backward and not a.workload.startswith("coo")
    if a.steps is None:
        a.steps = 200 if short else 100 if short_bwd else 20
    if a.warmup is None:
        a.warmup = 20 if short else 10 if short_bwd else 3
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: this path is a single-GPU kernel and every box here has "
                 "one GPU; run with --gpus 1")

    import torch
    import spfa_synth as syn
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    torch.cuda.set_device(0)
    dtype = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[a.dtype]
    lib = load_library()
    if a.planned and not (a.workload.startswith(("csr", "coo")) or (a.workload == "bigbird" and a.backward)):
        sys.exit("bench.py: --planned applies to the explicit-mask workloads (csr_*, coo_*; bigbird with --backward)")
    if a.tokens is not None and (a.workload != "csr_zipf" or not 2048 <= a.tokens <= 1 << 20):
        sys.exit("bench.py: --tokens applies to the csr_zipf workload, 2048 ... 1048576")
    if a.heads > 1 and not (a.workload.startswith("csr") or a.workload == "local"):
        sys.exit("bench.py: --heads applies to the csr_* and local workloads")
    w = make_workload(a.workload, dtype, torch, syn, int(lib.spfa_explicit_inline_row_limit()), a.planned,
                      max(1, a.heads), a.loop_heads, a.d, a.tokens)
    n, d, nnz = w["n"], w["d"], w["nnz"]

    n_states = a.steps + a.warmup
    state_bytes = max(1, a.heads) * n * d * torch.tensor([], dtype=dtype).element_size()
    n_alloc = max(1, min(n_states, int(32e9 // max(1, state_bytes))))
    def new_state():
        if a.heads > 1:
            per = [syn.fresh_state(n, d, dtype=dtype, device="cuda", state_dtype=torch.float32)
                   for _ in range(a.heads)]
            return tuple(torch.stack([p[j] for p in per]) for j in range(3))
        return syn.fresh_state(n, d, dtype=dtype, device="cuda", state_dtype=torch.float32)
    states = [new_state() for _ in range(n_alloc)]

    def fresh(i):
        st = states[i % n_alloc]
        if i >= n_alloc:  # recycled: reset outside the timed region is not possible, so do it here
            st[0].fill_(-float("inf"))
            st[1].zero_()
        return st

    if a.backward:
        return bench_backward(a, w, states[0], dtype, torch, syn, lib)

    n_ev = min(a.steps, 10)
    evs = [HipEvents() for _ in range(n_ev)]
    for i in range(a.warmup):
        w["call"](fresh(i))
    torch.cuda.synchronize()

    if a.graph:
        # one step = reset of (m, l) + the call, captured once; the timed region replays it K times
        gst = states[0]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            w["call"](gst)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            gst[0].fill_(-float("inf"))
            gst[1].zero_()
            w["call"](gst)
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(a.steps):
            graph.replay()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        # (events cannot be recorded inside a captured graph: one eager step is timed for the kernel)
        lib.spfa_set_kernel_events(evs[0].start, evs[0].stop)
        w["call"](fresh(0))
        lib.spfa_set_kernel_events(None, None)
        torch.cuda.synchronize()
        evs = evs[:1]
    else:
        # timed region: exactly K steps, back to back on the stream.  In the last n_ev of them the
        # library records an event pair around its dominant kernel (no host synchronisation), so the
        # kernel times come out of the very steps that ms_per_step averages over.
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(a.steps):
            j = i - (a.steps - n_ev)
            if j >= 0:
                lib.spfa_set_kernel_events(evs[j].start, evs[j].stop)
            w["call"](fresh(a.warmup + i))
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        lib.spfa_set_kernel_events(None, None)
    ms_per_step = dt / a.steps * 1e3
    kernel_ms = [e.elapsed_ms() for e in evs]
    k_avg = sum(kernel_ms) / len(kernel_ms)

    # one call at a time (synchronised before and after): latency of a single call
    call_ms = []
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(min(a.steps, 10)):
        st = states[i % n_alloc]
        st[0].fill_(-float("inf"))
        st[1].zero_()
        torch.cuda.synchronize()
        c0.record()
        w["call"](st)
        c1.record()
        c1.synchronize()
        call_ms.append(c0.elapsed_time(c1))
    torch.cuda.synchronize()
    copy_gbs = measured_copy_bandwidth(torch)

    if a.copy_calibration:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    err, checked = verify_sample(w, states[0], torch)
    tol = 1e-4 if dtype == torch.float32 else 2e-2

    flops = syn.attention_flops(nnz, d)
    es = torch.tensor([], dtype=dtype).element_size()
    explicit = a.workload.startswith(("csr", "coo"))
    if explicit or w.get("whole_call"):
        # Gather work: bound by the memory system.  Which level binds depends on where K and V
        # live: every XCD's 4 MiB L2, the 256 MiB memory-side cache, or HBM.  The 8 TB/s HBM figure
        # is only a ceiling when K and V do not fit the memory-side cache; below that the ceiling
        # is what the same gather without arithmetic sustains at this working set (measured here).
        on_grid = lib.spfa_explicit_long_rows_on_grid(int(w["k"].shape[-2]), int(d), {"f32": 0, "f16": 1, "bf16": 2}[a.dtype])
        kernel_name = "items_grid_kernel" if on_grid else "segments_kernel"
        if on_grid and explicit and w["n"] * w.get("heads", 1) <= lib.spfa_explicit_one_launch_row_limit():
            w = dict(w, whole_call=True)  # (the row kernels of such a call are one launch)
        if w.get("whole_call") or w["kernel_nnz"] == 0:
            # no row is long enough for the segment kernel, or several kernels share the call: the
            # whole call stands in, with the call's algorithmic bytes
            k_avg, kernel_ms = ms_per_step, [ms_per_step]
            kernel_name = "whole call (several kernels, none dominant)"
            w = dict(w, kernel_bytes=w["bytes_total"], kernel_nnz=w["nnz"],
                     kernel_rows=w["n"] * w.get("heads", 1))
        achieved_gbs = w["kernel_bytes"] / (k_avg * 1e-3) / 1e9
        kv_bytes = 2 * w["k"].numel() * es
        traffic, traffic_src = measured_traffic(a.workload, a.dtype)
        if traffic is not None:
            traffic_src = "read from %s (two rocprofv3 --pmc runs of this command, FETCH_SIZE and " \
                          "WRITE_SIZE scaled by a copy kernel); not measured by this process" % traffic_src
        gather = measured_gather_ceiling(lib, w, torch)
        if kv_bytes <= 4 << 20:
            bound = "l2"
        elif kv_bytes <= 256 << 20:
            bound = "infinity_cache"
        else:
            bound = "hbm"
        peak = HBM_PEAK_GBS if bound == "hbm" or gather is None else gather["GBs"]
        roofline = {"bound": bound, "achieved": achieved_gbs, "peak": peak, "unit": "GB/s",
                    "frac": achieved_gbs / peak,
                    "peak_source": "MI355X HBM3E, published" if peak == HBM_PEAK_GBS else
                                   "measured on this device: the same gather without arithmetic "
                                   "(spfa_probe_gather) over this K and V and this column list",
                    "traffic": traffic, "traffic_source": traffic_src, "kernel": kernel_name,
                    "kv_working_set_bytes": kv_bytes,
                    "hbm_peak_GBs": HBM_PEAK_GBS, "achieved_over_hbm_peak": achieved_gbs / HBM_PEAK_GBS}
        if gather is not None:
            roofline["measured_gather_GBs"] = gather["GBs"]
            roofline["frac_of_measured_gather"] = achieved_gbs / gather["GBs"]
            roofline["measured_gather"] = gather["how"]
        roofline["measured_copy_GBs"] = copy_gbs
    else:
        # dense tiles: the roofline time is the larger of the HBM time of the compulsory bytes and
        # the matrix-pipe time of the live flops; whichever is larger names the bound.  The global
        # mask runs two tile kernels; the timed one (global rows against every key) reads K and V
        # once and computes the global rows' positions.
        mfma_peak = FP32_PEAK_TFLOPS if a.dtype == "f32" else HALF_PEAK_TFLOPS
        if a.workload == "global":
            kernel_flops = 4.0 * d * w["n_global_rows_nnz"]
            kernel_bytes = 2 * n * d * es
            # (half types, at most 64 listed tokens, d = 32 / 64: the streaming row kernel)
            streamed = a.dtype != "f32" and w["params"]["n_globals"] <= 64 and d in (32, 64)
            kernel_name = "global_rows_dma_kernel" if streamed else "tile_kernel (global rows)"
            w = dict(w, kernel_bytes=kernel_bytes, kernel_nnz=w["n_global_rows_nnz"],
                     kernel_rows=w["params"]["n_globals"])
        else:
            kernel_flops, kernel_bytes = flops, w["bytes_total"]
            # tiles straight to LDS: half types at d = 32, 64, 128, 256, fp32 at d = 64, 128
            kernel_name = ("band_dma_kernel" if d in (32, 64, 128, 256) else "tile_kernel") if a.dtype != "f32" else \
                "band_dma_f32_kernel" if d in (64, 128) else "tile_kernel"
        hbm_ms = kernel_bytes / (HBM_PEAK_GBS * 1e9) * 1e3
        mfma_ms = kernel_flops / (mfma_peak * 1e12) * 1e3
        if hbm_ms >= mfma_ms:
            achieved, peak, unit, bound = kernel_bytes / (k_avg * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s", "hbm"
        else:
            achieved, peak, unit, bound = kernel_flops / (k_avg * 1e-3) / 1e12, mfma_peak, "TFLOP/s", "mfma"
        roofline = {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit,
                    "frac": achieved / peak, "traffic": None, "kernel": kernel_name,
                    "hbm_time_ms": hbm_ms, "mfma_time_ms": mfma_ms, "roofline_time_ms": max(hbm_ms, mfma_ms),
                    "kernel_TFLOPs": kernel_flops / (k_avg * 1e-3) / 1e12,
                    "kernel_compulsory_GBs": kernel_bytes / (k_avg * 1e-3) / 1e9,
                    "call_hbm_time_ms": w["bytes_total"] / (HBM_PEAK_GBS * 1e9) * 1e3,
                    "call_mfma_time_ms": flops / (mfma_peak * 1e12) * 1e3,
                    "measured_copy_GBs": copy_gbs,
                    "hbm_time_at_measured_copy_ms": kernel_bytes / (copy_gbs * 1e9) * 1e3}
    roofline["frac_above_one"] = bool(roofline["frac"] > 1.0)
    call_sorted = sorted(call_ms)
    roofline.update({"kernel_ms_avg": k_avg, "kernel_ms_min": min(kernel_ms),
                     "kernel_ms_from": "start / stop events attached to the kernel's own dispatch "
                                       "(hipExtLaunchKernelGGL) in the last %d steps of the timed loop"
                                       % len(kernel_ms),
                     "algorithmic_bytes": w["kernel_bytes"], "kernel_nnz": w["kernel_nnz"],
                     "kernel_rows": w["kernel_rows"], "call_algorithmic_bytes": w["bytes_total"],
                     "call_gathered_bytes": w["bytes_gathered"]})
    out = {
        "metric": "masked-attn GFLOP/s (nnz-counted) + effective HBM GB/s, CSR N=128K d=64 fp32" if a.tokens is None else
                  "masked-attn GFLOP/s (nnz-counted) + effective HBM GB/s, CSR N=%d d=64" % a.tokens,
        "value": flops / (ms_per_step * 1e-3) / 1e9,
        "unit": "GFLOP/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic",
        "config": {"workload": w["desc"], "n": n, "d": d, "nnz": nnz, "seed": 0,
                   "index_dtypes": "uint64 offsets / uint32 columns", "state": "fresh m=-inf l=0 each step",
                   "mask_plan": "reused (built outside the timed region)" if a.planned else "rebuilt every call",
                   "heads": max(1, a.heads), "hip_graph": bool(a.graph),
                   "heads_call": ("one call per head" if a.loop_heads else "one batched call") if a.heads > 1 else "single",
                   "composite_call": (("three chained calls" if a.loop_heads else "one call (spfa_bigbird)")
                                      if a.workload == "bigbird" else None)},
        "call_ms_median": call_sorted[len(call_sorted) // 2], "call_ms_min": call_sorted[0],
        "effective_gathered_GBs": w["bytes_gathered"] / (ms_per_step * 1e-3) / 1e9,
        "effective_gathered_over_hbm_peak": w["bytes_gathered"] / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "algorithmic_GBs": w["bytes_total"] / (ms_per_step * 1e-3) / 1e9,
        "roofline": roofline,
        "parity": {"max_abs_err": err, "rows_checked": checked, "tolerance": tol, "ok": bool(err <= tol)},
    }
    if not a.no_cpu:
        cb = cpu_baseline(w, torch)
        if cb is not None:
            out["cpu_baseline"] = cb
            sp = cpu_sparse_port(w, torch)
            if sp is not None:
                out["cpu_sparse_port"] = sp
    print(json.dumps(out))
    if err > tol:
        sys.exit("parity check failed: max abs error %.3e > %.1e" % (err, tol))


if __name__ == "__main__":
    main()
