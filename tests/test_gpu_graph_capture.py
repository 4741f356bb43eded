"""The calls enqueue kernels only (no allocation inside the library, no memset nodes, no host
synchronisation), so a caller can capture them in a HIP graph.  Each replay is checked against
the eager result, with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

import spfa_synth as syn
from helpers import np64
from oracle import spfa_oracle as so

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_chained_forward_and_backward_replay_from_a_graph(mods):
    n, d, w = 1024, 64, 16
    globs = torch.tensor([3, 500], dtype=torch.int32, device=DEV)
    rng = np.random.default_rng(7)
    union = so.mask_local_dense(n, w) | so.mask_global_no_local_dense(n, [3, 500], w)
    rand = (rng.random((n, n)) < 0.02) & ~union
    ro, ci = so.csr_from_dense(rand)
    ro_t = torch.as_tensor(ro).to(torch.uint64).to(DEV)
    ci_t = torch.as_tensor(ci).to(torch.uint32).to(DEV)
    val = torch.empty(0, device=DEV)
    tr = mods["spfa_csr"].transpose(ro_t, ci_t, n)
    q, k, v = syn.qkv(n, d, device=DEV, seed=3)
    d_out = torch.randn(n, d, device=DEV, generator=torch.Generator(device=DEV).manual_seed(4))
    m = torch.empty(n, device=DEV)
    l = torch.empty(n, device=DEV)
    o = torch.empty(n, d, device=DEV)
    dq, dk, dv = (torch.empty(n, d, device=DEV) for _ in range(3))

    def step():
        m.fill_(-float("inf"))
        l.zero_()
        o.zero_()
        for g in (dq, dk, dv):
            g.zero_()
        mods["spfa_bigbird"].forward(q, k, v, m, l, o, w, globs, ro_t, ci_t, val)
        mods["spfa_bigbird"].backward(q, k, v, m, l, o, w, globs, ro_t, ci_t, val, d_out, dq, dk, dv, *tr)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # warm-up outside the capture (one-time set-up inside the library and torch)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = [x.clone() for x in (o, m, l, dq, dk, dv)]
    ref = so.dense_masked_attention(np64(q), np64(k), np64(v), union | rand)[0]
    assert np.abs(np64(o) - ref).max() <= 1e-4

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for x in (o, m, l, dq, dk, dv):
            x.fill_(123.0)  # eager work between the replays; stale results must not survive
        torch.cuda.synchronize()
        q.mul_(1.0)  # (the inputs are read in place by the replay)
        graph.replay()
        torch.cuda.synchronize()
        for name, got, want in zip(("out", "m", "l", "dq", "dk", "dv"), (o, m, l, dq, dk, dv), eager):
            assert torch.allclose(got, want, atol=1e-5, rtol=1e-5), "replay %d: %s differs from the eager run" % (rep, name)
