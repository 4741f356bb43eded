"""Writes tests/golden/spfa_golden.npz: small seeded inputs and expected outputs for the six mask
kinds, computed WITHOUT the repository's oracle or kernels.

Expected outputs come from torch's CPU ``scaled_dot_product_attention`` in float64 (the library
routine the reference's own check is built on, verification/verify.py:61-63) applied to boolean
masks that are spelled out here with plain loops, following the mask constructions of
verification/verify.py (:194-205 global-minus-local, :253-256 local, :376-382 1D-dilated,
:423-431 2D-dilated).  Rows without a live column are stored as NaN (recent torch versions return
zeros for such rows; the reference's convention with use_nan=True is NaN).  The running-softmax
statistics are stored as logsumexp = m + log(l), computed with torch.logsumexp.

Run from the repository root:  python tests/golden/make_golden.py
"""
import math
import os

import numpy as np
import torch

N, D = 64, 8


def sdpa(q, k, v, mask):
    out = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    dead = ~mask.any(dim=1)
    out[dead] = float("nan")
    s = (q @ k.T) / math.sqrt(q.shape[1])
    s = s.masked_fill(~mask, -float("inf"))
    lse = torch.logsumexp(s, dim=1)
    return out.numpy(), lse.numpy()


def main():
    g = torch.Generator().manual_seed(20250202)
    q = torch.randn(N, D, generator=g, dtype=torch.float64)
    k = torch.randn(N, D, generator=g, dtype=torch.float64)
    v = torch.randn(N, D, generator=g, dtype=torch.float64)
    # keep the inputs exactly representable in fp32, fp16 and bf16
    q, k, v = [(x * 8).round() / 8 for x in (q, k, v)]
    data = {"q": q.numpy(), "k": k.numpy(), "v": v.numpy()}

    # explicit random mask with some empty rows, a full row and a one-entry row
    rnd = torch.rand(N, N, generator=g) < 0.15
    rnd[3, :] = False
    rnd[17, :] = False
    rnd[5, :] = True
    rnd[9, :] = False
    rnd[9, 60] = True
    data["csr_mask"] = rnd.numpy()
    data["csr_out"], data["csr_lse"] = sdpa(q, k, v, rnd)

    w = 5
    loc = torch.zeros(N, N, dtype=torch.bool)
    for i in range(N):
        loc[i, max(0, i - w):min(N, i + w + 1)] = True
    data["local_w"] = np.int64(w)
    data["local_out"], data["local_lse"] = sdpa(q, k, v, loc)

    w1, dil1 = 4, 2
    m1 = torch.zeros(N, N, dtype=torch.bool)
    for i in range(N):
        start = max(i - w1 * (dil1 + 1), i % (dil1 + 1))
        end = min(i + w1 * (dil1 + 1), N - 1)
        for j in range((end - start) // (dil1 + 1) + 1):
            m1[i, start + j * (dil1 + 1)] = True
    data["d1_w"], data["d1_dil"] = np.int64(w1), np.int64(dil1)
    data["d1_out"], data["d1_lse"] = sdpa(q, k, v, m1)

    blk, dil2 = 16, 1
    m2 = torch.zeros(N, N, dtype=torch.bool)
    for i in range(N):
        start = (i // blk) * blk
        count = min(blk, (blk - 1) // (dil2 + 1) + 1)
        if (i - start) % (dil2 + 1) == 0:
            for j in range(count):
                m2[i, start + j * (dil2 + 1)] = True
    data["d2_block"], data["d2_dil"] = np.int64(blk), np.int64(dil2)
    data["d2_out"], data["d2_lse"] = sdpa(q, k, v, m2)

    globs = [0, 1, 10, 40]
    wg = 6
    mg = torch.zeros(N, N, dtype=torch.bool)
    for gi in globs:
        mg[gi, :] = True
        mg[:, gi] = True
    for i in range(N):
        mg[i, max(0, i - wg):min(N, i + wg) + 1] = False
    data["glob_inds"] = np.array(globs, dtype=np.int32)
    data["glob_w"] = np.int64(wg)
    data["glob_out"], data["glob_lse"] = sdpa(q, k, v, mg)

    # union of local(w) + global-minus-local(globs, w) + a random remainder: the chained case
    # (verification/verify.py:296-362)
    wu = 6
    locu = torch.zeros(N, N, dtype=torch.bool)
    for i in range(N):
        locu[i, max(0, i - wu):min(N, i + wu + 1)] = True
    rest = (torch.rand(N, N, generator=g) < 0.1) & ~locu & ~mg
    data["union_rest_mask"] = rest.numpy()
    data["union_out"], data["union_lse"] = sdpa(q, k, v, locu | mg | rest)

    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "spfa_golden.npz")
    np.savez_compressed(out, **data)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
