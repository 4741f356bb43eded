"""libspfa_probe.so (include/spfa_probe.h): the gather without arithmetic that bench.py prices the
explicit-mask kernels against.  It computes nothing, so what can be checked is that it walks the
whole list (the work cursor ends where it must), that entries at or beyond n_rows - top bit
set or merely out of range - are skipped instead of read, and that its argument checks hold."""
import ctypes
import os

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "graph-processing-attention-ipdps-2025_amd", "libspfa_probe.so")


@pytest.fixture(scope="module")
def probe():
    L = ctypes.CDLL(LIB)
    L.spfa_probe_gather.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                    ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                    ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    return L


@pytest.mark.gpu
@pytest.mark.parametrize("row_bytes,in_flight,wg,chunk", [(64, 16, 1, 64), (128, 8, 2, 64), (256, 16, 1, 64),
                                                          (256, 32, 2, 1024), (512, 32, 1, 64), (256, 8, 0, 1024),
                                                          (128, 16, 0, 64)])
def test_probe_walks_the_list_and_skips_rows_beyond_the_tensor(probe, row_bytes, in_flight, wg, chunk):
    dev = "cuda:0"
    n_rows, n_idx = 1000, 200001
    k = torch.randn(n_rows, row_bytes // 4, device=dev)
    v = torch.randn(n_rows, row_bytes // 4, device=dev)
    g = torch.Generator(device=dev).manual_seed(3)
    idx = torch.randint(0, n_rows, (n_idx,), generator=g, device=dev, dtype=torch.int64)
    # every third entry is no row of the tensor: top bit set, just past the end, far past the end
    idx[0::9] = 0x80000000 + 5
    idx[3::9] = n_rows
    idx[6::9] = 0x7fffffff
    idx32 = idx.to(torch.uint32)
    cursor = torch.full((16,), 999, dtype=torch.int32, device=dev)
    rc = probe.spfa_probe_gather(k.data_ptr(), v.data_ptr(), n_rows, row_bytes, idx32.data_ptr(), n_idx, chunk,
                                 wg, in_flight, cursor.data_ptr(), None, None,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    n_chunks = (n_idx + chunk - 1) // chunk
    n_waves = 4 * wg * torch.cuda.get_device_properties(0).multi_processor_count
    # A wavefront's first run is the one with its own number, the cursor hands out the later ones:
    # with fewer wavefronts than runs every wavefront leaves with one pull beyond the end of the
    # list; an ordinary grid (wg = 0) and a persistent one with a wavefront for every run never pull.
    if 0 < n_waves < n_chunks:
        assert int(cursor[0]) == n_chunks
    else:
        assert int(cursor[0]) == 0
    assert (cursor[1:] == 999).all()


def test_probe_argument_checks(probe):
    """Returned from the host-side checks, before any device work (no GPU needed)."""
    buf = ctypes.create_string_buffer(256)
    a = ctypes.addressof(buf)
    a16 = (a + 15) // 16 * 16
    ok = dict(k=a16, v=a16, n_rows=4, row_bytes=64, idx=a16, n_idx=4, chunk=64, wg=1, fl=16, cur=a16)

    def call(**kw):
        x = dict(ok, **kw)
        return probe.spfa_probe_gather(x["k"], x["v"], x["n_rows"], x["row_bytes"], x["idx"], x["n_idx"], x["chunk"],
                                       x["wg"], x["fl"], x["cur"], None, None, None)
    assert call(k=None) == 1
    assert call(idx=None) == 1
    assert call(n_rows=0) == 1
    assert call(n_rows=1 << 31) == 1
    assert call(chunk=32) == 1
    assert call(wg=9) == 1
    assert call(wg=-1) == 1
    assert call(k=a16 + 4) == 1
    assert call(row_bytes=96) == 2
