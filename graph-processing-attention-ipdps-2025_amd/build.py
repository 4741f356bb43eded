"""Build libspfa_hip.so (HIP kernels + C ABI, gfx950), libspfa_probe.so (a measurement aid for
benchmarks, include/spfa_probe.h) and the torch host wrappers in-tree.

    python build.py            # everything
    python build.py --lib      # only libspfa_hip.so and libspfa_probe.so
    python build.py --ext      # only the spfa_* Python modules

The wrappers are host-only C++ (g++): they check tensors the way the reference bindings do and
call the C ABI.  All device code is in libspfa_hip.so, compiled by hipcc for gfx950 only.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
EXT = os.path.join(HERE, "ext")
OBJ = os.path.join(HERE, "build")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # keep the compiler from forming packed-fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", INCLUDE, "-I", CSRC,
]

ELEM_TYPES = {"f32": "float", "f16": "spfa::f16", "bf16": "spfa::bf16"}
MASK_KINDS = {"csr": 0, "stride": 1, "global": 2}

MODULES = ["spfa_csr", "spfa_coo", "spfa_local", "spfa_local_1d_dilated", "spfa_local_2d_dilated",
           "spfa_global_no_local", "spfa_bigbird"]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + p.stdout + "\n")
        raise RuntimeError("build step failed: " + os.path.basename(cmd[-1]))
    return p.stdout


def lib_jobs():
    jobs = []
    for mname, mid in MASK_KINDS.items():
        for tname, tcpp in ELEM_TYPES.items():
            obj = os.path.join(OBJ, "inst_%s_%s.o" % (mname, tname))
            jobs.append((obj, [HIPCC, *HIP_FLAGS, "-DSPFA_INST_MASK=%d" % mid,
                               "-DSPFA_INST_T=%s" % tcpp, "-c",
                               os.path.join(CSRC, "spfa_inst.hip"), "-o", obj]))
            obj = os.path.join(OBJ, "grad_%s_%s.o" % (mname, tname))
            jobs.append((obj, [HIPCC, *HIP_FLAGS, "-DSPFA_INST_MASK=%d" % mid,
                               "-DSPFA_INST_T=%s" % tcpp, "-c",
                               os.path.join(CSRC, "spfa_grad_inst.hip"), "-o", obj]))
    for src in sorted(os.listdir(CSRC)):
        if src.endswith(".hip") and src not in ("spfa_inst.hip", "spfa_grad_inst.hip"):
            obj = os.path.join(OBJ, src[:-4] + ".o")
            jobs.append((obj, [HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]))
    return jobs


def build_lib(workers: int) -> str:
    os.makedirs(OBJ, exist_ok=True)
    jobs = lib_jobs()
    with cf.ThreadPoolExecutor(max_workers=workers) as ex:
        list(ex.map(lambda j: _run(j[1]), jobs))
    out = os.path.join(HERE, "libspfa_hip.so")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *[j[0] for j in jobs]])
    return out


def build_probe() -> str:
    """libspfa_probe.so: the gather probe that bench.py prices the explicit-mask kernels against
    (csrc/probe/, apart from the attention library)."""
    os.makedirs(OBJ, exist_ok=True)
    out = os.path.join(HERE, "libspfa_probe.so")
    _run([HIPCC, *HIP_FLAGS, "-shared", "-o", out, os.path.join(CSRC, "probe", "spfa_probe.hip")])
    return out


def build_ext(workers: int):
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(OBJ, exist_ok=True)
    inc = []
    for p in ce.include_paths("cuda"):  # on torch-ROCm this adds the HIP headers
        inc += ["-I", p]
    inc += ["-I", os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "include")]
    inc += ["-I", sysconfig.get_paths()["include"], "-I", INCLUDE, "-I", EXT]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cxx = os.environ.get("CXX", "g++")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    outs = []
    jobs = []
    for mod in MODULES:
        out = os.path.join(HERE, mod + ".so")
        outs.append(out)
        jobs.append([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
                     "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=" + mod,
                     "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
                     "-Wno-deprecated-declarations", *inc,
                     os.path.join(EXT, mod + ".cpp"), "-o", out,
                     "-L", HERE, "-lspfa_hip", "-L", torch_lib, "-ltorch_python", "-ltorch",
                     "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
                     "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib])
    with cf.ThreadPoolExecutor(max_workers=workers) as ex:
        list(ex.map(_run, jobs))
    return outs


def _source_loop_depth(kname: str) -> int:
    """Loop-nest depth the source of a kernel has: work loop (segments_kernel only) > index-chunk
    loop > batch loop; the batch loop is only a real loop when a chunk holds more than two
    batches (it is unrolled otherwise)."""
    import re
    if "11tile_kernelI" in kname:
        # key-tile loop; the global-columns mode (third template argument 2, before the flag for
        # padded rows) also loops over query tiles
        return 2 if re.search(r"Li2ELb[01]EEEv", kname) else 1
    whole = "17whole_rows_kernelI" in kname  # (a medium-row walk inside its loop over long rows)
    if "20explicit_rows_kernelI" in kname:
        # the item, medium-row and short-row kernels in one launch: the deepest nest of the three
        # (the first two with the layout's own batch size)
        # (its third template argument is the medium rows' batch size; the items keep the layout's)
        as_items = re.sub(r"MaskELi\d+EEEv", "MaskEEEv", kname).replace("20explicit_rows_kernelI", "18medium_rows_kernelI")
        return max(_source_loop_depth(kname.replace("20explicit_rows_kernelI", "18medium_rows_kernelI")),
                   _source_loop_depth(as_items),
                   _source_loop_depth(kname.replace("20explicit_rows_kernelI", "11rows_kernelI")))
    med = "18medium_rows_kernelI" in kname or "17items_grid_kernelI" in kname or whole
    if "15segments_kernelI" not in kname and "11rows_kernelI" not in kname and not med:
        return 1
    seg = "15segments_kernelI" in kname
    m = re.search(r"6VecLayI\w+?Li(\d+)E", kname)
    if m:
        lpr, unroll = int(m.group(1)), (16 if seg else 8 if med else 4)
    elif "7WideLayI" in kname:
        nch = int(re.search(r"7WideLayI\w+?Li(\d+)E", kname).group(1))
        u = 16 // nch
        lpr, unroll = 32, (u if seg else max(u // 2, 1) if med else max(u // 4, 1))
    else:
        m = re.search(r"6GenLayI\w+?Li(\d+)E", kname)
        lpr, unroll = 64, (8 if int(m.group(1)) <= 2 else 2)
    if med and not whole:
        # medium_rows_kernel and items_grid_kernel name their batch size as a third template argument
        m = re.search(r"MaskELi(\d+)EEEv", kname)
        if m:
            unroll = min(unroll, int(m.group(1)))
    span = 64 if (seg or med) else lpr
    groups = span // lpr
    unroll = min(unroll, span // groups)
    parts = span // (unroll * groups)
    return (2 if (seg or whole) else 1) + (1 if parts > 2 else 0)


def check_loop_nests(workers: int | None = None) -> None:
    """Compile the engine to assembly and check the loop nests the compiler formed.

    segments_kernel fetches its work index with a cross-lane read at the top of its work loop, so
    every lane of a wavefront must take every trip of that loop together.  The optimiser has been
    seen to split the loop into an outer and an inner loop (one back edge for the lanes that write
    the row statistics, one for the rest), after which the inner loop spins on work index 0.  The
    source keeps a convergent operation in the loop's single latch; this check fails the build if a
    kernel ever shows a deeper loop nest than its source has.
    """
    import re
    workers = workers or min(8, os.cpu_count() or 4)
    os.makedirs(OBJ, exist_ok=True)
    jobs = []
    for mname, mid in MASK_KINDS.items():
        for tname, tcpp in ELEM_TYPES.items():
            asm = os.path.join(OBJ, "inst_%s_%s.s" % (mname, tname))
            jobs.append((asm, [HIPCC, *HIP_FLAGS, "-DSPFA_INST_MASK=%d" % mid,
                               "-DSPFA_INST_T=%s" % tcpp, "-S", "--cuda-device-only",
                               os.path.join(CSRC, "spfa_inst.hip"), "-o", asm]))
    with cf.ThreadPoolExecutor(max_workers=workers) as ex:
        list(ex.map(lambda j: _run(j[1]), jobs))
    for asm, _ in jobs:
        depth, name = {}, None
        for line in open(asm):
            m = re.match(r"^(_ZN4spfa\w+):", line)
            if m:
                name = m.group(1)
                depth[name] = 0
            m = re.search(r"Loop Header: Depth=(\d+)", line)
            if m and name:
                depth[name] = max(depth[name], int(m.group(1)))
        for kname, dep in depth.items():
            limit = _source_loop_depth(kname)
            if dep > limit:
                raise RuntimeError("%s: %s has loop depth %d (source has %d): a loop was split"
                                   % (os.path.basename(asm), kname, dep, limit))
        if not any("segments_kernel" in k for k in depth):
            raise RuntimeError("no segments_kernel found in " + asm)


def build_all(workers: int | None = None):
    workers = workers or min(8, os.cpu_count() or 4)
    lib = build_lib(workers)
    probe = build_probe()
    exts = build_ext(min(workers, 6))
    return [lib, probe, *exts]


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--lib", action="store_true")
    ap.add_argument("--ext", action="store_true")
    ap.add_argument("--check", action="store_true", help="only check the compiled loop nests")
    ap.add_argument("-j", type=int, default=None)
    a = ap.parse_args()
    w = a.j or min(8, os.cpu_count() or 4)
    if a.check:
        check_loop_nests(w)
        print("loop nests ok")
        sys.exit(0)
    if a.lib or not a.ext:
        print(build_lib(w))
        print(build_probe())
    if a.ext or not a.lib:
        for o in build_ext(min(w, 6)):
            print(o)
