"""Build step for libsharpnet_hip.so (hipcc, gfx950 only).

Run as ``python -m sharpnet_amd.build``; ``__graft_entry__.build()`` calls
``build_library(force=True)``.  The library is written next to this file so it
is found by ``hiplib.load_library`` and travels with the source tree.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libsharpnet_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

MAIN_SOURCE = os.path.join(CSRC, "sharpnet_hip.hip")       # C ABI, dispatch, small kernels
KERNEL_SOURCE = os.path.join(CSRC, "gemm_kernels.hip")     # GEMM kernels, compiled once per group of kernel_list.hpp
KERNEL_GROUPS = 10                                         # SNHIP_NUM_KERNEL_GROUPS
SOURCES = [MAIN_SOURCE, KERNEL_SOURCE]
HEADERS = [os.path.join(CSRC, n) for n in ("sgemm_mfma.hpp", "bgemm_mfma.hpp", "rowops.hpp", "kernel_list.hpp", "attention_mfma.hpp", "rnn_cells.hpp", "rnn_layers.hpp", "sgemm_ksplit.hpp", "sgemm_stream.hpp", "bgemm_dtl.hpp")] + \
          [os.path.join(REPO, "include", "sharpnet_hip.h")]
# what gemm_kernels.hip includes; the other headers belong to the translation unit with the C ABI
KERNEL_HEADERS = [os.path.join(CSRC, n) for n in ("sgemm_mfma.hpp", "bgemm_mfma.hpp", "kernel_list.hpp")]
OBJ_DIR = os.path.join(HERE, "_obj")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # packed fp32 VALU forms are switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # some fully unrolled staging loops of the bf16-input kernel keep a rolled remainder; that is fine, not worth a warning
    "-Wno-pass-failed",
]


def find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def is_stale():
    if not os.path.exists(LIB_PATH):
        return True
    built = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(p) > built for p in SOURCES + HEADERS)


def _run(cmd, verbose):
    if verbose:
        print("[sharpnet_amd.build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is harmless
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_library(force=False, verbose=True, jobs=None):
    """Compile the HIP sources into libsharpnet_hip.so.  Returns the library path.

    The GEMM kernels are split into KERNEL_GROUPS translation units that are compiled side by side
    (``jobs`` at a time, default min(8, cpu count)); one more unit holds the C ABI.  Everything is linked into
    one shared library.
    """
    if not force and not is_stale():
        return LIB_PATH
    from concurrent.futures import ThreadPoolExecutor
    hipcc = find_hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    inc = ["-I", os.path.join(REPO, "include")]
    units = [([hipcc] + HIPCC_FLAGS + inc + ["-c", MAIN_SOURCE, "-o", os.path.join(OBJ_DIR, "sharpnet_hip.o")])]
    for g in range(KERNEL_GROUPS):
        units.append([hipcc] + HIPCC_FLAGS + inc + ["-DSNHIP_KERNEL_GROUP=%d" % g, "-c", KERNEL_SOURCE, "-o",
                                                    os.path.join(OBJ_DIR, "gemm_kernels_%d.o" % g)])
    jobs = jobs or max(1, min(8, os.cpu_count() or 1))
    objs = [u[-1] for u in units]
    if not force:
        # rebuild only the objects that are older than their own source or a header they include
        def fresh(unit):
            obj, src = unit[-1], unit[-3]
            deps = HEADERS if src == MAIN_SOURCE else KERNEL_HEADERS
            return os.path.exists(obj) and all(os.path.getmtime(p) <= os.path.getmtime(obj) for p in [src] + deps)
        units = [u for u in units if not fresh(u)]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        outs = list(pool.map(lambda c: _run(c, verbose), units))
    outs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH + ".tmp"] + objs, verbose))
    if verbose:
        for out in outs:
            if out.strip():
                print(out)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force="--incremental" not in sys.argv))
