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

SOURCES = [os.path.join(CSRC, "sharpnet_hip.hip")]
HEADERS = [os.path.join(CSRC, "sgemm_mfma.hpp"), os.path.join(REPO, "include", "sharpnet_hip.h")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 VALU forms are switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
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


def build_library(force=False, verbose=True):
    """Compile the HIP sources into libsharpnet_hip.so.  Returns the library path."""
    if not force and not is_stale():
        return LIB_PATH
    cmd = [find_hipcc()] + HIPCC_FLAGS + ["-I", os.path.join(REPO, "include"), "-o", LIB_PATH + ".tmp"] + SOURCES
    if verbose:
        print("[sharpnet_amd.build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is harmless
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force="--force" in sys.argv or True))
