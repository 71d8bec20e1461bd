"""Compiles the HIP sources under dlf_amd/csrc into dlf_amd/lib/libdlfx.so for gfx950.

hipcc cross-compiles without a GPU.  Object files go to dlf_amd/csrc/obj/ and
are rebuilt only when a source or header is newer, unless force=True.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "obj")
LIB = os.path.join(HERE, "lib", "libdlfx.so")

# (the longest compilations first; topk_wide.hip and topk_narrow.hip include topk.hip)
SOURCES = ["topk.hip", "topk_wide.hip", "topk_narrow.hip", "scan.hip", "softmax.hip", "sort.hip", "sort_split.hip", "reduce.hip", "lib.hip",
           "nonzero.hip", "merge.hip", "copy.hip"]
INCLUDES = {"topk_wide.hip": ["topk.hip"], "topk_narrow.hip": ["topk.hip"]}

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unused-const-variable", "-Wno-pass-failed",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _newest_header():
    t = 0.0
    for root in (CSRC, os.path.join(HERE, "..", "include")):
        for f in os.listdir(root):
            if f.endswith(".h"):
                t = max(t, os.path.getmtime(os.path.join(root, f)))
    return t


def _compile(src, force, header_time):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    srcp = os.path.join(CSRC, src)
    newest = max([os.path.getmtime(srcp), header_time] + [os.path.getmtime(os.path.join(CSRC, f)) for f in INCLUDES.get(src, [])])
    if not force and os.path.exists(obj) and os.path.getmtime(obj) > newest:
        return obj
    cmd = [_hipcc()] + HIPCC_FLAGS + ["-c", srcp, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_all(force=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    jobs = jobs or min(8, len(sources))
    ht = _newest_header()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, ht), sources))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


VENEER_TEST_SRC = os.path.join(HERE, "..", "tests", "cpp", "veneer_test.cpp")
VENEER_TEST_BIN = os.path.join(HERE, "..", "tests", "cpp", "veneer_test.bin")


def build_veneer_test(force=False):
    """Compiles the C++ host veneer's test program (host code + HIP runtime only)."""
    src, out = os.path.abspath(VENEER_TEST_SRC), os.path.abspath(VENEER_TEST_BIN)
    if not os.path.exists(src):
        return None
    inc = os.path.join(HERE, "include")
    newest = max([os.path.getmtime(src)] + [os.path.getmtime(os.path.join(inc, f)) for f in os.listdir(inc)])
    if not force and os.path.exists(out) and os.path.getmtime(out) > newest:
        return out
    cmd = [_hipcc(), "-O2", "-std=c++17", "-I", inc, "-I", os.path.join(HERE, "..", "include"), src, "-o", out,
           "-pthread", "-L", os.path.dirname(LIB), "-ldlfx", "-Wl,-rpath,$ORIGIN/../../dlf_amd/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("veneer test build failed:\n" + r.stderr)
    return out


if __name__ == "__main__":
    print(build_all(force="--force" in sys.argv))
    print(build_veneer_test(force="--force" in sys.argv))
