"""Builds libsplatad_hip.so (gfx950) in-tree with hipcc.

    python -m splatad_amd.build            # compile if sources are newer than the library
    python -m splatad_amd.build --force    # always compile

The library is a plain C-ABI shared object (see include/splatad_hip.h); it does not link
against torch.  Packed FP32 instructions are disabled for every device translation unit.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libsplatad_hip.so")
OBJ_DIR = os.path.join(PKG_DIR, "csrc", "_obj")

ARCH = "gfx950"
COMMON = ["-O3", "-fPIC", "-std=c++17", f"--offload-arch={ARCH}",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wall", "-Wno-unused-function", "-Wno-unused-command-line-argument"]
# per-file extra flags: the tile bounds of the intersection code must not be contracted
EXTRA = {"intersect.hip": ["-ffp-contract=off"]}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _stale():
    if not os.path.exists(LIB_PATH):
        return True
    lib_m = os.path.getmtime(LIB_PATH)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp", ".h"))]
    deps.append(os.path.join(PKG_DIR, "..", "include", "splatad_hip.h"))
    return any(os.path.getmtime(d) > lib_m for d in deps)


def _compile(src):
    obj = os.path.join(OBJ_DIR, src + ".o")
    cmd = [_hipcc(), *COMMON, *EXTRA.get(src, []), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    return obj, out


def build(force: bool = False, verbose: bool = False) -> str:
    if not force and not _stale():
        return LIB_PATH
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        results = list(pool.map(_compile, sources()))
    for _, out in results:
        if verbose and out.strip():
            print(out)
    objs = [o for o, _ in results]
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", LIB_PATH]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}")
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--force" in sys.argv, verbose=True)
    print(path)
