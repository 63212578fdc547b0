"""Builds the HIP library (csrc/*.hip -> csrc/libqwen_tailor_hip.so) for gfx950 with hipcc, in-tree."""
from __future__ import annotations

import glob
import hashlib
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
SO = os.path.join(CSRC, "libqwen_tailor_hip.so")
FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


HASH = SO + ".srchash"


def source_hash() -> str:
    """sha256 over the names and contents of every source the library is built from (csrc/*.hip, csrc/*.h) and the flags"""
    h = hashlib.sha256(" ".join(FLAGS).encode())
    for path in sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def is_current() -> bool:
    """True if the built library exists and was built from the sources as they are now."""
    try:
        with open(HASH) as f:
            return os.path.exists(SO) and f.read().strip() == source_hash()
    except OSError:
        return False


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False, jobs: int = 8) -> str:
    """Compile every csrc/*.hip and link them into one shared library.  Always recompiles."""
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    hipcc = _hipcc()
    digest = source_hash()                  # taken before compiling: an edit made during the build leaves the library stale
    objs = [s[:-4] + ".o" for s in srcs]

    def one(pair):
        src, obj = pair
        cmd = [hipcc, *FLAGS, "-c", src, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
        if verbose and r.stderr.strip():
            print(r.stderr)

    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(srcs)))) as ex:
        list(ex.map(one, zip(srcs, objs)))
    r = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", SO + ".tmp"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(SO + ".tmp", SO)
    with open(HASH, "w") as f:
        f.write(digest + "\n")
    return SO


if __name__ == "__main__":
    print(build(verbose=True))
