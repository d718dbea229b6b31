"""Builds libcosmos_dm_hip.so (gfx950) in-tree with hipcc.  ``python -m cosmos_amd.build``."""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcosmos_dm_hip.so")
SOURCES = ["api.hip", "norm.hip", "rope.hip", "gemm.hip", "attn.hip", "step.hip"]
# packed fp32 VALU forms are switched off on purpose (hipcc's host pass warns that it does not
# know the feature; that warning is harmless)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


INCLUDE = os.path.join(os.path.dirname(HERE), "include")
HASH_MARKER = b"CDM_SRC_HASH="


def source_hash() -> str:
    """16 hex digits over every file the library is built from (kernels, shared headers, the public header)."""
    h = hashlib.sha256()
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith((".hip", ".h"))]
    files += [os.path.join(INCLUDE, f) for f in sorted(os.listdir(INCLUDE)) if f.endswith(".h")]
    for path in files:
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def built_hash(path: str = LIB_PATH) -> str:
    """The source hash a built library carries ("" if the file is missing or carries none)."""
    try:
        with open(path, "rb") as fh:
            blob = fh.read()
    except OSError:
        return ""
    i = blob.find(HASH_MARKER)
    return blob[i + len(HASH_MARKER):i + len(HASH_MARKER) + 16].decode("ascii", "replace") if i >= 0 else ""


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, f'-DCDM_SOURCE_HASH="{source_hash()}"', "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr[-4000:]}")
    return obj


def build(verbose: bool = True) -> str:
    """Compile every HIP source for gfx950 and link the shared library. Always recompiles."""
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(6, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
