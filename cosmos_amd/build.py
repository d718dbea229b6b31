"""Builds the HIP libraries (gfx950) in-tree with hipcc.  ``python -m cosmos_amd.build``.

Two libraries come out of the same sources:
  * ``libcosmos_dm_hip.so``            - the product: the default kernels, no process-wide state;
  * ``libcosmos_dm_hip_crosscheck.so`` - compiled with ``-DCDM_CROSSCHECK``: additionally carries the superseded kernels
    and ``cdm_set_variant``; only the parity tests and measurement aids load it (``ops.set_variant``).
"""
from __future__ import annotations

import fcntl
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcosmos_dm_hip.so")
CROSSCHECK_PATH = os.path.join(LIB_DIR, "libcosmos_dm_hip_crosscheck.so")
SOURCES = ["api.hip", "norm.hip", "rope.hip", "gemm.hip", "attn.hip", "step.hip", "edge.hip"]
# packed fp32 VALU forms are switched off on purpose (hipcc's host pass warns that it does not
# know the feature; that warning is harmless)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
CROSSCHECK_FLAGS = ["-DCDM_CROSSCHECK"]


INCLUDE = os.path.join(os.path.dirname(HERE), "include")
HASH_MARKER = b"CDM_SRC_HASH="


def source_hash() -> str:
    """16 hex digits over everything a library is built from: kernels, shared headers, the public header and the
    compiler flags."""
    h = hashlib.sha256()
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith((".hip", ".h"))]
    files += [os.path.join(INCLUDE, f) for f in sorted(os.listdir(INCLUDE)) if f.endswith(".h")]
    for path in files:
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as fh:
            h.update(fh.read())
    h.update("\0".join(FLAGS + ["|"] + CROSSCHECK_FLAGS).encode())
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


def _compile(job) -> str:
    src, extra, out_dir, want = job
    obj = os.path.join(out_dir, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, *extra, f'-DCDM_SOURCE_HASH="{want}"', "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr[-4000:]}")
    return obj


def build(verbose: bool = True, only_if_stale: bool = False) -> str:
    """Compile every HIP source for gfx950 and link both shared libraries.  Recompiles every time it is called, unless
    ``only_if_stale`` is set and both libraries already carry the hash of the present sources (the loader's case).
    Builds go to a temporary directory and are moved into place under a file lock, so that processes which find a
    stale library at the same time neither overwrite each other's objects nor load a half-written file."""
    os.makedirs(LIB_DIR, exist_ok=True)
    want = source_hash()
    with open(os.path.join(LIB_DIR, ".build.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        try:
            if only_if_stale and built_hash(LIB_PATH) == want and built_hash(CROSSCHECK_PATH) == want:
                return LIB_PATH             # another process built it while this one waited for the lock
            tmp = tempfile.mkdtemp(prefix=".build-", dir=LIB_DIR)
            try:
                targets = [(LIB_PATH, [], os.path.join(tmp, "product")), (CROSSCHECK_PATH, CROSSCHECK_FLAGS, os.path.join(tmp, "crosscheck"))]
                jobs = []
                for _, extra, out_dir in targets:
                    os.makedirs(out_dir)
                    jobs += [(src, extra, out_dir, want) for src in SOURCES]
                with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1, len(jobs))) as ex:
                    objs = list(ex.map(_compile, jobs))
                for i, (path, _, out_dir) in enumerate(targets):
                    so = os.path.join(out_dir, os.path.basename(path))
                    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", so, *objs[i * len(SOURCES):(i + 1) * len(SOURCES)]]
                    r = subprocess.run(cmd, capture_output=True, text=True)
                    if r.returncode != 0:
                        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
                for path, _, out_dir in targets:
                    os.replace(os.path.join(out_dir, os.path.basename(path)), path)
            finally:
                shutil.rmtree(tmp, ignore_errors=True)
        finally:
            fcntl.flock(lock, fcntl.LOCK_UN)
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes) and {os.path.basename(CROSSCHECK_PATH)} "
              f"({os.path.getsize(CROSSCHECK_PATH)} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
