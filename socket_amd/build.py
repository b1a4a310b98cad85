"""Builds libsocket_hip.so (gfx950) from socket_amd/csrc with hipcc.

Run as `python -m socket_amd.build`; `__graft_entry__.build()` calls `build()`.
Objects are compiled in parallel, one translation unit per kernel family, and
linked into socket_amd/libsocket_hip.so next to this file.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libsocket_hip.so")
SOURCES = ["common.hip", "score.hip", "collide.hip", "topk.hip", "attend.hip", "hash.hip", "softhash.hip", "decode_ops.hip", "block_sparse.hip"]
ARCH = "gfx950"
# Packed-FP32 VALU ops are switched off for every device translation unit.
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# Per-file additions.  block_sparse.hip: keep MFMA accumulators in ordinary
# registers (its softmax reads and rescales them every tile; the default form
# parks them in the accumulator file and moves them back and forth).
FILE_FLAGS = {
    "block_sparse.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "attend.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],     # the MFMA dense flash-decode, for the same reason
}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libsocket_hip.so cannot be built")
    return exe


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), p.stdout))
    lines = [ln for ln in p.stdout.splitlines() if "not a recognized feature" not in ln]
    return "\n".join(lines)


def _stale(src_path: str, obj: str) -> bool:
    """True if the object is older than its source or any header beside it."""
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src_path, os.path.join(CSRC, "socket_common.h"), os.path.join(HERE, "..", "include", "socket_hip.h")]
    return any(os.path.getmtime(d) > t for d in deps)


def build(verbose: bool = False, extra_flags=(), only_changed: bool = False) -> str:
    """Compile every source (or, with only_changed, those newer than their
    object) and link the library."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        if only_changed and not _stale(os.path.join(CSRC, src), obj):
            return obj
        out = _run([hipcc, *FLAGS, *FILE_FLAGS.get(src, []), *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, only_changed="--changed" in sys.argv))
