"""Builds libnsa_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(OUT_DIR, "libnsa_hip.so")
SOURCES = ["prep.hip", "attn.hip", "cmp_select.hip", "select.hip", "slc_block.hip", "bwd.hip", "compress_bwd.hip", "combine.hip", "qkv_rope.hip", "decode.hip", "decode_split.hip", "capi.hip"]
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-fno-honor-nans", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]


def sources_digest() -> str:
    """First 12 hex digits of the SHA-256 over the kernel sources (file names and contents, sorted): names the
    build a measurement was taken on."""
    import hashlib
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:12]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str, extra) -> str:
    obj = os.path.join(OUT_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr[-8000:]))
    return obj


def build(verbose: bool = False, extra_flags=()) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        objs = list(ex.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    cmd = [_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr[-8000:])
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__" and sys.argv[1:] == ["--digest"]:
    print(sources_digest())
    sys.exit(0)

if __name__ == "__main__":
    build(verbose=True, extra_flags=sys.argv[1:])
