"""Build libtrimkv_hip.so (the C-ABI library of HIP kernels) in-tree for gfx950.

Usage: ``python -m trimkv_amd.build [--changed]`` (hipcc cross-compiles without a GPU; ``--changed`` recompiles only
the sources whose object file is older than its inputs).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_PATH = os.path.join(HERE, "libtrimkv_hip.so")
SOURCES = ["api.hip", "append.hip", "evict.hip", "attn_decode.hip", "attn_decode_append.hip", "attn_decode_pieces.hip", "attn_decode_append_pieces.hip", "attn_decode_append_gated.hip", "attn_decode_append_pieces_gated.hip", "pieces_plan.hip", "attn_prefill.hip", "gate.hip", "stream_probe.hip", "decoder_ops.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + INCLUDE, "-I" + CSRC,
    # packed fp32 VALU ops are kept out of every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _stale(src: str, obj: str) -> bool:
    """An object is stale when its source, any header beside it or the public header is newer."""
    if not os.path.exists(obj):
        return True
    deps = [os.path.join(CSRC, src)] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    deps += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE)]
    return any(os.path.getmtime(d) > os.path.getmtime(obj) for d in deps)


def build(verbose: bool = True, only_changed: bool = False) -> str:
    """Compile every source (or, with ``only_changed``, the ones whose object is older than its inputs) and link."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in srcs]
    all_objs = objs
    if only_changed:
        keep = [i for i, (s, o) in enumerate(zip(srcs, objs)) if _stale(s, o)]
        srcs, objs = [srcs[i] for i in keep], [objs[i] for i in keep]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])

    if srcs:
        with ThreadPoolExecutor(max_workers=min(os.cpu_count() or 4, 8, len(srcs))) as ex:
            for src, out in zip(srcs, ex.map(compile_one, zip(srcs, objs))):
                if verbose and out.strip():
                    print("[%s]\n%s" % (src, out))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + all_objs)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build(only_changed="--changed" in sys.argv[1:])
    sys.exit(0)
