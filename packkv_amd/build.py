"""Builds libpackkv_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m packkv_amd.build          # compile every kernel source and link
    python -m packkv_amd.build --changed   # recompile only what is older than its sources
    python -m packkv_amd.build --define PKV_ATTN_PROBE=30 --out /tmp/libpackkv_probe.so
                                        # a development build with extra -D flags under another name (objects in a
                                        # directory of their own); PACKKV_HIP_LIB=/tmp/libpackkv_probe.so loads it

The library has no PyTorch dependency: it is a plain C-ABI shared object (include/packkv.h)
that takes raw device pointers and a hipStream_t.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libpackkv_hip.so")
SOURCES = ["pkv_runtime.hip", "pkv_codec.hip", "pkv_codec_long.hip", "pkv_quant.hip", "pkv_legacy.hip", "pkv_attn.hip", "pkv_repack.hip", "pkv_cache.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


def _stale(src, obj):
    """True when `obj` is older than the source, any header beside it or the public header."""
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [os.path.join(CSRC, src), os.path.join(HERE, "..", "include", "packkv.h"), os.path.abspath(__file__)]
    deps += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, only_stale=False, defines=(), obj_dir=OBJ):
    obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
    if only_stale and not _stale(src, obj):
        return obj
    cmd = [_hipcc()] + FLAGS + ["-D" + d for d in defines] + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines()
                    if "packed-fp32-ops" not in l and "warning generated" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err:
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True, only_stale=False, defines=(), out=None):
    """Compile and link.  only_stale=True (``--changed`` on the command line) recompiles only the sources whose
    object file is older than the source or a header.  `defines` / `out`: a development build with extra -D flags,
    linked under another name."""
    lib = out or LIB
    obj_dir = OBJ if not defines else OBJ + "_" + "_".join(d.replace("=", "-") for d in defines)
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda src: _compile(src, only_stale, defines, obj_dir), SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", lib)
    return lib


if __name__ == "__main__":
    argv = sys.argv[1:]
    defs = [argv[i + 1] for i, a in enumerate(argv) if a == "--define" and i + 1 < len(argv)]
    outs = [argv[i + 1] for i, a in enumerate(argv) if a == "--out" and i + 1 < len(argv)]
    if defs and not outs:
        raise SystemExit("--define needs --out: a build with extra flags does not replace the library")
    build(only_stale="--changed" in argv, defines=tuple(defs), out=outs[0] if outs else None)
