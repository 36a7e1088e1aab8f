"""Build the gfx950 shared library (hipcc cross-compiles without a GPU).

    python -m ktransformers_amd.build [--force]

Every csrc/*.hip is compiled to its own object (in parallel, only when it or a header it may include changed) and the
objects are linked into ktransformers_amd/lib/libktx_hip.so (git-ignored, travels with the gpurun snapshot).
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB = os.path.join(LIBDIR, "libktx_hip.so")
# the sequence-mixer, hybrid-decoder and window-attention / scan kernels alone (include/ktx_seq.h, ktx_hyb.h, ktx_swa.h): what the fp32-residual families need, built in
# well under a minute
SEQ_LIB = os.path.join(LIBDIR, "libktx_seq.so")
SEQ_SOURCES = ("ktx_seq.hip", "ktx_hyb.hip", "ktx_swa.hip", "ktx_err.hip")

# -ffp-contract=off: the parity contract needs every fp32 op rounded exactly as the reference's AVX512 code does;
# FMAs appear only where the reference issues one (explicit fmaf()).
CFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fPIC", "-Wno-unused-value"]


# per-source extra flags: the sequence-mixer kernels keep fp32 state and norms on the vector ALUs and are built without the packed
# fp32 instructions (scalar v_fma / v_mul only)
_NO_PACKED_FP32 = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
EXTRA_CFLAGS = {"ktx_seq.hip": _NO_PACKED_FP32, "ktx_hyb.hip": _NO_PACKED_FP32, "ktx_swa.hip": _NO_PACKED_FP32}


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _headers() -> list[str]:
    return (glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(CSRC, "*.inc"))
            + glob.glob(os.path.join(HERE, "..", "include", "*.h")))


def _deps(src: str, seen: set | None = None) -> list[str]:
    """The headers a source reaches through its quoted #include lines (searched beside the including file and in include/)."""
    import re
    seen = set() if seen is None else seen
    out = []
    try:
        text = open(src, encoding="utf-8", errors="replace").read()
    except OSError:
        return out
    for inc in re.findall(r'^\s*#\s*include\s*"([^"]+)"', text, flags=re.M):
        for base in (os.path.dirname(src), CSRC, os.path.join(HERE, "..", "include")):
            path = os.path.normpath(os.path.join(base, inc))
            if os.path.exists(path):
                if path not in seen:
                    seen.add(path)
                    out.append(path)
                    out.extend(_deps(path, seen))
                break
    return out


def _obj(src: str) -> str:
    return os.path.join(OBJDIR, os.path.basename(src)[:-4] + ".o")


def _stale(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build_seq(force: bool = False, verbose: bool = False) -> str:
    """libktx_seq.so from SEQ_SOURCES only (ktransformers_amd._native_seq loads it when libktx_hip.so is absent)."""
    srcs = [os.path.join(CSRC, n) for n in SEQ_SOURCES]
    if not force and not _stale(SEQ_LIB, [d for s in srcs for d in [s] + _deps(s)]):
        return SEQ_LIB
    os.makedirs(OBJDIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

    def compile_one(src: str) -> None:
        cmd = [hipcc, *CFLAGS, *EXTRA_CFLAGS.get(os.path.basename(src), []), "-c", src, "-o", _obj(src)]
        if verbose:
            print(" ".join(cmd), file=sys.stderr)
        subprocess.run(cmd, check=True)

    todo = [s for s in srcs if force or _stale(_obj(s), [s] + _deps(s))]
    with ThreadPoolExecutor(max_workers=max(1, min(len(todo), os.cpu_count() or 4))) as ex:
        list(ex.map(compile_one, todo))
    tmp = SEQ_LIB + f".tmp{os.getpid()}"
    subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[_obj(s) for s in srcs], "-o", tmp], check=True)
    os.replace(tmp, SEQ_LIB)
    return SEQ_LIB


def needs_build() -> bool:
    return _stale(LIB, sources() + _headers())


def build(force: bool = False, verbose: bool = False) -> str:
    if not force and not needs_build():
        return LIB
    os.makedirs(OBJDIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    hdrs = _headers()
    todo = [s for s in sources() if force or _stale(_obj(s), [s] + (_deps(s) or hdrs))]

    def compile_one(src: str) -> None:
        cmd = [hipcc, *CFLAGS, *EXTRA_CFLAGS.get(os.path.basename(src), []), "-c", src, "-o", _obj(src)]
        if verbose:
            print(" ".join(cmd), file=sys.stderr)
        subprocess.run(cmd, check=True)

    with ThreadPoolExecutor(max_workers=max(1, min(len(todo), os.cpu_count() or 4))) as ex:
        list(ex.map(compile_one, todo))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[_obj(s) for s in sources()], "-o", LIB]
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    if "--seq" in sys.argv:
        print(build_seq(force="--force" in sys.argv, verbose=True))
    else:
        print(build(force="--force" in sys.argv, verbose=True))
