"""Build the package's HIP libraries (gfx950) in-tree with hipcc.  No GPU is needed to build.

Three libraries, each from its own folder of translation units, so that a model only waits for what it runs on:
  qlinear  csrc/*.hip         -> nanovllm/_lib/libqlinear.so   (quantized linears, Qwen3 operators, attention)
  seqmix   csrc/seqmix/*.hip  -> nanovllm/_lib/libseqmix.so    (multi-stream residuals, short convolutions, latent
                                                                attention with or without a rotated part and a window,
                                                                PolyNorm / clamped GLU / GELU experts, expert routing)
  hymix    csrc/hymix/*.hip   -> nanovllm/_lib/libhymix.so     (gated, grouped-norm and tanh-norm residuals, token shift,
                                                                attention with sinks, windows, pooled blocks, chunked
                                                                masks and sigmoid weights over a paged cache, delta-rule
                                                                and constant-decay recurrences)
``python build.py [--force] [qlinear|seqmix|hymix]`` builds one of them, or all without a name."""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "nanovllm", "_lib")
LIB = os.path.join(OUT_DIR, "libqlinear.so")
SEQMIX_LIB = os.path.join(OUT_DIR, "libseqmix.so")
HYMIX_LIB = os.path.join(OUT_DIR, "libhymix.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fno-gpu-rdc"]
# the packed-f32 VALU forms stay off in the newer library (plain f32 code only)
NO_PACKED_F32 = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
TARGETS = {
    "qlinear": dict(src=CSRC, lib=LIB, header="qlinear.h", flags=FLAGS, obj=""),
    "seqmix": dict(src=os.path.join(CSRC, "seqmix"), lib=SEQMIX_LIB, header="seqmix.h", flags=FLAGS + NO_PACKED_F32, obj="seqmix_"),
    "hymix": dict(src=os.path.join(CSRC, "hymix"), lib=HYMIX_LIB, header="hymix.h", flags=FLAGS + NO_PACKED_F32, obj="hymix_"),
}


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True, target="qlinear"):
    """Compile one library (``target`` = "qlinear" | "seqmix") or all of them ("all"); returns the path of the (last) library."""
    if target == "all":
        for name in TARGETS:
            lib = build(force, verbose, name)
        return lib
    spec = TARGETS[target]
    CSRC, LIB, FLAGS = spec["src"], spec["lib"], spec["flags"]
    os.makedirs(OUT_DIR, exist_ok=True)
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    hipcc = _hipcc()
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(HERE, "..", "include", spec["header"]))
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))      # every translation unit of the folder

    def compile_one(src):
        obj = os.path.join(objdir, spec["obj"] + src.replace(".hip", ".o"))
        path = os.path.join(CSRC, src)
        if force or _stale(obj, [path] + headers):
            cmd = [hipcc] + FLAGS + ["-c", path, "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            subprocess.check_call(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(compile_one, srcs))
    if force or _stale(LIB, objs):
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    names = [a for a in sys.argv[1:] if not a.startswith("-")] or ["all"]
    for name in names:
        print(build(force="--force" in sys.argv, target=name))
