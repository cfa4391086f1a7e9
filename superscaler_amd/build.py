"""Builds libace_eval.so (HIP, gfx950) in-tree with hipcc; cross-compiles without a GPU."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libace_eval.so")
SOURCES = [os.path.join(HERE, "csrc", "ace_eval.hip")]
HEADERS = [os.path.join(HERE, "csrc", "ace_plan_state.h"), os.path.join(HERE, "csrc", "ace_score_loop.h"),
           os.path.join(HERE, "csrc", "ace_score_loop_asm.inc"), os.path.join(HERE, "csrc", "ace_edit_kernels.h"),
           os.path.join(ROOT, "include", "ace_eval.h")]

# -ffp-contract=off: the scoring arithmetic must round exactly like the reference's Python floats,
# so a*b+c may never be fused.  packed-fp32 ops are switched off for the whole translation unit.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "csrc")]


def source_hash() -> str:
    """sha256 over the library's sources (the files `build` compiles, in a fixed order): names what a set of
    profile readings was taken on."""
    import hashlib
    h = hashlib.sha256()
    for path in sorted(SOURCES + HEADERS):
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def build(verbose: bool = True) -> str:
    hipcc = os.environ.get("HIPCC", "hipcc")
    cmd = [hipcc] + FLAGS + SOURCES + ["-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


def is_stale() -> bool:
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    return any(os.path.getmtime(p) > t for p in SOURCES + HEADERS)


if __name__ == "__main__":
    build()
    sys.exit(0)
