"""Build libeagle_mi355x.so (the C-ABI library) in-tree with hipcc for gfx950.

    python -m mlx_eagle_spec_decoding_tree_amd.build        # or build.build()

hipcc cross-compiles without a GPU.  Packed fp32 instructions are disabled for
all device code (-packed-fp32-ops).
"""
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libeagle_mi355x.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-fvisibility=hidden", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the HIP extension cannot be built")


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose=False, jobs=8):
    """Compile every csrc/*.hip to an object (in parallel) and link the library."""
    cc = hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    flags = [f for f in FLAGS if f != "-shared"]
    for src in sources():
        obj = os.path.join(objdir, os.path.basename(src) + ".o")
        objs.append(obj)
        cmd = [cc, *flags, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        while sum(p.poll() is None for _, p in procs) >= jobs:
            procs[0][1].wait()
    for src, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        noise = "is not a recognized feature for this target"
        text = "\n".join(l for l in text.splitlines() if noise not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{text}")
        if verbose and text.strip():
            print(text)
    tmp = LIB + ".tmp"
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout.decode(errors="replace"))
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
