"""Build libeagle_mi355x.so (the C-ABI library) in-tree with hipcc for gfx950.

    python -m mlx_eagle_spec_decoding_tree_amd.build        # or build.build()

hipcc cross-compiles without a GPU.  Packed fp32 instructions are disabled for
all device code (-packed-fp32-ops).

The compile also asks the backend for every kernel's resource usage
(-Rpass-analysis=kernel-resource-usage) and fails if a kernel that is not on
the list below keeps registers in scratch memory: a spill in a kernel of the
verification step or of the draft loop is a build error, not a slow surprise.
"""
import glob
import os
import re
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
    "-Rpass-analysis=kernel-resource-usage",
]

# Kernels that may spill, by a pattern on the demangled-free (mangled) name, with the reason.
# None of them runs in the verification step or in the draft loop of the benchmark configurations.
SCRATCH_ALLOWED = [
    # prompt chunks of 128 x rows by 256 weight rows: 128 accumulator registers plus the
    # operands of two weight tiles in flight; the 128 x 128 blocks do not spill
    (r"qmm_gemm_w4g64_kernelILi2ELi4E", "prompt GEMM, 128 x 256 blocks"),
    # sixteen waves (K above 3072) leave a wave 128 registers: too few with a second weight tile
    # (SwiGLU, rope) or with the norm weights of three chunks; the drafter's K is 896 there
    (r"qmm_small_kernelILi16ELi\dELi[12]E", "small-row kernel, sixteen waves, two tiles"),
    (r"qmm_small_kernelILi16ELi\dELi0ELb1E", "small-row kernel, sixteen waves, norm folded in"),
    # one query head per KV group at head dimension 128 on a tree above 32 tokens
    (r"tree_attn_split_kernelILi128ELb1ELi8ELi1ELi1E", "attention split, eight vectors per thread"),
]

_NAME = re.compile(r"Function Name: (\S+)")
_SCRATCH = re.compile(r"ScratchSize \[bytes/lane\]: (\d+)")


def scratch_report(text):
    """{kernel name: scratch bytes per lane} from the resource-usage remarks of one compile."""
    out = {}
    name = None
    for line in text.splitlines():
        m = _NAME.search(line)
        if m:
            name = m.group(1)
            continue
        m = _SCRATCH.search(line)
        if m and name:
            out[name] = int(m.group(1))
            name = None
    return out


def check_scratch(report):
    """Raise if a kernel outside SCRATCH_ALLOWED spills; returns the allowed ones that do."""
    allowed, bad = {}, {}
    for name, nbytes in report.items():
        if nbytes == 0:
            continue
        why = next((w for pat, w in SCRATCH_ALLOWED if re.search(pat, name)), None)
        (allowed if why else bad)[name] = (nbytes, why)
    if bad:
        lines = "\n".join(f"  {n}: {b} bytes per lane" for n, (b, _) in sorted(bad.items()))
        raise RuntimeError("kernels with registers spilled to scratch memory:\n" + lines)
    return allowed


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
    report = {}
    for src, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        report.update(scratch_report(text))
        noise = ("is not a recognized feature for this target", "-Rpass-analysis=kernel-resource-usage")
        text = "\n".join(l for l in text.splitlines() if not any(n in l for n in noise))
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{text}")
        if verbose and text.strip():
            print(text)
    if not report:
        raise RuntimeError("the compiler reported no kernel resource usage: the scratch check cannot run")
    allowed = check_scratch(report)
    if verbose:
        print(f"[build] {len(report)} kernels, {len(allowed)} on the allowed list use scratch memory")
        for n, (b, why) in sorted(allowed.items()):
            print(f"[build]   {b:4d} B/lane  {why}: {n}")
    tmp = LIB + ".tmp"
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout.decode(errors="replace"))
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
