"""Compile the HIP sources under csrc/ into csrc/libancora_optim.so for gfx950.

    python -m ancora_cutile_amd.build

hipcc cross-compiles without a GPU. Flags: no FMA contraction (the AdamW kernel must
reproduce a numpy fp32 evaluation operation by operation), correctly rounded fp32
divide/sqrt, packed-fp32 instruction selection switched off.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(CSRC, "libancora_optim.so")

FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
         "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-inline-asm"]


def build(verbose=True):
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    target, objdir = OUT, CSRC
    objs = []
    procs = []
    for s in srcs:
        o = os.path.join(objdir, os.path.basename(s)[:-4] + ".o")
        cmd = [hipcc, *[f for f in FLAGS if f != "-shared"], "-c", s, "-o", o]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(o)
    failed = False
    for s, p in procs:
        out = p.communicate()[0].decode("utf-8", "replace")
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l]
        if lines and verbose:
            print("\n".join(lines))
        if p.returncode != 0:
            print(out, file=sys.stderr)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", target]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return target


if __name__ == "__main__":
    print(build())
