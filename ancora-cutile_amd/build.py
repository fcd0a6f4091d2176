"""Compile the HIP sources under csrc/ into csrc/libancora_optim.so for gfx950.

    python -m ancora_cutile_amd.build
    python -m ancora_cutile_amd.build --define ANC_DBG_NOEPI --out /tmp/noepi.so

The second form builds an ablation variant somewhere else (objects in a temporary directory,
the product library untouched); `ANCORA_OPTIM_LIB=/tmp/noepi.so` makes the host layer load it.
Ablation switches of csrc/ns_gemm_big.hip: ANC_DBG_NOEPI (no epilogue), ANC_DBG_NODMA (operand
tiles fetched for the first K tiles only), ANC_DBG_NOMFMA (matrix instructions replaced by an add),
ANC_DBG_TRACE (per-workgroup timestamps of K loop and epilogue, read with anc_dbg_trace_read),
ANC_DBG_KNOWAIT (K loop does not wait for its DMA), ANC_DBG_EPI_NOST / ANC_DBG_EPI_NOLD (epilogue
without its global stores / without its input DMA); of csrc/ns.hip: ANC_DBG_SAMEOPS (every matrix of
a batch multiplies the first matrix's operands, i.e. cache-resident operands). All of these but
TRACE give wrong results: timing only. Two more switch an optimisation off and leave the results'
bits alone: ANC_DBG_NOSTEADY (the K loop always runs its branching body), ANC_DBG_BX_NT
(X = a X + B X fetches B by rows m in 64-byte pieces at every size; identical bits except for
chains with residual terms at M >= 1024).

hipcc cross-compiles without a GPU. Flags: no FMA contraction (the AdamW kernel must
reproduce a numpy fp32 evaluation operation by operation), correctly rounded fp32
divide/sqrt, packed-fp32 instruction selection switched off.
"""
import glob
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(CSRC, "libancora_optim.so")

FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
         "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-inline-asm"]


def build(verbose=True, defines=(), out=None):
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    target = out or OUT
    objdir = CSRC if target == OUT else tempfile.mkdtemp(prefix="ancora_build_")
    objs = []
    procs = []
    for s in srcs:
        o = os.path.join(objdir, os.path.basename(s)[:-4] + ".o")
        cmd = [hipcc, *[f for f in FLAGS if f != "-shared"], *[f"-D{d}" for d in defines], "-c", s, "-o", o]
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
    import argparse
    ap = argparse.ArgumentParser()
    ap.add_argument("--define", action="append", default=[], help="extra -D for every source")
    ap.add_argument("--out", default=None, help="output library (default: csrc/libancora_optim.so)")
    a = ap.parse_args()
    print(build(defines=a.define, out=a.out))
