"""CPU restatement (numpy) of the reference's Muon + AdamW optimizer step.

TEST INFRASTRUCTURE ONLY. Nothing in the product package imports this directory; it is
used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py, and
only as the checker or the timed baseline, never as the thing shipped.

Every function cites the reference lines (path:line under the reference repository
root) it restates; the reference itself cannot be imported (its modules import
cuda.tile and a Windows-only ancora.env at module top), so the restatement was written
from the source text.

How each function is pinned (see tests/test_oracle_*.py):
  adamw_step_div / adamw_step_ibc   reference-held case of tests/optim/test_adamw.py:19-43
                                    (seed 0, 5 steps, rel < 1e-5 between the two forms);
                                    closed forms: t=1 gives dp = -lr*g/(|g|+eps) - lr*wd*p,
                                    g=0 decays m and v only, an fp64 evaluation agrees to 1e-6
  bf16_rne_bits                     exhaustive halfway/tie cases and a value-level definition
                                    (nearest bf16, ties to even) by brute force over candidates
  sr_dither / bf16_sr_bits          exact-grid invariance and unbiasedness over 400 seeds
                                    (tests/kernels/_probe_sr_ops.py:41-66), hand-computed hash
  gradnorm_f64 / gradnorm_fixed     closed forms (constant vectors, 3-4-5), fsum brute force,
                                    the two agree to 1 ulp
  newton_schulz5 / host_ns          SVD cross-check U p(S) V^T, transpose equivariance, scale
                                    invariance, zero input, ortho_err(PE5) < ortho_err(Keller5)
                                    (tests/kernels/_probe_polar_express_device.py:83)
  muon_step / hybrid routing        table-driven over the Qwen3 / MoE name lists, shape scale
                                    sqrt(max(1, rows/cols)) on square, wide and tall weights
  quant_mxfp8_w / e4m3_rne          (quant_ref.py) format constants, midpoints and their neighbours,
                                    an independent integer-bit formulation over every bf16 input
                                    and every reachable scale, powers of two, zero blocks, the
                                    format's error bound and the reference-held 8 % acceptance
                                    (tests/kernels/test_gpu_quant.py:45-47,68)
  gemm_dw                           (gemm_ref.py) the reference's own checker, an fp64 library
                                    matrix product of the bf16 inputs (tests/kernels/test_gemm_bwd.py:40-44)
  id_groups / embed_dw_rows /       (embed_ref.py) defining properties of the group arrays (permutation,
  embed_dw_scatter                  stability, counts), an exact integer case, the reference-held gate
                                    against an fp64 scatter-add (tests/kernels/test_embed_dw_scatter.py:55-61,91)
ns_chain_model.py and ns_inputs.py are not restatements of the reference: the first models the
arithmetic of this library's bf16 chain (rounding points, plan, gate statistics, the 8-bit low
half), the second holds input families for walking its thresholds. The model is pinned to the GPU
by tests/test_gpu_ns_model.py (errors against host_ns to three digits, gate decisions, two-step
results to 2e-6); the parity target of every Newton-Schulz test stays host_ns.
No function of the optimizer step is "parity unpinned". quant_mxfp8_w has three edge behaviours
that no reference-held vector fixes (blocks with amax < 2**-120, bf16 subnormal inputs,
non-finite inputs): they are parity unpinned and listed in the header of quant_ref.py.
"""
