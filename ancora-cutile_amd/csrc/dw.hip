// Weight-gradient GEMM dW (+)= x^T dy: the producer of the gradients the optimizer step reads.
//
// Replaces `_gemm_dW` / `_gemm_dW_acc` (ancora/kernels/fused.py:190-219, launched per weight at
// ancora/model/resident_train.py:285-287): x (T, K) and dy (T, N) bf16, fp32 accumulation over the
// T tokens, fp32 result, optionally added onto the existing dW (gradient accumulation in place).
// Here the product runs on the Newton-Schulz chain's X = a X + B X K loop (128x256 tiles, bf16
// MFMA, LDS-DMA stage ring): B = dy as it lies, and A either the activations as they lie, x (T, K)
// (`x_row_major`: the A tile is then [tokens][128 columns] and its fragments come from transposing
// LDS reads, like B's), or x^T (K, T) for a caller that keeps the activations transposed.
//
// By default one workgroup owns one output tile and runs the whole token axis, tokens in ascending
// order, one accumulator per element: fixed tiles, no split-K, so a gradient's bits are a function
// of x and dy alone, whatever shares the call and however the caller groups its calls. A single
// weight is only 50-200 tiles, far fewer than the 512 a launch needs to fill 256 CUs: a caller
// fills the GPU by handing over the 7 weights of a layer in one call (480 tiles at Qwen3-0.6B
// shapes). A caller that cannot do that may opt into cutting the token axis into S segments
// (`segments` > 1, or -1 for a rule that depends on the problem's shape alone): segment s of every
// tile is then its own workgroup and leaves an fp32 partial tile in the workspace, and a second,
// HBM-bound kernel adds the S partials in ascending order (and the old dW when accumulating) and
// can emit the bf16 copy the optimizer step reads. That split is deterministic, but the bits then
// depend on S (not on what else is in the call).
#include "reduce.h"
#include "ns_common.h"

namespace {

constexpr int kThreads = anc_reduce::kThreads;

// Segments of the token axis: the smallest power of two that gives the problem at least 256
// workgroups (one per CU), with at least 256 tokens per segment and segment length a multiple
// of 32.
int dw_segments(int64_t T, int64_t K, int64_t N) {
  const int64_t tiles = (K / 128) * (N / 256);
  int s = 1;
  while (tiles * s < 256 && T % (2 * s * 32) == 0 && T / (2 * s) >= 256) s *= 2;
  return s;
}

struct DwReduce {
  const float *part;     // (S, n) partials
  float *dW;             // (n)
  uint16_t *g16;         // (n) or null
  double *gn;            // (n / ANC_GN_CHUNK) grad-norm partials or null
  int64_t n;
  int S;
  int accumulate;
};
struct DwReduceMulti {
  int count;
  int64_t blk0[kMaxGroups + 1];
  DwReduce r[kMaxGroups];
};

// One block per 8192-element chunk of the flat gradient, elements dealt to the lanes exactly as
// the grad-norm kernel deals them (anc_reduce: run j*256 + lane = 8 consecutive elements), so that
// the chunk's sum of squares -- of the bf16 copy if one is emitted, else of the fp32 gradient --
// comes out with the bits the grad-norm kernel would produce from the stored gradient.
__global__ void __launch_bounds__(kThreads) k_dw_reduce(DwReduceMulti m) {
  using namespace anc_reduce;
  int q = 0;
  while (q + 1 < m.count && (int64_t)blockIdx.x >= m.blk0[q + 1]) ++q;
  const DwReduce &r = m.r[q];
  const int64_t chunk = (int64_t)blockIdx.x - m.blk0[q];
  float ss[kIters];
#pragma unroll
  for (int j = 0; j < kIters; ++j) {
    const int64_t i = chunk * (int64_t)ANC_GN_CHUNK + ((int64_t)j * kThreads + threadIdx.x) * kRun;
    anc_f32x4 a0 = {0.0f, 0.0f, 0.0f, 0.0f}, a1 = a0;
    if (r.accumulate) {
      a0 = anc_ld_stream((const anc_f32x4 *)(r.dW + i));
      a1 = anc_ld_stream((const anc_f32x4 *)(r.dW + i + 4));
    }
    for (int s = 0; s < r.S; ++s) {
      const float *pp = r.part + (int64_t)s * r.n + i;
      const anc_f32x4 v0 = anc_ld_stream((const anc_f32x4 *)pp);
      const anc_f32x4 v1 = anc_ld_stream((const anc_f32x4 *)(pp + 4));
      a0.x = a0.x + v0.x; a0.y = a0.y + v0.y; a0.z = a0.z + v0.z; a0.w = a0.w + v0.w;
      a1.x = a1.x + v1.x; a1.y = a1.y + v1.y; a1.z = a1.z + v1.z; a1.w = a1.w + v1.w;
    }
    anc_st_stream((anc_f32x4 *)(r.dW + i), a0);
    anc_st_stream((anc_f32x4 *)(r.dW + i + 4), a1);
    float x[kRun] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    if (r.g16 != nullptr) {
      uint32_t hb[kRun];
#pragma unroll
      for (int k = 0; k < kRun; ++k) {
        hb[k] = anc_bf16_rne_bits(x[k]);
        x[k] = anc_bf16_bits_to_f32(hb[k]);
      }
      const anc_u32x4 h = {hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16), hb[4] | (hb[5] << 16), hb[6] | (hb[7] << 16)};
      anc_st_stream((anc_u32x4 *)(r.g16 + i), h);
    }
    float sq = x[0] * x[0];
#pragma unroll
    for (int k = 1; k < kRun; ++k) sq = sq + x[k] * x[k];
    ss[j] = sq;
  }
  if (r.gn != nullptr) chunk_finish(ss, r.gn + chunk);      // uniform over the block
}

int check_dw(const anc_dw_problem_t &b, const char *who) {
  ANC_REQUIRE(b.T > 0 && b.K > 0 && b.N > 0 && b.T % 32 == 0 && b.K % 128 == 0 && b.N % 256 == 0,
              "%s: needs T %% 32 == 0, K %% 128 == 0, N %% 256 == 0 (T=%lld K=%lld N=%lld)", who,
              (long long)b.T, (long long)b.K, (long long)b.N);
  ANC_REQUIRE(b.T < (1ll << 31) && b.K < (1ll << 24) && b.N < (1ll << 24), "%s: dimension too large", who);
  return ANC_OK;
}

}  // namespace

extern "C" int64_t anc_gemm_dw_workspace_bytes(int64_t T, int64_t K, int64_t N) {
  anc_dw_problem_t b{};
  b.T = T; b.K = K; b.N = N;
  if (check_dw(b, "anc_gemm_dw_workspace_bytes")) return -1;
  return (int64_t)dw_segments(T, K, N) * K * N * 4;
}

extern "C" int anc_gemm_dw_multi(const anc_dw_problem_t *probs, int32_t n_probs, uint64_t stream) {
  ANC_REQUIRE(probs != nullptr && n_probs >= 1 && n_probs <= kMaxGroups, "anc_gemm_dw_multi: 1..%d problems",
              kMaxGroups);
  hipStream_t s = anc_stream(stream);
  NsGemm g[kMaxGroups];
  int64_t Es[kMaxGroups];
  DwReduceMulti rm{};
  rm.count = n_probs;
  int64_t blocks = 0;
  const bool tn = probs[0].x_row_major != 0;
  for (int q = 0; q < n_probs; ++q) {
    const anc_dw_problem_t &b = probs[q];
    if (int rc = check_dw(b, "anc_gemm_dw_multi")) return rc;
    // 0 or 1: no split of the token axis (the default: fixed tiles, no split-K, bits a function of
    // the inputs alone); -1: the shape rule; S > 1: S segments
    const int S = b.segments > 0 ? b.segments : b.segments == 0 ? 1 : dw_segments(b.T, b.K, b.N);
    ANC_REQUIRE(b.segments >= -1 && S <= 256 && b.T % ((int64_t)S * 32) == 0,
                "anc_gemm_dw_multi: segments=%d must be 0 or 1 (none), -1 (shape rule) or divide T=%lld into multiples of 32 tokens",
                (int)b.segments, (long long)b.T);
    // One segment and no grad-norm sums wanted: the GEMM's epilogue finishes the gradient itself
    // (old dW or 0 + product, bf16 copy), no partial tile and no second kernel. Same bits as
    // the two-kernel route: one fp32 addition per element onto the same accumulator value.
    const bool direct = S == 1 && b.gn_partials == 0;
    ANC_REQUIRE(b.xT != 0 && b.dy != 0 && b.dW != 0 && (direct || b.workspace != 0) &&
                ((b.xT | b.dy | b.dW | b.workspace | b.g16) & 15) == 0 && (b.gn_partials & 7) == 0,
                "anc_gemm_dw_multi: null or misaligned pointer");
    ANC_REQUIRE(direct || b.workspace_bytes >= (int64_t)S * b.K * b.N * 4,
                "anc_gemm_dw_multi: workspace holds %lld bytes, %lld needed",
                (long long)b.workspace_bytes, (long long)S * b.K * b.N * 4);
    ANC_REQUIRE((b.x_row_major != 0) == tn, "anc_gemm_dw_multi: the problems of a call must agree on x_row_major");
    const int64_t seg = b.T / S;
    NsGemm p{};
    p.A[0] = (const uint16_t *)b.xT;
    p.B[0] = (const uint16_t *)b.dy;
    p.nterms = 1;
    p.K = (int)seg;
    p.ldA = tn ? (int)b.K : (int)b.T;
    p.strideA = tn ? seg * b.K : seg;  // segment e starts seg rows further down x / seg elements further along every row of x^T
    p.strideB = seg * b.N;           // and seg rows further down dy
    p.M = (int)b.K;
    p.N = (int)b.N;
    p.X32 = (float *)b.workspace;    // partial e at e * K * N
    if (direct) {
      p.plain_sum = 1;
      p.X32 = (float *)b.dW;
      p.A32 = b.accumulate ? (float *)b.dW : nullptr;
      p.Yh = (uint16_t *)b.g16;
    }
    g[q] = p;
    Es[q] = S;
    rm.r[q] = DwReduce{(const float *)b.workspace, (float *)b.dW, (uint16_t *)b.g16, (double *)b.gn_partials,
                       b.K * b.N, S, b.accumulate ? 1 : 0};
    rm.blk0[q] = blocks;
    if (!direct) blocks += b.K * b.N / ANC_GN_CHUNK;     // K % 128 and N % 256: whole chunks only
  }
  rm.blk0[n_probs] = blocks;
  ANC_REQUIRE(blocks < (1ll << 31), "anc_gemm_dw_multi: too large");
  {
    AncProfScope prof(ANC_PROF_DW_GEMM, s);
    if (int rc = anc_ns_gemm_big_plain(g, Es, n_probs, s, tn)) return rc;
  }
  if (blocks > 0) {
    AncProfScope prof(ANC_PROF_DW_REDUCE, s);
    hipLaunchKernelGGL(k_dw_reduce, dim3((unsigned)blocks), dim3(kThreads), 0, s, rm);
  }
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

// Executed = dense FLOPs of one problem (every tile is multiplied in full) and the number of
// token segments it is cut into.
extern "C" int anc_gemm_dw_info(int64_t T, int64_t K, int64_t N, double *flops, int32_t *segments) {
  anc_dw_problem_t b{};
  b.T = T; b.K = K; b.N = N;
  if (int rc = check_dw(b, "anc_gemm_dw_info")) return rc;
  ANC_REQUIRE(flops != nullptr && segments != nullptr, "anc_gemm_dw_info: null output");
  *flops = 2.0 * (double)T * (double)K * (double)N;
  *segments = dw_segments(T, K, N);
  return ANC_OK;
}
