// Deterministic global gradient norm for gfx950, no atomics.
//
// The reference has no gradient norm; the reduction shape follows its two fixed-order
// patterns: the single-block sum of `_fro_recip` (ancora/kernels/muon_ns.py:156-165)
// and the partial + reduce pair of the RMSNorm weight gradient
// (ancora/model/resident_train.py:295-298).
//
// Stage 1, one block of 256 lanes per chunk of ANC_GN_CHUNK = 8192 elements (chunk
// boundaries are fixed relative to the tensor start, elements past the end count as 0):
//   for j in 0..3: lane t takes the 8 consecutive elements of vector j*256 + t, adds
//     their squares left to right in fp32 (a bf16 square is exact in fp32), widens the
//     8-sum to fp64 and adds it to its fp64 accumulator;
//   the 64 lanes of a wavefront are combined by an xor butterfly (32,16,...,1);
//   the 4 wavefront sums are added in wavefront order.
// Stage 2, one block of 1024 lanes: lane t adds partials t, t+1024, ... in order, then
// the same butterfly, then the 16 wavefront sums in order. The result depends on the
// tensor sizes only: never on the grid, the launch grouping or the run.
#include <atomic>

#include "reduce.h"

namespace {

using namespace anc_reduce;

template <int GD>
__global__ void __launch_bounds__(kThreads)
k_gn_partials(const void *__restrict__ g, int64_t n, double *__restrict__ partials) {
  chunk_partial<GD>(g, n, (int64_t)blockIdx.x, partials + blockIdx.x);
}

__global__ void __launch_bounds__(kThreads)
k_gn_partials_multi(const anc_gn_desc_t *__restrict__ table, int n_tensors,
                    double *__restrict__ partials) {
  const int64_t chunk = (int64_t)blockIdx.x;
  int lo = 0, hi = n_tensors - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid].chunk0 <= chunk) lo = mid; else hi = mid - 1;
  }
  const anc_gn_desc_t d = table[lo];
  const int64_t local = chunk - d.chunk0;
  double *out = partials + d.part0 + local;
  if (d.dtype == ANC_BF16) chunk_partial<ANC_BF16>((const void *)d.g, d.n, local, out);
  else                     chunk_partial<ANC_F32>((const void *)d.g, d.n, local, out);
}

constexpr int kFinThreads = 1024;

__global__ void __launch_bounds__(kFinThreads)
k_gn_finalize(const double *__restrict__ partials, int64_t n_partials, float max_norm, float eps,
              int count_step, anc_step_ctl_t *__restrict__ ctl) {
  __shared__ double wave_sum[kFinThreads / 64];
  double acc = 0.0;
  for (int64_t i = threadIdx.x; i < n_partials; i += kFinThreads) acc = acc + partials[i];
  acc = anc_wave_sum_f64(acc);
  if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double t = wave_sum[0];
#pragma unroll
    for (int w = 1; w < kFinThreads / 64; ++w) t = t + wave_sum[w];
    const bool finite = (t == t) && (t - t == 0.0);   // neither NaN nor Inf
    const float norm = (float)sqrt(t);
    float clip = 1.0f;
    if (finite && max_norm > 0.0f) {
      const float s = max_norm / (norm + eps);
      clip = s < 1.0f ? s : 1.0f;
    }
    ctl->sumsq = t;
    ctl->norm = norm;
    ctl->clip_scale = clip;
    ctl->skip = finite ? 0u : 1u;
    if (count_step && finite) ctl->t = ctl->t + 1u;      // a skipped step is not counted
    ctl->reserved[0] = ctl->reserved[1] = 0u;
  }
}

}  // namespace

extern "C" int64_t anc_gradnorm_num_partials(int64_t n) {
  return n <= 0 ? 0 : (n + ANC_GN_CHUNK - 1) / ANC_GN_CHUNK;
}

extern "C" int anc_gradnorm_partials(uint64_t g, int64_t n, int g_dtype, uint64_t partials,
                                     int64_t part_offset, uint64_t stream) {
  ANC_REQUIRE(g != 0 && partials != 0 && n > 0 && part_offset >= 0,
              "anc_gradnorm_partials: bad arguments (n=%lld)", (long long)n);
  ANC_REQUIRE(g_dtype == ANC_F32 || g_dtype == ANC_BF16, "anc_gradnorm_partials: bad dtype %d",
              g_dtype);
  ANC_REQUIRE((g & 15) == 0 && (partials & 7) == 0, "anc_gradnorm_partials: misaligned pointers");
  const int64_t chunks = anc_gradnorm_num_partials(n);
  ANC_REQUIRE(chunks < (1ll << 31), "anc_gradnorm_partials: tensor too large for one launch");
  double *out = (double *)partials + part_offset;
  AncProfScope prof(ANC_PROF_GN_PARTIALS, anc_stream(stream));
  if (g_dtype == ANC_BF16)
    hipLaunchKernelGGL(k_gn_partials<ANC_BF16>, dim3((unsigned)chunks), dim3(kThreads), 0,
                       anc_stream(stream), (const void *)g, n, out);
  else
    hipLaunchKernelGGL(k_gn_partials<ANC_F32>, dim3((unsigned)chunks), dim3(kThreads), 0,
                       anc_stream(stream), (const void *)g, n, out);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_gradnorm_partials_multi(uint64_t desc_table, int32_t n_tensors,
                                           int64_t total_chunks, uint64_t partials,
                                           uint64_t stream) {
  ANC_REQUIRE(desc_table != 0 && n_tensors > 0 && partials != 0,
              "anc_gradnorm_partials_multi: bad arguments");
  ANC_REQUIRE(total_chunks > 0 && total_chunks < (1ll << 31),
              "anc_gradnorm_partials_multi: total_chunks=%lld out of range", (long long)total_chunks);
  AncProfScope prof(ANC_PROF_GN_PARTIALS, anc_stream(stream));
  hipLaunchKernelGGL(k_gn_partials_multi, dim3((unsigned)total_chunks), dim3(kThreads), 0,
                     anc_stream(stream), (const anc_gn_desc_t *)desc_table, (int)n_tensors,
                     (double *)partials);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_gradnorm_finalize(uint64_t partials, int64_t n_partials, float max_norm,
                                     float eps, int32_t count_step, uint64_t ctl, uint64_t stream) {
  ANC_REQUIRE(partials != 0 && ctl != 0 && n_partials > 0,
              "anc_gradnorm_finalize: bad arguments (n_partials=%lld)", (long long)n_partials);
  ANC_REQUIRE((ctl & 7) == 0, "anc_gradnorm_finalize: ctl must be 8-byte aligned");
  AncProfScope prof(ANC_PROF_GN_FINALIZE, anc_stream(stream));
  hipLaunchKernelGGL(k_gn_finalize, dim3(1), dim3(kFinThreads), 0, anc_stream(stream),
                     (const double *)partials, n_partials, max_norm, eps, (int)count_step, (anc_step_ctl_t *)ctl);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

// ------------------------------------------------------------------ no-allocation variant
// anc_gradnorm_static keeps the stage-1 partial sums in a file-scope device array instead of a
// caller-owned buffer, for callers that cannot allocate (HIP graph capture, tight serving loops).
// Every GPU holds its own copy of the array at its own address; the address is looked up once
// per device (anc_gradnorm_static_init, called by anc_init, or lazily on a device's first call)
// and host code only ever uses that looked-up pointer: the array's name is a host-side stand-in,
// not a device address.
#define ANC_GN_STATIC_MAX_PARTIALS 262144          /* 2 MiB of fp64 partials: n <= 2^31 elements */
static __device__ __align__(256) double scratch[ANC_GN_STATIC_MAX_PARTIALS];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<double *> g_scratch_ptr[kMaxDevices];
}  // namespace

// Look up the device address of `scratch` on the current device (once per device).
int anc_gradnorm_static_init(void) {
  int dev = 0;
  ANC_HIP(hipGetDevice(&dev));
  ANC_REQUIRE(dev >= 0 && dev < kMaxDevices, "anc_gradnorm_static: device index %d beyond %d", dev, kMaxDevices);
  if (g_scratch_ptr[dev].load(std::memory_order_acquire) != nullptr) return ANC_OK;
  double *ptr = nullptr;
  ANC_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
  ANC_REQUIRE(ptr != nullptr, "anc_gradnorm_static: null address for the scratch array");
  g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  return ANC_OK;
}

extern "C" int64_t anc_gradnorm_static_max_elements(void) {
  return (int64_t)ANC_GN_STATIC_MAX_PARTIALS * ANC_GN_CHUNK;
}

extern "C" int anc_gradnorm_static(uint64_t g, int64_t n, int g_dtype, float max_norm, float eps,
                                   uint64_t ctl, uint64_t stream) {
  ANC_REQUIRE(g != 0 && ctl != 0 && n > 0, "anc_gradnorm_static: bad arguments (n=%lld)", (long long)n);
  ANC_REQUIRE(g_dtype == ANC_F32 || g_dtype == ANC_BF16, "anc_gradnorm_static: bad dtype %d", g_dtype);
  ANC_REQUIRE((g & 15) == 0 && (ctl & 7) == 0, "anc_gradnorm_static: misaligned pointers");
  const int64_t chunks = anc_gradnorm_num_partials(n);
  ANC_REQUIRE(chunks <= ANC_GN_STATIC_MAX_PARTIALS,
              "anc_gradnorm_static: n=%lld exceeds the built-in scratch (at most %lld elements); use "
              "anc_gradnorm_partials + anc_gradnorm_finalize with a caller-owned buffer",
              (long long)n, (long long)anc_gradnorm_static_max_elements());
  if (int rc = anc_gradnorm_static_init()) return rc;
  int dev = 0;
  ANC_HIP(hipGetDevice(&dev));
  double *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  // Stage 1 overwrites partials [0, chunks) and stage 2 reads exactly those: nothing of an
  // earlier call is read, so nothing needs clearing.
  hipStream_t s = anc_stream(stream);
  if (g_dtype == ANC_BF16)
    hipLaunchKernelGGL(k_gn_partials<ANC_BF16>, dim3((unsigned)chunks), dim3(kThreads), 0, s, (const void *)g, n, ptr);
  else
    hipLaunchKernelGGL(k_gn_partials<ANC_F32>, dim3((unsigned)chunks), dim3(kThreads), 0, s, (const void *)g, n, ptr);
  ANC_LAUNCH_CHECK();
  hipLaunchKernelGGL(k_gn_finalize, dim3(1), dim3(kFinThreads), 0, s, (const double *)ptr, chunks, max_norm, eps, 0,
                     (anc_step_ctl_t *)ctl);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}
