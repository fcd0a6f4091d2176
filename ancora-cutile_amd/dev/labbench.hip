// Lab bench, not part of libancora_optim.so: what this board's memory system and matrix pipe give
// kernels shaped like the optimizer's, as reference points beside the nominal 8 TB/s and
// 2.5 PFLOP/s (the reference's own method is a timed copy beside its AdamW kernel,
// tests/hardware/_probe_adamw_bw.py:24-25,58-91). Built on request into dev/liblabbench.so by
// `python -m ancora_cutile_amd.dev.labbench`, which also times the launches and prints the tables.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

typedef uint32_t anc_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t anc_u32x2 __attribute__((ext_vector_type(2)));
#define ANC_OK 0
#define ANC_REQUIRE(cond, ...) do { if (!(cond)) { fprintf(stderr, __VA_ARGS__); fputc('\n', stderr); return 2; } } while (0)
#define ANC_HIP(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_)); return 1; } } while (0)
#define ANC_LAUNCH_CHECK() ANC_HIP(hipGetLastError())

// ---- copy shapes: what bounds a streaming kernel on this memory system ------------------
// The same bytes moved by differently shaped kernels: the reference points for "how close to the
// achievable rate is an elementwise optimizer kernel", whose access mix (AdamW: four read and four
// write streams, 14 B each way per element) is not a plain copy's.
enum {
  COPY_NT = 0,         // the library's copy kernel: 256 lanes, 4 x 16 B in flight per lane, non-temporal
  COPY_PLAIN = 1,      // the same with ordinary loads and stores
  COPY_WIDE = 2,       // 256 lanes, 8 x 16 B in flight per lane
  COPY_PERSIST = 3,    // 2048 workgroups walking the buffer grid-stride, 4 x 16 B in flight
  COPY_B1024 = 4,      // 1024 lanes per workgroup, 4 x 16 B in flight
  COPY_READ = 5,       // read only (folded into one word per workgroup)
  COPY_WRITE = 6,      // write only
  COPY_ADAMW_MIX = 7,  // AdamW's streams without its arithmetic: per 4096-element block read
                       // 2+4+4+4 B/element from four arrays, write 4+4+4+2 to four arrays
  COPY_MOM_MIX = 8,    // momentum's: read 2+4, write 4+2+2
  COPY_SHAPES = 9
};

template <int INFLIGHT, bool NT, int THREADS>
__global__ void __launch_bounds__(THREADS) k_copy_shape(const anc_u32x4 *__restrict__ src,
                                                        anc_u32x4 *__restrict__ dst, int64_t n_vec, int persist) {
  const int64_t per = (int64_t)THREADS * INFLIGHT;
  for (int64_t blk = blockIdx.x; blk * per < n_vec; blk += persist ? gridDim.x : n_vec) {
    const int64_t base = blk * per + threadIdx.x;
    anc_u32x4 r[INFLIGHT];
#pragma unroll
    for (int j = 0; j < INFLIGHT; ++j) {
      const int64_t i = base + (int64_t)j * THREADS;
      if (i < n_vec) r[j] = NT ? __builtin_nontemporal_load(&src[i]) : src[i];
    }
#pragma unroll
    for (int j = 0; j < INFLIGHT; ++j) {
      const int64_t i = base + (int64_t)j * THREADS;
      if (i < n_vec) { if (NT) __builtin_nontemporal_store(r[j], &dst[i]); else dst[i] = r[j]; }
    }
  }
}
__global__ void __launch_bounds__(256) k_read_only(const anc_u32x4 *__restrict__ src, uint32_t *__restrict__ sink,
                                                  int64_t n_vec) {
  const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  uint32_t acc = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t i = base + j * 256;
    if (i < n_vec) { const anc_u32x4 r = __builtin_nontemporal_load(&src[i]); acc ^= r.x ^ r.y ^ r.z ^ r.w; }
  }
  if (acc == 0x9E3779B1u) sink[blockIdx.x & 255] = acc;      // practically never: keeps the loads alive
}
__global__ void __launch_bounds__(256) k_write_only(anc_u32x4 *__restrict__ dst, int64_t n_vec) {
  const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  const anc_u32x4 v = {1u, 2u, 3u, 4u};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t i = base + j * 256;
    if (i < n_vec) __builtin_nontemporal_store(v, &dst[i]);
  }
}
// Element-indexed streams as the optimizer kernels have them: block b owns elements
// [4096 b, 4096 b + 4096), lane t of slab j the four elements at 1024 j + 4 t.
template <bool MOM>
__global__ void __launch_bounds__(256) k_mix(const char *__restrict__ src, char *__restrict__ dst, int64_t n) {
  const int64_t base = (int64_t)blockIdx.x * 4096 + threadIdx.x * 4;
  // reads: a 2 B stream then 4 B streams; writes: 4 B streams then 2 B streams
  const anc_u32x2 *r2 = (const anc_u32x2 *)src;
  const anc_u32x4 *r4a = (const anc_u32x4 *)(src + 2 * n), *r4b = (const anc_u32x4 *)(src + 6 * n),
                  *r4c = (const anc_u32x4 *)(src + 10 * n);
  anc_u32x4 *w4a = (anc_u32x4 *)dst, *w4b = (anc_u32x4 *)(dst + 4 * n), *w4c = (anc_u32x4 *)(dst + 8 * n);
  anc_u32x2 *w2a = (anc_u32x2 *)(dst + (MOM ? 4 : 12) * n), *w2b = (anc_u32x2 *)(dst + 6 * n);
  anc_u32x2 g[4];
  anc_u32x4 a[4], b[4], c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t e = (base + j * 1024) / 4;
    g[j] = __builtin_nontemporal_load(&r2[e]);
    a[j] = __builtin_nontemporal_load(&r4a[e]);
    if (!MOM) { b[j] = __builtin_nontemporal_load(&r4b[e]); c[j] = __builtin_nontemporal_load(&r4c[e]); }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t e = (base + j * 1024) / 4;
    a[j].x ^= g[j].x; a[j].y ^= g[j].y;
    __builtin_nontemporal_store(a[j], &w4a[e]);
    if (!MOM) {
      __builtin_nontemporal_store(b[j], &w4b[e]);
      __builtin_nontemporal_store(c[j], &w4c[e]);
      __builtin_nontemporal_store(anc_u32x2{c[j].x, c[j].z}, &w2a[e]);
    } else {
      __builtin_nontemporal_store(anc_u32x2{a[j].x, a[j].z}, &w2a[e]);
      __builtin_nontemporal_store(anc_u32x2{a[j].y, a[j].w}, &w2b[e]);
    }
  }
}

extern "C" int lab_copy_shape(uint64_t dst, uint64_t src, int64_t n_bytes, int shape, int64_t *bytes_moved,
                              uint64_t stream) {
  ANC_REQUIRE(dst != 0 && src != 0 && n_bytes >= (1 << 20) && n_bytes % (1 << 20) == 0 && (dst & 255) == 0 &&
                  (src & 255) == 0 && bytes_moved != nullptr,
              "lab_copy_shape: buffers must be 256-byte aligned and a multiple of 1 MiB long");
  ANC_REQUIRE(shape >= 0 && shape < COPY_SHAPES, "lab_copy_shape: shape 0..%d", COPY_SHAPES - 1);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int64_t n_vec = n_bytes / 16;
  const auto grid = [&](int64_t per) { return dim3((unsigned)((n_vec + per - 1) / per)); };
  ANC_REQUIRE(n_vec / 1024 < (1ll << 31), "lab_copy_shape: size too large");
  *bytes_moved = 2 * n_bytes;
  switch (shape) {
    case COPY_NT: hipLaunchKernelGGL((k_copy_shape<4, true, 256>), grid(1024), dim3(256), 0, s, (const anc_u32x4 *)src, (anc_u32x4 *)dst, n_vec, 0); break;
    case COPY_PLAIN: hipLaunchKernelGGL((k_copy_shape<4, false, 256>), grid(1024), dim3(256), 0, s, (const anc_u32x4 *)src, (anc_u32x4 *)dst, n_vec, 0); break;
    case COPY_WIDE: hipLaunchKernelGGL((k_copy_shape<8, true, 256>), grid(2048), dim3(256), 0, s, (const anc_u32x4 *)src, (anc_u32x4 *)dst, n_vec, 0); break;
    case COPY_PERSIST: hipLaunchKernelGGL((k_copy_shape<4, true, 256>), dim3(2048), dim3(256), 0, s, (const anc_u32x4 *)src, (anc_u32x4 *)dst, n_vec, 1); break;
    case COPY_B1024: hipLaunchKernelGGL((k_copy_shape<4, true, 1024>), grid(4096), dim3(1024), 0, s, (const anc_u32x4 *)src, (anc_u32x4 *)dst, n_vec, 0); break;
    case COPY_READ: *bytes_moved = n_bytes; hipLaunchKernelGGL(k_read_only, grid(1024), dim3(256), 0, s, (const anc_u32x4 *)src, (uint32_t *)dst, n_vec); break;
    case COPY_WRITE: *bytes_moved = n_bytes; hipLaunchKernelGGL(k_write_only, grid(1024), dim3(256), 0, s, (anc_u32x4 *)dst, n_vec); break;
    case COPY_ADAMW_MIX: {
      const int64_t n = n_bytes / 14 / 4096 * 4096;          // elements: 14 B of each buffer per element
      *bytes_moved = 28 * n;
      hipLaunchKernelGGL(k_mix<false>, dim3((unsigned)(n / 4096)), dim3(256), 0, s, (const char *)src, (char *)dst, n);
      break;
    }
    default: {
      const int64_t n = n_bytes / 8 / 4096 * 4096;           // read 6 B, write 8 B per element
      *bytes_moved = 14 * n;
      hipLaunchKernelGGL(k_mix<true>, dim3((unsigned)(n / 4096)), dim3(256), 0, s, (const char *)src, (char *)dst, n);
    }
  }
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

// ------------------------------------------------------------------ matrix-core reference rate
// The matrix instruction of the Newton-Schulz GEMMs (v_mfma_f32_32x32x16_bf16) on register
// operands only, two wavefronts per SIMD on every CU, eight accumulator blocks per wavefront
// (the GEMM's register tile). What it sustains depends on the operand VALUES: the board runs
// under a power limit, and products of varying bf16 values draw more than products of zeros
// or of one constant. values: 0 zeros, 1 one constant pair, 2 pseudo-random values in
// (-0.05, 0.05), two fragment sets alternating. The counterpart of lab_copy_shape for the
// matrix pipe: the rate a GEMM's K loop could not exceed on this board with such operands.
typedef __bf16 mr_bf16x8 __attribute__((ext_vector_type(8)));
typedef float mr_f32x16 __attribute__((ext_vector_type(16)));
__device__ __forceinline__ uint32_t mr_hash(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}
__global__ void __launch_bounds__(512) k_mfma_rate(int values, int64_t iters, float *sink) {
  mr_f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  mr_bf16x8 a[2][4], b[2][2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
#pragma unroll
    for (int i = 0; i < 6; ++i)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t h = mr_hash(((uint32_t)threadIdx.x * 128u + (uint32_t)(s * 48 + i * 8 + e)) * 2654435761u + blockIdx.x);
        const float v = values == 0 ? 0.0f : values == 1 ? (i < 4 ? 0.5f : 0.25f)
                                                         : (float)((int)(h & 0xFFFFu) - 32768) * (0.05f / 32768.0f);
        if (i < 4) a[s][i][e] = (__bf16)v; else b[s][i - 4][e] = (__bf16)v;
      }
  }
  for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
  }
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) t += acc[i][j][0];
  if (t == 12345.0f) sink[threadIdx.x] = t;      // never true for these operands; keeps the loop alive
}

extern "C" int lab_mfma_rate(int values, int64_t iters, uint64_t sink, double *flops, uint64_t stream) {
  ANC_REQUIRE(values >= 0 && values <= 2 && iters > 0 && iters <= (1ll << 24) && sink != 0 && (sink & 3) == 0 &&
                  flops != nullptr,
              "lab_mfma_rate: values 0..2, iters 1..2^24, sink a device buffer of at least 2 KiB");
  hipDeviceProp_t pr;
  int dev = 0;
  ANC_HIP(hipGetDevice(&dev));
  ANC_HIP(hipGetDeviceProperties(&pr, dev));
  const int blocks = pr.multiProcessorCount;      // one 8-wavefront workgroup per CU
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(k_mfma_rate, dim3((unsigned)blocks), dim3(512), 0, s, values, iters, (float *)sink);
  ANC_LAUNCH_CHECK();
  *flops = (double)blocks * 8.0 * (double)iters * 16.0 * 2.0 * 32.0 * 32.0 * 16.0;
  return ANC_OK;
}
