// Shared helpers for the gfx950 optimizer kernels: status handling, bf16 bit
// arithmetic, the counter-based dither hash, wavefront reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/anc_optim.h"

void anc_set_error(const char *fmt, ...);
int anc_hip_fail(hipError_t e, const char *what, const char *file, int line);

#define ANC_HIP(call)                                                       \
  do {                                                                      \
    hipError_t e_ = (call);                                                 \
    if (e_ != hipSuccess) return anc_hip_fail(e_, #call, __FILE__, __LINE__); \
  } while (0)

#define ANC_REQUIRE(cond, ...)                                              \
  do {                                                                      \
    if (!(cond)) { anc_set_error(__VA_ARGS__); return ANC_ERR_ARG; }        \
  } while (0)

// Launch check: hipGetLastError right after a launch catches bad configurations.
#define ANC_LAUNCH_CHECK() ANC_HIP(hipGetLastError())

static inline hipStream_t anc_stream(uint64_t s) { return reinterpret_cast<hipStream_t>(s); }

// Optional per-launch timing (anc_profile_enable): when on, every kernel launch of the
// library is bracketed by a pair of HIP events on its stream, attributed to a kernel kind.
void anc_prof_begin(int kind, hipStream_t s);
void anc_prof_end(hipStream_t s);
struct AncProfScope {
  hipStream_t s;
  AncProfScope(int kind, hipStream_t st) : s(st) { anc_prof_begin(kind, s); }
  ~AncProfScope() { anc_prof_end(s); }
};

// ---------------------------------------------------------------- bf16 bits
// Round-to-nearest-even fp32 -> bf16 as the integer formula the reference uses on
// the host (ancora/optim/adamw.py:63-65): u + 0x7FFF + ((u >> 16) & 1), then >> 16.
__device__ __forceinline__ uint32_t anc_bf16_rne_bits(float x) {
  uint32_t u = __float_as_uint(x);
  u = u + 0x7FFFu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ float anc_bf16_bits_to_f32(uint32_t b) {
  return __uint_as_float(b << 16);
}

// Dither of the stochastic downcast (ancora/kernels/fused.py:154-161): a 16-bit
// hash of the element's global (row, col) and the per-step seed, all uint32.
__device__ __forceinline__ uint32_t anc_sr_dither(uint32_t row, uint32_t col, uint32_t seed) {
  uint32_t h = ((row * 73856093u) ^ (col * 19349663u) ^ seed) * 0x9E3779B1u;
  h ^= h >> 16;
  h *= 0x85EBCA6Bu;
  h ^= h >> 13;
  return h & 0xFFFFu;
}
// Stochastic rounding fp32 -> bf16 bits: (bits + dither) >> 16. Inf/NaN pass through
// (a NaN keeps a non-zero mantissa) instead of carrying into the sign bit.
__device__ __forceinline__ uint32_t anc_bf16_sr_bits(float x, uint32_t row, uint32_t col,
                                                     uint32_t seed) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7F800000u) == 0x7F800000u) {
    uint32_t b = u >> 16;
    if (u & 0x007FFFFFu) b |= 0x0040u;
    return b;
  }
  return (u + anc_sr_dither(row, col, seed)) >> 16;
}

// ------------------------------------------------------- wavefront reductions
// Butterfly over the 64 lanes with a fixed xor pattern: every lane ends with the
// same value, and the association order is the same on every run.
__device__ __forceinline__ double anc_wave_sum_f64(double v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float anc_wave_sum_f32(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Clang vector types: 8- and 16-byte global accesses, usable with the
// non-temporal load/store builtins.
typedef uint32_t anc_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t anc_u32x2 __attribute__((ext_vector_type(2)));
typedef float    anc_f32x4 __attribute__((ext_vector_type(4)));
typedef float    anc_f32x2 __attribute__((ext_vector_type(2)));

// Streaming accesses: every optimizer tensor is touched once per step, so loads and
// stores carry the non-temporal hint and do not displace reusable lines in L2.
template <typename T> __device__ __forceinline__ T anc_ld_stream(const T *p) {
  return __builtin_nontemporal_load(p);
}
template <typename T> __device__ __forceinline__ void anc_st_stream(T *p, T v) {
  __builtin_nontemporal_store(v, p);
}
