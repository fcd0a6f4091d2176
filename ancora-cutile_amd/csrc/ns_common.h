// Shared declarations of the Newton-Schulz GEMM kernels: the argument block, the
// epilogue kinds, the XCD-aware tile remap.
#pragma once
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int PITCH = BK + 8;            // bf16 elements per LDS row: 144 bytes
constexpr int kGemmThreads = 256;
constexpr int kXcds = 8;

enum { EPI_GRAM = 0, EPI_BMAT = 1, EPI_BX = 2 };

// Workgroup id -> logical tile id such that logical ids [start(x), start(x+1)) run on XCD x
// (hardware deals consecutive workgroup ids round-robin over the 8 XCDs).
__device__ __forceinline__ int xcd_remap(int bid, int grid) {
  const int x = bid % kXcds, q = bid / kXcds;
  const int base = grid / kXcds, rem = grid % kXcds;
  return x * base + (x < rem ? x : rem) + q;
}

struct NsGemm {
  const uint16_t *A[3];      // term t: rows of the output  (tiles_m*128 rows, ld = K)
  const uint16_t *B[3];      // term t: columns of the output (tiles_n*128 rows, ld = K)
  int nterms;
  int K;
  int64_t strideA, strideB;  // elements between consecutive matrices
  int tiles_m, tiles_n;
  int lower;                 // symmetric output: tiles with tn <= tm only, mirrored
  int M, N;                  // matrix dims of the chain (A, B are MxM; X is MxN)
  float ca, cb, cc;
  float *A32;                // (E,M,M) fp32 A            GRAM out, BMAT in
  uint16_t *Fh;              // (E,M,M) bf16 off-diag A   GRAM out
  uint16_t *Fl, *Bl;         // bf16 residuals of F and Boff; null unless this step splits them
  float *dA;                 // (E,M)   diag A            GRAM out, BMAT in
  uint16_t *Bh;              // (E,M,M) bf16 off-diag B   BMAT out
  float *dB;                 // (E,M)   diag B            BMAT out, BX in
  float *X32;                // (E,M,N) fp32 iterate      BX in/out
  uint16_t *Yh, *YhT;        // next iterate bf16 (M,N) and (N,M); null on the last step
  uint16_t *Yl, *YlT;        // bf16 residual copies; null unless the next step splits
};


// 256x256-tile kernel (ns_gemm_big.hip): same products, same accumulation order and
// therefore the same bits as the 128x128 kernel; used when M and N are multiples of 256.
int anc_ns_gemm_big(int epi, const NsGemm &p, int64_t E, hipStream_t s);
