// Shared declarations of the Newton-Schulz GEMM kernels: the argument block, the
// epilogue kinds, the XCD-aware tile remap.
#pragma once
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

// B-operand fragment of v_mfma_f32_32x32x16_bf16 from a (k, n) row-major LDS tile: two
// ds_read_b64_tr_b16. Within each group of 16 lanes, lane i receives the i%4-th 16-bit element
// of the 8 bytes addressed by lanes i/4, i/4+4, i/4+8, i/4+12 of the group. With lane s of a
// group pointing at row k0 + s/4, columns n0 + 4*(s%4) .. +3, lane i therefore receives
// column n0 + i of rows k0 .. k0+3. `p0` addresses rows k0.., `p1` rows k0+4..; the result
// holds 8 consecutive k of one column, the layout the matrix instruction wants.
__device__ __forceinline__ bf16x8 anc_lds_tr_frag(const void *p0, const void *p1) {
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)p0);
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)p1);
  const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// Two fp32 -> one dword of two bf16 (round to nearest even, v_cvt_pk_bf16_f32): a in the low half.
typedef __bf16 anc_bf16x2 __attribute__((ext_vector_type(2)));
typedef float anc_f32x2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t anc_pk_bf16(float a, float b) {
  const anc_f32x2v v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, anc_bf16x2));
}
// The bf16 pair of two values: hi = bf16(x), lo = bf16(x - hi), each packed as above.
__device__ __forceinline__ void anc_pk_pair(float a, float b, uint32_t &hi, uint32_t &lo) {
  hi = anc_pk_bf16(a, b);
  lo = anc_pk_bf16(a - __uint_as_float(hi << 16), b - __uint_as_float(hi & 0xFFFF0000u));
}

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int kCondParts = 8;            // partial sums per matrix of the conditioning proxy
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
  const uint16_t *B[3];      // term t: columns of the output. GRAM, BMAT: one row per column, ld = K
                             // ("NT" product); BX: the iterate itself, (K, N) row-major, ld = N
  int nterms;
  int K;
  int ldA;                   // elements between consecutive rows of A; 0 means K (only the plain
                             // product sets it: its A is a K-range of a longer row)
  int64_t strideA, strideB;  // elements between consecutive matrices
  int tiles_m, tiles_n;
  int lower;                 // symmetric output: tiles with tn <= tm only, mirrored
  int plain_sum;             // plain product: 1 = write X32 = (A32, if not null, else 0) + A B and, if Yh is
                             // not null, its bf16 copy (RNE) to Yh; 0 = write X32 = A B
  int blk_r, blk_c;          // plain product and X = a X + B X: the tile sequence of a matrix runs block by block, blocks of
                             // blk_r x blk_c tiles (rows x columns): (tiles_m, 1) = column panel by column
                             // panel, (1, tiles_n) or 0 = row by row
  int M, N;                  // matrix dims of the chain (A, B are MxM; X is MxN)
  float ca, cb, cc;
  float *A32;                // (E,M,M) fp32 A            GRAM out, BMAT in
  // With a32_gated set the fp32 copy of A exists only for the matrices that a32_flag marks (a null
  // a32_flag marks none): GRAM writes A32 for those alone and BMAT takes the off-diagonal entries
  // of A from Fh (bf16) for every other matrix. Fh is then read at the output position, which for
  // the 256-tile kernel means panel layout.
  int a32_gated;
  const int32_t *a32_flag;   // (E)
  uint16_t *Fh;              // (E,M,M) bf16 off-diag A   GRAM out
  uint16_t *Fl, *Bl;         // bf16 residuals of F and Boff; null unless this step splits them
  float *dA;                 // (E,M)   diag A            GRAM out, BMAT in
  uint16_t *Bh;              // (E,M,M) bf16 off-diag B   BMAT out
  float *dB;                 // (E,M)   diag B            BMAT out, BX in
  const uint16_t *Xh, *Xl;   // (E,M,N) current iterate as a bf16 pair, X = Xh + Xl   BX in
  uint16_t *Yh, *Yl;         // (E,M,N) next iterate as a bf16 pair   BX out, null on the last step
  float *X32;                // (E,M,N) fp32 result                   BX out on the last step, else null
  const anc_muon_desc_t *upd;  // BX, last step only: if set, matrix e is the Newton-Schulz result of the
                             // weight upd[e] and the epilogue applies W -= lr*O to it (p32, p16) instead
                             // of writing X32
  const double *cond;        // null, or (E, kCondParts) partial sums of the conditioning proxy (see
                             // k_ns_cond): a matrix whose sum exceeds cond_thresh multiplies
                             // nterms_hard terms instead of nterms (its list is a prefix of the hard one)
  double cond_thresh;
  int nterms_hard;
  // Second gate: a matrix that k_ns_classify flagged (a spectrum spread over decades, many
  // moderately large columns, a low-rank signal over weak noise) multiplies nterms_wide terms;
  // wide_flag null or nterms_wide 0 = no such gate. It takes precedence over the gate above. With
  // lo_gated set, the residual outputs Fl / Bl are written for such matrices only (else for every
  // matrix when non-null).
  const int32_t *wide_flag;  // (E)
  int nterms_wide;
  int lo_gated;
  const float *scale;        // (E) or null. The operands are an unnormalised iterate U and the step
                             // acts on X = scale*U: GRAM multiplies its accumulator by scale^2, BX
                             // multiplies the accumulator and the epilogue's X by scale.
  // Panel layout of a bf16 matrix with R rows: element (r, c) at ((c / 32) * R + r) * 32 + c % 32,
  // i.e. 32-column panels, each (R, 32) row-major. The K tile of a product is one panel, so the
  // rows a tile fetches are one contiguous block instead of 64-byte pieces of rows that lie a
  // whole row pitch apart. 256-tile kernel only; R = M for every matrix of the chain.
  int f_panel;               // Fh, Fl, Bh, Bl are in panel layout (GRAM, BMAT write them so; BMAT, BX read them so)
  int x_panel;               // the input iterate (operands X of GRAM and BX, Xh/Xl of the BX epilogue)
  int y_panel;               // the output iterate Yh/Yl of BX
  // 8-bit low halves (256-tile X = a X + B X, panel layout only). Where the low half of a matrix's
  // iterate is never a matrix-core operand it is kept as one byte per element (anc_low8_encode), in the first M*N bytes of the matrix's Xl (Yl) region, panels of
  // (M, 32) bytes: the epilogue then reads and writes 3 instead of 4 bytes per element. A matrix
  // takes the format on the input side if l8_in > 0, it is not flagged in l8_wide and its proxy
  // sum (l8_cond, the units of cond_thresh) does not exceed l8_in; l8_out likewise for the output.
  // The launches that read an iterate must be given the threshold it was written with.
  const double *l8_cond;     // (E, kCondParts) or null (no matrix takes the format)
  const int32_t *l8_wide;    // (E) or null
  double l8_in, l8_out;
};


// Per-matrix statistics and flags were written by earlier kernels and are the same for every lane:
// read through the constant address space they come in by scalar loads, which neither occupy the
// vector memory counter nor wait behind the kernel's own vector traffic.
template <typename T> __device__ __forceinline__ T anc_ld_const(const T *p) {
  return *(const __attribute__((address_space(4))) T *)(p);
}

// Number of accumulation terms of matrix e: p.nterms, or p.nterms_hard for a matrix that the
// conditioning proxy marks as hard. The partial sums are added in a fixed order, so every
// workgroup of every launch takes the same decision for a matrix.
__device__ __forceinline__ double anc_cond_sum(const double *cond, int e) {
  const double *c = cond + (int64_t)e * kCondParts;
  double s = anc_ld_const(c);
#pragma unroll
  for (int i = 1; i < kCondParts; ++i) s = s + anc_ld_const(c + i);
  return s;
}
__device__ __forceinline__ double anc_ns_proxy(const NsGemm &p, int e) { return anc_cond_sum(p.cond, e); }
// Did the classification flag matrix e for the second gate?
__device__ __forceinline__ bool anc_ns_wide(const NsGemm &p, int e) {
  return p.wide_flag != nullptr && anc_ld_const(p.wide_flag + e) != 0;
}
// Does matrix e keep the fp32 copy of A (GRAM writes it, BMAT reads it)?
__device__ __forceinline__ bool anc_ns_has_a32(const NsGemm &p, int e) {
  if (p.A32 == nullptr) return false;
  return p.a32_gated == 0 || (p.a32_flag != nullptr && anc_ld_const(p.a32_flag + e) != 0);
}
// Is the low half of matrix e's iterate one byte per element (thresh = p.l8_in or p.l8_out)?
__device__ __forceinline__ bool anc_ns_low8(const NsGemm &p, int e, double thresh) {
  if (!(thresh > 0.0) || p.l8_cond == nullptr) return false;
  if (p.l8_wide != nullptr && anc_ld_const(p.l8_wide + e) != 0) return false;
  return !(anc_cond_sum(p.l8_cond, e) > thresh);
}
// The 8-bit low half of y next to its high half h = bf16(y), in the integer space of the fp32 bit
// patterns, where rounding to bf16 is rounding to a multiple of 0x10000: d = bits(y) - (h << 16) lies
// in -0x8000 .. 0x8000, and q = (d + 0x80) >> 8 (capped at 127) is d rounded to 8 bits. The pair reads
// back as the float whose bits are (h << 16) + (q << 8): y to 24 bits, exponent carries and borrows
// included, no special cases. `htop` is h in the upper half of a dword (lower half zero).
__device__ __forceinline__ uint32_t anc_low8_encode(float y, uint32_t htop) {
  int d = (int)(__float_as_uint(y) - htop) + 0x80;
  d = d < 0x7FFF ? d : 0x7FFF;
  return ((uint32_t)d >> 8) & 0xFFu;
}
// x = Xh + Xl from htop and the byte q, sign-extended
__device__ __forceinline__ float anc_low8_decode(uint32_t htop, int q) {
  return __uint_as_float(htop + ((uint32_t)q << 8));
}
__device__ __forceinline__ int anc_ns_terms(const NsGemm &p, int e) {
  if (p.nterms_wide > 0 && anc_ns_wide(p, e)) return p.nterms_wide;
  if (p.cond == nullptr) return p.nterms;
  return anc_ns_proxy(p, e) > p.cond_thresh ? p.nterms_hard : p.nterms;
}

// Up to 8 independent problems of the same kind (the same product of different shape groups)
// in one launch: tiles[k] workgroups belong to problem k. One launch over all groups keeps the
// CUs busy where separate launches would each end in a partly filled last wave.
#ifndef ANC_MAX_GROUPS
#define ANC_MAX_GROUPS 8
#endif
constexpr int kMaxGroups = ANC_MAX_GROUPS;
struct NsGemmMulti {
  int n;
  int seq;                   // plain product: 1 = anc_seq_tile dealing, 0 = anc_group_tile
  int tiles[kMaxGroups];     // 0 past n
  int seg_start[kXcds + 1];  // anc_group_tile: first logical tile of each XCD's segment (anc_fill_segments)
  NsGemm g[kMaxGroups];
  // fused weight update (problems with `upd` set): lr*shape_scale by descriptor scale index,
  // stochastic-rounding switch and seed, the step's control block (skip flag) or null
  float lr[ANC_MUON_MAX_SCALES];
  int sr;
  uint32_t seed_base;
  const anc_step_ctl_t *ctl;
};
// Segment x holds the x-th eighth of every problem's tiles, problems in the order given.
inline void anc_fill_segments(NsGemmMulti &pm) {
  int at = 0;
  for (int x = 0; x < kXcds; ++x) {
    pm.seg_start[x] = at;
    for (int k = 0; k < pm.n; ++k) at += pm.tiles[k] / kXcds + (x < pm.tiles[k] % kXcds ? 1 : 0);
  }
  pm.seg_start[kXcds] = at;
}
struct NsUpdate {
  float lr[ANC_MUON_MAX_SCALES];
  int sr;
  uint32_t seed_base;
  const anc_step_ctl_t *ctl;
};

// Workgroup id -> (problem, tile index inside the problem). The logical tile sequence is cut
// into 8 segments, one per XCD (xcd_remap hands XCD x a contiguous range that coincides with
// segment x up to a few tiles); segment x holds the x-th eighth of every problem's tiles,
// problems in the order given (longest tiles first), so that every XCD gets the same mix and a
// problem's consecutive tiles -- the tiles of one matrix -- stay on one XCD.
__device__ __forceinline__ void anc_group_tile(const NsGemmMulti &pm, int bid, int grid, int &g, int &L) {
  int pos = xcd_remap(bid, grid);
  g = 0;
  L = pos;
  if (pm.n == 1) return;
  // the segment, from the starts the host summed up (anc_fill_segments); then the problem inside
  // it: all in scalar registers, no memory access inside the loops
  int T[kMaxGroups];
#pragma unroll
  for (int k = 0; k < kMaxGroups; ++k) T[k] = pm.tiles[k];          // (entries past pm.n are 0)
  int x = 0, start = 0;
#pragma unroll
  for (int xx = 1; xx < kXcds; ++xx) {
    const int st = pm.seg_start[xx];
    if (pos >= st) { x = xx; start = st; }
  }
  pos -= start;
  bool found = false;
#pragma unroll
  for (int k = 0; k < kMaxGroups; ++k) {
    const int base = T[k] / kXcds, rem = T[k] % kXcds;
    const int c = base + (x < rem ? 1 : 0);
    if (!found && pos < c) {
      found = true;
      g = k;
      L = x * base + (x < rem ? x : rem) + pos;
    }
    if (!found) pos -= c;
  }
}

// The other dealing: the problems' tile sequences one after the other, cut into 8 contiguous runs,
// one per XCD. An XCD then works on one or two problems only and fetches their operands into its
// L2 once, where the dealing above makes every XCD fetch a part of every problem's operands. For
// launches whose tiles all cost the same (the plain product: one K length).
__device__ __forceinline__ void anc_seq_tile(const NsGemmMulti &pm, int bid, int grid, int &g, int &L) {
  int pos = xcd_remap(bid, grid);
  g = 0;
  while (g + 1 < pm.n && pos >= pm.tiles[g]) { pos -= pm.tiles[g]; ++g; }
  L = pos;
}

// 256x256-tile kernel (ns_gemm_big.hip): same products, same accumulation order and
// therefore the same bits as the 128x128 kernel; used when M and N are multiples of 256.
int anc_ns_gemm_big(int epi, const NsGemm &p, int64_t E, hipStream_t s);
// The same for n <= kMaxGroups problems in one launch (ps[k] with batch size Es[k]).
// `upd` (may be null) carries the scalars of the fused weight update for problems whose `upd` is set.
int anc_ns_gemm_big_multi(int epi, const NsGemm *ps, const int64_t *Es, int n, hipStream_t s,
                          const NsUpdate *upd = nullptr);
// Bare fp32 products C[e] = A[e] B[e] on the same K loop (ns_gemm_big.hip); a_transposed: A is
// given as (K, M) row-major with row pitch ldA (and strideA between matrices), C = A^T B.
int anc_ns_gemm_big_plain(const NsGemm *ps, const int64_t *Es, int n, hipStream_t s, bool a_transposed = false);
