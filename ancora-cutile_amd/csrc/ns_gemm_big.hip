// Tiled bf16 matrix-core GEMM of the Newton-Schulz chain for gfx950 (the three products
// A = X X^T, B = b A + c A A, X = a X + B X with their fused epilogues; see ns.hip for the
// arithmetic), for shapes that are multiples of 256.
//
// Tile. A 128x128 tile moves 64 FLOP per byte staged, which at the matrix-core rate asks more
// of the per-XCD L2 than it delivers. Every wavefront here owns 128x64 outputs: 8 accumulator
// blocks of 32x32 (128 accumulator registers per lane), 6 operand fragments per 8 MFMAs.
//   symmetric products (A, B): 256x256x32 tile, 8 wavefronts (2 x 4), four 32 KiB LDS stages,
//     128 FLOP per byte staged, one workgroup per CU;
//   X = a X + B X: 128x256x32 tile, 4 wavefronts (1 x 4), three 24 KiB stages, two workgroups
//     per CU. Its epilogue moves 8 bytes of HBM traffic per element (the bf16 pair of the
//     iterate read and written) and runs at the HBM rate.
//
// Data path. Operand tiles go from HBM/L2 straight into LDS with global_load_lds_dwordx4 (no
// register staging): one instruction moves 1 KiB, a lane writes 16 bytes at lds_base + 16*lane.
// "NT" operand tiles ([row][k], TK*2-byte rows, no padding) avoid bank conflicts by an XOR
// swizzle of the 16-byte chunk index with row bits (bits 1..3 for 128-byte rows, bits 2..3 for
// 64-byte rows), applied when choosing which global chunk a lane fetches and undone when a
// fragment is read: 16 consecutive rows then cover all 64 banks once. The B operand of
// X = a X + B X is the iterate itself, (k, n) row-major: its tile is [k][256 columns], fetched
// as whole 512-byte rows, and its fragments come from transposing LDS reads
// (ds_read_b64_tr_b16), so no transposed copy of the iterate exists anywhere.
// Operands in panel layout (NsGemm::f_panel, x_panel) land in the same LDS positions; only the
// global addresses differ: an [row][k] tile is one contiguous block (rows 64 bytes apart, the
// next K tile one panel further), a [k][n] tile one 2 KiB block per 32 columns.
//
// Stage ring. Tile k of the K loop lives in stage k % NS, each stage a __shared__ array of its
// own. The DMA instructions of tile k+NS-1 go out between the MFMAs of tile k's first k-step;
// before the last k-step of tile k a wavefront waits (s_waitcnt vmcnt) only for its own DMA of
// tile k+1, then the workgroup synchronises with a barrier that orders LDS traffic only. The DMA instructions and these
// waits are inline assembly: left to itself the compiler drains every outstanding LDS-DMA
// load before an LDS read it cannot prove disjoint, and at __syncthreads().
//
// Epilogue. What an epilogue reads at the output position (fp32 A32 for B, the bf16 pair of the
// iterate for X = a X + B X, the diagonal vectors) arrives by LDS-DMA in buffers private to the
// wavefront, two 32-row slabs ahead; a slab waits with an exact vmcnt for its own fetch only.
// bf16 outputs are converted with v_cvt_pk_bf16_f32 and pass through LDS so that rows and
// mirrored rows leave as 16-byte nontemporal stores. X = a X + B X issues its MFMAs with the
// operands exchanged (transposed accumulator layout: a lane holds runs of 4 consecutive columns
// of one output row) and reads and writes LDS 8 or 16 bytes at a time.
//
// One launch covers up to 8 problems (the shape groups of an optimizer step), see NsGemmMulti.
//
// Accumulation order per output element is the same in every tile configuration and in the
// 128x128 kernel of ns.hip (terms in order, k ascending, one accumulator).
#include <type_traits>

#include "ns_common.h"

// Epilogue store: streaming, the written tile is not read again by this launch.
template <typename T> __device__ __forceinline__ void epi_st(T *p, T v) { anc_st_stream(p, v); }

namespace {

#define LDS3(p) ((__attribute__((address_space(3))) void *)(p))
#define GLB1(p) ((const __attribute__((address_space(1))) void *)(p))

// X = a X + B X reads its symmetric B operand by rows k (see AT below).
constexpr bool kBxReadsBByRows = true;

struct Frags {
  bf16x8 a[4], b[2];
};

template <int TK>
__device__ __forceinline__ void load_frags(const unsigned char *sa, const unsigned char *sb, int a_base,
                                           int b_base, int swz, Frags &f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) f.a[i] = *(const bf16x8 *)(sa + a_base + i * (32 * TK * 2) + swz);
#pragma unroll
  for (int i = 0; i < 2; ++i) f.b[i] = *(const bf16x8 *)(sb + b_base + i * (32 * TK * 2) + swz);
}

// Same fragments when the B tile is stored (k, n) row-major with 512-byte rows (the X = a X + B X
// product reads the iterate as it lies in memory): the A fragments as above, the B fragments
// through transposing LDS reads. tb[bj] is the lane's byte offset for k-step 0 of column
// block bj (it carries the swizzle); a k-step advances 16 rows, the second read 4 rows.
template <int TK>
__device__ __forceinline__ void load_frags_bt(const unsigned char *st, int a_base, int swz, const int (&tb)[2],
                                              int kk, Frags &f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) f.a[i] = *(const bf16x8 *)(st + a_base + i * (32 * TK * 2) + swz);
#pragma unroll
  for (int i = 0; i < 2; ++i)
    f.b[i] = anc_lds_tr_frag(st + tb[i] + kk * (16 * 512), st + tb[i] + kk * (16 * 512) + 4 * 512);
}

// SWAP = false: accumulator block (bi,bj) holds C[32 bi + row][32 bj + col] with col = lane%32
// and element r = row 8*(r/4) + 4*(lane/32) + r%4. SWAP = true computes the transposed block
// (operands exchanged, same products, same order of summation): row = lane%32 and element
// r = col 8*(r/4) + 4*(lane/32) + r%4, i.e. a lane holds runs of 4 consecutive columns of one
// output row, which is what a row-major epilogue wants.
template <bool SWAP>
__device__ __forceinline__ void mfma1(const Frags &f, f32x16 (&acc)[4][2], int idx) {
  const int bi = idx >> 1, bj = idx & 1;
  acc[bi][bj] = SWAP ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.b[bj], f.a[bi], acc[bi][bj], 0, 0, 0)
                     : __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[bi], f.b[bj], acc[bi][bj], 0, 0, 0);
}
template <bool SWAP>
__device__ __forceinline__ void mfma8(const Frags &f, f32x16 (&acc)[4][2]) {
#pragma unroll
  for (int bi = 0; bi < 4; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
      acc[bi][bj] = SWAP ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.b[bj], f.a[bi], acc[bi][bj], 0, 0, 0)
                         : __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[bi], f.b[bj], acc[bi][bj], 0, 0, 0);
}

// bf16 tile staging through LDS. `v` holds, for the wavefront's 32-row slab, the bf16 values of
// its 2 column blocks in accumulator layout (element r: row 8*(r/4) + 4*(lane/32) + r%4, column
// bj*32 + lane%32), packed two per dword: v[bj][i] = elements r = 2i (low half), 2i+1 (high).
// Row-major output: out[row*ld + col]; transposed: outT[col*ldT + row].
// With pstride > 0 the output is in panel layout: `out` addresses the slab's first row in its
// first 32-column panel, rows lie 32 elements apart and the second panel pstride elements further.
__device__ __forceinline__ void stage_rows(unsigned char *region, const uint32_t (&v)[2][8], int lane,
                                           uint16_t *out, int64_t ld, int64_t pstride = 0) {
  uint16_t *t = (uint16_t *)region;                 // [32][72]
#pragma unroll
  for (int bj = 0; bj < 2; ++bj)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      t[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * 72 + bj * 32 + (lane & 31)] =
          (uint16_t)((r & 1) ? (v[bj][r >> 1] >> 16) : (v[bj][r >> 1] & 0xFFFFu));
  __builtin_amdgcn_s_waitcnt(0xC07F);               // lgkmcnt(0): this wavefront's LDS writes landed
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int idx = p * 64 + lane, row = idx >> 3, c8 = (idx & 7) * 8;
    const anc_u32x4 q = *(const anc_u32x4 *)(t + row * 72 + c8);
    if (pstride > 0) epi_st((anc_u32x4 *)(out + (int64_t)(c8 >> 5) * pstride + row * 32 + (c8 & 31)), q);
    else epi_st((anc_u32x4 *)(out + (int64_t)row * ld + c8), q);
  }
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_wave_barrier();
}
// Transposed: a lane's 4 consecutive rows are 4 consecutive elements of an output row, so they
// go to LDS as one 8-byte write.
__device__ __forceinline__ void stage_cols(unsigned char *region, const uint32_t (&v)[2][8], int lane,
                                           uint16_t *outT, int64_t ldT) {
  uint16_t *t = (uint16_t *)region;                 // [64][40]
#pragma unroll
  for (int bj = 0; bj < 2; ++bj)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const anc_u32x2 w = {v[bj][2 * q], v[bj][2 * q + 1]};
      *(anc_u32x2 *)(t + (bj * 32 + (lane & 31)) * 40 + 8 * q + 4 * (lane >> 5)) = w;
    }
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int idx = p * 64 + lane, col = idx >> 2, r8 = (idx & 3) * 8;
    const anc_u32x4 q = *(const anc_u32x4 *)(t + col * 40 + r8);
    epi_st((anc_u32x4 *)(outT + (int64_t)col * ldT + r8), q);
  }
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_wave_barrier();
}

constexpr int kStageRegion = 6144;      // bytes of epilogue staging per wavefront (>= 64*40*2)

// vmcnt(n): wait until at most n vector-memory operations of this wavefront are outstanding
// (they complete in issue order), leaving lgkmcnt/expcnt alone.
template <int N> __device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// One LDS-DMA instruction: lane l of the wavefront copies 16 bytes from g (per lane) to LDS byte
// address lds_base + 16*l (lds_base wavefront-uniform, carried in M0). Written as inline
// assembly so that the stage ring's explicit vmcnt waits are the only ones: the compiler's own
// wait insertion is conservative about LDS-DMA writes that it cannot prove distinct from later
// LDS reads and would drain the ring on every tile.
__device__ __forceinline__ void dma16(const void *g, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(g)
               : "memory", "m0");
}
__device__ __forceinline__ void dma16_epi(const void *g, uint32_t lds_base) { dma16(g, lds_base); }
__device__ __forceinline__ uint32_t lds_addr(const void *p) {
  return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const void *)p);
}

// Workgroup barrier that orders LDS traffic only: this wavefront's LDS reads and writes have
// completed (lgkmcnt 0) before it arrives. Unlike __syncthreads() it carries no fence over
// global memory, so LDS-DMA loads of younger stages stay in flight across it; the caller waits
// (wait_vm<N>) for the DMA it needs before calling this.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// VAR (X = a X + B X only) selects a variant of the epilogue as its own instantiation, so that
// the extra registers and branches do not weigh on the other launches: VAR_UPDATE applies the
// weight update; VAR_PLAIN is the bare product C = A B written as fp32 (no iterate at the output
// position, no row scaling), which the weight-gradient GEMM uses; with `plain_sum` set it writes
// C = (A32 or 0) + A B and, if Yh is set, the bf16 copy of C.
// AT (X = a X + B X kernel only): the A operand is read transposed, from a (K, M) row-major matrix
// with row pitch ldA: its tile is [k][128 columns] like the B tile, fetched in 256-byte rows
// instead of 64-byte row pieces, and its fragments come from transposing LDS reads too. Used
// for the activations of a weight-gradient GEMM as they lie (C = x^T dy) and for the chain's
// own B X, whose B is symmetric (stored in full): B read by rows k is B^T read by rows m, the
// same values in the same order of summation.
enum { VAR_NONE = 0, VAR_UPDATE = 1, VAR_PLAIN = 2 };
template <int EPI, int TM, int TN, int TK, int NS, int MINBLOCKS, int VAR = VAR_NONE, bool AT = false>
__global__ void __launch_bounds__((TM / 128) * (TN / 64) * 64, MINBLOCKS) k_ns_gemm_big(NsGemmMulti pm) {
  constexpr int NWN = TN / 64, NWAVES = (TM / 128) * NWN;
  constexpr int ROWB = TK * 2;                      // bytes per LDS row
  constexpr int CPR = TK / 8;                       // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;                     // rows per DMA instruction
  constexpr int IA = TM / RPI / NWAVES, IB = TN / RPI / NWAVES;   // DMA instructions per wavefront
  constexpr int KSTEPS = TK / 16;
  constexpr int kStage = (TM + TN) * ROWB;
  constexpr int IPS = IA + IB;                      // DMA instructions per wavefront per stage
  constexpr int WPS = kStage / kStageRegion;        // wavefronts whose epilogue staging fits in a stage
  static_assert(NS >= 2 && NS <= 4 && (NS - 2) * IPS < 64, "stage ring");
  static_assert(WPS * NS >= NWAVES, "epilogue staging must fit in the stages");
  static_assert(TM % (RPI * NWAVES) == 0 && TN % (RPI * NWAVES) == 0, "DMA split");
  // NS stages, each its own __shared__ array (distinct objects for the compiler's alias analysis)
  __shared__ __attribute__((aligned(1024))) unsigned char stage0[kStage];
  __shared__ __attribute__((aligned(1024))) unsigned char stage1[kStage];
  __shared__ __attribute__((aligned(1024))) unsigned char stage2[NS > 2 ? kStage : 16];
  __shared__ __attribute__((aligned(1024))) unsigned char stage3[NS > 3 ? kStage : 16];
  auto st = [&](int i) -> unsigned char * {
    return i == 0 ? stage0 : i == 1 ? stage1 : i == 2 ? stage2 : stage3;
  };
  // B = b A + c A A: per-wavefront copy of the dA entries of its 128 rows and 64 columns;
  // X = a X + B X: of the dB entries of its 128 rows
  __shared__ __attribute__((aligned(1024))) unsigned char aux[EPI != EPI_GRAM ? NWAVES * 1024 : 16];

  int gsel, L;
  constexpr bool PLAINV = (VAR == VAR_PLAIN);
  if (PLAINV && pm.seq) anc_seq_tile(pm, (int)blockIdx.x, (int)gridDim.x, gsel, L);
  else anc_group_tile(pm, (int)blockIdx.x, (int)gridDim.x, gsel, L);
  const NsGemm &p = pm.g[gsel];
  // Symmetric outputs: only tiles that reach the diagonal or lie below it. Row tm of TM-row
  // tiles has tm/R + 1 of them (R = TN/TM); a tile entirely below the diagonal is mirrored.
  constexpr int R = TN / TM;
  static_assert(TN % TM == 0, "tile ratio");
  int tiles_per;
  if (p.lower) {
    const int q = p.tiles_m / R, r = p.tiles_m % R;          // sum over tm of (tm/R + 1)
    tiles_per = R * q * (q + 1) / 2 + r * (q + 1);
  } else {
    tiles_per = p.tiles_m * p.tiles_n;
  }
  const int e = L / tiles_per;
  const int t = L % tiles_per;
  int tm, tn;
  if (p.lower) {
    tm = 0;
    int left = t;
    while (left >= tm / R + 1) { left -= tm / R + 1; ++tm; }
    tn = left;
  } else if (p.blk_r > 0) {
    const int per = p.blk_r * p.blk_c, b = t / per, i = t % per, across = p.tiles_n / p.blk_c;
    tm = (b / across) * p.blk_r + i / p.blk_c;
    tn = (b % across) * p.blk_c + i % p.blk_c;
  } else {
    tm = t / p.tiles_n;
    tn = t % p.tiles_n;
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / NWN, wn = wave % NWN;
  const int K = p.K, nk = K / TK, total = anc_ns_terms(p, e) * nk;

  // ---- DMA addressing: this wavefront moves IA*RPI rows of the A tile and IB*RPI rows of the B
  //      tile, RPI rows per instruction; lane -> (row lane/CPR, physical chunk lane%CPR). The
  //      global address is a wavefront-uniform base plus a per-lane byte offset that carries
  //      the swizzle: 128-byte rows use chunk ^ ((row>>1)&7), which alternates with the parity
  //      of the instruction index (RPI = 8); 64-byte rows use chunk ^ ((row>>2)&3), the same
  //      for every instruction (RPI = 16).
  // Panel layout (see NsGemm): rows of a tile lie 64 bytes apart, consecutive K tiles one panel
  // (rows_of_the_matrix * 64 bytes) apart; a (k, n) tile is one 2 KiB block per 32 columns.
  const int ldA = p.ldA > 0 ? p.ldA : K;
  static_assert(TK == 32, "a K tile is one 32-column panel");
  const bool a_pan = !PLAINV && (EPI == EPI_GRAM ? p.x_panel != 0 : p.f_panel != 0);
  const bool b_pan = !PLAINV && (EPI == EPI_BMAT ? p.f_panel != 0 : p.x_panel != 0);
  const int64_t panel = (int64_t)p.M * 64;          // bytes per panel (every matrix of the chain has M rows)
  const int rpA = a_pan ? 64 : ldA * 2;             // bytes between consecutive rows of the A operand
  const int rpB = b_pan ? 64 : K * 2;               // the same for an "NT" B operand
  const int lrow = lane / CPR, pchunk = lane % CPR;
  const int key0 = (TK == 64) ? (lrow >> 1) : ((lrow >> 2) & 3);
  const uint32_t voff0 = (uint32_t)(lrow * rpA + ((pchunk ^ key0) * 16));
  const uint32_t voff1 = (uint32_t)(lrow * rpA + ((pchunk ^ key0 ^ (TK == 64 ? 4 : 0)) * 16));
  const uint32_t voffN0 = (uint32_t)(lrow * rpB + ((pchunk ^ key0) * 16));
  const uint32_t voffN1 = (uint32_t)(lrow * rpB + ((pchunk ^ key0 ^ (TK == 64 ? 4 : 0)) * 16));
  // (k, m) A tile (AT): TK rows of TM*2 = 256 bytes, four rows per DMA instruction; lane -> (row
  // lane/16, physical chunk lane%16), chunk index XORed with 4*(row&3) as for the B tile.
  static_assert(!AT || (TM == 128 && IA * NWAVES * 4 == TK), "(k,m) tile layout");
  const int catl = (lane & 15) ^ ((lane >> 4) << 2);          // logical 16-byte chunk of the (k, m) row
  const uint32_t voffAT = a_pan ? (uint32_t)((lane >> 4) * 64 + (int64_t)(catl >> 2) * panel + (catl & 3) * 16)
                                : (uint32_t)((lane >> 4) * ldA * 2 + catl * 16);
  const int64_t ubaseA = AT ? (a_pan ? (int64_t)e * p.strideA * 2 + (int64_t)(tm * (TM / 32)) * panel + (int64_t)(wave * IA * 4) * 64
                                     : ((int64_t)e * p.strideA + (int64_t)tm * TM + (int64_t)(wave * IA * 4) * ldA) * 2)
                            : (int64_t)e * p.strideA * 2 + (int64_t)(tm * TM + wave * (IA * RPI)) * rpA;   // bytes
  const int64_t ubaseB = (int64_t)e * p.strideB * 2 + (int64_t)(tn * TN + wave * (IB * RPI)) * rpB;
  // (k, n) B tile: TK rows of TN*2 = 512 bytes, two rows per DMA instruction; lane -> (row
  // lane/32, physical chunk lane%32); the chunk index is XORed with 4*(row&3), so that the 4
  // rows a transposing read touches per 32 lanes fall into 4 different 64-byte bank windows.
  // row&3 = 2*(instruction parity) + lane/32.
  constexpr bool BT = (EPI == EPI_BX);
  static_assert(!BT || (TN == 256 && IB % 2 == 0 && IB * NWAVES * 2 == TK), "(k,n) tile layout");
  const int ldn = p.N;
  const int cb0 = (lane & 31) ^ ((lane >> 5) << 2), cb1 = (lane & 31) ^ ((2 + (lane >> 5)) << 2);
  const uint32_t voffB0 = b_pan ? (uint32_t)((lane >> 5) * 64 + (int64_t)(cb0 >> 2) * panel + (cb0 & 3) * 16)
                                : (uint32_t)((lane >> 5) * ldn * 2 + cb0 * 16);
  const uint32_t voffB1 = b_pan ? (uint32_t)((lane >> 5) * 64 + (int64_t)(cb1 >> 2) * panel + (cb1 & 3) * 16)
                                : (uint32_t)((lane >> 5) * ldn * 2 + cb1 * 16);
  const int64_t ubaseBT = b_pan ? (int64_t)e * p.strideB * 2 + (int64_t)(tn * (TN / 32)) * panel + (int64_t)(wave * IB * 2) * 64
                                : ((int64_t)e * p.strideB + (int64_t)tn * TN + (int64_t)(wave * IB * 2) * ldn) * 2;

  // Operand pointers of the three terms are fetched from the argument block once, here: a
  // scalar load inside the K loop would have to be waited for with lgkmcnt(0), which also
  // waits for the LDS fragment reads in flight. K tiles are issued strictly in order, so the
  // running pointers just advance.
  const char *Abase[3], *Bbase[3];
#pragma unroll
  for (int t3 = 0; t3 < 3; ++t3) {
    Abase[t3] = (const char *)p.A[t3] + ubaseA;
    Bbase[t3] = (const char *)p.B[t3] + (BT ? ubaseBT : ubaseB);
  }
  // bytes from one K tile to the next, and from one DMA instruction of a tile to the next
  const int64_t advB = BT ? (b_pan ? (int64_t)TK * 64 : (int64_t)TK * ldn * 2) : (b_pan ? panel : (int64_t)ROWB);
  const int64_t advA = AT ? (a_pan ? (int64_t)TK * 64 : (int64_t)TK * ldA * 2) : (a_pan ? panel : (int64_t)ROWB);
  const int64_t roA = AT ? (a_pan ? (int64_t)4 * 64 : (int64_t)4 * ldA * 2) : (int64_t)RPI * rpA;
  const int64_t roB = BT ? (b_pan ? (int64_t)2 * 64 : (int64_t)2 * ldn * 2) : (int64_t)RPI * rpB;
  const char *curA = Abase[0], *curB = Bbase[0];
  int is_kt = 0, is_term = 0;
  // DMA instruction i of a stage (0 .. IPS-1: the A tile's IA, then the B tile's IB)
  auto issue_piece = [&](int i, unsigned char *stage) {
    if (i < IA) {
      const uint32_t vo = AT ? voffAT : ((i & 1) ? voff1 : voff0);
      dma16(curA + i * roA + vo, lds_addr(stage + (wave * IA + i) * 1024));
    } else {
      const int j = i - IA;
      const uint32_t vo = BT ? ((j & 1) ? voffB1 : voffB0) : ((j & 1) ? voffN1 : voffN0);
      dma16(curB + j * roB + vo, lds_addr(stage + TM * ROWB + (wave * IB + j) * 1024));
    }
  };
  auto issue_advance = [&]() {
    curA += advA;
    curB += advB;
    if (++is_kt == nk) {
      is_kt = 0;
      ++is_term;
      curA = is_term == 1 ? Abase[1] : Abase[2];
      curB = is_term == 1 ? Bbase[1] : Bbase[2];
    }
  };
  auto issue = [&](unsigned char *stage) {
#pragma unroll
    for (int i = 0; i < IPS; ++i) issue_piece(i, stage);
    issue_advance();
  };

  // ---- fragment addressing
  const int a_base = (wm * 128 + (lane & 31)) * ROWB;
  const int b_base = TM * ROWB + (wn * 64 + (lane & 31)) * ROWB;
  int swz[KSTEPS];
#pragma unroll
  for (int kk = 0; kk < KSTEPS; ++kk)
    swz[kk] = ((kk * 2 + (lane >> 5)) ^ (TK == 64 ? ((lane >> 1) & 7) : ((lane >> 2) & 3))) * 16;

  int tb[2] = {0, 0};
  if (BT) {
    const int s16 = lane & 15, g16 = lane >> 4;
#pragma unroll
    for (int bj = 0; bj < 2; ++bj) {
      const int chunk = wn * 8 + bj * 4 + 2 * (g16 & 1) + ((s16 & 3) >> 1);
      tb[bj] = TM * ROWB + (8 * (g16 >> 1) + (s16 >> 2)) * 512 + ((chunk ^ ((s16 >> 2) << 2)) * 16) + (s16 & 1) * 8;
    }
  }
  int ta[4] = {0, 0, 0, 0};
  if (AT) {
    const int s16 = lane & 15, g16 = lane >> 4;
#pragma unroll
    for (int bi = 0; bi < 4; ++bi) {
      const int chunk = bi * 4 + 2 * (g16 & 1) + ((s16 & 3) >> 1);
      ta[bi] = (8 * (g16 >> 1) + (s16 >> 2)) * 256 + ((chunk ^ ((s16 >> 2) << 2)) * 16) + (s16 & 1) * 8;
    }
  }
  auto frags = [&](const unsigned char *stg, int kk, Frags &f) {
    if (AT) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        f.a[i] = anc_lds_tr_frag(stg + ta[i] + kk * (16 * 256), stg + ta[i] + kk * (16 * 256) + 4 * 256);
#pragma unroll
      for (int i = 0; i < 2; ++i)
        f.b[i] = anc_lds_tr_frag(stg + tb[i] + kk * (16 * 512), stg + tb[i] + kk * (16 * 512) + 4 * 512);
    } else if (BT) load_frags_bt<TK>(stg, a_base, swz[kk], tb, kk, f);
    else load_frags<TK>(stg, stg, a_base, b_base, swz[kk], f);
  };

  f32x16 acc[4][2];
#pragma unroll
  for (int bi = 0; bi < 4; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bi][bj][r] = 0.0f;

  // Stage ring. Tile k lives in stage k % NS. The DMA of tile k+NS-1 is started at the top of
  // tile k, into the stage that tile k-1 was read from (every wavefront left it before the
  // barrier inside tile k-1). Before the last k-step of tile k each wavefront waits until its
  // own DMA of tile k+1 has landed (NS-2 younger tiles may still be in flight), all
  // wavefronts synchronise, and the first fragments of tile k+1 load under the last MFMAs.
  Frags f[2];
#pragma unroll
  for (int s0 = 0; s0 < NS - 1; ++s0)
    if (s0 < total) issue(st(s0));
  if (total >= NS - 1) wait_vm<(NS - 2) * IPS>(); else wait_vm<0>();
  lds_barrier();
  frags(stage0, 0, f[0]);

  // f[kk&1] holds k-step kk (KSTEPS is even, so every tile starts on f[0] and ends on f[1]).
  // `steady` (a std::true_type): the caller knows that this tile refills the ring and has a
  // successor, so the body carries no branch.
  auto body = [&](auto steady, int step, unsigned char *cur, unsigned char *nxt, unsigned char *fill) {
    constexpr bool kSteady = decltype(steady)::value;
    const bool more = kSteady || step + 1 < total;
    const bool refill = kSteady || step + NS - 1 < total;
    if (KSTEPS == 2) {
      // The stage's DMA instructions go out between the MFMAs of the first k-step, one every
      // 8/IPS matrix instructions, instead of as a burst during which the matrix pipe idles.
      frags(cur, 1, f[1]);
#pragma unroll
      for (int idx = 0; idx < 8; ++idx) {
        mfma1<BT>(f[0], acc, idx);
#pragma unroll
        for (int i = 0; i < IPS; ++i)
          if (((i + 1) * 8 + IPS - 1) / IPS - 1 == idx) {
            __builtin_amdgcn_sched_barrier(0);
            if (refill) issue_piece(i, fill);
            __builtin_amdgcn_sched_barrier(0);
          }
      }
      if (refill) issue_advance();
    } else {
      if (refill) issue(fill);
#pragma unroll
      for (int kk = 0; kk < KSTEPS - 1; ++kk) {
        frags(cur, kk + 1, f[(kk + 1) & 1]);
        mfma8<BT>(f[kk & 1], acc);
      }
    }
    if (refill) wait_vm<(NS - 2) * IPS>(); else wait_vm<0>();
    lds_barrier();
    if (more) frags(nxt, 0, f[0]);
    mfma8<BT>(f[(KSTEPS - 1) & 1], acc);
  };
  int step = 0;
  // rounds of NS tiles in which even the last tile (step + NS - 1) still refills the ring
  for (; step + 2 * NS - 2 < total; step += NS) {
#pragma unroll
    for (int s0 = 0; s0 < NS; ++s0)
      body(std::true_type{}, step + s0, st(s0), st((s0 + 1) % NS), st((s0 + NS - 1) % NS));
  }
  for (; step < total; step += NS) {
#pragma unroll
    for (int s0 = 0; s0 < NS; ++s0)
      if (step + s0 < total) body(std::false_type{}, step + s0, st(s0), st((s0 + 1) % NS), st((s0 + NS - 1) % NS));
  }
  __syncthreads();

  // ---- epilogue
  if (VAR == VAR_UPDATE && pm.ctl != nullptr && pm.ctl->skip != 0u) return;   // skipped step
  const int M = p.M, N = p.N;
  const int64_t mm = (int64_t)e * M * M, mn = (int64_t)e * M * N, mv = (int64_t)e * M;
  unsigned char *region = st(wave / WPS) + (wave % WPS) * kStageRegion;
  const int gi0w = tm * TM + wm * 128, gj0w = tn * TN + wn * 64;
  const bool mirror = (EPI != EPI_BX) && (TN * (tn + 1) <= TM * tm);
  float sc = 1.0f;
  if (EPI != EPI_BMAT && p.scale != nullptr) sc = anc_ld_const(p.scale + e);
  const float acc_scale = (EPI == EPI_GRAM) ? sc * sc : sc;
  // residual output (Fl of GRAM, Bl of BMAT): for every matrix, or only for those in the band of
  // the second conditioning gate (uniform over the workgroup: a function of the matrix)
  const bool write_lo = (EPI == EPI_GRAM ? p.Fl != nullptr : EPI == EPI_BMAT ? p.Bl != nullptr : false) &&
                        (p.lo_gated == 0 || anc_ns_wide(p, e));

  // X = a X + B X reads the iterate at the output position (the bf16 pair Xh, Xl). A 32x64 slab
  // of each is 32 rows of 128 bytes: 4 DMA instructions (8 rows each, lane -> row lane/8, chunk
  // lane%8) put it into a buffer private to the wavefront, two slabs ahead of the arithmetic, so
  // that full cache lines are requested and the latency runs under the previous slabs. The
  // 16-byte chunk index is XORed with (row&7) ^ ((row>>3)&1) (see the epilogue). The same
  // buffer stages the slab's outputs.
  constexpr int kInBuf = 8192, kBufPerStage = kStage / kInBuf;
  static_assert(EPI != EPI_BMAT || kBufPerStage * NS >= 2 * NWAVES, "epilogue buffers");
  static_assert(EPI != EPI_BX || (kBufPerStage * NS >= 2 * NWAVES && kInBuf >= kStageRegion), "epilogue buffers");
  auto inbuf = [&](int bi) -> unsigned char * {
    const int q = wave * 2 + (bi & 1);
    return st(q / kBufPerStage) + (q % kBufPerStage) * kInBuf;
  };
  // (panel layout: the slab is two 2 KiB blocks, rows 64 bytes apart)
  const bool x_pan = !PLAINV && p.x_panel != 0;
  const int ci0 = (lane & 7) ^ (lane >> 3), ci1 = ci0 ^ 1;
  const uint32_t vo_in0 = x_pan ? (uint32_t)((lane >> 3) * 64 + (int64_t)(ci0 >> 2) * panel + (ci0 & 3) * 16)
                                : (uint32_t)((lane >> 3) * N * 2 + ci0 * 16);
  const uint32_t vo_in1 = x_pan ? (uint32_t)((lane >> 3) * 64 + (int64_t)(ci1 >> 2) * panel + (ci1 & 3) * 16)
                                : (uint32_t)((lane >> 3) * N * 2 + ci1 * 16);
  const int64_t in_row = x_pan ? 64 : (int64_t)N * 2;       // bytes between consecutive rows of the slab
  // 8-bit low halves (NsGemm::l8_in, l8_out; uniform over the workgroup: a function of the
  // matrix): a 32x64 slab of bytes is 32 rows of two (M, 32)-byte panels, 1 KiB contiguous each: 2
  // DMA instructions instead of 4, in the buffer [panel][row][32 bytes].
  // (readfirstlane: the flags live in scalar registers, so the branches on them are scalar branches)
  const bool in8 = EPI == EPI_BX && !PLAINV && __builtin_amdgcn_readfirstlane((int)anc_ns_low8(p, e, p.l8_in)) != 0;
  const bool out8 = EPI == EPI_BX && !PLAINV && __builtin_amdgcn_readfirstlane((int)anc_ns_low8(p, e, p.l8_out)) != 0;
  // In the buffer the two 16-byte halves of a row's 32 bytes are swapped for rows with bit 3 set:
  // LDS chunk l holds row l/2, half (l%2) ^ ((l/16)%2), which halves the bank conflicts of the
  // 4-byte accesses below (rows 8 apart would otherwise meet in one bank four at a time).
  const int l8_src = (lane >> 1) * 32 + (((lane & 1) ^ ((lane >> 4) & 1)) * 16);
  auto fetch_in = [&](int bi) {
    const int64_t ub = x_pan ? mn * 2 + (int64_t)(gj0w / 32) * panel + (int64_t)(gi0w + bi * 32) * 64
                             : (mn + (int64_t)(gi0w + bi * 32) * N + gj0w) * 2;
    unsigned char *b = inbuf(bi);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t ro = (int64_t)(8 * j) * in_row;
      const uint32_t vo = (j & 1) ? vo_in1 : vo_in0;
      dma16_epi((const char *)p.Xh + ub + ro + vo, lds_addr(b + j * 1024));
      if (!in8) dma16_epi((const char *)p.Xl + ub + ro + vo, lds_addr(b + 4096 + j * 1024));
    }
    if (in8) {
#pragma unroll
      for (int j = 0; j < 2; ++j)
        dma16_epi((const char *)p.Xl + mn * 2 + ((int64_t)(gj0w / 32 + j) * M + gi0w + bi * 32) * 32 + l8_src,
                  lds_addr(b + 4096 + j * 1024));
    }
  };
  // B = b A + c A A reads A32 at the output position the same way: a 32x64 fp32 slab is 32 rows
  // of 256 bytes, 8 DMA instructions (4 rows each, lane -> row lane/16, chunk lane%16), chunk
  // index XORed with 8*((row>>2)&1).
  const uint32_t vo_a0 = (uint32_t)((lane >> 4) * M * 4 + ((lane & 15) * 16));
  const uint32_t vo_a1 = (uint32_t)((lane >> 4) * M * 4 + (((lane & 15) ^ 8) * 16));
  auto fetch_a32 = [&](int bi) {
    const int64_t ub = (mm + (int64_t)(gi0w + bi * 32) * M + gj0w) * 4;
    unsigned char *b = inbuf(bi);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      dma16_epi((const char *)p.A32 + ub + (int64_t)(4 * j) * M * 4 + ((j & 1) ? vo_a1 : vo_a0), lds_addr(b + j * 1024));
  };
  // Without an fp32 copy of A (see NsGemm::a32_gated) B takes the off-diagonal entries of A from
  // Fh: in panel layout a 32x64 slab is 32 rows of two panels, 2 KiB contiguous each, 4 DMA
  // instructions (16 rows of one panel each); in the buffer [panel][row][32 columns].
  const bool has_a32 = EPI != EPI_BX && anc_ns_has_a32(p, e);
  auto fetch_fh = [&](int bi) {
    unsigned char *b = inbuf(bi);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t el = mm + ((int64_t)(gj0w / 32 + (j >> 1)) * M + gi0w + bi * 32 + (j & 1) * 16) * 32;
      dma16_epi((const char *)(p.Fh + el) + lane * 16, lds_addr(b + j * 1024));
    }
  };
  auto fetch_a = [&](int bi) { if (has_a32) fetch_a32(bi); else fetch_fh(bi); };
  int in_lane[2] = {0, 0};
  unsigned char *aux_w = aux + (EPI != EPI_GRAM ? wave * 1024 : 0);
  if (EPI == EPI_BMAT) {
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
      in_lane[bj] = 4 * (lane >> 5) * 256 + (((bj * 8 + ((lane & 31) >> 2)) ^ ((lane >> 5) << 3)) * 16) + (lane & 3) * 4;
    // dA of the wavefront's rows (lanes 0..31) and columns (lanes 32..47, repeated by 48..63)
    const float *dsrc = (lane < 32) ? p.dA + mv + gi0w + lane * 4 : p.dA + mv + gj0w + (lane & 15) * 4;
    dma16(dsrc, lds_addr(aux_w));
    fetch_a(0);
    fetch_a(1);
  }
  unsigned char *dvec_lds = aux_w;
  if (EPI == EPI_BX && !PLAINV) {
    asm volatile("" : "+v"(sc));      // the scale has arrived before the first DMA is issued
    // dB of the tile's 128 rows, one private copy per wavefront (lanes 32..63 repeat lanes 0..31),
    // fetched first: any ordinary load issued after the slab fetches would, completing in
    // order, wait for them.
    dma16((const char *)(p.dB + mv + gi0w) + (lane & 31) * 16, lds_addr(dvec_lds));
    fetch_in(0);
    fetch_in(1);
  }
  if (EPI == EPI_BX) {
    // Transposed accumulator layout (see mfma8): lane l holds row l%32 of the slab and, per
    // column block bj and q = 0..3, the 4 consecutive columns bj*32 + 8q + 4*(l/32) .. +3.
    // Inputs (the bf16 pair) are 8-byte LDS reads, outputs 8-byte (pair) or 16-byte (fp32
    // result) LDS writes into the slab's own buffer, which then leaves as whole rows.
    // Pair layout in the buffer: [32 rows][8 chunks of 16 B], chunk index XORed with
    // (row&7) ^ ((row>>3)&1): the 32 rows a read touches spread over all banks.
    const int rr = lane & 31, hh = lane >> 5;
    const int key = (rr & 7) ^ ((rr >> 3) & 1);
    const bool fp32_out = p.X32 != nullptr;
    // Fused weight update (last step): the slab is the Newton-Schulz result O of a 32x64 (or,
    // for a tall weight whose chain ran on its transpose, 64x32) block of the weight W; the
    // epilogue reads that block of the fp32 master, subtracts lr*O, writes it back together with
    // its bf16 copy. The master block is requested (8 x 16 bytes per lane) before the wait for
    // the slab's DMA, so that its latency runs under the wait and the arithmetic.
    constexpr bool fused = (VAR == VAR_UPDATE);
    constexpr bool plain = PLAINV;
    float *W32 = nullptr;
    uint16_t *W16 = nullptr;
    float wlr = 0.0f;
    uint32_t wseed = 0;
    int wN = 0;
    bool wtr = false;
    if (fused) {
      const anc_muon_desc_t &d = p.upd[e];
      W32 = (float *)d.p32;
      W16 = (uint16_t *)d.p16;
      wN = d.N;
      wtr = d.transpose != 0;
      wlr = pm.lr[d.scale_idx & (ANC_MUON_MAX_SCALES - 1)];
      wseed = pm.seed_base + d.seed + ((pm.sr & ANC_SR_STEP_SEED) ? ANC_SR_SEED_STRIDE * pm.ctl->t : 0u);
    }
    // element offset in W of the 4 values lane-piece pz handles
    auto w_off = [&](int gi0, int pz) -> int64_t {
      const int idx = pz * 64 + lane;
      if (!wtr) return (int64_t)(gi0 + (idx >> 4)) * wN + gj0w + (idx & 15) * 4;
      return (int64_t)(gj0w + (idx >> 3)) * wN + gi0 + (idx & 7) * 4;
    };
#pragma unroll
    for (int bi = 0; bi < 4; ++bi) {
      const int gi0 = gi0w + bi * 32;
      anc_f32x4 pv[8];
      if (fused) {
#pragma unroll
        for (int pz = 0; pz < 8; ++pz) pv[pz] = anc_ld_stream((const anc_f32x4 *)(W32 + w_off(gi0, pz)));
      }
      // Plain product with an addend (C = A32 + A B, in place when A32 == X32): same early request
      const bool plain_add = plain && p.plain_sum && p.A32 != nullptr;
      if (plain_add) {
#pragma unroll
        for (int pz = 0; pz < 8; ++pz) {
          const int idx = pz * 64 + lane;
          pv[pz] = anc_ld_stream((const anc_f32x4 *)(p.A32 + mn + (int64_t)(gi0 + (idx >> 4)) * N + gj0w + (idx & 15) * 4));
        }
      }
      // Wait for this slab's DMA only. Vector memory operations complete in issue order; after
      // the fetch of slab bi this wavefront issued the 8 row stores of slab bi-1 and the fetch
      // of slab bi+1 (8 DMA); in the fused update the stores of a slab are 8 (master) + 8 (bf16
      // copy, if there is one) and the 8 master loads of slab bi are younger too.
      // A slab's fetch is 8 DMA instructions, 6 with an 8-bit low half; its pair stores 8 or 6.
      if (plain) {
        // no inputs: nothing to wait for
      } else if (!fused) {
        if (bi == 0) { if (in8) wait_vm<6>(); else wait_vm<8>(); }
        else if (bi == 3) { if (out8) wait_vm<6>(); else wait_vm<8>(); }
        else if (in8 && out8) wait_vm<12>();
        else if (in8 || out8) wait_vm<14>();
        else wait_vm<16>();
      } else {
        // (the fused launch writes no iterate: out8 does not occur)
        if (W16 != nullptr) {
          if (bi == 0) { if (in8) wait_vm<14>(); else wait_vm<16>(); }
          else if (bi == 3) wait_vm<24>();
          else if (in8) wait_vm<30>();
          else wait_vm<32>();
        } else {
          if (bi == 0) { if (in8) wait_vm<14>(); else wait_vm<16>(); }
          else if (bi == 3) wait_vm<16>();
          else if (in8) wait_vm<22>();
          else wait_vm<24>();
        }
      }
      unsigned char *b = inbuf(bi);
      float y[2][16];
      if (plain) {
#pragma unroll
        for (int bj = 0; bj < 2; ++bj)
#pragma unroll
          for (int r = 0; r < 16; ++r) y[bj][r] = acc[bi][bj][r];
      } else {
        const float dr = *(const float *)(dvec_lds + (bi * 32 + rr) * 4);
        const float cf = p.ca + dr;
        if (!in8) {
          anc_u32x2 xh[2][4], xl[2][4];
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int off = rr * 128 + (((bj * 4 + q) ^ key) * 16) + hh * 8;
              xh[bj][q] = *(const anc_u32x2 *)(b + off);
              xl[bj][q] = *(const anc_u32x2 *)(b + 4096 + off);
            }
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const uint32_t wh = (r & 2) ? xh[bj][r >> 2].y : xh[bj][r >> 2].x;
              const uint32_t wl = (r & 2) ? xl[bj][r >> 2].y : xl[bj][r >> 2].x;
              const float x = ((r & 1) ? __uint_as_float(wh & 0xFFFF0000u) : __uint_as_float(wh << 16)) +
                              ((r & 1) ? __uint_as_float(wl & 0xFFFF0000u) : __uint_as_float(wl << 16));
              y[bj][r] = x;
            }
        } else {
          // 8-bit low halves: w8[bj][q] holds the 4 bytes of columns bj*32 + 8q + 4hh .. +3 of row
          // rr, which with the high half give x directly
          anc_u32x2 xh[2][4];
          uint32_t w8[2][4];
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              xh[bj][q] = *(const anc_u32x2 *)(b + rr * 128 + (((bj * 4 + q) ^ key) * 16) + hh * 8);
              w8[bj][q] = *(const uint32_t *)(b + 4096 + bj * 1024 + rr * 32 + (((q >> 1) ^ ((rr >> 3) & 1)) * 16) + (q & 1) * 8 + hh * 4);
            }
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const uint32_t wh = (r & 2) ? xh[bj][r >> 2].y : xh[bj][r >> 2].x;
              const uint32_t htop = (r & 1) ? (wh & 0xFFFF0000u) : (wh << 16);
              y[bj][r] = anc_low8_decode(htop, (int)(w8[bj][r >> 2] << (24 - 8 * (r & 3))) >> 24);
            }
        }
        // y = (a + dB) x + B X; only the first iteration carries the input's scale (times 1.0f is the
        // identity, so leaving the factors out elsewhere changes no bit; the fused instantiation,
        // which has no register to spare for a second version, keeps them)
        if (fused || p.scale != nullptr) {
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int r = 0; r < 16; ++r) y[bj][r] = cf * (y[bj][r] * sc) + acc[bi][bj][r] * acc_scale;
        } else {
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int r = 0; r < 16; ++r) y[bj][r] = cf * y[bj][r] + acc[bi][bj][r];
        }
      }
      if (fp32_out || fused || plain) {
        // fp32 result: [32 rows][16 chunks of 16 B], chunk XOR (row & 15)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const anc_f32x4 v4 = {y[bj][4 * q], y[bj][4 * q + 1], y[bj][4 * q + 2], y[bj][4 * q + 3]};
            *(anc_f32x4 *)(b + rr * 256 + (((bj * 8 + 2 * q + hh) ^ (rr & 15)) * 16)) = v4;
          }
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_wave_barrier();
        if (plain && p.plain_sum) {
          // C = (A32 or 0) + A B, and its bf16 copy (round to nearest even) if Yh is set
#pragma unroll
          for (int pz = 0; pz < 8; ++pz) {
            const int idx = pz * 64 + lane, row = idx >> 4, c = idx & 15;
            const anc_f32x4 v4 = *(const anc_f32x4 *)(b + row * 256 + ((c ^ (row & 15)) * 16));
            const anc_f32x4 a4 = plain_add ? pv[pz] : anc_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            const anc_f32x4 o4 = {a4.x + v4.x, a4.y + v4.y, a4.z + v4.z, a4.w + v4.w};
            const int64_t off = mn + (int64_t)(gi0 + row) * N + gj0w + c * 4;
            epi_st((anc_f32x4 *)(p.X32 + off), o4);
            if (p.Yh != nullptr) {
              const anc_u32x2 ho = {(anc_bf16_rne_bits(o4.x) & 0xFFFFu) | (anc_bf16_rne_bits(o4.y) << 16),
                                    (anc_bf16_rne_bits(o4.z) & 0xFFFFu) | (anc_bf16_rne_bits(o4.w) << 16)};
              epi_st((anc_u32x2 *)(p.Yh + off), ho);
            }
          }
        } else if (!fused) {
#pragma unroll
          for (int pz = 0; pz < 8; ++pz) {
            const int idx = pz * 64 + lane, row = idx >> 4, c = idx & 15;
            const anc_f32x4 v4 = *(const anc_f32x4 *)(b + row * 256 + ((c ^ (row & 15)) * 16));
            epi_st((anc_f32x4 *)(p.X32 + mn + (int64_t)(gi0 + row) * N + gj0w + c * 4), v4);
          }
        } else {
#pragma unroll
          for (int pz = 0; pz < 8; ++pz) {
            const int idx = pz * 64 + lane;
            float o[4];
            if (!wtr) {
              const int row = idx >> 4, c = idx & 15;
              const anc_f32x4 v4 = *(const anc_f32x4 *)(b + row * 256 + ((c ^ (row & 15)) * 16));
              o[0] = v4.x; o[1] = v4.y; o[2] = v4.z; o[3] = v4.w;
            } else {
              // W row = column `col` of the slab, W columns = slab rows 4c .. 4c+3
              const int col = idx >> 3, c = idx & 7;
#pragma unroll
              for (int t4 = 0; t4 < 4; ++t4) {
                const int row = 4 * c + t4;
                o[t4] = *(const float *)(b + row * 256 + (((col >> 2) ^ (row & 15)) * 16) + (col & 3) * 4);
              }
            }
            const int64_t we = w_off(gi0, pz);
            float pp[4] = {pv[pz].x, pv[pz].y, pv[pz].z, pv[pz].w};
            uint32_t hb[4];
#pragma unroll
            for (int k4 = 0; k4 < 4; ++k4) {
              pp[k4] = pp[k4] - wlr * o[k4];
              const uint64_t i = (uint64_t)(we + k4);
              hb[k4] = (pm.sr & ANC_SR_ON) ? anc_bf16_sr_bits(pp[k4], (uint32_t)(i >> 6), (uint32_t)(i & 63u), wseed)
                             : anc_bf16_rne_bits(pp[k4]);
            }
            const anc_f32x4 po = {pp[0], pp[1], pp[2], pp[3]};
            epi_st((anc_f32x4 *)(W32 + we), po);
            if (W16 != nullptr) {
              const anc_u32x2 ho = {(hb[0] & 0xFFFFu) | (hb[1] << 16), (hb[2] & 0xFFFFu) | (hb[3] << 16)};
              epi_st((anc_u32x2 *)(W16 + we), ho);
            }
          }
        }
      } else {
        if (!out8) {
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              uint32_t h0, l0, h1, l1;
              anc_pk_pair(y[bj][4 * q], y[bj][4 * q + 1], h0, l0);
              anc_pk_pair(y[bj][4 * q + 2], y[bj][4 * q + 3], h1, l1);
              const anc_u32x2 wh = {h0, h1}, wl = {l0, l1};
              const int off = rr * 128 + (((bj * 4 + q) ^ key) * 16) + hh * 8;
              *(anc_u32x2 *)(b + off) = wh;
              *(anc_u32x2 *)(b + 4096 + off) = wl;
            }
        } else {
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const uint32_t h0 = anc_pk_bf16(y[bj][4 * q], y[bj][4 * q + 1]);
              const uint32_t h1 = anc_pk_bf16(y[bj][4 * q + 2], y[bj][4 * q + 3]);
              const anc_u32x2 wh = {h0, h1};
              *(anc_u32x2 *)(b + rr * 128 + (((bj * 4 + q) ^ key) * 16) + hh * 8) = wh;
              const uint32_t q0 = anc_low8_encode(y[bj][4 * q], h0 << 16);
              const uint32_t q1 = anc_low8_encode(y[bj][4 * q + 1], h0 & 0xFFFF0000u);
              const uint32_t q2 = anc_low8_encode(y[bj][4 * q + 2], h1 << 16);
              const uint32_t q3 = anc_low8_encode(y[bj][4 * q + 3], h1 & 0xFFFF0000u);
              *(uint32_t *)(b + 4096 + bj * 1024 + rr * 32 + (((q >> 1) ^ ((rr >> 3) & 1)) * 16) + (q & 1) * 8 + hh * 4) =
                  q0 | (q1 << 8) | (q2 << 16) | (q3 << 24);
            }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_wave_barrier();
        // element offset of chunk c (8 columns) of slab row `row` in the output iterate
        const bool y_pan = p.y_panel != 0;
        auto y_off = [&](int row, int c) -> int64_t {
          return y_pan ? mn + ((int64_t)(gj0w / 32 + (c >> 2)) * M + gi0 + row) * 32 + (c & 3) * 8
                       : mn + (int64_t)(gi0 + row) * N + gj0w + c * 8;
        };
#pragma unroll
        for (int pz = 0; pz < 4; ++pz) {
          const int idx = pz * 64 + lane, row = idx >> 3, c = idx & 7;
          const int off = row * 128 + ((c ^ ((row & 7) ^ ((row >> 3) & 1))) * 16);
          const anc_u32x4 qh = *(const anc_u32x4 *)(b + off);
          epi_st((anc_u32x4 *)(p.Yh + y_off(row, c)), qh);
        }
        if (!out8) {
#pragma unroll
          for (int pz = 0; pz < 4; ++pz) {
            const int idx = pz * 64 + lane, row = idx >> 3, c = idx & 7;
            const int off = row * 128 + ((c ^ ((row & 7) ^ ((row >> 3) & 1))) * 16);
            const anc_u32x4 ql = *(const anc_u32x4 *)(b + 4096 + off);
            epi_st((anc_u32x4 *)(p.Yl + y_off(row, c)), ql);
          }
        } else {
          // one byte per element: the slab's 32 rows of a panel are 1 KiB contiguous
#pragma unroll
          for (int pz = 0; pz < 2; ++pz) {
            const anc_u32x4 ql = *(const anc_u32x4 *)(b + 4096 + pz * 1024 + lane * 16);
            epi_st((anc_u32x4 *)((char *)p.Yl + mn * 2 + ((int64_t)(gj0w / 32 + pz) * M + gi0) * 32 + l8_src), ql);
          }
        }
      }
      // the buffer is free again once the staged rows have been read back
      __builtin_amdgcn_s_waitcnt(0xC07F);
      __builtin_amdgcn_wave_barrier();
      asm volatile("" ::: "memory");
      if (!plain && bi + 2 < 4) fetch_in(bi + 2);
    }
    return;
  }
#pragma unroll
  for (int bi = 0; bi < 4; ++bi) {
    const int gi0 = gi0w + bi * 32;
    // operands of the epilogue first (all loads in flight together), arithmetic after
    float in[2][16], drow[16], dcol[2];
    if (EPI == EPI_BMAT) {
      // Wait for this slab's DMA only (see the X = a X + B X branch). Stores of a slab: 4 per
      // staged bf16 block (Bh, its mirror, and the same for Bl); the conditional dB stores of
      // diagonal tiles only add to what may stay outstanding, so leaving them out is safe.
      // A slab's fetch is 8 DMA instructions (A32) or 4 (Fh).
      const int nst = 4 * ((mirror ? 2 : 1) * (write_lo ? 2 : 1));
      const int young = bi == 0 ? (has_a32 ? 8 : 4) : bi == 3 ? nst : nst + (has_a32 ? 8 : 4);
      if (young >= 24) wait_vm<24>();
      else if (young >= 20) wait_vm<20>();
      else if (young >= 16) wait_vm<16>();
      else if (young >= 12) wait_vm<12>();
      else if (young >= 8) wait_vm<8>();
      else wait_vm<4>();
      const unsigned char *b = inbuf(bi);
      if (has_a32) {
#pragma unroll
        for (int bj = 0; bj < 2; ++bj)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            in[bj][r] = *(const float *)(b + in_lane[bj] + (8 * (r >> 2) + (r & 3)) * 256);
      } else {
#pragma unroll
        for (int bj = 0; bj < 2; ++bj)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            in[bj][r] = anc_bf16_bits_to_f32(*(const uint16_t *)(b + bj * 2048 + row * 64 + (lane & 31) * 2));
          }
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const anc_f32x4 d4 = *(const anc_f32x4 *)(aux_w + (bi * 32 + 8 * q + 4 * (lane >> 5)) * 4);
        drow[4 * q] = d4.x; drow[4 * q + 1] = d4.y; drow[4 * q + 2] = d4.z; drow[4 * q + 3] = d4.w;
      }
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) dcol[bj] = *(const float *)(aux_w + 512 + (bj * 32 + (lane & 31)) * 4);
      region = const_cast<unsigned char *>(b);
    }
    float ov[2][16];          // the values that leave as bf16 (pairs)
    // Only a slab whose rows gi0 .. gi0+31 meet its columns gj0w .. gj0w+63 holds diagonal elements
    // (the same for every lane of the wavefront): every other slab runs without the per-element test.
    const bool slab_diag = gi0 + 31 >= gj0w && gi0 <= gj0w + 63;
    if (EPI == EPI_GRAM && has_a32) {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int gi = gi0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          const int gj = gj0w + bj * 32 + (lane & 31);
          p.A32[mm + (int64_t)gi * M + gj] = acc[bi][bj][r] * acc_scale;
        }
    }
    if (!slab_diag) {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (EPI == EPI_GRAM) {
            ov[bj][r] = acc[bi][bj][r] * acc_scale;
          } else {
            const float v = acc[bi][bj][r], a = in[bj][r];
            const float a2 = v + (drow[r] * a + a * dcol[bj]);   // symmetric in (i,j)
            ov[bj][r] = p.cb * a + p.cc * a2;
          }
        }
    } else {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int gi = gi0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          const int gj = gj0w + bj * 32 + (lane & 31);
          const float v = (EPI == EPI_BMAT) ? acc[bi][bj][r] : acc[bi][bj][r] * acc_scale;
          if (EPI == EPI_GRAM) {
            const bool diag = gi == gj;
            ov[bj][r] = diag ? 0.0f : v;
            if (diag) p.dA[mv + gi] = v;
          } else if (EPI == EPI_BMAT) {
            const float a = in[bj][r];
            const float di = drow[r], dj = dcol[bj];
            if (gi != gj) {
              const float a2 = v + (di * a + a * dj);   // symmetric in (i,j)
              ov[bj][r] = p.cb * a + p.cc * a2;
            } else {
              const float a2 = v + di * di;
              p.dB[mv + gi] = p.cb * di + p.cc * a2;
              ov[bj][r] = 0.0f;
            }
          }
        }
      }
    }
    uint32_t hv[2][8], lv[2][8];
    if (write_lo) {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int i = 0; i < 8; ++i) anc_pk_pair(ov[bj][2 * i], ov[bj][2 * i + 1], hv[bj][i], lv[bj][i]);
    } else {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int i = 0; i < 8; ++i) { hv[bj][i] = anc_pk_bf16(ov[bj][2 * i], ov[bj][2 * i + 1]); lv[bj][i] = 0u; }
    }
    // Where the slab (rows gi0.., columns gj0w..) and its mirror image (rows gj0w.., columns gi0..:
    // 64 rows of one 32-column panel, a contiguous 4 KiB in panel layout) go in an (M, M) matrix.
    const bool f_pan = p.f_panel != 0;
    const int64_t o_rows = f_pan ? mm + ((int64_t)(gj0w / 32) * M + gi0) * 32 : mm + (int64_t)gi0 * M + gj0w;
    const int64_t o_cols = f_pan ? mm + ((int64_t)(gi0 / 32) * M + gj0w) * 32 : mm + (int64_t)gj0w * M + gi0;
    const int64_t ps = f_pan ? (int64_t)M * 32 : 0, ldT = f_pan ? 32 : M;
    if (EPI == EPI_GRAM) {
      stage_rows(region, hv, lane, p.Fh + o_rows, M, ps);
      if (mirror) stage_cols(region, hv, lane, p.Fh + o_cols, ldT);
      if (write_lo) {
        stage_rows(region, lv, lane, p.Fl + o_rows, M, ps);
        if (mirror) stage_cols(region, lv, lane, p.Fl + o_cols, ldT);
      }
    } else if (EPI == EPI_BMAT) {
      stage_rows(region, hv, lane, p.Bh + o_rows, M, ps);
      if (mirror) stage_cols(region, hv, lane, p.Bh + o_cols, ldT);
      if (write_lo) {
        stage_rows(region, lv, lane, p.Bl + o_rows, M, ps);
        if (mirror) stage_cols(region, lv, lane, p.Bl + o_cols, ldT);
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);
      asm volatile("" ::: "memory");
      if (bi + 2 < 4) fetch_a(bi + 2);
    }
  }
}

template <int EPI>
int launch_sym(const NsGemm *ps, const int64_t *Es, int n, hipStream_t s) {
  NsGemmMulti pm{};
  pm.n = n;
  int64_t grid = 0;
  for (int k = 0; k < n; ++k) {
    ANC_REQUIRE(!ps[k].a32_gated || ps[k].f_panel, "anc_ns_gemm_big: A taken from Fh needs the panel layout");
    pm.g[k] = ps[k];
    pm.g[k].tiles_m = pm.g[k].tiles_n = ps[k].M / 256;
    const int64_t t = Es[k] * ((int64_t)pm.g[k].tiles_m * (pm.g[k].tiles_m + 1) / 2);
    ANC_REQUIRE(t > 0 && t < (1ll << 30), "anc_ns_gemm_big: grid out of range");
    pm.tiles[k] = (int)t;
    grid += t;
  }
  ANC_REQUIRE(grid < (1ll << 31), "anc_ns_gemm_big: grid out of range");
  anc_fill_segments(pm);
  hipLaunchKernelGGL((k_ns_gemm_big<EPI, 256, 256, 32, 4, 1>), dim3((unsigned)grid), dim3(512), 0, s, pm);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

}  // namespace

namespace {

// One X = a X + B X launch over the given problems, B fetched by rows k or by rows m.
int launch_bx(const NsGemm *ps, const int64_t *Es, int n, hipStream_t s, const NsUpdate *upd, bool by_rows) {
  NsGemmMulti pm{};
  pm.n = n;
  int64_t grid = 0;
  for (int k = 0; k < n; ++k) {
    pm.g[k] = ps[k];
    pm.g[k].tiles_m = ps[k].M / 128;
    pm.g[k].tiles_n = ps[k].N / 256;
    pm.g[k].lower = 0;
    ANC_REQUIRE(!(ps[k].l8_in > 0.0) || (ps[k].x_panel && ps[k].Xl != nullptr),
                "anc_ns_gemm_big: 8-bit low halves of the input need the panel layout");
    ANC_REQUIRE(!(ps[k].l8_out > 0.0) || (ps[k].y_panel && ps[k].Yl != nullptr),
                "anc_ns_gemm_big: 8-bit low halves of the output need the panel layout");
    // A matrix's tiles are walked in blocks of 4 x 2 tiles (512 rows of B, 512 columns of X) instead
    // of row by row: the 64 workgroups an XCD runs together then share 4 row blocks of B and a few
    // column blocks of X per matrix instead of all of X, and its L2 fetches X from HBM about once
    // (HBM reads of a Qwen3-0.6B launch: 4.10 GiB row by row, 3.39 in these blocks, 3.24 .. 3.37 in
    // blocks of 8 x 1 .. 8 x 4, 4.02 in 2 x 1; the launch takes the same time in every order). The
    // order does not enter a tile's arithmetic.
    {
      NsGemm &g = pm.g[k];
      const int br = g.tiles_m % 4 == 0 ? 4 : g.tiles_m % 2 == 0 ? 2 : 1;
      const int bc = g.tiles_n % 2 == 0 ? 2 : 1;
      g.blk_r = br; g.blk_c = bc;
    }
    const int64_t t = Es[k] * (int64_t)pm.g[k].tiles_m * pm.g[k].tiles_n;
    ANC_REQUIRE(t > 0 && t < (1ll << 30), "anc_ns_gemm_big: grid out of range");
    pm.tiles[k] = (int)t;
    grid += t;
  }
  ANC_REQUIRE(grid < (1ll << 31), "anc_ns_gemm_big: grid out of range");
  anc_fill_segments(pm);
  const bool fused = ps[0].upd != nullptr;
  if (fused) {
    for (int k = 0; k < ANC_MUON_MAX_SCALES; ++k) pm.lr[k] = upd->lr[k];
    pm.sr = upd->sr;
    pm.seed_base = upd->seed_base;
    pm.ctl = upd->ctl;
  }
  if (fused) {
    if (by_rows)
      hipLaunchKernelGGL((k_ns_gemm_big<EPI_BX, 128, 256, 32, 3, 2, VAR_UPDATE, true>), dim3((unsigned)grid), dim3(256), 0, s, pm);
    else
      hipLaunchKernelGGL((k_ns_gemm_big<EPI_BX, 128, 256, 32, 3, 2, VAR_UPDATE, false>), dim3((unsigned)grid), dim3(256), 0, s, pm);
  } else {
    if (by_rows)
      hipLaunchKernelGGL((k_ns_gemm_big<EPI_BX, 128, 256, 32, 3, 2, VAR_NONE, true>), dim3((unsigned)grid), dim3(256), 0, s, pm);
    else
      hipLaunchKernelGGL((k_ns_gemm_big<EPI_BX, 128, 256, 32, 3, 2, VAR_NONE, false>), dim3((unsigned)grid), dim3(256), 0, s, pm);
  }
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

}  // namespace

// Symmetric products run on 256x256 tiles (lower triangle); X = a X + B X runs on 128x256 tiles
// (the tile counts of the problems are recomputed here).
int anc_ns_gemm_big_multi(int epi, const NsGemm *ps, const int64_t *Es, int n, hipStream_t s,
                          const NsUpdate *upd) {
  ANC_REQUIRE(n >= 1 && n <= kMaxGroups, "anc_ns_gemm_big: 1..%d problems per launch", kMaxGroups);
  for (int k = 0; k < n; ++k)
    ANC_REQUIRE(ps[k].M % 256 == 0 && ps[k].N % 256 == 0 && ps[k].K % 32 == 0,
                "anc_ns_gemm_big: dims must be multiples of 256");
  if (epi == EPI_GRAM) return launch_sym<EPI_GRAM>(ps, Es, n, s);
  if (epi == EPI_BMAT) return launch_sym<EPI_BMAT>(ps, Es, n, s);
  bool any_upd = false, all_upd = true;
  for (int k = 0; k < n; ++k) { any_upd = any_upd || ps[k].upd != nullptr; all_upd = all_upd && ps[k].upd != nullptr; }
  ANC_REQUIRE(any_upd == all_upd, "anc_ns_gemm_big: the fused update applies to every problem of a launch or to none");
  ANC_REQUIRE(!any_upd || upd != nullptr, "anc_ns_gemm_big: fused update without its scalars");
  // B is symmetric and stored in full, so its tile can be fetched by rows k (256-byte rows) as
  // well as by rows m (64-byte row pieces). Measured per 5 launches: 84 x (1024, 3072) 4.12
  // against 4.27 ms, 208 x (1024, 1024) 3.37 against 3.56 ms, but 64 x (512, 512) 0.238 against
  // 0.212 ms: by rows k from M = 1024 on. The two ways read the same values except inside the
  // diagonal 256x256 tiles of a B that descends from an A = X X^T with residual terms: there
  // element (i, j) and element (j, i) add the same products in a different order and may differ
  // in the last bit. So the way of reading is a property of the problem's shape, never of what
  // it shares a call with: a call with problems of both kinds becomes two launches.
  NsGemm part[kMaxGroups];
  int64_t pe[kMaxGroups];
  for (int pass = 0; pass < 2; ++pass) {
    const bool by_rows = pass == 0;
    int m = 0;
    for (int k = 0; k < n; ++k)
      if ((kBxReadsBByRows && ps[k].M >= 1024) == by_rows) { part[m] = ps[k]; pe[m] = Es[k]; ++m; }
    if (m > 0)
      if (int rc = launch_bx(part, pe, m, s, upd, by_rows)) return rc;
  }
  return ANC_OK;
}

// Bare products C[e] = A[e] B[e] (fp32 out, p.X32), A (M, K) with row pitch p.ldA -- or, with
// a_transposed, (K, M) with row pitch p.ldA >= M (a multiple of 8) --, B (K, N) row-major, on the X = a X + B X kernel's K loop: 128x256 tiles, M % 128 == 0, N % 256 == 0,
// K % 32 == 0.
int anc_ns_gemm_big_plain(const NsGemm *ps, const int64_t *Es, int n, hipStream_t s, bool a_transposed) {
  ANC_REQUIRE(n >= 1 && n <= kMaxGroups, "anc_ns_gemm_big_plain: 1..%d problems per launch", kMaxGroups);
  NsGemmMulti pm{};
  pm.n = n;
  int64_t grid = 0;
  for (int k = 0; k < n; ++k) {
    ANC_REQUIRE(ps[k].M % 128 == 0 && ps[k].N % 256 == 0 && ps[k].K % 32 == 0 && ps[k].K >= 32,
                "anc_ns_gemm_big_plain: needs M % 128 == 0, N % 256 == 0, K % 32 == 0");
    ANC_REQUIRE(ps[k].X32 != nullptr && ps[k].nterms == 1 && ps[k].scale == nullptr && ps[k].upd == nullptr &&
                (ps[k].plain_sum || (ps[k].A32 == nullptr && ps[k].Yh == nullptr)),
                "anc_ns_gemm_big_plain: bad problem");
    pm.g[k] = ps[k];
    pm.g[k].tiles_m = ps[k].M / 128;
    pm.g[k].tiles_n = ps[k].N / 256;
    pm.g[k].lower = 0;
    const int64_t t = Es[k] * (int64_t)pm.g[k].tiles_m * pm.g[k].tiles_n;
    ANC_REQUIRE(t > 0 && t < (1ll << 30), "anc_ns_gemm_big_plain: grid out of range");
    pm.tiles[k] = (int)t;
    grid += t;
  }
  ANC_REQUIRE(grid < (1ll << 31), "anc_ns_gemm_big_plain: grid out of range");
  anc_fill_segments(pm);
  // Every XCD has an L2 of its own, so which tiles it runs decides how often an operand byte is
  // fetched from HBM. A launch that fits the GPU's 512 workgroup slots runs in one round: its
  // problems' tile sequences are dealt one after the other (anc_seq_tile), an XCD works on one or
  // two problems, and a problem's tile grid is walked along its smaller operand -- column panel by
  // column panel when A = (M, K) is the smaller one, so that a run of tiles reads all of A once
  // and only its own panels of B; row by row when B is. (One layer of Qwen3-0.6B weight
  // gradients, 480 tiles: 744 MiB of HBM reads per launch; with an eighth of every problem on
  // every XCD in row order 1800 MiB.) Larger launches measured better with an eighth of every
  // problem on every XCD (anc_group_tile), each eighth a compact block of the tile grid: the grid
  // cut 1x8, 2x4, 4x2 or 8x1, whichever needs the fewest operand bytes per block.
  pm.seq = grid <= 512 ? 1 : 0;
  for (int k = 0; k < n; ++k) {
    NsGemm &g = pm.g[k];
    if (pm.seq) {
      if (g.M <= g.N) { g.blk_r = g.tiles_m; g.blk_c = 1; }
      else { g.blk_r = 1; g.blk_c = g.tiles_n; }
      continue;
    }
    int best = 0;
    g.blk_r = g.blk_c = 0;
    for (int gx = 1; gx <= 8; gx *= 2) {
      const int gy = 8 / gx;
      if (g.tiles_m % gx != 0 || g.tiles_n % gy != 0) continue;
      const int cost = 128 * (g.tiles_m / gx) + 256 * (g.tiles_n / gy);
      if (best == 0 || cost < best) { best = cost; g.blk_r = g.tiles_m / gx; g.blk_c = g.tiles_n / gy; }
    }
  }
  if (a_transposed)
    hipLaunchKernelGGL((k_ns_gemm_big<EPI_BX, 128, 256, 32, 3, 2, VAR_PLAIN, true>), dim3((unsigned)grid), dim3(256), 0, s, pm);
  else
    hipLaunchKernelGGL((k_ns_gemm_big<EPI_BX, 128, 256, 32, 3, 2, VAR_PLAIN>), dim3((unsigned)grid), dim3(256), 0, s, pm);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

int anc_ns_gemm_big(int epi, const NsGemm &p, int64_t E, hipStream_t s) {
  return anc_ns_gemm_big_multi(epi, &p, &E, 1, s, nullptr);
}
