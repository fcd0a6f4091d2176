// Input-embedding weight gradient by deterministic sorted scatter, for gfx950.
// Replaces `_embed_dw_scatter` (ancora/kernels/fused.py:387-408; host side `build_id_groups`,
// :411-424; launched from ancora/model/resident_moe_model.py:333-334):
//     out[gid[g]] += sum over r < cnt[g] of f32(bf16 dy[srt[start[g] + r]])
// The host stable-sorts the token ids into groups (one per distinct id, rows in their original
// order). One workgroup owns one (group, 256-column chunk): a single writer per output element,
// no atomics, and the rows of a group are added one after the other in sorted order starting from
// zero, then added onto `out`: the association order of the reference's loop, so the result is
// bit-identical to a sequential fp32 evaluation and the same on every run. Eight row loads are in
// flight at a time; the additions stay in order.
#include "common.h"

namespace {

constexpr int kChunk = 256;     // columns per workgroup: 64 lanes x 4

__global__ void __launch_bounds__(64)
k_embed_dw_scatter(const int32_t *__restrict__ cnt, const int32_t *__restrict__ start,
                   const int32_t *__restrict__ gid, const int32_t *__restrict__ srt,
                   const uint16_t *__restrict__ dy, float *__restrict__ out, float *__restrict__ compact,
                   int H, int64_t M, int64_t V) {
  const int g = (int)blockIdx.x;
  const int n = cnt[g];
  if (n <= 0) return;                                   // padding group
  const int st = start[g];
  const int64_t row = gid[g];
  if (st < 0 || (int64_t)st + n > M || row < 0 || (compact == nullptr && row >= V)) return;   // malformed group: no write
  const int c0 = (int)blockIdx.y * kChunk + (int)threadIdx.x * 4;
  if (c0 >= H) return;
  float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  bool bad = false;                                     // an index outside dy: the group writes nothing
  for (int r0 = 0; r0 < n; r0 += 8) {
    anc_u32x2 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (r0 + j < n) {
        int64_t sr = srt[st + r0 + j];
        if (sr < 0 || sr >= M) { sr = 0; bad = true; }  // malformed index: stay inside dy
        v[j] = *(const anc_u32x2 *)(dy + sr * H + c0);
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (r0 + j < n) {
        acc[0] = acc[0] + __uint_as_float(v[j].x << 16);
        acc[1] = acc[1] + __uint_as_float(v[j].x & 0xFFFF0000u);
        acc[2] = acc[2] + __uint_as_float(v[j].y << 16);
        acc[3] = acc[3] + __uint_as_float(v[j].y & 0xFFFF0000u);
      }
    }
  }
  if (bad) return;
  if (compact != nullptr) {
    const anc_f32x4 o = {acc[0], acc[1], acc[2], acc[3]};
    *(anc_f32x4 *)(compact + (int64_t)g * H + c0) = o;
  } else {
    float *p = out + row * H + c0;
    const anc_f32x4 b = *(const anc_f32x4 *)p;
    const anc_f32x4 o = {b.x + acc[0], b.y + acc[1], b.z + acc[2], b.w + acc[3]};
    *(anc_f32x4 *)p = o;
  }
}

}  // namespace

extern "C" int anc_embed_dw_scatter(uint64_t cnt, uint64_t start, uint64_t gid, uint64_t srt, uint64_t dy,
                                    uint64_t out, uint64_t compact, int64_t M, int64_t V, int64_t H,
                                    uint64_t stream) {
  ANC_REQUIRE(cnt && start && gid && srt && dy && (out != 0) != (compact != 0),
              "anc_embed_dw_scatter: null pointer, or both / neither of out and compact given");
  ANC_REQUIRE(M > 0 && M < (1ll << 31) && H > 0 && H % 64 == 0 && H <= 65536 * (int64_t)kChunk && (out == 0 || V > 0),
              "anc_embed_dw_scatter: M=%lld, V=%lld, H=%lld (H must be a multiple of 64)", (long long)M,
              (long long)V, (long long)H);
  ANC_REQUIRE(((cnt | start | gid | srt) & 3) == 0 && (dy & 7) == 0 && ((out | compact) & 15) == 0,
              "anc_embed_dw_scatter: misaligned pointers");
  AncProfScope prof(ANC_PROF_MISC, anc_stream(stream));
  hipLaunchKernelGGL(k_embed_dw_scatter, dim3((unsigned)M, (unsigned)((H + kChunk - 1) / kChunk)), dim3(64), 0,
                     anc_stream(stream), (const int32_t *)cnt, (const int32_t *)start, (const int32_t *)gid,
                     (const int32_t *)srt, (const uint16_t *)dy, (float *)out, (float *)compact, (int)H, M, V);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}
