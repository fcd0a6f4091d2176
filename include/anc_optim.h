/*
 * anc_optim.h — C ABI of libancora_optim.so: the Muon + AdamW optimizer step of
 * MythosAd/ancora-cutile (ancora/optim + ancora/kernels/muon_ns.py) as hand-written
 * HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - every device pointer crosses the boundary as a raw 64-bit address (uint64_t),
 *     every size as int64_t, every stream/event as an opaque uint64_t handle
 *     (0 = the null stream);
 *   - every entry point returns an int status: 0 = ok, non-zero = error, with a
 *     human-readable description available from anc_last_error();
 *   - all launches are asynchronous on the given stream; the library owns no hidden
 *     state: optimizer state, scratch and partial-sum buffers are caller-owned, so
 *     the aliasing the reference relies on (p16 IS the model's GEMM weight buffer,
 *     ancora/model/resident_train.py:96-102) keeps working;
 *   - bf16 travels as uint16 bit patterns, exactly as in the reference
 *     (ancora/optim/adamw.py:63-66);
 *   - results are bitwise reproducible run to run and independent of how tensors are
 *     batched into launches: fixed tiles, no split-K, no atomics, fixed reduction order.
 *
 * Each declaration cites the reference interface (path:line under the reference
 * repository root) that it replaces.
 */
#ifndef ANC_OPTIM_H
#define ANC_OPTIM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ status */

#define ANC_OK               0
#define ANC_ERR_HIP          1   /* a HIP runtime call failed                         */
#define ANC_ERR_ARG          2   /* bad argument: null pointer, misaligned shape, ... */
#define ANC_ERR_UNSUPPORTED  3   /* valid request outside what the kernels implement  */

/* Text of the last error raised on the calling thread ("" if none). */
const char *anc_last_error(void);

/* ABI version: bumped whenever a signature or struct layout below changes. */
int anc_abi_version(void);

/* ----------------------------------------------------- device and memory ---
 * Replaces the cuda.bindings driver calls the reference makes directly
 * (cuMemAlloc/cuMemcpyHtoD/cuMemcpyDtoH/cuMemFree: ancora/optim/adamw.py:51-60,
 *  ancora/kernels/loss.py:277-294, ancora/model/resident.py:52-94) and its stream
 * bootstrap (tests/optim/test_adamw.py:14-16). */

typedef struct {
  int32_t cu_count;          /* compute units                                  */
  int32_t clock_khz;         /* peak engine clock                              */
  int32_t mem_clock_khz;     /* peak memory clock                              */
  int32_t mem_bus_bits;      /* memory bus width                               */
  int32_t wavefront;         /* lanes per wavefront (64 on gfx950)             */
  int32_t lds_bytes_per_block;
  int64_t hbm_bytes;         /* total device memory                            */
  int64_t l2_bytes;
  char    name[64];
  char    arch[64];          /* gcnArchName, e.g. "gfx950:sramecc+:xnack-"     */
} anc_device_info_t;

int anc_init(int device);                        /* hipSetDevice + arch check (gfx950 only) */
int anc_device_info(anc_device_info_t *out);
int anc_malloc(uint64_t *dptr, int64_t bytes);
int anc_free(uint64_t dptr);
int anc_host_alloc(void **hptr, int64_t bytes);  /* pinned host memory */
int anc_host_free(void *hptr);
int anc_mem_info(int64_t *free_bytes, int64_t *total_bytes);
/* Fill with a 32-bit pattern using a kernel (safe inside graph capture). */
int anc_fill_u32(uint64_t dptr, uint32_t value, int64_t n_words, uint64_t stream);
int anc_memcpy_h2d(uint64_t dst, const void *src, int64_t bytes, uint64_t stream);
int anc_memcpy_d2h(void *dst, uint64_t src, int64_t bytes, uint64_t stream);
int anc_memcpy_d2d(uint64_t dst, uint64_t src, int64_t bytes, uint64_t stream);
int anc_stream_create(uint64_t *stream);
int anc_stream_destroy(uint64_t stream);
int anc_stream_sync(uint64_t stream);
int anc_device_sync(void);
int anc_event_create(uint64_t *event);
int anc_event_destroy(uint64_t event);
int anc_event_record(uint64_t event, uint64_t stream);
int anc_event_sync(uint64_t event);
/* Make `stream` wait for `event` (fork/join of the per-shape-group chains onto their own
 * streams; all streams stay at the default priority). */
int anc_stream_wait_event(uint64_t stream, uint64_t event);
int anc_event_elapsed_ms(uint64_t start, uint64_t stop, float *ms);
/* Plain streaming copy kernel of n_bytes (multiple of 16): the calibration
 * reference for HBM traffic counters and the measured copy ceiling. */
int anc_copy_kernel(uint64_t dst, uint64_t src, int64_t n_bytes, uint64_t stream);

/* ------------------------------------------------------------- profiling ----
 * Per-kernel timing with HIP events on the launch stream, for the benchmarks (the
 * reference times with perf_counter around cudaStreamSynchronize,
 * tests/kernels/_bench_ns_fused.py:34-40). While enabled every kernel launch of the
 * library is bracketed by an event pair; anc_profile_read synchronises the device,
 * adds the elapsed times per kernel kind and clears the record. */
#define ANC_PROF_ADAMW        0
#define ANC_PROF_GN_PARTIALS  1
#define ANC_PROF_GN_FINALIZE  2
#define ANC_PROF_MUON_MOM     3
#define ANC_PROF_MUON_UPD     4
#define ANC_PROF_NS_FRO       5
#define ANC_PROF_NS_PREP      6
#define ANC_PROF_NS_GRAM      7   /* A = X X^T           (bf16 matrix-core GEMM) */
#define ANC_PROF_NS_BMAT      8   /* B = b A + c A A     (bf16 matrix-core GEMM) */
#define ANC_PROF_NS_BX        9   /* X = a X + B X       (bf16 matrix-core GEMM) */
#define ANC_PROF_NS_GEMM_F32 10   /* any GEMM of the fp32 validation chain        */
#define ANC_PROF_MISC        11   /* casts, conversions, transposes, fill         */
#define ANC_PROF_COPY        12
#define ANC_PROF_NS_BX_UPD   13   /* X = a X + B X whose epilogue applies the weight update */
#define ANC_PROF_DW_GEMM     14   /* weight-gradient product, partial tiles (bf16 matrix-core GEMM) */
#define ANC_PROF_DW_REDUCE   15   /* sum of the token segments, accumulation, bf16 emission */
#define ANC_PROF_KINDS       16
int anc_profile_enable(int on);
int anc_profile_read(float *ms /* [ANC_PROF_KINDS] */, int64_t *launches /* [ANC_PROF_KINDS] */);

/* --------------------------------------------------------- element types --- */
#define ANC_F32   0
#define ANC_BF16  1

/* ------------------------------------------------- step control block -------
 * 32 bytes in device memory, written by anc_gradnorm_finalize and read by every
 * update kernel, so that clip and skip decisions never need a host round trip.
 * No reference counterpart: the reference has no grad-norm, clip or non-finite
 * guard (its closest pattern is the single-block fixed-order reduction of
 * ancora/kernels/muon_ns.py:156-165). Passing ctl = 0 to an update kernel means
 * "clip_scale = 1, never skip".
 * `t` counts the steps that passed the guard: anc_gradnorm_finalize with count_step != 0
 * advances it when the step is not skipped, so a skipped step needs no undo on the host and the
 * whole guarded step can be issued without a host synchronisation (the reference's resident
 * step never synchronises, ancora/model/resident_train.py:338-339). The update kernels take the
 * step's bias corrections and rounding seed from it on request (anc_adamw_hyper_t.step_table,
 * ANC_SR_STEP_SEED). The caller zeroes the block once (or sets t when resuming). */
typedef struct {
  double   sumsq;        /* sum of g*g over every gradient element, fp64          */
  float    norm;         /* (float)sqrt(sumsq)                                    */
  float    clip_scale;   /* min(1, max_norm / (norm + eps)); 1 if max_norm <= 0   */
  uint32_t skip;         /* 1 if sumsq is not finite: update kernels write nothing */
  uint32_t t;            /* steps counted so far, this one included if not skipped */
  uint32_t reserved[2];
} anc_step_ctl_t;
/* Stochastic-rounding switch of the update kernels (`sr` arguments and anc_adamw_hyper_t.sr):
 * 0 = round to nearest even; ANC_SR_ON = stochastic rounding with the seed base given;
 * ANC_SR_ON | ANC_SR_STEP_SEED = the seed base of the call is seed_base +
 * ANC_SR_SEED_STRIDE * ctl->t (uint32 wrap-around), i.e. the per-step seed is formed on the device
 * from the step count of the control block (ctl must not be 0). */
#define ANC_SR_ON           1
#define ANC_SR_STEP_SEED    2
#define ANC_SR_SEED_STRIDE  1000003u

/* ------------------------------------------------------------ grad-norm ----
 * Deterministic global gradient norm, no atomics. Stage 1 writes one fp64
 * partial per ANC_GN_CHUNK-element chunk of the tensor (lane-strided exact
 * products, wavefront shuffle reduction, fixed LDS tree); chunk boundaries are
 * fixed relative to the tensor start, so the partials do not depend on the grid
 * or on which tensors share a launch. Stage 2 reduces the whole partial array
 * in a fixed order and writes the control block. */
#define ANC_GN_CHUNK 8192
int64_t anc_gradnorm_num_partials(int64_t n);
int anc_gradnorm_partials(uint64_t g, int64_t n, int g_dtype,
                          uint64_t partials /* double[] */, int64_t part_offset,
                          uint64_t stream);
typedef struct {
  uint64_t g;            /* gradient tensor                                    */
  int64_t  n;            /* elements                                           */
  int64_t  chunk0;       /* index of this tensor's first chunk in the launch   */
  int64_t  part0;        /* index of its first partial in the partial array    */
  int32_t  dtype;        /* ANC_F32 or ANC_BF16                                */
  int32_t  pad;
} anc_gn_desc_t;
/* One launch over n_tensors tensors described by a device-resident table. */
int anc_gradnorm_partials_multi(uint64_t desc_table, int32_t n_tensors,
                                int64_t total_chunks, uint64_t partials,
                                uint64_t stream);
/* count_step != 0: ctl->t is advanced by one unless the step is skipped; 0: ctl->t is left as it is. */
int anc_gradnorm_finalize(uint64_t partials, int64_t n_partials,
                          float max_norm, float eps, int32_t count_step,
                          uint64_t ctl /* anc_step_ctl_t* */, uint64_t stream);

/* The same norm for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference. One
 * tensor of n elements; result in ctl bit-identical to anc_gradnorm_partials(g, n, g_dtype, buf, 0)
 * followed by anc_gradnorm_finalize(buf, anc_gradnorm_num_partials(n), ..., count_step = 0, ...).
 * The stage-1 partial
 * sums live in a 2 MiB array built into the library (one copy per GPU, held until the process
 * ends), so n is limited to anc_gradnorm_static_max_elements() = 2^31; larger n returns
 * ANC_ERR_ARG. The call allocates nothing (no hipMalloc/hipFree, no events, and it is not seen
 * by anc_profile_*). All calls on one GPU share that array: calls that overlap in time on one
 * GPU (different streams without ordering) race and must be serialised by the caller: issue them
 * on one stream, or order the streams with events. (The library cannot check this for the caller
 * without allocating: it holds no event, and a remembered stream handle may be stale.) */
int64_t anc_gradnorm_static_max_elements(void);
int anc_gradnorm_static(uint64_t g, int64_t n, int g_dtype, float max_norm, float eps,
                        uint64_t ctl /* anc_step_ctl_t* */, uint64_t stream);

/* ---------------------------------------------------------------- AdamW ----
 * Replaces the `_adamw` cuda-tile kernel and its launch tuple
 * (g, m, v, p32, p16, OTM, beta1, beta2, eps, lr, wd, ibc1, ibc2)
 * (ancora/optim/adamw.py:23-41, launched at :94-97, also from
 *  ancora/model/resident_train.py:350-353, resident_model.py:162-166,
 *  ancora/kernels/moe.py:586-588,603-604).
 *
 * One pass per element: read g (fp32 or bf16), m, v, p32; write m, v, p32 and the
 * bf16 copy p16. All scalars are rounded to fp32 once on the host, so the kernel
 * reproduces a numpy fp32 evaluation operation by operation (no FMA contraction,
 * correctly rounded divide and sqrt).
 *
 *   form ANC_ADAMW_FORM_DIV  (numpy oracle, tests/optim/test_adamw.py:37-41):
 *       g' = g * clip_scale
 *       m  = beta1*m + omb1*g'            v = beta2*v + (omb2*g')*g'
 *       p  = p - lr * ((m/bc1) / (sqrt(v/bc2) + eps) + wd*p)
 *   form ANC_ADAMW_FORM_IBC  (the reference kernel, ancora/optim/adamw.py:34-37):
 *       m  = beta1*m + (1.0f-beta1)*g'    v = beta2*v + ((1.0f-beta2)*g')*g'
 *       p  = p - lr * ((m*bc1) / (sqrt(v*bc2) + eps) + wd*p)     (bc = 1/(1-beta^t))
 *
 * p16 = round-to-nearest-even bf16 of the new p (ancora/optim/adamw.py:41,63-65), or,
 * with sr != 0, the stochastic rounding (bits(p) + dither) >> 16 with the counter-based
 * dither of ancora/kernels/fused.py:154-161 keyed on (row = i/64, col = i%64, seed),
 * non-finite values passed through unchanged. */
#define ANC_ADAMW_FORM_DIV 0
#define ANC_ADAMW_FORM_IBC 1
typedef struct {
  float   beta1, beta2;
  float   omb1, omb2;    /* fp32(1-beta1), fp32(1-beta2) — used by FORM_DIV only   */
  float   eps, lr;
  float   bc1, bc2;      /* FORM_DIV: fp32(1-beta^t); FORM_IBC: fp32(1/(1-beta^t)) */
  int32_t form;
  int32_t sr;            /* 0 = RNE downcast, ANC_SR_ON (| ANC_SR_STEP_SEED)        */
  uint32_t seed_base;    /* per-step SR seed; a tensor's seed is seed_base + its own */
  int32_t step_cap;      /* entries 1 .. step_cap of step_table are valid           */
  uint64_t step_table;   /* 0, or a device array of anc_adamw_step_t: bc1 and bc2 are then taken
                            from entry min(ctl->t, step_cap) instead of from this block (steps
                            counted on the device; ctl must not be 0). The host fills the table
                            ahead with the same fp32 values it would pass per step; once both
                            corrections have reached 1.0f the last entry serves every later step */
} anc_adamw_hyper_t;
/* One entry per counted step (entry 0 unused): the scalars of that step. The dense kernels read
 * bc1 and bc2; anc_adamw_rows reads all four. */
typedef struct { float bc1, bc2, lr; uint32_t seed_base; } anc_adamw_step_t;

int anc_adamw(uint64_t g, uint64_t m, uint64_t v, uint64_t p32, uint64_t p16,
              int64_t n /* multiple of 64, as ancora/optim/adamw.py:20,79 */,
              int g_dtype, const anc_adamw_hyper_t *h, float wd, uint32_t seed,
              uint64_t ctl, uint64_t stream);

typedef struct {
  uint64_t g, m, v, p32, p16;
  int64_t  n;            /* elements, multiple of 64                            */
  int64_t  blk0;         /* index of this tensor's first block in the launch    */
  float    wd;           /* per-tensor weight decay (0 for no_decay names)      */
  uint32_t seed;         /* per-tensor SR seed offset (added to seed_base)      */
  int32_t  g_dtype;
  int32_t  pad;
} anc_adamw_desc_t;
int64_t anc_adamw_num_blocks(int64_t n);   /* blocks one tensor of n elements occupies */
/* The whole AdamW parameter group in ONE launch (the reference launches once per
 * tensor, ancora/optim/adamw.py:92-97). Per-element results are identical to anc_adamw. */
int anc_adamw_multi(uint64_t desc_table, int32_t n_tensors, int64_t total_blocks,
                    const anc_adamw_hyper_t *h, uint64_t ctl, uint64_t stream);

/* Row-sparse AdamW on a (V, H) tensor whose gradient touches few rows per step (an input
 * embedding not tied to the output head), with the results of the dense kernel. The
 * reference has only the dense kernel (ancora/optim/adamw.py:92-97). A
 * dense step moves rows with zero gradient too (moment decay, bias-corrected momentum, weight
 * decay), so each row carries the last counted step it is current for (last_step, int32[V], zero
 * at the start) and the steps it missed are replayed on it, with g = 0 and that step's own
 * scalars from step_table (device array of anc_adamw_step_t {bc1, bc2, lr, seed_base} per counted
 * step, entries 1 .. t_now, bc as in anc_adamw_hyper_t for the chosen form), before anything else
 * is done to it. m, v, p32 and p16 of a current row are bit-identical to anc_adamw's.
 *   grads != 0: rows[i]'s gradient is row i of grads, (n_rows, H) fp32: replay through t_now - 1,
 *               then step t_now (clip scale and skip flag from ctl as in anc_adamw).
 *   grads == 0: replay through t_now (what the forward must call for the rows it is about to
 *               gather; with rows == 0 and n_rows == V: every row, e.g. before a checkpoint).
 * rows: distinct int32 indices on the device. beta1, beta2, omb1, omb2, eps, form and sr are taken
 * from h; bc1, bc2, lr and seed_base of h are ignored (the table carries them per step). */
int anc_adamw_rows(uint64_t rows, int64_t n_rows, uint64_t grads, uint64_t m, uint64_t v,
                   uint64_t p32, uint64_t p16, uint64_t last_step, int64_t V, int64_t H,
                   uint64_t step_table, int32_t t_now, const anc_adamw_hyper_t *h, float wd,
                   uint32_t seed, uint64_t ctl, uint64_t stream);

/* Input-embedding weight gradient by deterministic sorted scatter: replaces `_embed_dw_scatter`
 * (ancora/kernels/fused.py:387-408, launched at ancora/model/resident_moe_model.py:333-334) with
 * the group arrays of `build_id_groups` (fused.py:411-424): cnt, start, gid (int32[M], groups
 * padded with cnt = 0) and srt (int32[M], the stable argsort of the token ids). dy: (M, H) bf16.
 *   out != 0:     out[gid[g]] += sum_r f32(dy[srt[start[g] + r]]), out (V, H) fp32 (the reference)
 *   compact != 0: compact[g]   = that sum, (M, H) fp32: the gradient rows anc_adamw_rows takes
 * Rows of a group are added in sorted order starting from zero, one writer per element, no
 * atomics: bit-identical to the sequential fp32 sum, and from run to run. H % 64 == 0. A group
 * whose start / count / id / sorted indices point outside the arrays writes nothing. */
int anc_embed_dw_scatter(uint64_t cnt, uint64_t start, uint64_t gid, uint64_t srt, uint64_t dy,
                         uint64_t out, uint64_t compact, int64_t M, int64_t V, int64_t H,
                         uint64_t stream);

/* p16 = bf16(p32): replaces `_cast_bf16` (ancora/kernels/fused.py:285-290). */
int anc_cast_bf16(uint64_t p32, uint64_t p16, int64_t n, int sr, uint32_t seed,
                  uint64_t stream);

/* ------------------------------------------------------ Muon elementwise ---
 * Momentum + Nesterov look-ahead, replaces `_muon_mom`, `_muon_mom_t`, `_e_muon_mom`
 * (ancora/kernels/muon_ns.py:177-186, 206-217, 409-418; numpy form
 *  ancora/optim/muon.py:303-305):
 *     g' = g*clip_scale;  buf = mom*buf + g';  u = nesterov ? g' + mom*buf : buf
 * buf is (K,N) fp32, g is (K,N) fp32 or bf16; u is written as (K,N), or as (N,K) when
 * transpose_out != 0 (tall weights enter Newton-Schulz transposed,
 * ancora/optim/muon.py:72-74), with dtype u_dtype: ANC_BF16 (RNE, the reference's
 * storage) or ANC_F32 (this library's precise chain). K and N multiples of 64. */
int anc_muon_momentum(uint64_t buf, uint64_t g, uint64_t u, int64_t K, int64_t N,
                      float mom, int nesterov, int transpose_out,
                      int g_dtype, int u_dtype, uint64_t ctl, uint64_t stream);

/* Master update + bf16 refresh, replaces `_muon_update`, `_muon_update_cast`,
 * `_muon_update_cast_t`, `_e_muon_update` (ancora/kernels/muon_ns.py:189-195,
 * 220-242, 421-427; numpy form ancora/optim/muon.py:308-309):
 *     p32 = p32 - lr_scale*O;   p16 = bf16(p32)   (RNE, or SR keyed as for AdamW)
 * O is (K,N), or (N,K) when transpose_in != 0; o_dtype ANC_BF16 or ANC_F32.
 * p16 = 0 skips the bf16 refresh. sr: 0 or ANC_SR_ON. */
int anc_muon_update(uint64_t p32, uint64_t p16, uint64_t O, int64_t K, int64_t N,
                    float lr_scale, int transpose_in, int o_dtype,
                    int sr, uint32_t seed, uint64_t ctl, uint64_t stream);

typedef struct {
  uint64_t buf, g, p32, p16;   /* per-weight state, (K,N) row-major               */
  uint64_t u;                  /* this weight's slice of the packed NS batch      */
  int32_t  K, N;
  int32_t  transpose;          /* 1 for tall weights (K > N)                      */
  int32_t  g_dtype;
  int32_t  scale_idx;          /* which of the launch's lr_scale values applies   */
  uint32_t seed;               /* per-weight SR seed offset (added to seed_base)  */
  int64_t  tile0;              /* index of this weight's first 4096-element block */
  uint64_t p16t;               /* 0, or a (N,K) bf16 copy of the weight that the update
                                  refreshes in the same pass (replaces the `_transpose_e`
                                  launch after the step, ancora/kernels/moe.py:593-597)   */
} anc_muon_desc_t;
#define ANC_MUON_MAX_SCALES 8
/* All weights of a packed batch in ONE launch each (the reference launches once per
 * weight, ancora/optim/muon.py:261-276). Per-element results equal the single calls. */
int anc_muon_momentum_multi(uint64_t desc_table, int32_t n_weights, int64_t total_tiles,
                            float mom, int nesterov, int u_dtype,
                            uint64_t ctl, uint64_t stream);
/* Momentum straight into the Newton-Schulz input format (replaces `_muon_mom`/`_muon_mom_t`
 * plus the norm pass `_fro`, ancora/kernels/muon_ns.py:156-186, 206-217). desc.u is each
 * weight's fp32 slice of the packed batch that starts at pair_base; the bf16 pair of u is
 * written at the same element offset into two bf16 arrays, hi at pair_base, lo
 * lo_offset_bytes behind it, and block b leaves the sum of its 4096 u*u (fp64, fixed
 * order) in fro_partials[b]: K*N/4096 consecutive partials per weight. */
int anc_muon_momentum_multi_pair(uint64_t desc_table, int32_t n_weights, int64_t total_tiles,
                                 float mom, int nesterov, uint64_t pair_base,
                                 int64_t lo_offset_bytes, uint64_t fro_partials,
                                 uint64_t ctl, uint64_t stream);
/* lr_scales: host array of ANC_MUON_MAX_SCALES values lr * sqrt(max(1, K/N))
 * (ancora/optim/muon.py:308), one per distinct weight shape class; the table itself
 * holds nothing that changes from step to step. sr: 0, ANC_SR_ON, or
 * ANC_SR_ON | ANC_SR_STEP_SEED (seed base formed from ctl->t on the device). */
int anc_muon_update_multi(uint64_t desc_table, int32_t n_weights, int64_t total_tiles,
                          const float *lr_scales, int o_dtype, int sr, uint32_t seed_base,
                          uint64_t ctl, uint64_t stream);

/* bf16 transpose XT(N,M) = X(M,N)^T: replaces `_transpose_mat`
 * (ancora/kernels/muon_ns.py:198-203) and, batched over E, `_transpose_e`
 * (ancora/kernels/moe.py:370-377). M, N multiples of 64. */
int anc_transpose_bf16(uint64_t X, uint64_t XT, int64_t E, int64_t M, int64_t N,
                       uint64_t stream);

/* ------------------------------------------------------ weight gradients ----
 * dW (+)= x^T dy for up to 8 weights per call: replaces `_gemm_dW` / `_gemm_dW_acc`
 * (ancora/kernels/fused.py:190-219, launched per weight at ancora/model/resident_train.py:285-287),
 * the producer of the fp32 gradients the optimizer step reads. xT is the activation matrix, either
 * transposed, (K, T) bf16 row-major, or as it lies, x (T, K), with x_row_major = 1; dy is (T, N) bf16; dW (K, N) fp32 is overwritten, or added onto when
 * `accumulate` is set (micro-batch accumulation in place); g16, if not 0, receives the bf16 copy
 * (RNE) of the final dW, the format the step reads.
 * Accumulation order. segments = 0 or 1 (the default): one workgroup owns one 128x256 output tile
 * and runs the whole token axis in ascending order with one fp32 accumulator per element: fixed
 * tiles, no split-K, the bits of dW are a function of x, dy (and the old dW) alone, independent of
 * what else is in the call and of how the caller groups its calls; the GEMM's epilogue adds onto
 * the old dW and writes g16 itself, no workspace is needed (with gn_partials set a second kernel
 * finishes the gradient and needs workspace K*N*4). A call fills the GPU when it carries about 500
 * tiles: the 7 weights of a Qwen3-0.6B layer in one call are 480. segments > 1, or -1 for
 * anc_gemm_dw_info's shape rule (the smallest power of two that gives the problem 256 workgroups
 * by itself): the token axis is cut into S equal pieces (T a multiple of 32 S), each piece of each
 * tile is one workgroup's whole K loop leaving an fp32 partial tile, and a second kernel adds the
 * pieces in ascending order: deterministic, but the bits then DEPEND ON S (and on nothing else);
 * workspace of S*K*N*4 bytes per problem (anc_gemm_dw_workspace_bytes for the shape rule), not
 * shared between the problems of a call.
 * T % 32, K % 128, N % 256 == 0 (the reference: all % 64); pointers and g16 16-byte aligned. */
typedef struct {
  uint64_t xT, dy, dW, g16, workspace;
  int64_t  T, K, N, workspace_bytes;
  int32_t  accumulate, segments;
  uint64_t gn_partials;        /* 0, or double[K*N / ANC_GN_CHUNK]: the grad-norm partial sums of this
                                  gradient (of its bf16 copy if g16 is set), bit-identical to what
                                  anc_gradnorm_partials would compute from the stored gradient, so
                                  that the step's norm needs no pass of its own over it */
  int32_t  x_row_major;        /* 1: `xT` points at the activations as they lie, x (T, K) row-major (the
                                  reference's argument); 0: at x^T (K, T). Same bits either way; all
                                  problems of a call must agree */
  int32_t  reserved;
} anc_dw_problem_t;
int64_t anc_gemm_dw_workspace_bytes(int64_t T, int64_t K, int64_t N);
int anc_gemm_dw_multi(const anc_dw_problem_t *problems, int32_t n_problems, uint64_t stream);
/* FLOPs of one problem (2 T K N, all executed) and the segment count of the shape rule (segments = -1). */
int anc_gemm_dw_info(int64_t T, int64_t K, int64_t N, double *flops, int32_t *segments);

/* MXFP8 re-quantisation of bf16 weights (E, K, N) after the step: per block of 32 consecutive K
 * and per column one E8M0 scale byte = (biased fp32 exponent of the block's amax) - 7 (0 below
 * 7), elements E4M3FN(w / 2^(byte-127)) rounded to nearest even. col_major = 0 writes
 * fp8_out (E, K, N) and scale_out (E, K/32, N): replaces `_quant_mxfp8_w`
 * (ancora/kernels/quant.py:60-73); col_major = 1 writes the transposed fp8_out (E, N, K) and
 * scale_out (E, N, K/32): replaces `_quant_mxfp8_w_cm` (quant.py:84-100). The reference launches
 * them per weight from the forward that follows a step (ancora/model/resident_train.py:190-199,
 * dirty flags set by the step at :354-357). K and N must be multiples of 128 (the reference:
 * K % 32, N % 128); w and fp8_out 16-byte, scale_out 8-byte aligned. bf16 subnormals count as
 * zero, Inf/NaN elements become the E4M3 NaN byte. */
int anc_quant_mxfp8_w(uint64_t w_bf16, uint64_t fp8_out, uint64_t scale_out, int64_t E, int64_t K,
                      int64_t N, int col_major, uint64_t stream);

/* --------------------------------------------------------- Newton-Schulz ---
 * Replaces the chains `newton_schulz_resident` / `newton_schulz_resident_e`
 * (ancora/kernels/muon_ns.py:245-283, 430-468) and the kernels they launch
 * (`_fro_recip`, `_scale`, `_gemm_nt_tril`, `_gemm_axpy_tril`, `_mirror`,
 *  `_gemm_axpy_bf16` and their `_e_` twins, :68-174, 293-406); numpy form
 * ancora/optim/muon.py:67-80 and tests/kernels/_probe_polar_express_device.py:27-34.
 *
 * X holds E matrices (M,N), M <= N, packed (E*M, N) row-major, fp32; it is
 * overwritten with the orthogonalised result. Per matrix:
 *     X = X / (||X||_F + eps)
 *     for k < steps: (a,b,c) = coef[3k..3k+2];  A = X X^T;  B = b A + c A A;  X = a X + B X
 *
 * Modes
 *   ANC_NS_BF16       GEMM operands are bf16 at the matrix-core input, fp32 accumulate (MFMA).
 *                     Between steps the iterate is a bf16 pair hi + lo (16 significant bits), the
 *                     diagonals of A and B stay fp32, and selected products add the bf16 residuals
 *                     of X, A, B as further accumulation terms: by shape (the plan) and, per
 *                     matrix, by the gates below.
 *   ANC_NS_BF16_FAST  the same without any residual term (15 GEMM passes); no accuracy bar of its
 *                     own (about 2.2e-3 on 1024x1024).
 *   ANC_NS_BF16_X3    the residuals of both operands in every product of every iteration: about
 *                     1e-5 from the fp32 chain whatever the input, three times the matrix-core work.
 *   ANC_NS_BF16_LATE3 for coefficients that do not drive the singular values to 1 (Keller's quintic,
 *                     ancora/kernels/muon_ns.py:21, leaves them in 0.7 .. 1.2, so operand rounding
 *                     stays a first-order error to the end: ANC_NS_BF16 reaches 2.8e-3 .. 5e-3 there).
 *                     Every matrix: residual of X from iteration 2 on, of A and B from iteration 3
 *                     on (the last three iterations of a chain shorter than 5 steps); the wide gate
 *                     below; 2.05 times the work of ANC_NS_BF16_FAST; 2e-5 .. 9e-4.
 *   ANC_NS_FP32       every product in fp32 (validation mode, 1e-5).
 *
 * Plan of ANC_NS_BF16 by shape
 *   M < 1024          residuals of X, A, B from iteration 1 on (iteration 0 below M = 256); no gates.
 *   M >= 1024, N < 2M residual of X in A = X X^T and X = a X + B X of the last iteration.
 *   M >= 1024, N >= 2M  no residual term; B = b A + c A A takes the off-diagonal entries of A from the
 *                     bf16 copy it multiplies anyway (no fp32 copy of A: 3 .. 8 % of accuracy); with
 *                     the 256-tile kernels the low half of the iterate is kept as 8 instead of 16
 *                     bits wherever no product multiplies it (the iterate to 24 bits).
 * Gates (M >= 1024), per matrix, from statistics of the matrix alone, so that a result never
 * depends on the batch: after the first A = X X^T, proxy = N * ||offdiag(A)||_F^2 (1.0 for independent
 * entries whatever the row scaling, 1.7 for columns scaled over 0.1 .. 3, about N/r when the mass sits
 * in r directions); for some ranges of it the column concentration colc = N * sum_j c_j^4 /
 * (sum_j c_j^2)^2 over the column norms c_j of the input (every fourth row), which equals the proxy
 * exactly when column norms explain it, and the share of the mass in the lightest 64-column block.
 *   proxy > 1.3, N < 2M     residual of X in both X-products of iterations 2 and 3 (5-step chains);
 *   proxy > 2.5             residual of X in A = X X^T of iteration 2 (N >= 2M; also iteration 1 in
 *                           chains shorter than 5 steps) or of iterations 1 and 2 (N < 2M);
 *   the wide gate           every residual in all three products from iteration 1 on (2.6 times the
 *                           work, for that matrix alone; it keeps the fp32 copy of A) if
 *                           2.5 < proxy < 40 (spectra spread over decades, many moderately large
 *                           columns), or proxy >= 40 and (colc < 0.85 proxy: a low-rank signal, a
 *                           steep spectrum, alone or mixed with outlier columns; or less than 3e-3 of
 *                           the mass outside the outlier columns), or just below the band, where the
 *                           column norms leave part of the proxy unexplained (a gap in the spectrum,
 *                           e.g. near-duplicate rows): N < 2M, 1.5 < proxy <= 2.5 and colc < 0.85
 *                           proxy; N >= 2M, 1.15 < proxy <= 2.5 and proxy - colc > 0.15.
 * Accuracy bar of ANC_NS_BF16 under the Polar-Express schedule (ANC_NS_BF16_LATE3 under Keller's):
 * 2e-3 relative Frobenius against the fp32 chain, held on independent, sparse and heavy-tailed
 * entries, row or column outliers (1 % x30 .. x3000, 10 % x10), scaled columns, log-uniform spectra
 * up to condition number 1e4, power-law spectra, low-rank signals over noise down to 1 %,
 * near-duplicate rows, shapes up to 4096x8192, chains of 3 .. 8 steps. Known limits: a low-rank
 * bulk hidden behind independent outlier columns (the column norms explain the proxy, the bulk's own
 * spectrum is not seen: 2.5e-3 at 1024x3072); under Keller a single element of 1000 standard
 * deviations (up to 3e-3). ANC_NS_BF16_X3 has neither.
 *
 * M and N must be multiples of 128 (the reference's tile alignment,
 * ancora/optim/muon.py:98). workspace must hold anc_ns_workspace_bytes(E,M,N,mode)
 * bytes; the chain keeps nothing in it between calls. */
#define ANC_NS_BF16 0
#define ANC_NS_FP32 1
#define ANC_NS_BF16_FAST 2
#define ANC_NS_BF16_X3 3
#define ANC_NS_BF16_LATE3 4
/* Flag OR-ed into a bf16 mode: use the 128x128-tile GEMM kernel even where the 256x256-tile
 * kernel applies. The two produce the same bits in ANC_NS_BF16_FAST (no residual terms). Residual
 * terms are added in an order that depends on which elements of a symmetric product are computed
 * and which are mirrored, hence on the tile size: the results then differ in the last fp32 bits
 * of A and B (1e-6 .. 4e-4 of the result, largest on gated outlier-column inputs). ANC_NS_BF16 on
 * N >= 2M keeps 8-bit low halves of the iterate with the 256-tile kernels only: the 24-bit iterate
 * differs from the 32-bit pair by 2^-16 per element, which the chain turns into another
 * realisation of its rounding error (the results are then 1.2e-3 apart, each inside the accuracy
 * bar). The flag exists so that tests can show both. */
#define ANC_NS_TILE128 0x100
int64_t anc_ns_workspace_bytes(int64_t E, int64_t M, int64_t N, int mode);
int anc_ns_batched(uint64_t X, int64_t E, int64_t M, int64_t N,
                   int steps, const float *coef /* host, 3*steps */, float eps,
                   int mode, uint64_t workspace, int64_t workspace_bytes,
                   uint64_t stream);

/* The same chain fed by anc_muon_momentum_multi_pair: the momentum kernel leaves the
 * unnormalised input U as a bf16 pair (Uh = bf16(u), Ul = bf16(u - Uh), both (E,M,N)) and
 * n_partials sums of u*u per matrix; the reference's separate norm and scale passes
 * (`_fro` + `_scale_e`, ancora/kernels/muon_ns.py:156-174, 387-406) disappear: the scale
 * 1/(||U||_F + eps) is applied inside the first step's epilogues (A = s^2 U U^T,
 * X1 = s (a U + B U)). The fp32 result goes to X32_out, which may overlay the input pair
 * (Uh at X32_out, Ul right behind it: the same 4 bytes per element); steps >= 2. bf16
 * modes only. Results differ from anc_ns_batched on the same data only by where the bf16
 * rounding of the first operand falls (before instead of after the scaling). The first products
 * run on the unnormalised values: a matrix whose sum of squares is below 2^-100 (||U||_F < 9e-16,
 * where products of two elements would underflow fp32) is first multiplied in place, Uh and Ul,
 * by the power of two that brings its norm into [1, 2), exactly, and its scale carries the
 * inverse; every other matrix is left as it is. */
int anc_ns_batched_pair(uint64_t Uh, uint64_t Ul, uint64_t fro_partials, int64_t n_partials,
                        uint64_t X32_out, int64_t E, int64_t M, int64_t N,
                        int steps, const float *coef, float eps, int mode,
                        uint64_t workspace, int64_t workspace_bytes, uint64_t stream);

/* Several batches (the shape groups of one optimizer step) through anc_ns_batched_pair side
 * by side: each of the three products of each step is ONE launch over all batches, so the
 * CUs stay busy where per-batch launches would each end in a partly filled last wave of
 * workgroups. No reference counterpart (the reference runs its shape groups one after the
 * other, ancora/optim/muon.py:257-277). Results equal anc_ns_batched_pair on each batch bit
 * for bit. n_probs <= 8; every M and N a multiple of 256; steps >= 2; bf16 modes. */
typedef struct {
  uint64_t Uh, Ul;            /* input bf16 pair, (E,M,N) each                        */
  uint64_t fro_partials;      /* n_partials sums of u*u per matrix                     */
  uint64_t X32_out;           /* fp32 result (may overlay the pair)                    */
  uint64_t workspace;         /* anc_ns_workspace_bytes(E,M,N,mode) bytes of its own   */
  int64_t  n_partials, E, M, N, workspace_bytes;
} anc_ns_problem_t;
int anc_ns_batched_pair_multi(const anc_ns_problem_t *probs, int32_t n_probs, int steps,
                              const float *coef, float eps, int mode, uint64_t stream);

/* anc_ns_batched_pair_multi followed by the Muon weight update of every matrix, the update
 * applied by the epilogue of the chain's last product instead of by a kernel of its own:
 * W -= lr_scales[scale_idx] * O, bf16 copy by RNE or stochastic rounding (`_muon_update_cast[_t]`,
 * ancora/kernels/muon_ns.py:189-242, launched after the chain at ancora/optim/muon.py:272-277).
 * desc_tables[q] is a device array of problems[q].E anc_muon_desc_t, entry e describing the weight
 * whose orthogonalised update is matrix e of the batch (fields read: p32, p16 (may be 0), K, N,
 * transpose, scale_idx, seed; p16t must be 0). X32_out of the problems is not used. Results in
 * p32 and p16 are bit-identical to the unfused sequence; the fp32 hand-off (8 bytes per parameter
 * of HBM traffic) disappears. ctl: the step's control block or 0 (skip flag honoured). sr as
 * for anc_muon_update_multi. */
int anc_muon_ns_update_multi(const anc_ns_problem_t *problems, int32_t n_problems,
                             const uint64_t *desc_tables, int steps, const float *coef, float eps,
                             int mode, const float *lr_scales /* [ANC_MUON_MAX_SCALES] */, int sr,
                             uint32_t seed_base, uint64_t ctl, uint64_t stream);

/* Matrix-core FLOPs of one anc_ns_batched call: `executed` counts the tiles and terms the
 * kernels really multiply (residual terms; of the symmetric products the tiles on or below the
 * diagonal, each in full: 256x256 tiles where dims are multiples of 256, i.e. 10/16 of the dense
 * product at M = 1024, else, or with ANC_NS_TILE128 in `mode`, 128x128 tiles, 36/64; the
 * profiler's matrix-instruction counter reads this number), `dense` is steps*(4 M^2 N + 2 M^3)
 * per matrix. Roofline figures use `executed`; matrices that take the conditioning gate add
 * anc_ns_hard_info's extra work. */
int anc_ns_flops(int64_t E, int64_t M, int64_t N, int steps, int mode,
                 double *executed, double *dense);
/* Of the E matrices of the last chain call that used `workspace`: how many took extra terms
 * through a conditioning gate, and the matrix-core work they add, all together, to
 * anc_ns_flops' `executed`. Synchronises `stream` and reads 64 bytes per matrix back. */
int anc_ns_hard_info(uint64_t workspace, int64_t E, int64_t M, int64_t N, int mode, int steps,
                     int32_t *n_gated, double *extra_flops, uint64_t stream);
/* Executed matrix-core work of one product of one iteration of that chain: iteration k in
 * 0..steps-1, product 0 (A = X X^T), 1 (B = b A + c A A) or 2 (X = a X + B X). */
int anc_ns_product_flops(int64_t E, int64_t M, int64_t N, int steps, int mode, int k, int product,
                         double *executed);

/* fp32 <-> bf16 conversion of packed batches (entry/exit of the bf16-typed
 * reference drivers): dst_f32 = float(src_bf16); dst_bf16 = RNE(src_f32). */
int anc_bf16_to_f32(uint64_t src, uint64_t dst, int64_t n, uint64_t stream);
int anc_f32_to_bf16(uint64_t src, uint64_t dst, int64_t n, uint64_t stream);

#ifdef __cplusplus
}
#endif
#endif /* ANC_OPTIM_H */
