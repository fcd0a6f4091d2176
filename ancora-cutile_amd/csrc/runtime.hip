// Device, memory, stream and event plumbing behind the C ABI, plus the two tiny
// utility kernels (fill, copy). Replaces the cuda.bindings driver calls the reference
// makes from Python (ancora/optim/adamw.py:51-60, ancora/model/resident.py:52-94).
#include "common.h"
#include <stdarg.h>
#include <string.h>

static thread_local char g_err[512] = "";

void anc_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int anc_hip_fail(hipError_t e, const char *what, const char *file, int line) {
  anc_set_error("HIP error %d (%s) at %s:%d in %s", (int)e, hipGetErrorString(e), file, line, what);
  return ANC_ERR_HIP;
}

extern "C" const char *anc_last_error(void) { return g_err; }

// ---- per-launch profiler -------------------------------------------------------------
#include <mutex>
#include <vector>
namespace {
struct ProfRec { int kind; hipEvent_t start, stop; };
std::mutex g_prof_mu;
bool g_prof_on = false;
std::vector<ProfRec> g_prof_recs;
std::vector<hipEvent_t> g_prof_pool;
hipEvent_t prof_event() {
  if (!g_prof_pool.empty()) { hipEvent_t e = g_prof_pool.back(); g_prof_pool.pop_back(); return e; }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}
}  // namespace

void anc_prof_begin(int kind, hipStream_t s) {
  if (!g_prof_on) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  ProfRec r{kind, prof_event(), prof_event()};
  if (r.start == nullptr || r.stop == nullptr) return;
  (void)hipEventRecord(r.start, s);
  g_prof_recs.push_back(r);
}
void anc_prof_end(hipStream_t s) {
  if (!g_prof_on) return;
  std::lock_guard<std::mutex> lk(g_prof_mu);
  if (!g_prof_recs.empty()) (void)hipEventRecord(g_prof_recs.back().stop, s);
}
extern "C" int anc_profile_enable(int on) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  g_prof_on = on != 0;
  return ANC_OK;
}
extern "C" int anc_profile_read(float *ms, int64_t *launches) {
  ANC_REQUIRE(ms != nullptr && launches != nullptr, "anc_profile_read: null output");
  ANC_HIP(hipDeviceSynchronize());
  std::lock_guard<std::mutex> lk(g_prof_mu);
  for (int k = 0; k < ANC_PROF_KINDS; ++k) { ms[k] = 0.0f; launches[k] = 0; }
  for (const ProfRec &r : g_prof_recs) {
    float t = 0.0f;
    if (hipEventElapsedTime(&t, r.start, r.stop) == hipSuccess && r.kind >= 0 && r.kind < ANC_PROF_KINDS) {
      ms[r.kind] += t;
      launches[r.kind] += 1;
    }
    g_prof_pool.push_back(r.start);
    g_prof_pool.push_back(r.stop);
  }
  g_prof_recs.clear();
  return ANC_OK;
}
extern "C" int anc_abi_version(void) { return 3; }

int anc_gradnorm_static_init(void);   // gradnorm.hip: per-device address of its built-in scratch

extern "C" int anc_init(int device) {
  int n = 0;
  ANC_HIP(hipGetDeviceCount(&n));
  ANC_REQUIRE(device >= 0 && device < n, "anc_init: device %d out of range (%d visible)", device, n);
  ANC_HIP(hipSetDevice(device));
  hipDeviceProp_t p;
  ANC_HIP(hipGetDeviceProperties(&p, device));
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
    anc_set_error("anc_init: device %d is %s; this library carries gfx950 code only", device,
                  p.gcnArchName);
    return ANC_ERR_UNSUPPORTED;
  }
  return anc_gradnorm_static_init();
}

extern "C" int anc_device_info(anc_device_info_t *out) {
  ANC_REQUIRE(out != nullptr, "anc_device_info: null output");
  int dev = 0;
  ANC_HIP(hipGetDevice(&dev));
  hipDeviceProp_t p;
  ANC_HIP(hipGetDeviceProperties(&p, dev));
  memset(out, 0, sizeof(*out));
  out->cu_count = p.multiProcessorCount;
  out->clock_khz = p.clockRate;
  out->mem_clock_khz = p.memoryClockRate;
  out->mem_bus_bits = p.memoryBusWidth;
  out->wavefront = p.warpSize;
  out->lds_bytes_per_block = (int32_t)p.sharedMemPerBlock;
  out->hbm_bytes = (int64_t)p.totalGlobalMem;
  out->l2_bytes = (int64_t)p.l2CacheSize;
  strncpy(out->name, p.name, sizeof(out->name) - 1);
  strncpy(out->arch, p.gcnArchName, sizeof(out->arch) - 1);
  return ANC_OK;
}

extern "C" int anc_malloc(uint64_t *dptr, int64_t bytes) {
  ANC_REQUIRE(dptr != nullptr && bytes > 0, "anc_malloc: bad arguments (bytes=%lld)", (long long)bytes);
  void *p = nullptr;
  ANC_HIP(hipMalloc(&p, (size_t)bytes));
  *dptr = (uint64_t)p;
  return ANC_OK;
}
extern "C" int anc_free(uint64_t dptr) {
  ANC_REQUIRE(dptr != 0, "anc_free: null pointer");
  ANC_HIP(hipFree((void *)dptr));
  return ANC_OK;
}
extern "C" int anc_host_alloc(void **hptr, int64_t bytes) {
  ANC_REQUIRE(hptr != nullptr && bytes > 0, "anc_host_alloc: bad arguments");
  ANC_HIP(hipHostMalloc(hptr, (size_t)bytes, hipHostMallocDefault));
  return ANC_OK;
}
extern "C" int anc_host_free(void *hptr) {
  ANC_REQUIRE(hptr != nullptr, "anc_host_free: null pointer");
  ANC_HIP(hipHostFree(hptr));
  return ANC_OK;
}
extern "C" int anc_mem_info(int64_t *free_bytes, int64_t *total_bytes) {
  size_t f = 0, t = 0;
  ANC_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = (int64_t)f;
  if (total_bytes) *total_bytes = (int64_t)t;
  return ANC_OK;
}

__global__ void __launch_bounds__(256) k_fill_u32(uint32_t *__restrict__ p, uint32_t v, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < n; i += stride) p[i] = v;
}
extern "C" int anc_fill_u32(uint64_t dptr, uint32_t value, int64_t n_words, uint64_t stream) {
  ANC_REQUIRE(dptr != 0 && n_words >= 0 && (dptr & 3) == 0, "anc_fill_u32: bad arguments");
  if (n_words == 0) return ANC_OK;
  int64_t blocks = (n_words + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  AncProfScope prof(ANC_PROF_MISC, anc_stream(stream));
  hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)blocks), dim3(256), 0, anc_stream(stream),
                     (uint32_t *)dptr, value, n_words);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_memcpy_h2d(uint64_t dst, const void *src, int64_t bytes, uint64_t stream) {
  ANC_REQUIRE(dst != 0 && src != nullptr && bytes >= 0, "anc_memcpy_h2d: bad arguments");
  if (bytes == 0) return ANC_OK;
  ANC_HIP(hipMemcpyAsync((void *)dst, src, (size_t)bytes, hipMemcpyHostToDevice, anc_stream(stream)));
  // Pageable host memory: make the call synchronous so the caller may reuse src at once.
  ANC_HIP(hipStreamSynchronize(anc_stream(stream)));
  return ANC_OK;
}
extern "C" int anc_memcpy_d2h(void *dst, uint64_t src, int64_t bytes, uint64_t stream) {
  ANC_REQUIRE(dst != nullptr && src != 0 && bytes >= 0, "anc_memcpy_d2h: bad arguments");
  if (bytes == 0) return ANC_OK;
  ANC_HIP(hipMemcpyAsync(dst, (const void *)src, (size_t)bytes, hipMemcpyDeviceToHost, anc_stream(stream)));
  ANC_HIP(hipStreamSynchronize(anc_stream(stream)));
  return ANC_OK;
}
extern "C" int anc_memcpy_d2d(uint64_t dst, uint64_t src, int64_t bytes, uint64_t stream) {
  ANC_REQUIRE(dst != 0 && src != 0 && bytes >= 0, "anc_memcpy_d2d: bad arguments");
  if (bytes == 0) return ANC_OK;
  ANC_HIP(hipMemcpyAsync((void *)dst, (const void *)src, (size_t)bytes, hipMemcpyDeviceToDevice,
                         anc_stream(stream)));
  return ANC_OK;
}

extern "C" int anc_stream_create(uint64_t *stream) {
  ANC_REQUIRE(stream != nullptr, "anc_stream_create: null output");
  hipStream_t s;
  ANC_HIP(hipStreamCreate(&s));   // default priority only
  *stream = (uint64_t)s;
  return ANC_OK;
}
extern "C" int anc_stream_destroy(uint64_t stream) {
  ANC_REQUIRE(stream != 0, "anc_stream_destroy: the null stream is not destroyable");
  ANC_HIP(hipStreamDestroy(anc_stream(stream)));
  return ANC_OK;
}
extern "C" int anc_stream_sync(uint64_t stream) {
  ANC_HIP(hipStreamSynchronize(anc_stream(stream)));
  return ANC_OK;
}
extern "C" int anc_device_sync(void) {
  ANC_HIP(hipDeviceSynchronize());
  return ANC_OK;
}
extern "C" int anc_event_create(uint64_t *event) {
  ANC_REQUIRE(event != nullptr, "anc_event_create: null output");
  hipEvent_t e;
  ANC_HIP(hipEventCreate(&e));
  *event = (uint64_t)e;
  return ANC_OK;
}
extern "C" int anc_event_destroy(uint64_t event) {
  ANC_REQUIRE(event != 0, "anc_event_destroy: null event");
  ANC_HIP(hipEventDestroy((hipEvent_t)event));
  return ANC_OK;
}
extern "C" int anc_event_record(uint64_t event, uint64_t stream) {
  ANC_REQUIRE(event != 0, "anc_event_record: null event");
  ANC_HIP(hipEventRecord((hipEvent_t)event, anc_stream(stream)));
  return ANC_OK;
}
extern "C" int anc_event_sync(uint64_t event) {
  ANC_REQUIRE(event != 0, "anc_event_sync: null event");
  ANC_HIP(hipEventSynchronize((hipEvent_t)event));
  return ANC_OK;
}
extern "C" int anc_stream_wait_event(uint64_t stream, uint64_t event) {
  ANC_REQUIRE(event != 0, "anc_stream_wait_event: null event");
  ANC_HIP(hipStreamWaitEvent(anc_stream(stream), (hipEvent_t)event, 0));
  return ANC_OK;
}
extern "C" int anc_event_elapsed_ms(uint64_t start, uint64_t stop, float *ms) {
  ANC_REQUIRE(start != 0 && stop != 0 && ms != nullptr, "anc_event_elapsed_ms: bad arguments");
  ANC_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return ANC_OK;
}

// Streaming copy: 16 bytes per lane per access, four accesses in flight per lane.
__global__ void __launch_bounds__(256) k_copy16(const anc_u32x4 *__restrict__ src,
                                                anc_u32x4 *__restrict__ dst, int64_t n_vec) {
  const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  anc_u32x4 r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int64_t i = base + j * 256;
    if (i < n_vec) r[j] = __builtin_nontemporal_load(&src[i]);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int64_t i = base + j * 256;
    if (i < n_vec) __builtin_nontemporal_store(r[j], &dst[i]);
  }
}
extern "C" int anc_copy_kernel(uint64_t dst, uint64_t src, int64_t n_bytes, uint64_t stream) {
  ANC_REQUIRE(dst != 0 && src != 0 && n_bytes > 0 && n_bytes % 16 == 0 && (dst & 15) == 0 &&
                  (src & 15) == 0,
              "anc_copy_kernel: pointers and size must be 16-byte aligned");
  int64_t n_vec = n_bytes / 16;
  int64_t blocks = (n_vec + 1023) / 1024;
  ANC_REQUIRE(blocks < (1ll << 31), "anc_copy_kernel: size too large");
  AncProfScope prof(ANC_PROF_COPY, anc_stream(stream));
  hipLaunchKernelGGL(k_copy16, dim3((unsigned)blocks), dim3(256), 0, anc_stream(stream),
                     (const anc_u32x4 *)src, (anc_u32x4 *)dst, n_vec);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}
