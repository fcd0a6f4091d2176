"""ctypes binding of libancora_optim.so (the C ABI declared in include/anc_optim.h).

The reference launches its cuda-tile kernels with `ct.launch(stream, grid, kernel, args)`
and talks to the driver through `cuda.bindings` (ancora/optim/adamw.py:51-60,94-97).
Here every kernel sits behind one C entry point; this module loads the library, declares
the prototypes and turns non-zero status codes into exceptions. There is no fallback:
if the library is missing or is not usable, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# ANCORA_OPTIM_LIB names another build of the same library (an ablation variant, see build.py)
LIB_PATH = os.environ.get("ANCORA_OPTIM_LIB") or os.path.join(_HERE, "csrc", "libancora_optim.so")

F32, BF16 = 0, 1                  # ANC_F32 / ANC_BF16
FORM_DIV, FORM_IBC = 0, 1         # ANC_ADAMW_FORM_*
NS_BF16, NS_FP32, NS_BF16_FAST, NS_BF16_X3, NS_BF16_LATE3 = 0, 1, 2, 3, 4   # ANC_NS_*
GN_CHUNK = 8192                   # ANC_GN_CHUNK
MUON_MAX_SCALES = 8               # ANC_MUON_MAX_SCALES
SR_ON, SR_STEP_SEED, SR_SEED_STRIDE = 1, 2, 1000003   # ANC_SR_*
ABI_VERSION = 3                   # the anc_abi_version() these prototypes were written for

u64, i64, i32, u32, f32 = C.c_uint64, C.c_int64, C.c_int32, C.c_uint32, C.c_float


class AncoraError(RuntimeError):
    """A libancora_optim.so call returned a non-zero status."""


class DeviceInfo(C.Structure):
    _fields_ = [("cu_count", i32), ("clock_khz", i32), ("mem_clock_khz", i32),
                ("mem_bus_bits", i32), ("wavefront", i32), ("lds_bytes_per_block", i32),
                ("hbm_bytes", i64), ("l2_bytes", i64), ("name", C.c_char * 64),
                ("arch", C.c_char * 64)]


class StepCtl(C.Structure):
    _fields_ = [("sumsq", C.c_double), ("norm", f32), ("clip_scale", f32), ("skip", u32),
                ("t", u32), ("reserved", u32 * 2)]


class AdamWHyper(C.Structure):
    _fields_ = [("beta1", f32), ("beta2", f32), ("omb1", f32), ("omb2", f32), ("eps", f32),
                ("lr", f32), ("bc1", f32), ("bc2", f32), ("form", i32), ("sr", i32),
                ("seed_base", u32), ("step_cap", i32), ("step_table", u64)]


class AdamWStepEntry(C.Structure):
    """anc_adamw_step_t: the scalars of one counted step."""
    _fields_ = [("bc1", f32), ("bc2", f32), ("lr", f32), ("seed_base", u32)]


class AdamWDesc(C.Structure):
    _fields_ = [("g", u64), ("m", u64), ("v", u64), ("p32", u64), ("p16", u64), ("n", i64),
                ("blk0", i64), ("wd", f32), ("seed", u32), ("g_dtype", i32), ("pad", i32)]


class GnDesc(C.Structure):
    _fields_ = [("g", u64), ("n", i64), ("chunk0", i64), ("part0", i64), ("dtype", i32),
                ("pad", i32)]


class MuonDesc(C.Structure):
    _fields_ = [("buf", u64), ("g", u64), ("p32", u64), ("p16", u64), ("u", u64), ("K", i32),
                ("N", i32), ("transpose", i32), ("g_dtype", i32), ("scale_idx", i32),
                ("seed", u32), ("tile0", i64), ("p16t", u64)]


class NsProblem(C.Structure):
    """anc_ns_problem_t: one batch of the multi-batch chain entry."""
    _fields_ = [("Uh", u64), ("Ul", u64), ("fro_partials", u64), ("X32_out", u64), ("workspace", u64),
                ("n_partials", i64), ("E", i64), ("M", i64), ("N", i64), ("workspace_bytes", i64)]


class DwProblem(C.Structure):
    """anc_dw_problem_t: one weight of the weight-gradient GEMM call."""
    _fields_ = [("xT", u64), ("dy", u64), ("dW", u64), ("g16", u64), ("workspace", u64),
                ("T", i64), ("K", i64), ("N", i64), ("workspace_bytes", i64),
                ("accumulate", i32), ("segments", i32), ("gn_partials", u64),
                ("x_row_major", i32), ("reserved", i32)]


# name -> (restype, argtypes); restype None means "int status, checked".
_PROTOS = {
    "anc_last_error": (C.c_char_p, []),
    "anc_abi_version": (C.c_int, []),
    "anc_init": (None, [C.c_int]),
    "anc_device_info": (None, [C.POINTER(DeviceInfo)]),
    "anc_malloc": (None, [C.POINTER(u64), i64]),
    "anc_free": (None, [u64]),
    "anc_host_alloc": (None, [C.POINTER(C.c_void_p), i64]),
    "anc_host_free": (None, [C.c_void_p]),
    "anc_mem_info": (None, [C.POINTER(i64), C.POINTER(i64)]),
    "anc_fill_u32": (None, [u64, u32, i64, u64]),
    "anc_memcpy_h2d": (None, [u64, C.c_void_p, i64, u64]),
    "anc_memcpy_d2h": (None, [C.c_void_p, u64, i64, u64]),
    "anc_memcpy_d2d": (None, [u64, u64, i64, u64]),
    "anc_stream_create": (None, [C.POINTER(u64)]),
    "anc_stream_destroy": (None, [u64]),
    "anc_stream_sync": (None, [u64]),
    "anc_device_sync": (None, []),
    "anc_event_create": (None, [C.POINTER(u64)]),
    "anc_event_destroy": (None, [u64]),
    "anc_event_record": (None, [u64, u64]),
    "anc_event_sync": (None, [u64]),
    "anc_stream_wait_event": (None, [u64, u64]),
    "anc_event_elapsed_ms": (None, [u64, u64, C.POINTER(f32)]),
    "anc_copy_kernel": (None, [u64, u64, i64, u64]),
    "anc_profile_enable": (None, [C.c_int]),
    "anc_profile_read": (None, [C.POINTER(f32), C.POINTER(i64)]),
    "anc_gradnorm_num_partials": (i64, [i64]),
    "anc_gradnorm_partials": (None, [u64, i64, C.c_int, u64, i64, u64]),
    "anc_gradnorm_partials_multi": (None, [u64, i32, i64, u64, u64]),
    "anc_gradnorm_finalize": (None, [u64, i64, f32, f32, i32, u64, u64]),
    "anc_gradnorm_static_max_elements": (i64, []),
    "anc_gradnorm_static": (None, [u64, i64, C.c_int, f32, f32, u64, u64]),
    "anc_adamw": (None, [u64, u64, u64, u64, u64, i64, C.c_int, C.POINTER(AdamWHyper), f32, u32,
                         u64, u64]),
    "anc_adamw_num_blocks": (i64, [i64]),
    "anc_adamw_multi": (None, [u64, i32, i64, C.POINTER(AdamWHyper), u64, u64]),
    "anc_adamw_rows": (None, [u64, i64, u64, u64, u64, u64, u64, u64, i64, i64, u64, i32,
                              C.POINTER(AdamWHyper), f32, u32, u64, u64]),
    "anc_embed_dw_scatter": (None, [u64, u64, u64, u64, u64, u64, u64, i64, i64, i64, u64]),
    "anc_cast_bf16": (None, [u64, u64, i64, C.c_int, u32, u64]),
    "anc_muon_momentum": (None, [u64, u64, u64, i64, i64, f32, C.c_int, C.c_int, C.c_int,
                                 C.c_int, u64, u64]),
    "anc_muon_update": (None, [u64, u64, u64, i64, i64, f32, C.c_int, C.c_int, C.c_int, u32, u64,
                               u64]),
    "anc_muon_momentum_multi": (None, [u64, i32, i64, f32, C.c_int, C.c_int, u64, u64]),
    "anc_muon_momentum_multi_pair": (None, [u64, i32, i64, f32, C.c_int, u64, i64, u64, u64, u64]),
    "anc_muon_update_multi": (None, [u64, i32, i64, C.POINTER(f32), C.c_int, C.c_int, u32, u64,
                                     u64]),
    "anc_transpose_bf16": (None, [u64, u64, i64, i64, i64, u64]),
    "anc_quant_mxfp8_w": (None, [u64, u64, u64, i64, i64, i64, C.c_int, u64]),
    "anc_gemm_dw_workspace_bytes": (i64, [i64, i64, i64]),
    "anc_gemm_dw_multi": (None, [C.POINTER(DwProblem), i32, u64]),
    "anc_gemm_dw_info": (None, [i64, i64, i64, C.POINTER(C.c_double), C.POINTER(i32)]),
    "anc_ns_workspace_bytes": (i64, [i64, i64, i64, C.c_int]),
    "anc_ns_batched": (None, [u64, i64, i64, i64, C.c_int, C.POINTER(f32), f32, C.c_int, u64, i64,
                              u64]),
    "anc_ns_batched_pair": (None, [u64, u64, u64, i64, u64, i64, i64, i64, C.c_int, C.POINTER(f32), f32,
                                   C.c_int, u64, i64, u64]),
    "anc_ns_batched_pair_multi": (None, [C.POINTER(NsProblem), i32, C.c_int, C.POINTER(f32), f32, C.c_int,
                                         u64]),
    "anc_muon_ns_update_multi": (None, [C.POINTER(NsProblem), i32, C.POINTER(u64), C.c_int, C.POINTER(f32), f32,
                                        C.c_int, C.POINTER(f32), C.c_int, u32, u64, u64]),
    "anc_ns_flops": (None, [i64, i64, i64, C.c_int, C.c_int, C.POINTER(C.c_double),
                            C.POINTER(C.c_double)]),
    "anc_ns_hard_info": (None, [u64, i64, i64, i64, C.c_int, C.c_int, C.POINTER(i32), C.POINTER(C.c_double), u64]),
    "anc_ns_product_flops": (None, [i64, i64, i64, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double)]),
    "anc_bf16_to_f32": (None, [u64, u64, i64, u64]),
    "anc_f32_to_bf16": (None, [u64, u64, i64, u64]),
}

EXPORTS = tuple(_PROTOS)

_lib = None
_initialised = False


def _checked(fn, name):
    def call(*args):
        rc = fn(*args)
        if rc != 0:
            msg = _lib.anc_last_error().decode("utf-8", "replace")
            raise AncoraError(f"{name} failed (status {rc}): {msg}")
    call.__name__ = name
    return call


class _Api:
    """Namespace of checked entry points: `api.anc_adamw(...)` raises on error."""


api = _Api()


def load(path=None):
    """Load the shared library and bind every prototype. Raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise AncoraError(
            f"{p} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()' "
            "or python -m ancora_cutile_amd.build). There is no CPU fallback for the optimizer step.")
    lib = C.CDLL(p)
    for name, (restype, argtypes) in _PROTOS.items():
        fn = getattr(lib, name)          # AttributeError if the export is missing
        fn.argtypes = argtypes
        fn.restype = C.c_int if restype is None else restype
        setattr(api, name, _checked(fn, name) if restype is None else fn)
    got = lib.anc_abi_version()
    if got != ABI_VERSION:
        raise AncoraError(f"{p} has ABI version {got}, this binding was written for {ABI_VERSION}: "
                          "rebuild the library (python -m ancora_cutile_amd.build)")
    _lib = lib
    return lib


def init(device=0):
    """Select the GPU (gfx950 only). Called lazily by the first device allocation."""
    global _initialised
    load()
    if not _initialised:
        api.anc_init(int(device))
        _initialised = True


def device_info():
    init()
    info = DeviceInfo()
    api.anc_device_info(C.byref(info))
    return {"cu_count": info.cu_count, "clock_khz": info.clock_khz,
            "mem_clock_khz": info.mem_clock_khz, "mem_bus_bits": info.mem_bus_bits,
            "wavefront": info.wavefront, "lds_bytes_per_block": info.lds_bytes_per_block,
            "hbm_bytes": info.hbm_bytes, "l2_bytes": info.l2_bytes,
            "name": info.name.decode(), "arch": info.arch.decode()}


def stream_create():
    init()
    s = u64(0)
    api.anc_stream_create(C.byref(s))
    return int(s.value)


def stream_sync(stream=0):
    api.anc_stream_sync(int(stream))


PROF_KINDS = ("adamw", "gradnorm_partials", "gradnorm_finalize", "muon_momentum", "muon_update",
              "ns_fro", "ns_prep", "ns_gemm_gram", "ns_gemm_bmat", "ns_gemm_bx", "ns_gemm_f32",
              "misc", "copy", "ns_gemm_bx_update", "dw_gemm", "dw_reduce")


def profile_enable(on=True):
    init()
    api.anc_profile_enable(int(bool(on)))


def profile_read():
    """{kind: (milliseconds, launches)} since the last read; synchronises the device."""
    n = len(PROF_KINDS)
    ms = (f32 * n)()
    cnt = (i64 * n)()
    api.anc_profile_read(ms, cnt)
    return {k: (float(ms[i]), int(cnt[i])) for i, k in enumerate(PROF_KINDS)}


class Event:
    """HIP event on a stream: the timing primitive of the benchmarks."""

    def __init__(self):
        init()
        e = u64(0)
        api.anc_event_create(C.byref(e))
        self.h = int(e.value)

    def record(self, stream=0):
        api.anc_event_record(self.h, int(stream))

    def sync(self):
        api.anc_event_sync(self.h)

    def wait_on(self, stream):
        """Make `stream` wait for this event."""
        api.anc_stream_wait_event(int(stream), self.h)

    def elapsed_ms(self, later):
        ms = f32(0)
        api.anc_event_elapsed_ms(self.h, later.h, C.byref(ms))
        return float(ms.value)

    def free(self):
        if self.h:
            api.anc_event_destroy(self.h)
            self.h = 0
