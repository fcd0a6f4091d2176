"""HIP device buffers: the persistent optimizer state lives in these.

One class replaces the reference's three raw-allocation wrappers — `adamw._Buf`
(ancora/optim/adamw.py:51-60), `loss._GpuArray` (ancora/kernels/loss.py:277-294) and
`resident._DBuf` (ancora/model/resident.py:52-94) — and `moe._View`
(ancora/kernels/moe.py:380-386), with the same methods: `zeros`, `view`, `at_pos`,
`to_numpy` / `numpy`, `upload`, `free`, and an integer device address in `.ptr`.
Views share the pointer and are never freed (ancora/model/resident.py:80).
bf16 data is held as uint16 bit patterns, as in the reference.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import api


class DevBuf:
    def __init__(self, arr=None, *, shape=None, dtype=None, ptr=None):
        """DevBuf(host_array) allocates and uploads; DevBuf(shape=, dtype=) allocates
        uninitialised memory; DevBuf(shape=, dtype=, ptr=) wraps memory owned elsewhere."""
        _lib.init()
        if arr is not None:
            arr = np.ascontiguousarray(arr)
            shape, dtype = arr.shape, arr.dtype
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        if self.nbytes <= 0:
            raise ValueError(f"DevBuf: empty shape {self.shape}")
        self._owner = ptr is None
        if ptr is None:
            p = C.c_uint64(0)
            api.anc_malloc(C.byref(p), self.nbytes)
            ptr = p.value
        self.ptr = int(ptr)
        if self.ptr == 0:
            raise _lib.AncoraError("DevBuf: null device pointer")
        if arr is not None:
            self.upload(arr)

    # same protocol dict the reference's buffers expose to its launcher
    @property
    def __cuda_array_interface__(self):
        return {"shape": self.shape, "typestr": self.dtype.str, "data": (self.ptr, False),
                "version": 3}

    @property
    def size(self):
        return self.nbytes // self.dtype.itemsize

    @classmethod
    def zeros(cls, shape, dtype=np.uint16, stream=0):
        b = cls(shape=shape, dtype=dtype)
        b.fill_zero(stream)
        return b

    @classmethod
    def empty(cls, shape, dtype):
        return cls(shape=shape, dtype=dtype)

    def fill_zero(self, stream=0):
        if self.nbytes % 4:
            raise ValueError("DevBuf.fill_zero: size must be a multiple of 4 bytes")
        api.anc_fill_u32(self.ptr, 0, self.nbytes // 4, int(stream))

    def view(self, shape, dtype=None):
        """Same memory under another declared shape (and dtype); must fit inside this buffer."""
        dtype = self.dtype if dtype is None else np.dtype(dtype)
        need = int(np.prod(shape, dtype=np.int64)) * dtype.itemsize
        if need > self.nbytes:
            raise ValueError(f"DevBuf.view: {shape} {dtype} needs {need} B, buffer has {self.nbytes} B")
        return DevBuf(shape=shape, dtype=dtype, ptr=self.ptr)

    def at_pos(self, rows):
        """View starting `rows` rows down a 2-D buffer (the packed-batch slice u.at_pos(i*M) of
        ancora/optim/muon.py:266)."""
        if len(self.shape) != 2 or not 0 <= rows < self.shape[0]:
            raise ValueError(f"DevBuf.at_pos({rows}) outside shape {self.shape}")
        off = rows * self.shape[1] * self.dtype.itemsize
        return DevBuf(shape=(self.shape[0] - rows, self.shape[1]), dtype=self.dtype,
                      ptr=self.ptr + off)

    def upload(self, arr, stream=0):
        arr = np.ascontiguousarray(arr)
        if arr.nbytes > self.nbytes:
            raise ValueError(f"DevBuf.upload: {arr.nbytes} B into a buffer of {self.nbytes} B")
        api.anc_memcpy_h2d(self.ptr, arr.ctypes.data_as(C.c_void_p), arr.nbytes, int(stream))

    def to_numpy(self, stream=0):
        out = np.empty(self.shape, self.dtype)
        api.anc_memcpy_d2h(out.ctypes.data_as(C.c_void_p), self.ptr, self.nbytes, int(stream))
        return out

    numpy = to_numpy

    def copy_from(self, other, stream=0):
        if other.nbytes > self.nbytes:
            raise ValueError("DevBuf.copy_from: source larger than destination")
        api.anc_memcpy_d2d(self.ptr, other.ptr, other.nbytes, int(stream))

    def free(self):
        if self._owner and self.ptr:
            api.anc_free(self.ptr)
        self.ptr = 0


def upload_table(structs):
    """Pack a list of ctypes structures into one device buffer (a descriptor table)."""
    n = len(structs)
    arr_t = type(structs[0]) * n
    host = arr_t(*structs)
    raw = np.frombuffer(bytes(host), dtype=np.uint8)
    pad = (-raw.size) % 4
    if pad:
        raw = np.concatenate([raw, np.zeros(pad, np.uint8)])
    return DevBuf(raw)
