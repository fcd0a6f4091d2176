"""Lab bench: what this board's memory system and matrix pipe give kernels shaped like the
optimizer's. Not part of the product library: `labbench.hip` is compiled on request into
dev/liblabbench.so and loaded here only.

    python3 -m ancora_cutile_amd.dev.labbench build
    python3 -m ancora_cutile_amd.dev.labbench copy [GiB] [reps]    nine streaming-kernel shapes, TB/s each
    python3 -m ancora_cutile_amd.dev.labbench mfma [launches]      register-only matrix-instruction loop on
                                      zero, constant and random operands, with the shader clock and
                                      package power sysfs reports while each runs
"""
import ctypes
import os
import subprocess
import sys
import threading
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "labbench.hip")
OUT = os.path.join(HERE, "liblabbench.so")


def build():
    from ..build import FLAGS
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    subprocess.run([hipcc, *FLAGS, SRC, "-o", OUT], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return OUT


def _load():
    if not os.path.exists(OUT):
        raise RuntimeError(f"{OUT} is not built: run `python3 -m ancora_cutile_amd.dev.labbench build` first")
    lab = ctypes.CDLL(OUT)
    lab.lab_copy_shape.argtypes = [ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int64, ctypes.c_int,
                                   ctypes.POINTER(ctypes.c_int64), ctypes.c_uint64]
    lab.lab_mfma_rate.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_uint64, ctypes.POINTER(ctypes.c_double),
                                  ctypes.c_uint64]
    return lab


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed with status {rc}")


def copy(gib=1.0, reps=5):
    from .. import DevBuf, _lib
    _lib.init(0)
    lab = _load()
    nb = int(gib * (1 << 30)) // (1 << 20) * (1 << 20)
    a, b = DevBuf.empty((nb // 4,), np.float32), DevBuf.empty((nb // 4,), np.float32)
    a.fill_zero(0)
    b.fill_zero(0)
    names = ("copy 4x16B nt", "copy 4x16B plain", "copy 8x16B nt", "copy persistent 2048 wg", "copy 1024-lane wg",
             "read only", "write only", "AdamW mix 4R+4W (14+14 B/elem)", "momentum mix 2R+3W (6+8 B/elem)")
    e0, e1 = _lib.Event(), _lib.Event()
    moved = ctypes.c_int64(0)
    print(f"two buffers of {nb / 2 ** 30:.2f} GiB, {reps} launches each, HIP events around the launches")
    for shape, name in enumerate(names):
        _check(lab.lab_copy_shape(b.ptr, a.ptr, nb, shape, ctypes.byref(moved), 0), "lab_copy_shape")
        e0.record(0)
        for _ in range(reps):
            _check(lab.lab_copy_shape(b.ptr, a.ptr, nb, shape, ctypes.byref(moved), 0), "lab_copy_shape")
        e1.record(0)
        e1.sync()
        ms = e0.elapsed_ms(e1) / reps
        print(f"  shape {shape}  {name:34s} {moved.value / 1e9:7.3f} GB in {ms * 1e3:8.1f} us = "
              f"{moved.value / ms / 1e9:6.3f} TB/s = {moved.value / ms / 1e9 / 8 * 100:5.1f} % of 8 TB/s")
    _lib.api.anc_device_sync()


def mfma(launches=12):
    from .. import DevBuf, _lib
    from ..sysfs import sclk_mhz as sclk, power_w
    _lib.init(0)
    lab = _load()
    sink = DevBuf.empty((1024,), np.float32)
    for name, values in (("zeros", 0), ("constant", 1), ("random", 2), ("zeros", 0), ("random", 2)):
        samples, watts, stop = [], [], threading.Event()

        def poll():
            time.sleep(0.5)
            while not stop.is_set():
                v, w = sclk(), power_w()
                if v:
                    samples.append(v)
                if w:
                    watts.append(w)
                time.sleep(0.02)

        th = threading.Thread(target=poll, daemon=True)
        th.start()
        fl = ctypes.c_double()
        rates = []
        for _ in range(launches):
            e0, e1 = _lib.Event(), _lib.Event()
            e0.record(0)
            _check(lab.lab_mfma_rate(values, 400000, sink.ptr, ctypes.byref(fl), 0), "lab_mfma_rate")
            e1.record(0)
            e1.sync()
            rates.append(fl.value / (e0.elapsed_ms(e1) * 1e-3) / 1e12)
        stop.set()
        th.join(timeout=15)
        busy = sorted(v for v in samples if v > 300)
        med = lambda xs: xs[len(xs) // 2] if xs else None       # noqa: E731
        print(f"{name:9s} first launch {rates[0]:7.1f}  last {rates[-1]:7.1f} TFLOP/s over {launches} launches; "
              f"sclk while running: median {med(busy)} MHz (min {busy[0] if busy else None}, max {busy[-1] if busy else None}, "
              f"{len(busy)} samples); package power median {med(sorted(watts))} W", flush=True)
    _lib.api.anc_device_sync()


def main(argv):
    if not argv or argv[0] == "build":
        print(build())
    elif argv[0] == "copy":
        copy(float(argv[1]) if len(argv) > 1 else 1.0, int(argv[2]) if len(argv) > 2 else 5)
    elif argv[0] == "mfma":
        mfma(int(argv[1]) if len(argv) > 1 else 12)
    else:
        raise SystemExit(__doc__)


if __name__ == "__main__":
    main(sys.argv[1:])
