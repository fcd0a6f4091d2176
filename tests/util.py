"""Shared helpers of the parity tests."""
import numpy as np


def ulp_diff(a, b):
    """Element-wise distance in units in the last place between two fp32 arrays."""
    a = np.ascontiguousarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    b = np.ascontiguousarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, np.int64(-2147483648) - a, a)
    b = np.where(b < 0, np.int64(-2147483648) - b, b)
    return np.abs(a - b)


def max_ulp(a, b):
    d = ulp_diff(a, b)
    return int(d.max()) if d.size else 0


def bits_equal(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and bool(np.array_equal(a.view(np.uint8), b.view(np.uint8)))


def rel_fro(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / (np.linalg.norm(b) + 1e-300))


def bf16_grad(rng, shape, std=1e-3):
    """bf16 gradient ~N(0, std) as uint16 bit patterns, plus its fp32 value."""
    from oracle.bf16_ref import bf16_rne_bits, bits_to_f32
    g = (rng.standard_normal(shape) * std).astype(np.float32)
    bits = bf16_rne_bits(g)
    return bits, bits_to_f32(bits).reshape(shape)


class StubMoELayer:
    """What `GroupedMoEFFN` carries when its optimizer methods run: masters in `w`, packed bf16
    forward weights and their transposes, fp32 gradient buffers, router buffers."""

    def __init__(self, E, H, rng, optimizer, device_route):
        from ancora_cutile_amd import DevBuf
        from ancora_cutile_amd.bf16 import bf16_bits
        self.E, self.H, self.Ie, self.optimizer, self.device_route = E, H, H, optimizer, device_route
        self.w = {k: (0.02 * rng.standard_normal((E, H, H))).astype(np.float32)
                  for k in ("gate_proj", "up_proj", "down_proj")}
        self.w["router"] = (0.02 * rng.standard_normal((H, E))).astype(np.float32)
        for attr, key in (("Wg", "gate_proj"), ("Wu", "up_proj"), ("Wd", "down_proj")):
            setattr(self, attr, DevBuf(bf16_bits(self.w[key]).reshape(E * H, H)))
            setattr(self, attr + "T", DevBuf.zeros((E * H, H), np.uint16))
            setattr(self, "d" + attr, DevBuf.zeros((E * H, H), np.float32))
        self.Wr_dev = DevBuf(self.w["router"].reshape(-1))
        self.G_router_dev = DevBuf.zeros((H * E,), np.float32)
        self.Gr_acc = DevBuf.zeros((H * E,), np.float32)
        self.G_router = np.zeros((H, E), np.float32)
        self._muon_lr = 0.02
