"""Position encodings as parts.  A mixer is handed one and asks it for what its kernels need.

RotaryHalfSplit: f_i = theta^(-2i/rotary_dim), angle = position * f_i, all in 32-bit; the pair
(d, d + rotary_dim/2) is rotated by the angle of d; dims above rotary_dim pass through.
Tables as crates/synaptix-ops/src/pos/rope_cache.rs:16-38 builds them, rotation as
crates/synaptix-ops/src/pos/rope.rs:81-97 (Split layout).
"""
from __future__ import annotations

import numpy as np
import torch

from .base import Part


class Position(Part):
    def tables(self, device):
        """(cos, sin) float [capacity, rotary_dim / 2] on `device`, or (None, None) for no rotation."""
        return None, None

    def score_slopes(self, n_heads: int, device):
        """A scheme that acts on the attention scores instead of on q and k: float [n_heads] on `device`, the
        score of query position p and key position j <= p then gets - slope[head] * (p - j) (the linear bias of
        crates/synaptix-ops/src/pos/alibi.rs:47-66); None (the default): nothing is added."""
        return None

    def score_log_bias(self, n_heads: int, device):
        """A scheme whose term on the scores grows with the logarithm of the distance: (r1, r2), float [n_heads] each
        on `device`, for - r1[head] * ln(1 + r2[head] * (p - j)); None (the default): nothing is added."""
        return None

    capacity = None  # positions at and beyond it cannot be encoded; None: no limit
    # which values a rotation pairs: "halves" (value i with value i + rotary_dim / 2) or "pairs" (value 2i with 2i + 1)
    pairing = "halves"


class NoPosition(Position):
    pass


class RotaryHalfSplit(Position):
    def __init__(self, theta: float, rotary_dim: int, capacity: int):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise ValueError(f"rotary_dim {rotary_dim} must be positive and even")
        if capacity <= 0:
            raise ValueError("capacity must be positive")
        self.theta = float(np.float32(theta))
        self.rotary_dim = rotary_dim
        self.capacity = capacity
        self._tables = {}

    def host_tables(self):
        half = self.rotary_dim // 2
        i = np.arange(half, dtype=np.float32)
        expo = -(np.float32(2.0) * i) / np.float32(self.rotary_dim)
        freqs = np.power(np.float32(self.theta), expo).astype(np.float32)
        t = np.arange(self.capacity, dtype=np.float32)
        ang = (t[:, None] * freqs[None, :]).astype(np.float32)
        return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)

    def tables(self, device):
        key = str(device)
        if key not in self._tables:
            cos, sin = self.host_tables()
            self._tables[key] = (torch.from_numpy(cos).to(device), torch.from_numpy(sin).to(device))
        return self._tables[key]


class LogDistanceBias(Position):
    """No rotation; the score of query position i and key position j <= i gets  - r1[h] * ln(1 + r2[h] * (i - j)),
    with one pair of numbers a head, read from the tensors `prefix + r1_name` and `prefix + r2_name` ([n_heads])."""
    capturable = True

    def __init__(self, prefix: str, n_heads: int, r1_name: str = "r1", r2_name: str = "r2"):
        self.n_heads = n_heads
        self.r1_name, self.r2_name = prefix + r1_name, prefix + r2_name
        self.r1 = self.r2 = None

    def tensor_specs(self):
        from ..weights.source import TensorSpec
        return {self.r1_name: TensorSpec((self.n_heads,), "positive"), self.r2_name: TensorSpec((self.n_heads,), "positive")}

    def load(self, get):
        self.r1 = get(self.r1_name).float().contiguous()
        self.r2 = get(self.r2_name).float().contiguous()

    def score_log_bias(self, n_heads: int, device):
        """(r1, r2) float [n_heads] on the device."""
        if n_heads != self.n_heads:
            raise ValueError(f"a distance bias for {self.n_heads} heads was asked for {n_heads}")
        return self.r1, self.r2


class RotaryInterleaved(Position):
    """A rotation of the pairs (2i, 2i + 1), i < dims / 2, of a vector's first `dims` values by the angle
    t_i = position * base^(-2i / dims), as a complex multiplication (x_2i + j x_2i+1) e^(j t_i); what lies behind `dims`
    passes unchanged.  Tables [capacity, dims / 2] are made on the host with 64-bit angles and kept in 32-bit, once for
    all parts with the same constants."""
    capturable = True
    pairing = "pairs"
    _shared: dict = {}

    def __init__(self, base: float, dims: int, capacity: int):
        if dims < 0 or dims % 2:
            raise ValueError(f"rotated dims {dims} must be even and not negative")
        if capacity <= 0:
            raise ValueError("capacity must be positive")
        self.base, self.dims, self.capacity = float(base), int(dims), int(capacity)

    def host_tables(self):
        half = self.dims // 2
        freqs = np.power(np.float64(self.base), -2.0 * np.arange(half, dtype=np.float64) / max(self.dims, 1))
        ang = np.arange(self.capacity, dtype=np.float64)[:, None] * freqs[None, :]
        return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)

    def tables(self, device):
        if self.dims == 0:
            return None, None
        key = (self.base, self.dims, self.capacity, str(device))
        if key not in self._shared:
            cos, sin = self.host_tables()
            self._shared[key] = (torch.from_numpy(cos).to(device), torch.from_numpy(sin).to(device))
        return self._shared[key]


class RotaryScaledHalfSplit(Position):
    """The half-split rotation (value i < dims / 2 paired with value i + dims / 2, the rest passes) whose long waves are
    stretched for contexts beyond the one the rates were made for.  With f_i = base^(-2i / dims) and, for a number of
    turns t over the `original` context, place(t) = dims ln(original / (2 pi t)) / (2 ln base):

        lo = max(floor(place(fast)), 0);  hi = min(ceil(place(slow)), dims - 1)
        ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
        rate_i = f_i / factor * ramp_i + f_i * (1 - ramp_i)

    and cos and sin both carry the factor 0.1 ln(factor) + 1.  factor None: the plain rates, no factor on cos and sin.
    Angles are position * rate in 32-bit; tables [capacity, dims / 2], kept once for equal constants."""
    capturable = True
    _shared: dict = {}

    def __init__(self, base: float, dims: int, capacity: int, factor: float | None = None, original: float | None = None,
                 fast: float | None = None, slow: float | None = None):
        if dims < 0 or dims % 2:
            raise ValueError(f"rotated dims {dims} must be even and not negative")
        if capacity <= 0:
            raise ValueError("capacity must be positive")
        if factor is not None and (original is None or fast is None or slow is None or not factor > 0.0):
            raise ValueError("a scaled rotation needs factor, original, fast and slow")
        self.base, self.dims, self.capacity = float(base), int(dims), int(capacity)
        self.factor, self.original, self.fast, self.slow = factor, original, fast, slow

    def rates(self):
        """(rate_i as float64 [dims / 2], the factor on cos and sin)."""
        import math
        half = self.dims // 2
        i = np.arange(half, dtype=np.float64)
        f = np.power(np.float64(self.base), -2.0 * i / max(self.dims, 1))
        if self.factor is None:
            return f, 1.0

        def place(turns):
            return self.dims * math.log(self.original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))

        lo, hi = max(math.floor(place(self.fast)), 0), min(math.ceil(place(self.slow)), self.dims - 1)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / self.factor * ramp + f * (1.0 - ramp), 0.1 * math.log(self.factor) + 1.0

    def host_tables(self):
        rates, mult = self.rates()
        ang = np.arange(self.capacity, dtype=np.float32)[:, None] * rates.astype(np.float32)[None, :]
        ang = ang.astype(np.float64)           # (the 32-bit angle itself, its cosine and sine taken exactly)
        return (np.cos(ang) * mult).astype(np.float32), (np.sin(ang) * mult).astype(np.float32)

    def tables(self, device):
        if self.dims == 0:
            return None, None
        key = (self.base, self.dims, self.capacity, self.factor, self.original, self.fast, self.slow, str(device))
        if key not in self._shared:
            cos, sin = self.host_tables()
            self._shared[key] = (torch.from_numpy(cos).to(device), torch.from_numpy(sin).to(device))
        return self._shared[key]


class RotaryByWavelength(Position):
    """A rotation of the first `dims` values whose rates depend on their wavelength, for contexts beyond the `original`
    one that the plain rates f_i = base^(-2i / dims) were made for.  With the wavelength l_i = 2 pi / f_i:

        l_i < original / high:   rate_i = f_i                       (fast waves stay)
        l_i > original / low:    rate_i = f_i / factor              (slow waves are stretched)
        else:                    s = (original / l_i - low) / (high - low);  rate_i = (1 - s) f_i / factor + s f_i

    factor None: the plain rates.  pairing "halves" (value i with i + dims / 2) or "pairs" (2i with 2i + 1); the mixer
    that takes the tables asks for it.  Tables [capacity, dims / 2] from 64-bit angles, kept in 32-bit, once for all parts
    with the same constants."""
    capturable = True
    _shared: dict = {}

    def __init__(self, base: float, dims: int, capacity: int, factor: float | None = None, low: float | None = None,
                 high: float | None = None, original: float | None = None, pairing: str = "halves"):
        if dims < 0 or dims % 2:
            raise ValueError(f"rotated dims {dims} must be even and not negative")
        if capacity <= 0:
            raise ValueError("capacity must be positive")
        if pairing not in ("halves", "pairs"):
            raise ValueError(f"pairing {pairing!r} ('halves' or 'pairs')")
        if factor is not None and (low is None or high is None or original is None or not factor > 0.0 or not high > low):
            raise ValueError("stretched rates need factor, low < high and original")
        self.base, self.dims, self.capacity, self.pairing = float(base), int(dims), int(capacity), pairing
        self.factor, self.low, self.high, self.original = factor, low, high, original

    def rates(self):
        """rate_i as float64 [dims / 2]."""
        import math
        f = np.power(np.float64(self.base), -2.0 * np.arange(self.dims // 2, dtype=np.float64) / max(self.dims, 1))
        if self.factor is None:
            return f
        wave = 2.0 * math.pi / f
        s = (self.original / wave - self.low) / (self.high - self.low)
        blend = (1.0 - s) * f / self.factor + s * f
        return np.where(wave < self.original / self.high, f, np.where(wave > self.original / self.low, f / self.factor, blend))

    def host_tables(self):
        ang = np.arange(self.capacity, dtype=np.float64)[:, None] * self.rates()[None, :]
        return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)

    def tables(self, device):
        if self.dims == 0:
            return None, None
        key = (self.base, self.dims, self.capacity, self.factor, self.low, self.high, self.original, str(device))
        if key not in self._shared:
            cos, sin = self.host_tables()
            self._shared[key] = (torch.from_numpy(cos).to(device), torch.from_numpy(sin).to(device))
        return self._shared[key]
