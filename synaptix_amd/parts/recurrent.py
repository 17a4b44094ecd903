"""Mixers whose memory of a sequence is a matrix for each head that is updated token by token, behind a short causal
convolution (csrc/recurrent.hip has the equations).

StateSpaceMixer: one fused projection [z | x | B | C | dt]; x, B and C pass the convolution and silu; per head a scalar
decay from the step size, S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x; y silu(z) is normed in equal parts and
multiplied by a gain; then the output product.

ChannelDeltaMixer: q, k, v pass convolutions of their own and silu; q and k become unit vectors; the state decays with a
rate for every (head, key channel), made by a product through a narrow middle, and is corrected by the delta rule with
a step sigmoid(W_b h); each head's read-out is divided by its root mean square, times a gain, times the sigmoid of a
gate that is also made through a narrow middle; then the output product.

Step sizes, decays, gates, unit norms, states and everything between the projections and the output product are 32-bit
in both engine types.  A sequence's state (the matrix, and the convolution's last inputs) starts at zero when its slot
is taken and is carried from step to step.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import StateNeed
from .linear import linear, linear_for_sum
from .mixer import Mixer, _projection


def conv_state_need(taps: int, channels: int) -> StateNeed:
    """What a short convolution keeps of a sequence: its last taps - 1 inputs."""
    return StateNeed((max(taps - 1, 0), channels))


class StateSpaceMixer(Mixer):
    takes_scaled_rows = False
    capturable = True

    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D",
             "norm": "norm", "o": "o"}

    def __init__(self, prefix: str, hidden: int, n_heads: int, vdim: int, n_state: int, n_groups: int, taps: int, *,
                 norm_groups: int = 1, norm_eps: float, names: dict | None = None):
        if n_groups <= 0 or n_heads % n_groups:
            raise ValueError(f"{prefix}: {n_heads} heads do not divide into {n_groups} groups")
        inner = n_heads * vdim
        if norm_groups <= 0 or inner % norm_groups:
            raise ValueError(f"{prefix}: {inner} values do not divide into {norm_groups} normed parts")
        self.prefix, self.hidden = prefix, hidden
        self.nh, self.vdim, self.ns, self.ng, self.taps = n_heads, vdim, n_state, n_groups, taps
        self.inner, self.norm_groups, self.norm_eps = inner, norm_groups, float(norm_eps)
        self.channels = inner + 2 * n_groups * n_state
        self.names = dict(self.NAMES, **(names or {}))
        self.w_in = self.w_o = self.conv = self.conv_bias = self.dt_bias = self.a_log = self.d = self.gain = None

    def _n(self, key):
        return self.prefix + self.names[key]

    def tensor_specs(self):
        return {self._n("in"): TensorSpec((self.inner + self.channels + self.nh, self.hidden)),
                self._n("conv"): TensorSpec((self.channels, self.taps), "filter"),
                self._n("conv_bias"): TensorSpec((self.channels,), "bias"),
                self._n("dt_bias"): TensorSpec((self.nh,), "bias"),
                self._n("a_log"): TensorSpec((self.nh,), "rate"),
                self._n("d"): TensorSpec((self.nh,), "gain"),
                self._n("norm"): TensorSpec((self.inner,), "gain"),
                self._n("o"): TensorSpec((self.hidden, self.inner))}

    def load(self, get):
        self.w_in = _projection(get(self._n("in")))
        self.w_o = _projection(get(self._n("o")))
        for attr, key in (("conv", "conv"), ("conv_bias", "conv_bias"), ("dt_bias", "dt_bias"), ("a_log", "a_log"),
                          ("d", "d"), ("gain", "norm")):
            setattr(self, attr, get(self._n(key)).float().contiguous())      # small: kept in 32-bit

    def cache_need(self):
        return (conv_state_need(self.taps, self.channels), StateNeed((self.nh, self.ns, self.vdim)))

    def check(self, dtype):
        if self.ns > ops.SCAN_MAX_ROWS or not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"{self.prefix}: a state of {self.ns} rows (at most {ops.SCAN_MAX_ROWS}), {self.taps} taps "
                             f"(at most {ops.SHORT_CONV_MAX_TAPS})")

    def forward(self, h, ctx, cache, owner=True):
        N, inner = h.shape[0], self.inner
        conv_state, cell = cache
        proj = linear(h, self.w_in, torch.float32)          # [N, z | x, B, C | dt] float
        xbc = torch.empty((N, self.channels), dtype=torch.float32, device=h.device)
        ops.short_conv(proj[:, inner:inner + self.channels], self.conv, self.conv_bias, conv_state.state, ctx.tok_seq,
                       ctx.tok_pos, ctx.seq_start, ctx.seq_past, ctx.seq_slot, xbc, silu=True)
        y = torch.empty((N, inner), dtype=torch.float32, device=h.device)
        ops.state_space_scan(xbc, proj[:, inner + self.channels:], self.dt_bias, self.a_log, self.d, cell.state,
                             ctx.seq_start, ctx.seq_slot, y, self.nh, self.vdim, self.ns, self.ng,
                             single_tokens=ctx.one_token_each)
        o = torch.empty((N, inner), dtype=h.dtype, device=h.device)
        ops.head_norm_gate(y, self.gain, self.norm_eps, proj[:, :inner], o, self.norm_groups, inner // self.norm_groups,
                           silu_first=True)
        return linear_for_sum(o, self.w_o)


class ChannelDeltaMixer(Mixer):
    takes_scaled_rows = False
    capturable = True

    NAMES = {"q": "q", "k": "k", "v": "v", "conv": ".conv", "b": "b", "a1": "a1", "a2": "a2", "a_bias": "dt_bias",
             "a_log": "A_log", "g1": "g1", "g2": "g2", "norm": "norm", "o": "o"}
    UNIT_EPS = 1e-6       # inside the root of the unit norm of q and k

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_key_heads: int, dim: int, vdim: int, taps: int, *,
                 norm_eps: float, q_scale: float | None = None, names: dict | None = None):
        if n_key_heads <= 0 or n_heads % n_key_heads:
            raise ValueError(f"{prefix}: {n_heads} heads do not divide into {n_key_heads} key heads")
        self.prefix, self.hidden = prefix, hidden
        self.nh, self.nk, self.dim, self.vdim, self.taps = n_heads, n_key_heads, dim, vdim, taps
        self.norm_eps = float(norm_eps)
        self.q_scale = float(q_scale) if q_scale is not None else dim ** -0.5
        self.channels = 2 * n_key_heads * dim + n_heads * vdim
        self.names = dict(self.NAMES, **(names or {}))
        self.rank_a = self.rank_g = None          # the narrow middles' sizes: None until set_ranks or load names them
        self.w_in = self.w_mid = self.w_o = self.conv = self.a_bias = self.a_log = self.gain = None

    def _n(self, key):
        return self.prefix + self.names[key]

    def _qkv(self):
        return [("q", self.nk * self.dim), ("k", self.nk * self.dim), ("v", self.nh * self.vdim)]

    def tensor_specs(self):
        ra, rg = self.rank_a, self.rank_g       # None: any size, which the stored tensors then decide
        specs = {}
        for k, n in self._qkv():
            specs[self._n(k)] = TensorSpec((n, self.hidden))
            specs[self._n(k) + self.names["conv"]] = TensorSpec((n, self.taps), "filter")
        specs.update({self._n("b"): TensorSpec((self.nh, self.hidden)),
                      self._n("a1"): TensorSpec((ra, self.hidden)), self._n("a2"): TensorSpec((self.nh * self.dim, ra)),
                      self._n("a_bias"): TensorSpec((self.nh * self.dim,), "bias"),
                      self._n("a_log"): TensorSpec((self.nh,), "rate"),
                      self._n("g1"): TensorSpec((rg, self.hidden)), self._n("g2"): TensorSpec((self.nh * self.vdim, rg)),
                      self._n("norm"): TensorSpec((self.vdim,), "gain"),
                      self._n("o"): TensorSpec((self.hidden, self.nh * self.vdim))})
        return specs

    def set_ranks(self, rank_a: int, rank_g: int):
        """The sizes of the two narrow middles (the decays' and the gate's).  Stored tensors bring them in their shapes
        (the specs then leave those sizes open); random weights need them named."""
        self.rank_a, self.rank_g = int(rank_a), int(rank_g)

    def load(self, get):
        a1, g1 = get(self._n("a1")), get(self._n("g1"))
        a2, g2 = get(self._n("a2")), get(self._n("g2"))
        if a2.shape[1] != a1.shape[0] or g2.shape[1] != g1.shape[0]:
            raise ValueError(f"{self.prefix}: the narrow middles of {a1.shape[0]} and {g1.shape[0]} values meet matrices for "
                             f"{a2.shape[1]} and {g2.shape[1]}")
        self.rank_a, self.rank_g = a1.shape[0], g1.shape[0]
        # one product for q, k, v and the step, one for the two narrow middles (their rows are rounded to the
        # activation type, as the input of the products that follow), and one for what comes out of the middles:
        # [a2 0; 0 g2] over [a1 | g1]
        self.w_in = _projection(torch.cat([get(self._n(k)) for k, _ in self._qkv()] + [get(self._n("b"))], 0))
        self.w_mid = _projection(torch.cat([a1, g1], 0))
        wide = torch.zeros((a2.shape[0] + g2.shape[0], self.rank_a + self.rank_g), dtype=a2.dtype, device=a2.device)
        wide[:a2.shape[0], :self.rank_a] = a2
        wide[a2.shape[0]:, self.rank_a:] = g2
        self.w_wide = _projection(wide)
        self.w_o = _projection(get(self._n("o")))
        self.conv = torch.cat([get(self._n(k) + self.names["conv"]) for k, _ in self._qkv()], 0).float().contiguous()
        self.a_bias = get(self._n("a_bias")).float().contiguous()
        self.a_log = get(self._n("a_log")).float().contiguous()
        self.gain = get(self._n("norm")).float().repeat(self.nh).contiguous()        # one gain for all heads

    def cache_need(self):
        return (conv_state_need(self.taps, self.channels), StateNeed((self.nh, self.dim, self.vdim)))

    def check(self, dtype):
        if self.dim > ops.SCAN_MAX_ROWS or not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"{self.prefix}: keys of {self.dim} values (at most {ops.SCAN_MAX_ROWS}), {self.taps} taps "
                             f"(at most {ops.SHORT_CONV_MAX_TAPS})")

    def forward(self, h, ctx, cache, owner=True):
        N, H = h.shape[0], self.nh
        conv_state, cell = cache
        proj = linear(h, self.w_in, torch.float32)          # [N, q | k | v | step] float
        mid = linear(h, self.w_mid, h.dtype)                # [N, decays' middle | gate's middle]
        wide = linear(mid, self.w_wide, torch.float32)      # [N, decays (heads x dim) | gate (heads x vdim)] float
        qkv = torch.empty((N, self.channels), dtype=torch.float32, device=h.device)
        ops.short_conv(proj[:, :self.channels], self.conv, None, conv_state.state, ctx.tok_seq, ctx.tok_pos, ctx.seq_start,
                       ctx.seq_past, ctx.seq_slot, qkv, silu=True)
        raw = torch.empty((N, H * self.vdim), dtype=torch.float32, device=h.device)
        ops.channel_delta_scan(qkv, proj[:, self.channels:], wide[:, :H * self.dim], self.a_bias, self.a_log, self.q_scale, self.UNIT_EPS,
                               cell.state, ctx.seq_start, ctx.seq_slot, raw, H, self.nk, self.dim, self.vdim,
                               single_tokens=ctx.one_token_each)
        o = torch.empty((N, H * self.vdim), dtype=h.dtype, device=h.device)
        ops.head_norm_gate(raw, self.gain, self.norm_eps, wide[:, H * self.dim:], o, H, self.vdim)
        return linear_for_sum(o, self.w_o)
