"""RMSNorm as a part: y = gain * x * rsqrt(mean(x^2) + eps), arithmetic in 32-bit.

Formula and order of the product as in crates/synaptix-ops/src/norm/rms_norm.rs:16-26 and
crates/synaptix-kernels-cuda/src/cu/reduction/rms_norm.cu:65-98 (plain gain `w`, not `1 + w`).
The residual sum of the block is fused in (`add_apply`), as the reference's graph path does with
crates/synaptix-kernels-cuda/src/cu/fused/norm/rmsnorm_residual.cu:97-159; here the residual stream
itself stays in 32-bit.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import Part
from .linear import DeferredProduct, ScaledRows, ChannelScaledDeltas, SummedDeltas


class RmsNorm(Part):
    capturable = True
    takes_deferred_product = True     # add_apply accepts a parts.linear.DeferredProduct as delta and may return ScaledRows

    def __init__(self, name: str, dim: int, eps: float, gain_offset: float = 0.0):
        """gain_offset: the gain is gain_offset + the stored tensor (0 here; 1 for checkpoints that store
        the gain as a difference from one, crates/synaptix-models/llm/common/src/config.rs:1-5)."""
        self.name = name          # full tensor name of the gain
        self.dim = dim
        self.eps = float(eps)
        self.gain_offset = float(gain_offset)
        self.gain = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.dim,), "gain")}

    def load(self, get):
        self.gain = get(self.name)

    def add_apply(self, resid, delta, out_dtype, rows=None):
        """resid [N, dim] float: with rows None, resid += delta (if any) in place and every row is
        normed; with rows [n] int32 only those rows of resid + delta are normed and resid is kept."""
        if isinstance(delta, SummedDeltas):
            # a sublayer's result in several terms (routed experts' partial sums, a gated shared expert)
            delta = delta.scaled() if len(delta.terms) <= 2 else delta.run()
        if isinstance(delta, ChannelScaledDeltas):
            # the results of sublayers that ran side by side, each with its channels' scales: added and normed in one pass
            if self.gain_offset == 0.0 and len(delta.terms) <= 2:
                n = resid.shape[0] if rows is None else rows.shape[0]
                out = torch.empty((n, self.dim), dtype=out_dtype, device=resid.device)
                ops.add_scaled_rmsnorm(resid, delta.terms, self.gain, self.eps, out, rows)
                return out
            delta = delta.run()
        if isinstance(delta, DeferredProduct):
            # a product over packed weights for few rows: it adds its sums into resid itself and leaves the rows with
            # the gain and the row statistic in groups; the product that follows applies the row's factor
            if (rows is None and out_dtype == torch.bfloat16 and delta.shape == tuple(resid.shape)
                    and self.dim % 16 == 0):
                xs = torch.empty(resid.shape, dtype=torch.bfloat16, device=resid.device)
                ss = torch.empty((resid.shape[0], self.dim // 16), dtype=torch.float32, device=resid.device)
                ops.gemm_packed(delta.x, delta.packed, None, resid_norm=(resid, self.gain, self.gain_offset, xs, ss))
                return ScaledRows(xs, ss, self.eps, resid, self)
            delta = delta.run()
        n = resid.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n, self.dim), dtype=out_dtype, device=resid.device)
        ops.add_rmsnorm(resid, delta, self.gain, self.eps, out, rows, self.gain_offset)
        return out

    def apply(self, x):
        """Norm over the last axis of a tensor in the activation type."""
        out = torch.empty_like(x)
        ops.rmsnorm_rows(x, self.gain, self.eps, out, self.gain_offset)
        return out


class DynamicTanh(Part):
    """y = tanh(alpha * x) * gain + shift with a scalar alpha: a norm that takes no mean and no variance.

    Tensors: `name` (gain [dim]), `name + alpha_suffix` (one number), `name + shift_suffix` ([dim]).  Arithmetic in
    32-bit.  The residual it reads may run in several streams [N, S, dim]: `add_apply` then norms their sum, or with
    `read` a weighted sum of them (what a block with hyper-connections hands its sublayers).
    """
    capturable = True
    takes_deferred_product = False

    def __init__(self, name: str, dim: int, alpha_suffix: str = ".alpha", shift_suffix: str = ".b"):
        self.name, self.dim = name, dim
        self.alpha_name, self.shift_name = name + alpha_suffix, name + shift_suffix
        self.gain = self.alpha = self.shift = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.dim,), "gain"), self.alpha_name: TensorSpec((), "gain"),
                self.shift_name: TensorSpec((self.dim,), "bias")}

    def load(self, get):
        # a few hundred numbers: kept in 32-bit whatever the engine's type
        self.gain = get(self.name).float().contiguous()
        self.alpha = get(self.alpha_name).float().reshape(1).contiguous()
        self.shift = get(self.shift_name).float().contiguous()

    def dyt_tensors(self):
        """(alpha, gain, shift): what the kernels that apply this norm on their way take."""
        return self.alpha, self.gain, self.shift

    def read(self, resid, in_weights, out_dtype, rows=None, delta=None):
        """The norm of sum_s in_weights[s] * resid[:, s] (in_weights None: of the sum of the streams)."""
        n = resid.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n, self.dim), dtype=out_dtype, device=resid.device)
        ops.streams_read_norm(resid, in_weights, out, dyt=(self.alpha, self.gain, self.shift), rows=rows, delta=delta)
        return out

    def add_apply(self, resid, delta, out_dtype, rows=None):
        """As RmsNorm.add_apply; a residual in several streams comes without a delta and is summed over its streams."""
        return self.read(resid, None, out_dtype, rows=rows, delta=delta)

    def apply(self, x):
        out = torch.empty_like(x)
        x32 = x if x.dtype == torch.float32 else x.float()
        ops.streams_read_norm(x32.reshape(-1, self.dim), None, out.view(-1, self.dim), dyt=(self.alpha, self.gain, self.shift))
        return out
