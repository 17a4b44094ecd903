"""A weight matrix [out, in] without bias: y = x . W^T, 32-bit accumulation.

crates/synaptix-nn/src/linear.rs:67-73; the decoder builds every projection without a bias
(crates/synaptix-models/llm/common/src/weights.rs:49).
"""
from __future__ import annotations

import torch

from ..kernels import ops


class Matrix:
    """A weight [N, K] as the products read it, kept once: a bf16 matrix whose sizes allow it (N a multiple of
    16, K of 32) lies in the order of the MFMA fragments (ops.pack_weight), which the products for single tokens
    need and the tiles for prompts read as well; any other lies in plain rows (`plain`)."""

    def __init__(self, w, keep_rows: bool = False):
        """keep_rows: leave w in plain rows whatever its sizes (a small matrix that only ever meets many rows)."""
        self.shape, self.dtype, self.device = tuple(w.shape), w.dtype, w.device
        self.packed = None if keep_rows else ops.pack_weight(w)
        self.plain = w if self.packed is None else None

    @property
    def data(self):
        """What ops.gemm, ops.gemm_swiglu and ops.embed take for this weight."""
        return self.plain if self.packed is None else self.packed

    def rows(self):
        """The matrix in plain rows (a copy, if it is kept in fragment order): for tests and tools."""
        return self.plain if self.packed is None else ops.unpack_weight(self.packed)

    def nbytes(self):
        t = self.data
        return t.numel() * t.element_size()


def _use_packed(x, m):
    return m.packed is not None and x.dtype == torch.bfloat16 and x.shape[0] <= ops.packed_max_rows(m.shape[0])


def _matrix(w):
    """The products below take a Matrix; a tensor [N, K] in plain rows is taken as it is."""
    return w if isinstance(w, Matrix) else Matrix(w, keep_rows=True)


class ScaledRows:
    """Rows on their way through an RMSNorm whose last step has not been taken: `rows` [M, dim] bf16 hold
    gain * x, `ss` [M, groups] float the sums of x^2 over groups of columns; the normed rows are
    rows[m] * rsqrt(sum(ss[m]) / dim + eps).  A product over packed weights takes them as they are and applies the
    row's factor to its finished sums (it is linear in its input); everything else asks for `plain()`, which norms
    the float rows `resid` they were made from.  Made by a norm from a DeferredProduct; has the shape, type and
    device of the normed rows, so that code which only passes them on need not know."""

    def __init__(self, rows, ss, eps, resid, norm):
        self.rows, self.ss, self.eps, self.resid, self.norm = rows, ss, float(eps), resid, norm
        self.shape, self.dtype, self.device = rows.shape, rows.dtype, rows.device
        self.dim = rows.shape[1]

    @property
    def row_scale(self):
        return (self.ss, self.dim, self.eps)

    def plain(self):
        return self.norm.add_apply(self.resid, None, self.dtype)


def as_rows(h):
    """The normed rows as a tensor, whatever form they arrive in."""
    return h.plain() if isinstance(h, ScaledRows) else h


class DeferredProduct:
    """A product x . W^T over packed weights that has not been run: the norm that receives it as the delta of
    the residual rows runs it with the residual sum and its own first half as the epilogue (ops.gemm_packed,
    resid_norm), or asks for `run()`, the float product itself."""

    def __init__(self, x, w):
        self.x, self.w, self.packed = x, w, w.packed
        self.shape = (x.shape[0], w.shape[0])

    def run(self):
        return linear_for_sum(self.x, self.w)


class WeightedDeltas:
    """A sublayer's result that is a sum of one or two scaled terms which have not been added yet:
    sum_i scale_i * (term_i + bias_i), each term a float tensor [N, hidden] or partial sums [P, N, hidden], each
    bias float [hidden] or None (two mixers side by side; a last product whose bias is still to come).  A block
    that says `takes_weighted_deltas` adds them while it writes the residual; everything else asks for `run()`."""

    def __init__(self, terms):
        self.terms = [(as_delta(t), float(c), b) for t, c, b in terms]
        first = self.terms[0][0]
        self.shape = tuple(first.shape[-2:])

    def run(self):
        first = self.terms[0][0]
        zero = torch.zeros(self.shape, dtype=torch.float32, device=first.device)
        one = torch.ones((1,), dtype=torch.float32, device=first.device)
        ops.streams_update(zero, one.view(1, 1), one, self.terms)
        return zero


class StreamsWrite:
    """A sublayer's result on its way into a residual that runs in streams, not yet written:
    X'[t] = sum_s mix[s, t] X[s] + out_w[t] y.  Whoever reads the streams next either takes it in, updating the
    streams and gathering its own input in one pass (`write_and_read`), or asks for `run()`, which writes the
    streams and leaves nothing to add (None)."""

    def __init__(self, resid, mix, out_w, y):
        self.resid, self.mix, self.out_w = resid, mix, out_w
        self.terms = y.terms if isinstance(y, WeightedDeltas) else [(as_delta(y), 1.0, None)]

    def run(self):
        ops.streams_update(self.resid, self.mix, self.out_w, self.terms)
        return None

    def write_and_read(self, in_w, dyt, out_dtype):
        """The streams written, and norm(sum_t in_w[t] X'[t]) of every row (dyt: a dynamic tanh's tensors or None)."""
        out = torch.empty((self.resid.shape[0], self.resid.shape[-1]), dtype=out_dtype, device=self.resid.device)
        ops.streams_update(self.resid, self.mix, self.out_w, self.terms, read=(in_w, dyt, out))
        return out


class ChannelScaledDeltas:
    """The results of one or two sublayers that ran side by side, not yet added to the residual:
    sum_i scale_i * term_i, each term a float tensor [N, hidden] or partial sums [P, N, hidden], each scale float
    [hidden] (one factor for every channel) or None.  A term may be a triple whose third member is a gate for every row
    (a float view [N, 1], a column of longer rows, or None): the term then counts sigmoid(gate) times.  A norm that
    takes it (RmsNorm) adds the terms into the residual and norms the rows in the same pass; everything else asks for
    `run()`, the sum as one tensor."""

    def __init__(self, terms):
        self.terms = [(as_delta(t[0]), t[1], t[2] if len(t) > 2 else None) for t in terms]
        self.shape = tuple(self.terms[0][0].shape[-2:])

    def run(self):
        first = self.terms[0][0]
        total = torch.zeros(self.shape, dtype=torch.float32, device=first.device)
        ops.add_scaled_rmsnorm(total, self.terms, None, 0.0, None)
        return total


class SummedDeltas:
    """A sublayer's result as several terms that have not been added yet (routed experts and an expert that every token
    passes), each a float tensor [N, hidden] or partial sums [P, N, hidden] (or a product that has not been run).
    `row_gates`: for each term None or a float view [N, 1] whose sigmoid multiplies the term's rows (an expert that
    every token passes through a gate of its own).  A block that scales its sublayers' results by channel hands the
    terms on, each with the scales; a norm takes them as they are (both as ChannelScaledDeltas); everything else asks
    for `run()`, the sum as one tensor."""

    def __init__(self, terms, row_gates=None):
        self.terms = [as_delta(t) for t in terms]
        self.row_gates = list(row_gates) if row_gates is not None else [None] * len(self.terms)
        if len(self.row_gates) != len(self.terms):
            raise ValueError("one gate (or None) for each term")
        self.shape = tuple(self.terms[0].shape[-2:])

    def scaled(self, scale=None):
        """The terms, each with the channels' scales `scale` (or none) and its rows' gate."""
        return ChannelScaledDeltas([(t, scale, g) for t, g in zip(self.terms, self.row_gates)])

    def run(self):
        return self.scaled().run()


def as_delta(d):
    """The delta of the residual rows as a tensor (or None), whatever form it arrives in."""
    if isinstance(d, (DeferredProduct, WeightedDeltas, StreamsWrite, ChannelScaledDeltas, SummedDeltas)):
        return d.run()
    return d


def deferred_product(x, w):
    """linear_for_sum, but where the product would run over few rows in one slice it is only described:
    the caller's result is the delta that a following norm adds to the residual rows, and that norm can take the
    product in (RmsNorm.add_apply)."""
    w = _matrix(w)
    if isinstance(x, torch.Tensor) and _use_packed(x, w) and ops.packed_slices(w.shape[0], w.shape[1]) <= 1:
        return DeferredProduct(x, w)
    return linear_for_sum(x, w)


def linear(x, w, out_dtype):
    """x [M, K] in the activation type, w a Matrix [N, K]; a weight kept in 32-bit takes the 32-bit product."""
    w = _matrix(w)
    if _use_packed(x, w) and out_dtype in (torch.bfloat16, torch.float32):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=x.device)
        if isinstance(x, ScaledRows):
            ops.gemm_packed(x.rows, w.packed, out, row_scale=x.row_scale)
        else:
            ops.gemm_packed(x, w.packed, out)
        return out
    x = as_rows(x)
    if w.dtype != x.dtype:
        if w.dtype == torch.float32:
            x = x.to(torch.float32)
        else:
            raise TypeError(f"linear: activation {x.dtype} with weight {w.dtype}")
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32 if x.dtype == torch.float32 else out_dtype,
                      device=x.device)
    ops.gemm(x, w.data, out)
    return out if out.dtype == out_dtype else out.to(out_dtype)


def product_slices(n_rows, w, dtype) -> int:
    """Into how many slices of K the product of n_rows rows with w is cut for a reader that adds partial sums."""
    if w.dtype != dtype or (w.packed is not None and w.shape[1] % 128):
        return 1            # (in fragment order the tiles for many rows take a K that is a multiple of 128 only)
    return ops.gemm_slices(n_rows, w.shape[0], w.shape[1], dtype)


def linear_for_sum(x, w):
    """The product as float partial sums for a consumer that adds them up (the residual sum fused
    into the next norm): [S, M, N] when cutting K into S slices gives a small product more
    workgroups, else [M, N]."""
    w = _matrix(w)
    if _use_packed(x, w):
        slices = ops.packed_slices(w.shape[0], w.shape[1])
        if slices <= 1:
            return linear(x, w, torch.float32)
        out = torch.empty((slices, x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device)
        if isinstance(x, ScaledRows):
            ops.gemm_packed(x.rows, w.packed, out, row_scale=x.row_scale)
        else:
            ops.gemm_packed(x, w.packed, out)
        return out
    x = as_rows(x)
    M = x.shape[0]
    slices = product_slices(M, w, x.dtype)
    if slices <= 1:
        return linear(x, w, torch.float32)
    out = torch.empty((slices, M, w.shape[0]), dtype=torch.float32, device=x.device)
    ops.gemm(x, w.data, out)
    return out
