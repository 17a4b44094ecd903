"""How a norm, a mixer, a second norm and a feed-forward are arranged in a layer.

PreNormBlock:  x <- x + mixer(norm1(x));  x <- x + ff(norm2(x))  (no post-norms),
crates/synaptix-models/llm/common/src/model.rs:1179-1199.  The residual stream x is float; each
sum x + delta is fused into the norm that follows it, so a block returns its last delta
unsummed and takes the previous block's.
"""
from __future__ import annotations

from .base import Part
from .linear import as_rows, as_delta


class Block(Part):
    """Interface: forward(resid, pending, ctx, cache, owner) -> pending.
    resid [N, hidden] float is updated in place; pending is a delta not yet added (or None)."""

    mixer = None
    # True: `pending` may arrive as a parts.linear.DeferredProduct (a product that the block's first norm can take
    # in); False (the default): the model runs such a product before it calls the block
    takes_deferred_product = False

    def forward(self, resid, pending, ctx, cache, owner=True):
        raise NotImplementedError


def _norm_input(norm, delta):
    return delta if getattr(norm, "takes_deferred_product", False) else as_delta(delta)


class PreNormBlock(Block):
    """x <- x + s1 * mixer(norm1(x));  x <- x + s2 * ff(norm2(x)).  scale_prefix: the results are multiplied channel by
    channel by the tensors scale_prefix + "ls1" and "ls2" ([hidden]; None: no scales).  A layer may have no
    feed-forward (norm2 and feed_forward None): it is its first half only."""
    takes_deferred_product = True

    def __init__(self, norm1, mixer, norm2=None, feed_forward=None, scale_prefix: str | None = None,
                 scale_names=("ls1", "ls2"), hidden: int | None = None):
        if (norm2 is None) != (feed_forward is None):
            raise ValueError("the second norm and the feed-forward come together")
        if scale_prefix is not None and hidden is None:
            raise ValueError("channel scales need the width of the residual")
        self.norm1, self.mixer, self.norm2, self.feed_forward = norm1, mixer, norm2, feed_forward
        self.scale_prefix, self.scale_names, self.hidden = scale_prefix, tuple(scale_names), hidden
        self.scales = [None, None]

    def _parts(self):
        return tuple(p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None)

    def _scale_names(self):
        if self.scale_prefix is None:
            return []
        return [self.scale_prefix + n for n in self.scale_names[:2 if self.feed_forward is not None else 1]]

    @property
    def capturable(self):
        return all(getattr(p, "capturable", False) for p in self._parts())

    def tensor_specs(self):
        from ..weights.source import TensorSpec
        specs = {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        specs.update({n: TensorSpec((self.hidden,), "gain") for n in self._scale_names()})
        return specs

    def load(self, get):
        for p in self._parts():
            p.load(get)
        for i, n in enumerate(self._scale_names()):
            self.scales[i] = get(n).float().contiguous()

    def check(self, dtype):
        for p in self._parts():
            p.check(dtype)

    def _scaled(self, delta, scale):
        """A sublayer's result with its channels' scales, left for whoever adds the residual next."""
        from .linear import ChannelScaledDeltas, SummedDeltas
        if scale is None:
            return delta
        if isinstance(delta, SummedDeltas):
            return delta.scaled(scale)
        return ChannelScaledDeltas([(delta, scale)])

    def forward(self, resid, pending, ctx, cache, owner=True):
        # a norm may hand on rows whose last step a product finishes, and take a product that has not been run
        # (parts.linear.ScaledRows, DeferredProduct); parts that do not say they take them get plain tensors
        h = self.norm1.add_apply(resid, _norm_input(self.norm1, pending), ctx.act_dtype)
        a = self._scaled(self.mixer.forward(h if self.mixer.takes_scaled_rows else as_rows(h), ctx, cache, owner),
                         self.scales[0])
        if self.feed_forward is None:
            return a
        h2 = self.norm2.add_apply(resid, _norm_input(self.norm2, a), ctx.act_dtype)
        return self._scaled(self.feed_forward.forward(h2 if self.feed_forward.takes_scaled_rows else as_rows(h2), ctx),
                            self.scales[1])


class HyperConnectionBlock(Block):
    """A pre-norm layer over a residual that runs in S streams X[:, s] (csrc/streams.hip).  For sublayer q (1: the
    mixer, 2: the feed-forward, if the layer has one):

        u = sum_s in_q[s] X[s];   y = sublayer(norm_q(u));   X'[t] = sum_s mix_q[s, t] X[s] + out_q[t] y

    with all streams written at once from the old ones.  Tensors: prefix + "hc<q>.in" [S], ".out" [S], ".mix" [S, S]
    (from, to).  A sublayer's result is written into the streams by the pass that gathers the next sublayer's input
    (parts.linear.StreamsWrite): the block's last one leaves as `pending`, for the next block or the final norm.
    """
    takes_deferred_product = True       # `pending` may be the StreamsWrite that the block before left

    def __init__(self, prefix: str, streams: int, norm1, mixer, norm2=None, feed_forward=None,
                 names=("hc1.", "hc2.")):
        if (norm2 is None) != (feed_forward is None):
            raise ValueError("the second norm and the feed-forward come together")
        self.prefix, self.streams, self.names = prefix, int(streams), names
        self.norm1, self.mixer, self.norm2, self.feed_forward = norm1, mixer, norm2, feed_forward
        self.hc = [None, None]

    def _parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    @property
    def capturable(self):
        return all(getattr(p, "capturable", False) for p in self._parts())

    def _subs(self):
        return range(2 if self.feed_forward is not None else 1)

    def tensor_specs(self):
        from ..weights.source import TensorSpec
        S, specs = self.streams, {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        for q in self._subs():
            n = self.prefix + self.names[q]
            specs.update({n + "in": TensorSpec((S,), "gain"), n + "out": TensorSpec((S,), "gain"),
                          n + "mix": TensorSpec((S, S), "mixing")})
        return specs

    def load(self, get):
        for p in self._parts():
            p.load(get)
        for q in self._subs():
            n = self.prefix + self.names[q]
            self.hc[q] = tuple(get(n + k).float().contiguous() for k in ("in", "out", "mix"))

    def check(self, dtype):
        for p in self._parts():
            p.check(dtype)

    def _read(self, norm, resid, in_w, dtype, pending=None):
        """The sublayer's input: the norm of the streams' weighted sum, after `pending` (a StreamsWrite) has been
        written; one pass where the norm can be applied on the way."""
        import torch
        from ..kernels import ops
        if pending is not None and hasattr(norm, "dyt_tensors"):
            return pending.write_and_read(in_w, norm.dyt_tensors(), dtype)
        if pending is not None:
            pending.run()
        if hasattr(norm, "read"):
            return norm.read(resid, in_w, dtype)
        u = torch.empty((resid.shape[0], resid.shape[2]), dtype=torch.float32, device=resid.device)
        ops.streams_read_norm(resid, in_w, u)
        return norm.add_apply(u, None, dtype)

    def forward(self, resid, pending, ctx, cache, owner=True):
        from .linear import StreamsWrite
        if pending is not None and not isinstance(pending, StreamsWrite):
            raise ValueError("a block over residual streams takes no pending delta but another such block's")
        if resid.dim() != 3 or resid.shape[1] != self.streams:
            raise ValueError(f"the residual has shape {list(resid.shape)}; this block reads {self.streams} streams")
        h = self._read(self.norm1, resid, self.hc[0][0], ctx.act_dtype, pending)
        pending = StreamsWrite(resid, self.hc[0][2], self.hc[0][1], self.mixer.forward(h, ctx, cache, owner))
        if self.feed_forward is not None:
            h2 = self._read(self.norm2, resid, self.hc[1][0], ctx.act_dtype, pending)
            pending = StreamsWrite(resid, self.hc[1][2], self.hc[1][1], self.feed_forward.forward(h2, ctx))
        return pending


class ParallelBlock(Block):
    """A layer whose mixer and feed-forward run side by side on the output of one norm:

        h = norm(x);   x <- x + mult * (scale1 * mixer(h) + scale2 * ff(h))

    with a scale for every channel of each sublayer's result (tensors prefix + "ls1", "ls2", [hidden]; `layer_scale`
    False: none) and one factor `mult`.  A layer may have no feed-forward.  The sum is left to whoever reads the
    residual next (parts.linear.ChannelScaledDeltas): a norm that takes it adds and norms in one pass."""
    takes_deferred_product = True       # `pending` may be the ChannelScaledDeltas that the block before left

    def __init__(self, prefix: str, hidden: int, norm, mixer, feed_forward=None, mult: float = 1.0,
                 layer_scale: bool = True, scale_names=("ls1", "ls2")):
        self.prefix, self.hidden, self.mult = prefix, hidden, float(mult)
        self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward
        self.layer_scale, self.scale_names = bool(layer_scale), tuple(scale_names)
        self.scales = [None, None]

    def _parts(self):
        return [p for p in (self.norm, self.mixer, self.feed_forward) if p is not None]

    @property
    def capturable(self):
        return all(getattr(p, "capturable", False) for p in self._parts())

    def _scale_names(self):
        n = 2 if self.feed_forward is not None else 1
        return [self.prefix + s for s in self.scale_names[:n]] if self.layer_scale else []

    def tensor_specs(self):
        from ..weights.source import TensorSpec
        specs = {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        specs.update({n: TensorSpec((self.hidden,), "gain") for n in self._scale_names()})
        return specs

    def load(self, get):
        import torch
        for p in self._parts():
            p.load(get)
        for i, n in enumerate(self._scale_names()):
            self.scales[i] = (get(n).float() * self.mult).contiguous()       # mult * scale, 32-bit
        if not self.layer_scale and self.mult != 1.0:
            dev = self.norm.gain.device
            self.scales = [torch.full((self.hidden,), self.mult, dtype=torch.float32, device=dev)] * 2

    def check(self, dtype):
        for p in self._parts():
            p.check(dtype)

    def forward(self, resid, pending, ctx, cache, owner=True):
        from .linear import ChannelScaledDeltas
        h = as_rows(self.norm.add_apply(resid, _norm_input(self.norm, pending), ctx.act_dtype))
        terms = [(as_delta(self.mixer.forward(h, ctx, cache, owner)), self.scales[0])]
        if self.feed_forward is not None:
            terms.append((as_delta(self.feed_forward.forward(h, ctx)), self.scales[1]))
        return ChannelScaledDeltas(terms)
