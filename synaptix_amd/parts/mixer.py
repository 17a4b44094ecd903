"""Token mixers.  Here: grouped-query attention over the paged cache.

GqaAttention: q/k/v projections (one fused product), optional per-head RMSNorm of q and k,
a position encoding, cache write, causal attention (optionally a window), output projection.
Order and formulas as crates/synaptix-models/llm/common/src/model.rs:1715-1734 (projections,
q/k norm before the rotation, the layer's eps), 1781-1782 (cache write), 1740-1869
(scores, scale, mask, softmax, PV), 1872-1878 (merge heads, o_proj).
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import Part, KvNeed
from .linear import (Matrix, linear, linear_for_sum, product_slices, deferred_product, as_rows, ScaledRows,
                     WeightedDeltas)
from .position import Position, NoPosition


class Mixer(Part):
    """Interface of a token mixer.

    cache_need(): KvNeed, StateNeed or None: what it keeps for each sequence.
    forward(h, ctx, cache, owner): h [N, hidden] in the activation type, ctx the step's
    StepContext, cache the view of its cache layer (None without a need); owner is False when the
    layer reads a cache that another layer writes.  Returns the residual delta as float [N, hidden],
    or as partial sums [S, N, hidden] that the following norm adds up.
    """

    # True: `h` may arrive as parts.linear.ScaledRows (rows whose norm a product over packed weights finishes)
    # and the returned delta may be a parts.linear.DeferredProduct; False (the default): plain tensors both ways
    takes_scaled_rows = False

    def cache_need(self):
        return None

    def forward(self, h, ctx, cache, owner=True):
        raise NotImplementedError


class GqaAttention(Mixer):
    takes_scaled_rows = True
    capturable = True

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, *,
                 position: Position | None = None, qk_norm_eps: float | None = None, scale: float | None = None,
                 window: int | None = None, qk_gain_offset: float = 0.0, score_softcap: float | None = None):
        if n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not divide into {n_kv_heads} kv heads")
        self.prefix = prefix
        self.hidden, self.nh, self.nkv, self.hd = hidden, n_heads, n_kv_heads, head_dim
        self.position = position or NoPosition()
        self.qk_norm_eps = qk_norm_eps
        self.qk_gain_offset = float(qk_gain_offset)     # the q/k gains are this + their tensors
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.window = window
        # a soft cap on the scaled scores, cap * tanh(score / cap); None: none.  What the position scheme adds to the
        # scores (Position.score_slopes) is asked for at the first step.
        self.score_softcap = float(score_softcap) if score_softcap else 0.0
        self._slopes = {}
        self.w_qkv = self.w_o = self.q_gain = self.k_gain = None

    def tensor_specs(self):
        p, hd = self.prefix, self.hd
        specs = {
            p + "q_proj.weight": TensorSpec((self.nh * hd, self.hidden)),
            p + "k_proj.weight": TensorSpec((self.nkv * hd, self.hidden)),
            p + "v_proj.weight": TensorSpec((self.nkv * hd, self.hidden)),
            p + "o_proj.weight": TensorSpec((self.hidden, self.nh * hd)),
        }
        if self.qk_norm_eps is not None:
            specs[p + "q_norm.weight"] = TensorSpec((hd,), "gain")
            specs[p + "k_norm.weight"] = TensorSpec((hd,), "gain")
        return specs

    def load(self, get):
        p = self.prefix
        # one product for q, k and v: rows of the three matrices one after another
        self.w_qkv = Matrix(torch.cat([get(p + "q_proj.weight"), get(p + "k_proj.weight"), get(p + "v_proj.weight")], 0))
        self.w_o = Matrix(get(p + "o_proj.weight"))
        if self.qk_norm_eps is not None:
            self.q_gain = get(p + "q_norm.weight")
            self.k_gain = get(p + "k_norm.weight").to(self.q_gain.dtype)

    def cache_need(self):
        return KvNeed(self.nkv, self.hd, self.window)

    def check(self, dtype):
        if self.hd % 2 or self.hd > ops.MAX_HEAD_DIM:
            raise ValueError(f"{self.prefix}: head size {self.hd} must be even and at most {ops.MAX_HEAD_DIM}")
        if dtype == torch.bfloat16 and self.hd % 16:
            raise ValueError(f"{self.prefix}: the bf16 attention kernels take head sizes in steps of 16 "
                             f"(16, 32, ..., {ops.MAX_HEAD_DIM}); {self.hd} runs in float32 only")

    def _score_terms(self, device):
        key = str(device)
        if key not in self._slopes:
            sl = self.position.score_slopes(self.nh, device)
            self._slopes[key] = None if sl is None else sl.to(device=device, dtype=torch.float32).contiguous()
        return dict(slopes=self._slopes[key], softcap=self.score_softcap)

    def _decode_work(self, ctx, cache, n_seqs):
        """For single tokens: the workspace of the splits' partial results, the number of splits, and
        what merges them inside the attention kernel (counters, and the step's work list if it keeps one)."""
        splits = ctx.decode_splits(self.nkv, cache.group)
        work = ctx.scratch("attention_decode", n_seqs * self.nh * splits * (self.hd + 2))
        merge = {}
        if splits > 1:
            chunks = -(-(self.nh // self.nkv) // 16)
            items = ctx.decode_items(cache.group)
            if items is not None and items.numel() != 4 * n_seqs * splits + 2 * n_seqs:
                items = None
            merge = dict(counters=ctx.counters("attention_decode_arrivals", n_seqs * self.nkv * chunks), items=items)
        return work, splits, merge

    def forward(self, h, ctx, cache, owner=True):
        nh, nkv, hd = self.nh, self.nkv, self.hd
        N, act = h.shape[0], h.dtype
        terms = self._score_terms(h.device)
        cap = self.position.capacity
        if cap is not None and ctx.max_position >= cap:
            raise ValueError(f"position {ctx.max_position} is beyond the position encoding's capacity {cap}")
        # single tokens: partial sums over slices of K, which the attention kernel adds; prompts: the plain product
        if self.w_qkv.packed is not None and N <= ops.PACKED_MAX_ROWS and act == torch.bfloat16:
            qkv = linear_for_sum(h, self.w_qkv)       # float partial sums [S, N, width]
            if qkv.dim() == 2:
                qkv = qkv.unsqueeze(0)
        else:
            h = as_rows(h)
            # (every kernel behind it adds partial sums itself; ops.gemm_slices cuts where the product would
            # otherwise leave compute units without work: single tokens and prompts up to about 1,200 tokens)
            sliced = product_slices(N, self.w_qkv, act) > 1
            qkv = linear_for_sum(h, self.w_qkv) if sliced else linear(h, self.w_qkv, act)
        cos, sin = self.position.tables(h.device)
        table = ctx.page_table(cache.group)
        o = torch.empty((N, nh * hd), dtype=act, device=h.device)
        window = self.window or 0
        if act == torch.bfloat16 and ctx.one_token_each:
            # single tokens: the attention kernel takes q, k and v from the projection itself
            work, splits, merge = self._decode_work(ctx, cache, N)
            ops.attention_decode_fused_bf16(qkv, cache.k_pages, cache.v_pages, table, ctx.seq_len, o, work, splits,
                                            self.scale, window, nh, nkv, hd, self.q_gain, self.k_gain,
                                            self.qk_norm_eps or 0.0, cos, sin, write_kv=owner,
                                            gain_offset=self.qk_gain_offset, **terms, **merge)
            return deferred_product(o, self.w_o)
        q = torch.empty((N, nh * hd), dtype=act, device=h.device)
        ops.qk_norm_rope_kv_write(qkv, q, cache.k_pages, cache.v_pages, table, ctx.tok_seq, ctx.tok_pos,
                                  self.q_gain, self.k_gain, self.qk_norm_eps or 0.0, cos, sin, nh, nkv, hd,
                                  write_kv=owner, gain_offset=self.qk_gain_offset)
        if act == torch.float32:
            ops.attention_f32(q, cache.k_pages, cache.v_pages, table, ctx.tok_seq, ctx.tok_pos, o, self.scale, window,
                              nh, nkv, hd, **terms)
        elif ctx.one_token_each:
            work, splits, merge = self._decode_work(ctx, cache, N)
            ops.attention_decode_bf16(q, cache.k_pages, cache.v_pages, table, ctx.seq_len, o, work, splits,
                                      self.scale, window, nh, nkv, hd, **terms, **merge)
        else:
            # a step of prompts and single tokens: the prompts' kernel leaves the single tokens out, and the kernel
            # for single tokens takes them (gathered, since it counts one row a sequence)
            singles = ctx.single_token_rows()
            ops.attention_prefill_bf16(q, cache.k_pages, cache.v_pages, table, ctx.seq_start, ctx.seq_past, o,
                                       self.scale, window, nh, nkv, hd, skip_below=2 if singles is not None else 0, **terms)
            if singles is not None:
                rows, seqs = singles
                n1 = rows.numel()
                q1, o1 = q.index_select(0, rows), torch.empty((n1, nh * hd), dtype=act, device=h.device)
                splits = ops.decode_splits(n1, nkv, table.shape[1])
                work = ctx.scratch("attention_decode", n1 * nh * splits * (hd + 2))
                ops.attention_decode_bf16(q1, cache.k_pages, cache.v_pages, table.index_select(0, seqs),
                                          ctx.seq_len.index_select(0, seqs), o1, work, splits, self.scale, window,
                                          nh, nkv, hd, **terms)
                o.index_copy_(0, rows, o1)
        return deferred_product(o, self.w_o)


def _projection(w):
    """A projection's weight as the products keep it: in fragment order only where the tiles for many rows read that
    order too (K a multiple of 128); other widths stay in plain rows."""
    return Matrix(w, keep_rows=w.shape[1] % 128 != 0)


def _whole_fragments(w):
    """A fused projection whose last piece is a few rows (one gate a head): rows of zeros behind it up to the next
    multiple of 16, so that the matrix can lie in fragment order; the product's rows get that much longer, and nobody
    reads the extra columns."""
    spare = -w.shape[0] % 16
    if spare == 0 or w.shape[1] % 128:
        return w
    return torch.cat([w, torch.zeros((spare, w.shape[1]), dtype=w.dtype, device=w.device)], 0)


class GatedWindowAttention(Mixer):
    """Grouped-query attention whose scores, mask and softmax are parameters (csrc/attention_window.hip):

        score(i, j) = scale q_i.k_j [soft cap] + what the position scheme puts on the scores
        key j is seen by i iff j <= i and (window is None or i - j < window or j < keep_first)
                                      and (chunk is None or j // chunk == i // chunk or j < keep_first)
        p_j = exp(score_j) / (sink + sum exp(score_j)),  sink = 1 with sink_one, exp(sink_h) with a learned `sink`

    Keys have `dim` values, values `v_dim`.  q, k and v may carry a bias (`bias`), the output product one of its own
    (`out_bias`); q and k heads may be normed (RMS over the head, one gain for all heads: `qk_norm_eps`); with `gate`
    the heads' results are multiplied by sigmoid(W_g h) before the output product (True or "value": one gate for every
    value; "head": one for each head).  The position scheme may act on the scores (Position.score_slopes,
    Position.score_log_bias) or turn the first values of every q and k head after the norm (Position.tables, in the
    pairing that Position.pairing names).  `chunk`: positions are counted in runs of that many from the sequence's
    first token, and a query sees the keys of its own run only.  Scores, weights, the rotation and the norms are 32-bit
    in both engine types.

    `shared_kv`: the layer has no keys and values of its own (no k and v tensors, biases or k norm): it reads the cache
    of an earlier layer with the same head counts and sizes (the model's schedule gives both runs the same cache), as
    that layer wrote it, with its own queries, mask, sink and gate.  `cache_window`: what the cache keeps where that is
    more than this layer's own mask needs (the layers that share a cache name the same).

    Tensor names: prefix + "q", "k", "v", "o" (+ ".b" for their biases), "q.norm", "k.norm", "g", "sink"; `names`
    renames them.
    """
    # (the input projection over packed weights finishes a norm's rows itself, and the output product without a bias
    # is left for the following norm to run with the residual sum as its epilogue: parts.linear)
    takes_scaled_rows = True
    capturable = True

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_norm": "q.norm", "k_norm": "k.norm", "bias": ".b",
             "sink": "sink"}
    _UNSET = object()

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, dim: int, v_dim: int | None = None, *,
                 position: Position | None = None, qk_norm_eps: float | None = None, scale: float | None = None,
                 window: int | None = None, keep_first: int = 0, sink_one: bool = False, bias: bool = False,
                 out_bias: bool = False, gate=False, score_softcap: float | None = None, names: dict | None = None,
                 chunk: int | None = None, sink: bool = False, shared_kv: bool = False, cache_window=_UNSET):
        if n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not divide into {n_kv_heads} kv heads")
        if gate not in (False, True, None, "value", "head"):
            raise ValueError(f"{prefix}: gate {gate!r} (False, 'value' or 'head')")
        if sink and sink_one:
            raise ValueError(f"{prefix}: a learned sink and a sink of one together")
        if chunk is not None and chunk <= 0:
            raise ValueError(f"{prefix}: chunks of {chunk} positions")
        self.prefix, self.hidden = prefix, hidden
        self.nh, self.nkv, self.dim, self.vdim = n_heads, n_kv_heads, dim, v_dim or dim
        self.position = position or NoPosition()
        self.qk_norm_eps = qk_norm_eps
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(dim)
        self.window, self.keep_first, self.sink_one = window, int(keep_first or 0), bool(sink_one)
        self.chunk, self.sink, self.shared_kv = chunk, bool(sink), bool(shared_kv)
        # what a query can see lies within the last `reach` positions (None: anywhere): a run of `chunk` positions is
        # never longer than that many
        reach = [n for n in (window, chunk) if n]
        self.reach = min(reach) if reach else None
        self.cache_window = self.reach if cache_window is self._UNSET else cache_window
        if self.cache_window is not None and (self.reach is None or self.cache_window < self.reach):
            raise ValueError(f"{prefix}: a cache of the last {self.cache_window} keys for a mask that reaches "
                             f"{'every key' if self.reach is None else self.reach}")
        self.bias, self.out_bias = bool(bias), bool(out_bias)
        self.gate = "head" if gate == "head" else ("value" if gate else None)
        self.score_softcap = float(score_softcap) if score_softcap else 0.0
        self.names = dict(self.NAMES, **(names or {}))
        self.w_in = self.w_o = self.b_in = self.b_o = self.q_gain = self.k_gain = self.sinks = None
        self._terms = None

    def _n(self, key, bias=False):
        return self.prefix + self.names[key] + (self.names["bias"] if bias else "")

    def _biased(self):
        """The pieces of the fused projection that carry a bias: q, and k and v where the layer has them."""
        return [("q", self.nh * self.dim)] + ([] if self.shared_kv else [("k", self.nkv * self.dim), ("v", self.nkv * self.vdim)])

    def _widths(self):
        gate = {None: 0, "head": self.nh, "value": self.nh * self.vdim}[self.gate]
        return self._biased() + ([("g", gate)] if self.gate else [])

    def tensor_specs(self):
        specs = {self._n(k): TensorSpec((n, self.hidden)) for k, n in self._widths()}
        specs[self._n("o")] = TensorSpec((self.hidden, self.nh * self.vdim))
        if self.bias:
            for k, n in self._biased():
                specs[self._n(k, True)] = TensorSpec((n,), "bias")
        if self.out_bias:
            specs[self._n("o", True)] = TensorSpec((self.hidden,), "bias")
        if self.qk_norm_eps is not None:
            specs[self._n("q_norm")] = TensorSpec((self.dim,), "gain")
            if not self.shared_kv:
                specs[self._n("k_norm")] = TensorSpec((self.dim,), "gain")
        if self.sink:
            specs[self._n("sink")] = TensorSpec((self.nh,), "bias")
        specs.update(self.position.tensor_specs())
        return specs

    def load(self, get):
        # one product for q, k, v and the gate: rows of the matrices one after another
        self.w_in = _projection(_whole_fragments(torch.cat([get(self._n(k)) for k, _ in self._widths()], 0)))
        self.w_o = _projection(get(self._n("o")))
        if self.bias:
            self.b_in = torch.cat([get(self._n(k, True)).float() for k, _ in self._biased()]).contiguous()
        if self.out_bias:
            self.b_o = get(self._n("o", True)).float().contiguous()
        if self.qk_norm_eps is not None:
            self.q_gain = get(self._n("q_norm")).float().contiguous()
            # (a layer without keys of its own hands the intake its query gain twice; the key gain is never read)
            self.k_gain = self.q_gain if self.shared_kv else get(self._n("k_norm")).float().contiguous()
        if self.sink:
            self.sinks = get(self._n("sink")).float().contiguous()
        self.position.load(get)

    def cache_need(self):
        return KvNeed(self.nkv, self.dim, self.cache_window, v_dim=self.vdim,
                      keep_first=self.keep_first if self.cache_window else 0)

    def check(self, dtype):
        if max(self.dim, self.vdim) > ops.WINDOW_ATTENTION_MAX_DIM:
            raise ValueError(f"{self.prefix}: head sizes {self.dim} and {self.vdim} (at most {ops.WINDOW_ATTENTION_MAX_DIM})")
        cos, _ = self.position.tables("cpu")
        if cos is not None and 2 * cos.shape[1] > self.dim:
            raise ValueError(f"{self.prefix}: the rotation turns {2 * cos.shape[1]} values of heads of {self.dim}")

    def _score_terms(self, device):
        if self._terms is None:
            sl = self.position.score_slopes(self.nh, device)
            self._terms = dict(slopes=None if sl is None else sl.to(device=device, dtype=torch.float32).contiguous(),
                               log_bias=self.position.score_log_bias(self.nh, device), softcap=self.score_softcap)
        return self._terms

    def forward(self, h, ctx, cache, owner=True):
        N, act = h.shape[0], h.dtype
        if owner == self.shared_kv:
            raise ValueError(f"{self.prefix}: a layer {'without' if owner else 'with'} keys and values of its own was "
                             f"scheduled as the cache's {'owner' if owner else 'reader'}")
        cap = self.position.capacity
        if cap is not None and ctx.max_position >= cap:
            raise ValueError(f"position {ctx.max_position} is beyond the position encoding's capacity {cap}")
        proj = linear(h, self.w_in, torch.float32)          # [N, q | k | v | gate] float (q | gate with shared_kv)
        q = torch.empty((N, self.nh * self.dim), dtype=act, device=h.device)
        table = ctx.page_table(cache.group)
        ops.window_intake(proj, self.b_in, q, cache.k_pages, cache.v_pages, table, ctx.tok_seq, ctx.tok_pos,
                          self.q_gain, self.k_gain, self.qk_norm_eps or 0.0, self.nh, self.nkv, self.dim, self.vdim,
                          write_kv=owner, rotation=self.position.tables(h.device), pairs=self.position.pairing == "pairs")
        o = torch.empty((N, self.nh * self.vdim), dtype=act, device=h.device)
        at = sum(n for _, n in self._biased())
        gate = proj[:, at:at + self._widths()[-1][1]] if self.gate else None
        how = dict(window=self.window or 0, keep_first=self.keep_first, sink_one=self.sink_one, gate=gate,
                   gate_per_head=self.gate == "head", sinks=self.sinks, chunk=self.chunk or 0,
                   **self._score_terms(h.device))
        if act == torch.bfloat16 and not ctx.one_token_each and ops.window_prefill_takes(self.dim, self.vdim):
            # prompts in bf16: tiles of queries on the matrix cores
            ops.window_attention_prefill_bf16(q, cache.k_pages, cache.v_pages, table, ctx.seq_start, ctx.seq_past, o,
                                              self.scale, self.nh, self.nkv, self.dim, self.vdim, **how)
        else:
            # 32-bit, single tokens, and head sizes that the tiles do not take: a wave (or eight) for each (token, head)
            ops.window_attention(q, cache.k_pages, cache.v_pages, table, ctx.tok_seq, ctx.tok_pos, o, self.scale, self.nh,
                                 self.nkv, self.dim, self.vdim, **how)
        if self.b_o is None:
            return deferred_product(o, self.w_o)
        return WeightedDeltas([(linear_for_sum(o, self.w_o), 1.0, self.b_o)])


class DifferentialAttention(Mixer):
    """Grouped-query attention in two softmax maps over the same values, joined by a difference:

        q [heads x 2 x dim], k [kv_heads x 2 x dim] (head by head: map 1, map 2), v [kv_heads x vdim];
        each of q, k, v passes a short causal convolution over time (one filter a channel, no activation);
        the position scheme turns the first values of every map's q and k;
        a_m = softmax_j(scale q_m . k_m) v over the keys j with 0 <= i - j (< window), m = 1, 2;
        lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff  (one number for the layer)
        o = rms_norm(a_1 - lambda a_2) (1 - diff)  per head over its vdim values, no gain;   W_o on the heads.

    It runs as grouped-query attention with 2 heads x 2 kv_heads of `dim` whose kv heads share their values in pairs
    (KvNeed.v_heads): the query rows are kept in the order (kv head, map, head of the group), so that a head's two maps
    read the key heads 2 g and 2 g + 1 of its group g.  The cache holds each token's keys for both maps, its values
    once, and the convolutions' last taps - 1 inputs.  Scores, weights, the rotation and the norm are 32-bit.

    Tensor names: prefix + "q", "k", "v" (+ ".conv" [channels, taps]), "lq1", "lk1", "lq2", "lk2" [dim], "o"."""
    takes_scaled_rows = False
    capturable = True

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "conv": ".conv", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, dim: int, v_dim: int, taps: int, *,
                 diff: float, norm_eps: float, position: Position | None = None, scale: float | None = None,
                 window: int | None = None, names: dict | None = None):
        if n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not divide into {n_kv_heads} kv heads")
        self.prefix, self.hidden = prefix, hidden
        self.nh, self.nkv, self.dim, self.vdim, self.taps = n_heads, n_kv_heads, dim, v_dim, taps
        self.diff, self.norm_eps = float(diff), float(norm_eps)
        self.position = position or NoPosition()
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(dim)
        self.window = window
        self.names = dict(self.NAMES, **(names or {}))
        self.channels = (2 * n_heads + 2 * n_kv_heads) * dim + n_kv_heads * v_dim
        self.w_in = self.w_o = self.conv = None
        self.lam = None

    def _n(self, key):
        return self.prefix + self.names[key]

    def _widths(self):
        return [("q", 2 * self.nh * self.dim), ("k", 2 * self.nkv * self.dim), ("v", self.nkv * self.vdim)]

    def tensor_specs(self):
        specs = {}
        for k, n in self._widths():
            specs[self._n(k)] = TensorSpec((n, self.hidden))
            specs[self._n(k) + self.names["conv"]] = TensorSpec((n, self.taps), "filter")
        for k in ("lq1", "lk1", "lq2", "lk2"):
            specs[self._n(k)] = TensorSpec((self.dim,), "bias")
        specs[self._n("o")] = TensorSpec((self.hidden, self.nh * self.vdim))
        return specs

    def _by_kv_head(self, rows):
        """Query rows [heads, 2, dim, ...] in the order (kv head, map, head of the group, dim)."""
        R = self.nh // self.nkv
        t = rows.reshape(self.nkv, R, 2, self.dim, -1).permute(0, 2, 1, 3, 4)
        return t.reshape(2 * self.nh * self.dim, -1)

    def load(self, get):
        q, qc = self._by_kv_head(get(self._n("q"))), self._by_kv_head(get(self._n("q") + self.names["conv"]))
        self.w_in = _projection(torch.cat([q, get(self._n("k")), get(self._n("v"))], 0).contiguous())
        self.conv = torch.cat([qc, get(self._n("k") + self.names["conv"]), get(self._n("v") + self.names["conv"])],
                              0).float().contiguous()
        self.w_o = _projection(get(self._n("o")))
        l = {k: get(self._n(k)).double() for k in ("lq1", "lk1", "lq2", "lk2")}
        # one number for the layer, made once from the stored vectors
        self.lam = float(torch.exp((l["lq1"] * l["lk1"]).sum()) - torch.exp((l["lq2"] * l["lk2"]).sum())) + self.diff

    def cache_need(self):
        from .base import StateNeed
        return (StateNeed((max(self.taps - 1, 0), self.channels)),
                KvNeed(2 * self.nkv, self.dim, self.window, v_dim=self.vdim, v_heads=self.nkv))

    def check(self, dtype):
        if max(self.dim, self.vdim) > ops.WINDOW_ATTENTION_MAX_DIM:
            raise ValueError(f"{self.prefix}: head sizes {self.dim} and {self.vdim} (at most {ops.WINDOW_ATTENTION_MAX_DIM})")
        if not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError(f"{self.prefix}: {self.taps} taps (at most {ops.SHORT_CONV_MAX_TAPS})")
        cos, _ = self.position.tables("cpu")
        if cos is not None and 2 * cos.shape[1] > self.dim:
            raise ValueError(f"{self.prefix}: the rotation turns {2 * cos.shape[1]} values of maps of {self.dim}")

    def forward(self, h, ctx, cache, owner=True):
        N, act, dev = h.shape[0], h.dtype, h.device
        conv_state, kv = cache
        nq, nk = 2 * self.nh, 2 * self.nkv
        cap = self.position.capacity
        if cap is not None and ctx.max_position >= cap:
            raise ValueError(f"position {ctx.max_position} is beyond the position encoding's capacity {cap}")
        proj = linear(h, self.w_in, torch.float32)          # [N, q | k | v] float
        mixed = torch.empty((N, self.channels), dtype=torch.float32, device=dev)
        ops.short_conv(proj, self.conv, None, conv_state.state, ctx.tok_seq, ctx.tok_pos, ctx.seq_start, ctx.seq_past,
                       ctx.seq_slot, mixed)
        q = torch.empty((N, nq * self.dim), dtype=act, device=dev)
        table = ctx.page_table(kv.group)
        ops.window_intake(mixed, None, q, kv.k_pages, kv.v_pages, table, ctx.tok_seq, ctx.tok_pos, None, None, 0.0,
                          nq, nk, self.dim, self.vdim, write_kv=owner, rotation=self.position.tables(dev), v_share=2)
        maps = torch.empty((N, nq * self.vdim), dtype=act, device=dev)
        if act == torch.bfloat16 and not ctx.one_token_each and ops.window_prefill_takes(self.dim, self.vdim):
            ops.window_attention_prefill_bf16(q, kv.k_pages, kv.v_pages, table, ctx.seq_start, ctx.seq_past, maps,
                                              self.scale, nq, nk, self.dim, self.vdim, window=self.window or 0, v_share=2)
        else:
            ops.window_attention(q, kv.k_pages, kv.v_pages, table, ctx.tok_seq, ctx.tok_pos, maps, self.scale, nq, nk,
                                 self.dim, self.vdim, window=self.window or 0, v_share=2)
        o = torch.empty((N, self.nh * self.vdim), dtype=act, device=dev)
        ops.diff_heads(maps, o, self.lam, self.norm_eps, 1.0 - self.diff, self.nkv, self.nh // self.nkv, self.vdim)
        return linear_for_sum(o, self.w_o)


class ParallelMixers(Mixer):
    """Several mixers side by side that read the same input; the result is sum_i scale_i * mixer_i(h).  Each keeps
    what it needs for a sequence: the cache need is the tuple of theirs, and so is the cache view."""
    takes_scaled_rows = False

    def __init__(self, mixers: list, scales: list):
        if len(mixers) != len(scales) or not mixers:
            raise ValueError("one scale for each of the mixers")
        self.mixers, self.scales = list(mixers), [float(s) for s in scales]

    @property
    def capturable(self):
        return all(getattr(m, "capturable", False) for m in self.mixers)

    def tensor_specs(self):
        specs = {}
        for m in self.mixers:
            specs.update(m.tensor_specs())
        return specs

    def load(self, get):
        for m in self.mixers:
            m.load(get)

    def check(self, dtype):
        for m in self.mixers:
            m.check(dtype)

    def cache_need(self):
        return tuple(m.cache_need() for m in self.mixers)

    def forward(self, h, ctx, cache, owner=True):
        terms = []
        for m, s, c in zip(self.mixers, self.scales, cache):
            y = m.forward(h, ctx, c, owner)
            if isinstance(y, WeightedDeltas):
                terms += [(t, s * w, b) for t, w, b in y.terms]
            else:
                terms.append((y, s, None))
        return WeightedDeltas(terms)
