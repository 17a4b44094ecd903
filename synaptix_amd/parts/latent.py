"""Latent attention: keys and values of all heads are made from one small latent a token, and only that latent and one
rotated key part are cached.

With h the mixer's input, per token:   q = W_q h, laid out head by head as [dim unrotated | rot_dim rotated];
W_dkv h = [latent (rank) | rotated key part (rot_dim)];  c = RMSNorm(latent) * gain;  per head the unrotated key is
W_uk[h] c and the value W_uv[h] c;  score = scale (q_nope . k_nope + rot(q_rot) . rot(k_rot));  causal, or a sliding
window of the last `window` keys;  softmax;  the heads' results times sigmoid of a gate (one number a head, or one a
value);  W_o on the concatenated heads.

Computed with the up-projections moved to the query's side, which is the same sums in another order:
    q_nope . (W_uk[h] c_j) = (W_uk[h]^T q_nope) . c_j          the query in the latent's space ("absorbed")
    sum_j p_j W_uv[h] c_j  = W_uv[h] (sum_j p_j c_j)           the weights meet the latents, then one small product
so that attention is one shared key row [c | k_rot] of rank + rot_dim values a token for all heads, whose first
`rank` values are also its value.  The cache group has one kv head with rows [c | k_rot] and the latent once more
transposed as the value page (what the attention kernels' second product reads along the keys).
Scores, weights, the latent's norm, the rotation and the gates are 32-bit in both engine types.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import KvNeed
from .linear import Matrix, linear, linear_for_sum, deferred_product
from .mixer import Mixer, _projection
from .position import Position, NoPosition


class LatentAttention(Mixer):
    takes_scaled_rows = True      # (as GatedWindowAttention: the products at both ends take a norm's halves)
    capturable = True

    NAMES = {"q": "q", "down": "dkv", "down_norm": "dkv.norm", "up_k": "uk", "up_v": "uv", "g": "g", "o": "o"}
    GATES = (None, "head", "value")

    def __init__(self, prefix: str, hidden: int, n_heads: int, dim: int, rot_dim: int, v_dim: int, rank: int, *,
                 position: Position | None = None, norm_eps: float = 1e-6, scale: float | None = None,
                 window: int | None = None, gate: str | None = None, names: dict | None = None):
        """position: a rotation of interleaved pairs (Position.tables) applied to the rot_dim parts of queries and
        keys; gate: None, "head" (sigmoid of one number a head) or "value" (of one number for each value)."""
        if gate not in self.GATES:
            raise ValueError(f"{prefix}: gate {gate!r} (one of {self.GATES})")
        if min(n_heads, dim, v_dim, rank) <= 0 or rot_dim < 0:
            raise ValueError(f"{prefix}: sizes must be positive")
        self.prefix, self.hidden = prefix, hidden
        self.nh, self.dim, self.rot, self.vdim, self.rank = n_heads, dim, rot_dim, v_dim, rank
        self.position = position or NoPosition()
        self.norm_eps = float(norm_eps)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(dim + rot_dim)
        self.window, self.gate = window, gate
        self.names = dict(self.NAMES, **(names or {}))
        self.w_in = self.w_o = self.w_uk_t = self.w_uv = self.gain = None

    def _n(self, key):
        return self.prefix + self.names[key]

    def _gate_width(self):
        return {None: 0, "head": self.nh, "value": self.nh * self.vdim}[self.gate]

    def tensor_specs(self):
        H = self.hidden
        specs = {self._n("q"): TensorSpec((self.nh * (self.dim + self.rot), H)),
                 self._n("down"): TensorSpec((self.rank + self.rot, H)),
                 self._n("down_norm"): TensorSpec((self.rank,), "gain"),
                 self._n("up_k"): TensorSpec((self.nh * self.dim, self.rank)),
                 self._n("up_v"): TensorSpec((self.nh * self.vdim, self.rank)),
                 self._n("o"): TensorSpec((H, self.nh * self.vdim))}
        if self.gate:
            specs[self._n("g")] = TensorSpec((self._gate_width(), H))
        return specs

    def load(self, get):
        # one product for the queries, the latent with its rotated key part, and the gate
        rows = [get(self._n("q")), get(self._n("down"))] + ([get(self._n("g"))] if self.gate else [])
        self.w_in = _projection(torch.cat(rows, 0))
        self.w_o = _projection(get(self._n("o")))
        self.gain = get(self._n("down_norm"))
        # W_uk[h] as [rank, dim]: the query's product with it runs along dim
        self.w_uk_t = get(self._n("up_k")).view(self.nh, self.dim, self.rank).transpose(1, 2).contiguous()
        self.w_uv = get(self._n("up_v")).view(self.nh, self.vdim, self.rank).contiguous()

    def cache_need(self):
        return KvNeed(1, self.rank + self.rot, self.window, v_dim=self.rank)

    def check(self, dtype):
        if not ops.latent_attention_takes(self.rank, self.rot, dtype):
            raise ValueError(f"{self.prefix}: a cache row of {self.rank} + {self.rot} values (at most "
                             f"{ops.LATENT_ATTENTION_MAX_ROW}; in bfloat16 multiples of 16 up to {ops.LATENT_TILED_MAX_RANK} "
                             f"and {ops.LATENT_TILED_MAX_ROW} together)")
        cos, _ = self.position.tables("cpu")
        if cos is not None and 2 * cos.shape[1] > self.rot:
            raise ValueError(f"{self.prefix}: the rotation turns {2 * cos.shape[1]} values, the rotated part has {self.rot}")

    def forward(self, h, ctx, cache, owner=True):
        N, act, dev = h.shape[0], h.dtype, h.device
        nh, dim, rot, rank, vdim = self.nh, self.dim, self.rot, self.rank, self.vdim
        R = rank + rot
        proj = linear(h, self.w_in, torch.float32)          # [N, queries | latent, key part | gate] float
        q_nope = torch.empty((N, nh * dim), dtype=act, device=dev)
        q_full = torch.empty((N, nh * R), dtype=act, device=dev)
        cos, sin = self.position.tables(dev)
        table = ctx.page_table(cache.group)
        # (bf16 whose sizes the tiles on the matrix cores take: the value pages lie in that kernel's order)
        tiled = act == torch.bfloat16 and ops.latent_attention_tiled(rank, rot)
        ops.latent_intake(proj, self.gain, self.norm_eps, cos, sin, q_nope, q_full, cache.k_pages, cache.v_pages, table,
                          ctx.tok_seq, ctx.tok_pos, nh, dim, rot, rank, ctx.max_position, write_kv=owner, v_fragments=tiled)
        # the query in the latent's space, into the first `rank` places of each head's row
        ops.heads_product(q_nope.view(N, nh, dim), self.w_uk_t, q_full.view(N, nh, R))
        o_lat = torch.empty((N, nh * rank), dtype=act, device=dev)
        floats = ops.latent_attention_workspace(N, nh, ctx.n_seqs, rank, table.shape[1]) if tiled else 0
        ops.latent_attention(q_full, cache.k_pages, cache.v_pages, table, ctx.tok_seq, ctx.tok_pos, o_lat, self.scale, nh,
                             rank, rot, window=self.window or 0, seqs=(ctx.seq_start, ctx.seq_past) if tiled else None,
                             workspace=ctx.scratch("latent_attention", floats) if floats else None)
        o = torch.empty((N, nh * vdim), dtype=act, device=dev)
        gate = proj[:, nh * (dim + rot) + R:] if self.gate else None
        ops.heads_product(o_lat.view(N, nh, rank), self.w_uv, o.view(N, nh, vdim), gate=gate,
                          gate_per_value=self.gate == "value")
        return deferred_product(o, self.w_o)
