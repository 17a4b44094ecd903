"""Feed-forward parts.  Here: the gated MLP  down( act(gate(h)) * up(h) ), dense.

crates/synaptix-models/llm/common/src/model.rs:1670-1691; activation silu(z) = z / (1 + e^-z) in
32-bit as crates/synaptix-kernels-cuda/src/cu/fused/mlp/silu_and_mul.cu:11-52.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import Part
from .linear import Matrix, linear, linear_for_sum, deferred_product, as_rows, ScaledRows


class FeedForward(Part):
    """Interface: forward(h [N, hidden] activation type, ctx) -> residual delta [N, hidden] float."""

    takes_scaled_rows = False     # as Mixer.takes_scaled_rows

    def forward(self, h, ctx):
        raise NotImplementedError


class GatedMlp(FeedForward):
    takes_scaled_rows = True
    capturable = True

    NAMES = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "silu", names=None):
        """names: the tensors of the gate, up and down products behind `prefix` (default: NAMES)."""
        self.names = tuple(names or self.NAMES)
        try:
            ops.activation_code(activation)       # the kernels apply it by its code; an unknown name is refused here
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        self.prefix, self.hidden, self.intermediate, self.activation = prefix, hidden, intermediate, activation
        self.w_gate_up = self.w_down = None
        self.paired = False      # gate and up rows in turns of 16: the activation runs inside the product

    def tensor_specs(self):
        p, (gate, up, down) = self.prefix, self.names
        return {
            p + gate: TensorSpec((self.intermediate, self.hidden)),
            p + up: TensorSpec((self.intermediate, self.hidden)),
            p + down: TensorSpec((self.hidden, self.intermediate)),
        }

    def load(self, get):
        p = self.prefix
        gate, up = get(p + self.names[0]), get(p + self.names[1])
        self.paired = (gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16
                       and self.intermediate % ops.PAIR == 0 and self.hidden % 8 == 0)
        self.w_gate_up = Matrix(ops.pair_rows(gate, up) if self.paired else torch.cat([gate, up], 0))
        self.w_down = Matrix(get(p + self.names[2]))

    def forward(self, h, ctx):
        m = torch.empty((h.shape[0], self.intermediate), dtype=h.dtype, device=h.device)
        if self.paired and h.dtype == torch.bfloat16:
            if self.w_gate_up.packed is not None and h.shape[0] <= ops.PACKED_MAX_ROWS_GATED:
                if isinstance(h, ScaledRows):      # the norm's last step is the product's epilogue
                    ops.gemm_packed(h.rows, self.w_gate_up.packed, m, paired=True, activation=self.activation,
                                    row_scale=h.row_scale)
                else:
                    ops.gemm_packed(h, self.w_gate_up.packed, m, paired=True, activation=self.activation)
            else:
                ops.gemm_swiglu(as_rows(h), self.w_gate_up.data, m, self.activation)
        else:
            h = as_rows(h)
            ops.swiglu(linear(h, self.w_gate_up, h.dtype), m, self.activation)
        return deferred_product(m, self.w_down)


class RoutedExperts(FeedForward):
    """A mixture of small experts: each token goes through `top` of them, chosen by a router, and gets the weighted sum
    of their results.

    The router (32-bit sums of the framework's own product z = W_router h), one of
        "top_logits"  the `top` largest z + bias; weights: softmax over the chosen logits only
        "scores"      s = softmax(z) over all router outputs; the choice is made on s + correction among the members of
                      the `keep_groups` best of `n_groups` equal groups of neighbours (a group's score: its largest choice
                      score); weights: the chosen s themselves (`renorm`: divided by their sum) times `route_scale`
    The experts, one of
        ungated       W_down act(W_up h), act the exact GELU
        gated         W_down act2(W_gate h, W_up h) with an activation of the gated products (ops.ACTIVATIONS; one with a
                      bound as the pair (name, bound))
    `identity`: the router's last `identity` outputs stand for experts without tensors whose result is h itself.
    `shared`: a feed-forward that every token passes as well (its result is a second term of the sum); with
    `shared_gate` that term is multiplied by sigmoid(w_sg . h), one number a token (tensor `shared_gate` [1, hidden],
    which rides along as one more row of the router's product).

    The tokens are sorted by expert on the device (no count comes back to the host), and each expert's rows meet its
    matrices in one launch for all experts (ops.experts_product).  Returns the `top` weighted results of every token
    as partial sums [top, N, hidden], which whoever adds the residual sums up (with `shared`: parts.SummedDeltas of
    those and the shared result).
    Tensors: prefix + "e<j>.up" [ff, hidden], "e<j>.down" [hidden, ff] (gated: "e<j>.gate" too), "router"
    [experts + identity, hidden], "router.b" or "correction"; `names` renames them."""
    takes_scaled_rows = False
    capturable = True

    ACTIVATIONS = ("gelu",)       # of ungated experts: the exact (erf) form, the products' epilogue
    ROUTERS = ("top_logits", "scores")

    def __init__(self, prefix: str, hidden: int, ff: int, n_experts: int, top: int, activation="gelu",
                 router_bias: bool = True, names=None, *, gated: bool = False, router: str = "top_logits",
                 n_groups: int = 1, keep_groups: int = 1, renorm: bool = False, identity: int = 0, shared=None,
                 route_scale: float = 1.0, shared_gate: str | None = None):
        if router not in self.ROUTERS:
            raise ValueError(f"{prefix}: router {router!r} (one of {self.ROUTERS})")
        if gated:
            try:
                ops.activation_code(activation)
            except ops.KernelError as e:
                raise ValueError(f"{prefix}: {e}") from None
        elif activation not in self.ACTIVATIONS:
            raise ValueError(f"{prefix}: activation {activation!r} (the experts' products apply {self.ACTIVATIONS})")
        total = n_experts + int(identity)
        if not 0 < top <= total or n_experts < 0 or identity < 0:
            raise ValueError(f"{prefix}: the {top} largest of {n_experts} experts and {identity} identities")
        if router == "scores" and (n_groups <= 0 or total % n_groups or not 0 < keep_groups <= n_groups
                                   or top > keep_groups * (total // n_groups)):
            raise ValueError(f"{prefix}: {total} router outputs in {n_groups} groups, {keep_groups} kept, {top} chosen")
        if identity and router != "scores":
            raise ValueError(f"{prefix}: identity experts come with the router that scores all outputs")
        if route_scale != 1.0 and router != "scores":
            raise ValueError(f"{prefix}: a factor on the weights comes with the router that scores all outputs")
        if shared_gate is not None and shared is None:
            raise ValueError(f"{prefix}: a gate for a shared expert that is not there")
        self.route_scale, self.shared_gate = float(route_scale), shared_gate
        self.prefix, self.hidden, self.ff, self.n_experts, self.top = prefix, hidden, ff, n_experts, top
        self.activation, self.gated, self.router = activation, bool(gated), router
        self.n_groups, self.keep_groups, self.renorm, self.identity = int(n_groups), int(keep_groups), bool(renorm), int(identity)
        self.total, self.shared = total, shared
        self.router_bias = bool(router_bias)
        if names is None:
            names = ("e{}.up", "e{}.down", "router", "correction" if router == "scores" else "router.b", "e{}.gate")
        self.names = tuple(names)
        self.w_up = self.w_down = self.w_router = self.b_router = None

    @property
    def capturable(self):
        return self.shared is None or bool(getattr(self.shared, "capturable", False))

    def tensor_specs(self):
        p, (up, down, router, bias) = self.prefix, self.names[:4]
        specs = {p + router: TensorSpec((self.total, self.hidden))}
        if self.router_bias:
            specs[p + bias] = TensorSpec((self.total,), "bias")
        for e in range(self.n_experts):
            if self.gated:
                specs[p + self.names[4].format(e)] = TensorSpec((self.ff, self.hidden))
            specs[p + up.format(e)] = TensorSpec((self.ff, self.hidden))
            specs[p + down.format(e)] = TensorSpec((self.hidden, self.ff))
        if self.shared is not None:
            specs.update(self.shared.tensor_specs())
        if self.shared_gate is not None:
            specs[p + self.shared_gate] = TensorSpec((1, self.hidden))
        return specs

    def load(self, get):
        p, (up, down, router, bias) = self.prefix, self.names[:4]
        # every expert's matrices kept once: in fragment order where type and sizes allow, else in plain rows
        if self.n_experts:
            if self.gated:      # an expert's gate and up rows in turns: one product for both, the activation its epilogue
                w_up = ops.pair_expert_rows(torch.stack([get(p + self.names[4].format(e)) for e in range(self.n_experts)]),
                                            torch.stack([get(p + up.format(e)) for e in range(self.n_experts)]))
            else:
                w_up = torch.stack([get(p + up.format(e)) for e in range(self.n_experts)]).contiguous()
            packed = ops.pack_expert_weights(w_up)
            self.w_up = w_up if packed is None else packed
            del w_up, packed
            w_down = torch.stack([get(p + down.format(e)) for e in range(self.n_experts)]).contiguous()
            packed = ops.pack_expert_weights(w_down)
            self.w_down = w_down if packed is None else packed
        rows = get(p + router)
        if self.shared_gate is not None:       # the shared expert's gate as one more row behind the router's
            rows = torch.cat([rows, get(p + self.shared_gate).to(rows.dtype)], 0)
            spare = -rows.shape[0] % 16            # (and rows of zeros up to whole fragments of 16, which nobody reads)
            if spare and rows.shape[1] % 32 == 0:
                rows = torch.cat([rows, torch.zeros((spare, rows.shape[1]), dtype=rows.dtype, device=rows.device)], 0)
        self.w_router = Matrix(rows)
        self.b_router = get(p + bias).float().contiguous() if self.router_bias else None
        if self.shared is not None:
            self.shared.load(get)

    def check(self, dtype):
        if self.total > ops.ROUTE_MAX_EXPERTS or self.top > ops.ROUTE_MAX_TOP:
            raise ValueError(f"{self.prefix}: {self.top} of {self.total} experts "
                             f"(at most {ops.ROUTE_MAX_TOP} of {ops.ROUTE_MAX_EXPERTS})")
        if self.shared is not None:
            self.shared.check(dtype)

    def forward(self, h, ctx):
        h = as_rows(h)
        N, dev = h.shape[0], h.device
        ids = torch.empty((N, self.top), dtype=torch.int32, device=dev)
        weights = torch.empty((N, self.top), dtype=torch.float32, device=dev)
        logits = linear(h, self.w_router, torch.float32)
        shared_gate = None
        if self.shared_gate is not None:
            logits, shared_gate = logits[:, :self.total], logits[:, self.total:self.total + 1]
        if self.router == "scores":
            ops.route_scores(logits, self.b_router, ids, weights, self.n_groups, self.keep_groups, self.renorm,
                             self.route_scale)
        else:
            ops.route_topk(logits.contiguous(), self.b_router, ids, weights)
        seg, tok_of, pair_of, part_of, weight_of = ops.route_sort(ids, weights, self.total)
        y = torch.empty((self.top, N, self.hidden), dtype=torch.float32, device=dev)
        if self.n_experts:
            real = seg[:self.n_experts + 1]          # the experts with matrices come first
            mid = torch.empty((N * self.top, self.ff), dtype=h.dtype, device=dev)
            if self.gated:
                ops.experts_product(h, self.w_up, mid, real, tok_of, pair_of, gated=self.activation)
            else:
                ops.experts_product(h, self.w_up, mid, real, tok_of, pair_of, gelu=True)
            ops.experts_product(mid, self.w_down, y.view(self.top * N, self.hidden), real, pair_of, part_of,
                                row_weight=weight_of)
        if self.identity:
            ops.route_identity(h, y.view(self.top * N, self.hidden), seg, self.n_experts, self.total, tok_of, part_of,
                               weight_of)
        if self.shared is not None:
            from .linear import SummedDeltas
            return SummedDeltas([y, self.shared.forward(h, ctx)], [None, shared_gate])
        return y
