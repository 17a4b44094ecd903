"""The Nilepel decoder put together from parts, and its entry in the registry.

Every layer is a pre-norm layer with RMSNorms (parts.PreNormBlock): x <- x + mixer(norm1(x)); x <- x + ff(norm2(x)), the
second half only where the layer has a feed-forward.  The mixer is one of three, chosen by the layer's type:
"attention": grouped-query attention without biases whose first values are turned in pairs (2i, 2i + 1), over runs of
positions counted from the sequence's start, with a learned sink in every softmax; "attention_2": the same with biases,
q/k norms, a rotation of halves whose long waves are stretched, a sliding window, and one output gate a head, whose
keys and values may be an earlier layer's (both parts.GatedWindowAttention); "latent_attention": keys and values of
all heads from one normed latent a token beside one turned key part, over a sliding window (parts.LatentAttention).
The feed-forward is a gated product with bounded inputs (parts.GatedMlp) or a mixture of silu-gated experts behind a
router that scores all experts, picks within the best groups and weighs with the scaled scores, beside one expert that
every token passes through a gate of its own (parts.RoutedExperts).  The embedding is scaled; RMSNorm and an output
matrix of its own at the end.  Layers take their sizes from their own entry of config.json's `layers`.
Tensor names: embed; l<i>.norm1|norm2; l<i>.mix.*; l<i>.mlp.gate|up|down; l<i>.mlp.e<j>.gate|up|down, l<i>.mlp.router,
l<i>.mlp.shared.gate|up|down|sg; final.norm; head.
"""
from __future__ import annotations

from ..config.nilepel import NilepelConfig
from ..config.registry import register_architecture
from ..parts import (RmsNorm, NoPosition, RotaryInterleaved, RotaryByWavelength, GatedWindowAttention, LatentAttention,
                     GatedMlp, RoutedExperts, PreNormBlock)
from .decoder import DecoderModel, LayerRun, TokenEmbedding, OutputHead

DEFAULT_POSITIONS = 1 << 16      # rows of the rotation's tables when the caller names no longest sequence


def _rotation(rot, capacity, pairing):
    if rot.dims == 0:
        return NoPosition()
    if pairing == "pairs" and rot.scaling is None:
        return RotaryInterleaved(rot.base, rot.dims, capacity)
    sc = rot.scaling
    return RotaryByWavelength(rot.base, rot.dims, capacity, pairing=pairing,
                              **({} if sc is None else dict(factor=sc.factor, low=sc.low, high=sc.high, original=sc.original)))


def _reach(layer):
    """How far back a layer's mask lets a query see (None: any distance)."""
    m = layer.mixer
    return m.chunk if layer.type == "attention" else m.window


def _mixer(cfg, i, p, capacity, cache_window):
    layer, W, eps = cfg.layers[i], cfg.width, cfg.eps_f32
    m = layer.mixer
    if layer.type == "latent_attention":
        return LatentAttention(p, W, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, position=_rotation(m.rot, capacity, "pairs"),
                               norm_eps=eps, scale=m.scale, window=m.window, gate=None)
    if layer.type == "attention":
        return GatedWindowAttention(p, W, m.heads, m.kv_heads, m.dim, m.vdim, position=_rotation(m.rot, capacity, "pairs"),
                                    scale=m.scale, chunk=m.chunk, sink=True, shared_kv=m.kv_from is not None,
                                    cache_window=cache_window)
    return GatedWindowAttention(p, W, m.heads, m.kv_heads, m.dim, m.vdim, position=_rotation(m.rot, capacity, "halves"),
                                qk_norm_eps=eps, scale=m.scale, window=m.window, sink=True, bias=True, gate="head",
                                shared_kv=m.kv_from is not None, cache_window=cache_window)


def _feed_forward(p, W, c):
    names = ("gate", "up", "down")
    if c.kind == "dense":
        return GatedMlp(p, W, c.ff, ("swiglu_limit", c.limit), names=names)
    shared = None if c.shared_ff is None else GatedMlp(p + "shared.", W, c.shared_ff, "silu", names=names)
    return RoutedExperts(p, W, c.ff, c.experts, c.top, "silu", router_bias=False, gated=True, router="scores",
                         n_groups=c.groups, keep_groups=c.keep_groups, shared=shared, route_scale=c.route_scale,
                         shared_gate=None if shared is None else "shared.sg")


def build_nilepel(cfg: NilepelConfig, max_positions: int | None = None) -> DecoderModel:
    W, eps = cfg.width, cfg.eps_f32
    capacity = max_positions or DEFAULT_POSITIONS
    n = len(cfg.layers)
    # layers that read one cache: it keeps what the one that sees furthest needs
    source = [cfg.kv_source(i) for i in range(n)]
    keeps = {}
    for i, s in enumerate(source):
        reach = _reach(cfg.layers[i])
        keeps[s] = None if (s in keeps and keeps[s] is None) or reach is None else max(keeps.get(s, 0), reach)
    caches = {s: c for c, s in enumerate(sorted(set(source)))}
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mixer = _mixer(cfg, i, p + "mix.", capacity, keeps[source[i]])
        norm2 = ff = None
        if layer.mlp is not None:
            norm2, ff = RmsNorm(p + "norm2", W, eps), _feed_forward(p + "mlp.", W, layer.mlp)
        blocks.append(PreNormBlock(RmsNorm(p + "norm1", W, eps), mixer, norm2, ff))
    schedule = [LayerRun(i, caches[source[i]]) for i in range(n)]
    embedding = TokenEmbedding("embed", cfg.vocab, W, scale=cfg.embedding_scale)
    return DecoderModel(cfg, embedding, blocks, schedule, RmsNorm("final.norm", W, eps), OutputHead("head", cfg.vocab, W))


NILEPEL = register_architecture("Nilepel", NilepelConfig, build_nilepel, model_types=("nilepel",))
