"""The Repolix decoder put together from parts, and its entry in the registry.

Every layer is a pre-norm layer with RMSNorms whose sublayers' results are multiplied channel by channel before they are
added (parts.PreNormBlock with scales): x <- x + ls1 * mixer(norm1(x)); x <- x + ls2 * ff(norm2(x)), the second half
only where the layer has a feed-forward.  The mixer is one of three, chosen by the layer's type: a state space with a
scalar decay a head (parts.StateSpaceMixer), the delta rule with a decay for every key channel
(parts.ChannelDeltaMixer), or grouped-query attention in two softmax maps over the same values behind short
convolutions, with a partial rotation whose long waves are stretched, and a sliding window
(parts.DifferentialAttention).  The feed-forward is a mixture of gated experts with bounded inputs behind a router that
scores all experts, picks within the best groups, and counts some of its outputs as the identity; one more such expert
is passed by every token (parts.RoutedExperts with a shared parts.GatedMlp).  The embedding is scaled; RMSNorm and an
output matrix of its own at the end.  Layers take their sizes from their own entry of config.json's `layers`.
Tensor names: embed; l<i>.norm1|norm2; l<i>.ls1|ls2; l<i>.mix.*; l<i>.mlp.e<j>.gate|up|down, l<i>.mlp.router|correction,
l<i>.mlp.shared.gate|up|down; final.norm; head.
"""
from __future__ import annotations

from ..config.repolix import RepolixConfig
from ..config.registry import register_architecture
from ..parts import (RmsNorm, RotaryScaledHalfSplit, StateSpaceMixer, ChannelDeltaMixer, DifferentialAttention, GatedMlp,
                     RoutedExperts, PreNormBlock)
from .decoder import DecoderModel, LayerRun, TokenEmbedding, OutputHead

DEFAULT_POSITIONS = 1 << 16      # rows of the rotation's tables when the caller names no longest sequence


def _mixer(kind, p, W, m, eps, max_positions, middle_rank):
    if kind == "mamba2":
        return StateSpaceMixer(p, W, m.heads, m.vdim, m.state, m.groups, m.conv, norm_groups=m.norm_groups, norm_eps=eps)
    if kind == "channel_delta":
        mixer = ChannelDeltaMixer(p, W, m.heads, m.kv_heads, m.dim, m.vdim, m.conv, norm_eps=eps)
        if middle_rank is not None:
            mixer.set_ranks(middle_rank, middle_rank)
        return mixer
    sc = m.rot_scaling
    position = RotaryScaledHalfSplit(m.rot_base, m.rot_dims, max_positions or DEFAULT_POSITIONS,
                                     **({} if sc is None else dict(factor=sc.factor, original=sc.original, fast=sc.fast,
                                                                   slow=sc.slow)))
    return DifferentialAttention(p, W, m.heads, m.kv_heads, m.dim, m.vdim, m.conv, diff=m.diff, norm_eps=eps,
                                 position=position, scale=m.scale, window=m.window)


def _feed_forward(p, W, c):
    act = lambda e: ("swiglu_limit", e.limit)
    shared = None
    if c.shared is not None:
        shared = GatedMlp(p + "shared.", W, c.shared.ff, act(c.shared), names=("gate", "up", "down"))
    return RoutedExperts(p, W, c.expert.ff, c.experts, c.top, act(c.expert), gated=True, router="scores",
                         n_groups=c.groups, keep_groups=c.keep_groups, identity=c.identity, shared=shared)


def build_repolix(cfg: RepolixConfig, max_positions: int | None = None) -> DecoderModel:
    W, eps = cfg.width, cfg.eps_f32
    embedding = TokenEmbedding("embed", cfg.vocab, W, scale=cfg.embedding_scale)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mixer = _mixer(layer.type, p + "mix.", W, layer.mixer, eps, max_positions, cfg.middle_rank)
        norm2 = ff = None
        if layer.mlp is not None:
            norm2, ff = RmsNorm(p + "norm2", W, eps), _feed_forward(p + "mlp.", W, layer.mlp)
        blocks.append(PreNormBlock(RmsNorm(p + "norm1", W, eps), mixer, norm2, ff, scale_prefix=p, hidden=W))
    schedule = [LayerRun(i, i) for i in range(len(blocks))]
    return DecoderModel(cfg, embedding, blocks, schedule, RmsNorm("final.norm", W, eps), OutputHead("head", cfg.vocab, W))


REPOLIX = register_architecture("Repolix", RepolixConfig, build_repolix, model_types=("repolix",))
