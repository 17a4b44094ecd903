"""Small Repolix configurations for the tests, their model folders (random weights), and the plain model's logits."""
from __future__ import annotations

import copy
import os
import tempfile

import torch

from synaptix_amd.config import RepolixConfig
from synaptix_amd import write_random_model
from plain_repolix import PlainRepolix


def ssm(heads, vdim, state, groups, conv, norm_groups=1):
    return "mamba2", {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}


def delta(heads, kv_heads, dim, vdim, conv):
    return "channel_delta", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def attn(heads, kv_heads, dim, vdim, conv, window=None, dims=None, base=10000.0, scaling=None, diff=0.4, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "diff": diff,
         "scale": scale if scale is not None else 5.0 * dim ** -0.5, "rot": {"base": base, "dims": dim if dims is None else dims}}
    if scaling is not None:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if window is not None:
        m["mask"] = {"size": window}
    return "attention", m


def moe(ff, experts, top, identity=0, groups=None, limit=1.25, shared=None):
    router = {"experts": experts, "top": top}
    if identity:
        router["identity"] = identity
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}
    if shared is not None:
        d["shared"] = {"ff": shared[0], "limit": shared[1]}
    return d


def config(vocab, width, layers, eps=1e-6, scale=None, rank=8):
    d = {"architecture": "Repolix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "middle_rank": rank,
         "layers": [{"type": t, "mixer": m, "mlp": f} for (t, m), f in layers]}
    if scale is not None:
        d["embedding"] = {"scale": scale}
    return d


# P: the three mixers in an order of their own, a window shorter than a page, part of a map's values turned with
#    stretched long waves, identity experts, groups of which half stay, a shared expert, one layer without a feed-forward.
# Q: sizes that are multiples of nothing (a width of 72, keys of 12, states of 7 rows, values of 10, an odd vocabulary),
#    one group and one normed part, a convolution of one tap (none at all) and one of five, a window of exactly one
#    page and one of a page and a token, no identity experts, no groups, no shared expert, no scale on the embedding.
# R: sizes at which the products run on the matrix cores and prompts' attention in tiles; a window that no test
#    sequence outgrows and a layer without any; sixteen experts in four groups; states of 128 rows.
# S: one head everywhere, windows of one and of two, one expert beside one identity, the top one of them only: a choice
#    that the rounding of bfloat16 activations can turn changes a token's result altogether, so this one is 32-bit only.
CONFIGS = {
    "P": config(300, 64, [(attn(4, 2, 16, 24, 3, window=20, dims=8, scaling=(4.0, 64, 16.0, 2.0)), moe(32, 6, 3, identity=2, groups=(4, 2), shared=(48, 0.9))),
                          (ssm(4, 16, 24, 2, 4, norm_groups=2), None),
                          (delta(4, 2, 16, 24, 3), moe(24, 4, 2, identity=1, limit=0.7, shared=(16, 2.0))),
                          (ssm(6, 8, 20, 3, 2, norm_groups=3), moe(32, 6, 3, identity=2, groups=(2, 1)))], scale=4.0),
    "Q": config(257, 72, [(ssm(3, 10, 7, 1, 1), moe(20, 3, 2)),
                          (attn(3, 3, 12, 10, 4, window=64, dims=12), moe(28, 5, 5, identity=0, limit=3.0)),
                          (delta(3, 1, 12, 20, 5), None),
                          (attn(2, 1, 20, 6, 1, window=65, dims=4, base=500.0, diff=0.8), moe(12, 2, 1, identity=2, groups=(2, 2)))],
                eps=1e-5, rank=5),
    "R": config(512, 128, [(delta(8, 4, 64, 32, 3), moe(64, 16, 4, groups=(4, 2), shared=(80, 1.1))),
                           (attn(4, 2, 32, 64, 3, window=4096, dims=32, scaling=(8.0, 128, 32.0, 1.0)), moe(64, 8, 2, identity=0)),
                           (ssm(8, 32, 128, 2, 4, norm_groups=4), moe(32, 6, 2, identity=2, shared=(64, 1.5))),
                           (attn(8, 2, 64, 32, 2, dims=16, base=1e6), None)], scale=11.3, rank=16),
    "S": config(101, 40, [(attn(1, 1, 8, 8, 2, window=1, dims=8), moe(16, 1, 1, identity=1)),
                          (ssm(1, 12, 5, 1, 3), None),
                          (attn(1, 1, 6, 12, 3, window=2, dims=2), moe(8, 2, 1)),
                          (delta(1, 1, 10, 6, 2), None)], scale=2.0, rank=3),
}
SEEDS = {"P": 31, "Q": 32, "R": 33, "S": 34}


def dtypes_of(name: str) -> list:
    return ["float32"] if name == "S" else ["float32", "bfloat16"]


def cases(names) -> list:
    """(configuration, engine type) pairs for pytest.mark.parametrize."""
    return [(n, d) for n in names for d in dtypes_of(n)]


_tmp = None
_folders, _plain, _logits = {}, {}, {}


def model_folder(name: str) -> str:
    """Random bf16 weights, drawn wide enough that every branch carries weight; the configurations' scales make the
    attention peaked, so that a lost or wrong key moves the logits.  The routers' weights are drawn wider still, so that
    the scores of a token's experts lie apart, and the corrections small beside those differences (the choice then
    follows the token, not the correction alone); where the rounding of bfloat16 activations turns a near tie between
    the last expert chosen and the first one left out, the expert in question carries a small weight."""
    global _tmp
    if name not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="synaptix_amd_repolix_")
        cfg = RepolixConfig.from_dict(copy.deepcopy(CONFIGS[name]))
        folder = os.path.join(_tmp.name, name)
        g = torch.Generator().manual_seed(800 + SEEDS[name])
        extra = {}
        for i, l in enumerate(cfg.layers):
            if l.mlp is not None:
                total = l.mlp.experts + l.mlp.identity
                extra[f"l{i}.mlp.router"] = (0.4 * torch.randn(total, cfg.width, generator=g)).to(torch.bfloat16)
                extra[f"l{i}.mlp.correction"] = (0.05 * torch.randn(total, generator=g)).to(torch.bfloat16)
        write_random_model(folder, cfg, SEEDS[name], std=0.08, gain_std=0.3, extra_tensors=extra)
        _folders[name] = folder
    return _folders[name]


def plain_model(name: str) -> PlainRepolix:
    if name not in _plain:
        _plain[name] = PlainRepolix.from_folder(model_folder(name))
    return _plain[name]


def plain_logits(name: str, tokens) -> torch.Tensor:
    key = (name, tuple(tokens))
    if key not in _logits:
        _logits[key] = plain_model(name).logits(list(tokens))
    return _logits[key]


def tokens_for(name: str, n: int, seed: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CONFIGS[name]["vocab"], (n,), generator=g).tolist()
