"""Small Nilepel configurations for the tests, their model folders (random weights), and the plain model's logits."""
from __future__ import annotations

import copy
import os
import tempfile

import torch

from synaptix_amd.config import NilepelConfig
from synaptix_amd import write_random_model
from plain_nilepel import PlainNilepel


def chunked(heads, kv_heads, dim, vdim, chunk=None, dims=None, base=10000.0, scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 8.0 * dim ** -0.5,
         "rot": {"base": base, "dims": dim if dims is None else dims}}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "attention", m


def windowed(heads, kv_heads, dim, vdim, window=None, dims=None, base=10000.0, scaling=None, kv_from=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 4.0 * dim ** -0.5,
         "rot": {"base": base, "dims": dim if dims is None else dims}}
    if scaling is not None:
        m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if window is not None:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "attention_2", m


def latent(heads, dim, rot_dim, vdim, rank, window=None, base=10000.0, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
         "scale": scale if scale is not None else 12.0 * (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": rot_dim}}
    if window is not None:
        m["mask"] = {"size": window}
    return "latent_attention", m


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff, experts, top, groups=None, scale=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    if scale is not None:
        router["scale"] = scale
    d = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        d["shared"] = {"ff": shared}
    return d


def config(vocab, width, layers, eps=1e-6, scale=None):
    d = {"architecture": "Nilepel", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "layers": [{"type": t, "mixer": m, "mlp": f} for (t, m), f in layers]}
    if scale is not None:
        d["embedding"] = {"scale": scale}
    return d


# P: the three mixers in an order of their own; windows and runs shorter than a page; a layer that reads the keys of the
#    first one through a longer window than its owner's (the cache keeps the longer one); values of another size than
#    the keys; part of a head turned, with stretched long waves; groups of which half stay; a shared expert; one layer
#    without a feed-forward.
# Q: sizes that are multiples of nothing (a width of 72, keys of 12, values of 10, a latent of 20 beside 6 turned values,
#    an odd vocabulary), as many kv heads as heads, a run of exactly one page and a window of a page and a token, a layer
#    that sees every earlier key, all experts chosen, no groups, no shared expert, no factor on the weights, no scale on
#    the embedding.
# R: sizes at which the products run on the matrix cores and prompts' attention in tiles; a window that no test sequence
#    outgrows; runs of two pages; sixteen experts in four groups; two layers reading one layer's keys.
# T: a width, feed-forwards and a vocabulary that are multiples of two at most; a layer over runs that reads the keys of a
#    windowed layer (turned in halves by that layer, its own queries in pairs); an expert layer whose groups all stay.
# S: one head everywhere, a window of one and of two, runs of one position, the top one of two experts: a choice that the
#    rounding of bfloat16 activations can turn changes a token's result altogether, so this one is 32-bit only.
CONFIGS = {
    "P": config(300, 64, [(windowed(4, 2, 16, 24, window=20, dims=8, scaling=(4.0, 1.0, 4.0, 64)), dense(48, 0.9)),
                          (latent(4, 8, 8, 12, 32, window=33), moe(32, 6, 2, groups=(2, 1), scale=1.5, shared=24)),
                          (chunked(6, 3, 16, 8, chunk=24, dims=12), None),
                          (windowed(4, 2, 16, 24, window=37, dims=8, scaling=(4.0, 1.0, 4.0, 64), kv_from=0),
                           moe(24, 8, 3, groups=(4, 2), scale=0.7, shared=16)),
                          (latent(2, 16, 4, 16, 16, window=5, base=500.0), dense(80, 2.0))], scale=3.0),
    "Q": config(257, 72, [(chunked(3, 3, 12, 10, chunk=64), moe(20, 5, 5)),
                          (latent(3, 10, 6, 14, 20, window=65), dense(50, 0.5)),
                          (windowed(2, 1, 20, 6, window=65, dims=4, base=300.0), moe(12, 3, 1, shared=28)),
                          (latent(5, 6, 2, 4, 9), None),
                          (chunked(4, 1, 10, 18, dims=2), dense(30, 3.0))], eps=1e-5),
    "R": config(512, 128, [(windowed(8, 2, 64, 32, window=4096, dims=32, scaling=(8.0, 1.0, 2.0, 128), base=1e6), moe(64, 16, 4, groups=(4, 2), scale=2.0, shared=80)),
                           (latent(4, 32, 16, 32, 64, window=100), dense(256, 1.5)),
                           (windowed(8, 2, 64, 32, window=70, dims=32, scaling=(8.0, 1.0, 2.0, 128), base=1e6, kv_from=0), None),
                           (chunked(4, 4, 32, 64, chunk=128, dims=16), moe(32, 8, 2, shared=64)),
                           (windowed(8, 2, 64, 32, dims=32, scaling=(8.0, 1.0, 2.0, 128), base=1e6, kv_from=2), dense(128, 1.0))],
                scale=11.3),
    "T": config(131, 90, [(windowed(5, 5, 6, 14, window=9, dims=6), moe(22, 6, 2, groups=(3, 3), scale=0.5, shared=10)),
                          (latent(3, 6, 4, 10, 14, window=70), dense(34, 1.2)),
                          (chunked(5, 5, 6, 14, chunk=40, dims=4, kv_from=0), dense(18, 0.8))], scale=1.7),
    "S": config(101, 40, [(windowed(1, 1, 8, 8, window=1), moe(16, 2, 1)),
                          (chunked(1, 1, 6, 12, chunk=1, dims=2), None),
                          (latent(1, 4, 2, 6, 5, window=2), dense(24, 1.0)),
                          (windowed(1, 1, 8, 8, window=2, kv_from=0), None)], scale=2.0),
}
SEEDS = {"P": 41, "Q": 42, "R": 43, "S": 44, "T": 45}


def dtypes_of(name: str) -> list:
    return ["float32"] if name == "S" else ["float32", "bfloat16"]


def cases(names) -> list:
    """(configuration, engine type) pairs for pytest.mark.parametrize."""
    return [(n, d) for n in names for d in dtypes_of(n)]


_tmp = None
_folders, _plain, _logits = {}, {}, {}


def model_folder(name: str) -> str:
    """Random bf16 weights, drawn wide enough that every branch carries weight; the configurations' scales make the
    attention peaked, so that a lost or wrong key moves the logits.  The sinks are drawn around 1.5 so that they hold a
    good part of most softmax sums, the shared experts' gates wide so that they differ from token to token, and the
    routers wider still so that the scores of a token's experts lie apart: where the rounding of bfloat16 activations
    turns a near tie between the last expert chosen and the first one left out, that expert carries a small weight."""
    global _tmp
    if name not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="synaptix_amd_nilepel_")
        cfg = NilepelConfig.from_dict(copy.deepcopy(CONFIGS[name]))
        folder = os.path.join(_tmp.name, name)
        g = torch.Generator().manual_seed(900 + SEEDS[name])
        extra = {}
        for i, l in enumerate(cfg.layers):
            if l.type != "latent_attention":
                extra[f"l{i}.mix.sink"] = (1.5 + torch.randn(l.mixer.heads, generator=g)).to(torch.bfloat16)
            if l.mlp is not None and l.mlp.kind == "moe":
                extra[f"l{i}.mlp.router"] = (0.7 * torch.randn(l.mlp.experts, cfg.width, generator=g)).to(torch.bfloat16)
                if l.mlp.shared_ff is not None:
                    extra[f"l{i}.mlp.shared.sg"] = (0.3 * torch.randn(1, cfg.width, generator=g)).to(torch.bfloat16)
        write_random_model(folder, cfg, SEEDS[name], std=0.08, gain_std=0.3, extra_tensors=extra)
        _folders[name] = folder
    return _folders[name]


def plain_model(name: str) -> PlainNilepel:
    if name not in _plain:
        _plain[name] = PlainNilepel.from_folder(model_folder(name))
    return _plain[name]


def plain_logits(name: str, tokens) -> torch.Tensor:
    key = (name, tuple(tokens))
    if key not in _logits:
        _logits[key] = plain_model(name).logits(list(tokens))
    return _logits[key]


def tokens_for(name: str, n: int, seed: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CONFIGS[name]["vocab"], (n,), generator=g).tolist()


def random_config(seed: int) -> dict:
    """A configuration drawn from a seed: layer kinds in any order, head counts, sizes (multiples of sixteen and not),
    masks from one position to none, readers of earlier layers' keys, every shape of the experts' router."""
    import random
    rng = random.Random(seed)
    width, vocab = rng.choice([64, 96, 128, 192, 256]), rng.choice([200, 384, 512, 1000])
    layers, owners = [], []
    for i in range(rng.randint(2, 6)):
        kind = rng.choice(["runs", "window", "latent"])
        heads = rng.choice([2, 4, 6, 8, 12])
        kv = rng.choice([h for h in (1, 2, 3, 4, 6, 8, 12) if heads % h == 0])
        dim, vdim = rng.choice([16, 32, 48, 64, 96, 128, 24, 40]), rng.choice([16, 32, 48, 64, 96, 24, 80])
        size = rng.choice([None, 1, 7, 16, 31, 64, 65, 100, 128, 200, 300])
        if kind == "runs":
            dims = rng.choice([n for n in (0, 2, 8, 16, dim) if n <= dim])
            mixer = chunked(heads, kv, dim, vdim, chunk=size, dims=dims, base=rng.choice([100.0, 1e4, 5e5]), scale=2.0 * dim ** -0.5)
            if dims == 0:
                mixer[1].pop("rot")
            owners.append((i, heads, kv, dim, vdim))
        elif kind == "window":
            dims = rng.choice([n for n in (2, 8, 16, 32, dim) if n <= dim])
            stretch = rng.choice([None, (4.0, 1.0, 4.0, 64), (8.0, 1.0, 4.0, 1024), (2.0, 0.5, 3.0, 300), (32.0, 1.0, 2.0, 16)])
            how = dict(window=size, scaling=stretch, base=rng.choice([1e4, 2.5e5]))
            if owners and rng.random() < 0.5:
                o = rng.choice(owners)
                mixer = windowed(o[1], o[2], o[3], o[4], dims=min(dims, o[3]) // 2 * 2, kv_from=o[0], scale=o[3] ** -0.5, **how)
            else:
                mixer = windowed(heads, kv, dim, vdim, dims=dims, scale=dim ** -0.5, **how)
                owners.append((i, heads, kv, dim, vdim))
        else:
            rot, nope = rng.choice([0, 2, 8, 16, 32, 64]), rng.choice([8, 16, 32, 64, 24])
            mixer = latent(heads, nope, rot, rng.choice([16, 32, 48, 64, 40]), rng.choice([16, 32, 64, 128, 96, 40, 256]),
                           window=size, scale=3.0 * (nope + rot) ** -0.5)
            if rot == 0:
                mixer[1].pop("rot")
        ff = rng.choice(["dense", "moe", "moe", None])
        if ff == "dense":
            mlp = dense(rng.choice([32, 64, 100, 256, 512]), rng.choice([0.5, 1.5, 7.0]))
        elif ff == "moe":
            groups = rng.choice([None, (1, 1), (2, 1), (4, 2), (4, 4), (8, 3)])
            per, count = rng.choice([1, 2, 4]), groups[0] if groups else rng.choice([1, 2, 3])
            top = rng.randint(1, min(per * (groups[1] if groups else count), 6))
            mlp = moe(rng.choice([16, 32, 64, 96, 40]), per * count, top, groups=groups, scale=rng.choice([None, 1.5, 0.5, 2.5]),
                      shared=rng.choice([None, 32, 64, 128, 24]))
        else:
            mlp = None
        layers.append((mixer, mlp))
    return config(vocab, width, layers, eps=rng.choice([1e-6, 1e-5]), scale=rng.choice([None, 0.5, 2.0, width ** 0.5]))


def random_model(seed: int):
    """(typed configuration, model folder, plain model) of random_config(seed)."""
    global _tmp
    if _tmp is None:
        _tmp = tempfile.TemporaryDirectory(prefix="synaptix_amd_nilepel_")
    cfg = NilepelConfig.from_dict(random_config(seed))
    folder = os.path.join(_tmp.name, f"random{seed}")
    if not os.path.isdir(folder):
        g = torch.Generator().manual_seed(seed)
        extra = {f"l{i}.mix.sink": (1.0 + torch.randn(l.mixer.heads, generator=g)).to(torch.bfloat16)
                 for i, l in enumerate(cfg.layers) if l.type != "latent_attention"}
        write_random_model(folder, cfg, seed, std=0.06, gain_std=0.3, extra_tensors=extra)
    return cfg, folder, PlainNilepel.from_folder(folder)
