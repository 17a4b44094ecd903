"""A plain, slow statement of the Nilepel decoder in float64 on the CPU: one function for each mechanism, whole
sequences only (no cache, no batches, no portions; attention is a full score matrix with a mask).  The oracle of the
GPU tests; it shares no code with the package.

Notation: T tokens, W the width; positions count from 0; a weight [out, in] meets a row x as x @ w.T.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def rms_norm(x, gain, eps):
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if gain is None else y * gain


# ---------------------------------------------------------------- rotations
def rates(base, dims):
    """f_i = base^(-2 i / dims), i < dims / 2."""
    return torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)


def stretched_rates(f, factor, low, high, original):
    """Long waves slowed down: wavelength l = 2 pi / f; l < original / high keeps f, l > original / low gets f / factor,
    between the two a straight blend in s = (original / l - low) / (high - low)."""
    out = f.clone()
    for i, fi in enumerate(f.tolist()):
        l = 2.0 * math.pi / fi
        if l < original / high:
            out[i] = fi
        elif l > original / low:
            out[i] = fi / factor
        else:
            s = (original / l - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate(x, f, layout, first=0):
    """x [T, ..., D]: the first 2 len(f) values of the last axis turned by position * f; the token at row t has position
    first + t.  layout "pairs": value 2i with 2i + 1; "halves": value i with i + len(f)."""
    T, n = x.shape[0], f.shape[0]
    pos = torch.arange(first, first + T, dtype=F64)
    ang = pos[:, None] * f[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [n]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    out = x.clone()
    if layout == "pairs":
        u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
        out[..., 0:2 * n:2] = u * c - v * s
        out[..., 1:2 * n:2] = v * c + u * s
    elif layout == "halves":
        u, v = x[..., :n], x[..., n:2 * n]
        out[..., :n] = u * c - v * s
        out[..., n:2 * n] = v * c + u * s
    else:
        raise ValueError(layout)
    return out


# ---------------------------------------------------------------- masks
def window_mask(T, size):
    """[T, T] bool: query i sees key j iff 0 <= i - j < size (size None: every earlier key)."""
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    m = j <= i
    return m if size is None else m & (i - j < size)


def chunk_mask(T, size):
    """[T, T] bool: query i sees key j iff j <= i and both lie in the same run of `size` positions counted from 0."""
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


# ---------------------------------------------------------------- softmax, with or without a sink
def attend(q, k, v, scale, mask, sink=None):
    """q [T, H, D], k [T, G, D], v [T, G, E], mask [T, T] bool, sink [H] or None -> [T, H, E].  Head h reads kv head
    h // (H / G).  The sink adds exp(sink_h) to the denominator and nothing to the numerator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, -math.inf)
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].expand_as(m))
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


# ---------------------------------------------------------------- mixers
def attention_chunked(h, w, p, c, kv=None):
    """Mixer "attention": no biases, pairs rotated, chunks, a sink.  Returns (delta, (k, v)) with the keys as a later
    layer would read them; with kv given it makes queries only."""
    T = h.shape[0]
    H, G, D, E = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    f = rates(c["rot"]["base"], c["rot"]["dims"])
    q = rotate((h @ w[p + "q"].T).view(T, H, D), f, "pairs")
    if kv is None:
        k = rotate((h @ w[p + "k"].T).view(T, G, D), f, "pairs")
        v = (h @ w[p + "v"].T).view(T, G, E)
    else:
        k, v = kv
    mask = chunk_mask(T, c["mask"]["size"]) if c.get("mask") else window_mask(T, None)
    o = attend(q, k, v, c["scale"], mask, w[p + "sink"])
    return o.reshape(T, H * E) @ w[p + "o"].T, (k, v)


def attention_windowed(h, w, p, c, eps, kv=None):
    """Mixer "attention_2": biases, q/k norm before the rotation of halves with stretched rates, a window, a sink, one
    output gate a head; with kv given (another layer's rotated keys and its values) it makes queries only."""
    T = h.shape[0]
    H, G, D, E = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    f = rates(c["rot"]["base"], c["rot"]["dims"])
    sc = c["rot"].get("scaling")
    if sc is not None:
        f = stretched_rates(f, sc["factor"], sc["low"], sc["high"], sc["original"])
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, D)
    q = rotate(rms_norm(q, w[p + "q.norm"], eps), f, "halves")
    if kv is None:
        k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, D)
        k = rotate(rms_norm(k, w[p + "k.norm"], eps), f, "halves")
        v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, E)
    else:
        k, v = kv
    o = attend(q, k, v, c["scale"], window_mask(T, c["mask"]["size"] if c.get("mask") else None), w[p + "sink"])
    o = o * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, H * E) @ w[p + "o"].T, (k, v)


def latent_attention(h, w, p, c, eps):
    """Mixer "latent_attention": per-head keys and values made from one normed latent a token, one rotated key part for
    all heads, a window, the ordinary softmax."""
    T = h.shape[0]
    H, D, R, E, C = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    f = rates(c["rot"]["base"], c["rot"]["dims"])
    q = (h @ w[p + "q"].T).view(T, H, D + R)
    q = torch.cat([q[..., :D], rotate(q[..., D:], f, "pairs")], -1)
    down = h @ w[p + "dkv"].T
    lat = rms_norm(down[:, :C], w[p + "dkv.norm"], eps)
    k_rot = rotate(down[:, C:].view(T, 1, R), f, "pairs")
    k = torch.cat([(lat @ w[p + "uk"].T).view(T, H, D), k_rot.expand(T, H, R)], -1)
    v = (lat @ w[p + "uv"].T).view(T, H, E)
    o = attend(q, k, v, c["scale"], window_mask(T, c["mask"]["size"] if c.get("mask") else None))
    return o.reshape(T, H * E) @ w[p + "o"].T


# ---------------------------------------------------------------- feed-forwards
def bounded_mlp(h, w, p, limit):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def silu_expert(h, w, p):
    z = h @ w[p + "gate"].T
    return (z * torch.sigmoid(z) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(z, top, groups, keep, scale):
    """z [T, E] router outputs -> (ids [T, top], weights [T, top]).  Scores are the softmax over all experts; only
    members of the `keep` groups with the largest best score can be chosen; the weights are scale * score."""
    T, E = z.shape
    s = torch.softmax(z, -1)
    allowed = torch.ones(T, E, dtype=torch.bool)
    if groups > 1:
        best = s.view(T, groups, E // groups).max(-1).values
        kept = best.topk(keep, -1).indices
        on = torch.zeros(T, groups, dtype=torch.bool)
        on.scatter_(1, kept, True)
        allowed = on[:, :, None].expand(T, groups, E // groups).reshape(T, E)
    ids = s.masked_fill(~allowed, -1.0).topk(top, -1).indices
    return ids, s.gather(1, ids) * scale


def experts(h, w, p, c):
    r = c["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    ids, wt = route(h @ w[p + "router"].T, r["top"], g["count"], g["keep"], r.get("scale", 1.0))
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), wt[t].tolist()):
            y[t] += a * silu_expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if c.get("shared") is not None:
        y = y + silu_expert(h, w, p + "shared.") * torch.sigmoid(h @ w[p + "shared.sg"].T)
    return y


# ---------------------------------------------------------------- the model
class PlainNilepel:
    def __init__(self, config: dict, weights: dict):
        self.c = config
        self.w = {k: v.to(F64) for k, v in weights.items()}

    @classmethod
    def from_folder(cls, folder):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            config = json.load(f)
        return cls(config, load_file(os.path.join(folder, "model.safetensors")))

    def residuals(self, tokens):
        """[layers, T, W]: the residual after each layer."""
        c, w = self.c, self.w
        eps = c["norm"]["eps"]
        x = w["embed"][torch.tensor(tokens)] * (c.get("embedding") or {}).get("scale", 1.0)
        out, kept = [], {}
        for i, layer in enumerate(c["layers"]):
            p, m = f"l{i}.", layer["mixer"]
            h = rms_norm(x, w[p + "norm1"], eps)
            src = m.get("kv_from")
            if layer["type"] == "attention":
                d, kept[i] = attention_chunked(h, w, p + "mix.", m, None if src is None else kept[src])
            elif layer["type"] == "attention_2":
                d, kept[i] = attention_windowed(h, w, p + "mix.", m, eps, None if src is None else kept[src])
            elif layer["type"] == "latent_attention":
                d = latent_attention(h, w, p + "mix.", m, eps)
            else:
                raise ValueError(layer["type"])
            x = x + d
            f = layer.get("mlp")
            if f is not None:
                h = rms_norm(x, w[p + "norm2"], eps)
                x = x + (bounded_mlp(h, w, p + "mlp.", f["limit"]) if f["kind"] == "dense" else experts(h, w, p + "mlp.", f))
            out.append(x)
        return torch.stack(out)

    def logits(self, tokens):
        x = self.residuals(tokens)[-1]
        return rms_norm(x, self.w["final.norm"], self.c["norm"]["eps"]) @ self.w["head"].T
