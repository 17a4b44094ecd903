"""A plain, slow statement of the Repolix decoder in float64 on the CPU: one function for each mechanism, whole
sequences only (no cache, no batches, no portions; every recurrence is a loop over the tokens).  The oracle of the GPU
tests; it shares no code with the package.

Notation: T tokens, W the width; positions count from 0; a weight [out, in] meets a row x as x @ w.T.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rms_norm(x, gain, eps):
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if gain is None else y * gain


def short_conv(u, w, bias=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the first token."""
    T, C = u.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j]
    return y if bias is None else y + bias


# ---------------------------------------------------------------- mixer: state space with a scalar decay a head
def state_space_cell(x, B, C, dt_raw, dt_bias, a_log, d_skip, S=None):
    """x [T, H, P], B and C [T, G, N], dt_raw [T, H] -> y [T, H, P]; S [H, N, P] is updated in place if given."""
    T, H, P = x.shape
    G, N = B.shape[1], B.shape[2]
    dt = softplus(dt_raw + dt_bias)
    decay = torch.exp(-torch.exp(a_log) * dt)
    S = torch.zeros(H, N, P, dtype=F64) if S is None else S
    y = torch.zeros(T, H, P, dtype=F64)
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            S[hd] = decay[t, hd] * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + d_skip[hd] * x[t, hd]
    return y


def state_space(h, w, p, c, eps):
    T = h.shape[0]
    H, P, N, G = c["heads"], c["vdim"], c["state"], c["groups"]
    inner = H * P
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    y = state_space_cell(x, B, C, dt, w[p + "dt_bias"], w[p + "A_log"], w[p + "D"])
    y = y.reshape(T, inner) * silu(z)
    parts = c["norm_groups"]
    y = rms_norm(y.view(T, parts, inner // parts), None, eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


# ---------------------------------------------------------------- mixer: delta rule with a decay for every key channel
def delta_cell(q, k, v, beta_raw, a_raw, a_bias, a_log, S=None):
    """q, k [T, K, D] (not yet unit vectors), v [T, H, E], beta_raw [T, H], a_raw [T, H, D], a_bias [H, D], a_log [H]
    -> o [T, H, E]; S [H, D, E] is updated in place if given."""
    T, K, D = q.shape
    H, E = v.shape[1], v.shape[2]

    def unit(x):
        return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)

    q, k = unit(q) * D ** -0.5, unit(k)
    beta = torch.sigmoid(beta_raw)
    decay = torch.exp(-torch.exp(a_log)[None, :, None] * softplus(a_raw + a_bias))
    S = torch.zeros(H, D, E, dtype=F64) if S is None else S
    o = torch.zeros(T, H, E, dtype=F64)
    for t in range(T):
        for hd in range(H):
            kv = hd // (H // K)
            S[hd] = decay[t, hd][:, None] * S[hd]
            u = beta[t, hd] * (v[t, hd] - S[hd].T @ k[t, kv])
            S[hd] = S[hd] + torch.outer(k[t, kv], u)
            o[t, hd] = S[hd].T @ q[t, kv]
    return o


def channel_delta(h, w, p, c, eps):
    T = h.shape[0]
    H, K, D, E = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, K, D)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, K, D)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, E)
    a = ((h @ w[p + "a1"].T) @ w[p + "a2"].T).view(T, H, D)
    o = delta_cell(q, k, v, h @ w[p + "b"].T, a, w[p + "dt_bias"].view(H, D), w[p + "A_log"])
    o = rms_norm(o, w[p + "norm"], eps)
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(T, H, E)
    return (o * gate).reshape(T, H * E) @ w[p + "o"].T


# ---------------------------------------------------------------- mixer: two softmax maps over the same values
def scaled_frequencies(rot):
    """The turning rates f_i, i < dims / 2, with the long waves slowed down by `factor`, and the factor on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if sc is None:
        return f, 1.0

    def place(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(place(sc["fast"])), 0)
    hi = min(math.ceil(place(sc["slow"])), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def turn_halves(x, positions, rot):
    """x [T, ..., n]: value i < dims / 2 is paired with value i + dims / 2; the rest passes."""
    dims = rot["dims"]
    if dims == 0:
        return x.clone()
    f, m = scaled_frequencies(rot)
    angle = positions.to(F64)[:, None] * f
    while angle.dim() < x.dim():
        angle = angle.unsqueeze(1)
    c, s = torch.cos(angle) * m, torch.sin(angle) * m
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    y = x.clone()
    y[..., :dims // 2] = u * c - v * s
    y[..., dims // 2:dims] = v * c + u * s
    return y


def window_softmax(q, k, scale, window):
    """q, k [T, n] -> weights [T, T] over the keys j with 0 <= i - j < window."""
    T = q.shape[0]
    d = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    seen = (d >= 0) if window is None else (d >= 0) & (d < window)
    return torch.softmax((scale * q @ k.T).masked_fill(~seen, -math.inf), -1)


def two_maps(q, k, v, scale, window, lam, eps, post):
    """q [T, H, 2, D], k [T, G, 2, D], v [T, G, E] -> [T, H, E]: rms_norm(a1 - lam a2) * post for each head."""
    T, H, G, E = q.shape[0], q.shape[1], k.shape[1], v.shape[2]
    o = torch.zeros(T, H, E, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        a1 = window_softmax(q[:, hd, 0], k[:, g, 0], scale, window) @ v[:, g]
        a2 = window_softmax(q[:, hd, 1], k[:, g, 1], scale, window) @ v[:, g]
        o[:, hd] = rms_norm(a1 - lam * a2, None, eps) * post
    return o


def differential_attention(h, w, p, c, eps, positions=None):
    T = h.shape[0]
    H, G, D, E = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    pos = torch.arange(T) if positions is None else positions
    q = short_conv(h @ w[p + "q"].T, w[p + "q.conv"]).view(T, H, 2, D)
    k = short_conv(h @ w[p + "k"].T, w[p + "k.conv"]).view(T, G, 2, D)
    v = short_conv(h @ w[p + "v"].T, w[p + "v.conv"]).view(T, G, E)
    q, k = turn_halves(q, pos, c["rot"]), turn_halves(k, pos, c["rot"])
    lam = (torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + c["diff"])
    window = (c.get("mask") or {}).get("size")
    o = two_maps(q, k, v, c["scale"], window, lam, eps, 1.0 - c["diff"])
    return o.reshape(T, H * E) @ w[p + "o"].T


# ---------------------------------------------------------------- feed-forward: routed experts, some of them the identity
def clamped_expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h, w, p, r):
    """(chosen [T, top], weights [T, top]): softmax over all router outputs; the choice adds the correction and keeps
    the best groups only; the weights are the chosen scores themselves."""
    total = r["experts"] + r.get("identity", 0)
    s = torch.softmax(h @ w[p + "router"].T, -1)
    choice = s + w[p + "correction"]
    groups = r.get("groups")
    if groups is not None:
        per = total // groups["count"]
        best = choice.view(-1, groups["count"], per).max(-1).values
        keep = torch.topk(best, groups["keep"], -1).indices
        allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, keep, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(per, 1), -math.inf)
    chosen = torch.topk(choice, r["top"], -1).indices
    return chosen, torch.gather(s, 1, chosen)


def routed_experts(h, w, p, c):
    r = c["router"]
    chosen, weights = route(h, w, p, r)
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, s in zip(chosen[t].tolist(), weights[t]):
            if e >= r["experts"]:
                y[t] += s * h[t]
            else:
                q = f"{p}e{e}."
                y[t] += s * clamped_expert(h[t:t + 1], w[q + "gate"], w[q + "up"], w[q + "down"], c["expert"]["limit"])[0]
    if c.get("shared") is not None:
        q = p + "shared."
        y = y + clamped_expert(h, w[q + "gate"], w[q + "up"], w[q + "down"], c["shared"]["limit"])
    return y


MIXERS = {"mamba2": lambda h, w, p, c, eps: state_space(h, w, p, c, eps),
          "channel_delta": lambda h, w, p, c, eps: channel_delta(h, w, p, c, eps),
          "attention": lambda h, w, p, c, eps: differential_attention(h, w, p, c, eps)}


class PlainRepolix:
    def __init__(self, config: dict, weights: dict):
        self.c = config
        self.w = {n: (t.to(F64) if t.is_floating_point() else t) for n, t in weights.items()}

    @classmethod
    def from_folder(cls, folder):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            c = json.load(f)
        return cls(c, load_file(os.path.join(folder, "model.safetensors")))

    def residuals(self, tokens):
        """The residual after every layer [layers, T, W] and the logits [T, vocab] of one whole sequence."""
        c, w = self.c, self.w
        eps = c["norm"]["eps"]
        x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * (c.get("embedding") or {}).get("scale", 1.0)
        after = []
        for i, layer in enumerate(c["layers"]):
            p = f"l{i}."
            x = x + w[p + "ls1"] * MIXERS[layer["type"]](rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps)
            if layer.get("mlp") is not None:
                x = x + w[p + "ls2"] * routed_experts(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"])
            after.append(x)
        return torch.stack(after), rms_norm(x, w["final.norm"], eps) @ w["head"].T

    def logits(self, tokens):
        return self.residuals(tokens)[1]
