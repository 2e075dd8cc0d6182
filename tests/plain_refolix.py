"""A plain, slow implementation of the Refolix decoder in float64 on the CPU, one function per
mechanism, written from the design's equations.  It shares no code with the library: it reads
``config.json`` and the safetensors file by itself and works on whole sequences with dense
masks, a token-by-token loop for every recurrence, and every expert run densely over all
tokens.

The design in this file's notation (h: what a sublayer reads, t: a position from 0):

* stream: ``x = E[token] * c_embed``; per layer ``x <- LN1(alpha x + ls1 * mixer(x))``, then
  ``x <- LN2(alpha x + ls2 * ff(x))``; LN is the layer norm with a weight and no bias.
* mixer "parallel": two mixers read the same h, ``(rms(left) w_l + rms(right) w_r) / 2``;
  left = windowed softmax attention with grouped keys, per-head RMS norm on q and k, a
  partial rotation of interleaved pairs with rescaled frequencies, and capped scores;
  right = the gated delta rule behind short causal convolutions.
* mixer "retention": a matrix state per head with a fixed decay, rotation of half-split pairs.
* feed-forward: a mixture of gated experts chosen by sigmoid scores with a correction that
  only the choice sees, group-limited, plus a shared expert behind a gate of one number.
"""
import json
import math
import os

import torch

from plain_llama import read_safetensors

F = torch.float64


def load_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    for k, v in read_safetensors(os.path.join(folder, "model.safetensors")).items():
        w[k] = v.to(F) if v.is_floating_point() else v.to(torch.int64)
    return cfg, w


# --------------------------------------------------------------------------- small pieces
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * weight; no bias."""
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# --------------------------------------------------------------------------- rotation
def rotary_frequencies(rot):
    """(frequencies [dims / 2], factor on cos and sin).  Plain ladder ``base^(-2i/dims)``; with
    ``scaling`` the slow end of the ladder is divided by ``factor`` along a linear ramp between
    the two places where a full turn takes ``original / fast`` and ``original / slow`` positions,
    and cos and sin grow by ``0.1 ln(factor) + 1``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def place(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(place(float(sc["fast"]))), 0)
    hi = min(math.ceil(place(float(sc["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=F)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot, layout):
    """x [T, heads, d]: the first ``rot.dims`` elements of every head turned by
    ``position * frequency``; pairs (2i, 2i + 1) for "interleaved", (i, i + dims/2) for
    "half".  (u, v) -> (u cos - v sin, v cos + u sin)."""
    if not rot or not int(rot.get("dims", 0)):
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f, grow = rotary_frequencies(rot)
    a = positions.to(F)[:, None] * f[None, :]                      # [T, half]
    cos, sin = (torch.cos(a) * grow)[:, None, :], (torch.sin(a) * grow)[:, None, :]
    out = x.clone()
    if layout == "interleaved":
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:dims] = v * cos + u * sin
    return out


# --------------------------------------------------------------------------- mixers
def window_mask(T, size):
    """[query, key]: key j is seen from i if 0 <= i - j < size (size None: every earlier key)."""
    i = torch.arange(T)
    d = i[:, None] - i[None, :]
    return (d >= 0) if size is None else (d >= 0) & (d < size)


def windowed_attention(h, w, p, m, eps):
    """The left half of a "parallel" mixer."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, d)
    k = (h @ w[p + "k"].T).view(T, G, d)
    v = (h @ w[p + "v"].T).view(T, G, dv)
    q = unit_rms(q, eps) * w[p + "q.norm"]
    k = unit_rms(k, eps) * w[p + "k.norm"]
    pos = torch.arange(T)
    q, k = rotate(q, pos, m.get("rot"), "interleaved"), rotate(k, pos, m.get("rot"), "interleaved")
    size = (m.get("mask") or {}).get("size")
    mask = window_mask(T, size)
    cap = m.get("softcap")
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~mask, -math.inf)
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, g]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def short_convolution(x, taps):
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, j] x[t - (K - 1) + j, c], zeros before the
    start; the last column weighs the current token."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j]
    return y


def delta_rule(h, w, p, m, eps):
    """The right half of a "parallel" mixer: per head a state S [d, dv] with
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, d)
    k = silu(short_convolution(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, d)
    v = silu(short_convolution(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)                                     # [T, H]
    g = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        kv = head // (H // G)
        S = torch.zeros(d, dv, dtype=F)
        for t in range(T):
            S = g[t, head] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            o[t, head] = S.T @ q[t, kv]
    o = unit_rms(o, eps) * w[p + "norm"]
    o = o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps):
    left = windowed_attention(h, w, p + "left.", m["left"], eps)
    right = delta_rule(h, w, p + "right.", m["right"], eps)
    return 0.5 * (unit_rms(left, eps) * w[p + "left.out"] + unit_rms(right, eps) * w[p + "right.out"])


def retention(h, w, p, m, eps):
    """S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t; no softmax, no denominator."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rotate((h @ w[p + "q"].T).view(T, H, d), pos, m.get("rot"), "half")
    k = rotate((h @ w[p + "k"].T).view(T, H, d), pos, m.get("rot"), "half") * d ** -0.5
    v = (h @ w[p + "v"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        S = torch.zeros(d, dv, dtype=F)
        for t in range(T):
            S = float(m["decay"][head]) * S + torch.outer(k[t, head], v[t, head])
            o[t, head] = S.T @ q[t, head]
    o = unit_rms(o, eps).reshape(T, H * dv) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


# --------------------------------------------------------------------------- feed-forward
def route(z, correction, top, groups, keep):
    """(chosen [T, top], weights [T, top]) from router logits z [T, E]: s = sigmoid(z); the
    choice is made on s + correction (a group counts by the sum of its two largest, only the
    ``keep`` best groups stay, the rest count as minus infinity); the weights are the chosen
    experts' s over their sum."""
    T, E = z.shape
    s = torch.sigmoid(z)
    c = s + correction
    size = E // groups
    by_group = c.view(T, groups, size)
    group_score = by_group.topk(min(2, size), dim=-1).values.sum(-1)           # [T, groups]
    best = group_score.topk(keep, dim=-1).indices
    allowed = torch.zeros(T, groups, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    c = c.masked_fill(~allowed[:, :, None].expand(T, groups, size).reshape(T, E), -math.inf)
    chosen = c.topk(top, dim=-1).indices
    picked = s.gather(1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def gated_expert(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def mixture(h, w, p, mlp):
    r = mlp["router"]
    groups = r.get("groups") or {}
    chosen, weights = route(h @ w[p + "router"].T, w[p + "correction"], r["top"],
                            int(groups.get("count", 1)), int(groups.get("keep", groups.get("count", 1))))
    y = torch.zeros_like(h)
    for e in range(r["experts"]):
        weight = (weights * (chosen == e)).sum(-1, keepdim=True)               # 0 where not chosen
        y = y + weight * gated_expert(h, w[f"{p}e{e}.gate"], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"])
    if mlp.get("shared"):
        y = y + torch.sigmoid(h @ w[p + "shared.sg"].T) * gated_expert(
            h, w[p + "shared.gate"], w[p + "shared.up"], w[p + "shared.down"])
    return y


# --------------------------------------------------------------------------- the model
def forward(w, cfg, tokens, layer_outputs=None):
    """float64 logits [T, vocab] of a whole sequence; ``layer_outputs``, a list, receives the
    stream after every layer."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = w["embed"][list(tokens)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] == "parallel":
            y = parallel_mixer(x, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "retention":
            y = retention(x, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = layer_norm(alpha * x + w[p + "ls1"] * y, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            y = mixture(x, w, p + "mlp.", layer["mlp"])
            x = layer_norm(alpha * x + w[p + "ls2"] * y, w[p + "norm2"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    x = layer_norm(x, w["final.norm"], eps)
    logits = (x @ w["head"].T) * cfg.get("logit_scale", 1.0)
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy_generate(w, cfg, prompt, max_new_tokens):
    tokens = list(prompt)
    for _ in range(max_new_tokens):
        tokens.append(int(forward(w, cfg, tokens)[-1].argmax()))
    return tokens[len(prompt):]
