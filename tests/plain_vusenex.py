"""A plain, slow implementation of the Vusenex decoder in float64 on the CPU, one function per
mechanism, written from the design's equations.  It shares no code with the library: it reads
``config.json`` and the safetensors file by itself and works on whole sequences with dense
masks, keys and values formed per head, and every expert run densely over all tokens.
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


def scalar_norm(x, g, eps):
    """x over its root mean square, times ONE number for all coordinates."""
    return unit_rms(x, eps) * g.reshape(())


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


# --------------------------------------------------------------------------- embedding
def pair_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for each token: a hash of (previous token, token); the first
    token of a sequence, which has no previous one, takes the table's last row."""
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets)
    return rows


def embed(w, cfg, tokens):
    b = cfg["embedding"]["bigram"]
    T = len(tokens)
    x = w["embed"][tokens]
    x = x + w["bigram"][pair_rows(tokens, b["buckets"], b["mul_prev"], b["mul_cur"])]
    return x + w["pos"][:T]


# --------------------------------------------------------------------------- mixers
def causal_mask(T):
    i = torch.arange(T)
    return i[None, :] <= i[:, None]                # [query, key]


def query_temperature(T, coef, every):
    """1 + coef ln(floor((p + 1) / every) + 1) per position p."""
    p = torch.arange(T)
    return 1.0 + coef * torch.log((torch.div(p + 1, every, rounding_mode="floor") + 1).to(F))


def sink_softmax(s, mask):
    """exp(s_j) / (1 + sum_j exp(s_j)) over the seen keys: one more key of score zero that
    carries no value."""
    s = s.masked_fill(~mask, -math.inf)
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def attention(h, w, p, m, eps):
    """Grouped-query attention whose values are the keys (as projected, before their norm);
    queries and keys normed over the whole projection; a temperature on the query by its
    position; a bias r1 ln(1 + r2 (i - j)) taken off the scores; a sink in the softmax."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = k.view(T, G, d)
    q = unit_rms(q, eps) * w[p + "q.norm"]
    k = unit_rms(k, eps) * w[p + "k.norm"]
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(T, qt["coef"], qt["every"])[:, None]
    q, k = q.view(T, H, d), k.view(T, G, d)
    i = torch.arange(T)
    dist = (i[:, None] - i[None, :]).clamp(min=0).to(F)
    mask = causal_mask(T)
    out = torch.zeros(T, H, d, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"]
        s = s - w[p + "r1"][hh] * torch.log1p(w[p + "r2"][hh] * dist)
        out[:, hh] = sink_softmax(s, mask) @ v[:, g]
    return out.reshape(T, H * d) @ w[p + "o"].T


def latent_attention(h, w, p, m, eps):
    """Every head's keys and values are expanded from one normed latent per token; no
    positions enter."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, d)
    c = unit_rms(h @ w[p + "dkv"].T, eps) * w[p + "dkv.norm"]
    k = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    mask = causal_mask(T)
    out = torch.zeros(T, H, dv, dtype=F)
    for hh in range(H):
        s = (q[:, hh] @ k[:, hh].T) * m["scale"]
        s = s.masked_fill(~mask, -math.inf)
        out[:, hh] = torch.softmax(s, -1) @ v[:, hh]
    return out.reshape(T, H * dv) @ w[p + "o"].T


MIXERS = {"attention": attention, "latent_attention": latent_attention}


# --------------------------------------------------------------------------- feed-forward
def route(z, top, groups, keep):
    """Softmax over all experts; only experts of the ``keep`` groups (of ``groups`` equal
    groups of neighbours) whose best score is largest can be chosen; the ``top`` largest
    among them, weighted by their scores over the scores' sum.  Returns [T, E] weights."""
    T, E = z.shape
    s = torch.softmax(z, -1)
    per = E // groups
    best = s.view(T, groups, per).max(-1).values
    allowed = torch.zeros(T, groups, dtype=torch.bool)
    allowed.scatter_(1, best.topk(keep, dim=-1).indices, True)
    allowed = allowed[:, :, None].expand(T, groups, per).reshape(T, E)
    chosen = s.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    picked = torch.zeros(T, E, dtype=F).scatter_(1, chosen, s.gather(1, chosen))
    return picked / (picked.sum(-1, keepdim=True) + 1e-20)


def expert(h, up, down):
    return gelu_erf(h @ up.T) @ down.T


def mixture(h, w, p, mlp):
    r = mlp["router"]
    weights = route(h @ w[p + "router"].T, r["top"], r["groups"]["count"], r["groups"]["keep"])
    y = torch.zeros_like(h)
    for e in range(r["experts"]):
        y = y + weights[:, e:e + 1] * expert(h, w[f"{p}e{e}.up"], w[f"{p}e{e}.down"])
    if mlp.get("shared"):
        y = y + expert(h, w[p + "shared.up"], w[p + "shared.down"])
    return y


# --------------------------------------------------------------------------- the stack
def gated(x, y, w, name):
    """A sublayer's result y times sigmoid(W x + b), element by element."""
    return y * torch.sigmoid(x @ w[name].T + w[name + ".b"])


def forward(w, cfg, tokens, layer_outputs=None):
    """Logits [T, vocab] of one whole sequence; ``layer_outputs`` collects the stream after
    every layer."""
    eps = cfg["norm"]["eps"]
    x = embed(w, cfg, list(tokens))
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[layer["type"]](x, w, p + "mix.", layer["mixer"], eps)
        x = x + scalar_norm(gated(x, y, w, p + "rg1"), w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            y = mixture(x, w, p + "mlp.", layer["mlp"])
            x = x + scalar_norm(gated(x, y, w, p + "rg2"), w[p + "norm2"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return scalar_norm(x, w["final.norm"], eps) @ w["head"].T


def greedy_generate(w, cfg, prompt, max_new_tokens):
    tokens = list(prompt)
    for _ in range(max_new_tokens):
        tokens.append(int(forward(w, cfg, tokens)[-1].argmax()))
    return tokens[len(prompt):]
