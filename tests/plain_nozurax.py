"""Plain, slow implementation of the Nozurax decoder: whole sequences, no cache, no batch.

One function per mechanism, written from the design's equations in this file's own notation.
It shares no code with the engine: it reads config.json and model.safetensors itself, keeps
every projection as a separate matrix, and runs the retention recurrence token by token.

The design, per layer (x is the residual stream, one row per token):
    h = x / sqrt(mean(x^2) + eps) * (1 + w_norm)
    x <- x + mixer(h) + feed_forward(h)              both sublayers read the same h
A layer entry with "weights_of": j runs layer j's tensors again (own cache / state).

Mixer "retention" (per head, state S [dim, vdim] starts at zero):
    q, k <- rotate the first R channels, pairs (i, i + R/2), angle p * base^(-2i/R)
    k <- k * dim^(-1/2)
    S_t = decay * S_(t-1) + k_t v_t^T ;  o_t = S_t^T q_t
    o_t <- o_t / sqrt(mean(o_t^2) + eps)   (per head, no weight)
    out = Wo (concat(o) * silu(Wg h))
Mixer "attention" (H query heads, G key/value heads, sizes dim / vdim):
    q = Wq h + bq ; k = Wk h + bk ; v = Wv h + bv
    q <- q / sqrt(mean(q^2) + eps) * wq    over the whole projection, before the split into heads
    k <- the same with wk
    q <- q * (1 + coef * ln(floor((p + 1) / every) + 1))
    s_ij = scale * q_i . k_j  (j <= i) ;  a_ij = exp(s_ij) / (exp(sink_h) + sum_j exp(s_ij))
    out = Wo concat(sum_j a_ij v_j)
Feed-forward "dense": Wdown (relu(Wgate h) * (Wup h)).
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def read_folder(path: str, dtype=torch.float64):
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    weights = {}
    with safe_open(os.path.join(path, "model.safetensors"), "pt", "cpu") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(dtype)
    return cfg, weights


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def one_plus_norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def rotate_half(x, positions, rot_dims, base):
    """x [T, heads, dim]; the first rot_dims channels of every head are rotated."""
    half = rot_dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = base ** (-2.0 * i / rot_dims)
    a = positions.to(x.dtype)[:, None] * freq[None, :]            # [T, half]
    cos, sin = a.cos()[:, None, :], a.sin()[:, None, :]
    u, v, rest = x[..., :half], x[..., half:rot_dims], x[..., rot_dims:]
    return torch.cat((u * cos - v * sin, v * cos + u * sin, rest), dim=-1)


def retention(h, w, prefix, m, eps, positions):
    T = h.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + "q"].T).reshape(T, heads, dim)
    k = (h @ w[prefix + "k"].T).reshape(T, heads, dim)
    v = (h @ w[prefix + "v"].T).reshape(T, heads, vdim)
    g = h @ w[prefix + "g"].T
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, positions, rot["dims"], rot["base"])
        k = rotate_half(k, positions, rot["dims"], rot["base"])
    k = k * dim ** -0.5
    o = torch.zeros((T, heads, vdim), dtype=h.dtype)
    for hd in range(heads):
        S = torch.zeros((dim, vdim), dtype=h.dtype)
        for t in range(T):
            S = m["decay"][hd] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps).reshape(T, heads * vdim)
    return (o * (g * torch.sigmoid(g))) @ w[prefix + "o"].T


def sink_attention(h, w, prefix, m, eps, positions):
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[prefix + "q"].T + w[prefix + "q.b"]
    k = h @ w[prefix + "k"].T + w[prefix + "k.b"]
    v = h @ w[prefix + "v"].T + w[prefix + "v.b"]
    q = unit_rms(q, eps) * w[prefix + "q.norm"]
    k = unit_rms(k, eps) * w[prefix + "k.norm"]
    temp = m.get("q_temp")
    if temp:
        steps = torch.floor((positions.to(h.dtype) + 1) / temp["every"])
        q = q * (1.0 + temp["coef"] * torch.log(steps + 1.0))[:, None]
    q, k, v = q.reshape(T, H, dim), k.reshape(T, G, dim), v.reshape(T, G, vdim)
    out = torch.zeros((T, H, vdim), dtype=h.dtype)
    sink = w[prefix + "sink"]
    for hd in range(H):
        kv = hd // (H // G)
        for t in range(T):
            s = (k[: t + 1, kv] @ q[t, hd]) * m["scale"]
            top = max(float(s.max()), float(sink[hd]))
            e = torch.exp(s - top)
            out[t, hd] = (e[:, None] * v[: t + 1, kv]).sum(0) / (e.sum() + math.exp(float(sink[hd]) - top))
    return out.reshape(T, H * vdim) @ w[prefix + "o"].T


def dense_relu_glu(h, w, prefix):
    return (torch.relu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


MIXERS = {"retention": retention, "attention": sink_attention}


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of a whole sequence (and the residual stream after every layer run)."""
    dtype = w["embed"].dtype
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    positions = torch.arange(len(tokens))
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        name = f"l{src}."
        h = one_plus_norm(x, w[name + "norm1"], eps)
        y = MIXERS[layer["type"]](h, w, name + "mix.", layer["mixer"], eps, positions)
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            y = y + dense_relu_glu(h, w, name + "mlp.")
        x = x + y
        streams.append(x)
    logits = one_plus_norm(x, w["final.norm"], eps) @ w["head"].T
    assert logits.dtype == dtype
    return (logits, torch.stack(streams)) if return_layers else logits


def greedy_generate(cfg, w, prompt, max_tokens):
    toks = list(prompt)
    for _ in range(max_tokens):
        toks.append(int(torch.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]
