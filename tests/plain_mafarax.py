"""Plain, slow implementation of the Mafarax decoder: whole sequences, no cache, no batch.

One function per mechanism, written from the design's equations in this file's own notation.  It
shares no code with the engine: it reads config.json and model.safetensors itself, keeps every
projection as a separate matrix, loops over the experts, and runs the state-space recurrence token by
token.  Everything is float64.

The design, per layer (r is the residual stream, one row per token):
    r <- r + mix(dyt1(r));   r <- r + moe(dyt2(r))   (the second only where the layer has a feed-forward)
    dyt(x) = tanh(alpha x) * w + b                    alpha one number, w and b vectors
mix(h) = ( unit(att(h)) * w_left + unit(ssm(h)) * w_right ) / 2,   unit(x) = x / sqrt(mean(x^2) + eps)
att: q = Wq h + bq, k = Wk h + bk, v = Wv h + bv in H query and G key/value heads; the first R channels of
    every q and k head turn in pairs (i, i + R/2) by the angle p * base^(-2i/R) / factor; token i reads the
    tokens j <= i with floor(j / c) = floor(i / c) (c: the chunk); softmax(scale q.k) v; Wo on the heads, + bo.
ssm: [z | x | B | C | dt] = W_in h;  (x, B, C) <- silu(conv over the last K tokens per channel + bias);
    dt <- softplus(dt + dt_bias);  S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T;  y_t = S_t^T C_t + D x_t
    per head (heads share B and C in groups);  y <- y silu(z);  y <- unit(y) in norm_groups parts, times w;  Wo y.
moe: s = sigmoid(Wr h); groups of neighbouring experts scored by their two best; experts of the best groups only;
    the top scores chosen; sum of scale * s_e * Wd_e relu(Wu_e h)^2 over the chosen, plus the shared expert.
logits = head dyt_final(r) * logit_scale.
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


def dynamic_tanh(x, w, name):
    return torch.tanh(w[name + ".alpha"] * x) * w[name] + w[name + ".b"]


def unit(x, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def turn_heads(x, rot):
    """x [T, heads, dim]: the first rot["dims"] channels of every head turned by the token's position."""
    if not rot:
        return x
    R = rot["dims"]
    half = R // 2
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    out = x.clone()
    for t in range(x.shape[0]):
        for i in range(half):
            angle = t * rot["base"] ** (-2.0 * i / R) / factor
            c, s = math.cos(angle), math.sin(angle)
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


def chunked_attention(h, m, w, p):
    T = h.shape[0]
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = turn_heads((h @ w[p + ".q"].T + w[p + ".q.b"]).reshape(T, H, D), m.get("rot"))
    k = turn_heads((h @ w[p + ".k"].T + w[p + ".k.b"]).reshape(T, G, D), m.get("rot"))
    v = (h @ w[p + ".v"].T + w[p + ".v.b"]).reshape(T, G, DV)
    c = m["mask"]["size"]
    heads_out = torch.zeros(T, H, DV, dtype=h.dtype)
    for i in range(T):
        lo = (i // c) * c
        for a in range(H):
            g = a // (H // G)
            scores = (k[lo:i + 1, g] @ q[i, a]) * m["scale"]
            heads_out[i, a] = torch.softmax(scores, dim=0) @ v[lo:i + 1, g]
    return heads_out.reshape(T, H * DV) @ w[p + ".o"].T + w[p + ".o.b"]


def silu(x):
    return x * torch.sigmoid(x)


def causal_conv(u, kernel, bias):
    """u [T, C]; kernel [C, K] with the current token's tap last; zeros before the sequence."""
    T, C = u.shape
    K = kernel.shape[1]
    out = torch.zeros_like(u)
    for t in range(T):
        acc = bias.clone()
        for j in range(K):
            src = t - (K - 1) + j
            if src >= 0:
                acc = acc + kernel[:, j] * u[src]
        out[t] = acc
    return out


def state_space(h, m, w, p, eps):
    T = h.shape[0]
    Hn, P, N, G = m["heads"], m["vdim"], m["state"], m.get("groups", 1)
    inner = Hn * P
    zxbcdt = h @ w[p + ".in"].T
    z = zxbcdt[:, :inner]
    xbc = zxbcdt[:, inner:2 * inner + 2 * G * N]
    dt = zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + ".conv"], w[p + ".conv.b"]))
    x = xbc[:, :inner].reshape(T, Hn, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = torch.log1p(torch.exp(dt + w[p + ".dt_bias"]))            # softplus, no clamp (float64 holds it)
    y = torch.zeros(T, Hn, P, dtype=h.dtype)
    for a in range(Hn):
        g = a // (Hn // G)
        S = torch.zeros(N, P, dtype=h.dtype)
        rate = torch.exp(w[p + ".A_log"][a])
        for t in range(T):
            S = torch.exp(-rate * dt[t, a]) * S + dt[t, a] * torch.outer(B[t, g], x[t, a])
            y[t, a] = S.T @ C[t, g] + w[p + ".D"][a] * x[t, a]
    y = y.reshape(T, inner) * silu(z)
    parts = m.get("norm_groups", 1)
    y = unit(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * w[p + ".norm"]
    return y @ w[p + ".o"].T


def choose_experts(scores, router):
    """scores [E] of one token -> the chosen experts, by the grouped rule."""
    E = router["experts"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    count, keep = groups["count"], groups["keep"]
    per = E // count
    group_score = []
    for g in range(count):
        best = sorted((float(s) for s in scores[g * per:(g + 1) * per]), reverse=True)
        group_score.append(sum(best[:2]))
    kept = sorted(range(count), key=lambda g: -group_score[g])[:keep]
    allowed = [e for e in range(E) if e // per in kept]
    return sorted(allowed, key=lambda e: -float(scores[e]))[:router["top"]]


def expert(h, w, p):
    return torch.relu(h @ w[p + ".up"].T).pow(2) @ w[p + ".down"].T


def mixture(h, mlp, w, p):
    router = mlp["router"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        s = torch.sigmoid(w[p + ".router"] @ h[t])
        for e in choose_experts(s, router):
            out[t] += router.get("scale", 1.0) * s[e] * expert(h[t], w, f"{p}.e{e}")
    if mlp.get("shared"):
        out = out + expert(h, w, p + ".shared")
    return out


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of a whole sequence; with return_layers also the stream after every layer."""
    eps = cfg["norm"]["eps"]
    r = w["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        h = dynamic_tanh(r, w, p + ".norm1")
        a = chunked_attention(h, layer["mixer"]["left"], w, p + ".mix.left")
        b = state_space(h, layer["mixer"]["right"], w, p + ".mix.right", eps)
        r = r + 0.5 * (unit(a, eps) * w[p + ".mix.left.out"] + unit(b, eps) * w[p + ".mix.right.out"])
        if layer.get("mlp"):
            r = r + mixture(dynamic_tanh(r, w, p + ".norm2"), layer["mlp"], w, p + ".mlp")
        streams.append(r.clone())
    logits = dynamic_tanh(r, w, "final.norm") @ w["head"].T * cfg.get("logit_scale", 1.0)
    return (logits, streams) if return_layers else logits


def greedy_generate(cfg, w, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(torch.argmax(forward(cfg, w, tokens)[-1])))
    return tokens[len(prompt):]
