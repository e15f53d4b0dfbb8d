"""Plain, slow implementation of the Kirisun decoder: whole sequences, no cache, no batch.

One function per mechanism, written from the design's equations in this file's own notation.  It
shares no code with the engine: it reads config.json and model.safetensors itself, keeps every
projection as a separate matrix, loops over heads, tokens and experts, and runs the delta rule token
by token.  Everything is float64.

The design (r is the residual stream, one row per token; c the residual multiplier):
    r = embed[token] * embedding scale
    per layer:  r <- r + c * nb1(mixer(n1(r)));   r <- r + c * nb2(moe(n2(r)))   (the second where there is one)
    n(x) = x / sqrt(mean(x^2) + eps) * w      for all four norms of a layer and the model's last one
    logits = head n_final(r)
mixer "attention": q = Wq h in H heads, k = Wk h and v = Wv h in G heads; q and k heads normed (n with a weight
    shared by the heads); the first R channels of each q and k head turn in pairs (i, i + R/2) by the angle
    p * base^(-2i/R) / factor; s_ij = cap * tanh(scale q_i.k_j / cap); token i reads j <= i with i - j < window
    or j < keep; weights e^s_ij / (1 + sum_j e^s_ij); the heads' outputs times sigmoid(Wg h); Wo.
mixer "channel_delta": q = Wq h, k = Wk h in G heads of D, v = Wv h in H heads of DV; each through a causal
    convolution per channel and silu; q, k <- x / sqrt(sum x^2 + 1e-6), q <- q D^-1/2; b = sigmoid(Wb h);
    a = exp(-exp(A_log_head) * softplus(Wa2 Wa1 h + dt_bias)) per head and key channel;
    S <- diag(a) S;  u = b (v - S^T k);  S <- S + k u^T;  o = S^T q;  o <- n(o) (weight shared by the heads)
    times sigmoid(Wg2 Wg1 h);  Wo.
moe: z = Wr h + br; the `top` largest z are chosen, weighted by the softmax over the chosen z alone;
    sum of weight * Wd_e (silu(Wgate_e h) * (Wup_e h)).
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
            t = f.get_tensor(name)
            weights[name] = t.to(dtype) if t.is_floating_point() else t
    return cfg, weights


def unit_mean(x, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def turn_heads(x, rot, first_position=0):
    """x [T, heads, dim]: the first rot["dims"] channels of every head turned by the token's position."""
    if not rot:
        return x
    R = rot["dims"]
    half = R // 2
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    out = x.clone()
    for t in range(x.shape[0]):
        for i in range(half):
            angle = (first_position + t) * (rot["base"] ** (-2.0 * i / R) / factor)
            c, s = math.cos(angle), math.sin(angle)
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


def sees(i, j, mask):
    """Whether the token at position i reads the token at position j."""
    if j > i:
        return False
    if not mask:
        return True
    return i - j < mask["size"] or j < mask.get("keep_first", 0)


def sink_softmax(scores):
    """e^s_j / (1 + sum e^s): one more term of score 0 in the denominator."""
    m = max(float(scores.max()), 0.0)
    e = torch.exp(scores - m)
    return e / (math.exp(-m) + e.sum())


def attend(q, k, v, m, rows=None):
    """q [T, H, D], k [T, G, D], v [T, G, DV] of a whole sequence, ready (normed, turned): every head's output
    [T, H, DV] (rows: only these positions are computed, the others stay zero)."""
    T, H = q.shape[0], q.shape[1]
    G, DV = k.shape[1], v.shape[2]
    cap = m.get("softcap")
    heads_out = torch.zeros(T, H, DV, dtype=q.dtype)
    for i in (range(T) if rows is None else rows):
        js = [j for j in range(i + 1) if sees(i, j, m.get("mask"))]
        for a in range(H):
            g = a // (H // G)
            s = (k[js, g] @ q[i, a]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            heads_out[i, a] = sink_softmax(s) @ v[js, g]
    return heads_out


def gated_attention(h, m, w, p, eps):
    T = h.shape[0]
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_mean((h @ w[p + ".q"].T).reshape(T, H, D), eps) * w[p + ".q.norm"]
    k = unit_mean((h @ w[p + ".k"].T).reshape(T, G, D), eps) * w[p + ".k.norm"]
    q, k = turn_heads(q, m.get("rot")), turn_heads(k, m.get("rot"))
    v = (h @ w[p + ".v"].T).reshape(T, G, DV)
    gate = torch.sigmoid(h @ w[p + ".g"].T)
    return (attend(q, k, v, m).reshape(T, H * DV) * gate) @ w[p + ".o"].T


def short_conv(u, kernel):
    """u [T, C]; kernel [C, K] with the current token's tap last; zeros before the sequence; no bias."""
    T, C = u.shape
    K = kernel.shape[1]
    out = torch.zeros_like(u)
    for t in range(T):
        for j in range(K):
            src = t - (K - 1) + j
            if src >= 0:
                out[t] += kernel[:, j] * u[src]
    return out


def unit_sum(x):
    return x / torch.sqrt(x.pow(2).sum(dim=-1, keepdim=True) + 1e-6)


def delta_of_projections(q_in, k_in, v_in, b_in, a_in, g_in, m, w, p, eps):
    """The mixer between its input projections and its output projection: q_in, k_in [T, G D], v_in [T, H DV],
    b_in [T, H], a_in [T, H D] (before dt_bias), g_in [T, H DV] (before the sigmoid)."""
    T = q_in.shape[0]
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(q_in, w[p + ".q.conv"])).reshape(T, G, D)
    k = silu(short_conv(k_in, w[p + ".k.conv"])).reshape(T, G, D)
    v = silu(short_conv(v_in, w[p + ".v.conv"])).reshape(T, H, DV)
    q = unit_sum(q) * D ** -0.5
    k = unit_sum(k)
    beta = torch.sigmoid(b_in)                                                          # [T, H]
    step = torch.log1p(torch.exp(a_in + w[p + ".dt_bias"])).reshape(T, H, D)
    decay = torch.exp(-torch.exp(w[p + ".A_log"])[None, :, None] * step)                # [T, H, D]
    o = torch.zeros(T, H, DV, dtype=q_in.dtype)
    for a in range(H):
        g = a // (H // G)
        S = torch.zeros(D, DV, dtype=q_in.dtype)
        for t in range(T):
            S = decay[t, a][:, None] * S
            u = beta[t, a] * (v[t, a] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, a] = S.T @ q[t, g]
    o = unit_mean(o, eps) * w[p + ".norm"]
    return o.reshape(T, H * DV) * torch.sigmoid(g_in)


def channel_delta(h, m, w, p, eps):
    y = delta_of_projections(h @ w[p + ".q"].T, h @ w[p + ".k"].T, h @ w[p + ".v"].T, h @ w[p + ".b"].T,
                             (h @ w[p + ".a1"].T) @ w[p + ".a2"].T, (h @ w[p + ".g1"].T) @ w[p + ".g2"].T, m, w, p, eps)
    return y @ w[p + ".o"].T


def chosen_experts(z, top):
    """The `top` largest logits of one token (ties to the lower number) and their softmax among themselves."""
    order = sorted(range(z.shape[0]), key=lambda e: (-float(z[e]), e))[:top]
    weights = torch.softmax(z[order], dim=0)
    return order, weights


def expert(h, w, p):
    return (silu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def mixture(h, mlp, w, p):
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        z = w[p + ".router"] @ h[t] + w[p + ".router.b"]
        ids, weights = chosen_experts(z, mlp["router"]["top"])
        for e, a in zip(ids, weights):
            out[t] += a * expert(h[t], w, f"{p}.e{e}")
    return out


def norm(x, w, name, eps):
    return unit_mean(x, eps) * w[name]


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of a whole sequence; with return_layers also the stream after every layer."""
    eps = cfg["norm"]["eps"]
    c = cfg.get("residual_mult", 1.0)
    r = w["embed"][torch.tensor(list(tokens), dtype=torch.long)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        h = norm(r, w, p + ".norm1", eps)
        mix = gated_attention if layer["type"] == "attention" else channel_delta
        r = r + c * norm(mix(h, layer["mixer"], w, p + ".mix", eps), w, p + ".norm1b", eps)
        if layer.get("mlp"):
            h = norm(r, w, p + ".norm2", eps)
            r = r + c * norm(mixture(h, layer["mlp"], w, p + ".mlp"), w, p + ".norm2b", eps)
        streams.append(r.clone())
    logits = norm(r, w, "final.norm", eps) @ w["head"].T
    return (logits, streams) if return_layers else logits


def greedy_generate(cfg, w, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(torch.argmax(forward(cfg, w, tokens)[-1])))
    return tokens[len(prompt):]
