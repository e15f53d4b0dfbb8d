"""Plain, slow implementation of the Pemuvik decoder: whole sequences, no cache, no batch.

One function per mechanism, written from the design's equations in this file's own notation.  It
shares no code with the engine: it reads config.json and model.safetensors itself, keeps every
projection as a separate matrix and loops over heads, tokens, keys and experts.  Everything is float64.

The design (r is the residual stream, one row per token):
    r = embed[token]
    per layer:  r <- r + ls1 * mixer(n1(r)) + ls2 * ff(n2(r))      (both read the same r; ff may be absent)
    n(x) = x / sqrt(mean(x^2) + eps) * w
    logits = embed n_final(r)                                      (the head is the embedding table)
Rotation: channels (2i, 2i + 1) of the first R channels of a head turn by p * base^(-2i/R).
mixer "attention": q = Wq h + bq in H heads of D, k = Wk h + bk in G heads of D, v = Wv h + bv in G heads of DV;
    q, k rotated; v <- v / rms(v) per head; in the layers that mix values, but the first of them,
    v <- (1 - lam) v + lam v1, v1 being the first such layer's v of the same token;
    token i reads j with 0 <= i - j < window; weight of j = sigmoid(scale q_i.k_j + pb_head), no normalisation;
    Wo (heads side by side) + bo.
mixer "latent_attention": q = Wq h in H heads of [D plain | R rotated]; [c | kr] = Wdkv h, c <- n(c) with a weight of
    its own, kr (R channels, one for all heads) rotated; per head kp = Wuk c, v = Wuv c;
    s_ij = scale (qp_i.kp_j + qr_i.kr_j), j <= i; weights e^s_ij / (e^sink_head + sum_j e^s_ij); Wo.
ff "dense": Wd (gelu_tanh(Wg h) * (Wu h)).
ff "moe": z = Wr h; s = softmax(z) over E experts and I identities; choice score = s + correction; the experts
    lie in equal groups of neighbours, a group counts by its best choice score, only the best groups' members
    can be chosen; the `top` best are; weights s_e / (sum of the chosen s + 1e-20); an expert gives
    Wd_e (silu(Wg_e h) * (Wu_e h)), an identity h itself; plus sigmoid(wsg.h) * shared expert (same form).
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


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def turn_pairs(x, rot, first_position=0):
    """x [T, heads, dim]: neighbouring channels (2i, 2i + 1) below rot["dims"] turned by the token's position."""
    if not rot:
        return x
    R = rot["dims"]
    out = x.clone()
    for t in range(x.shape[0]):
        for i in range(R // 2):
            angle = (first_position + t) * rot["base"] ** (-2.0 * i / R)
            c, s = math.cos(angle), math.sin(angle)
            u, v = x[t, :, 2 * i], x[t, :, 2 * i + 1]
            out[t, :, 2 * i] = u * c - v * s
            out[t, :, 2 * i + 1] = v * c + u * s
    return out


def window_values(h, m, w, p, eps, shared):
    """The values a window-attention layer caches; `shared` carries the first mixing layer's from layer to layer."""
    T = h.shape[0]
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, m["kv_heads"], m["vdim"])
    v = unit_mean(v, eps)
    if m.get("v_mix"):
        if "first" not in shared:
            shared["first"] = v
        else:
            lam = w[p + "vmix"]
            v = (1.0 - lam) * v + lam * shared["first"]
    return v


def sigmoid_window_attend(q, k, v, m, bias, rows=None):
    """q [T, H, D], k [T, G, D], v [T, G, DV] -> [T, H * DV]: every visible key weighs sigmoid(score + bias).
    rows: the tokens whose output is wanted (default all; the others' stay zero)."""
    T, H = q.shape[0], q.shape[1]
    per = H // k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for head in range(H):
        g = head // per
        for i in (range(T) if rows is None else rows):
            for j in range(max(0, i - m["mask"]["size"] + 1) if m.get("mask") else 0, i + 1):
                weight = torch.sigmoid(torch.dot(q[i, head], k[j, g]) * m["scale"] + bias[head])
                out[i, head] += weight * v[j, g]
    return out.reshape(T, -1)


def window_attention(h, m, w, p, eps, shared):
    T = h.shape[0]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, m["heads"], m["dim"])
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, m["kv_heads"], m["dim"])
    q, k = turn_pairs(q, m.get("rot")), turn_pairs(k, m.get("rot"))
    v = window_values(h, m, w, p, eps, shared)
    o = sigmoid_window_attend(q, k, v, m, w[p + "pb"])
    return o @ w[p + "o"].T + w[p + "o.b"]


def sink_softmax_rows(scores, sink):
    """scores [n] of the visible keys -> weights whose denominator also holds e^sink."""
    top = max(float(scores.max()), float(sink))
    e = torch.exp(scores - top)
    return e / (e.sum() + math.exp(float(sink) - top))


def latent_attention(h, m, w, p, eps):
    T, H, D, R, DV, C = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w[p + "q"].T).view(T, H, D + R)
    q_plain, q_turn = q[:, :, :D], turn_pairs(q[:, :, D:], m["rot"])
    low = h @ w[p + "dkv"].T
    c = unit_mean(low[:, :C], eps) * w[p + "dkv.norm"]
    k_turn = turn_pairs(low[:, C:].reshape(T, 1, R), m["rot"])[:, 0]
    k_plain = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, DV)
    out = torch.zeros(T, H, DV, dtype=h.dtype)
    for head in range(H):
        for i in range(T):
            s = (k_plain[: i + 1, head] @ q_plain[i, head] + k_turn[: i + 1] @ q_turn[i, head]) * m["scale"]
            out[i, head] = sink_softmax_rows(s, w[p + "sink"][head]) @ v[: i + 1, head]
    return out.reshape(T, -1) @ w[p + "o"].T


def gated_unit(h, w, p, act):
    return (act(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def chosen_experts(s, correction, router):
    """s [n] the softmax scores of one token -> (indices chosen, their weights)."""
    n = s.shape[0]
    choice = s + correction
    groups = (router.get("groups") or {})
    count, keep = groups.get("count", 1), groups.get("keep", 1)
    if count > 1:
        size = n // count
        best = [float(choice[g * size: (g + 1) * size].max()) for g in range(count)]
        kept = sorted(range(count), key=lambda g: (-best[g], g))[:keep]
        allowed = [e for e in range(n) if e // size in kept]
    else:
        allowed = list(range(n))
    picked = sorted(allowed, key=lambda e: (-float(choice[e]), e))[: router["top"]]
    weights = s[picked] / (s[picked].sum() + 1e-20)
    return picked, weights


def mixture(h, mlp, w, p):
    router = mlp["router"]
    E, I = router["experts"], router.get("identity", 0)
    z = h @ w[p + "router"].T
    s = torch.softmax(z, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        picked, weights = chosen_experts(s[t], w[p + "correction"], router)
        for e, weight in zip(picked, weights):
            out[t] += weight * (h[t] if e >= E else gated_unit(h[t], w, f"{p}e{e}.", silu))
    if mlp.get("shared"):
        gate = torch.sigmoid(h @ w[p + "shared.sg"].reshape(-1))
        out = out + gate[:, None] * gated_unit(h, w, p + "shared.", silu)
    return out


def feed_forward(h, mlp, w, p):
    if mlp["kind"] == "dense":
        return gated_unit(h, w, p, gelu_tanh)
    return mixture(h, mlp, w, p)


def forward(cfg, w, tokens, return_layers=False):
    eps = cfg["norm"]["eps"]
    r = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    shared, layers = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = unit_mean(r, eps) * w[p + "norm1"]
        if layer["type"] == "attention":
            add = window_attention(h, layer["mixer"], w, p + "mix.", eps, shared)
        else:
            add = latent_attention(h, layer["mixer"], w, p + "mix.", eps)
        add = add * w[p + "ls1"]
        if layer.get("mlp"):
            add = add + feed_forward(unit_mean(r, eps) * w[p + "norm2"], layer["mlp"], w, p + "mlp.") * w[p + "ls2"]
        r = r + add
        layers.append(r)
    logits = (unit_mean(r, eps) * w["final.norm"]) @ w["embed"].T
    return (logits, torch.stack(layers)) if return_layers else logits


def greedy_generate(cfg, w, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(forward(cfg, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]
