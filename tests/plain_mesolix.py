"""Mesolix, plainly: whole sequences in float64, dense masks, every head's keys and values made from the
latents in full, python loops over tokens for the convolution and the recurrence and over tokens and
experts for the mixture.  One function per mechanism, written from the design's equations; it shares
nothing with the engine (which keeps pages and state slots, never expands a latent per key, sorts
tokens by expert and runs ragged batches).

``weights`` maps tensor names to tensors; ``cfg`` is the config.json dictionary.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def stream_norm(x, w, eps):
    """The norm of the residual stream: the weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


def embedding(W, tokens):
    n = len(tokens)
    return W["embed"][torch.tensor(tokens)] + W["pos"][:n]


# when a list: for every query and head of every attention (both kinds), (query, head, the key with the largest
# weight, that weight) is appended (tests that make attention sharp look where it points)
ATTENTION_PEAKS: Optional[list] = None


def latent_attention(W, p: str, m: dict, eps: float, h):
    n, H, d, vd = h.shape[0], m["heads"], m["dim"], m["vdim"]
    c_q = rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (c_q @ W[p + "uq"].T).view(n, H, d)
    c = rms(h @ W[p + "dkv"].T, eps) * W[p + "dkv.norm"]
    k = (c @ W[p + "uk"].T).view(n, H, d)
    v = (c @ W[p + "uv"].T).view(n, H, vd)
    out = torch.zeros(n, H, vd, dtype=F)
    for i in range(n):
        for hd in range(H):
            s = (k[: i + 1, hd] @ q[i, hd]) * m["scale"]
            top = max(float(s.max()), float(W[p + "sink"][hd]))
            e = torch.exp(s - top)
            den = e.sum() + math.exp(float(W[p + "sink"][hd]) - top)
            out[i, hd] = (e / den) @ v[: i + 1, hd]
            if ATTENTION_PEAKS is not None:
                ATTENTION_PEAKS.append((i, hd, int(torch.argmax(e)), float((e / den).max())))
    gate = torch.sigmoid(h @ W[p + "g"].T)
    return (out.reshape(n, H * vd) * gate) @ W[p + "o"].T


def distance_bucket(n: int, rows: int, far: float) -> int:
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def window_attention(W, p: str, m: dict, h):
    n, H, G, d, vd = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(n, H, d)
    k = (h @ W[p + "k"].T).view(n, G, d)
    v = (h @ W[p + "v"].T).view(n, G, vd)
    rel = W[p + "rel"]
    size = m["mask"]["size"] if m.get("mask") else None
    out = torch.zeros(n, H, vd, dtype=F)
    for i in range(n):
        first = 0 if size is None else max(0, i - size + 1)
        for hd in range(H):
            g = hd // (H // G)
            s = (k[first: i + 1, g] @ q[i, hd]) * m["scale"]
            s = s + torch.stack([rel[distance_bucket(i - j, rel.shape[0], m["bias_max"]), hd] for j in range(first, i + 1)])
            w = torch.softmax(s, 0)
            out[i, hd] = w @ v[first: i + 1, g]
            if ATTENTION_PEAKS is not None:
                ATTENTION_PEAKS.append((i, hd, first + int(torch.argmax(w)), float(w.max())))
    gate = torch.sigmoid(h @ W[p + "g"].T)
    return (out.reshape(n, H * vd) * gate) @ W[p + "o"].T


def mamba2(W, p: str, m: dict, eps: float, h):
    n, H, P, N, G, taps = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * P
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner: 2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    conv = torch.zeros_like(xbc)
    for t in range(n):
        acc = W[p + "conv.b"].clone()
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                acc = acc + W[p + "conv"][:, j] * xbc[src]
        conv[t] = acc * torch.sigmoid(acc)
    x = conv[:, :inner].view(n, H, P)
    B = conv[:, inner: inner + G * N].view(n, G, N)
    C = conv[:, inner + G * N:].view(n, G, N)
    dt = torch.nn.functional.softplus(dt + W[p + "dt_bias"])
    y = torch.zeros(n, H, P, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=F)
        a = -torch.exp(W[p + "A_log"][hd])
        for t in range(n):
            S = torch.exp(a * dt[t, hd]) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + W[p + "D"][hd] * x[t, hd]
    y = y.reshape(n, inner) * (z * torch.sigmoid(z))
    parts = m["norm_groups"]
    y = rms(y.view(n, parts, inner // parts), eps).reshape(n, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def dense_ff(W, p: str, f: dict, h):
    lim = f["limit"]
    g = torch.clamp(h @ W[p + "gate"].T, max=lim)
    u = torch.clamp(h @ W[p + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def silu_expert(W, p: str, h):
    g = h @ W[p + "gate"].T
    return ((g * torch.sigmoid(g)) * (h @ W[p + "up"].T)) @ W[p + "down"].T


# when a list: every token's gap between the last chosen expert's logit and the best one left out is appended
# (tests pick weights for which no choice is a close call)
ROUTER_GAPS: Optional[list] = None


def moe_ff(W, p: str, f: dict, h):
    n = h.shape[0]
    logits = h @ W[p + "router"].T
    scores = torch.sigmoid(logits)
    out = torch.zeros(n, W[p + "e0.down"].shape[0], dtype=F)
    top = f["router"]["top"]
    for t in range(n):
        chosen = torch.topk(scores[t], top).indices.tolist()
        if ROUTER_GAPS is not None and top < logits.shape[1]:
            ranked = torch.sort(logits[t], descending=True).values
            ROUTER_GAPS.append(float(ranked[top - 1] - ranked[top]))
        for e in chosen:
            out[t] += silu_expert(W, f"{p}e{e}.", (scores[t, e] * h[t])[None])[0]
    if f.get("shared"):
        out = out + silu_expert(W, p + "shared.", h)
    return out


def forward(weights: Dict[str, torch.Tensor], cfg: dict, tokens: List[int], streams: Optional[list] = None):
    """float64 logits [len(tokens), vocab]; ``streams`` (a list) receives the residual stream after every layer run."""
    W = {k: v.to(F) if v.is_floating_point() else v for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = embedding(W, tokens)
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        p, m = f"l{src}.", layer["mixer"]
        h = stream_norm(x, W[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            x = x + latent_attention(W, p + "mix.", m, eps, h)
        elif layer["type"] == "attention":
            x = x + window_attention(W, p + "mix.", m, h)
        elif layer["type"] == "mamba2":
            x = x + mamba2(W, p + "mix.", m, eps, h)
        else:
            raise ValueError(layer["type"])
        f = layer.get("mlp")
        if f is not None:
            h = stream_norm(x, W[p + "norm2"], eps)
            x = x + (dense_ff(W, p + "mlp.", f, h) if f["kind"] == "dense" else moe_ff(W, p + "mlp.", f, h))
        if streams is not None:
            streams.append(x.clone())
    return stream_norm(x, W["final.norm"], eps) @ W["head"].T
