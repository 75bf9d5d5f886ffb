"""Bekedra, plainly: whole sequences in float64, dense loops over queries and heads for both attentions and over
tokens and experts for the mixture.  One function per mechanism, written from the design's equations; it shares
nothing with the engine (which keeps pages, runs ragged batches, sorts tokens by expert and fuses steps).

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
    return rms(x, eps) * w


def embedding(W, cfg, tokens):
    return W["embed"][torch.tensor(tokens)] * float(cfg["embedding"]["scale"])


# when a list: for every query and head of every attention, (query, head, the key with the largest weight, that
# weight) is appended (tests that make attention sharp look where it points)
ATTENTION_PEAKS: Optional[list] = None


def query_temperature(n: int, coef: float, every: int):
    """1 + coef ln(floor((p + 1) / every) + 1) for p = 0 .. n - 1."""
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in range(n)], dtype=F)


def tempered_attention(W, p: str, m: dict, eps: float, h):
    """Mixer "attention": biased q and k, the values are the keys as projected, a norm over all heads at once, a
    query temperature by position, plain softmax over every earlier key."""
    n, H, G, d = h.shape[0], m["heads"], m["kv_heads"], m["dim"]
    q = h @ W[p + "q"].T + W[p + "q.b"]
    k = h @ W[p + "k"].T + W[p + "k.b"]
    v = k.view(n, G, d)  # before the norm
    q = rms(q, eps) * W[p + "q.norm"]
    k = rms(k, eps) * W[p + "k.norm"]
    t = m.get("q_temp")
    if t is not None:
        q = q * query_temperature(n, float(t["coef"]), int(t["every"]))[:, None]
    q, k = q.view(n, H, d), k.view(n, G, d)
    out = torch.zeros(n, H, d, dtype=F)
    for i in range(n):
        for hd in range(H):
            g = hd // (H // G)
            s = (k[: i + 1, g] @ q[i, hd]) * m["scale"]
            w = torch.softmax(s, dim=0)
            out[i, hd] = w @ v[: i + 1, g]
            if ATTENTION_PEAKS is not None:
                ATTENTION_PEAKS.append((i, hd, int(torch.argmax(w)), float(w.max())))
    return out.reshape(n, H * d) @ W[p + "o"].T


def rotary_frequencies(rot: dict):
    """f_i = base^(-2i / dims), then the three bands by wavelength."""
    dims, base = int(rot["dims"]), float(rot["base"])
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        sc = rot.get("scaling")
        if sc is not None:
            wave = 2.0 * math.pi / f
            original, low, high, factor = float(sc["original"]), float(sc["low"]), float(sc["high"]), float(sc["factor"])
            if wave < original / high:
                pass
            elif wave > original / low:
                f = f / factor
            else:
                s = (original / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F)


def rotate(x, rot: dict):
    """x [n, heads, dim]: the first dims elements of every head turn, pairs (i, i + dims / 2)."""
    n, dims = x.shape[0], int(rot["dims"])
    half = dims // 2
    angle = torch.arange(n, dtype=F)[:, None] * rotary_frequencies(rot)[None, :]  # [n, half]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def sink_attention(W, p: str, m: dict, eps: float, h):
    """Mixer "attention_2": a norm per head, partial rotation, capped scores, a sink in the denominator, a gate
    per output element."""
    n, H, G, d, vd = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(n, H, d)
    k = (h @ W[p + "k"].T).view(n, G, d)
    v = (h @ W[p + "v"].T).view(n, G, vd)
    q = rms(q, eps) * W[p + "q.norm"]
    k = rms(k, eps) * W[p + "k.norm"]
    if m.get("rot") is not None:
        q, k = rotate(q, m["rot"]), rotate(k, m["rot"])
    cap = m.get("softcap")
    out = torch.zeros(n, H, vd, dtype=F)
    for i in range(n):
        for hd in range(H):
            g = hd // (H // G)
            s = (k[: i + 1, g] @ q[i, hd]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            sink = float(W[p + "sink"][hd])
            top = max(float(s.max()), sink)
            e = torch.exp(s - top)
            den = e.sum() + math.exp(sink - top)
            out[i, hd] = (e / den) @ v[: i + 1, g]
            if ATTENTION_PEAKS is not None:
                ATTENTION_PEAKS.append((i, hd, int(torch.argmax(e)), float((e / den).max())))
    gate = torch.sigmoid(h @ W[p + "g"].T)
    return (out.reshape(n, H * vd) * gate) @ W[p + "o"].T


# when a list: every token's gap between the last chosen expert's logit and the best one left out is appended
ROUTER_GAPS: Optional[list] = None


def expert(W, p: str, x):
    a = torch.relu(x @ W[p + "up"].T)
    return (a * a) @ W[p + "down"].T


def moe_ff(W, p: str, f: dict, h):
    n, top = h.shape[0], int(f["router"]["top"])
    logits = h @ W[p + "router"].T + W[p + "router.b"]
    out = torch.zeros(n, W[p + "e0.down"].shape[0], dtype=F)
    for t in range(n):
        ranked = torch.sort(logits[t], descending=True, stable=True)
        chosen = ranked.indices[:top].tolist()
        if ROUTER_GAPS is not None and top < logits.shape[1]:
            ROUTER_GAPS.append(float(ranked.values[top - 1] - ranked.values[top]))
        weight = torch.softmax(logits[t][chosen], dim=0)
        for w, e in zip(weight, chosen):
            out[t] += w * expert(W, f"{p}e{e}.", h[t][None])[0]
    return out


def run_layer(W, cfg: dict, i: int, x):
    layer = cfg["layers"][i]
    p, m, eps = f"l{i}.", layer["mixer"], cfg["norm"]["eps"]
    h = stream_norm(x, W[p + "norm1"], eps)
    if layer["type"] == "attention":
        y = tempered_attention(W, p + "mix.", m, eps, h)
    elif layer["type"] == "attention_2":
        y = sink_attention(W, p + "mix.", m, eps, h)
    else:
        raise ValueError(layer["type"])
    f = layer.get("mlp")
    if f is not None:
        y = y + moe_ff(W, p + "mlp.", f, h)
    return x + y


def layer_runs(cfg: dict):
    """(layer, the pass it begins or None) in the order the layers run."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if loop is None:
        return [(i, None) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, None) for i in range(start)]
    for t in range(times):
        runs += [(i, t if i == start else None) for i in range(start, stop)]
    return runs + [(i, None) for i in range(stop, n)]


def forward(weights: Dict[str, torch.Tensor], cfg: dict, tokens: List[int], streams: Optional[list] = None):
    """float64 logits [len(tokens), vocab]; ``streams`` (a list) receives the residual stream after every layer run."""
    W = {k: v.to(F) if v.is_floating_point() else v for k, v in weights.items()}
    x = embedding(W, cfg, tokens)
    for i, begins in layer_runs(cfg):
        if begins is not None:
            x = x + W["loop.step"][begins]
        x = run_layer(W, cfg, i, x)
        if streams is not None:
            streams.append(x.clone())
    return stream_norm(x, W["final.norm"], cfg["norm"]["eps"]) @ W["embed"].T
