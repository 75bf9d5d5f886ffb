"""Small Bekedra configurations that differ from each other in every size and option, random weights for them,
and helpers to run them through the engine and the plain implementation."""
from __future__ import annotations

import copy
from typing import Dict, List, Sequence

import torch

import plain_bekedra as P
from mesolix_cases import CLOSE_CALL, assert_matches, make_requests, relative_error  # noqa: F401  (shared test equipment)
from yalis_amd.config.runtime import EngineConfig
from yalis_amd.engine.factory import build_model, tensor_specs_for
from yalis_amd.engine.step import ModelRunner


def tempered(heads, kv_heads, dim, scale, coef=None, every=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if coef is not None:
        m["q_temp"] = {"coef": coef, "every": every}
    return {"type": "attention", "mixer": m}


def sinked(heads, kv_heads, dim, vdim, scale, softcap=None, rot=None):
    """rot: (dims, base) or (dims, base, factor, low, high, original)."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap is not None:
        m["softcap"] = softcap
    if rot is not None:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
        if len(rot) > 2:
            m["rot"]["scaling"] = {"factor": rot[2], "low": rot[3], "high": rot[4], "original": rot[5]}
    return {"type": "attention_2", "mixer": m}


def moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def model(vocab, width, eps, scale, layers, loop=None):
    out = []
    for layer, mlp in layers:
        entry = copy.deepcopy(layer)
        entry["mlp"] = copy.deepcopy(mlp)
        out.append(entry)
    cfg = {"architecture": "Bekedra", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps}, "layers": out}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


CONFIGS = {
    # nothing a multiple of 8; values narrower than keys; a layer without feed-forward; every expert chosen; one key
    # head; a rotation over the whole head without scaling; no cap; the middle layers three times
    "odd": model(70, 40, 1e-5, 3.0, [
        (tempered(3, 3, 10, 0.3, 0.7, 5), moe(5, 2, 12)),
        (sinked(6, 2, 12, 10, 0.2, softcap=5.0, rot=(6, 100.0, 4.0, 1.0, 3.0, 16)), None),
        (tempered(4, 1, 6, 0.4), moe(3, 3, 9)),
        (sinked(2, 2, 8, 8, 0.35, rot=(8, 50.0)), moe(4, 1, 7)),
    ], loop=(1, 3, 3)),
    # no loop; an embedding that is not scaled; a temperature that steps every 16 tokens; values wider than keys
    "mix": model(128, 64, 1e-6, 1.0, [
        (sinked(4, 1, 16, 24, 0.25, softcap=30.0, rot=(8, 10000.0, 8.0, 1.0, 4.0, 32)), moe(4, 1, 32)),
        (tempered(2, 2, 32, 0.18, 0.4, 16), None),
        (sinked(2, 2, 24, 8, 0.2, rot=(24, 500.0, 2.0, 0.5, 2.0, 8)), moe(6, 3, 16)),
        (tempered(8, 4, 8, 0.35, 1.5, 1), moe(2, 2, 40)),
    ]),
    # sizes of whole wavefronts (the matrix-core attention and grouped products in bfloat16); the loop begins with the
    # first layer and takes in all of them
    "wide": model(200, 128, 1e-6, 8.0, [
        (sinked(4, 2, 64, 64, 0.125, softcap=25.0, rot=(32, 30000.0, 8.0, 1.0, 4.0, 64)), moe(8, 2, 64)),
        (tempered(4, 2, 64, 0.125, 0.4, 48), moe(8, 2, 64)),
        (sinked(2, 1, 128, 128, 0.09, softcap=50.0, rot=(128, 10000.0)), moe(4, 2, 96)),
    ], loop=(0, 3, 2)),
}
PAGE = {"odd": 16, "mix": 32, "wide": 64}
LENGTHS = {"odd": [1, 23, 50, 9, 37, 64], "mix": [70, 3, 41, 129, 18], "wide": [150, 40, 97, 2, 66]}


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Float32 weights by tensor name; values that bfloat16 holds exactly, so that both engines and the plain
    implementation read the same numbers."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in tensor_specs_for(cfg).items():
        last = name.rsplit(".", 1)[-1]
        offset = 0.0
        if last.startswith("norm"):
            std, offset = 0.3, 1.0  # plain weights
        elif last == "sink":
            std = 1.0
        elif last == "b":
            std = 0.5
        elif last == "router":
            std = 4.0 / (spec.shape[-1] ** 0.5)
        elif name == "loop.step":
            std = 0.5
        elif name == "embed":
            std = 1.0 / float(cfg["embedding"]["scale"])
        else:
            std = 1.5 / (spec.shape[-1] ** 0.5)
        out[name] = (torch.randn(spec.shape, generator=g) * std + offset).to(torch.bfloat16).float()
    return out


def make_runner(cfg, weights, dtype, device, ops, page_size, num_pages, max_seqs=4, max_len=512) -> ModelRunner:
    eng = EngineConfig(page_size=page_size, num_pages=num_pages, max_num_seqs=max_seqs, max_model_len=max_len,
                       max_num_batched_tokens=max_len, dtype=dtype, device=device)
    m = build_model(cfg, eng, ops=ops)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    m.load({k: v.to(wd).to(device) for k, v in weights.items()})
    return ModelRunner(m, eng)


def plain_logits(cfg, weights, reqs) -> Dict[str, torch.Tensor]:
    return {rid: P.forward(weights, cfg, toks) for rid, toks in reqs.items()}


def plain_logits_and_gaps(cfg, weights, reqs):
    """The plain logits, and for every position the smallest gap, over the layer runs with a router, between the
    last chosen expert's logit and the best one left out (infinite where every expert is chosen).  An engine that
    rounds what a router reads may send a token whose gap is tiny to another expert, which is then another model:
    the comparisons leave such positions out."""
    want, gaps = {}, {}
    for rid, toks in reqs.items():
        P.ROUTER_GAPS = seen = []
        try:
            want[rid] = P.forward(weights, cfg, toks)
        finally:
            P.ROUTER_GAPS = None
        n = len(toks)
        gaps[rid] = torch.tensor(seen, dtype=torch.float64).view(-1, n).min(0).values if seen else torch.full((n,), float("inf"), dtype=torch.float64)
    return want, gaps
