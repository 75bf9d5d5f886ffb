"""Small Mesolix configurations that differ from each other in every size and option, random weights for
them, and helpers to run them through the engine and the plain implementation."""
from __future__ import annotations

import copy
from typing import Dict, List, Sequence

import torch

import plain_mesolix as P
from yalis_amd.config.runtime import EngineConfig
from yalis_amd.engine.factory import build_model, tensor_specs_for
from yalis_amd.engine.step import ModelRunner


def latent(heads, dim, vdim, kv_rank, q_rank, scale):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale}}


def ssd(heads, vdim, state, groups, conv, norm_groups):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}}


def window(heads, kv_heads, dim, vdim, scale, size, bias_rows, bias_max):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": bias_max, "bias_rows": bias_rows}
    if size is not None:
        m["mask"] = {"size": size}
    return {"type": "attention", "mixer": m}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, shared=None):
    f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        f["shared"] = {"ff": shared}
    return f


def again(j: int):
    """A layer that runs layer j's weights once more."""
    return {"weights_of": j}


def model(vocab, width, eps, max_positions, layers):
    out = []
    for layer, mlp in layers:
        if "weights_of" in layer:
            entry = copy.deepcopy(out[layer["weights_of"]])
            entry["weights_of"] = layer["weights_of"]
        else:
            entry = copy.deepcopy(layer)
            entry["mlp"] = copy.deepcopy(mlp)
        out.append(entry)
    return {"architecture": "Mesolix", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": eps}, "layers": out}


CONFIGS = {
    # nothing a multiple of 8; a recurrent layer first, with a group per head and one part to norm; a layer
    # without feed-forward; every expert chosen; no window; layers run twice
    "odd": model(70, 40, 1e-5, 300, [
        (ssd(3, 6, 10, 3, 3, 1), moe(5, 2, 12)),
        (latent(3, 10, 14, 20, 12, 0.3), None),
        (window(6, 2, 12, 10, 0.2, 13, 10, 40.0), dense(24, 0.8)),
        (again(1), None),
        (window(3, 3, 5, 7, 0.45, None, 6, 100.0), moe(3, 3, 9, shared=7)),
        (again(0), None),
    ]),
    # one tap; one group for all heads; a window longer than a page; one key head; one expert of four
    "mix": model(128, 64, 1e-6, 512, [
        (latent(2, 32, 16, 24, 40, 0.2), moe(4, 1, 32, shared=16)),
        (ssd(4, 16, 16, 1, 1, 4), dense(48, 2.5)),
        (window(4, 1, 16, 16, 0.25, 40, 8, 64.0), None),
        (ssd(2, 32, 24, 2, 4, 2), moe(6, 3, 16)),
        (again(2), None),
        (latent(6, 8, 8, 48, 16, 0.35), dense(32, 0.5)),
        (again(0), None),
    ]),
    # sizes of whole wavefronts: latents of 128 (the matrix-core attention in bfloat16), states of 64 rows
    "wide": model(200, 128, 1e-6, 512, [
        (latent(8, 64, 64, 128, 96, 0.1), dense(256, 1.0)),
        (ssd(4, 64, 64, 2, 4, 2), moe(8, 2, 64, shared=128)),
        (window(4, 2, 64, 64, 0.125, 100, 32, 256.0), moe(8, 2, 64, shared=128)),
        (again(0), None),
    ]),
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
        if last.startswith("norm") and not name.endswith("mix.norm"):
            std = 0.3  # a norm of the stream: stored around zero
        elif last == "norm":
            std, offset = 0.3, 1.0  # the latents' and the read-out's norms: plain weights
        elif last == "conv":
            std = 0.5
        elif name.endswith("conv.b"):
            std = 0.2
        elif last in ("A_log", "dt_bias"):
            std = 0.7
        elif last == "D":
            std, offset = 0.5, 1.0
        elif last in ("sink", "rel"):
            std = 1.0
        elif last == "router":
            std = 4.0 / (spec.shape[-1] ** 0.5)
        elif name in ("embed", "pos"):
            std = 1.0 if name == "embed" else 0.5
        else:
            std = 1.5 / (spec.shape[-1] ** 0.5)
        out[name] = (torch.randn(spec.shape, generator=g) * std + offset).to(torch.bfloat16).float()
    return out


def make_requests(cfg: dict, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def make_runner(cfg, weights, dtype, device, ops, page_size, num_pages, max_seqs=4, max_len=None) -> ModelRunner:
    max_len = max_len or cfg["max_positions"]
    eng = EngineConfig(page_size=page_size, num_pages=num_pages, max_num_seqs=max_seqs, max_model_len=max_len,
                       max_num_batched_tokens=max_len, dtype=dtype, device=device)
    m = build_model(cfg, eng, ops=ops)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    m.load({k: v.to(wd).to(device) for k, v in weights.items()})
    return ModelRunner(m, eng)


def plain_logits(cfg, weights, reqs) -> Dict[str, torch.Tensor]:
    return {rid: P.forward(weights, cfg, toks) for rid, toks in reqs.items()}


def plain_logits_and_gaps(cfg, weights, reqs):
    """The plain logits, and for every position the smallest gap, over the layers with a router, between the last
    chosen expert's logit and the best one left out (infinite where every expert is chosen).  An engine that rounds
    what a router reads may send a token whose gap is tiny to another expert, which is then another model: the
    comparisons leave such positions out."""
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


def relative_error(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per position: the root mean square of the logits' difference (its mean taken off) against that of the logits."""
    d = got.double() - want
    d = d - d.mean(dim=1, keepdim=True)
    w = want - want.mean(dim=1, keepdim=True)
    return d.pow(2).mean(dim=1).sqrt() / w.pow(2).mean(dim=1).sqrt().clamp_min(1e-30)


F32_TOL = 1e-4
# bfloat16 against the unrounded float64 implementation: most positions within BF16_TOL, none beyond BF16_WORST;
# positions whose router gap is below CLOSE_CALL are left out (see plain_logits_and_gaps)
BF16_TOL = 6e-2
BF16_FEW = 0.1
BF16_WORST = 0.5
CLOSE_CALL = {True: 0.25, False: 1e-3}


def assert_matches(got, want, bf16: bool, what: str, gaps=None) -> None:
    over = total = 0
    for rid, w in want.items():
        g = got[rid]
        assert g.shape == w.shape, f"{what}: request {rid} has {tuple(g.shape)} logits, expected {tuple(w.shape)}"
        assert torch.isfinite(g).all(), f"{what}: request {rid} has non-finite logits"
        err = relative_error(g, w)
        if gaps is not None:
            err = err[gaps[rid] >= CLOSE_CALL[bf16]]
        tol = BF16_WORST if bf16 else F32_TOL
        if (err > tol).any():
            first = int(torch.nonzero(err > tol)[0])
            raise AssertionError(f"{what}: request {rid} first differs at the {first}th of {len(err)} compared positions "
                                 f"(relative error {err[first].item():.3e}, tolerance {tol:.1e}, largest {err.max().item():.3e})")
        over += int((err > BF16_TOL).sum())
        total += len(err)
    assert total > 0, f"{what}: nothing was compared"
    if bf16:
        assert over <= max(1, BF16_FEW * total), f"{what}: {over} of {total} positions differ by more than {BF16_TOL:.1e}"
