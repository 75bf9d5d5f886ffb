"""Named shapes of the Llama 3 family as config.json dictionaries, for runs with random
weights: the command line's ``--random NAME`` and the benchmark take them from here (the
reference's example script names its model as a constant at its top, examples/infer.py:13-16,
and needs the checkpoint; here a name stands for the layer sizes alone).
"""
from __future__ import annotations

from typing import Dict, Tuple

LLAMA3_8B = {
    "architectures": ["LlamaForCausalLM"],
    "hidden_size": 4096,
    "num_hidden_layers": 32,
    "num_attention_heads": 32,
    "num_key_value_heads": 8,
    "head_dim": 128,
    "intermediate_size": 14336,
    "vocab_size": 128256,
    "rms_norm_eps": 1e-5,
    "rope_theta": 500000.0,
    "rope_scaling": None,
    "max_position_embeddings": 8192,
    "tie_word_embeddings": False,
}
_LLAMA3_SCALING = {"rope_type": "llama3", "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                   "original_max_position_embeddings": 8192}
LLAMA32_3B = dict(LLAMA3_8B, hidden_size=3072, num_hidden_layers=28, num_attention_heads=24, intermediate_size=8192,
                  rope_scaling=dict(_LLAMA3_SCALING, factor=32.0), tie_word_embeddings=True)
LLAMA32_1B = dict(LLAMA3_8B, hidden_size=2048, num_hidden_layers=16, num_attention_heads=32, head_dim=64, intermediate_size=8192,
                  rope_scaling=dict(_LLAMA3_SCALING, factor=32.0), tie_word_embeddings=True)
LLAMA31_70B = dict(LLAMA3_8B, hidden_size=8192, num_hidden_layers=80, num_attention_heads=64, intermediate_size=28672,
                   rope_scaling=dict(_LLAMA3_SCALING, factor=8.0))
# two shapes of a few thousand parameters that differ in every size and option
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 192, "vocab_size": 256, "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0, "rope_scaling": None, "max_position_embeddings": 128, "tie_word_embeddings": False,
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 128, "num_hidden_layers": 3, "num_attention_heads": 4,
    "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 352, "vocab_size": 384, "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "max_position_embeddings": 256, "tie_word_embeddings": True,
}



def suranex_shape(width: int, vocab: int, heads: int, kv_heads: int, dim: int, window: int, recurrent_width: int, blocks: int,
                  experts: int, top: int, ff: int, shared_ff: int, pattern=("attention", "attention", "rglru"), repeats: int = 2) -> dict:
    """A Suranex config.json of the given layer sizes: ``pattern`` repeated ``repeats`` times, every
    layer with a mixture of experts and a shared expert."""
    att = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "softcap": 30.0,
           "mask": {"size": window, "keep_first": 4},
           "rot": {"base": 10000.0, "dims": dim, "scaling": {"factor": 8.0, "original": 4096, "fast": 16.0, "slow": 2.0}}}
    rec = {"width": recurrent_width, "blocks": blocks, "conv": 4}
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": 7.0},
           "shared": {"ff": shared_ff, "limit": 7.0}}
    layers = [{"type": kind, "mixer": dict(att if kind == "attention" else rec), "mlp": dict(mlp)} for kind in pattern * repeats]
    return {"architecture": "Suranex", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "layers": layers}


def nutavik_shape(width: int, vocab: int, heads: int, dim: int, rot_dim: int, kv_rank: int, q_rank: int, delta_heads: int,
                  delta_kv_heads: int, gla_heads: int, gla_dim: int, gla_vdim: int, ff: int, repeats: int = 2) -> dict:
    """A Nutavik config.json of the given layer sizes: (latent attention, delta rule, gated linear
    attention) repeated ``repeats`` times, every layer with a dense feed-forward; latent-attention
    layers after the first read the first one's cache."""
    rot = {"base": 10000.0, "dims": rot_dim, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}
    att = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": dim, "kv_rank": kv_rank, "q_rank": q_rank,
           "scale": (dim + rot_dim) ** -0.5, "rot": rot}
    dl = {"heads": delta_heads, "kv_heads": delta_kv_heads, "dim": dim, "vdim": dim, "conv": 4}
    gl = {"heads": gla_heads, "dim": gla_dim, "vdim": gla_vdim, "tau": 16.0, "low_rank": 16}
    layers = []
    for r in range(repeats):
        layers.append({"type": "latent_attention", "mixer": dict(att, **({"kv_from": 0} if r else {})), "mlp": {"kind": "dense", "ff": ff}})
        layers.append({"type": "delta", "mixer": dict(dl), "mlp": {"kind": "dense", "ff": ff}})
        layers.append({"type": "gla", "mixer": dict(gl), "mlp": {"kind": "dense", "ff": ff}})
    return {"architecture": "Nutavik", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "residual_mult": 0.5, "logit_scale": 1.0,
            "layers": layers}


def mesolix_shape(width: int, vocab: int, heads: int, kv_heads: int, dim: int, kv_rank: int, q_rank: int, window: int, ssd_heads: int,
                  ssd_vdim: int, state: int, groups: int, ff: int, experts: int, top: int, expert_ff: int, shared_ff: int,
                  bias_rows: int = 32, max_positions: int = 8192, repeats: int = 2, again: bool = False) -> dict:
    """A Mesolix config.json of the given layer sizes: (latent attention, state space duality, windowed attention
    with a bias per distance) repeated ``repeats`` times, dense and routed feed-forwards in turn; with ``again`` a last
    layer runs the first one's weights once more."""
    lat = {"heads": heads, "dim": dim, "vdim": dim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": dim ** -0.5}
    ssd = {"heads": ssd_heads, "vdim": ssd_vdim, "state": state, "groups": groups, "conv": 4, "norm_groups": groups}
    att = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "bias_max": float(2 * window),
           "bias_rows": bias_rows, "mask": {"size": window}}
    dense = {"kind": "dense", "ff": ff, "limit": 7.0}
    moe = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff}, "shared": {"ff": shared_ff}}
    layers = []
    for r in range(repeats):
        for i, (kind, mixer) in enumerate((("latent_attention", lat), ("mamba2", ssd), ("attention", att))):
            layers.append({"type": kind, "mixer": dict(mixer), "mlp": dict(dense if (3 * r + i) % 2 == 0 else moe)})
    if again:
        layers.append(dict(layers[0], weights_of=0))
    return {"architecture": "Mesolix", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": 1e-6}, "layers": layers}


def bekedra_shape(width: int, vocab: int, heads: int, kv_heads: int, dim: int, experts: int, top: int, expert_ff: int,
                  pattern=("attention_2", "attention", "attention", "attention_2"), loop=(1, 3, 2), original: int = 4096) -> dict:
    """A Bekedra config.json of the given layer sizes: the mixers of ``pattern``, every layer with a mixture of experts,
    the layers loop[0] .. loop[1] - 1 run loop[2] times in a row."""
    first = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "q_temp": {"coef": 0.1, "every": 1024}}
    second = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "softcap": 30.0,
              "rot": {"base": 500000.0, "dims": dim // 2, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": original}}}
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff}}
    layers = [{"type": kind, "mixer": dict(first if kind == "attention" else second), "mlp": dict(mlp)} for kind in pattern]
    cfg = {"architecture": "Bekedra", "vocab": vocab, "width": width, "embedding": {"scale": float(width) ** 0.5}, "norm": {"eps": 1e-6},
           "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def layer_runs(design: dict) -> int:
    """How many layers a token passes through (a looped stretch counts every pass)."""
    loop = design.get("loop")
    n = len(design["layers"])
    return n if not loop else n + (loop["stop"] - loop["start"]) * (loop["times"] - 1)


def llama_like(design: dict) -> dict:
    """The Llama configuration of equal size.  For Suranex: the same width, layer count, vocabulary
    and (first attention layer's) heads, a feed-forward as wide as what a token uses of the mixture
    (its top experts and the shared one).  For Nutavik: the same width, layer count, vocabulary and
    attention heads (keys as wide as its unrotated and rotated parts together, a quarter as many key
    heads), a gated feed-forward with as many weights as its dense one (two thirds as wide)."""
    if design.get("architecture") == "Bekedra":
        # the same width, vocabulary and heads, as many layers as a token passes through, a feed-forward with as many
        # weights as what a token uses of the mixture (three matrices against an expert's two)
        att = design["layers"][0]["mixer"]
        f = next(layer["mlp"] for layer in design["layers"] if layer["mlp"] is not None)
        inter = (2 * f["router"]["top"] * f["expert"]["ff"] // 3 + 255) // 256 * 256
        return dict(LLAMA3_8B, hidden_size=design["width"], num_hidden_layers=layer_runs(design), num_attention_heads=att["heads"],
                    num_key_value_heads=att["kv_heads"], head_dim=att["dim"], intermediate_size=inter, vocab_size=design["vocab"])
    if design.get("architecture") == "Mesolix":
        # the same width, layer count, vocabulary and (windowed attention's) heads; a feed-forward with as many
        # weights as the mean of what a token uses of the dense and the routed ones
        att = next(layer["mixer"] for layer in design["layers"] if layer["type"] == "attention")
        used = []
        for layer in design["layers"]:
            f = layer["mlp"]
            if f is not None:
                used.append(f["ff"] if f["kind"] == "dense" else f["router"]["top"] * f["expert"]["ff"] + (f["shared"]["ff"] if f.get("shared") else 0))
        inter = (sum(used) // max(len(used), 1) + 255) // 256 * 256
        return dict(LLAMA3_8B, hidden_size=design["width"], num_hidden_layers=len(design["layers"]), num_attention_heads=att["heads"],
                    num_key_value_heads=att["kv_heads"], head_dim=att["dim"], intermediate_size=inter, vocab_size=design["vocab"])
    if design.get("architecture") == "Nutavik":
        att = next(layer["mixer"] for layer in design["layers"] if layer["type"] == "latent_attention")
        ff = next(layer["mlp"]["ff"] for layer in design["layers"] if layer["mlp"] is not None)
        head_dim = 128 if att["dim"] + att["rot_dim"] > 64 else 64
        return dict(LLAMA3_8B, hidden_size=design["width"], num_hidden_layers=len(design["layers"]), num_attention_heads=att["heads"],
                    num_key_value_heads=max(1, att["heads"] // 4), head_dim=head_dim, intermediate_size=(2 * ff // 3 + 255) // 256 * 256,
                    vocab_size=design["vocab"])
    suranex = design
    att = next(layer["mixer"] for layer in suranex["layers"] if layer["type"] == "attention")
    mlp = next(layer["mlp"] for layer in suranex["layers"] if layer["mlp"] is not None)
    inter = mlp["router"]["top"] * mlp["expert"]["ff"] + (mlp["shared"]["ff"] if mlp.get("shared") else 0)
    return dict(LLAMA3_8B, hidden_size=suranex["width"], num_hidden_layers=len(suranex["layers"]), num_attention_heads=att["heads"],
                num_key_value_heads=att["kv_heads"], head_dim=att["dim"], intermediate_size=inter, vocab_size=suranex["vocab"])


def nutavik_like(design: dict) -> dict:
    """The Nutavik configuration of a Mesolix one's size: the same width, vocabulary and layer count (in threes), a
    latent attention of the same heads and ranks with a rotated part of 64 (or a quarter of the latent) on top, the
    two recurrences with as many heads and as wide keys and values as the state-space layer's state and channels,
    a dense feed-forward as wide as Mesolix's dense one."""
    lat = next(layer["mixer"] for layer in design["layers"] if layer["type"] == "latent_attention")
    ssd = next(layer["mixer"] for layer in design["layers"] if layer["type"] == "mamba2")
    ff = next(layer["mlp"]["ff"] for layer in design["layers"] if layer["mlp"] is not None and layer["mlp"]["kind"] == "dense")
    rot = 64 if lat["kv_rank"] >= 256 else max(2, lat["kv_rank"] // 4)
    return nutavik_shape(design["width"], design["vocab"], lat["heads"], lat["dim"], rot, lat["kv_rank"], lat["q_rank"], ssd["heads"],
                         max(1, ssd["heads"] // 2), ssd["heads"], ssd["state"], ssd["vdim"], ff, repeats=max(1, len(design["layers"]) // 3))


def mesolix_like(design: dict) -> dict:
    """The Mesolix configuration of a Bekedra one's size: the same width, vocabulary, heads and experts (no shared
    expert), as many layers as a token passes through (in threes), a window as long as the benchmark's prompts."""
    att = design["layers"][0]["mixer"]
    f = next(layer["mlp"] for layer in design["layers"] if layer["mlp"] is not None)
    width = design["width"]
    cfg = mesolix_shape(width, design["vocab"], att["heads"], att["kv_heads"], att["dim"], 512, 768 * width // 2048, 2048, 2 * att["heads"], 64, 128,
                        max(1, att["heads"] // 8), 4 * width, f["router"]["experts"], f["router"]["top"], f["expert"]["ff"], f["expert"]["ff"],
                        repeats=max(1, layer_runs(design) // 3))
    for layer in cfg["layers"]:
        if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe":
            layer["mlp"].pop("shared", None)
    return cfg


SURANEX_2K = suranex_shape(2048, 32768, 16, 4, 128, 1024, 2560, 10, 16, 2, 1024, 2048)
SURANEX_4K = suranex_shape(4096, 65536, 32, 8, 128, 2048, 5120, 20, 32, 4, 1024, 4096, repeats=1)
SURANEX_TINY = suranex_shape(64, 256, 4, 2, 16, 24, 96, 3, 4, 2, 32, 48, repeats=1)
NUTAVIK_2K = nutavik_shape(2048, 32768, 16, 128, 64, 512, 768, 16, 8, 4, 256, 512, 8192)
NUTAVIK_4K = nutavik_shape(4096, 65536, 32, 128, 64, 512, 1536, 32, 16, 8, 256, 512, 16384, repeats=1)
NUTAVIK_TINY = nutavik_shape(64, 256, 4, 16, 8, 24, 32, 4, 2, 2, 16, 32, 96, repeats=1)
MESOLIX_2K = mesolix_shape(2048, 32768, 16, 4, 128, 512, 768, 1024, 32, 64, 128, 2, 8192, 16, 2, 1024, 2048)
MESOLIX_4K = mesolix_shape(4096, 65536, 32, 8, 128, 512, 1536, 2048, 64, 64, 128, 4, 16384, 32, 4, 1024, 4096, repeats=1)
MESOLIX_TINY = mesolix_shape(64, 256, 4, 2, 16, 24, 32, 24, 4, 8, 16, 2, 96, 4, 2, 32, 48, bias_rows=8, max_positions=256, repeats=1, again=True)

BEKEDRA_2K = bekedra_shape(2048, 32768, 16, 4, 128, 16, 2, 1024)
BEKEDRA_4K = bekedra_shape(4096, 65536, 32, 8, 128, 32, 4, 1024, pattern=("attention_2", "attention"), loop=(1, 2, 2))
BEKEDRA_TINY = bekedra_shape(64, 256, 4, 2, 16, 4, 2, 32, pattern=("attention_2", "attention", "attention_2"), loop=(0, 2, 2), original=32)

# name -> (what to call it, config.json dictionary)
SHAPES: Dict[str, Tuple[str, dict]] = {
    "8b": ("Llama-3-8B", LLAMA3_8B),
    "3b": ("Llama-3.2-3B", LLAMA32_3B),
    "1b": ("Llama-3.2-1B", LLAMA32_1B),
    "70b": ("Llama-3.1-70B", LLAMA31_70B),
    "tiny-a": ("tiny Llama A", TINY_A),
    "tiny-b": ("tiny Llama B", TINY_B),
    "suranex-2k": ("Suranex, width 2,048", SURANEX_2K),
    "suranex-4k": ("Suranex, width 4,096", SURANEX_4K),
    "suranex-tiny": ("tiny Suranex", SURANEX_TINY),
    "nutavik-2k": ("Nutavik, width 2,048", NUTAVIK_2K),
    "nutavik-4k": ("Nutavik, width 4,096", NUTAVIK_4K),
    "nutavik-tiny": ("tiny Nutavik", NUTAVIK_TINY),
    "mesolix-2k": ("Mesolix, width 2,048", MESOLIX_2K),
    "mesolix-4k": ("Mesolix, width 4,096", MESOLIX_4K),
    "mesolix-tiny": ("tiny Mesolix", MESOLIX_TINY),
    "bekedra-2k": ("Bekedra, width 2,048", BEKEDRA_2K),
    "bekedra-4k": ("Bekedra, width 4,096", BEKEDRA_4K),
    "bekedra-tiny": ("tiny Bekedra", BEKEDRA_TINY),
}


def shape(name: str) -> Tuple[str, dict]:
    if name not in SHAPES:
        raise ValueError(f"unknown shape {name!r}; known: {sorted(SHAPES)}")
    label, cfg = SHAPES[name]
    return label, dict(cfg)
