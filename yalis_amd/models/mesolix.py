"""Mesolix: a small decoder whose config.json lists its layers one by one, each with one of three mixers and a
dense or routed feed-forward (or none), in pre-norm blocks; a layer may run another layer's weights again with a
cache and state of its own.

What the design fixes (everything else is read from config.json or a tensor's shape):
  * the stream starts as embed[token] + pos[position], a learned vector per absolute position;
  * a layer is  x += mixer(norm1(x));  x += ff(norm2(x))  with RMS norms whose weight is stored around zero
    (multiplied as 1 + w); the final norm is of the same kind, the head a matrix of its own;
  * mixer "latent_attention": queries through a normed latent (``q_rank``), keys and values through a normed latent
    of ``kv_rank`` elements, which is all the cache holds; no rotated part and no positions beyond the causal mask;
    a learned sink per head in the softmax's denominator; the concatenated heads gated element by element with the
    sigmoid of a projection of the mixer's input;
  * mixer "mamba2": state space duality (parts/linear_state.py), B and C shared by groups of heads, a causal
    convolution with bias and silu on x, B and C, the read-out gated by silu(z) and then normed in
    ``norm_groups`` parts;
  * mixer "attention": grouped query heads without any rotation; a learned bias per head and bucket of distance
    added to the scaled scores (the table's rows are read from the tensor, ``bias_max`` is where the last bucket
    ends); a sliding window of ``mask.size`` keys; the same element-wise gate;
  * feed-forward "dense": min(g, limit) sigmoid(1.702 min(g, limit)) (clamp(u, -limit, limit) + 1);
  * feed-forward "moe": a router with sigmoid scores chooses ``top`` experts, whose scores multiply their inputs
    and are not renormalised; experts and the optional shared expert are silu-gated feed-forwards.

config.json: {"architecture": "Mesolix", "vocab", "width", "max_positions", "norm": {"eps"}, "layers": [{"type",
"mixer": {...}, "mlp": {...} | null, "weights_of": j (optional)}]}; tensors "embed", "pos", "l<i>.norm1",
"l<i>.norm2", "l<i>.mix.*", "l<i>.mlp.*", "final.norm", "head".
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.reader import ConfigError, KeyReader
from ..config.registry import register_architecture
from ..config.specs import LayerSpec, ModelSpec, PartSpec, RunEntry

ARCHITECTURE_NAME = "Mesolix"
SWISH_SLOPE = 1.702  # the sigmoid's slope in the dense feed-forward's gated pair
MIXERS = ("latent_attention", "mamba2", "attention")


@dataclass(frozen=True)
class MesolixLayer:
    kind: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]
    weights_of: Optional[int]  # the layer whose tensors this one runs again (None: its own)


@dataclass(frozen=True)
class MesolixConfig:
    vocab: int
    width: int
    eps: float
    max_positions: int
    layers: Tuple[MesolixLayer, ...]
    raw: Dict[str, Any]

    @staticmethod
    def _latent_attention(m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = {"heads": r.integer("heads", minimum=1), "dim": r.integer("dim", minimum=1), "vdim": r.integer("vdim", minimum=1),
               "kv_rank": r.integer("kv_rank", minimum=1), "q_rank": r.integer("q_rank", minimum=1),
               "scale": r.number("scale", positive=True)}
        r.finish()
        return out

    @staticmethod
    def _mamba2(m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = {"heads": r.integer("heads", minimum=1), "vdim": r.integer("vdim", minimum=1), "state": r.integer("state", minimum=1),
               "groups": r.integer("groups", minimum=1), "conv": r.integer("conv", minimum=1),
               "norm_groups": r.integer("norm_groups", minimum=1)}
        if out["heads"] % out["groups"]:
            raise ConfigError(f"{where}: heads={out['heads']} is not a multiple of groups={out['groups']}")
        if (out["heads"] * out["vdim"]) % out["norm_groups"]:
            raise ConfigError(f"{where}: heads * vdim = {out['heads'] * out['vdim']} does not divide into norm_groups={out['norm_groups']} parts")
        r.finish()
        return out

    @staticmethod
    def _attention(m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = {"heads": r.integer("heads", minimum=1), "kv_heads": r.integer("kv_heads", minimum=1), "dim": r.integer("dim", minimum=1),
               "vdim": r.integer("vdim", minimum=1), "scale": r.number("scale", positive=True),
               "bias_max": r.number("bias_max", positive=True),
               # the table's rows: read from the tensor unless given (random weights need a number)
               "bias_rows": r.integer("bias_rows", default=None, minimum=2), "window": None}
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"{where}: heads={out['heads']} is not a multiple of kv_heads={out['kv_heads']}")
        mask = r.mapping("mask", default=None)
        if mask is not None:
            mr = KeyReader(mask, where=where + " mask")
            out["window"] = mr.integer("size", default=None, minimum=1)
            mr.finish()
        r.finish()
        return out

    @staticmethod
    def _mlp(f: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(f, where=where)
        kind = r.require_value("kind", ["dense", "moe"], None)
        if kind == "dense":
            out = {"kind": "dense", "ff": r.integer("ff", minimum=1), "limit": r.number("limit", positive=True)}
            r.finish()
            return out
        router = KeyReader(r.mapping("router"), where=where + " router")
        expert = KeyReader(r.mapping("expert"), where=where + " expert")
        out = {"kind": "moe", "experts": router.integer("experts", minimum=1), "top": router.integer("top", minimum=1),
               "ff": expert.integer("ff", minimum=1), "shared": None}
        if out["top"] > out["experts"]:
            raise ConfigError(f"{where}: top={out['top']} of {out['experts']} experts")
        shared = r.mapping("shared", default=None)
        if shared is not None:
            sr = KeyReader(shared, where=where + " shared")
            out["shared"] = {"ff": sr.integer("ff", minimum=1)}
            sr.finish()
        router.finish()
        expert.finish()
        r.finish()
        return out

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], strict: bool = False) -> "MesolixConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab", minimum=1), r.integer("width", minimum=1)
        max_positions = r.integer("max_positions", minimum=1)
        eps = KeyReader(r.mapping("norm"), where="config.json norm").number("eps", positive=True)
        listed = r.raw_value("layers", None)
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        readers = {"latent_attention": cls._latent_attention, "mamba2": cls._mamba2, "attention": cls._attention}
        layers = []
        for i, entry in enumerate(listed):
            where = f"config.json layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{where} must be an object")
            er = KeyReader(entry, where=where)
            kind = er.string("type")
            if kind not in readers:
                raise ConfigError(f"{where}: mixer type {kind!r} is not one of this design's {MIXERS}")
            m = readers[kind](er.mapping("mixer"), where + " mixer")
            mlp = er.mapping("mlp", default=None)
            layers.append(MesolixLayer(kind, m, None if mlp is None else cls._mlp(mlp, where + " mlp"),
                                       er.integer("weights_of", default=None, minimum=0)))
            er.finish()
        for i, layer in enumerate(layers):
            j = layer.weights_of
            if j is None:
                continue
            where = f"config.json layers[{i}]"
            if not j < i or layers[j].weights_of is not None:
                raise ConfigError(f"{where}: weights_of={j} must name an earlier layer that has tensors of its own")
            if (layers[j].kind, layers[j].mixer, layers[j].mlp) != (layer.kind, layer.mixer, layer.mlp):
                raise ConfigError(f"{where}: a layer that runs layer {j}'s weights again has layer {j}'s type, mixer and mlp")
        r.taken.add("architecture")
        r.finish(strict=strict)
        return cls(vocab, width, eps, max_positions, tuple(layers), dict(raw))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def build_mesolix_spec(cfg: MesolixConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"name": name, "size": cfg.width, "eps": cfg.eps, "unit_offset": True})

    layers, spec_index = [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p, m = f"l{i}", layer.mixer
        common = {"prefix": f"{p}.mix", "hidden_size": cfg.width}
        if layer.kind == "latent_attention":
            mixer = PartSpec("latent_attention", dict(
                common, num_heads=m["heads"], head_dim=m["dim"], rot_dim=0, value_dim=m["vdim"], kv_rank=m["kv_rank"], q_rank=m["q_rank"],
                scale=m["scale"], latent_eps=cfg.eps, gate="g", gate_per="element", sink="sink", position=None))
        elif layer.kind == "mamba2":
            mixer = PartSpec("state_space_duality", dict(
                common, num_heads=m["heads"], value_dim=m["vdim"], state_dim=m["state"], groups=m["groups"], conv_taps=m["conv"],
                norm_groups=m["norm_groups"], out_norm_eps=cfg.eps))
        else:
            mixer = PartSpec("attention", dict(
                common, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"], scale=m["scale"],
                window=m["window"], names={"q": "q", "k": "k", "v": "v", "o": "o"}, position=None, gate="g", gate_per="element",
                distance_bias={"name": "rel", "far": m["bias_max"], "buckets": m["bias_rows"]}))
        ffn = ffn_norm = None
        f = layer.mlp
        if f is not None and f["kind"] == "dense":
            ffn = PartSpec("gated_mlp", {"prefix": f"{p}.mlp", "hidden_size": cfg.width, "intermediate_size": f["ff"],
                                         "activation": ("clamped_swish", f["limit"], SWISH_SLOPE),
                                         "names": {"gate": "gate", "up": "up", "down": "down"}})
        elif f is not None:
            ffn = PartSpec("routed_moe", {
                "prefix": f"{p}.mlp", "hidden_size": cfg.width, "experts": f["experts"], "top": f["top"], "intermediate_size": f["ff"],
                "activation": "silu",
                "shared": None if f["shared"] is None else {"intermediate_size": f["shared"]["ff"], "activation": "silu"}})
        if ffn is not None:
            ffn_norm = norm(f"{p}.norm2")
        spec_index[i] = len(layers)
        layers.append(LayerSpec.of(p, "prenorm", mixer_norm=norm(f"{p}.norm1"), mixer=mixer, feed_forward_norm=ffn_norm, feed_forward=ffn))
    # a layer with weights_of runs the named layer's parts once more: another entry of the run order, which has a
    # cache or state of its own
    order = tuple(RunEntry(layer=spec_index[i if layer.weights_of is None else layer.weights_of]) for i, layer in enumerate(cfg.layers))
    spec = ModelSpec(
        architecture=ARCHITECTURE_NAME,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=cfg.max_positions,
        embedding=PartSpec("token_position_embedding", {"name": "embed", "position_name": "pos", "vocab_size": cfg.vocab,
                                                        "hidden_size": cfg.width, "max_positions": cfg.max_positions}),
        layers=tuple(layers),
        run_order=order,
        final_norm=norm("final.norm"),
        head=PartSpec("lm_head", {"name": "head", "tied_to": None, "vocab_size": cfg.vocab, "hidden_size": cfg.width}),
    )
    spec.validate()
    return spec


register_architecture(ARCHITECTURE_NAME, MesolixConfig, build_mesolix_spec)
