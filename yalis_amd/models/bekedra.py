"""Bekedra: a small decoder whose config.json lists its layers one by one, each with one of two attention mixers
and a routed mixture of experts (or no feed-forward), in parallel blocks; a stretch of the layers may run several
times in a row with the same weights.

What the design fixes (everything else is read from config.json or a tensor's shape):
  * the stream starts as embed[token] * embedding.scale; the head is the embedding table itself, unscaled;
  * a layer is  x += mixer(norm1(x)) + ff(norm1(x)): one RMS norm (plain weight) that both branches read;
  * ``loop``: layers start .. stop - 1 run ``times`` times in a row; every pass has pages of its own, and before
    a pass's first layer row t of the tensor "loop.step" is added to the stream (t the pass's number);
  * mixer "attention": grouped heads; q and k with biases; the values are the keys as projected (with the bias,
    before any norm; there is no v projection); one RMS norm over all of a token's query heads at once and one over
    all its key heads, with weights as wide as the projections; no rotation; queries multiplied by
    1 + coef ln(floor((p + 1) / every) + 1) at position p; plain softmax over every earlier key;
  * mixer "attention_2": grouped heads without biases; an RMS norm per head on queries and keys (one weight of
    ``dim`` elements for all heads) before the rotation; rotary positions on the first ``rot.dims`` elements of a
    head, pairs (i, i + dims / 2), with the three-band frequency scaling by wavelength; scores squashed to
    softcap tanh(s / softcap); a learned sink per head in the softmax's denominator; the concatenated heads gated
    element by element with the sigmoid of a projection of the mixer's input;
  * feed-forward "moe": router logits W h + b in float32, the ``top`` largest chosen, their weights the softmax
    over the chosen logits; an expert is down(relu(up h)^2) without biases; the weighted sum of their outputs.

config.json: {"architecture": "Bekedra", "vocab", "width", "embedding": {"scale"}, "norm": {"eps"}, "layers":
[{"type", "mixer": {...}, "mlp": {...} | null}], "loop": {"start", "stop", "times"} (optional)}; tensors "embed",
"loop.step", "l<i>.norm1", "l<i>.mix.*", "l<i>.mlp.*", "final.norm".
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.reader import ConfigError, KeyReader
from ..config.registry import register_architecture
from ..config.specs import LayerSpec, ModelSpec, PartSpec, RunEntry

ARCHITECTURE_NAME = "Bekedra"
MIXERS = ("attention", "attention_2")
# the design names no longest sequence; tables by position are made for the engine's own limit
MAX_POSITIONS = 1 << 20


@dataclass(frozen=True)
class BekedraLayer:
    kind: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


@dataclass(frozen=True)
class BekedraConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    layers: Tuple[BekedraLayer, ...]
    loop: Optional[Tuple[int, int, int]]  # (start, stop, times)
    raw: Dict[str, Any]

    @staticmethod
    def _heads(r: KeyReader, where: str) -> Dict[str, Any]:
        out = {"heads": r.integer("heads", minimum=1), "kv_heads": r.integer("kv_heads", minimum=1), "dim": r.integer("dim", minimum=1),
               "vdim": r.integer("vdim", minimum=1), "scale": r.number("scale", positive=True)}
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"{where}: heads={out['heads']} is not a multiple of kv_heads={out['kv_heads']}")
        return out

    @classmethod
    def _attention(cls, m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = cls._heads(r, where)
        if out["vdim"] != out["dim"]:
            raise ConfigError(f"{where}: the values are the keys, so vdim={out['vdim']} must equal dim={out['dim']}")
        out["q_temp"] = None
        temp = r.mapping("q_temp", default=None)
        if temp is not None:
            tr = KeyReader(temp, where=where + " q_temp")
            out["q_temp"] = {"coef": tr.number("coef"), "every": tr.integer("every", minimum=1)}
            tr.finish()
        r.finish()
        return out

    @classmethod
    def _attention_2(cls, m: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(m, where=where)
        out = cls._heads(r, where)
        out["softcap"] = r.number("softcap", default=None, positive=True)
        out["rot"] = None
        rot = r.mapping("rot", default=None)
        if rot is not None:
            rr = KeyReader(rot, where=where + " rot")
            dims = rr.integer("dims", minimum=2)
            if dims % 2 or dims > out["dim"]:
                raise ConfigError(f"{where} rot: dims={dims} must be even and at most dim={out['dim']}")
            out["rot"] = {"dims": dims, "base": rr.number("base", positive=True), "scaling": None}
            scaling = rr.mapping("scaling", default=None)
            if scaling is not None:
                sr = KeyReader(scaling, where=where + " rot scaling")
                out["rot"]["scaling"] = {
                    "kind": "llama3", "factor": sr.number("factor", positive=True), "low_freq_factor": sr.number("low", positive=True),
                    "high_freq_factor": sr.number("high", positive=True),
                    "original_max_position_embeddings": sr.number("original", positive=True)}
                if out["rot"]["scaling"]["high_freq_factor"] <= out["rot"]["scaling"]["low_freq_factor"]:
                    raise ConfigError(f"{where} rot scaling: 'high' must be larger than 'low'")
                sr.finish()
            rr.finish()
        r.finish()
        return out

    @staticmethod
    def _mlp(f: Dict[str, Any], where: str) -> Dict[str, Any]:
        r = KeyReader(f, where=where)
        r.require_value("kind", ["moe"], None)
        router = KeyReader(r.mapping("router"), where=where + " router")
        expert = KeyReader(r.mapping("expert"), where=where + " expert")
        out = {"experts": router.integer("experts", minimum=1), "top": router.integer("top", minimum=1), "ff": expert.integer("ff", minimum=1)}
        if out["top"] > out["experts"]:
            raise ConfigError(f"{where}: top={out['top']} of {out['experts']} experts")
        router.finish()
        expert.finish()
        r.finish()
        return out

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], strict: bool = False) -> "BekedraConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab", minimum=1), r.integer("width", minimum=1)
        eps = KeyReader(r.mapping("norm"), where="config.json norm").number("eps", positive=True)
        embedding = r.mapping("embedding", default=None)  # (left out: the rows as they are)
        scale = 1.0 if embedding is None else KeyReader(embedding, where="config.json embedding").number("scale", positive=True)
        listed = r.raw_value("layers", None)
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        readers = {"attention": cls._attention, "attention_2": cls._attention_2}
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
            layers.append(BekedraLayer(kind, m, None if mlp is None else cls._mlp(mlp, where + " mlp")))
            er.finish()
        loop = None
        looped = r.mapping("loop", default=None)
        if looped is not None:
            lr = KeyReader(looped, where="config.json loop")
            loop = (lr.integer("start", minimum=0), lr.integer("stop", minimum=1), lr.integer("times", minimum=1))
            if not loop[0] < loop[1] <= len(layers):
                raise ConfigError(f"config.json loop: start={loop[0]} .. stop={loop[1]} is no stretch of the {len(layers)} layers")
            lr.finish()
        r.taken.add("architecture")
        r.finish(strict=strict)
        return cls(vocab, width, eps, scale, tuple(layers), loop, dict(raw))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def build_bekedra_spec(cfg: BekedraConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"name": name, "size": cfg.width, "eps": cfg.eps, "unit_offset": False})

    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer.mixer
        common = {"prefix": f"{p}.mix", "hidden_size": cfg.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                  "head_dim": m["dim"], "value_dim": m["vdim"], "scale": m["scale"], "window": None}
        if layer.kind == "attention":
            mixer = PartSpec("attention", dict(
                common, names={"q": "q", "k": "k", "o": "o"}, position=None, values_from_keys=True,
                projection_bias={"q": "q.b", "k": "k.b"},
                qk_norm={"q": "q.norm", "k": "k.norm", "eps": cfg.eps, "over": "projection"},
                query_temperature=None if m["q_temp"] is None else {"coef": m["q_temp"]["coef"], "every": m["q_temp"]["every"]}))
        else:
            rot = m["rot"]
            mixer = PartSpec("attention", dict(
                common, names={"q": "q", "k": "k", "v": "v", "o": "o"},
                position=None if rot is None else PartSpec("rotary", {"rotary_dim": rot["dims"], "theta": rot["base"], "pairing": "half",
                                                                     "scaling": rot["scaling"]}),
                qk_norm={"q": "q.norm", "k": "k.norm", "eps": cfg.eps}, softcap=m["softcap"], sink="sink", gate="g", gate_per="element"))
        ffn = None
        if layer.mlp is not None:
            f = layer.mlp
            ffn = PartSpec("routed_moe", {
                "prefix": f"{p}.mlp", "hidden_size": cfg.width, "experts": f["experts"], "top": f["top"], "intermediate_size": f["ff"],
                "gated": False, "activation": "relu2", "router_bias": "router.b", "scores": "softmax_of_chosen", "weighs": "output"})
        layers.append(LayerSpec.of(p, "parallel", norm=norm(f"{p}.norm1"), mixer=mixer, feed_forward=ffn))
    n = len(layers)
    if cfg.loop is None:
        order = [RunEntry(layer=i) for i in range(n)]
    else:
        start, stop, times = cfg.loop
        order = [RunEntry(layer=i) for i in range(start)]
        for t in range(times):
            # a pass begins with its row of the table of steps; every pass's entries keep pages of their own
            order += [RunEntry(layer=i, added_row=("loop.step", t, times) if i == start else None) for i in range(start, stop)]
        order += [RunEntry(layer=i) for i in range(stop, n)]
    spec = ModelSpec(
        architecture=ARCHITECTURE_NAME,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=MAX_POSITIONS,
        embedding=PartSpec("token_embedding", {"name": "embed", "vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                               "scale": cfg.embedding_scale}),
        layers=tuple(layers),
        run_order=tuple(order),
        final_norm=norm("final.norm"),
        head=PartSpec("lm_head", {"name": "head", "tied_to": "embed", "vocab_size": cfg.vocab, "hidden_size": cfg.width}),
    )
    spec.validate()
    return spec


register_architecture(ARCHITECTURE_NAME, BekedraConfig, build_bekedra_spec)
