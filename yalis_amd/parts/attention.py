"""Causal self-attention with grouped key/value heads over a paged cache.

Reference: yalis/external/model.py:525-608 (projection, split into heads, rotary,
attention, output projection); the mask and softmax rules are those of
yalis/attention/backend_impl/sdpa_and_flex.py:15-19, 85-90, 300-312: query head h
reads key/value head h // (H/G), key j is visible to the query at position p iff
j <= p, softmax in float32.  The reference stores q, k and v rows interleaved per
group in one matrix (yalis/external/model.py:445-456); here the three checkpoint
matrices are stacked [q; k; v], which is the same arithmetic.

params: prefix, hidden_size, num_heads, num_kv_heads, head_dim, scale, window
(None: every earlier key), position (a PartSpec or None; this mixer uses a position
encoding's ``rotation()``), names (optional overrides of the tensor names below the
prefix), bias (False; True: the four projections have biases ``*.bias`` beside their
weights, which Llama's do not).

Options beyond the plain causal form (any of them sends the layer through the kernels that
prepare, mask and finish heads in general, ``ops.qkv_prepare`` / ``ops.attention_masked``):
value_dim (values narrower or wider than keys), qk_norm ({"q": name, "k": name, "eps": e}: an RMS
norm per head on queries and keys before the rotation, its weight of head_dim elements shared by
the heads), value_norm_eps (values divided by their root mean square per head before they are
cached), value_position (a rotary PartSpec over all of value_dim: values are cached rotated by
their position and a head's output is turned back by the query's position, so that what reaches
the output depends on distances), softcap (scores squashed to softcap * tanh(s / softcap)),
keep_first (that many first keys stay visible below the window), gate (a tensor name below the
prefix, [num_heads, hidden]: a head's output is multiplied by the sigmoid of its row's product with
the mixer's input; with gate_per "element" the tensor is [num_heads * value_dim, hidden] and the
concatenated heads are multiplied element by element), distance_bias ({"name": tensor below the
prefix, [buckets, num_heads]; "far": D; "buckets": B or None, the tensor's rows}: a learned number per
head added to the scaled score of a key n positions back, row bucket(n) of the tensor with bucket(n) =
n below B/2 and min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(D / (B/2)) * (B - B/2))) from there on, so
that distances up to B/2 have a row each and the rows beyond cover distances that grow
geometrically up to D), sink (a tensor name below the prefix, [num_heads]: exp(sink_h) joins the
softmax's denominator of head h once; it has no key and no value and is neither scaled nor squashed),
values_from_keys (True: there is no v projection; a token's values are its keys as projected, with
their bias and before any norm; value_dim = head_dim), projection_bias ({"q": name, "k": name}:
biases of the q and k projections below the prefix, added in float32 before everything else),
qk_norm["over"] ("head", the default, or "projection": one RMS norm over all of a token's query
heads together, and one over all its key heads, with weights as wide as the projections),
query_temperature ({"coef": c, "every": e}: the query at position p is multiplied by
1 + c ln(floor((p + 1) / e) + 1), after the norm).  A layer may have no position encoding at all
(``position`` None).
"""
from __future__ import annotations

import math
from typing import Dict, Mapping

import numpy as np
import torch

from ..config.specs import PartSpec
from ..engine.batch import attention_tiles, attention_token_columns
from ..weights.loader import TensorSpec
from .base import POSITIONS, KVNeed, Mixer, Runtime, register_mixer


@register_mixer("attention")
class Attention(Mixer):

    graph_capturable = True
    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.n_heads = int(params["num_heads"])
        self.n_kv = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        self.scale = float(params["scale"])
        self.window = params.get("window")
        if self.n_heads % self.n_kv:
            raise ValueError(f"num_heads={self.n_heads} is not a multiple of num_kv_heads={self.n_kv}")
        names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight"}
        names.update(params.get("names", {}))
        self.names = {k: f"{self.prefix}.{v}" for k, v in names.items()}
        # False when every run entry of this layer borrows another entry's cache
        self.projects_kv = bool(params.get("projects_kv", True))
        self.bias = bool(params.get("bias", False))
        pos: PartSpec = params.get("position")
        self.position = None if pos is None else POSITIONS.get(pos.kind)(pos.params, rt)
        # what this mixer takes of a position encoding: a rotation of queries and keys
        self.rotation = None if self.position is None else self.position.rotation()
        if self.position is not None and self.rotation is None:
            raise ValueError(f"{self.prefix}: position encoding {pos.kind!r} offers no rotation, which is all this mixer applies")
        if self.rotation is not None and self.rotation.rotary_dim > self.head_dim:
            raise ValueError("rotary_dim exceeds head_dim")
        self.value_dim = int(params.get("value_dim") or self.head_dim)
        self.qk_norm = params.get("qk_norm")
        self.value_norm_eps = params.get("value_norm_eps")
        vpos: PartSpec = params.get("value_position")
        self.value_position = None if vpos is None else POSITIONS.get(vpos.kind)(vpos.params, rt)
        self.value_rotation = None if self.value_position is None else self.value_position.rotation()
        if self.value_rotation is not None and self.value_rotation.rotary_dim != self.value_dim:
            raise ValueError(f"{self.prefix}: values rotate over all of value_dim={self.value_dim}")
        self.softcap = float(params.get("softcap") or 0.0)
        self.keep_first = int(params.get("keep_first") or 0)
        self.gate_name = params.get("gate")
        self.gate_per = params.get("gate_per", "head")
        if self.gate_per not in ("head", "element"):
            raise ValueError(f"{self.prefix}: gate_per is 'head' or 'element', got {self.gate_per!r}")
        self.gate_elems = self.value_dim if self.gate_per == "element" else 1
        self.distance_bias = params.get("distance_bias")
        self.bias_by_distance = None
        self.sink_name = params.get("sink")
        self.sink = None
        self.values_from_keys = bool(params.get("values_from_keys", False))
        if self.values_from_keys and self.value_dim != self.head_dim:
            raise ValueError(f"{self.prefix}: values that are the keys are as wide as the keys")
        self.projection_bias = dict(params.get("projection_bias") or {})
        if set(self.projection_bias) - {"q", "k"}:
            raise ValueError(f"{self.prefix}: projection_bias names the biases of q and k")
        self.norm_over_projection = bool(self.qk_norm) and self.qk_norm.get("over", "head") == "projection"
        if self.qk_norm and self.qk_norm.get("over", "head") not in ("head", "projection"):
            raise ValueError(f"{self.prefix}: qk_norm is over 'head' or 'projection'")
        self.query_temperature = params.get("query_temperature")
        if self.query_temperature is not None and int(self.query_temperature["every"]) < 1:
            raise ValueError(f"{self.prefix}: query_temperature every must be at least 1")
        self.b_proj = None
        self.masked = bool(
            self.value_dim != self.head_dim or self.qk_norm or self.value_norm_eps is not None or self.value_rotation is not None
            or self.softcap or self.keep_first or self.gate_name or self.distance_bias or self.sink_name or self.values_from_keys
            or self.projection_bias or self.query_temperature
        )
        self.w_qn = self.w_kn = None
        if self.masked:
            if self.bias:
                raise ValueError(f"{self.prefix}: the four biases are not offered together with the masked attention's options "
                                 "(projection_bias gives q and k theirs)")
            self.group = None
            self.w_qkv = self.w_q = self.w_o = None
            self.b_qkv = self.b_q = self.b_o = None
            self.rotates_in_launch = False
            # the matrix-core kernels take these options too, where they take the sizes (bfloat16, keys and
            # values of 64 or 128 elements alike); everything else runs on the general float32-arithmetic kernel
            can = getattr(rt.ops, "attention_can_rotate", None)
            self.on_matrix_cores = bool(can is not None and self.value_dim == self.head_dim and can(rt.act_dtype, self.head_dim) is True)
            if self.on_matrix_cores and self.sink_name:
                with_sink = getattr(rt.ops, "attention_takes_sink", None)
                self.on_matrix_cores = bool(with_sink is not None and with_sink(rt.act_dtype, self.head_dim) is True)
            if self.on_matrix_cores:
                self._tile_sizes(rt)
            return
        rt.ops.check_attention_sizes(self.n_heads, self.n_kv, self.head_dim, rt.page_size)
        self.on_matrix_cores = True  # (where the kernel library has them for these sizes: it decides per call)
        self._tile_sizes(rt)
        self.group = None
        self.w_qkv = self.w_q = self.w_o = None
        # whether the kernel library's attention can rotate and append inside its own launch
        # for steps of single tokens (one kernel fewer per layer), and what it needs for that
        can = getattr(rt.ops, "attention_can_rotate", None)
        self.rotates_in_launch = bool(can is not None and can(rt.act_dtype, self.head_dim))
        if self.rotates_in_launch:
            self.rope_in_launch = {append: rt.ops.rope_in_launch(self.rotation, append) for append in (False, True)}
        self.b_qkv = self.b_q = self.b_o = None

    def _tile_sizes(self, rt) -> None:
        self.tokens_per_tile = rt.ops.attention_tokens_per_tile(self.n_heads, self.n_kv)
        # spans longer than `long_tile` go to the kernel for long spans, in tiles of that many
        # tokens or twice as many (`long_tiles_of`: the step's choice)
        self.long_tile = rt.ops.attention_long_span_tile(self.n_heads, self.n_kv)
        self.long_tile_2 = rt.ops.attention_long_span_tile(self.n_heads, self.n_kv, 2)
        self.layout = f"h{self.n_heads}g{self.n_kv}"

    # ---- what it needs
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        hd = self.n_heads * self.head_dim
        kd = self.n_kv * self.head_dim
        specs = {
            self.names["q"]: TensorSpec((hd, self.hidden)),
            self.names["o"]: TensorSpec((self.hidden, self.n_heads * self.value_dim)),
        }
        if self.projects_kv:
            specs[self.names["k"]] = TensorSpec((kd, self.hidden))
            if not self.values_from_keys:
                specs[self.names["v"]] = TensorSpec((self.n_kv * self.value_dim, self.hidden))
        if self.qk_norm:
            qn, kn = (hd, kd) if self.norm_over_projection else (self.head_dim, self.head_dim)
            specs[f"{self.prefix}.{self.qk_norm['q']}"] = TensorSpec((qn,), "float", ("one_plus_normal", 0.1))
            if self.projects_kv:
                specs[f"{self.prefix}.{self.qk_norm['k']}"] = TensorSpec((kn,), "float", ("one_plus_normal", 0.1))
        if "q" in self.projection_bias:
            specs[f"{self.prefix}.{self.projection_bias['q']}"] = TensorSpec((hd,), "float", ("normal", 0.1))
        if "k" in self.projection_bias and self.projects_kv:
            specs[f"{self.prefix}.{self.projection_bias['k']}"] = TensorSpec((kd,), "float", ("normal", 0.1))
        if self.sink_name:
            specs[f"{self.prefix}.{self.sink_name}"] = TensorSpec((self.n_heads,), "float", ("normal", 1.0))
        if self.gate_name:
            specs[f"{self.prefix}.{self.gate_name}"] = TensorSpec((self.n_heads * self.gate_elems, self.hidden))
        if self.distance_bias:
            rows = self.distance_bias.get("buckets")
            specs[f"{self.prefix}.{self.distance_bias['name']}"] = TensorSpec((int(rows or 16), self.n_heads), "float", ("normal", 1.0),
                                                                              free_axes=() if rows else (0,))
        if self.bias:
            for which, spec in list(specs.items()):
                specs[self._bias_name(which)] = TensorSpec((spec.shape[0],), "float", ("normal", 0.02))
        return specs

    @staticmethod
    def _bias_name(weight_name: str) -> str:
        return weight_name[: -len("weight")] + "bias" if weight_name.endswith("weight") else weight_name + ".bias"

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        q = tensors[self.names["q"]]
        if self.masked:
            # one projection for everything that reads the mixer's input: [q; k; v; gates], its rows
            # padded to a multiple of 8 so that the few-row product's tiles take it
            parts = [q]
            if self.projects_kv:
                parts.append(tensors[self.names["k"]])
                if not self.values_from_keys:
                    parts.append(tensors[self.names["v"]])
            if self.gate_name:
                parts.append(tensors[f"{self.prefix}.{self.gate_name}"])
            rows = sum(p.shape[0] for p in parts)
            pad = -rows % 16
            if pad:
                parts.append(torch.zeros((pad, self.hidden), dtype=q.dtype, device=q.device))
            self.w_qkv = torch.cat(parts, dim=0).contiguous()
            self.w_o = tensors[self.names["o"]]
            if self.qk_norm:
                self.w_qn = tensors[f"{self.prefix}.{self.qk_norm['q']}"]
                self.w_kn = tensors[f"{self.prefix}.{self.qk_norm['k']}"] if self.projects_kv else self.w_qn
            if self.distance_bias:
                self.bias_by_distance = self._bias_by_distance(tensors[f"{self.prefix}.{self.distance_bias['name']}"])
            if self.sink_name:
                self.sink = tensors[f"{self.prefix}.{self.sink_name}"].to(torch.float32).contiguous()
            if self.projection_bias:
                # one float32 vector over the projection's columns: the biases where they are, zeros elsewhere
                b = torch.zeros(self.w_qkv.shape[0], dtype=torch.float32, device=q.device)
                if "q" in self.projection_bias:
                    b[: q.shape[0]] = tensors[f"{self.prefix}.{self.projection_bias['q']}"].to(torch.float32)
                if "k" in self.projection_bias and self.projects_kv:
                    kd = self.n_kv * self.head_dim
                    b[q.shape[0]: q.shape[0] + kd] = tensors[f"{self.prefix}.{self.projection_bias['k']}"].to(torch.float32)
                self.b_proj = b
            return
        if self.projects_kv:
            self.w_qkv = torch.cat([q, tensors[self.names["k"]], tensors[self.names["v"]]], dim=0).contiguous()
            self.w_q = self.w_qkv[: q.shape[0]]
        else:
            self.w_q = q
        self.w_o = tensors[self.names["o"]]
        if self.bias:
            b = lambda which: tensors[self._bias_name(self.names[which])]
            if self.projects_kv:
                self.b_qkv = torch.cat([b("q"), b("k"), b("v")]).contiguous()
                self.b_q = self.b_qkv[: q.shape[0]]
            else:
                self.b_q = b("q")
            self.b_o = b("o")

    @staticmethod
    def distance_bucket(n: int, buckets: int, far: float) -> int:
        half = buckets // 2
        if n < half:
            return n
        return min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (buckets - half))))

    def _bias_by_distance(self, table: torch.Tensor) -> torch.Tensor:
        """The table [buckets, heads] spread out as float32 [distances, heads], a row per distance a key can have:
        up to the window, or to where the last bucket begins (every larger distance reads the last row)."""
        buckets, far = int(table.shape[0]), float(self.distance_bias["far"])
        if buckets < 2 or far <= buckets // 2:
            raise ValueError(f"{self.prefix}: a distance bias needs at least two buckets and far={far} beyond the {buckets // 2} exact ones")
        reach = self.rt.max_positions if not self.window else min(int(self.window), self.rt.max_positions)
        rows = []
        for n in range(max(reach, 1)):
            rows.append(self.distance_bucket(n, buckets, far))
            if rows[-1] == buckets - 1:
                break
        index = torch.tensor(rows, dtype=torch.long, device=table.device)
        return table.float().index_select(0, index).contiguous()

    def kv_need(self) -> KVNeed:
        return KVNeed(self.n_kv, self.head_dim, self.window, None if self.value_dim == self.head_dim else self.value_dim,
                      self.keep_first if self.window else 0)

    def products(self):
        hd, kd = self.n_heads * self.head_dim, self.n_kv * self.head_dim
        if self.masked:
            v_rows = 0 if self.values_from_keys else self.n_kv * self.value_dim
            rows = hd + (kd + v_rows if self.projects_kv else 0) + (self.n_heads * self.gate_elems if self.gate_name else 0)
            return ((rows + (-rows % 16), self.hidden), (self.hidden, self.n_heads * self.value_dim))
        return ((hd + 2 * kd if self.projects_kv else hd, self.hidden), (self.hidden, hd))

    def long_col_tiles(self, hb) -> int:
        """Column tiles per wave for this step's long spans (1 or 2), from what the host
        knows of the batch: how many workgroups the larger tiles would make, and the fewest
        keys any long span has cached before it."""
        long_spans = hb.seq_qlen > self.long_tile
        if not long_spans.any():
            return 1
        qlen = hb.seq_qlen[long_spans].astype(np.int64)
        tiles = int((-(-qlen // self.long_tile_2)).sum())
        heads_per_tile = min(self.n_heads // self.n_kv, 16)
        chunks = -(-(self.n_heads // self.n_kv) // heads_per_tile)
        fewest = int((hb.seq_ctx[long_spans] - hb.seq_qlen[long_spans]).min())
        return self.rt.ops.attention_long_col_tiles(tiles * self.n_kv * chunks, fewest)

    def step_inputs(self):
        if self.masked and not self.on_matrix_cores:
            return {}
        # spans of more than one large tile go to the kernel for long spans, the rest
        # (single decoded tokens, short portions) to the one that splits the keys
        tpt = self.tokens_per_tile
        big, big2 = self.long_tile, self.long_tile_2
        none = np.zeros((0, 4), dtype=np.int32)
        # (the long tiles carry the head layout in their names: which of the two lists a step
        # fills depends on it, and layers with another layout must not read this one's choice)
        return {
            f"attention_tiles_{tpt}_upto{big}": lambda hb: attention_tiles(hb, tpt, 1, big),
            f"attention_token_columns_{tpt}_upto{big}": lambda hb: attention_token_columns(hb, tpt, 1, big),
            f"attention_long_tiles_{big}_{self.layout}": lambda hb: attention_tiles(hb, big, big + 1, longest_first=True)
            if self.long_col_tiles(hb) == 1 else none,
            f"attention_long_tiles_{big2}_{self.layout}": lambda hb: attention_tiles(hb, big2, big + 1, longest_first=True)
            if self.long_col_tiles(hb) == 2 else none,
        }

    # ---- what it computes
    def _forward_masked(self, h: torch.Tensor, ctx, site) -> torch.Tensor:
        ops = self.rt.ops
        if site.owns_cache != self.projects_kv:
            raise RuntimeError(f"{self.prefix}: a layer whose run entries both own and borrow caches is not offered with these options")
        proj = ops.linear(h, self.w_qkv, self.rt.act_dtype, partial_ok=True)
        n_kv_rows = self.n_kv if site.owns_cache else 0
        k_cache, v_cache = site.kv()
        more = {}
        if self.norm_over_projection or self.query_temperature is not None:
            # what a token's queries and keys are multiplied with as wholes: the inverse root mean square over all
            # heads at once, and the temperature of the token's position
            temp = self.query_temperature
            more["row_scales"] = ops.qk_row_scales(
                proj, self.n_heads * self.head_dim, n_kv_rows * self.head_dim, ctx.arrays["positions"], bias=self.b_proj,
                eps=float(self.qk_norm["eps"]) if self.norm_over_projection else None,
                temperature=None if temp is None else (float(temp["coef"]), int(temp["every"])))
        if self.norm_over_projection:
            more["norm_over_projection"] = True
        if self.b_proj is not None:
            more["bias"] = self.b_proj
        if self.values_from_keys:
            more["values_from_keys"] = True
        q = ops.qkv_prepare(
            proj, self.n_heads, n_kv_rows, self.head_dim, self.value_dim, ctx.arrays["positions"], self.rt.act_dtype,
            q_norm=self.w_qn, k_norm=self.w_kn, qk_eps=float(self.qk_norm["eps"]) if self.qk_norm else 0.0,
            rotation=self.rotation, value_norm_eps=self.value_norm_eps, value_rotation=self.value_rotation,
            k_cache=k_cache, v_cache=v_cache, slots=ctx.arrays[f"slots_g{site.group}"] if n_kv_rows else None,
            page_size=self.rt.page_size, **more,
        )
        gate_col = self.n_heads * self.head_dim + n_kv_rows * (self.head_dim + (0 if self.values_from_keys else self.value_dim))
        sink = {} if self.sink is None else {"sink": self.sink}
        if self.on_matrix_cores:
            memo_key = f"attention_long_col_tiles_{self.layout}"
            col_tiles = ctx.memo.get(memo_key)
            if col_tiles is None:
                col_tiles = ctx.memo[memo_key] = self.long_col_tiles(ctx.host)
            out = ops.attention(
                q, self.n_heads, self.n_kv, self.head_dim, k_cache, v_cache, self.rt.page_size, self.scale,
                0 if self.window is None else int(self.window), ctx, site.group,
                ctx.arrays[f"attention_tiles_{self.tokens_per_tile}_upto{self.long_tile}"],
                ctx.arrays[f"attention_long_tiles_{self.long_tile_2 if col_tiles == 2 else self.long_tile}_{self.layout}"],
                long_col_tiles=col_tiles, keep_first=self.keep_first if self.window else 0, softcap=self.softcap,
                distance_bias=self.bias_by_distance, **sink,
            )
            if self.value_rotation is not None or self.gate_name:
                ops.attention_finish(out, ctx.arrays["positions"], self.n_heads, self.value_dim, self.value_rotation,
                                     gate=proj if self.gate_name else None, gate_col=gate_col, gate_elems=self.gate_elems)
            return ops.linear(out, self.w_o, self.rt.act_dtype, partial_ok=True)
        out = ops.attention_masked(
            q, self.n_heads, self.n_kv, self.head_dim, self.value_dim, k_cache, v_cache, self.rt.page_size, self.scale, ctx,
            site.group, window=0 if self.window is None else int(self.window), keep_first=self.keep_first,
            softcap=self.softcap, value_rotation=self.value_rotation, gate=proj if self.gate_name else None, gate_col=gate_col,
            gate_elems=self.gate_elems, distance_bias=self.bias_by_distance, **sink,
        )
        return ops.linear(out, self.w_o, self.rt.act_dtype, partial_ok=True)

    def forward(self, h: torch.Tensor, ctx, site) -> torch.Tensor:
        if self.masked:
            return self._forward_masked(h, ctx, site)
        ops = self.rt.ops
        if site.owns_cache:
            if not self.projects_kv:
                raise RuntimeError(f"{self.prefix}: run entry owns a cache but the layer has no k/v projections")
            qkv = self._project(h, self.w_qkv, self.b_qkv)
            n_kv_rows = self.n_kv
        else:
            qkv = self._project(h, self.w_q, self.b_q)
            n_kv_rows = 0
        k_cache, v_cache = site.kv()
        memo_key = f"attention_long_col_tiles_{self.layout}"
        col_tiles = ctx.memo.get(memo_key)
        if col_tiles is None:
            col_tiles = ctx.memo[memo_key] = self.long_col_tiles(ctx.host)
        pos = self.rotation
        tiles = ctx.arrays[f"attention_tiles_{self.tokens_per_tile}_upto{self.long_tile}"]
        token_cols = ctx.arrays[f"attention_token_columns_{self.tokens_per_tile}_upto{self.long_tile}"]
        if ctx.max_qlen == 1 and self.rotates_in_launch:
            # a step of single tokens: rotary + append happen inside the attention launch
            out = ops.attention(
                qkv, self.n_heads, self.n_kv, self.head_dim, k_cache, v_cache, self.rt.page_size, self.scale,
                0 if self.window is None else int(self.window), ctx, site.group, tiles, token_cols=token_cols,
                rope=self.rope_in_launch[bool(n_kv_rows)],
            )
            return self._project(out, self.w_o, self.b_o)
        q = ops.rope_append(
            qkv,
            self.n_heads,
            n_kv_rows,
            self.head_dim,
            ctx.arrays["positions"],
            None if pos is None else pos.cos,
            None if pos is None else pos.sin,
            0 if pos is None else pos.rotary_dim,
            False if pos is None else pos.interleaved,
            k_cache,
            v_cache,
            ctx.arrays[f"slots_g{site.group}"],
            self.rt.page_size,
        )
        out = ops.attention(
            q,
            self.n_heads,
            self.n_kv,
            self.head_dim,
            k_cache,
            v_cache,
            self.rt.page_size,
            self.scale,
            0 if self.window is None else int(self.window),
            ctx,
            site.group,
            tiles,
            ctx.arrays[f"attention_long_tiles_{self.long_tile_2 if col_tiles == 2 else self.long_tile}_{self.layout}"],
            long_col_tiles=col_tiles,
            token_cols=token_cols,
        )
        return self._project(out, self.w_o, self.b_o)

    def _project(self, x, w, b):
        """x . w^T (+ b); without a bias the product may come as unreduced K slices."""
        if b is None:
            return self.rt.ops.linear(x, w, self.rt.act_dtype, partial_ok=True)
        return self.rt.ops.linear(x, w, self.rt.act_dtype, bias=b)
