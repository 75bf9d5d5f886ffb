"""Causal attention whose keys and values come from one small latent per token.

For a token with mixer input h and position p, per head (dim unrotated, rot_dim rotated query and
key elements, value_dim value elements):
    c_q = rmsnorm(W_dq h) * w_dq          q = W_uq c_q, head by head [dim | rot_dim]
    [l ; r] = W_dkv h                     c = rmsnorm(l) * w_dkv  (kv_rank)    kr = turn(r, p)  (rot_dim, one for all heads)
    k_head = W_uk,head c                  v_head = W_uv,head c
    score(i, j) = (q_i[:dim] . k_head,j + turn(q_i[dim:], i) . kr_j) * scale,  softmax over j <= i
    out = W_o concat_heads(sigmoid(W_g h)_head * sum_j p_ij v_head,j)
A token's page row holds [c | kr] and nothing else (where the kernel library's matrix-core attention
takes the sizes, c is kept a second time transposed, as value pages); a layer may read another layer's pages
(``RunEntry.cache_from``) with W_uk, W_uv and queries of its own.

The up-projections never touch the cached rows: since q[:dim] . (W_uk c) = (W_uk^T q[:dim]) . c and
sum_j p_j W_uv c_j = W_uv sum_j p_j c_j, the queries are taken into the latent's space once per
token ([W_uk^T q[:dim] | turned q[dim:]], float32), the attention runs over the page rows as they
are, with one shared "key" of kv_rank + rot_dim elements and the latent itself as the value, and
W_uv is applied to the kv_rank-wide result of each head.

params: prefix, hidden_size, num_heads, head_dim, rot_dim, value_dim, kv_rank, q_rank, scale,
latent_eps (of the two latent norms), gate (tensor name below the prefix or None), position (a
PartSpec whose ``rotation()`` covers exactly rot_dim elements; None with rot_dim 0: no rotated part,
the page row is the latent alone and positions enter through the causal mask only), gate_per
("head": the gate's tensor has a row per head; "element": one per head and value element, and the
concatenated heads are multiplied element by element), sink (tensor name below the prefix or None:
a learned number per head whose exponential joins the softmax's denominator, a score that has no
key and no value and is not scaled), names (optional overrides).
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..config.specs import PartSpec
from ..engine.batch import attention_tiles
from ..weights.loader import TensorSpec
from .base import POSITIONS, KVNeed, Mixer, Runtime, register_mixer


def _pad_rows(parts, multiple: int):
    rows = sum(p.shape[0] for p in parts)
    pad = -rows % multiple
    if pad:
        parts = list(parts) + [torch.zeros((pad, parts[0].shape[1]), dtype=parts[0].dtype, device=parts[0].device)]
    return torch.cat(list(parts), dim=0).contiguous()


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.n_heads = int(params["num_heads"])
        self.head_dim = int(params["head_dim"])
        self.rot_dim = int(params["rot_dim"])
        self.value_dim = int(params["value_dim"])
        self.kv_rank = int(params["kv_rank"])
        self.q_rank = int(params["q_rank"])
        self.scale = float(params["scale"])
        self.eps = float(params["latent_eps"])
        self.gate_name = params.get("gate")
        self.projects_kv = bool(params.get("projects_kv", True))
        self.sink_name = params.get("sink")
        self.gate_per = params.get("gate_per", "head")
        if self.gate_per not in ("head", "element"):
            raise ValueError(f"{self.prefix}: gate_per is 'head' or 'element', got {self.gate_per!r}")
        self.gate_elems = self.value_dim if self.gate_per == "element" else 1
        pos: PartSpec = params.get("position")
        self.position = None if pos is None else POSITIONS.get(pos.kind)(pos.params, rt)
        self.rotation = None if self.position is None else self.position.rotation()
        if (self.rot_dim or self.position is not None) and (self.rotation is None or self.rotation.rotary_dim != self.rot_dim):
            raise ValueError(f"{self.prefix}: the position encoding must rotate exactly the rot_dim={self.rot_dim} elements of the rotated part")
        names = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o"}
        names.update(params.get("names", {}))
        self.names = {k: f"{self.prefix}.{v}" for k, v in names.items()}
        self.w_down = self.w_qn = self.w_kvn = self.w_uq = self.w_uk = self.w_uv_t = self.w_o = self.w_uk_t = self.w_uv = None
        self.sink = None
        # columns of the stacked down-projection: [dq | dkv (where the layer keeps a cache) | gates], each
        # section starting at a multiple of 8
        up8 = lambda n: n + (-n % 8)
        self.kv_col = up8(self.q_rank)
        self.gate_col = self.kv_col + (up8(self.kv_rank + self.rot_dim) if self.projects_kv else 0)
        self.down_rows = self.gate_col + (self.n_heads * self.gate_elems if self.gate_name else 0)
        self.down_rows += -self.down_rows % 16
        # where the kernel library has its matrix-core attention for these sizes the latent is kept a second
        # time, transposed, in value pages (that form's second product reads a column's slots side by side)
        self.on_matrix_cores = bool(rt.ops.latent_attention_on_matrix_cores(rt.act_dtype, self.kv_rank, self.rot_dim, rt.page_size))
        # consecutive tokens of a request that one tile of the attention takes
        self.tile_tokens = int(rt.ops.latent_tile_tokens(self.n_heads, self.on_matrix_cores))

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, H = self.names, self.n_heads
        specs = {
            n["dq"]: TensorSpec((self.q_rank, self.hidden)), n["dq_norm"]: TensorSpec((self.q_rank,), "float", ("one_plus_normal", 0.1)),
            n["uq"]: TensorSpec((H * (self.head_dim + self.rot_dim), self.q_rank)),
            n["uk"]: TensorSpec((H * self.head_dim, self.kv_rank)), n["uv"]: TensorSpec((H * self.value_dim, self.kv_rank)),
            n["o"]: TensorSpec((self.hidden, H * self.value_dim)),
        }
        if self.projects_kv:
            specs[n["dkv"]] = TensorSpec((self.kv_rank + self.rot_dim, self.hidden))
            specs[n["dkv_norm"]] = TensorSpec((self.kv_rank,), "float", ("one_plus_normal", 0.1))
        if self.gate_name:
            specs[f"{self.prefix}.{self.gate_name}"] = TensorSpec((H * self.gate_elems, self.hidden))
        if self.sink_name:
            specs[f"{self.prefix}.{self.sink_name}"] = TensorSpec((H,), "float", ("normal", 1.0))
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n, H = self.names, self.n_heads
        dq = tensors[n["dq"]]
        zeros = lambda rows: torch.zeros((rows, self.hidden), dtype=dq.dtype, device=dq.device)
        parts = [dq, zeros(self.kv_col - self.q_rank)]
        if self.projects_kv:
            parts += [tensors[n["dkv"]], zeros(self.gate_col - self.kv_col - self.kv_rank - self.rot_dim)]
            self.w_kvn = tensors[n["dkv_norm"]].contiguous()
        if self.gate_name:
            parts.append(tensors[f"{self.prefix}.{self.gate_name}"])
        parts.append(zeros(self.down_rows - sum(p.shape[0] for p in parts)))
        self.w_down = torch.cat([p for p in parts if p.shape[0]], dim=0).contiguous()
        self.w_qn = tensors[n["dq_norm"]].contiguous()
        if self.sink_name:
            self.sink = tensors[f"{self.prefix}.{self.sink_name}"].float().contiguous()
        self.w_uq = tensors[n["uq"]]
        # per head [in][out]: W_uk as it is stored ([head][dim][kv_rank]: out = kv_rank), W_uv transposed
        # ([head][kv_rank][value_dim])
        self.w_uk = tensors[n["uk"]].view(H, self.head_dim, self.kv_rank).contiguous()
        self.w_uv_t = tensors[n["uv"]].view(H, self.value_dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_o = tensors[n["o"]]
        # the same weights [head][out][in] where the kernel library's matrix-core products want them
        transposed = getattr(self.rt.ops, "head_weights_transposed", None)
        self.w_uk_t = transposed(self.w_uk) if transposed is not None else None
        self.w_uv = transposed(self.w_uv_t) if transposed is not None else None

    def kv_need(self) -> KVNeed:
        # one row of kv_rank + rot_dim elements per token and no values: the row serves as both
        return KVNeed(1, self.kv_rank + self.rot_dim, None, self.kv_rank if self.on_matrix_cores else 0)

    def products(self):
        H = self.n_heads
        return ((self.down_rows, self.hidden), (H * (self.head_dim + self.rot_dim), self.q_rank), (self.hidden, H * self.value_dim))

    def step_inputs(self):
        n = self.tile_tokens
        # (the tiles with the most keys first: their workgroups start first, the short ones fill the end)
        return {f"latent_tiles_{n}": lambda hb: attention_tiles(hb, n, longest_first=True)}

    def forward(self, h: torch.Tensor, ctx, site) -> torch.Tensor:
        ops, act = self.rt.ops, self.rt.act_dtype
        if site.owns_cache != self.projects_kv:
            raise RuntimeError(f"{self.prefix}: a layer whose run entries both own and borrow caches is not offered")
        proj = ops.linear(h, self.w_down, act)
        pages, values = site.kv()
        c_q = ops.latent_prepare(
            proj, self.q_rank, self.w_qn, self.eps, act, kv_col=self.kv_col, kv_rank=self.kv_rank if site.owns_cache else 0,
            rot_dim=self.rot_dim, kv_norm=self.w_kvn, rotation=self.rotation, positions=ctx.arrays["positions"], pages=pages,
            slots=ctx.arrays[f"slots_g{site.group}"], page_size=self.rt.page_size, values=values,
        )
        q = ops.linear(c_q, self.w_uq, act)
        # queries in the latent's space: [W_uk^T q[:dim] | q[dim:] turned by the position], float32
        q_lat = ops.head_linear(q, self.w_uk, self.n_heads, self.head_dim, self.kv_rank, torch.float32, tail=self.rot_dim,
                                rotation=self.rotation, positions=ctx.arrays["positions"], w_t=self.w_uk_t)
        o_lat = ops.latent_attention(q_lat, pages, self.n_heads, self.kv_rank, self.rot_dim, self.scale, ctx, site.group,
                                     self.rt.page_size, tiles=ctx.arrays[f"latent_tiles_{self.tile_tokens}"], values=values,
                                     sink=self.sink)
        o = ops.head_linear(o_lat, self.w_uv_t, self.n_heads, self.kv_rank, self.value_dim, act,
                            gate=proj if self.gate_name else None, gate_col=self.gate_col, w_t=self.w_uv, gate_elems=self.gate_elems)
        return ops.linear(o, self.w_o, act, partial_ok=True)
