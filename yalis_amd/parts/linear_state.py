"""Mixers that keep a matrix per head as their memory: S [dim, value_dim], float32, one per request
and head in the request's state slot, zero before the first token.  Every token decays S, writes an
outer product k u^T into it and reads q out of it:

    S <- diag(a) S  (a one decay for the head, or one per key channel)
    u  = v                          plain write           ("gated_linear_attention")
    u  = beta (v - S^T k)           the delta rule        ("delta_rule")
    S <- S + k u^T,   o = S^T q     (the read-out sees the token's own write)

and each head's o is divided by its root mean square, multiplied by a weight shared by the heads and
by silu of a projection of the mixer's input, and projected back.  Decays, write strengths, unit
norms, S and the read-out norm are float32 in both engines; one kernel (``ops.linear_state_scan``)
walks every request's span with S in registers, one column of S to a group of lanes.

"delta_rule" (Yang et al., "Gated Delta Networks: Improving Mamba2 with Delta Rule"): q and k (``num_kv_heads`` heads of ``head_dim``, shared
by groups of value heads) and v pass a causal convolution per channel (``conv_taps``, silu), q and
k are made unit vectors (q also times head_dim^-1/2); beta = sigmoid(W_b h) and the head's decay
exp(-exp(A_log) softplus(W_a h + dt_bias)).  The convolution's last inputs are a second state.

"gated_linear_attention" (Yang et al., "Gated Linear Attention Transformers with Hardware-Efficient Training"): q times head_dim^-1/2, decay per key
channel sigmoid(z)^(1/tau) with z = W_a2 (W_a1 h) + b.

"state_space_duality" (Dao and Gu, "Transformers are SSMs: Generalized Models and Efficient Algorithms Through Structured State Space
Duality"): the same memory read as a selective state space.  One projection gives [z | x | B | C | dt]; x, B and C
pass a causal convolution per channel with a bias and silu; the step dt = softplus(dt + dt_bias) makes the head's
decay exp(-exp(A_log) dt) and the strength of its write, S <- a S + dt B x^T (k = B, u = dt x), the read-out is
S^T C + D x (q = C, a skip per head); B and C are shared by groups of heads.  The read-out is gated first, by
silu(z), and then normed in ``norm_groups`` equal parts, each by its own root mean square, with a weight as wide as
the read-out.
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..weights.loader import TensorSpec
from .base import Mixer, Runtime, StateNeed, register_mixer
from .latent_attention import _pad_rows


class _MatrixStateMixer(Mixer):
    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.n_heads = int(params["num_heads"])
        self.n_kv = int(params.get("num_kv_heads", self.n_heads))
        self.head_dim = int(params["head_dim"])
        self.value_dim = int(params["value_dim"])
        self.out_eps = float(params["out_norm_eps"])
        self.q_scale = float(params.get("q_scale", self.head_dim ** -0.5))
        if self.n_heads % self.n_kv:
            raise ValueError(f"{self.prefix}: num_heads={self.n_heads} is not a multiple of num_kv_heads={self.n_kv}")
        self.qk_cols = 2 * self.n_kv * self.head_dim
        self.v_cols = self.n_heads * self.value_dim
        self.w_in = self.w_norm = self.w_o = None

    def _name(self, short: str) -> str:
        return f"{self.prefix}.{self.params.get('names', {}).get(short, short)}"

    def _common_specs(self) -> Dict[str, TensorSpec]:
        kd = self.n_kv * self.head_dim
        return {
            self._name("q"): TensorSpec((kd, self.hidden)), self._name("k"): TensorSpec((kd, self.hidden)),
            self._name("v"): TensorSpec((self.v_cols, self.hidden)), self._name("g"): TensorSpec((self.v_cols, self.hidden)),
            self._name("o"): TensorSpec((self.hidden, self.v_cols)),
            self._name("norm"): TensorSpec((self.value_dim,), "float", ("one_plus_normal", 0.1)),
        }

    def _state(self) -> StateNeed:
        return StateNeed((self.n_heads, self.head_dim, self.value_dim), torch.float32, 0.0)

    def _finish(self, o, proj, gate_col):
        ops = self.rt.ops
        y = ops.gated_head_norm(o, self.w_norm, self.out_eps, proj, gate_col, self.n_heads, self.value_dim, self.rt.act_dtype)
        return ops.linear(y, self.w_o, self.rt.act_dtype, partial_ok=True)


@register_mixer("delta_rule")
class DeltaRule(_MatrixStateMixer):
    """params: prefix, hidden_size, num_heads, num_kv_heads, head_dim, value_dim, conv_taps, unit_eps
    (under the root of the unit norms), out_norm_eps, q_scale (head_dim^-1/2), names."""

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.taps = int(params["conv_taps"])
        self.unit_eps = float(params.get("unit_eps", 1e-6))
        self.conv_cols = self.qk_cols + self.v_cols
        self.gate_col = self.conv_cols + (-self.conv_cols % 8)
        self.w_conv = self.w_ba = self.a_log = self.dt_bias = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = self._common_specs()
        kd, H = self.n_kv * self.head_dim, self.n_heads
        conv = ("normal", 0.4)
        specs.update({
            self._name("q.conv"): TensorSpec((kd, self.taps), "float", conv), self._name("k.conv"): TensorSpec((kd, self.taps), "float", conv),
            self._name("v.conv"): TensorSpec((self.v_cols, self.taps), "float", conv),
            self._name("b"): TensorSpec((H, self.hidden)), self._name("a"): TensorSpec((H, self.hidden)),
            self._name("A_log"): TensorSpec((H,), "float", ("normal", 0.5)), self._name("dt_bias"): TensorSpec((H,), "float", ("normal", 0.5)),
        })
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        t = lambda short: tensors[self._name(short)]
        q = t("q")
        pad = torch.zeros((self.gate_col - self.conv_cols, self.hidden), dtype=q.dtype, device=q.device)
        self.w_in = _pad_rows([p for p in (q, t("k"), t("v"), pad, t("g")) if p.shape[0]], 16)
        self.w_ba = _pad_rows([t("b"), t("a")], 16)
        self.w_conv = torch.cat([t("q.conv"), t("k.conv"), t("v.conv")], dim=0).contiguous()
        self.a_log, self.dt_bias = t("A_log").float().contiguous(), t("dt_bias").float().contiguous()
        self.w_norm, self.w_o = t("norm").contiguous(), t("o")

    def state_need(self):
        needs = [self._state()]
        if self.taps > 1:
            needs.append(StateNeed((self.taps - 1, self.conv_cols), self.rt.act_dtype, 0.0))
        return tuple(needs)

    def products(self):
        rows = self.gate_col + self.v_cols
        return ((rows + (-rows % 16), self.hidden), (2 * self.n_heads + (-2 * self.n_heads % 16), self.hidden), (self.hidden, self.v_cols))

    def forward(self, h: torch.Tensor, ctx, site) -> torch.Tensor:
        ops, act = self.rt.ops, self.rt.act_dtype
        proj = ops.linear(h, self.w_in, act)
        ba = ops.linear(h, self.w_ba, torch.float32)  # [beta's logit | the decay's] per head, float32
        x = proj[:, : self.conv_cols]
        conv_state = site.state(1) if self.taps > 1 else None
        u = ops.causal_conv(x, self.w_conv, None, conv_state, ctx, act="silu")
        if conv_state is not None:
            ops.conv_state_push(x, conv_state, ctx)
        o = ops.linear_state_scan(
            u, self.n_heads, self.n_kv, self.head_dim, self.value_dim, site.state(0), ctx, q_scale=self.q_scale,
            unit_eps=self.unit_eps, decay=("head", ba, self.n_heads, self.a_log, self.dt_bias), beta=(ba, 0),
        )
        return self._finish(o, proj, self.gate_col)


@register_mixer("gated_linear_attention")
class GatedLinearAttention(_MatrixStateMixer):
    """params: prefix, hidden_size, num_heads, head_dim, value_dim, tau, out_norm_eps, q_scale, names.
    The low rank of the decay's projections is read from the tensors' shapes."""

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.tau = float(params["tau"])
        self.low_rank = params.get("low_rank")  # None: whatever the checkpoint's a1 has
        self.qkv_cols = self.qk_cols + self.v_cols
        self.gate_col = self.qkv_cols + (-self.qkv_cols % 8)
        self.a1_col = self.gate_col + self.v_cols + (-self.v_cols % 8)
        self.w_a2 = self.b_a2 = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = self._common_specs()
        low = int(self.low_rank or 16)
        specs.update({
            self._name("a1"): TensorSpec((low, self.hidden), free_axes=() if self.low_rank else (0,)),
            self._name("a2"): TensorSpec((self.n_heads * self.head_dim, low), free_axes=() if self.low_rank else (1,)),
            self._name("a2.b"): TensorSpec((self.n_heads * self.head_dim,), "float", ("normal", 1.0)),
        })
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        t = lambda short: tensors[self._name(short)]
        q, a1 = t("q"), t("a1")
        zeros = lambda rows: torch.zeros((rows, self.hidden), dtype=q.dtype, device=q.device)
        parts = [q, t("k"), t("v"), zeros(self.gate_col - self.qkv_cols), t("g"), zeros(self.a1_col - self.gate_col - self.v_cols), a1]
        self.low = int(a1.shape[0])
        if t("a2").shape[1] != self.low:
            raise ValueError(f"{self.prefix}: the decay's two projections disagree on their rank")
        self.w_in = _pad_rows([p for p in parts if p.shape[0]], 16)
        self.w_a2, self.b_a2 = t("a2").contiguous(), t("a2.b").float().contiguous()
        self.w_norm, self.w_o = t("norm").contiguous(), t("o")

    def state_need(self):
        return self._state()

    def products(self):
        low = int(getattr(self, "low", self.low_rank or 16))
        rows = self.a1_col + low
        return ((rows + (-rows % 16), self.hidden), (self.n_heads * self.head_dim, low), (self.hidden, self.v_cols))

    def forward(self, h: torch.Tensor, ctx, site) -> torch.Tensor:
        ops, act = self.rt.ops, self.rt.act_dtype
        proj = ops.linear(h, self.w_in, act)
        z = ops.linear(proj[:, self.a1_col: self.a1_col + self.low], self.w_a2, torch.float32)  # the decays' logits, float32
        o = ops.linear_state_scan(
            proj, self.n_heads, self.n_heads, self.head_dim, self.value_dim, site.state(0), ctx, q_scale=self.q_scale,
            unit_eps=None, decay=("channel", z, 0, self.b_a2, self.tau), beta=None,
        )
        return self._finish(o, proj, self.gate_col)


@register_mixer("state_space_duality")
class StateSpaceDuality(Mixer):
    """params: prefix, hidden_size, num_heads, value_dim (a head's channels), state_dim (rows of S), groups (of heads
    that share B and C), conv_taps, norm_groups, out_norm_eps, names (optional overrides: in, conv, conv_bias, dt_bias,
    A_log, D, norm, o)."""

    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.n_heads = int(params["num_heads"])
        self.value_dim = int(params["value_dim"])
        self.state_dim = int(params["state_dim"])
        self.groups = int(params["groups"])
        self.taps = int(params["conv_taps"])
        self.norm_groups = int(params["norm_groups"])
        self.out_eps = float(params["out_norm_eps"])
        self.inner = self.n_heads * self.value_dim
        if self.n_heads % self.groups:
            raise ValueError(f"{self.prefix}: num_heads={self.n_heads} is not a multiple of groups={self.groups}")
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.prefix}: {self.inner} channels do not divide into norm_groups={self.norm_groups} equal parts")
        self.bc_cols = self.groups * self.state_dim
        self.conv_cols = self.inner + 2 * self.bc_cols  # [x | B | C]
        self.main_rows = 2 * self.inner + 2 * self.bc_cols  # [z | x | B | C]; dt follows in the checkpoint's matrix
        self.w_main = self.w_dt = self.w_conv = self.b_conv = self.dt_bias = self.a_log = self.skip = self.w_norm = self.w_o = None

    def _name(self, short: str) -> str:
        default = {"conv_bias": "conv.b"}.get(short, short)
        return f"{self.prefix}.{self.params.get('names', {}).get(short, default)}"

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        H = self.n_heads
        return {
            self._name("in"): TensorSpec((self.main_rows + H, self.hidden)),
            self._name("conv"): TensorSpec((self.conv_cols, self.taps), "float", ("normal", 0.4)),
            self._name("conv_bias"): TensorSpec((self.conv_cols,), "float", ("normal", 0.1)),
            self._name("dt_bias"): TensorSpec((H,), "float", ("normal", 0.5)), self._name("A_log"): TensorSpec((H,), "float", ("normal", 0.5)),
            self._name("D"): TensorSpec((H,), "float", ("one_plus_normal", 0.1)),
            self._name("norm"): TensorSpec((self.inner,), "float", ("one_plus_normal", 0.1)),
            self._name("o"): TensorSpec((self.hidden, self.inner)),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        t = lambda short: tensors[self._name(short)]
        w_in = t("in")
        self.w_main = _pad_rows([w_in[: self.main_rows]], 16)
        self.w_dt = _pad_rows([w_in[self.main_rows:]], 16)
        self.w_conv, self.b_conv = t("conv").contiguous(), t("conv_bias").contiguous()
        if self.b_conv.dtype != self.w_conv.dtype:
            self.w_conv, self.b_conv = self.w_conv.float(), self.b_conv.float()
        self.dt_bias, self.a_log, self.skip = (t(n).float().contiguous() for n in ("dt_bias", "A_log", "D"))
        self.w_norm, self.w_o = t("norm").contiguous(), t("o")

    def state_need(self):
        needs = [StateNeed((self.n_heads, self.state_dim, self.value_dim), torch.float32, 0.0)]
        if self.taps > 1:
            needs.append(StateNeed((self.taps - 1, self.conv_cols), self.rt.act_dtype, 0.0))
        return tuple(needs)

    def products(self):
        up16 = lambda n: n + (-n % 16)
        return ((up16(self.main_rows), self.hidden), (up16(self.n_heads), self.hidden), (self.hidden, self.inner))

    def forward(self, h: torch.Tensor, ctx, site) -> torch.Tensor:
        ops, act = self.rt.ops, self.rt.act_dtype
        proj = ops.linear(h, self.w_main, act)
        dt = ops.linear(h, self.w_dt, torch.float32)  # the steps' logits per head, float32
        xbc = proj[:, self.inner: self.inner + self.conv_cols]
        conv_state = site.state(1) if self.taps > 1 else None
        u = ops.causal_conv(xbc, self.w_conv, self.b_conv, conv_state, ctx, act="silu")
        if conv_state is not None:
            ops.conv_state_push(xbc, conv_state, ctx)
        o = ops.linear_state_scan(
            u, self.n_heads, self.groups, self.state_dim, self.value_dim, site.state(0), ctx, q_scale=1.0, unit_eps=None,
            decay=("head", dt, 0, self.a_log, self.dt_bias), beta="step",
            columns=(self.inner + self.bc_cols, self.inner, 0), skip=self.skip,
        )
        y = ops.gated_head_norm(o, self.w_norm, self.out_eps, proj, 0, self.norm_groups, self.inner // self.norm_groups, act,
                                gate_first=True)
        return ops.linear(y, self.w_o, act, partial_ok=True)
