"""RMS normalisation (reference: yalis/external/model.py:957-989).

out = x * rsqrt(mean(x^2) + eps) * weight, all in float32 with one rounding at
the end; ``unit_offset`` multiplies by (1 + weight) instead (a flag of the same
class in the reference, :984).  The kernel fuses the residual sum that precedes
every norm of a pre-norm block: the float32 residual stream is updated in place
and normalised in one pass.  ``norm_add`` is the other way round, for blocks that norm a
branch's output instead of its input: residual += norm(branch), again one pass.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..weights.loader import TensorSpec
from .base import ExpertRows, Norm, NormedBranch, PlusRow, Runtime, Settled, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """params: name (checkpoint tensor), size, eps, unit_offset."""

    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.name = params["name"]
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.unit_offset = bool(params.get("unit_offset", False))
        self.weight: Optional[torch.Tensor] = None
        self.takes_embedded_rows = hasattr(rt.ops, "embedded_rows")

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        # (random weights: around the value that leaves a row as it is, 0 where 1 is added)
        return {self.name: TensorSpec((self.size,), "float", ("normal", 0.1) if self.unit_offset else ("one_plus_normal", 0.1))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name]

    def norm(self, x):
        return self.rt.ops.rmsnorm(x, self.weight, self.eps, self.unit_offset, self.rt.act_dtype)

    def add_norm(self, residual, delta):
        row = None
        if isinstance(delta, PlusRow):  # a vector for every token joins the stream in the same pass
            delta, row = delta.inner, delta.row
        if isinstance(delta, NormedBranch):
            delta = delta.settle(residual)
        if isinstance(delta, Settled):
            delta = None
        if row is not None:
            return self.rt.ops.add_rmsnorm(residual, delta, self.weight, self.eps, self.unit_offset, self.rt.act_dtype, row=row)
        return self.rt.ops.add_rmsnorm(
            residual, delta, self.weight, self.eps, self.unit_offset, self.rt.act_dtype
        )

    def norm_add(self, residual, branch, expert_rows=None, expert_weight=1.0, scale=1.0):
        if scale != 1.0:
            raise ValueError("this norm adds its branch unscaled")
        if isinstance(branch, ExpertRows) and branch.row_weights is not None:
            branch = branch.combine()  # (rows with weights of their own are summed first)
        if isinstance(branch, ExpertRows):
            branch, expert_rows, expert_weight = branch.dense, branch.rows, branch.weight
        return self.rt.ops.norm_add(residual, branch, self.weight, self.eps, self.unit_offset, self.rt.act_dtype,
                                    expert_rows=expert_rows, expert_weight=expert_weight)

    def gather_add_norm(self, residual, delta, rows):
        if isinstance(delta, PlusRow):
            delta = delta.settle(residual)
        if isinstance(delta, NormedBranch):
            delta = delta.settle(residual)
        if isinstance(delta, Settled):
            delta = None
        return self.rt.ops.gather_add_rmsnorm(
            residual, delta, rows, self.weight, self.eps, self.unit_offset, self.rt.act_dtype
        )


@register_norm("layernorm")
class LayerNorm(Norm):
    """(x - mean) / sqrt(variance + eps) * weight + bias over a row, the variance the mean of the
    squared deviations; float32 arithmetic, one rounding at the end.

    params: name (weight tensor), bias (bias tensor's name, or None: no bias), size, eps, center
    (True; False: no mean is taken off, which makes it an RMS norm with an optional bias).

    One kernel (``ops.sandwich_norm``) serves every place a block may put it: a pending
    contribution, plain or itself normed and scaled (``NormedBranch``), is added into the float32
    residual and the new residual normed in the same pass."""

    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.name = params["name"]
        self.bias_name = params.get("bias")
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.center = bool(params.get("center", True))
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {self.name: TensorSpec((self.size,), "float", ("one_plus_normal", 0.1))}
        if self.bias_name:
            specs[self.bias_name] = TensorSpec((self.size,), "float", ("normal", 0.1))
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name].contiguous()
        self.bias = tensors[self.bias_name].contiguous() if self.bias_name else None
        if self.bias is not None and self.bias.dtype != self.weight.dtype:
            self.weight, self.bias = self.weight.float(), self.bias.float()

    def constants(self):
        """What the kernel library needs of a norm: (weight, bias or None, eps, center)."""
        return (self.weight, self.bias, self.eps, self.center)

    def _pending(self, residual, delta):
        """(branch, its norm's constants or None, scale) of a pending contribution."""
        if isinstance(delta, PlusRow):
            delta = delta.settle(residual)
        if isinstance(delta, Settled) or delta is None:
            return None, None, 1.0
        if isinstance(delta, NormedBranch):
            if not isinstance(delta.norm, LayerNorm):
                delta.settle(residual)
                return None, None, 1.0
            return delta.branch, delta.norm.constants(), delta.scale
        return delta, None, 1.0

    def norm(self, x):
        return self.rt.ops.sandwich_norm(None, x, None, 1.0, self.constants(), None, self.rt.act_dtype)

    def add_norm(self, residual, delta):
        branch, post, scale = self._pending(residual, delta)
        return self.rt.ops.sandwich_norm(residual, branch, post, scale, self.constants(), None, self.rt.act_dtype)

    def gather_add_norm(self, residual, delta, rows):
        branch, post, scale = self._pending(residual, delta)
        return self.rt.ops.sandwich_norm(residual, branch, post, scale, self.constants(), rows, self.rt.act_dtype)

    def norm_add(self, residual, branch, expert_rows=None, expert_weight=1.0, scale=1.0):
        if isinstance(branch, ExpertRows):
            branch = branch.combine()
        elif expert_rows is not None:
            raise ValueError("this norm takes its branch combined")
        self.rt.ops.sandwich_norm(residual, branch, self.constants(), scale, None, None, self.rt.act_dtype)
        return self.rt.ops.round_rows(residual, self.rt.act_dtype)
