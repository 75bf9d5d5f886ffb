"""Block arrangements: how norms, mixer and feed-forward sit around the residual.

"prenorm" is the reference's sequential pre-norm block
(yalis/external/model.py:414-439 with parallel_residual=False and identity
post-norms): x = x + mixer(norm_1(x)); x = x + feed_forward(norm_2(x)); a layer may leave the
feed-forward and its norm out.

The residual stream is float32.  A block receives the residual and the previous
block's not-yet-added contribution ``delta``; each norm kernel adds the pending
contribution and normalises in one pass, so no separate addition runs.  The block
returns its own last contribution, to be added by whoever comes next.
"""
from __future__ import annotations

from .base import Block, ExpertRows, NormedBranch, PlusRow, Settled, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    roles = {
        "mixer_norm": ("norm", True),
        "mixer": ("mixer", True),
        "feed_forward_norm": ("norm", False),
        "feed_forward": ("feed_forward", False),
    }

    def __init__(self, mixer_norm, mixer, feed_forward_norm=None, feed_forward=None):
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a prenorm block has a feed-forward and its norm, or neither")
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.feed_forward_norm = feed_forward_norm
        self.feed_forward = feed_forward

    @property
    def takes_embedded_rows(self):
        return bool(getattr(self.mixer_norm, "takes_embedded_rows", False))

    def forward(self, residual, delta, ctx, site):
        h = self.mixer_norm.add_norm(residual, delta)
        a = self.mixer.forward(h, ctx, site)
        if self.feed_forward is None:  # a layer that is its mixer alone: the mixer's output waits for the next norm
            return a
        h = self.feed_forward_norm.add_norm(residual, a)
        return self.feed_forward.forward(h, ctx)


@register_block("parallel")
class ParallelBlock(Block):
    """One norm that both branches read: h = norm(x); x = x + (mixer(h) + feed_forward(h)).  A layer may leave
    the feed-forward out.  The two outputs are summed in float32 by one kernel (``ops.moe_combine``: the mixer's
    output, possibly still a product's unreduced slices, plus a mixture's uncombined rows times their weights) and
    handed on as one pending contribution."""

    roles = {
        "norm": ("norm", True),
        "mixer": ("mixer", True),
        "feed_forward": ("feed_forward", False),
    }

    def __init__(self, norm, mixer, feed_forward=None):
        self.norm = norm
        self.mixer = mixer
        self.feed_forward = feed_forward

    @property
    def takes_embedded_rows(self):
        return bool(getattr(self.norm, "takes_embedded_rows", False))

    def forward(self, residual, delta, ctx, site):
        h = self.norm.add_norm(residual, delta)
        if self.feed_forward is None:
            return self.mixer.forward(h, ctx, site)
        # the feed-forward first: what it hands on is settled in tensors of its own before the mixer runs, and the
        # mixer's output (possibly a product's unreduced slices in the library's workspace) is consumed right after
        f = self.feed_forward.forward(h, ctx)
        ops = self.mixer.rt.ops
        if not isinstance(f, ExpertRows):  # any other feed-forward: its output is one row a token
            f = ExpertRows(None, f.float().contiguous(), 1, 1.0)
        dense = None if f.dense is None else f.dense.float().contiguous()
        a = self.mixer.forward(h, ctx, site)
        if dense is not None:
            a = ops.moe_combine(a, dense, 1, 1.0)
        return ops.moe_combine(a, f.rows, f.top, f.weight, row_weights=f.row_weights)


@register_block("branch_norm")
class BranchNormBlock(Block):
    """Norms on the branches' outputs only: x = x + norm_1(mixer(x)); x = x + norm_2(feed_forward(x)).
    The branches read the stream itself.  A layer may leave the feed-forward (and its norm) out.

    Every addition happens inside the block (a pending contribution would have to wait for a norm
    that is not there), so what it hands on is ``Settled``: the stream in the activation dtype,
    which the norm's kernel writes beside the float32 residual in the same pass, and which the next
    block of this kind reads instead of rounding the residual again."""

    roles = {
        "mixer": ("mixer", True),
        "mixer_norm": ("norm", True),
        "feed_forward": ("feed_forward", False),
        "feed_forward_norm": ("norm", False),
    }

    def __init__(self, mixer, mixer_norm, feed_forward=None, feed_forward_norm=None):
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a branch_norm block has a feed-forward and its norm, or neither")
        self.mixer = mixer
        self.mixer_norm = mixer_norm
        self.feed_forward = feed_forward
        self.feed_forward_norm = feed_forward_norm

    def forward(self, residual, delta, ctx, site):
        if isinstance(delta, PlusRow):
            delta = delta.settle(residual)
        if isinstance(delta, Settled):
            h = delta.activations
        else:
            if delta is not None:  # a block of another kind left a contribution: it is added as it is
                residual += delta.float()
            h = self.mixer.rt.ops.round_rows(residual, self.mixer.rt.act_dtype)
        h = self.mixer_norm.norm_add(residual, self.mixer.forward(h, ctx, site))
        if self.feed_forward is not None:
            h = self.feed_forward_norm.norm_add(residual, self.feed_forward.forward(h, ctx))
        return Settled(h)


@register_block("sandwich")
class SandwichBlock(Block):
    """Norms before and after every branch, and a multiplier on what the branches add:
    x = x + s * post_1(mixer(pre_1(x))); x = x + s * post_2(feed_forward(pre_2(x))).
    A layer may leave the feed-forward (and its two norms) out.  ``branch_scale`` is s.

    Between two branches the stream is touched once: the norm that reads it next adds the pending
    branch (through that branch's own norm, scaled) and norms the sum in the same pass.  The last
    branch is handed on the same way (``NormedBranch``) to whatever norms the stream next."""

    roles = {
        "mixer_norm": ("norm", True),
        "mixer": ("mixer", True),
        "mixer_out_norm": ("norm", True),
        "feed_forward_norm": ("norm", False),
        "feed_forward": ("feed_forward", False),
        "feed_forward_out_norm": ("norm", False),
    }

    def __init__(self, mixer_norm, mixer, mixer_out_norm, feed_forward_norm=None, feed_forward=None, feed_forward_out_norm=None,
                 branch_scale: float = 1.0):
        if len({feed_forward is None, feed_forward_norm is None, feed_forward_out_norm is None}) != 1:
            raise ValueError("a sandwich block has a feed-forward with both of its norms, or none of the three")
        self.mixer_norm, self.mixer, self.mixer_out_norm = mixer_norm, mixer, mixer_out_norm
        self.feed_forward_norm, self.feed_forward, self.feed_forward_out_norm = feed_forward_norm, feed_forward, feed_forward_out_norm
        self.branch_scale = float(branch_scale)

    def forward(self, residual, delta, ctx, site):
        h = self.mixer_norm.add_norm(residual, delta)
        pending = NormedBranch(self.mixer.forward(h, ctx, site), self.mixer_out_norm, self.branch_scale)
        if self.feed_forward is None:
            return pending
        h = self.feed_forward_norm.add_norm(residual, pending)
        return NormedBranch(self.feed_forward.forward(h, ctx), self.feed_forward_out_norm, self.branch_scale)
