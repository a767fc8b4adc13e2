"""Arrangement of a layer's parts around the residual stream.

Pre-norm with two residual sums, ``x += mixer(norm(x)); x += ffn(norm(x))``
(/root/reference/src/engine/tq_transformer.c:2494,2531,2685-2701).  The sums are not done here: a part's
output travels as ``pending`` to the next norm, which adds it into the stream in float32 in the same
pass that normalises.
"""
from __future__ import annotations

import torch

from .base import Part, register_part


@register_part("block", "prenorm")
class PreNormBlock(Part):
    graph_safe = True
    # the parts a layer of this arrangement is made of, and the registry each comes from
    slots = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "ffn"}

    def __init__(self, mixer_norm, mixer, ffn_norm, ffn):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need()

    def native(self):
        from ..csrc import host_api
        norm1, mixer, norm2, ffn = (p.native() for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn))
        if not (isinstance(norm1, host_api.NormDesc) and isinstance(mixer, host_api.AttentionDesc)
                and isinstance(norm2, host_api.NormDesc) and isinstance(ffn, (host_api.DenseFfnDesc, host_api.MoeFfnDesc))):
            return None
        layer = host_api.LayerDesc()
        layer.mixer_norm, layer.attention, layer.ffn_norm = norm1, mixer, norm2
        if isinstance(ffn, host_api.DenseFfnDesc):
            layer.ffn_kind, layer.dense = host_api.FFN_DENSE, ffn
        else:
            layer.ffn_kind, layer.moe = host_api.FFN_MOE, ffn
        return layer

    def forward(self, x, pending, ctx, entry):
        normed, _ = self.mixer_norm.forward(x, pending, ctx)
        pending = self.mixer.forward(normed, ctx, entry)
        want32 = getattr(self.ffn, "wants_f32", False)
        normed, normed32 = self.ffn_norm.forward(x, pending, ctx, want_f32=want32)
        return self.ffn.forward(normed, normed32, ctx)


@register_part("block", "sandwich")
class SandwichBlock(Part):
    """A norm before and a norm after every part: ``x += norm_b(mixer(norm_a(x))); x += norm_d(ffn(norm_c(x)))``, the
    feed-forward half optional (``ffn``, ``ffn_norm`` and ``ffn_post_norm`` None: the layer is its mixer alone).  A
    part's output travels to the next norm wrapped with the weights of the norm it has to pass first
    (``ops.NormedDelta``), and that norm's kernel norms it, adds it into the stream and norms the stream in one pass."""
    graph_safe = True
    slots = {"mixer_norm": "norm", "mixer": "mixer", "mixer_post_norm": "norm", "ffn_norm": "norm", "ffn": "ffn",
             "ffn_post_norm": "norm"}
    optional = ("ffn_norm", "ffn", "ffn_post_norm")

    def __init__(self, mixer_norm, mixer, mixer_post_norm, ffn_norm=None, ffn=None, ffn_post_norm=None):
        if len({ffn_norm is None, ffn is None, ffn_post_norm is None}) != 1:
            raise ValueError("a layer has a feed-forward with both its norms, or none of the three")
        self.mixer_norm, self.mixer, self.mixer_post_norm = mixer_norm, mixer, mixer_post_norm
        self.ffn_norm, self.ffn, self.ffn_post_norm = ffn_norm, ffn, ffn_post_norm

    def children(self):
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "mixer_post_norm": self.mixer_post_norm,
                 "ffn_norm": self.ffn_norm, "ffn": self.ffn, "ffn_post_norm": self.ffn_post_norm}
        return {k: v for k, v in parts.items() if v is not None}

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need()

    def forward(self, x, pending, ctx, entry):
        from ..csrc import ops
        normed, _ = self.mixer_norm.forward(x, pending, ctx)
        pending = ops.NormedDelta(self.mixer.forward(normed, ctx, entry), self.mixer_post_norm.weight, self.mixer_post_norm.eps)
        if self.ffn is None:
            return pending
        want32 = getattr(self.ffn, "wants_f32", False)
        normed, normed32 = self.ffn_norm.forward(x, pending, ctx, want_f32=want32)
        return ops.NormedDelta(self.ffn.forward(normed, normed32, ctx), self.ffn_post_norm.weight, self.ffn_post_norm.eps)


@register_part("block", "outnorm")
class OutputNormBlock(Part):
    """A norm on every part's output only: ``x += norm_a(mixer(x)); x += norm_b(ffn(x))``.  The parts read the residual
    stream itself, un-normed, in the activation type; the feed-forward half is optional (``ffn`` and ``ffn_norm`` None: the
    layer is its mixer alone).  A part's output travels on wrapped with the weights of its norm (``ops.NormedDelta``), and
    the kernel that sums it into the stream norms it in the same pass and hands the summed stream to the next part.
    ``mixer_shift`` (optional, a part of the "shift" registry): the mixer reads the stream blended token by token with the
    row before (``parts/shift.py``) instead of the stream itself; the feed-forward still reads the stream.  What the shift
    keeps per sequence is the layer's state, so it goes with mixers that keep none of their own.  A feed-forward that wants
    its input in float32 as well (a router) is given the stream itself."""
    graph_safe = True
    slots = {"mixer": "mixer", "mixer_norm": "norm", "ffn": "ffn", "ffn_norm": "norm", "mixer_shift": "shift"}
    optional = ("ffn", "ffn_norm", "mixer_shift")

    def __init__(self, mixer, mixer_norm, ffn=None, ffn_norm=None, mixer_shift=None):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a layer has a feed-forward with its norm, or neither")
        if mixer_shift is not None and mixer.state_need() is not None:
            raise ValueError("a shifted input goes with a mixer that keeps no state of its own per sequence")
        self.mixer, self.mixer_norm, self.ffn, self.ffn_norm, self.mixer_shift = mixer, mixer_norm, ffn, ffn_norm, mixer_shift

    def children(self):
        parts = {"mixer": self.mixer, "mixer_norm": self.mixer_norm, "ffn": self.ffn, "ffn_norm": self.ffn_norm,
                 "mixer_shift": self.mixer_shift}
        return {k: v for k, v in parts.items() if v is not None}

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need() if self.mixer_shift is None else self.mixer_shift.state_need()

    def forward(self, x, pending, ctx, entry):
        from ..csrc import ops
        if pending is not None and not isinstance(pending, ops.NormedDelta):     # a layer of another arrangement before this one
            ops.add_rmsnorm(x, pending, self.mixer_norm.weight, self.mixer_norm.eps, ctx.act, want_act=False)
            pending = None
        if self.mixer_shift is None:
            h, _ = ops.add_rmsnorm(x, pending, None, 0.0, ctx.act, stream=True)
        else:       # the sum alone, then the blend with the row before from the float32 stream; one launch where that can be
            behind = self.mixer_shift.behind_sum(ctx, entry) if pending is not None and pending.weight.dtype == torch.float32 else None
            if behind is not None:
                h, _ = ops.add_rmsnorm(x, pending, None, 0.0, ctx.act, stream=True, shift=behind)
            else:
                if pending is not None:
                    ops.add_rmsnorm(x, pending, None, 0.0, ctx.act)
                h = self.mixer_shift.forward(x, ctx, entry)
        pending = ops.NormedDelta(self.mixer.forward(h, ctx, entry), self.mixer_norm.weight, self.mixer_norm.eps)
        if self.ffn is None:
            return pending
        h, _ = ops.add_rmsnorm(x, pending, None, 0.0, ctx.act, stream=True)
        # (a feed-forward that reads float32 rows reads the stream; what it hands on may name those rows, and the kernel
        # that sums it into the stream reads a row whole before it writes that row)
        return ops.NormedDelta(self.ffn.forward(h, x if getattr(self.ffn, "wants_f32", False) else None, ctx),
                               self.ffn_norm.weight, self.ffn_norm.eps)
