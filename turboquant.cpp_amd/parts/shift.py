"""Token shift: what a mixer reads is every token blended with the token before it.

``h_t = x_t + (x_(t-1) - x_t) * weight`` element by element, ``x_(t-1)`` being the row of the sequence's token before as it
was before any blending, zeros for a sequence's first token.  Between steps a sequence keeps the last row it brought: one
float32 row of state per slot (``StateNeed``), which the kernel finds through the step's slots on the device, so that a
captured decode step replays for other slots.  The blend is taken in float32 from the float32 stream; the result is in the
activation type, as a mixer reads it.  In a step of one token per sequence the blend rides in the launch that sums the
part before into the stream (``behind_sum``); elsewhere it is a launch of its own.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import ParamSpec, Part, StateNeed, register_part


@register_part("shift", "token_shift")
class TokenShift(Part):
    graph_safe = True

    def __init__(self, size: int):
        self.size = size
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), role="scale")}

    def state_need(self) -> StateNeed:
        return StateNeed((self.size,), torch.float32)

    def prepare(self, device, act):
        self.weight = self.weight.float().contiguous()      # it enters float arithmetic only

    def forward(self, x, ctx, entry):
        return ops.token_shift(x, self.weight, ctx.state(entry), ctx.batch.runs(), ctx.act)

    def behind_sum(self, ctx, entry):
        """What ``ops.add_rmsnorm(shift=)`` takes to blend in the launch that sums a part into the stream, or None where
        the step is not one token per sequence (then a row's blend needs the summed row before it, which another
        workgroup of that launch writes)."""
        b = ctx.batch
        return (self.weight, ctx.state(entry), b.slots_dev) if b.is_decode else None
