"""Linear attention with a constant decay per head ("lightning attention").

q = silu(W_q x) and k = silu(W_k x) ([heads, dim]), v = silu(W_v x) ([heads, vdim]).  Per head, a state S [dim, vdim] that
starts at zero and is carried from token to token of a sequence:

    S <- decay_h S + k v^T;   o = S^T q                      (no other scale)

The read-outs of all heads of a token are RMS-normed together with one weight vector [heads * vdim] (``eps``), multiplied
by sigmoid(W_g x) and go through the output product.  ``decay`` is a number per head, a constant of the model.

The sequence's state is one row of float32 per slot (``StateNeed``): S as [heads, dim, vdim].  Activations of the
projections, the recurrence, the norm and the gate are float32 on both libraries; the two products are the activation
type's, the first one leaving its result in float32.  Four launches a decode step: the product of all
projections (q | k | v | gate: one matrix), ``lightning_scan`` (the recurrence over each sequence's run of tokens, from
and into the state of its slot, which the kernel finds through the slots on the device, so that a captured decode step
replays for other slots), ``lightning_out`` (norm, weight, gate), the output product.  A step with a run of
``chunked_from`` tokens or more takes ``lightning_chunked`` in the scan's place: the same sums over chunks of 64 tokens on
the matrix cores in float32, every chunk's products side by side and only the states between chunks in order.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import ParamSpec, Part, StateNeed, register_part


@register_part("mixer", "lightning")
class LightningAttention(Part):
    graph_safe = True       # what changes from step to step is read from the batch's device arrays only
    chunked_from = 32       # a step whose longest run has this many tokens takes the chunked form

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay, eps: float):
        decay = [float(d) for d in decay]
        if len(decay) != num_heads:
            raise ValueError(f"{len(decay)} decays for {num_heads} heads")
        if not all(0.0 <= d <= 1.0 for d in decay):
            raise ValueError("a decay lies between 0 and 1")
        if not 1 <= head_dim <= 256:
            raise ValueError(f"a key width of {head_dim} is beyond the 256 that the recurrence's kernel takes")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.decay_values, self.eps = decay, eps
        for name in self.param_specs():
            setattr(self, name, None)
        self.in_weight = self.decay = None     # made by prepare()

    def param_specs(self):
        H, D, V, W = self.num_heads, self.head_dim, self.value_dim, self.hidden_size
        return {"q_weight": ParamSpec((H * D, W)), "k_weight": ParamSpec((H * D, W)), "v_weight": ParamSpec((H * V, W)),
                "g_weight": ParamSpec((H * V, W)), "out_norm": ParamSpec((H * V,), role="scale"),
                "out_weight": ParamSpec((W, H * V))}

    def cache_need(self):
        return None

    def state_need(self) -> StateNeed:
        return StateNeed((self.num_heads * self.head_dim * self.value_dim,), torch.float32)

    def prepare(self, device, act):
        if self.in_weight is not None:
            return
        self.in_weight = torch.cat([self.q_weight, self.k_weight, self.v_weight, self.g_weight]).contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=device)
        self.q_weight = self.k_weight = self.v_weight = self.g_weight = None

    def forward(self, normed, ctx, entry):
        H, D, V = self.num_heads, self.head_dim, self.value_dim
        proj = ops.gemm(normed, self.in_weight, ctx.act)                            # float32 [T, q | k | v | gate]
        runs = ctx.batch.runs()
        if not runs["decode"] and runs["max_new"] >= self.chunked_from and not ctx.capturing:
            o = ops.lightning_chunked(proj, self.decay, runs, ctx.state(entry), H, D, V, ctx.act)
        else:
            o = ops.lightning_scan(proj, self.decay, runs, ctx.state(entry), H, D, V, ctx.act)
        out = ops.lightning_out(o, proj[:, 2 * H * D + H * V:], self.out_norm, self.eps, ctx.act)
        return ops.gemm(out, self.out_weight, ctx.act, partial_sums=True)
