"""Attention over one compressed row per position, with or without a rotated part of the keys.

Every position keeps a latent c = rmsnorm(W_dkv x) of ``kv_rank`` numbers, and nothing else.  Head h has matrices of its
own that would expand it, k_h = W_uk,h c and v_h = W_uv,h c; the score of query position i and key position j <= i is
(q_h,i . k_h,j) * scale, the softmax is the ordinary one, the concatenated heads are multiplied element by element by
sigmoid(W_g x) and go through the output product.

In the folded form the keys and values are never expanded.  Since q . (W_uk c) = (W_uk^T q) . c, each head's key matrix is folded into its
query (one product per head, ``ops.head_gemm``), and since sum_j p_j W_uv c_j = W_uv sum_j p_j c_j, each head's value
matrix is applied to its weighted sum of latents afterwards (a second product per head, whose epilogue applies the output
gate).  In between runs the library's attention over the paged cache as for any mixer with one key/value head shared by
all query heads, of width ``kv_rank`` rounded up to a multiple of 16 (the added columns are zeros in the folded queries
and in the cache): the cache holds the latent as a key row and, transposed, as a value row, the layouts that the
attention kernels' operands take.  Decoded tokens and portions of prompts that go on from earlier tokens take this form:
it reads ``kv_rank`` numbers per position whatever the number of heads.

A step whose sequences all start at their first token takes the other, expanded form, since per pair of positions the folded form
costs heads x 2 ``kv_rank`` multiply-adds and the expanded one heads x (dim + vdim): one product expands the step's
latents into every head's keys and values, which are laid into pages that live for the step only
(``StepBatch.own_pages``), and the library's attention runs over them with as many key/value heads as heads; the output
gate is applied to its result.  The latents go into the cache all the same, for the steps that follow.  Both forms are
the same function of the same rounded latents; they differ in the rounding of what comes after.

Options: ``q_rank`` (the queries go through a latent of their own: c_q = rmsnorm(W_dq x), q = W_uq c_q); ``rot_dim`` with
a ``position`` part (a head's query is [dim plain | rot_dim rotated]; W_dkv has ``rot_dim`` more rows, which are not normed
and are one rotated key part for all heads; score = (q_plain . W_uk c + q_rot . k_rot) * scale; the cached row is
[k_rot rotated | c], the rotated part first so that the rotation's kernel finds it at a head's start, and the matrices
that fold and expand carry an identity block that passes it through); ``gate_activation`` None (no output gate);
``window`` n (position i sees j only if 0 <= i - j < n; the cache keeps the window only).

``shares_latent``: the mixer has no W_dkv; its schedule entry reads the cache of an earlier entry (another layer's
latents, written earlier in the same step) with its own W_uk, W_uv, queries, gate and output product.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from ..config.plan import PartSpec
from .base import CacheNeed, ParamSpec, Part, build_part, register_part
from .rope import NoRotation


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, kv_rank: int, scale: float,
                 eps: float, shares_latent: bool = False, gate_activation: str | None = "sigmoid", q_rank: int | None = None,
                 rot_dim: int = 0, position=None, window: int | None = None):
        if window is not None and window < 1:
            raise ValueError(f"window must be positive, got {window}")
        self.window = window
        if min(num_heads, head_dim, value_dim, kv_rank) < 1:
            raise ValueError("heads, widths and the latent's size must be positive")
        if rot_dim < 0 or rot_dim % 2 or (rot_dim > 0) != (position is not None):
            raise ValueError("a rotated key part has an even width and a position part, or there is neither")
        if kv_rank + rot_dim > 512:
            raise ValueError(f"a cached row of {kv_rank + rot_dim} numbers is beyond the 512 that the attention kernels take as a head")
        if max(head_dim + rot_dim, value_dim) > 512:
            raise ValueError(f"heads of {max(head_dim + rot_dim, value_dim)} are beyond the 512 that the attention kernels take")
        if gate_activation is not None and gate_activation not in ops.GATES:
            raise ValueError(f"unknown activation {gate_activation!r}; known: {', '.join(sorted(ops.GATES))}")
        if q_rank is not None and q_rank < 1:
            raise ValueError("q_rank must be positive")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.kv_rank, self.scale, self.eps, self.shares_latent = kv_rank, float(scale), eps, shares_latent
        self.gate_activation, self.q_rank, self.rot_dim = gate_activation, q_rank, rot_dim
        self.position = (build_part("position", position) if isinstance(position, PartSpec) else position) or NoRotation()
        if rot_dim and self.position.rotary_dim != rot_dim:
            raise ValueError(f"the position part turns {self.position.rotary_dim} numbers, the rotated key part has {rot_dim}")
        self.width = -(-(kv_rank + rot_dim) // 16) * 16          # the cached row's width, in the cache and in the attention kernels
        # the width at which a head's queries, gates and outputs are laid out: the expanded form's attention has keys and
        # values of one width, a multiple of 16; the added rows and columns of the matrices are zeros
        self.head_width = -(-max(head_dim + rot_dim, value_dim) // 16) * 16
        self.q_rank_width = None if q_rank is None else -(-q_rank // 8) * 8
        for name in self.param_specs():
            setattr(self, name, None)
        self.in_weight = self.fold_weight = self.expand_weight = self.kv_weight = self.uq_weight_laid = None      # made by prepare()

    def children(self):
        return {"position": self.position}

    def param_specs(self):
        H, K, V, R, W, Rr = self.num_heads, self.head_dim, self.value_dim, self.kv_rank, self.hidden_size, self.rot_dim
        specs = {"uk_weight": ParamSpec((H * K, R)), "uv_weight": ParamSpec((H * V, R)), "out_weight": ParamSpec((W, H * V))}
        if self.q_rank is None:
            specs["q_weight"] = ParamSpec((H * (K + Rr), W))
        else:
            specs.update({"dq_weight": ParamSpec((self.q_rank, W)), "dq_norm": ParamSpec((self.q_rank,), role="scale"),
                          "uq_weight": ParamSpec((H * (K + Rr), self.q_rank))})
        if self.gate_activation is not None:
            specs["g_weight"] = ParamSpec((H * V, W))
        if not self.shares_latent:
            specs.update({"dkv_weight": ParamSpec((R + Rr, W)), "dkv_norm": ParamSpec((R,), role="scale")})
        return specs

    def cache_need(self) -> CacheNeed:
        return CacheNeed(1, self.width, self.window)

    def state_need(self):
        return None

    def prepare(self, device, act):
        if self.in_weight is not None:
            return
        H, K, V, R, Rp, D, Rr = self.num_heads, self.head_dim, self.value_dim, self.kv_rank, self.width, self.head_width, self.rot_dim

        def heads_padded(t, n):          # [H * n, ...] -> [H * D, ...], rows n .. D - 1 of every head zeros
            if n == D:
                return t
            out = t.new_zeros((H, D) + tuple(t.shape[1:]))
            out[:, :n] = t.view(H, n, *t.shape[1:])
            return out.view(H * D, *t.shape[1:])

        def rotated_first(t):            # a head's rows [K plain | Rr rotated] -> [Rr rotated | K plain], then padded to D
            if Rr == 0:
                return heads_padded(t, K)
            t = t.view(H, K + Rr, *t.shape[1:])
            return heads_padded(torch.cat([t[:, K:], t[:, :K]], dim=1).reshape(H * (K + Rr), *t.shape[2:]), K + Rr)

        first = []
        if self.q_rank is None:
            first.append(rotated_first(self.q_weight))
        else:
            first.append(self.dq_weight)
            # the second product of the queries, its k filled with zeros up to a multiple of 8
            uq = rotated_first(self.uq_weight)
            laid = uq.new_zeros((uq.shape[0], self.q_rank_width))
            laid[:, :self.q_rank] = uq
            self.uq_weight_laid = laid.contiguous()
        if not self.shares_latent:
            first.append(self.dkv_weight)
        if self.gate_activation is not None:
            first.append(heads_padded(self.g_weight, V))
        self.in_weight = torch.cat(first).contiguous()          # q (or its latent) | (latent, rotated key part) | gate
        # W_uk,h^T [R, K] per head behind an identity for the rotated part; rows and columns beyond them zeros
        fold = self.uk_weight.new_zeros((H, Rp, D))
        fold[:, Rr:Rr + R, Rr:Rr + K] = self.uk_weight.view(H, K, R).transpose(1, 2)
        # W_uv,h [V, R] per head, read from the cached row's columns behind the rotated part
        expand = self.uv_weight.new_zeros((H, D, Rp))
        expand[:, :V, Rr:Rr + R] = self.uv_weight.view(H, V, R)
        # every head's keys, then every head's values, from a cached row: [2 H D, Rp]
        kv = self.uk_weight.new_zeros((2, H, D, Rp))
        kv[0, :, Rr:Rr + K, Rr:Rr + R] = self.uk_weight.view(H, K, R)
        kv[1, :, :V, Rr:Rr + R] = self.uv_weight.view(H, V, R)
        for i in range(Rr):
            fold[:, i, i] = 1.0
            kv[0, :, i, i] = 1.0
        self.fold_weight, self.expand_weight = fold.contiguous(), expand.contiguous()
        self.kv_weight = kv.view(2 * H * D, Rp).contiguous()
        if V != D:
            out = self.out_weight.new_zeros((self.hidden_size, H, D))
            out[:, :, :V] = self.out_weight.view(self.hidden_size, H, V)
            self.out_weight = out.view(self.hidden_size, H * D).contiguous()
        for name in ("q_weight", "dq_weight", "uq_weight", "dkv_weight", "g_weight", "uk_weight", "uv_weight"):
            setattr(self, name, None)

    def _queries(self, proj, ctx):
        """The heads' queries, float32 [T, H * D], each head [rotated part | plain part | zeros], not yet rotated; and the
        column of ``proj`` behind what made them."""
        H, D = self.num_heads, self.head_width
        if self.q_rank is None:
            return proj[:, :H * D], H * D
        cq = ops.lead_norm(proj[:, :self.q_rank], self.q_rank, self.dq_norm, self.eps, 1, self.q_rank_width, ctx.act, out_act=True)
        return ops.gemm(cq, self.uq_weight_laid, ctx.act), self.q_rank

    def _latent_rows(self, down, copies, ctx, out=None):
        """``copies`` times [rotated key part as projected | normed latent | zeros] from the down projection's columns."""
        if self.rot_dim == 0:
            if out is None:
                out = torch.empty((down.shape[0], copies * self.width), dtype=torch.float32, device=down.device)
            ops.latent_norm(down, self.dkv_norm, self.eps, out, copies, self.width, ctx.act)
            return out
        return ops.lead_norm(down, self.kv_rank, self.dkv_norm, self.eps, copies, self.width, ctx.act, out=out)

    def forward(self, normed, ctx, entry):
        b, kv = ctx.batch, ctx.kv(entry)
        H, R, Rp, D, Rr = self.num_heads, self.kv_rank, self.width, self.head_width, self.rot_dim
        T = normed.shape[0]
        proj = ops.gemm(normed, self.in_weight, ctx.act)                    # float32 [T, q | (latent) | gate]
        q, at = self._queries(proj, ctx)
        down = None if self.shares_latent else proj[:, at:at + R + Rr]
        gate = proj[:, proj.shape[1] - H * D:] if self.gate_activation is not None else None
        if kv.owns != (not self.shares_latent):
            raise ValueError("a latent attention keeps a cache of its own exactly if it has a latent of its own")
        pos = self.position
        angles = (pos.table(ctx.device), pos.pairing_code, pos.rotary_dim)
        amp = getattr(pos, "amplitude", 1.0)
        if not b.is_decode and b.is_fresh and not ctx.capturing:
            return self._expanded(q, down, gate, ctx, kv, angles, amp)
        if kv.owns:
            # folded queries, then the cached row twice (the key row and the value row), as the cache write reads them
            rows = torch.empty((T, (H + 2) * Rp), dtype=torch.float32, device=normed.device)
            ops.head_gemm(q, self.fold_weight, ctx.act, out=rows[:, :H * Rp])
            self._latent_rows(down, 2, ctx, out=rows[:, H * Rp:])
            folded = ops.rope_kv_write(rows, b.positions, b.slot_of_token, kv.table, *angles,
                                       kv.k_pages, kv.v_pages, kv.layer_offset, kv.page_size, kv.page_stride, H, 1, Rp,
                                       ctx.act, runs=b.runs(), amplitude=amp)
        elif Rr == 0:
            folded = ops.head_gemm(q, self.fold_weight, ctx.act, out_act=True)
        else:
            folded = ops.rope_kv_write(ops.head_gemm(q, self.fold_weight, ctx.act), b.positions, b.slot_of_token, kv.table,
                                       *angles, None, None, kv.layer_offset, kv.page_size, kv.page_stride, H, 0, Rp, ctx.act,
                                       runs=b.runs(), amplitude=amp)
        mixed = ops.attention(folded, kv.k_pages, kv.v_pages, kv.layer_offset, b.positions, b.slot_of_token, kv.table,
                              kv.page_size, kv.page_stride, H, 1, Rp, self.window, self.scale, ctx.act, runs=b.runs())
        out = ops.head_gemm(mixed, self.expand_weight, ctx.act, out_act=True, gate=gate,
                            **({} if gate is None else {"activation": self.gate_activation}))
        return ops.gemm(out, self.out_weight, ctx.act, partial_sums=True)

    def _expanded(self, q, down, gate, ctx, kv, angles, amp):
        """A step of whole prompts: every head's keys and values from the step's cached rows, in pages of the step's own."""
        b = ctx.batch
        H, R, Rp, D, Rr = self.num_heads, self.kv_rank, self.width, self.head_width, self.rot_dim
        T = q.shape[0]
        runs = b.runs()
        no_angles = (_NO_ROTATION.table(ctx.device), 0, 0)
        shared = ("latents", kv.k_pages.data_ptr(), kv.layer_offset)     # the same for every entry that reads this cache
        if kv.owns and Rr == 0:
            rows = self._latent_rows(down, 2, ctx)
            ops.rope_kv_write(rows, b.positions, b.slot_of_token, kv.table, *no_angles, kv.k_pages, kv.v_pages,
                              kv.layer_offset, kv.page_size, kv.page_stride, 0, 1, Rp, ctx.act, runs=runs)
            latents = b.scratch[shared] = ops.act_rows(rows[:, :Rp], None, None, ctx.act)       # as the cache holds them
        elif kv.owns:
            # the row a third time, as a query head: what comes back is the row as the cache holds it, rotated part turned
            rows = self._latent_rows(down, 3, ctx)
            latents = b.scratch[shared] = ops.rope_kv_write(rows, b.positions, b.slot_of_token, kv.table, *angles, kv.k_pages,
                                                            kv.v_pages, kv.layer_offset, kv.page_size, kv.page_stride, 1, 1,
                                                            Rp, ctx.act, runs=runs, amplitude=amp)
        else:
            latents = b.scratch[shared]
        table, n_pages = b.own_pages(kv.page_size)
        stride = H * kv.page_size * D
        # (cleared: a page's places behind a sequence's last token are multiplied by weights of zero, and must be numbers)
        pages = torch.zeros((2, n_pages, stride), dtype=latents.dtype, device=q.device)
        ops.rope_kv_write(ops.gemm(latents, self.kv_weight, ctx.act), b.positions, b.slot_of_token, table, *no_angles,
                          pages[0], pages[1], 0, kv.page_size, stride, 0, H, D, ctx.act, runs=runs)
        if Rr == 0:
            queries = ops.act_rows(q, None, None, ctx.act)
        else:
            queries = ops.rope_kv_write(q, b.positions, b.slot_of_token, table, *angles, None, None, 0, kv.page_size, stride,
                                        H, 0, D, ctx.act, runs=runs, amplitude=amp)
        mixed = ops.attention(queries, pages[0], pages[1], 0, b.positions, b.slot_of_token, table,
                              kv.page_size, stride, H, H, D, self.window, self.scale, ctx.act, runs=runs,
                              value_width=-(-self.value_dim // 16) * 16)
        if gate is not None:
            ops.gate_rows(mixed, gate, self.gate_activation, ctx.act)
        return ops.gemm(mixed, self.out_weight, ctx.act, partial_sums=True)


_NO_ROTATION = NoRotation()
