"""Grouped-query attention over the paged cache.

In the reference's order (/root/reference/src/engine/tq_transformer.c:934-2269, Qwen2 path):
q, k, v = W x (+ bias) (:1031-1093); rotation of q and k (:1342-1344); k and v written at the token's
position (:1363-1371, :1451-1455); per head, scores of the positions in reach scaled by 1/sqrt(head_dim),
softmax, weighted sum of values (:1908-1976); output projection (:2239-2240).  Query head h reads
kv head h / (heads / kv_heads) (:1675-1679).  With a window a token reaches the last ``window``
positions, itself included (:1646-1654).  With ``qk_norm_eps`` set, every head of q and of k is RMS-normed with
weights of its own between the product and the rotation (:1111-1124), which this architecture does not use.

Options for other designs, all off by default: ``position`` of kind "none" (no rotation: positions enter elsewhere);
``score_cap`` c (a scaled score s becomes c tanh(s / c)); ``distance_bias`` (two numbers per head, r1 and r2:
r1 ln(1 + r2 (i - j)) is taken off the score of query position i and key position j); ``chunk`` n (position i sees
j <= i only if i // n == j // n, chunks counted from position 0 of the sequence); ``value_dim`` (values of another width
than keys); ``separate_qkv`` (q, k, v and their biases are parameters of their own, joined when the part is prepared);
``sink`` (a learned number per head whose exponential joins the softmax's denominator: a score with no key and no value,
neither scaled nor capped, counted once).
``rotated_norm_eps`` (behind the rotation every query and key head is divided by its root mean square over the head, no
weights: the cache holds the keys so normed); ``head_gate`` (a matrix [heads, hidden]: head h's output is multiplied by
the sigmoid of row h's product with the layer's input, before the output product); ``shares_kv`` (the mixer has no key and
value matrices: its schedule entry reads the cache of an earlier entry, with queries, window and everything else of its
own); ``cache_window`` (what the cache keeps where that is more than the mixer's own window, because a later layer that
reads this cache looks further back; None: everything).  A position part may scale its sines and cosines (``amplitude``).
``value_norm_eps`` (every value head is divided by its root mean square over its width, no weights: the cache holds the
values so normed); ``value_mix`` ("source": the layer leaves its values, as it caches them, for later layers of the same
step; "mix": its values become (1 - mix) v + mix v_source, ``mix`` a learned number, before they are cached; both kinds
carry the parameter, which a source does not use); ``sigmoid_bias`` (no softmax: the weight of a visible key is
sigmoid(score + b_h), b a learned number per head, and the weights are not normalised over the keys); ``keep_first`` n
(with a window: the sequence's first n positions stay visible to every later token and stay in the cache).
With ``separate_qkv`` the heads are laid out at a kernel width that is the larger of key and value width rounded up to
16: the added rows and columns of the matrices are zeros, which change no score and no output, and every head size
then runs on the matrix-core kernels of both libraries.
"""
from __future__ import annotations

import math

import torch

from ..config.plan import PartSpec
from ..csrc import ops
from .base import CacheNeed, ParamSpec, Part, build_part, register_part


@register_part("mixer", "gqa_attention")
class GroupedQueryAttention(Part):
    graph_safe = True
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, position,
                 qkv_bias: bool = False, out_bias: bool = False, window: int | None = None,
                 scale: float | None = None, qk_norm_eps: float | None = None, score_cap: float | None = None,
                 distance_bias: bool = False, chunk: int | None = None, value_dim: int | None = None,
                 separate_qkv: bool = False, sink: bool = False, rotated_norm_eps: float | None = None,
                 head_gate: bool = False, shares_kv: bool = False, cache_window: int | None | str = "own",
                 value_norm_eps: float | None = None, value_mix: str | None = None, sigmoid_bias: bool = False,
                 keep_first: int = 0):
        if value_mix not in (None, "source", "mix"):
            raise ValueError(f"value_mix is None, 'source' or 'mix', got {value_mix!r}")
        if (value_norm_eps is not None or value_mix is not None or sigmoid_bias or keep_first) and not separate_qkv:
            raise ValueError("normed or mixed values, sigmoid weights and kept first positions need separate_qkv")
        if value_norm_eps is not None and not value_norm_eps > 0:
            raise ValueError(f"value_norm_eps must be positive, got {value_norm_eps}")
        if value_mix is not None and shares_kv:
            raise ValueError("a layer that reads another layer's values has none of its own to mix")
        if sigmoid_bias and sink:
            raise ValueError("sigmoid weights have no denominator for a sink to join")
        if keep_first < 0:
            raise ValueError(f"keep_first counts positions, got {keep_first}")
        self.value_norm_eps, self.value_mix, self.has_sigmoid_bias = value_norm_eps, value_mix, sigmoid_bias
        self.keep_first = int(keep_first) if window is not None else 0      # without a window everything stays visible anyway
        self.mix = self.score_bias = None
        if (head_gate or shares_kv) and not separate_qkv:
            raise ValueError("a gate per head and a cache shared with another layer need separate_qkv")
        if rotated_norm_eps is not None and not rotated_norm_eps > 0:
            raise ValueError(f"rotated_norm_eps must be positive, got {rotated_norm_eps}")
        if cache_window != "own" and cache_window is not None and (window is None or cache_window < window):
            raise ValueError(f"the cache must keep at least the mixer's own window {window}, got {cache_window}")
        self.rotated_norm_eps, self.has_head_gate, self.shares_kv = rotated_norm_eps, head_gate, shares_kv
        self.cache_window = window if cache_window == "own" else cache_window
        self.gate_weight = None
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if window is not None and window < 1:
            raise ValueError(f"window must be positive, got {window}")
        if chunk is not None and chunk < 1:
            raise ValueError(f"chunk must be positive, got {chunk}")
        if score_cap is not None and not score_cap > 0:
            raise ValueError(f"score_cap must be positive, got {score_cap}")
        if value_dim not in (None, head_dim) and not separate_qkv:
            raise ValueError("values of another width than keys need separate_qkv")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.score_cap, self.has_distance_bias, self.chunk, self.separate_qkv = score_cap, distance_bias, chunk, separate_qkv
        # what the checkpoint's heads measure (key width, value width); head_dim becomes the kernels' width
        self.key_dim, self.value_dim = head_dim, head_dim if value_dim is None else value_dim
        if separate_qkv:
            self.head_dim = -(-max(self.key_dim, self.value_dim) // 16) * 16
        self.r1 = self.r2 = None
        self.has_sink, self.sink = sink, None
        self.q_weight = self.k_weight = self.v_weight = self.q_bias = self.k_bias = self.v_bias = None
        self.has_qkv_bias, self.has_out_bias, self.window = qkv_bias, out_bias, window
        self.qk_norm_eps = qk_norm_eps
        self.q_norm = self.k_norm = None
        self.scale = scale if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position = build_part("position", position) if isinstance(position, PartSpec) else position
        self.qkv_weight = self.qkv_bias = self.out_weight = self.out_bias = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def param_specs(self):
        if self.separate_qkv:
            H, G, K, V, W = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim, self.hidden_size
            specs = {"q_weight": ParamSpec((H * K, W)), "out_weight": ParamSpec((W, H * V))}
            if not self.shares_kv:
                specs.update({"k_weight": ParamSpec((G * K, W)), "v_weight": ParamSpec((G * V, W))})
            if self.has_head_gate:
                specs["gate_weight"] = ParamSpec((H, W))
            if self.has_qkv_bias:
                specs["q_bias"] = ParamSpec((H * K,), role="bias")
                if not self.shares_kv:
                    specs.update({"k_bias": ParamSpec((G * K,), role="bias"), "v_bias": ParamSpec((G * V,), role="bias")})
            if self.has_out_bias:
                specs["out_bias"] = ParamSpec((W,), role="bias")
            if self.has_distance_bias:
                specs.update({"r1": ParamSpec((H,), role="scale"), "r2": ParamSpec((H,), role="scale")})
            if self.qk_norm_eps is not None:
                specs.update({"q_norm": ParamSpec((K,), role="scale"), "k_norm": ParamSpec((K,), role="scale")})
            if self.has_sink:
                specs["sink"] = ParamSpec((H,), role="scale")
            if self.has_sigmoid_bias:
                specs["score_bias"] = ParamSpec((H,), role="scale")
            if self.value_mix is not None:
                specs["mix"] = ParamSpec((), role="scale")
            return specs
        rows = self.q_size + 2 * self.kv_size
        splits = (self.q_size, self.kv_size, self.kv_size)
        specs = {
            "qkv_weight": ParamSpec((rows, self.hidden_size), splits=splits),
            "out_weight": ParamSpec((self.hidden_size, self.q_size)),
        }
        if self.has_qkv_bias:
            specs["qkv_bias"] = ParamSpec((rows,), role="bias", splits=splits)
        if self.has_out_bias:
            specs["out_bias"] = ParamSpec((self.hidden_size,), role="bias")
        if self.qk_norm_eps is not None:
            specs["q_norm"] = ParamSpec((self.head_dim,), role="scale")
            specs["k_norm"] = ParamSpec((self.head_dim,), role="scale")
        if self.has_distance_bias:
            specs.update({"r1": ParamSpec((self.num_heads,), role="scale"), "r2": ParamSpec((self.num_heads,), role="scale")})
        if self.has_sink:
            specs["sink"] = ParamSpec((self.num_heads,), role="scale")
        return specs

    def prepare(self, device, act):
        if self.has_distance_bias:      # they enter float arithmetic only
            self.r1, self.r2 = self.r1.float().contiguous(), self.r2.float().contiguous()
        if self.has_sink:
            self.sink = self.sink.float().contiguous()
        if self.has_sigmoid_bias:
            self.score_bias = self.score_bias.float().contiguous()
        if self.value_mix is not None:
            self.mix = self.mix.reshape(1).contiguous()
        if not self.separate_qkv or self.qkv_weight is not None:
            return
        D = self.head_dim

        def heads_padded(t, heads, width):
            """[heads * width, ...] -> [heads * D, ...], zeros behind each head's rows."""
            out = t.new_zeros((heads, D, *t.shape[1:]))
            out[:, :width] = t.view(heads, width, *t.shape[1:])
            return out.view(heads * D, *t.shape[1:])

        H, G, K, V = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        if self.qk_norm_eps is not None and K != D:     # zeros behind the head's own values: they norm zeros to zeros
            self.q_norm, self.k_norm = (torch.cat([w, w.new_zeros(D - K)]) for w in (self.q_norm, self.k_norm))
        rows = [heads_padded(self.q_weight, H, K)]
        if not self.shares_kv:
            rows += [heads_padded(self.k_weight, G, K), heads_padded(self.v_weight, G, V)]
        if self.has_head_gate:      # the gate's rows ride in the same product, filled up to a multiple of four rows
            fill = -H % 4
            rows += [self.gate_weight, self.gate_weight.new_zeros((fill, self.hidden_size))]
        self.qkv_weight = torch.cat(rows).contiguous()
        if self.has_qkv_bias:
            bias = [heads_padded(self.q_bias, H, K)]
            if not self.shares_kv:
                bias += [heads_padded(self.k_bias, G, K), heads_padded(self.v_bias, G, V)]
            if self.has_head_gate:
                bias.append(bias[0].new_zeros((H + -H % 4,)))
            self.qkv_bias = torch.cat(bias).contiguous()
        self.gate_weight = None
        if V != D:
            out = self.out_weight.new_zeros((self.hidden_size, H, D))
            out[:, :, :V] = self.out_weight.view(self.hidden_size, H, V)
            self.out_weight = out.view(self.hidden_size, H * D).contiguous()
        self.q_weight = self.k_weight = self.v_weight = self.q_bias = self.k_bias = self.v_bias = None

    def children(self):
        return {"position": self.position}

    def cache_need(self) -> CacheNeed:
        return CacheNeed(self.num_kv_heads, self.head_dim, self.cache_window, chunk=self.chunk,
                         keep_first=self.keep_first if self.cache_window is not None else 0)

    def state_need(self):
        return None

    def native(self):
        from ..csrc import host_api
        if self.qk_norm_eps is not None:        # the executor has no form with a norm of the heads
            return None
        if self.score_cap is not None or self.has_distance_bias or self.chunk is not None or self.separate_qkv or self.has_sink:
            return None                         # nor one with changed scores or chunks
        if self.rotated_norm_eps is not None or getattr(self.position, "amplitude", 1.0) != 1.0:
            return None
        table = self.position.table(self.qkv_weight.device)
        if table.dtype != torch.float32 or not table.is_contiguous() or table.numel() * 2 != self.position.rotary_dim:
            return None
        return host_api.AttentionDesc(self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.window or 0,
                                      self.position.pairing_code, self.position.rotary_dim, self.scale,
                                      host_api.weight(self.qkv_weight), host_api.weight(self.qkv_bias),
                                      host_api.weight(self.out_weight), host_api.weight(self.out_bias), table.data_ptr())

    def _score_options(self) -> dict:
        """What the attention kernels are told beyond the plain formula; nothing for a mixer that leaves it all off."""
        opts = {}
        if self.score_cap is not None:
            opts["softcap"] = self.score_cap
        if self.has_distance_bias:
            opts["distance_bias"] = (self.r1, self.r2)
        if self.chunk is not None:
            opts["chunk"] = self.chunk
        if self.has_sink:
            opts["sink"] = self.sink
        if self.has_sigmoid_bias:
            opts["sigmoid_bias"] = self.score_bias
        if self.keep_first:
            opts["keep_first"] = self.keep_first
        return opts

    def forward(self, normed, ctx, entry):
        b, kv = ctx.batch, ctx.kv(entry)
        amplitude = getattr(self.position, "amplitude", 1.0)
        if (self.rotated_norm_eps is not None or self.has_head_gate or self.shares_kv or amplitude != 1.0
                or self.value_norm_eps is not None or self.value_mix is not None):
            return self._forward_extended(normed, ctx, b, kv, amplitude)
        rope = (b.positions, b.slot_of_token, kv.table, self.position.table(ctx.device), self.position.pairing_code,
                self.position.rotary_dim, kv.k_pages if kv.owns else None, kv.v_pages if kv.owns else None,
                kv.layer_offset, kv.page_size, kv.page_stride, self.num_heads, self.num_kv_heads, self.head_dim, ctx.act)
        if self.qk_norm_eps is None:
            q = ops.qkv_rope_write(normed, self.qkv_weight, self.qkv_bias, *rope, runs=b.runs())
        else:
            qkv = ops.gemm(normed, self.qkv_weight, ctx.act, bias=self.qkv_bias)
            ops.head_rmsnorm(qkv, self.q_norm, self.k_norm, self.qk_norm_eps, self.num_heads, self.num_kv_heads,
                             self.head_dim, ctx.act, norm_dim=self.key_dim)
            q = ops.rope_kv_write(qkv, *rope, runs=b.runs())
        o = ops.attention(q, kv.k_pages, kv.v_pages, kv.layer_offset, b.positions, b.slot_of_token, kv.table,
                          kv.page_size, kv.page_stride, self.num_heads, self.num_kv_heads, self.head_dim,
                          self.window, self.scale, ctx.act, runs=b.runs(), **self._score_options())
        return ops.gemm(o, self.out_weight, ctx.act, bias=self.out_bias, partial_sums=True)

    def _forward_extended(self, normed, ctx, b, kv, amplitude):
        """The forms with a norm behind the rotation, scaled sines and cosines, a gate per head, another layer's keys
        and values, or values that are normed or mixed with an earlier layer's: one product of the layer's input (q | k | v | gate rows), the rotation with its norm and the cache
        write in one launch, attention with the gate where it normalises its output, the output product."""
        if kv.owns == self.shares_kv:
            raise ValueError("an attention keeps a cache of its own exactly if it has keys and values of its own")
        H, G, D = self.num_heads, 0 if self.shares_kv else self.num_kv_heads, self.head_dim
        proj = ops.gemm(normed, self.qkv_weight, ctx.act, bias=self.qkv_bias)
        width = (H + 2 * G) * D
        qkv = proj[:, :width]
        if (self.value_norm_eps is not None or self.value_mix is not None) and kv.owns and self.rotated_norm_eps is None:
            # head norms, unit values and their mix, rotation and cache write: one pass over a token's row
            first, first_dim = b.scratch[("value_mix",)] if self.value_mix == "mix" else (None, None)
            q = ops.attn_prep_kv_write(qkv, b.positions, b.slot_of_token, kv.table, self.position.table(ctx.device),
                                       self.position.pairing_code, self.position.rotary_dim, kv.k_pages, kv.v_pages,
                                       kv.layer_offset, kv.page_size, kv.page_stride, H, G, D, ctx.act, runs=b.runs(),
                                       amplitude=amplitude, q_weight=self.q_norm, k_weight=self.k_norm,
                                       qk_eps=self.qk_norm_eps or 0.0, norm_dim=self.key_dim,
                                       value_eps=self.value_norm_eps or 0.0, value_dim=self.value_dim, first=first,
                                       first_head_dim=first_dim, mix=self.mix if first is not None else None)
            if self.value_mix == "source":
                b.scratch[("value_mix",)] = (qkv[:, (H + G) * D:], D)
            o = ops.attention(q, kv.k_pages, kv.v_pages, kv.layer_offset, b.positions, b.slot_of_token, kv.table,
                              kv.page_size, kv.page_stride, H, self.num_kv_heads, D, self.window, self.scale, ctx.act,
                              runs=b.runs(), head_gate=proj[:, width:width + H] if self.has_head_gate else None,
                              **self._score_options())
            return ops.gemm(o, self.out_weight, ctx.act, bias=self.out_bias, partial_sums=True)
        if self.qk_norm_eps is not None:
            if proj.shape[1] != width:
                raise ValueError("the norm of the heads before the rotation does not go with a gate per head")
            ops.head_rmsnorm(qkv, self.q_norm, None if self.shares_kv else self.k_norm, self.qk_norm_eps, H, G, D, ctx.act,
                             norm_dim=self.key_dim)
        if self.value_norm_eps is not None or self.value_mix is not None:
            # the values as the cache will hold them: unit root mean square per head, then the blend with the values that
            # the source layer left for this step's tokens
            v = qkv[:, (H + G) * D:]
            first, first_dim = b.scratch[("value_mix",)] if self.value_mix == "mix" else (None, None)
            ops.value_norm_mix(v, G, D, self.value_dim, self.value_norm_eps or 0.0, ctx.act, first=first,
                               first_head_dim=first_dim, mix=self.mix if first is not None else None)
            if self.value_mix == "source":
                b.scratch[("value_mix",)] = (v, D)
        q = ops.rope_kv_write(qkv, b.positions, b.slot_of_token, kv.table, self.position.table(ctx.device),
                              self.position.pairing_code, self.position.rotary_dim, kv.k_pages if kv.owns else None,
                              kv.v_pages if kv.owns else None, kv.layer_offset, kv.page_size, kv.page_stride, H, G, D, ctx.act,
                              runs=b.runs(), amplitude=amplitude, norm_eps=self.rotated_norm_eps, norm_dim=self.key_dim)
        o = ops.attention(q, kv.k_pages, kv.v_pages, kv.layer_offset, b.positions, b.slot_of_token, kv.table,
                          kv.page_size, kv.page_stride, H, self.num_kv_heads, D, self.window, self.scale, ctx.act,
                          runs=b.runs(), head_gate=proj[:, width:width + H] if self.has_head_gate else None,
                          **self._score_options())
        return ops.gemm(o, self.out_weight, ctx.act, bias=self.out_bias, partial_sums=True)
