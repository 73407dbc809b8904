"""Attention whose heads talk to each other before the softmax, over the paged cache.

q, k, v and the output gate are one product with the concatenated matrix.  The whole query projection is normed as one
vector (RMSNorm over heads * head_dim values with a weight a lane), the whole key projection likewise; rotary on the first
lanes of every head; keys and values (of widths of their own) go into the pages of the row's request.  A score is
q_g . k * scale * temp[g]; head h then takes sum_g talk[h, g] * score_g, softmax over the keys the row sees: those of
its own chunk of `chunk` positions up to itself (chunks counted from the request's first position; None: all keys up
to itself).  Head h's output is multiplied by sigmoid(gate_h), gate = W_g n with the mixer's own input n, and the
concatenated heads go through the output projection into the residual stream.
"""
from __future__ import annotations

import torch

from ..config.spec import PartSpec
from ..registry import part_class, register_part
from .base import INIT_MATRIX, INIT_NORM, KVNeed, Mixer, fused_form


class TalkingAttention(Mixer):
    graph_safe = True      # forward launches kernels only: no per-step decision on the host

    @classmethod
    def tensor_shapes(cls, spec):
        h, nh, nkv, d = spec["hidden_size"], spec["num_heads"], spec["num_kv_heads"], spec["head_dim"]
        dv = spec.get("value_head_dim") or d
        return {
            "q": ((nh * d, h), INIT_MATRIX), "k": ((nkv * d, h), INIT_MATRIX), "v": ((nkv * dv, h), INIT_MATRIX),
            "o": ((h, nh * dv), INIT_MATRIX), "gate": ((nh, h), INIT_MATRIX),
            "q_norm": ((nh * d,), INIT_NORM), "k_norm": ((nkv * d,), INIT_NORM),
            "talk": ((nh, nh), INIT_MATRIX), "temp": ((nh,), INIT_NORM),
        }

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.k_dim = int(spec["head_dim"])
        self.v_dim = int(spec.get("value_head_dim") or self.k_dim)
        self.scale = float(spec["scale"])
        self.chunk = spec.get("chunk")
        self.eps = float(spec["qk_norm_eps"])
        if self.heads % self.kv_heads != 0:
            raise ValueError(f"head count {self.heads} is not a multiple of key/value head count {self.kv_heads}")
        if self.chunk is not None and self.chunk <= 0:
            raise ValueError("a chunk of positions must be positive")
        # keys lie in chunks of 8 values inside a page where the head size allows it (what the matrix-core kernels
        # read); other head sizes store keys lane by lane and run the plain kernels
        self.key_chunk = 8 if self.k_dim % 8 == 0 else 1
        position = spec.get("position")
        self.position = None
        if position is not None:
            position = dict(position)
            kind = position.pop("kind")
            self.position = part_class("position", kind)(PartSpec(kind, position), {}, rt)
            if self.position.pairing != 0:
                raise ValueError("this attention rotates lane i with lane i + dims / 2 only")
            if self.position.dims > self.k_dim:
                raise ValueError(f"{self.position.dims} rotated lanes in heads of {self.k_dim}")
        # one matrix for q, k, v and the gate: the normed input is read once.  Zero rows bring the width to a multiple
        # of 8, so that every row of the product begins on 16 bytes.
        parts = [rt.matrix(weights["q"]), rt.matrix(weights["k"]), rt.matrix(weights["v"]), rt.matrix(weights["gate"])]
        used = sum(p.shape[0] for p in parts)
        if used % 8:
            parts.append(torch.zeros((8 - used % 8, self.hidden), dtype=parts[0].dtype, device=rt.device))
        self.w_qkvg = torch.cat(parts, dim=0).contiguous()
        self.gate_at = self.heads * self.k_dim + self.kv_heads * (self.k_dim + self.v_dim)
        self.w_o = rt.matrix(weights["o"])
        rt.tile_for_decode(self.w_o)
        rt.tile_for_decode(self.w_qkvg, priority=1)
        self.q_norm = rt.vector(weights["q_norm"])
        self.k_norm = rt.vector(weights["k_norm"])
        self.talk = rt.vector(weights["talk"])
        self.temp = rt.vector(weights["temp"])

    def cache_need(self):
        # every key is kept: a row sees back to the start of its chunk only, but the pages of earlier chunks stay with
        # the request until it ends
        return KVNeed(self.kv_heads, self.k_dim, self.v_dim, None, key_chunk=self.key_chunk)

    def project_from_residual(self, ctx, residual, norm):
        """Decode-sized steps in bfloat16: the norm before the mixer and the joint product are one kernel that reads the
        residual stream; `attend` goes on from the product.  None: not taken."""
        rt, ops = self.rt, self.rt.ops
        rows = residual.shape[0]
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        if rt.dtype != torch.bfloat16 or prologue is None or not hasattr(ops, "norm_linear"):
            return None
        if fused_form(ops, rows, self.hidden, self.w_qkvg) != "resident":
            return None
        qkvg = rt.empty((rows, self.w_qkvg.shape[0]))
        ops.norm_linear(residual, prologue[0], prologue[1], self.w_qkvg, qkvg)
        return qkvg

    def forward(self, ctx, h, residual, binding):
        qkvg = self.rt.empty((h.shape[0], self.w_qkvg.shape[0]))
        self.rt.ops.linear(h, self.w_qkvg, qkvg)
        self.attend(ctx, qkvg, residual, binding)

    def attend(self, ctx, qkvg, residual, binding):
        """From the joint product [q | k | v | gate] of the step's rows to the sum into the residual stream."""
        rt, ops = self.rt, self.rt.ops
        rows = qkvg.shape[0]
        nh, nkv, d, dv = self.heads, self.kv_heads, self.k_dim, self.v_dim
        tables = ctx.tables[binding.group]
        if self.position is not None:
            cos, sin, dims = self.position.cos, self.position.sin, self.position.dims
        else:
            cos, sin, dims, _ = ctx.no_rotation(rt)
        q = rt.empty((rows, nh * d))
        ops.qk_norm_rope_store(qkvg, self.q_norm, self.k_norm, self.eps, q, ctx.row_pos, ctx.row_seg, tables, cos, sin,
                               binding.k_pages if binding.writes else None, binding.v_pages if binding.writes else None,
                               nh, nkv, d, dv, dims, binding.page_size, self.key_chunk)
        out = rt.empty((rows, nh * dv))
        # few row tiles (a decode step has one a request): several workgroups share a tile's keys and meet in a workspace
        extra = {"single_rows": True} if getattr(ctx, "uniform_rows", False) and hasattr(ops, "talking_attention_splits") else {}
        split = getattr(ops, "talking_attention_splits", None)
        if split is not None and rt.dtype == torch.bfloat16:
            segments = ctx.seg_start.numel() - 1
            splits = split(rows, segments, self.chunk, ctx.max_context)
            if splits > 1:
                extra = {**extra, "splits": splits, "workspace": rt.empty((ops.talking_attention_workspace(rows, segments, nh, dv, splits),),
                                                                 dtype=torch.float32)}
        ops.talking_attention(q, qkvg[:, self.gate_at:self.gate_at + nh], binding.k_pages, binding.v_pages, tables,
                              ctx.row_pos, ctx.row_seg, ctx.seg_start, self.talk, self.temp, out, nh, nkv, d, dv,
                              binding.page_size, self.scale, self.chunk, self.key_chunk, ctx.max_context, **extra)
        ops.linear(out, self.w_o, residual, accumulate=True)


register_part("mixer", "talking_attention", TalkingAttention)
