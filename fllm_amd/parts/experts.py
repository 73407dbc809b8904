"""A feed-forward of many small gated layers of which every token uses a few.

Router: z = W_router n in float32, score = sigmoid(z); the `top` experts with the largest scores are a token's picks (the
lower index among equal scores) and the scores themselves are their weights, not renormalized.  A pick's weight multiplies
the expert's INPUT: y = sum over the picks of W_down_e (a(W_gate_e (s_e n)) * (W_up_e (s_e n) + up_offset)) with
a(g) = g * sigmoid(alpha g), operands clamped to `limit` where there is one (the constants of `ClampedGLU`; the defaults
are SwiGLU).  The experts' matrices are stacked at load: [experts, 2 * inter, width] (gate rows, then up rows) and
[experts, width, inter], so that a kernel finds an expert by its index.
"""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import INIT_MATRIX, FeedForward


class RoutedExperts(FeedForward):
    graph_safe = True      # the picks stay on the device: no per-step decision on the host
    stores_branch = True   # forward(..., branch=t) stores the output in t (float32) instead of adding it to the stream

    @classmethod
    def tensor_shapes(cls, spec):
        h, i, n = spec["hidden_size"], spec["intermediate_size"], spec["experts"]
        shapes = {"router": ((n, h), INIT_MATRIX)}
        for e in range(n):
            shapes[f"gate_{e}"] = ((i, h), INIT_MATRIX)
            shapes[f"up_{e}"] = ((i, h), INIT_MATRIX)
            shapes[f"down_{e}"] = ((h, i), INIT_MATRIX)
        return shapes

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.experts = int(spec["experts"])
        self.top = int(spec["top"])
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"{self.top} picks among {self.experts} experts")
        if spec.get("score", "sigmoid") != "sigmoid":
            raise ValueError(f"router score {spec.get('score')!r}: the router's kernel scores with a sigmoid")
        self.limit = float(spec.get("limit") or 0.0)          # 0: nothing is clamped
        self.alpha = float(spec.get("alpha", 1.0))
        self.up_offset = float(spec.get("up_offset", 0.0))
        self.w_router = rt.matrix(weights["router"])
        n = self.experts
        self.w_gate_up = torch.stack([torch.cat([rt.matrix(weights[f"gate_{e}"]), rt.matrix(weights[f"up_{e}"])], dim=0)
                                      for e in range(n)]).contiguous()
        self.w_down = torch.stack([rt.matrix(weights[f"down_{e}"]) for e in range(n)]).contiguous()

    @property
    def branch_parts(self) -> int:
        """Rows of a stored branch that make up one token's output: a token's picks leave their outputs one after the
        other, and whoever adds the branch to the stream sums them in pick order."""
        return self.top

    def forward(self, ctx, h, residual, branch=None):
        """`branch`: float32 [rows * top, width], row r's picks at r * top ..; None: the sum goes into `residual`."""
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        ids = rt.empty((rows, self.top), torch.int32)
        weights = rt.empty((rows, self.top), torch.float32)
        ops.route_topk(h, self.w_router, self.top, ids, weights)
        parts = branch if branch is not None else rt.empty((rows * self.top, self.hidden), torch.float32)
        grouped = getattr(ops, "experts_grouped", None)
        if grouped is None or not grouped(h, ids, weights, self.w_gate_up, self.w_down, parts, self.limit, self.alpha, self.up_offset):
            act = rt.empty((rows * self.top, self.inter))
            ops.experts_gate_up(h, ids, weights, self.w_gate_up, act, self.limit, self.alpha, self.up_offset)
            ops.experts_down(act, ids, self.w_down, parts)
        if branch is None:
            ones = rt.shared.get(("ones", self.hidden))
            if ones is None:
                ones = rt.shared[("ones", self.hidden)] = torch.ones(self.hidden, dtype=torch.float32, device=rt.device)
            ops.postnorm_add(residual, parts, ones, None, parts=self.top)


register_part("feed_forward", "routed_experts", RoutedExperts)
