"""Arrangement of parts in a layer.  `prenorm`: x += mixer(norm(x)); x += feed_forward(norm(x))
(rust/engine/src/rust_decoder.rs:8764-8766, :9059-9088).  `parallel`: x += mixer(norm_a(x)) + feed_forward(norm_b(x)),
both branches behind norms of their own of the same x.  `sandwich`: a norm before and a norm behind each part,
x += m * s_a * norm_a'(mixer(norm_a(x))); x += m * s_b * norm_b'(feed_forward(norm_b(x))), with a constant m and
learned vectors s (a scale a lane of each branch)."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import INIT_NORM, Block


class PreNormBlock(Block):
    def __init__(self, spec, weights, rt, mixer=None, feed_forward=None, norms=None):
        super().__init__(spec, weights, rt)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = norms["mixer"]
        self.feed_forward_norm = norms["feed_forward"] if feed_forward is not None else None

    def first_norm(self):
        return self.mixer_norm

    takes_pending = True     # forward accepts a branch that the block before has not added yet, and may hand one on

    def forward(self, ctx, residual, binding, pending=None):
        """Runs the layer on the residual stream.  `pending`: the output of the block before, still
        to be added; the return value is this block's own such output, or None when everything has
        been added.  Where a sum can ride on the norm that follows it, it costs no pass of its own."""
        ops = self.rt.ops
        # a norm prepared ahead: what the block before left for this block's first norm, and the norms that this
        # block's own sums are read by (the feed-forward's; the first norm of the block after)
        incoming, ctx.prepared = getattr(ctx, "prepared", None), None
        after = getattr(ctx, "next_norm", None)
        try:
            return self._forward(ctx, residual, binding, pending, incoming, after)
        finally:
            ctx.then_norm = None
            left = getattr(ctx, "prepared", None)
            if left is not None and (after is None or left[0] is not after):
                ctx.prepared = None          # nothing outlives the sum it was made from

    def _forward(self, ctx, residual, binding, pending, incoming, after):
        ops = self.rt.ops
        add_mixer_norm = getattr(self.mixer_norm, "add_forward", None)
        add_ff_norm = getattr(self.feed_forward_norm, "add_forward", None) if self.feed_forward is not None else None
        # a part may take the residual stream and the norm before it in one fused kernel
        fused = getattr(self.mixer, "forward_from_residual", None)
        if pending is not None:
            if add_mixer_norm is None:
                ops.add_residual(residual, pending)
                pending = None
            else:
                fused = None     # the fused kernels read the finished residual stream: the sum rides on the norm instead
        if fused is not None and pending is None:
            ctx.prepared = incoming
        ctx.then_norm = self.feed_forward_norm if self.feed_forward is not None else after
        taken = fused is not None and fused(ctx, residual, self.mixer_norm, binding)
        ctx.then_norm = None
        if not taken:
            ctx.prepared = None
            if pending is not None:
                h = add_mixer_norm(ctx, residual, pending)
            else:
                h = self.mixer_norm.forward(ctx, residual)
            # a mixer may hand back its output instead of adding it: the add then rides on the next norm
            as_branch = getattr(self.mixer, "forward_branch", None)
            branch = as_branch(ctx, h, binding) if as_branch is not None and add_ff_norm is not None else None
            if branch is not None:
                h = add_ff_norm(ctx, residual, branch)
                ff_branch = getattr(self.feed_forward, "forward_branch", None)
                out = ff_branch(ctx, h) if ff_branch is not None else None
                if out is None:
                    self.feed_forward.forward(ctx, h, residual)
                return out
            self.mixer.forward(ctx, h, residual, binding)
        if self.feed_forward is None:
            return None                  # a layer of a mixer alone
        left = getattr(ctx, "prepared", None)
        if left is not None and left[0] is not self.feed_forward_norm:
            ctx.prepared = None
        fused = getattr(self.feed_forward, "forward_from_residual", None)
        ctx.then_norm = after
        taken = fused is not None and fused(ctx, residual, self.feed_forward_norm)
        ctx.then_norm = None
        if not taken:
            ctx.prepared = None
            h = self.feed_forward_norm.forward(ctx, residual)
            self.feed_forward.forward(ctx, h, residual)
        return None


class ParallelBlock(Block):
    """Both branches read the stream as the layer found it, each through its own norm; their outputs are added to it.
    Where both norms are of the form x * rsqrt(mean x^2 + eps) * w they share one pass over the rows."""

    def __init__(self, spec, weights, rt, mixer=None, feed_forward=None, norms=None):
        super().__init__(spec, weights, rt)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = norms["mixer"]
        self.feed_forward_norm = norms["feed_forward"] if feed_forward is not None else None

    def forward(self, ctx, residual, binding):
        rt, ops = self.rt, self.rt.ops
        ctx.then_norm = ctx.prepared = None          # the sums of this block's parts are not read by a norm they know
        # a part may read the stream through its norm in one kernel with its first product, and add to it later: every
        # reader of the stream runs before the first sum into it
        project = getattr(self.mixer, "project_from_residual", None)
        projected = project(ctx, residual, self.mixer_norm) if project is not None else None
        if self.feed_forward is None:
            if projected is not None:
                self.mixer.attend(ctx, projected, residual, binding)
            else:
                self.mixer.forward(ctx, self.mixer_norm.forward(ctx, residual), residual, binding)
            return
        begin = getattr(self.feed_forward, "begin_from_residual", None)
        begun = begin(ctx, residual, self.feed_forward_norm) if begin is not None else None
        h_mixer = h_ff = None
        if projected is None and begun is None:
            first = getattr(self.mixer_norm, "fused_prologue", lambda: None)()
            second = getattr(self.feed_forward_norm, "fused_prologue", lambda: None)()
            pair = getattr(ops, "rmsnorm_pair", None)
            if pair is not None and first is not None and second is not None:
                h_mixer, h_ff = rt.empty(tuple(residual.shape)), rt.empty(tuple(residual.shape))
                pair(residual, first[0], first[1], h_mixer, second[0], second[1], h_ff)
        if projected is None and h_mixer is None:
            h_mixer = self.mixer_norm.forward(ctx, residual)
        if begun is None and h_ff is None:
            h_ff = self.feed_forward_norm.forward(ctx, residual)
        if projected is not None:
            self.mixer.attend(ctx, projected, residual, binding)
        else:
            self.mixer.forward(ctx, h_mixer, residual, binding)
        if begun is not None:
            self.feed_forward.finish(ctx, begun, residual)
        else:
            self.feed_forward.forward(ctx, h_ff, residual)


class SandwichBlock(Block):
    """x += gain_a * rms'(mixer(norm_a x)); x += gain_b * rms'(feed_forward(norm_b x)): every branch is normed again
    (RMS over its own lanes) before it joins the stream.  gain = residual_mult * layer scale * the second norm's weight,
    one float32 vector a branch, made once: the kernel that adds a branch norms it on the way (`postnorm_add`).  The
    norms behind the parts are `mixer_out` and `feed_forward_out` (absent: the branch is scaled and added as it is); the
    layer scales are the block's own tensors `mixer_scale` and `feed_forward_scale` (optional).

    A part with `stores_branch` writes its output (float32) where the block tells it to (`branch=`); any other part adds
    into a zeroed buffer that stands in for the stream.  A part may leave several partial rows a token (`branch_parts`),
    which the adding kernel sums first."""

    @classmethod
    def tensor_shapes(cls, spec):
        return {"mixer_scale": ((spec["size"],), INIT_NORM), "feed_forward_scale": ((spec["size"],), INIT_NORM)}

    def __init__(self, spec, weights, rt, mixer=None, feed_forward=None, norms=None):
        super().__init__(spec, weights, rt)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.size = int(spec["size"])
        self.mixer_norm = norms["mixer"]
        self.feed_forward_norm = norms["feed_forward"] if feed_forward is not None else None
        mult = float(spec.get("residual_mult", 1.0))
        self.mixer_gain, self.mixer_eps = self._gain(mult, weights.get("mixer_scale"), norms.get("mixer_out"))
        if feed_forward is not None:
            self.feed_forward_gain, self.feed_forward_eps = self._gain(mult, weights.get("feed_forward_scale"),
                                                                       norms.get("feed_forward_out"))

    def _gain(self, mult, scale, out_norm):
        """(gain vector, eps of the norm behind the part or None when there is none)."""
        gain = torch.full((self.size,), mult, dtype=torch.float32, device=self.rt.device)
        eps = None
        if out_norm is not None:
            prologue = getattr(out_norm, "fused_prologue", lambda: None)()
            if prologue is None:
                raise ValueError("the norm behind a part must be of the form x * rsqrt(mean x^2 + eps) * weight")
            gain = gain * prologue[0]
            eps = float(prologue[1])
        if scale is not None:
            gain = gain * self.rt.vector(scale)
        return gain.contiguous(), eps

    def first_norm(self):
        return None          # this block's first norm rides on the sum before it only inside the block itself

    def _branch(self, part, rows):
        return self.rt.empty((rows * int(getattr(part, "branch_parts", 1)), self.size), torch.float32)

    def forward(self, ctx, residual, binding):
        rt, ops = self.rt, self.rt.ops
        rows = residual.shape[0]
        ctx.then_norm = ctx.prepared = None          # no sum of this block's parts is read by a norm the parts know
        # ---- mixer
        mixer = self.mixer
        if getattr(mixer, "stores_branch", False):
            branch = self._branch(mixer, rows)
            fused = getattr(mixer, "forward_from_residual", None)
            if fused is None or not fused(ctx, residual, self.mixer_norm, binding, branch=branch):
                mixer.forward(ctx, self.mixer_norm.forward(ctx, residual), None, binding, branch=branch)
        else:
            branch = torch.zeros((rows, self.size), dtype=torch.float32, device=rt.device)
            mixer.forward(ctx, self.mixer_norm.forward(ctx, residual), branch, binding)
        ff = self.feed_forward
        if ff is None:
            ops.postnorm_add(residual, branch, self.mixer_gain, self.mixer_eps, parts=branch.shape[0] // rows)
            return
        # the sum of the mixer's branch and the norm before the feed-forward are one pass over the row, unless the
        # feed-forward reads the stream through its norm itself
        begin = getattr(ff, "begin_from_residual", None) if getattr(ff, "stores_branch", False) else None
        prologue = getattr(self.feed_forward_norm, "fused_prologue", lambda: None)()
        takes_stream = begin is not None and getattr(ff, "begins_from_residual", lambda rows: False)(rows)
        h = None
        if prologue is not None and not takes_stream:
            h = rt.empty((rows, self.size))
            ops.postnorm_add(residual, branch, self.mixer_gain, self.mixer_eps, parts=branch.shape[0] // rows,
                             next_weight=prologue[0], next_eps=prologue[1], next_out=h)
        else:
            ops.postnorm_add(residual, branch, self.mixer_gain, self.mixer_eps, parts=branch.shape[0] // rows)
        # ---- feed-forward
        if getattr(ff, "stores_branch", False):
            branch = self._branch(ff, rows)
            begun = begin(ctx, residual, self.feed_forward_norm) if takes_stream else None
            if begun is not None:
                ff.finish(ctx, begun, None, branch=branch)
            else:
                ff.forward(ctx, h if h is not None else self.feed_forward_norm.forward(ctx, residual), None, branch=branch)
        else:
            branch = torch.zeros((rows, self.size), dtype=torch.float32, device=rt.device)
            ff.forward(ctx, h if h is not None else self.feed_forward_norm.forward(ctx, residual), branch)
        ops.postnorm_add(residual, branch, self.feed_forward_gain, self.feed_forward_eps, parts=branch.shape[0] // rows)


register_part("block", "prenorm", PreNormBlock)
register_part("block", "sandwich", SandwichBlock)
register_part("block", "parallel", ParallelBlock)
