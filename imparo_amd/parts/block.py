"""How a layer's parts are arranged.

pre_norm: x += mixer(norm_a(x)); x += ffn(norm_b(x)) -- no post-norms
(/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:8-15). Each
delta is left pending on the residual stream so that the next norm, whichever
block it belongs to, adds it while reading the row.

Two optional parts widen the arrangement: `shift` (role "shift") mixes what
the mixer reads with the token before it and keeps the last token's input as
state of the block's own, beside the mixer's; a layer without `ffn` and
`ffn_norm` has no feed-forward."""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.pages import with_fixed_arrays
from ..kernels import ops
from .base import Residual, StepContext, emits
from .registry import register_part


class PreNormBlock:
    """Reads its parts by name: mixer_norm, mixer, ffn_norm, ffn; optionally shift; ffn_norm and ffn may be absent."""
    role = "block"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    def __init__(self, parts: Dict[str, object]):
        self.parts = parts
        self.mixer_norm, self.mixer = parts["mixer_norm"], parts["mixer"]
        self.ffn_norm, self.ffn = parts.get("ffn_norm"), parts.get("ffn")
        self.shift = parts.get("shift")
        if (self.ffn is None) != (self.ffn_norm is None):
            raise ValueError("a block has a feed-forward and the norm before it, or neither")

    def cache_spec(self, page_size: int):
        """What a call of this block keeps between steps: its mixer's state and,
        with a token shift, the input that the request's last token left."""
        spec = self.mixer.cache_spec(page_size)
        if self.shift is not None:
            spec = with_fixed_arrays(spec, self.shift.state_arrays())
        return spec

    def forward(self, ctx: StepContext, res: Residual, site: int, owns_cache: bool) -> None:
        if self.shift is None:
            h = self.mixer_norm.forward(ctx, res, self.mixer.in_dtype)
        elif not owns_cache:
            raise ValueError("a token shift's state cannot be read from another layer")
        elif ctx.max_seg_len == 1 and hasattr(self.mixer_norm, "forward_shifted"):
            # every row brings one token: the shift rides in the norm's launch
            h = self.mixer_norm.forward_shifted(ctx, res, self.mixer.in_dtype, self.shift.mix,
                                                self.shift.state(ctx, site))
        else:
            h = self.shift.forward(ctx, site, self.mixer_norm.forward(ctx, res, torch.float32, name="normed_f32"),
                                   self.mixer.in_dtype)
        res.pending = self._delta(ctx, res, lambda: self.mixer.forward(ctx, site, owns_cache, h))
        if self.ffn is not None:
            n = self.ffn_norm.forward(ctx, res, self.ffn.in_dtype)
            res.pending = self._delta(ctx, res, lambda: self.ffn.forward(ctx, n))

    def can_emit(self) -> bool:
        if self.shift is not None or self.ffn is None:
            return False          # the step program knows the four-part block only
        parts = (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)
        return all(emits(p) and getattr(p, "can_emit", lambda: True)() for p in parts)

    def emit(self, program, site: int, owns_cache: bool) -> None:
        """Appends `forward` to a native step program: the four parts in the order they run."""
        self.mixer_norm.emit(program, self.mixer.in_dtype)
        self.mixer.emit(program, site, owns_cache)
        self.ffn_norm.emit(program, self.ffn.in_dtype)
        self.ffn.emit(program)

    @staticmethod
    def _delta(ctx: StepContext, res: Residual, run):
        """Runs a part whose result goes into the stream. With nothing pending the part may add its
        result to the stream itself (it then returns the stream); otherwise it returns a delta."""
        ctx.stream = res.x if res.pending is None else None
        try:
            delta = run()
        finally:
            ctx.stream = None
        return None if delta is res.x else delta


class SandwichBlock(PreNormBlock):
    """x += post_a(mixer(norm_a(x))); x += post_b(ffn(norm_b(x))): a norm before and behind each
    sublayer. The parts `mixer_post` and `ffn_post` are norms (their weights may carry a layer
    scale and a residual multiplier); a sublayer's result is left pending on the stream together
    with its norm, and the next norm that reads the stream, whichever block it belongs to, applies
    that norm, adds and norms the sum in one launch."""

    def __init__(self, parts: Dict[str, object]):
        super().__init__(parts)
        if self.shift is not None:
            raise ValueError("this arrangement has no token shift")
        self.mixer_post, self.ffn_post = parts["mixer_post"], parts.get("ffn_post")
        if (self.ffn is None) != (self.ffn_post is None):
            raise ValueError("a block has a feed-forward and the norm behind it, or neither")

    def forward(self, ctx: StepContext, res: Residual, site: int, owns_cache: bool) -> None:
        h = self.mixer_norm.forward(ctx, res, self.mixer.in_dtype)
        res.pending, res.post = self.mixer.forward(ctx, site, owns_cache, h), self.mixer_post.as_post()
        if self.ffn is not None:
            # (a buffer of its own: the feed-forward may leave this input to be read by the launch of the next
            # norm, which writes its own result where norms usually do)
            n = self.ffn_norm.forward(ctx, res, self.ffn.in_dtype, name="normed_ffn")
            # a feed-forward that can leave its last sum to the norm's launch does (`forward_rows`)
            run = getattr(self.ffn, "forward_rows", None) or self.ffn.forward
            res.pending, res.post = run(ctx, n), self.ffn_post.as_post()

    def can_emit(self) -> bool:
        return False          # the step program knows the pre-norm block only


class ParallelBlock:
    """x += gate_a * mixer(h) + gate_b * ffn(h) with h = norm(x): one norm feeds both sublayers, and each
    result is multiplied by sigmoid(W h + b) of that same input (`mixer_gate`, `ffn_gate`: both gates are
    one projection). Optional parts: `ffn` with `ffn_gate` (a layer may have no feed-forward), and `side`, a
    per-layer input from the token itself that reads the stream behind the sum; its result is left pending on
    the stream together with its norm, so that the next norm, whichever block it belongs to, applies it,
    adds and norms the sum in one launch."""
    role = "block"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    def __init__(self, parts: Dict[str, object]):
        from .gate import SigmoidGate
        self.parts = parts
        self.mixer_norm, self.mixer, self.mixer_gate = parts["mixer_norm"], parts["mixer"], parts["mixer_gate"]
        self.ffn, self.ffn_gate = parts.get("ffn"), parts.get("ffn_gate")
        self.side = parts.get("side")
        if (self.ffn is None) != (self.ffn_gate is None):
            raise ValueError("a block has a feed-forward and its gate, or neither")
        self.gates = SigmoidGate.together([self.mixer_gate] + ([self.ffn_gate] if self.ffn is not None else []))

    def cache_spec(self, page_size: int):
        return self.mixer.cache_spec(page_size)

    def forward(self, ctx: StepContext, res: Residual, site: int, owns_cache: bool) -> None:
        # the norm's output once per dtype its readers ask for (one, unless some projection's sizes keep it in float32)
        normed = {}

        def h_in(dtype):
            if dtype not in normed:
                normed[dtype] = self.mixer_norm.forward(ctx, res, dtype, name=f"normed_{len(normed)}" if normed else "normed")
            return normed[dtype]

        h = h_in(self.mixer.in_dtype)
        gates = self.gates(ctx, h_in(self.gates.in_dtype), torch.float32, "gates")
        m = self.mixer.forward(ctx, site, owns_cache, h)
        f = None if self.ffn is None else self.ffn.forward(ctx, h_in(self.ffn.in_dtype))
        copy = None
        if self.side is not None:
            copy = ctx.workspace.get("stream_copy", tuple(res.x.shape), self.side.in_dtype)
        ops.gated_sum(res.x, m, f, gates, copy)
        if self.side is not None:
            res.pending, res.post = self.side.forward(ctx, copy), self.side.as_post()

    def can_emit(self) -> bool:
        return False          # the step program knows the pre-norm block only


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "sandwich", SandwichBlock)
