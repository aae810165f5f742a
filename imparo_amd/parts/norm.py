"""RMS norm: y = x * rsqrt(mean(x^2) + eps) * w, no offset, no bias
(/root/reference/crates/imparo-cpu/src/ops.rs:6-22). The residual add that
precedes a norm is fused into it (the reference's add_rms_norm,
/root/reference/crates/imparo-backend/src/lib.rs:2603-2609).

With `groups` > 1 the row is cut into that many equal consecutive parts and
each is divided by its own root mean square; the weight spans the whole row.
`tensor` names the weight outright where a checkpoint does not call it
`<prefix>.weight`. `offset` is added to the stored weight (1 where a file keeps a weight's
distance from one). `scale_tensor` names a second vector of the row's width and
`multiplier` a constant that the normed row is multiplied by as well (a layer
scale and a residual multiplier on a norm that sits behind a sublayer): all
three are folded into one float32 weight when the model is loaded. `scalar`: the
stored weight is a single number for the whole row (a tensor without
dimensions), spread over the row's width when the model is loaded.

A block may leave its sublayer's result pending on the stream together with
the norm it goes through before the add (`Residual.post`); this norm then
applies that norm, adds, and norms the sum in one launch."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, Residual, StepContext
from .linear import place_vector
from .registry import register_part


class RmsNorm:
    role = "norm"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @staticmethod
    def _tensor(spec: PartSpec) -> str:
        return spec.get("tensor") or f"{spec.prefix}.weight"

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        # a weight that an offset of 1 is added to is drawn near zero
        shape = () if spec.get("scalar") else (spec["width"],)
        out = {cls._tensor(spec): (TensorDecl(shape, "vector"), "bias" if spec.get("offset") else "norm")}
        if spec.get("scale_tensor"):
            out[spec["scale_tensor"]] = (TensorDecl((spec["width"],), "vector"), "norm")
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        self.width = spec["width"]
        self.eps = float(spec["eps"])
        self.groups = int(spec.get("groups") or 1)
        if self.groups < 1 or self.width % self.groups:
            raise ValueError(f"a norm over {self.width} values cannot be cut into {self.groups} equal parts")
        weight = tensors[self._tensor(spec)].to(torch.float32) + float(spec.get("offset") or 0.0)
        if spec.get("scalar"):
            weight = weight.reshape(1).expand(self.width)
        if spec.get("scale_tensor"):
            weight = weight * tensors[spec["scale_tensor"]].to(torch.float32)
        if spec.get("multiplier") is not None:
            weight = weight * float(spec["multiplier"])
        self.weight = place_vector(weight, device)

    def as_post(self):
        """(weight, eps) for `Residual.post`: this norm applied to a sublayer's result by whoever adds it."""
        if self.groups != 1:
            raise ValueError("a norm behind a sublayer does not cut rows into groups")
        return self.weight, self.eps

    def forward(self, ctx: StepContext, res: Residual, out_dtype: torch.dtype, name: str = "normed") -> torch.Tensor:
        """Adds the pending delta into the stream (if any) and returns the
        normed rows in `out_dtype`."""
        out = ctx.workspace.get(name, tuple(res.x.shape), out_dtype)
        pending, res.pending = res.pending, None
        post, res.post = res.post, None
        if post is not None and pending is not None:
            if self.groups > 1:
                raise ValueError("a norm in groups cannot take a sublayer's result through a norm of its own")
            ops.post_norm_add(res.x, pending, post[0], post[1], self.weight, self.eps, out)
        elif self.groups > 1:
            ops.group_rms_norm(res.x, self.weight, self.groups, self.eps, out, delta=pending,
                               write_back=pending is not None)
        elif pending is not None:
            ops.rms_norm(res.x, self.weight, self.eps, out, delta=pending, write_back=True)
        else:
            ops.rms_norm(res.x, self.weight, self.eps, out)
        return out

    def forward_shifted(self, ctx: StepContext, res: Residual, out_dtype: torch.dtype, mix: torch.Tensor,
                        state: torch.Tensor, name: str = "normed") -> torch.Tensor:
        """`forward` for a step whose rows all bring one token, with the token shift behind the norm in
        the same launch: out = h + (prev - h) * mix, where the request's prev (state[slot]) becomes h."""
        out = ctx.workspace.get(name, tuple(res.x.shape), out_dtype)
        if res.post is not None:
            raise ValueError("the norm with the token shift does not take a sublayer's result through a norm of its own")
        pending, res.pending = res.pending, None
        ops.group_rms_norm(res.x, self.weight, self.groups, self.eps, out, delta=pending,
                           write_back=pending is not None, shift_mix=mix, shift_state=state, slot=ctx.slot)
        return out

    def can_emit(self) -> bool:
        return self.groups == 1

    def emit(self, program, out_dtype: torch.dtype) -> None:
        """Appends `forward` to a native step program."""
        if self.groups != 1:
            raise ValueError("the step program's norm does not cut rows into groups")
        program.norm(self.weight, self.eps, self.width, out_dtype)

    def emit_head(self, program, head_linear) -> None:
        """Appends `forward_rows` followed by the head's projection."""
        program.head(self.weight, self.eps, self.width, head_linear)

    def forward_rows(self, ctx: StepContext, res: Residual, rows: torch.Tensor, out_dtype: torch.dtype,
                     name: str = "normed_rows") -> torch.Tensor:
        """Norm of selected rows only (the rows whose logits are wanted); the
        stream itself is left as it is."""
        out = ctx.workspace.get(name, (rows.shape[0], self.width), out_dtype)
        if res.post is not None and res.pending is not None:
            if self.groups > 1:
                raise ValueError("a norm in groups cannot take a sublayer's result through a norm of its own")
            ops.post_norm_add(res.x, res.pending, res.post[0], res.post[1], self.weight, self.eps, out, rows=rows)
        elif self.groups > 1:
            ops.group_rms_norm(res.x, self.weight, self.groups, self.eps, out, delta=res.pending, rows=rows)
        else:
            ops.rms_norm(res.x, self.weight, self.eps, out, delta=res.pending, rows=rows)
        return out


class NoNorm:
    """No norm where a block has a place for one: the sublayer reads the stream itself. What is
    pending on the stream is added first, through the norm it carries if it carries one, in the
    same launch that hands the rows on in the dtype the reader asks for."""
    role = "norm"
    graph_safe = True     # launches kernels only: a step made of such parts can be captured

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        return {}

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        self.width = spec["width"]

    @staticmethod
    def _add_plain(res: Residual, pending) -> None:
        """A delta that carries no norm: its slices are added to the stream in order."""
        if not isinstance(pending, torch.Tensor):
            raise ValueError("rows that a routed feed-forward left to be combined go through a norm behind it")
        for part in (pending if pending.dim() == res.x.dim() + 1 else [pending]):
            ops.add_rows(res.x, part)

    def forward(self, ctx: StepContext, res: Residual, out_dtype: torch.dtype, name: str = "normed") -> torch.Tensor:
        pending, res.pending = res.pending, None
        post, res.post = res.post, None
        if pending is not None and post is None:
            self._add_plain(res, pending)
            pending = None
        if pending is None and out_dtype == torch.float32:
            return res.x          # readers do not write into what they read
        out = ctx.workspace.get(name, tuple(res.x.shape), out_dtype)
        if pending is None:
            return ops.cast_rows(res.x, out)
        ops.post_norm_add(res.x, pending, post[0], post[1], None, 0.0, out)
        return out

    def forward_rows(self, ctx: StepContext, res: Residual, rows: torch.Tensor, out_dtype: torch.dtype,
                     name: str = "normed_rows") -> torch.Tensor:
        """The chosen rows as they would be after the pending add; the stream itself is left as it is."""
        out = ctx.workspace.get(name, (rows.shape[0], self.width), out_dtype)
        if res.pending is None:
            return ops.cast_rows(res.x, out, rows)
        if res.post is None:
            raise ValueError("rows are chosen from a stream whose pending delta goes through a norm, or has none pending")
        ops.post_norm_add(res.x, res.pending, res.post[0], res.post[1], None, 0.0, out, rows=rows)
        return out


register_part("norm", "rms_norm", RmsNorm)
register_part("norm", "none", NoNorm)
