"""Two mixers side by side on the same input.

Both read the same h. Each result is divided by its root mean square over the
model's width and multiplied by a weight of its own (plain, not one-plus), and
the mixer's result is `factor` times their sum (one half unless given).

The two are any registered mixers (`left`, `right`: their PartSpecs). What
they keep between steps lives in one cache site: the pages of the one that
keeps pages (at most one may) and the fixed-size arrays of both, under the
names `left.<array>` and `right.<array>`; each mixer sees its own arrays under
its own names through a view of the step's context, and the left one keeps its
scratch under names of its own, since its result must outlive the right one's
run.

Parameters: width, eps, left, right, factor, names (left_out, right_out).
"""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.pages import FixedArray, FixedSpec, PagedSpec, fixed_part
from ..config.plan import PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Declared, StepContext
from .linear import place_vector
from .registry import part_class, register_part

_DEFAULT_NAMES = dict(left_out="left.out", right_out="right.out")


class _ScopedWorkspace:
    """A workspace whose names (and alias groups) carry a prefix."""

    def __init__(self, workspace, prefix: str):
        self._workspace, self._prefix = workspace, prefix

    def get(self, name, shape, dtype, alias=None):
        return self._workspace.get(self._prefix + name, shape, dtype,
                                   alias=None if alias is None else self._prefix + alias)

    def __getattr__(self, name):
        return getattr(self._workspace, name)


class _Scoped:
    """The step's context as one of the two mixers sees it: the site's fixed-size arrays that are
    its own, under its own names; no stream to add into (the pair's result is made of both)."""

    def __init__(self, ctx: StepContext, prefix: str, scratch_prefix: str = ""):
        self._ctx, self._prefix = ctx, prefix
        self.workspace = _ScopedWorkspace(ctx.workspace, scratch_prefix) if scratch_prefix else ctx.workspace
        self.stream = None

    def __getattr__(self, name):
        return getattr(self._ctx, name)

    def fixed_arrays(self, site: int) -> Dict[str, torch.Tensor]:
        p = self._prefix
        return {k[len(p):]: v for k, v in self._ctx.fixed_arrays(site).items() if k.startswith(p)}

    def fixed_state(self, site: int) -> torch.Tensor:
        arrays = self.fixed_arrays(site)
        return arrays["state"] if "state" in arrays else next(iter(arrays.values()))


class MixerPair:
    role = "mixer"

    @staticmethod
    def _names(spec: PartSpec) -> Dict[str, str]:
        names = dict(_DEFAULT_NAMES)
        names.update(spec.get("names") or {})
        return {k: f"{spec.prefix}.{v}" for k, v in names.items()}

    @classmethod
    def declare(cls, spec: PartSpec) -> Declared:
        n = cls._names(spec)
        out: Declared = {n["left_out"]: (TensorDecl((spec["width"],), "vector"), "norm"),
                         n["right_out"]: (TensorDecl((spec["width"],), "vector"), "norm")}
        for side in ("left", "right"):
            out.update(part_class("mixer", spec[side].kind).declare(spec[side]))
        return out

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], device: torch.device,
                 engine_dtype: torch.dtype):
        n = self._names(spec)
        self.width, self.eps = spec["width"], float(spec["eps"])
        self.factor = float(spec.get("factor", 0.5))
        self.left = part_class("mixer", spec["left"].kind)(spec["left"], tensors, device, engine_dtype)
        self.right = part_class("mixer", spec["right"].kind)(spec["right"], tensors, device, engine_dtype)
        if self.left.in_dtype != self.right.in_dtype:
            raise ValueError("two mixers side by side read their input in one dtype")
        self.left_out = place_vector(tensors[n["left_out"]], device)
        self.right_out = place_vector(tensors[n["right_out"]], device)
        self.graph_safe = bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))

    @property
    def in_dtype(self) -> torch.dtype:
        return self.left.in_dtype

    def cache_spec(self, page_size: int):
        specs = {"left.": self.left.cache_spec(page_size), "right.": self.right.cache_spec(page_size)}
        paged = [s for s in specs.values() if isinstance(s, PagedSpec)]
        if len(paged) > 1:
            raise ValueError("of two mixers side by side at most one keeps pages")
        arrays = ()
        for prefix, s in specs.items():
            fixed = fixed_part(s)
            if fixed is not None:
                arrays += tuple(FixedArray(prefix + a.name, a.shape, a.dtype, a.init) for a in fixed.all_arrays())
        fixed = FixedSpec(arrays=arrays) if arrays else None
        if paged:
            return PagedSpec(paged[0].arrays, paged[0].window, fixed, paged[0].chunk)
        return fixed

    def forward(self, ctx: StepContext, site: int, owns_cache: bool, h: torch.Tensor) -> torch.Tensor:
        a = self.left.forward(_Scoped(ctx, "left.", "left:"), site, owns_cache, h)
        b = self.right.forward(_Scoped(ctx, "right."), site, owns_cache, h)
        out = ctx.workspace.get("pair_out", (h.shape[0], self.width), torch.float32)
        return ops.normed_sum(a, self.left_out, b, self.right_out, self.eps, self.factor, out)


register_part("mixer", "mixer_pair", MixerPair)
