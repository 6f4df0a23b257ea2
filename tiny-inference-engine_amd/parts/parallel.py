"""Two (or more) mixers side by side: all read the same rows, their outputs are added with a factor each.

``y = sum_i scale_i * mixer_i(h)``. A branch is any registered mixer; its factor is handed to it as the parameter
``output_scale``, and the branch folds it into something it computes in float32 anyway (a convolution's weights, a
norm's weights), so that no pass over the rows is spent on it. The branches' cache needs are declared together, in
order (``Mixer.cache_need`` as a tuple), and every branch is bound to its own. Parameters: ``hidden``, ``branches``
(a list of ``(PartSpec of the mixer family, scale)``).
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..errors import InvalidArgument
from .base import Mixer, Part, PartSpec, StepContext, build_part, register_part


def _needs_of(mixer) -> tuple:
    need = mixer.cache_need()
    if need is None:
        return ()
    return tuple(need) if isinstance(need, (tuple, list)) else (need,)


@register_part("mixer", "parallel")
class ParallelMixer(Mixer):
    capturable = True
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.branches: List[Mixer] = []
        for spec, scale in params["branches"]:
            branch_params = dict(spec.params)
            branch_params["output_scale"] = float(scale) * float(branch_params.get("output_scale", 1.0))
            self.branches.append(build_part("mixer", PartSpec(spec.kind, branch_params)))
        if not self.branches:
            raise InvalidArgument("a parallel mixer needs at least one branch")
        self.counts = [len(_needs_of(b)) for b in self.branches]

    def children(self) -> List[Part]:
        return list(self.branches)

    def cache_need(self):
        needs = tuple(n for b in self.branches for n in _needs_of(b))
        return needs or None

    def _caches(self, cache):
        """Every branch's own binding(s), in the shape it declared them."""
        bindings = () if cache is None else (tuple(cache) if isinstance(cache, tuple) else (cache,))
        out, at = [], 0
        for branch, count in zip(self.branches, self.counts):
            mine = bindings[at:at + count]
            at += count
            declared = branch.cache_need()
            out.append(None if count == 0 else (mine if isinstance(declared, (tuple, list)) else mine[0]))
        return out

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: Optional[torch.Tensor]):
        caches = self._caches(cache)
        target = residual
        first = 0
        if target is None:
            # The first branch's result becomes the sum the others add to.
            y = self.branches[0].forward(ctx, h, caches[0], None) \
                if getattr(self.branches[0], "returns_result", False) else None
            ctx.settle()
            if isinstance(y, torch.Tensor) and y.dim() == 2:
                target, first = y, 1
            else:
                target = ctx.scratch("parallel.result", (h.shape[0], self.hidden), torch.float32)
                target.zero_()
                if isinstance(y, torch.Tensor):
                    kernels.add_partials(target, y)
                    first = 1
        for branch, binding in zip(self.branches[first:], caches[first:]):
            branch.forward(ctx, h, binding, target)
        if residual is None:
            ctx.settle()
            return target
        return None
