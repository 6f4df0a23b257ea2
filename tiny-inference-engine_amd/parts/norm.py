"""Norms over the rows of the stream. RMSNorm: ``out = (x * inv) * w`` with ``inv = 1 / sqrt(mean(x^2) + eps)``.

The weight multiplies after normalisation and is the plain ``w`` (not ``1 + w``);
no bias, no mean subtraction; statistics in float32
(``src/backend/cpu/cpu_backend.cpp:141-159``). Parameters: ``dim``, ``eps``,
``weight`` (tensor name) and, for designs that store the weight around zero, ``one_plus`` (True: the norm
multiplies by ``1 + w``; the sum is formed once at load time, in float32, which is the value the multiplication
would see anyway).

``layer_norm`` subtracts the row's mean first: ``out = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w``, a weight and
no bias, statistics in float32. Parameters: ``dim``, ``eps``, ``weight``.

``dynamic_tanh`` computes no mean and no variance: ``out = tanh(alpha * x) * w + b`` element by element, with the
scalar ``alpha`` and the vectors ``w`` and ``b`` stored. It has an eps in no formula. Parameters: ``dim``, ``weight``,
``bias``, ``alpha`` (tensor names).

``add_normed`` is the norm applied to a sub-layer's OUTPUT on its way into the stream, for arrangements that norm
both sides of a sub-layer: ``x += RMSNorm(y) * w``, optionally with the next norm of the stream in the same pass.
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from .base import Norm, StepContext, TensorSpec, register_part


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    adds_owed = True
    leaves_row_scale = True

    def __init__(self, params):
        super().__init__(params)
        self.dim = int(params["dim"])
        self.eps = float(params["eps"])
        self.weight_name = params["weight"]
        self.one_plus = bool(params.get("one_plus", False))
        self.weight: torch.Tensor = None

    def tensors(self) -> List[TensorSpec]:
        init = ("normal", 0.1) if self.one_plus else ("one_plus_uniform", 0.1)
        return [TensorSpec(self.weight_name, (self.dim,), "vector", init)]

    def load(self, fetch, mode, device) -> None:
        self.weight = fetch(self.weight_name, "vector")
        if self.one_plus:
            self.weight = (self.weight.to(torch.float32) + 1.0).contiguous()

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                out_name: str = "norm.out", out_dtype: torch.dtype = None, lazy: bool = False) -> torch.Tensor:
        """``lazy``: the caller's consumer applies a row scale (``Block.normed``). If the product that ends the
        sub-layer before is still pending, it is launched here with an epilogue that adds it to ``x`` and leaves
        ``x * weight`` and the rows' sums of squares: the result lacks its ``1 / rms``, which the consumer's
        products apply (``ctx.row_scale_of``), and no norm kernel runs."""
        count = x.shape[0] if rows is None else rows.numel()
        out = ctx.scratch(out_name, (count, self.dim), out_dtype or ctx.act_dtype)
        if lazy and rows is None and out.dtype == torch.bfloat16 and self.dim % 16 == 0:
            pending = ctx.take_pending_product(x)
            if pending is not None:
                linear, rows_in = pending
                squares = ctx.scratch(out_name + ".squares", (count, self.dim // 16), torch.float32)
                linear.add_to_and_prepare_norm(rows_in, x, self.weight, out, squares)
                ctx.set_row_scale(out, kernels.RowScale(squares, self.dim, self.eps))
                return out
        ctx.set_row_scale(out, None)
        owed = ctx.take_owed(x)
        if owed is not None and rows is None:
            kernels.add_partials(x, owed, self.weight, self.eps, out)   # x += owed sums; out = norm(x), one pass
            return out
        if owed is not None:
            kernels.add_partials(x, owed)
        kernels.rms_norm(x, self.weight, self.eps, out, rows)
        return out

    def add_normed(self, ctx: StepContext, y, x: torch.Tensor, next_norm: "RMSNorm" = None,
                   out_name: str = "norm.out") -> Optional[torch.Tensor]:
        """``x += RMSNorm(y) * weight`` for a sub-layer's result ``y`` (float32 rows, planes of partial sums, or a
        routed feed-forward's parts still to be combined). With ``next_norm`` (another RMSNorm over the stream) the
        same kernel also leaves ``next_norm(x)`` of the updated rows and returns it."""
        ctx.settle()
        out = None
        if next_norm is not None:
            out = ctx.scratch(out_name, (x.shape[0], self.dim), ctx.act_dtype)
            ctx.set_row_scale(out, None)
        kernels.norm_add_norm(y, self.weight, self.eps, x, next_norm.weight if next_norm is not None else None,
                              next_norm.eps if next_norm is not None else 0.0, out)
        return out


@register_part("norm", "layer_norm")
class LayerNorm(Norm):
    capturable = True
    replayable = True

    def __init__(self, params):
        super().__init__(params)
        self.dim = int(params["dim"])
        self.eps = float(params["eps"])
        self.weight_name = params["weight"]
        self.weight: torch.Tensor = None

    def tensors(self) -> List[TensorSpec]:
        return [TensorSpec(self.weight_name, (self.dim,), "vector", ("one_plus_uniform", 0.1))]

    def load(self, fetch, mode, device) -> None:
        self.weight = fetch(self.weight_name, "vector")

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                out_name: str = "norm.out", out_dtype: torch.dtype = None) -> torch.Tensor:
        count = x.shape[0] if rows is None else rows.numel()
        out = ctx.scratch(out_name, (count, self.dim), out_dtype or ctx.act_dtype)
        ctx.set_row_scale(out, None)
        kernels.layer_norm(x, self.weight, self.eps, out, rows)
        return out


@register_part("norm", "dynamic_tanh")
class DynamicTanh(Norm):
    capturable = True
    replayable = True
    adds_owed = True       # the pass that reads the stream adds the partial sums still owed to it

    def __init__(self, params):
        super().__init__(params)
        self.dim = int(params["dim"])
        self.weight_name = params["weight"]
        self.bias_name = params["bias"]
        self.alpha_name = params["alpha"]
        self.weight: torch.Tensor = None
        self.bias: torch.Tensor = None
        self.alpha: torch.Tensor = None

    def tensors(self) -> List[TensorSpec]:
        return [TensorSpec(self.weight_name, (self.dim,), "vector", ("one_plus_uniform", 0.1)),
                TensorSpec(self.bias_name, (self.dim,), "vector", ("normal", 0.05)),
                TensorSpec(self.alpha_name, (1,), "vector", ("one_plus_uniform", 0.5))]   # a stored scalar reads as [1]

    def load(self, fetch, mode, device) -> None:
        self.weight = fetch(self.weight_name, "vector")
        self.bias = fetch(self.bias_name, "vector")
        self.alpha = fetch(self.alpha_name, "vector").reshape(1).contiguous()

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                out_name: str = "norm.out", out_dtype: torch.dtype = None) -> torch.Tensor:
        count = x.shape[0] if rows is None else rows.numel()
        out = ctx.scratch(out_name, (count, self.dim), out_dtype or ctx.act_dtype)
        ctx.set_row_scale(out, None)
        owed = ctx.take_owed(x)
        if owed is not None and rows is not None:
            kernels.add_partials(x, owed)
            owed = None
        kernels.dynamic_tanh(x, self.alpha, self.weight, self.bias, out, rows, owed)
        return out
