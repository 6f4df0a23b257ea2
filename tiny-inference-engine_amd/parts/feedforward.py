"""Feed-forwards: the dense SwiGLU, a dense two-matrix one with an activation between, and a routed mixture.

SwiGLU:

``g = h @ Wg^T``, ``u = h @ Wu^T``, ``a = g / (1 + exp(-g)) * u`` evaluated left
to right, ``out = a @ Wd^T``, added to the residual; no bias, no experts
(``src/model/qwen3.cpp:235-239``, ``src/backend/cpu/cpu_backend.cpp:195-207``).
Gate and up run as one product over the two matrices side by side; with bfloat16 weights
their rows are interleaved in blocks of 8 and the product's epilogue applies the activation.
Parameters: ``hidden``, ``intermediate``, ``names`` (``gate``, ``up``, ``down``) and, for designs whose gate goes
through another function, ``activation``: ``silu`` (the default) or ``gelu_tanh``,
``0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))``.

``mlp`` is ``down(act(up(h)))`` without a gate; ``activation`` names the function (``gelu``: the exact form,
``0.5 z (1 + erf(z / sqrt 2))``; ``poly_norm``: ``a N(z) + b N(z^2) + c N(z^3) + e`` with powers taken element by
element, ``N(y) = y / sqrt(mean(y^2) + eps)`` over the row, and the four numbers a stored tensor, named by
``activation_weight``, with ``activation_eps``). Parameters: ``hidden``, ``intermediate``, ``activation``, ``names``
(``up``, ``down``).

``routed_experts`` is a mixture of SiLU-gated experts, ``down_e(silu(gate_e h) * (up_e h))``, of which every row
uses ``top``. The router is one matrix over all experts; its logits are float32 (bfloat16 operands, float32
sums). ``scoring`` ``softmax`` turns them into scores over all experts. The CHOICE looks at score + ``correction``
(a stored vector that steers the choice and nothing else): the experts form ``groups`` equal groups of
neighbours, a group scores its best member, only members of the ``keep_groups`` best groups stay eligible, and
the ``top`` best of those are chosen. The WEIGHTS are the scores of the chosen, as they are (``renormalize``
False). The last ``identity_experts`` router outputs are experts without weights that return their input. The
result is the weighted sum of the chosen experts' results. Parameters: ``hidden``, ``expert_intermediate``,
``experts``, ``identity_experts``, ``top``, ``groups``, ``keep_groups``, ``scoring``, ``renormalize``, ``names``
(``router``, ``correction`` or None, and lists ``gate``, ``up``, ``down`` with one name an expert).

For designs that have them: ``scoring`` ``sigmoid`` (scores are ``sigmoid(logits)`` expert by expert);
``group_top`` n (a group scores the sum of its n best members instead of its best); ``renormalize`` True (the
weights are the chosen scores divided by their sum + ``renorm_eps``); ``weight_scale`` (a factor on the weights);
``expert_activation`` ``relu_squared`` with no ``gate`` names (experts without a gate, ``down_e(relu(up_e h)^2)``);
``shared`` ``{"intermediate", "up", "down", "gate_logit"}`` (and ``"gate"`` for gated experts): one more expert of the
same form that every row uses, its result multiplied by ``sigmoid(w_gate_logit . h)``, one number a row. It runs as
pieces of the routed experts' size among them (further experts that every row chooses, all with that weight), so
the same launches carry it; its gate's logit is one more column of the router's product.

Nothing of a step is read on the host: the rows are sorted by expert on the device and the experts' products
run over a tile list that lives there (``kernels.moe_align``), so routed layers are recorded and replayed like
dense ones.

Every feed-forward here returns its result instead of adding it when ``residual`` is None.
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..errors import InvalidArgument, UnsupportedError
from .base import FeedForward, StepContext, TensorSpec, register_part
from .linear import Linear


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    takes_row_scale = True   # h goes into the gate/up product only
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.intermediate = int(params["intermediate"])
        self.activation = params.get("activation") or "silu"
        if self.activation not in kernels.GATE_ACTIVATIONS:
            raise UnsupportedError(f"a gate's activation '{self.activation}' (supported: "
                                   f"{', '.join(kernels.GATE_ACTIVATIONS)})")
        names = params["names"]
        self.gate_up = Linear([names["gate"], names["up"]], [self.intermediate, self.intermediate], self.hidden)
        self.down = Linear([names["down"]], [self.hidden], self.intermediate)

    def tensors(self) -> List[TensorSpec]:
        return self.gate_up.tensors() + self.down.tensors()

    def load(self, fetch, mode, device) -> None:
        self.down.load(fetch)
        gate, up = fetch(self.gate_up.names[0], "matrix"), fetch(self.gate_up.names[1], "matrix")
        # bfloat16 weights and widths in steps of 8: gate and up rows are interleaved so that one
        # product computes both and its epilogue applies silu(gate) * up before anything is stored.
        self.fused = gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16 and \
            self.intermediate % 8 == 0 and self.hidden % 8 == 0
        if self.fused:
            self.gate_up.set_weight(kernels.interleave_gate_up(gate, up))
        else:
            self.gate_up.load(fetch)

    def forward(self, ctx: StepContext, h: torch.Tensor, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        act = ctx.scratch("swiglu.act", (T, self.intermediate))
        if self.fused and h.dtype == torch.bfloat16:
            kernels.linear_swiglu(h, self.gate_up.weight, act, row_scale=Linear.row_scale_for(ctx, h, self.gate_up.weight),
                                  activation=self.activation)
        else:
            gate_up = ctx.scratch("swiglu.gate_up", (T, 2 * self.intermediate))
            self.gate_up(h, gate_up, ctx=ctx)
            kernels.swiglu(gate_up, act, self.activation)
        return _finish(ctx, self.down, act, residual, "feed_forward.result")


def _finish(ctx: StepContext, down: Linear, act: torch.Tensor, residual: Optional[torch.Tensor], name: str):
    """The last product of a feed-forward: added to ``residual``, or (None) returned as rows or planes of partial sums."""
    if residual is not None:
        down(act, residual, accumulate=True, ctx=ctx)
        return None
    ctx.settle()
    planes = down.partial_planes(ctx, act, name + "_planes")
    if planes is not None:
        return planes
    result = ctx.scratch(name, (act.shape[0], down.total_out), torch.float32)
    down(act, result, accumulate=False, ctx=ctx)
    return result


@register_part("feed_forward", "mlp")
class Mlp(FeedForward):
    capturable = True
    replayable = True
    returns_result = True
    ACTIVATIONS = ("gelu", "poly_norm")

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.intermediate = int(params["intermediate"])
        self.activation = params.get("activation", "gelu")
        if self.activation not in self.ACTIVATIONS:
            raise UnsupportedError(f"activation '{self.activation}' (supported: {', '.join(self.ACTIVATIONS)})")
        self.activation_weight_name = params.get("activation_weight")
        self.activation_eps = float(params.get("activation_eps") or 0.0)
        self.activation_weight: torch.Tensor = None
        if self.activation == "poly_norm" and not self.activation_weight_name:
            raise InvalidArgument("the poly_norm activation needs the name of its four coefficients")
        names = params["names"]
        self.up = Linear([names["up"]], [self.intermediate], self.hidden)
        self.down = Linear([names["down"]], [self.hidden], self.intermediate)

    def tensors(self) -> List[TensorSpec]:
        specs = self.up.tensors() + self.down.tensors()
        if self.activation == "poly_norm":
            specs.append(TensorSpec(self.activation_weight_name, (4,), "vector", ("normal", 0.5)))
        return specs

    def load(self, fetch, mode, device) -> None:
        self.up.load(fetch)
        self.down.load(fetch)
        if self.activation == "poly_norm":
            self.activation_weight = fetch(self.activation_weight_name, "vector").to(torch.float32).contiguous()

    def forward(self, ctx: StepContext, h: torch.Tensor, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        pre = ctx.scratch("mlp.pre", (T, self.intermediate), torch.float32)     # the activation reads float32 sums
        self.up(h, pre, ctx=ctx)
        act = ctx.scratch("mlp.act", (T, self.intermediate))
        if self.activation == "poly_norm":
            kernels.poly_norm(pre, self.activation_weight, self.activation_eps, act)
        else:
            kernels.gelu(pre, act)
        return _finish(ctx, self.down, act, residual, "feed_forward.result")


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    capturable = True
    replayable = True
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.intermediate = int(params["expert_intermediate"])
        self.experts = int(params["experts"])
        self.identity = int(params.get("identity_experts") or 0)
        self.outputs = self.experts + self.identity
        self.top = int(params["top"])
        self.groups = int(params.get("groups") or 1)
        self.keep_groups = int(params.get("keep_groups") or self.groups)
        self.scoring = params.get("scoring") or "softmax"
        if self.scoring not in ("softmax", "sigmoid"):
            raise UnsupportedError(f"router scoring '{self.scoring}' (supported: softmax, sigmoid)")
        self.group_top = int(params.get("group_top") or 1)
        self.renormalize = bool(params.get("renormalize"))
        self.renorm_eps = float(params.get("renorm_eps") or 0.0)
        self.weight_scale = float(params.get("weight_scale") if params.get("weight_scale") is not None else 1.0)
        names = params["names"]
        self.gated = bool(names.get("gate"))
        self.activation = params.get("expert_activation") or ("silu" if self.gated else "relu_squared")
        if (self.gated and self.activation != "silu") or (not self.gated and self.activation != "relu_squared"):
            raise UnsupportedError(f"experts {'with' if self.gated else 'without'} a gate and the activation "
                                   f"'{self.activation}' (supported: silu with a gate, relu_squared without)")
        if self.experts <= 0 or self.identity < 0 or self.outputs > kernels.MOE_MAX_EXPERTS:
            raise InvalidArgument(f"a routed feed-forward takes 1 to {kernels.MOE_MAX_EXPERTS} experts, got "
                                  f"{self.experts} + {self.identity}")
        if self.outputs % self.groups or not 0 < self.keep_groups <= self.groups or \
                not 0 < self.top <= self.keep_groups * (self.outputs // self.groups) or \
                not 0 < self.group_top <= kernels.MOE_MAX_GROUP_TOP:
            raise InvalidArgument(f"{self.outputs} experts in {self.groups} groups scored by their {self.group_top} "
                                  f"best, {self.keep_groups} kept, top {self.top}: no such choice")
        for key in ("gate", "up", "down") if self.gated else ("up", "down"):
            if len(names[key]) != self.experts:
                raise InvalidArgument(f"a routed feed-forward needs one '{key}' tensor name per expert")
        self.names = names
        # The expert every row uses, cut into pieces of the routed experts' size that sit behind them.
        self.shared = dict(params["shared"]) if params.get("shared") else None
        self.shared_intermediate = int(self.shared["intermediate"]) if self.shared else 0
        self.shared_pieces = -(-self.shared_intermediate // self.intermediate) if self.shared else 0
        if self.shared:
            if self.identity:
                raise InvalidArgument("a shared expert beside experts that return their input is not supported")
            if self.shared_intermediate <= 0 or self.experts + self.shared_pieces > kernels.MOE_MAX_EXPERTS:
                raise InvalidArgument(f"a shared expert of inner size {self.shared_intermediate} does not fit")
            router_names, router_sizes = [names["router"], self.shared["gate_logit"]], [self.outputs, 1]
        else:
            router_names, router_sizes = [names["router"]], [self.outputs]
        self.router = Linear(router_names, router_sizes, self.hidden)
        self.correction: torch.Tensor = None
        self.gate: torch.Tensor = None        # [experts (+ shared pieces), intermediate, hidden]
        self.up: torch.Tensor = None
        self.down: torch.Tensor = None        # [experts (+ shared pieces), hidden, intermediate]

    def tensors(self) -> List[TensorSpec]:
        specs = self.router.tensors()
        if self.names.get("correction"):
            specs.append(TensorSpec(self.names["correction"], (self.outputs,), "vector", ("normal", 0.02)))
        inner = ("gate", "up") if self.gated else ("up",)
        for e in range(self.experts):
            for key in inner:
                specs.append(TensorSpec(self.names[key][e], (self.intermediate, self.hidden), "matrix", ("normal", 0.02)))
            specs.append(TensorSpec(self.names["down"][e], (self.hidden, self.intermediate), "matrix", ("normal", 0.02)))
        if self.shared:
            for key in inner:
                specs.append(TensorSpec(self.shared[key], (self.shared_intermediate, self.hidden), "matrix", ("normal", 0.02)))
            specs.append(TensorSpec(self.shared["down"], (self.hidden, self.shared_intermediate), "matrix", ("normal", 0.02)))
        return specs

    def load(self, fetch, mode, device) -> None:
        self.router.load(fetch)
        if self.names.get("correction"):
            self.correction = fetch(self.names["correction"], "vector")
        F_, pieces = self.intermediate, self.shared_pieces

        def stack(key, inner_rows: bool):
            parts = [fetch(n, "matrix") for n in self.names[key]]
            if self.shared:
                w = fetch(self.shared[key], "matrix")
                # zero rows of an up (or gate) matrix give zero activations; they meet zero columns of the down matrix
                wide = w.new_zeros((pieces * F_, self.hidden) if inner_rows else (self.hidden, pieces * F_))
                if inner_rows:
                    wide[:self.shared_intermediate] = w
                    parts += list(wide.view(pieces, F_, self.hidden).unbind(0))
                else:
                    wide[:, :self.shared_intermediate] = w
                    parts += list(wide.view(self.hidden, pieces, F_).unbind(1))
            if len({p.dtype for p in parts}) > 1:
                parts = [p.to(torch.float32) for p in parts]
            return torch.stack(parts).contiguous()

        self.gate = stack("gate", True) if self.gated else None
        self.up, self.down = stack("up", True), stack("down", False)

    def forward(self, ctx: StepContext, h: torch.Tensor, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        slots, real = self.top + self.shared_pieces, self.experts + self.shared_pieces
        logits = ctx.scratch("moe.logits", (T, self.router.total_out), torch.float32)
        self.router(h, logits, ctx=ctx)
        ids = ctx.scratch("moe.ids", (T, slots), torch.int32)
        weights = ctx.scratch("moe.weights", (T, slots), torch.float32)
        kernels.moe_route(logits, self.correction, self.groups, self.keep_groups, self.top, ids, weights,
                          scoring=self.scoring, group_top=self.group_top, renormalize=self.renormalize,
                          renorm_eps=self.renorm_eps, weight_scale=self.weight_scale, shared=self.shared_pieces)
        tile_rows = kernels.moe_tile_rows(h.dtype, self.up.dtype, self.hidden, self.intermediate, T * slots, real)
        rows = kernels.moe_align(ids, real, tile_rows, ctx.scratch)
        act = ctx.scratch("moe.act", (T * slots, self.intermediate))
        kernels.moe_gate_up(h, self.gate, self.up, rows, act)
        parts = ctx.scratch("moe.parts", (T * slots, self.hidden), torch.float32)
        kernels.moe_down(act, self.down, rows, parts)
        routed = kernels.RoutedParts(parts, rows.where, weights, h)
        if residual is None:
            return routed
        ctx.settle()
        kernels.moe_combine(routed, residual, accumulate=True)
        return None
