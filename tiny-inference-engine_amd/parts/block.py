"""Arrangements of a layer's parts.

``pre_norm`` is the reference's block (``src/model/qwen3.cpp:216-239``):
``x += mixer(norm(x)); x += feed_forward(norm(x))`` with the norms named
``pre_mixer`` and ``pre_feed_forward`` in the layer's spec and nothing applied
to the sub-layer outputs. A layer that has only one of the two parts runs that
half alone (and needs that half's norm only).

``sandwich_norm`` norms both sides of each sub-layer: ``x += post_mixer(mixer(pre_mixer(x)))`` and then
``x += post_feed_forward(feed_forward(pre_feed_forward(x)))``. The sub-layers are asked for their result instead of
adding it (``forward(..., residual=None)``); the norm over the result, the addition to the stream and the norm
that the stream meets next run as one kernel where the norms can (``Norm.add_normed``).

``pre_norm_token_side`` is ``pre_norm`` followed by a third step that feeds every layer a vector of its own per
token: with ``e = table[token]`` restricted to the layer's ``dim`` columns (``first .. first + dim`` of a table all
layers share), ``g = gelu_tanh(W_gate x) * e`` from the stream itself (no norm before it), ``y = W_proj g`` and
``x += y / sqrt(mean(y^2) + eps) * w``. Parameters: ``hidden``, ``dim``, ``vocab``, ``table`` (tensor name),
``table_columns``, ``first``, ``eps``, ``names`` (``gate``, ``proj``, ``norm``).

``hyper_connections`` keeps ``streams`` copies of the residual instead of one. All start as the embedding's rows.
Sub-layer q of a layer (its mixer, then its feed-forward) has three small tensors ``in`` ``[streams]``, ``out``
``[streams]`` and ``mix`` ``[streams, streams]`` (from, to): it reads ``u = sum_s in[s] x_s``, computes
``y = sublayer(norm(u))``, and every stream becomes ``x_t <- sum_s mix[s, t] x_s + out[t] y``, all from the old
streams. The model's single residual row receives the sum of the streams behind every layer (what the head
norms, and what a layer hook sees). The streams live in step scratch memory: they never outlast a step. One
kernel does a sub-layer's write and the next sub-layer's read with its norm. Parameters: ``streams``, ``hidden``,
``names`` (``mixer`` and ``feed_forward``, each ``{"in", "out", "mix"}``).
"""

from __future__ import annotations

from typing import List

import torch

from .. import kernels
from ..errors import InvalidArgument
from .base import Block, StepContext, TensorSpec, register_part
from .linear import Linear


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    NORMS = ("pre_mixer", "pre_feed_forward")

    def forward(self, ctx: StepContext, x: torch.Tensor, layer, cache) -> None:
        if layer.mixer is not None:
            h = self.normed(ctx, layer.norms["pre_mixer"], x, consumer=layer.mixer)
            layer.mixer.forward(ctx, h, cache, x)
        if layer.feed_forward is not None:
            h = self.normed(ctx, layer.norms["pre_feed_forward"], x, consumer=layer.feed_forward)
            layer.feed_forward.forward(ctx, h, x)

    @classmethod
    def check_layer(cls, layer) -> None:
        needed = [n for n, part in zip(cls.NORMS, (layer.mixer, layer.feed_forward)) if part is not None]
        if not needed:
            raise InvalidArgument("a pre_norm block needs a mixer, a feed-forward or both")
        missing = [n for n in needed if n not in layer.norms]
        if missing:
            raise InvalidArgument(f"a pre_norm block needs the norms {', '.join(needed)}; missing {', '.join(missing)}")


@register_part("block", "pre_norm_token_side")
class TokenSideBlock(PreNormBlock):
    capturable = True
    replayable = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.dim = int(params["dim"])
        self.vocab = int(params["vocab"])
        self.table_name = params["table"]
        self.table_columns = int(params["table_columns"])
        self.first = int(params["first"])
        self.eps = float(params["eps"])
        if self.dim <= 0 or self.first < 0 or self.first + self.dim > self.table_columns:
            raise InvalidArgument(f"columns {self.first} .. {self.first + self.dim} do not lie in a per-token table of "
                                  f"{self.table_columns} columns")
        names = params["names"]
        self.gate = Linear([names["gate"]], [self.dim], self.hidden)
        self.proj = Linear([names["proj"]], [self.hidden], self.dim)
        self.norm_name = names["norm"]
        self.norm_weight: torch.Tensor = None
        self.table: torch.Tensor = None          # this layer's columns of the shared table, [vocab, dim]

    def tensors(self) -> List[TensorSpec]:
        return self.gate.tensors() + self.proj.tensors() + [
            TensorSpec(self.norm_name, (self.hidden,), "vector", ("one_plus_uniform", 0.1)),
            TensorSpec(self.table_name, (self.vocab, self.table_columns), "matrix", ("normal", 0.5))]

    def load(self, fetch, mode, device) -> None:
        self.gate.load(fetch)
        self.proj.load(fetch)
        self.norm_weight = fetch(self.norm_name, "vector")
        # a copy of the layer's own columns: a token's vector is then one piece of consecutive memory, and layers of
        # one shape differ in addresses only
        self.table = fetch(self.table_name, "matrix")[:, self.first:self.first + self.dim].contiguous()

    def forward(self, ctx: StepContext, x: torch.Tensor, layer, cache) -> None:
        super().forward(ctx, x, layer, cache)
        T = x.shape[0]
        if ctx.act_dtype == torch.float32:
            ctx.settle()
            rows = x
        else:
            # the stream in the products' type, in the pass that adds what the feed-forward still owes it
            ctx.run_late()
            owed = ctx.take_owed(x)
            rows = ctx.scratch("token_side.rows", (T, self.hidden), ctx.act_dtype)
            ctx.set_row_scale(rows, None)
            kernels.dynamic_tanh(x, None, None, None, rows, None, owed)
        gate = ctx.scratch("token_side.gate", (T, self.dim), torch.float32)
        self.gate(rows, gate, ctx=ctx)
        gated = ctx.scratch("token_side.gated", (T, self.dim), ctx.act_dtype)
        ctx.set_row_scale(gated, None)
        kernels.token_gate(gate, ctx.batch.tokens, self.table, 0, gated)
        y = self.proj.partial_planes(ctx, gated, "token_side.result_planes")
        if y is None:
            y = ctx.scratch("token_side.result", (T, self.hidden), torch.float32)
            self.proj(gated, y, ctx=ctx)
        kernels.norm_add_norm(y, self.norm_weight, self.eps, x)


@register_part("block", "sandwich_norm")
class SandwichNormBlock(Block):
    capturable = True
    replayable = True
    MIXER_NORMS = ("pre_mixer", "post_mixer")
    FEED_FORWARD_NORMS = ("pre_feed_forward", "post_feed_forward")

    @staticmethod
    def _result(ctx: StepContext, part, run):
        """The sub-layer's result: its own (``residual=None``), or for a part that can only add, what it adds to zeros."""
        if getattr(part, "returns_result", False):
            return run(None)
        zeros = ctx.scratch("block.sublayer_result", (ctx.num_tokens, part.hidden), torch.float32)
        zeros.zero_()
        run(zeros)
        ctx.settle()
        return zeros

    @staticmethod
    def _place(ctx: StepContext, post, y, x: torch.Tensor, following=None):
        if hasattr(post, "add_normed"):
            fused = following if isinstance(following, type(post)) else None
            h = post.add_normed(ctx, y, x, next_norm=fused)
            return h
        if not isinstance(y, torch.Tensor) or y.dim() != 2:
            raise InvalidArgument("this norm takes a sub-layer's result as plain rows only")
        x.add_(post.forward(ctx, y, out_name="norm.post", out_dtype=torch.float32))
        return None

    def forward(self, ctx: StepContext, x: torch.Tensor, layer, cache) -> None:
        norms = layer.norms
        h = None
        if layer.mixer is not None:
            h = self.normed(ctx, norms["pre_mixer"], x)
            y = self._result(ctx, layer.mixer, lambda residual: layer.mixer.forward(ctx, h, cache, residual))
            following = norms["pre_feed_forward"] if layer.feed_forward is not None else None
            h = self._place(ctx, norms["post_mixer"], y, x, following)
        if layer.feed_forward is not None:
            if h is None:
                h = self.normed(ctx, norms["pre_feed_forward"], x)
            rows = h
            y = self._result(ctx, layer.feed_forward, lambda residual: layer.feed_forward.forward(ctx, rows, residual))
            self._place(ctx, norms["post_feed_forward"], y, x)

    @classmethod
    def check_layer(cls, layer) -> None:
        needed = (cls.MIXER_NORMS if layer.mixer is not None else ()) + \
            (cls.FEED_FORWARD_NORMS if layer.feed_forward is not None else ())
        if not needed:
            raise InvalidArgument("a sandwich_norm block needs a mixer, a feed-forward or both")
        missing = [n for n in needed if n not in layer.norms]
        if missing:
            raise InvalidArgument(f"a sandwich_norm block needs the norms {', '.join(needed)}; missing {', '.join(missing)}")


@register_part("block", "hyper_connections")
class HyperConnectionsBlock(Block):
    capturable = True
    replayable = False     # the first block of a step makes the streams: what a layer launches depends on its place
    NORMS = ("pre_mixer", "pre_feed_forward")
    SUBLAYERS = ("mixer", "feed_forward")

    def __init__(self, params):
        super().__init__(params)
        self.streams = int(params["streams"])
        self.hidden = int(params["hidden"])
        if not 0 < self.streams <= kernels.HYPER_MAX_STREAMS:
            raise InvalidArgument(f"{self.streams} residual streams: 1 to {kernels.HYPER_MAX_STREAMS} are supported")
        self.names = {k: dict(v) for k, v in params["names"].items()}
        self.weights = {}

    def tensors(self) -> List[TensorSpec]:
        s, specs = self.streams, []
        for names in self.names.values():
            specs.append(TensorSpec(names["in"], (s,), "vector", ("normal", 0.5)))
            specs.append(TensorSpec(names["out"], (s,), "vector", ("one_plus_uniform", 0.2)))
            specs.append(TensorSpec(names["mix"], (s, s), "vector", ("normal", 0.4)))
        return specs

    def load(self, fetch, mode, device) -> None:
        for sub, names in self.names.items():
            self.weights[sub] = tuple(fetch(names[k], "vector").to(torch.float32).contiguous()
                                      for k in ("in", "out", "mix"))

    @classmethod
    def check_layer(cls, layer) -> None:
        needed = [n for n, part in zip(cls.NORMS, (layer.mixer, layer.feed_forward)) if part is not None]
        if not needed:
            raise InvalidArgument("a hyper_connections block needs a mixer, a feed-forward or both")
        missing = [n for n in needed if n not in layer.norms]
        missing += [s for s, part in zip(cls.SUBLAYERS, (layer.mixer, layer.feed_forward))
                    if part is not None and s not in layer.block.names]
        if missing:
            raise InvalidArgument(f"a hyper_connections block lacks {', '.join(missing)}")

    def _read(self, ctx: StepContext, sub: str, norm, T: int):
        """What the pass over the streams needs to also make the rows sub-layer ``sub`` reads: the kernel applies a
        layer norm or an RMS norm itself and hands any other norm the float32 sum."""
        kind = {"LayerNorm": "layer_norm", "RMSNorm": "rms_norm"}.get(type(norm).__name__)
        if kind is not None and hasattr(norm, "weight") and hasattr(norm, "eps"):
            h = ctx.scratch("hyper.normed", (T, self.hidden), ctx.act_dtype)
            ctx.set_row_scale(h, None)
            return (self.weights[sub][0], kind, norm.weight, norm.eps, h), h, None
        u = ctx.scratch("hyper.sum", (T, self.hidden), torch.float32)
        return (self.weights[sub][0], None, None, 0.0, u), None, u

    @staticmethod
    def _result(ctx: StepContext, part, run, T: int, hidden: int) -> torch.Tensor:
        """The sub-layer's result as float32 rows or planes of partial sums."""
        if getattr(part, "returns_result", False):
            y = run(None)
            ctx.settle()
            if isinstance(y, torch.Tensor):
                return y
            rows = ctx.scratch("hyper.sublayer_result", (T, hidden), torch.float32)
            kernels.moe_combine(y, rows)            # a routed feed-forward's parts
            return rows
        zeros = ctx.scratch("hyper.sublayer_result", (T, hidden), torch.float32)
        zeros.zero_()
        run(zeros)
        ctx.settle()
        return zeros

    def forward(self, ctx: StepContext, x: torch.Tensor, layer, cache) -> None:
        T = x.shape[0]
        # the layer before may have left its last write for this layer's first pass (same streams, same rows)
        left = ctx.take_late(("hyper.write", self.streams, T, self.hidden))
        ctx.settle()
        streams = ctx.scratch("hyper.streams", (self.streams, T, self.hidden), torch.float32)
        subs = [(s, part, layer.norms[n]) for s, n, part in
                zip(self.SUBLAYERS, self.NORMS, (layer.mixer, layer.feed_forward)) if part is not None]
        fresh = ctx.notes.get("hyper.streams") is None     # the first layer of the step: the streams are x
        ctx.notes["hyper.streams"] = streams
        read, h, u = self._read(ctx, subs[0][0], subs[0][2], T)
        if left is not None and not fresh:
            kernels.hyper_connection(streams, x, write=left, read=read)       # x is not needed in between
        else:
            if left is not None:
                kernels.hyper_connection(streams, x, fold=True, write=left)
            kernels.hyper_connection(streams, x, from_x=fresh, read=read)
        for i, (sub, part, norm) in enumerate(subs):
            if h is None:
                h = norm.forward(ctx, u)
            rows = h
            if sub == "mixer":
                y = self._result(ctx, part, lambda residual: part.forward(ctx, rows, cache, residual), T, self.hidden)
            else:
                y = self._result(ctx, part, lambda residual: part.forward(ctx, rows, residual), T, self.hidden)
            last = i + 1 == len(subs)
            read = h = u = None
            if not last:
                read, h, u = self._read(ctx, subs[i + 1][0], subs[i + 1][2], T)
            _, out_w, mix = self.weights[sub]
            if last:
                # left for the next layer's first pass; settle() (the model's end, a hook, another kind of block)
                # runs it with the fold of the streams' sum into x
                ctx.leave_late(("hyper.write", self.streams, T, self.hidden),
                               lambda write: kernels.hyper_connection(streams, x, fold=True, write=write),
                               (y, mix, out_w))
            else:
                kernels.hyper_connection(streams, x, write=(y, mix, out_w), read=read)
