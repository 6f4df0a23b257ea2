"""Attention over a cached latent: a token leaves one small vector and one rotated key part for all heads.

    q = Wq h              per head [dim unrotated | rot_dim rotated]; or, with ``q_rank``, through a latent of their
                          own: c_q = RMSnorm(Wdq h) (weight ``dq_norm``), q = Wuq c_q
    Wdkv h                [kv_rank | rot_dim]: the first part RMS-normed (weight ``dkv_norm``) is the latent c, the
                          second, rotated by position, is the one rotated key part all heads share
    head h:  key = [Wuk[h] c | rotated part],  value = Wuv[h] c
             score = (q_unrotated . Wuk[h] c + q_rotated . k_rotated) * scale
    softmax over the window (or all keys), with exp(sink[h]) as one more term of the denominator where sinks exist
    y = Wo (heads side by side * sigmoid(Wg h))            (the gate only where ``g`` is named)

What is cached is c and the rotated key part, nothing per head. The scores need no key per head either:
``q_unrotated . Wuk[h] c = (Wuk[h]^T q_unrotated) . c``, so the query's unrotated part goes through ``Wuk[h]^T`` once
and attention runs with ALL heads over ONE key/value head ``[c | rotated part]`` whose values are the latents; ``Wuv[h]``
is applied to the attention's output, which is linear in the values. The cache is an ordinary paged group of one
head of size kv_rank + rot_dim (rounded up to a multiple of 16), so windows, sinks, page tables and all three attention
kernels are the ones every other attention here uses. Prompt portions and decoded tokens run the same arithmetic.

Parameters: ``hidden``, ``num_heads``, ``head_dim`` (unrotated), ``rope_dim``, ``value_dim``, ``kv_rank``, ``scale``,
``window`` (None: all keys), ``sink`` (tensor name or None), ``eps``, ``position`` (a PartSpec of the position family
that describes a rotation table over ``rope_dim``), ``names`` (``q``, ``dkv``, ``dkv_norm``, ``uk``, ``uv``, ``o`` and
optionally ``g``; with ``q_rank`` ``dq``, ``dq_norm`` and ``uq`` instead of ``q``), ``output_scale`` (a factor on the
result, folded into the latent-to-value matrices).
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..cache.spec import PagedKV
from ..errors import InvalidArgument
from .base import Mixer, Part, PartSpec, StepContext, TensorSpec, build_part, register_part
from .linear import Linear


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    capturable = True
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.num_heads = int(params["num_heads"])
        self.dim = int(params["head_dim"])
        self.rope_dim = int(params["rope_dim"])
        self.value_dim = int(params.get("value_dim") or self.dim)
        self.kv_rank = int(params["kv_rank"])
        self.scale = float(params["scale"])
        self.window: Optional[int] = params.get("window")
        self.eps = float(params["eps"])
        self.output_scale = float(params.get("output_scale", 1.0))
        self.sink_name: Optional[str] = params.get("sink")
        self.sinks: torch.Tensor = None
        # the one cached head: [latent | rotated key part], in steps of 16 for the matrix-core kernels
        self.cache_dim = -(-(self.kv_rank + self.rope_dim) // 16) * 16
        kernels.check_attention_sizes(self.num_heads, 1, self.cache_dim)
        names = dict(params["names"])
        self.names = names
        H = self.num_heads
        self.q_width = H * (self.dim + self.rope_dim)
        self.latent_width = self.kv_rank + self.rope_dim
        self.gated = bool(names.get("g"))
        self.q_rank = int(params.get("q_rank") or 0)
        first, first_width = (names["dq"], self.q_rank) if self.q_rank else (names["q"], self.q_width)
        self.first_width = first_width
        inputs = [first, names["dkv"]] + ([names["g"]] if self.gated else [])
        sizes = [first_width, self.latent_width] + ([H * self.value_dim] if self.gated else [])
        self.inputs = Linear(inputs, sizes, self.hidden)
        self.q_up = Linear([names["uq"]], [self.q_width], self.q_rank) if self.q_rank else None
        self.q_norm: torch.Tensor = None
        self.out = Linear([names["o"]], [self.hidden], H * self.value_dim)
        self.position = build_part("position", params.get("position") or PartSpec("none"))
        table = self.position.rotary_table()
        if table is None:
            raise InvalidArgument("a latent attention takes a position encoding that is a rotation table (or none)")
        self.rotary_dim = int(table[1]) if table[0] is not None or table[1] else 0
        self.pairing = table[2] if self.rotary_dim else "rotate_half"
        if self.rotary_dim > self.rope_dim:
            raise InvalidArgument(f"{self.rotary_dim} rotated dimensions do not fit a rotated part of {self.rope_dim}")
        self.latent_norm: torch.Tensor = None
        self.uk_t: torch.Tensor = None       # [H, kv_rank, dim]: the unrotated query part -> the latent's space
        self.uv: torch.Tensor = None         # [H, value_dim, kv_rank]: the attended latent -> the head's value

    def children(self) -> List[Part]:
        return [self.position]

    def cache_need(self):
        return PagedKV(1, self.cache_dim, self.window)

    def tensors(self) -> List[TensorSpec]:
        H, n = self.num_heads, self.names
        specs = self.inputs.tensors() + self.out.tensors()
        if self.q_rank:
            specs += self.q_up.tensors()
            specs.append(TensorSpec(n["dq_norm"], (self.q_rank,), "vector", ("one_plus_uniform", 0.1)))
        specs.append(TensorSpec(n["dkv_norm"], (self.kv_rank,), "vector", ("one_plus_uniform", 0.1)))
        specs.append(TensorSpec(n["uk"], (H * self.dim, self.kv_rank), "matrix", ("normal", 0.05)))
        specs.append(TensorSpec(n["uv"], (H * self.value_dim, self.kv_rank), "matrix", ("normal", 0.05)))
        if self.sink_name:
            specs.append(TensorSpec(self.sink_name, (H,), "vector", ("normal", 1.0)))
        return specs

    def load(self, fetch, mode, device) -> None:
        H = self.num_heads
        self.inputs.load(fetch)
        self.out.load(fetch)
        self.latent_norm = fetch(self.names["dkv_norm"], "vector")
        if self.q_rank:
            self.q_up.load(fetch)
            self.q_norm = fetch(self.names["dq_norm"], "vector")
        uk = fetch(self.names["uk"], "matrix")
        self.uk_t = uk.view(H, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        uv = fetch(self.names["uv"], "matrix").view(H, self.value_dim, self.kv_rank)
        if self.output_scale != 1.0:
            uv = (uv.to(torch.float32) * self.output_scale).to(uv.dtype)
        self.uv = uv.contiguous()
        if self.sink_name:
            self.sinks = fetch(self.sink_name, "vector").to(torch.float32).contiguous()

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: Optional[torch.Tensor]):
        T, H, D = h.shape[0], self.num_heads, self.cache_dim
        proj = ctx.scratch("latent.proj", (T, self.inputs.total_out), torch.float32)
        self.inputs(h, proj, ctx=ctx)
        q_plain = ctx.scratch("latent.q_plain", (T, H * self.dim))
        q_latent = ctx.scratch("latent.q", (T, H * D))
        step = cache.step
        queries, latent_rows = proj, None
        if self.q_rank:
            # the queries' own latent: normed out of the first columns, then taken up to the heads
            c_q = ctx.scratch("latent.c_q", (T, self.q_rank))
            ctx.set_row_scale(c_q, None)
            kernels.rms_norm_columns(proj[:, :self.q_rank], self.q_norm, self.eps, c_q)
            queries = ctx.scratch("latent.queries", (T, self.q_width), torch.float32)
            self.q_up(c_q, queries, ctx=ctx)
            latent_rows = proj[:, self.q_rank:]
        kernels.latent_prepare(queries, self.latent_norm, self.eps,
                               self.position.angles(ctx) if self.rotary_dim else None, self.rotary_dim, self.pairing,
                               step.slot_mapping, cache.k_cache, cache.v_cache, cache.block_size, cache.writes,
                               q_plain, q_latent, H, self.dim, self.rope_dim, self.kv_rank, latent_rows=latent_rows)
        q_heads = q_latent.view(T, H, D)
        kernels.head_linear(q_plain.view(T, H, self.dim), self.uk_t, q_heads[:, :, :self.kv_rank])
        attn = ctx.scratch("latent.attended", (T, H * D))
        kernels.paged_attention(q_latent, cache.k_cache, cache.v_cache, attn, step, ctx.batch, H, self.scale,
                                self.window, scratch=ctx.scratch, sinks=self.sinks)
        heads = ctx.scratch("latent.heads", (T, H * self.value_dim))
        gate = proj[:, self.first_width + self.latent_width:].unflatten(1, (H, self.value_dim)) if self.gated else None
        kernels.head_linear(attn.view(T, H, D)[:, :, :self.kv_rank], self.uv, heads.view(T, H, self.value_dim), gate)
        if residual is not None:
            self.out(heads, residual, accumulate=True, ctx=ctx)
            return None
        ctx.settle()
        planes = self.out.partial_planes(ctx, heads, "latent.result_planes")
        if planes is not None:
            return planes
        result = ctx.scratch("latent.result", (T, self.hidden), torch.float32)
        self.out(heads, result, accumulate=False, ctx=ctx)
        return result
