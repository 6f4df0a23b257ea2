"""Mixers whose memory is a state of fixed size per request instead of a cache of keys.

``decay_attention`` is a linear attention with a fixed decay per head and a gated, normed output:

    q, k = act(Wq h), act(Wk h)   (heads x key_dim)        v = act(Wv h)   (heads x value_dim)
    per head   S_t = decay[head] * S_(t-1) + k_t v_t^T ,   o_t = S_t^T q_t          (no other scale)
    y = Wo ( RMSNorm(o_t, all heads side by side; weight ``norm``) * sigmoid(Wg h) )

``min_gru`` is a gated recurrence whose gates read the current token only:

    z = sigmoid(Wz h + bz),   u = Wx h + bx,   candidate = u + 1/2 for u >= 0, sigmoid(u) below
    S_t = (1 - z) S_(t-1) + z * candidate   element by element,      y = Wo (S_t * silu(Wg h))

``gated_delta_rule`` keeps a matrix per value head and corrects it by what it already answers for the key:

    q, k = silu(conv(Wq h)), silu(conv(Wk h))   (kv_heads x key_dim)      v = silu(conv(Wv h))   (heads x value_dim)
    q, k <- x / sqrt(sum(x^2) + 1e-6) per head,  q also times key_dim^(-1/2);  head i reads q/k head i // (heads / kv_heads)
    beta = sigmoid(Wb h)  (one a head)     g = exp(-exp(A_log[head]) * softplus(Wa2 (Wa1 h) + dt_bias))  (heads x key_dim)
    per head   S <- diag(g) S ;  u = beta (v - S^T k) ;  S <- S + k u^T ;  o = S^T q        (S: key_dim x value_dim)
    y = Wo ( o / rms(o over value_dim) * norm * sigmoid(Wg2 (Wg1 h)) )

``conv`` is a short causal convolution over time per channel (weights ``[channels, taps]``, the last tap the current
token's); its last ``taps - 1`` inputs are a second state of the mixer, so it declares two needs. The two-step
projections (``a1``/``a2``, ``g1``/``g2``) run as one product each: the second over the block-diagonal of the two
matrices. Everything behind the products is float32. Parameters: ``hidden``, ``heads``, ``kv_heads``, ``key_dim``,
``value_dim``, ``conv``, ``eps``, ``names`` (``q``, ``k``, ``v``, ``b``, ``a1``, ``a2``, ``g1``, ``g2``, ``o``, ``A_log``,
``dt_bias``, ``norm``, ``q_conv``, ``k_conv``, ``v_conv``), ``low_rank`` (the inner size of the two-step projections
where random weights are made; a file's tensors say their own), ``output_scale`` (a factor on the result, folded into the
norm's weight).

All states start at zero (a slot is cleared when a request takes it), live in float32 whatever the compute mode,
and are carried from step to step in the request's state slot. The projections of a mixer run as one product; the
recurrences, their gates, activations and the norm are float32 on the product's float32 sums. Everything that
differs between steps is read on the device (``query_start``, ``state_slots``), so decode steps are recorded. A
step with a long prompt portion runs the recurrences chunk beside chunk (``kernels.scan_chunks``: three launches
instead of one token after the other in a handful of waves); such steps are never recorded.

Parameters. ``decay_attention``: ``hidden``, ``heads``, ``key_dim``, ``value_dim``, ``decay`` (one number a head),
``activation`` ("silu" or "none"), ``eps``, ``names`` (``q``, ``k``, ``v``, ``g``, ``o``, ``norm``).
``min_gru``: ``hidden``, ``width``, ``names`` (``z``, ``x``, ``g``, ``o``) and ``bias`` (``z``, ``x``).
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..cache.spec import FixedState
from ..errors import InvalidArgument
from .base import Mixer, StepContext, TensorSpec, register_part
from .linear import Linear


def _finish(ctx: StepContext, out: Linear, rows: torch.Tensor, residual: Optional[torch.Tensor], name: str):
    """The output projection: added to ``residual``, or (None) returned as float32 rows."""
    if residual is not None:
        out(rows, residual, accumulate=True, ctx=ctx)
        return None
    ctx.settle()
    result = ctx.scratch(name, (rows.shape[0], out.total_out), torch.float32)
    out(rows, result, accumulate=False, ctx=ctx)
    return result


@register_part("mixer", "decay_attention")
class DecayAttention(Mixer):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    takes_row_scale = True   # h goes into the one projection only, through Linear with the step context
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.heads = int(params["heads"])
        self.key_dim = int(params["key_dim"])
        self.value_dim = int(params.get("value_dim") or self.key_dim)
        self.decay_values = [float(d) for d in params["decay"]]
        self.activation = params.get("activation", "silu")
        self.eps = float(params["eps"])
        if len(self.decay_values) != self.heads:
            raise InvalidArgument(f"{self.heads} heads need {self.heads} decays, got {len(self.decay_values)}")
        if self.key_dim > kernels.DECAY_ATTENTION_MAX_DIM:
            raise InvalidArgument(f"a key size of {self.key_dim} exceeds {kernels.DECAY_ATTENTION_MAX_DIM}")
        names = params["names"]
        self.qk_width, self.v_width = self.heads * self.key_dim, self.heads * self.value_dim
        self.inputs = Linear([names["q"], names["k"], names["v"], names["g"]],
                             [self.qk_width, self.qk_width, self.v_width, self.v_width], self.hidden)
        self.out = Linear([names["o"]], [self.hidden], self.v_width)
        self.norm_name = names["norm"]
        self.norm_weight: torch.Tensor = None
        self.decay: torch.Tensor = None

    def cache_need(self):
        return FixedState((self.heads, self.key_dim, self.value_dim))

    def tensors(self) -> List[TensorSpec]:
        return self.inputs.tensors() + self.out.tensors() + \
            [TensorSpec(self.norm_name, (self.v_width,), "vector", ("one_plus_uniform", 0.1))]

    def load(self, fetch, mode, device) -> None:
        self.inputs.load(fetch)
        self.out.load(fetch)
        self.norm_weight = fetch(self.norm_name, "vector")
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32).to(device)

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        proj = ctx.scratch("decay_attention.proj", (T, self.inputs.total_out), torch.float32)
        self.inputs(h, proj, ctx=ctx)
        o = ctx.scratch("decay_attention.o", (T, self.v_width), torch.float32)
        kernels.decay_attention_scan(proj, o, cache.state, ctx.batch.query_start, cache.state_slots, self.decay,
                                     ctx.batch.num_seqs, self.heads, self.key_dim, self.value_dim, self.activation,
                                     chunks=kernels.scan_chunks(ctx.batch, ctx.device), scratch=ctx.scratch)
        gated = ctx.scratch("decay_attention.gated", (T, self.v_width))
        kernels.gated_rms_norm(o, self.norm_weight, self.eps, proj[:, 2 * self.qk_width + self.v_width:], gated)
        return _finish(ctx, self.out, gated, residual, "decay_attention.result")


@register_part("mixer", "min_gru")
class MinGru(Mixer):
    capturable = True
    takes_row_scale = True
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.width = int(params["width"])
        names = params["names"]
        bias = params.get("bias") or {}
        # The projection itself carries no bias: the recurrence kernel adds the vectors as it reads the sums, so the
        # product keeps its ways of running at decode sizes (planes of partial sums are not used here: the kernel
        # reads plain rows) and no pass over the rows is spent on the addition.
        self.inputs = Linear([names["z"], names["x"], names["g"]], [self.width] * 3, self.hidden)
        self.bias_names = [bias.get("z"), bias.get("x"), bias.get("g")] if bias else None
        self.bias: torch.Tensor = None
        self.out = Linear([names["o"]], [self.hidden], self.width)

    def cache_need(self):
        return FixedState((self.width,))

    def tensors(self) -> List[TensorSpec]:
        specs = self.inputs.tensors() + self.out.tensors()
        for name in self.bias_names or ():
            if name is not None:
                specs.append(TensorSpec(name, (self.width,), "vector", ("normal", 0.02)))
        return specs

    def load(self, fetch, mode, device) -> None:
        self.inputs.load(fetch)
        self.out.load(fetch)
        if self.bias_names is not None:
            self.bias = torch.cat([fetch(name, "vector").to(torch.float32) if name is not None else
                                   torch.zeros(self.width, dtype=torch.float32, device=device)
                                   for name in self.bias_names]).contiguous()

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        proj = ctx.scratch("min_gru.proj", (T, 3 * self.width), torch.float32)
        self.inputs(h, proj, ctx=ctx)
        rows = ctx.scratch("min_gru.rows", (T, self.width))
        kernels.min_gru_scan(proj, rows, cache.state, ctx.batch.query_start, cache.state_slots, ctx.batch.num_seqs,
                             self.width, chunks=kernels.scan_chunks(ctx.batch, ctx.device), scratch=ctx.scratch,
                             bias=self.bias)
        return _finish(ctx, self.out, rows, residual, "min_gru.result")


@register_part("mixer", "gated_delta_rule")
class GatedDeltaRule(Mixer):
    capturable = True
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.heads = int(params["heads"])
        self.kv_heads = int(params.get("kv_heads") or self.heads)
        self.key_dim = int(params["key_dim"])
        self.value_dim = int(params.get("value_dim") or self.key_dim)
        self.taps = int(params.get("conv") or 1)
        self.eps = float(params["eps"])
        self.output_scale = float(params.get("output_scale", 1.0))
        self.low_rank = int(params.get("low_rank") or 16)        # for random weights only: a file's own size counts
        if self.heads % self.kv_heads:
            raise InvalidArgument(f"{self.heads} value heads are no multiple of {self.kv_heads} query/key heads")
        if self.key_dim > kernels.DELTA_RULE_MAX_DIM:
            raise InvalidArgument(f"a key size of {self.key_dim} exceeds {kernels.DELTA_RULE_MAX_DIM}")
        if not 1 <= self.taps <= kernels.CONV_MAX_TAPS:
            raise InvalidArgument(f"a convolution of {self.taps} taps: 1 to {kernels.CONV_MAX_TAPS} are supported")
        n = self.names = dict(params["names"])
        self.qk_width, self.v_width = self.kv_heads * self.key_dim, self.heads * self.value_dim
        self.decay_width = self.heads * self.key_dim
        self.channels = 2 * self.qk_width + self.v_width          # what the convolution runs over
        self.inputs = Linear([n["q"], n["k"], n["v"], n["b"]],
                             [self.qk_width, self.qk_width, self.v_width, self.heads], self.hidden)
        self.low_ranks = None                                      # (rank of a1, rank of g1): from the stored shapes
        self.low: Linear = None
        self.second: Linear = None
        self.out = Linear([n["o"]], [self.hidden], self.v_width)
        self.conv_weight = self.A_log = self.dt_bias = self.norm_weight = None

    def cache_need(self):
        state = FixedState((self.heads, self.key_dim, self.value_dim))
        if self.taps > 1:
            return (state, FixedState((self.taps - 1, self.channels)))
        return state

    def tensors(self) -> List[TensorSpec]:
        n = self.names
        specs = self.inputs.tensors() + self.out.tensors()
        # The inner size of the two-step projections is whatever the file holds (None: any).
        specs += [TensorSpec(n["a1"], (None, self.hidden), "matrix", ("normal", 0.02), free_dims=(self.low_rank,)),
                  TensorSpec(n["a2"], (self.decay_width, None), "matrix", ("normal", 0.1), free_dims=(self.low_rank,)),
                  TensorSpec(n["g1"], (None, self.hidden), "matrix", ("normal", 0.02), free_dims=(self.low_rank,)),
                  TensorSpec(n["g2"], (self.v_width, None), "matrix", ("normal", 0.1), free_dims=(self.low_rank,))]
        specs += [TensorSpec(n["A_log"], (self.heads,), "vector", ("normal", 0.5)),
                  TensorSpec(n["dt_bias"], (self.decay_width,), "vector", ("normal", 0.5)),
                  TensorSpec(n["norm"], (self.value_dim,), "vector", ("one_plus_uniform", 0.1))]
        for key, width in (("q_conv", self.qk_width), ("k_conv", self.qk_width), ("v_conv", self.v_width)):
            specs.append(TensorSpec(n[key], (width, self.taps), "vector", ("normal", 0.4)))
        return specs

    def load(self, fetch, mode, device) -> None:
        n = self.names
        self.inputs.load(fetch)
        self.out.load(fetch)
        a1, a2, g1, g2 = (fetch(n[k], "matrix") for k in ("a1", "a2", "g1", "g2"))
        ra, rg = a1.shape[0], g1.shape[0]
        if a2.shape[1] != ra or g2.shape[1] != rg:
            raise InvalidArgument(f"{n['a2']} / {n['g2']} do not take what {n['a1']} / {n['g1']} give")
        self.low_ranks = (ra, rg)
        self.low = Linear([n["a1"], n["g1"]], [ra, rg], self.hidden)
        self.low.set_weight(torch.cat([a1, g1], dim=0).contiguous())
        both = a2.new_zeros((self.decay_width + self.v_width, ra + rg))
        both[:self.decay_width, :ra] = a2
        both[self.decay_width:, ra:] = g2
        self.second = Linear(["(a2 | g2)"], [self.decay_width + self.v_width], ra + rg)
        self.second.set_weight(both)
        self.conv_weight = torch.cat([fetch(n[k], "vector").to(torch.float32).reshape(-1, self.taps)
                                      for k in ("q_conv", "k_conv", "v_conv")]).contiguous()
        self.A_log = fetch(n["A_log"], "vector").to(torch.float32).contiguous()
        self.dt_bias = fetch(n["dt_bias"], "vector").to(torch.float32).contiguous()
        self.norm_weight = (fetch(n["norm"], "vector").to(torch.float32) * self.output_scale).contiguous()

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        state, conv_state = (cache[0], cache[1].state) if isinstance(cache, tuple) else (cache, None)
        proj = ctx.scratch("delta_rule.proj", (T, self.inputs.total_out), torch.float32)
        self.inputs(h, proj, ctx=ctx)
        low = ctx.scratch("delta_rule.low", (T, sum(self.low_ranks)))
        self.low(h, low, ctx=ctx)
        second = ctx.scratch("delta_rule.second", (T, self.decay_width + self.v_width), torch.float32)
        self.second(low, second)
        tok = ctx.scratch("delta_rule.tokens", (T, self.channels + self.heads + self.decay_width), torch.float32)
        kernels.delta_prepare(proj, self.conv_weight, self.taps, conv_state, ctx.batch, second[:, :self.decay_width],
                              self.A_log, self.dt_bias, self.kv_heads, self.heads, self.key_dim, self.value_dim, tok)
        if conv_state is not None and state.writes:
            kernels.conv_state_update(proj, self.taps, conv_state, ctx.batch, self.channels)
        o = ctx.scratch("delta_rule.o", (T, self.v_width), torch.float32)
        chunks = None
        if max(ctx.batch.host_new_tokens) >= kernels.DELTA_CHUNKS_FROM:      # such steps are never recorded
            chunks = kernels.scan_chunks(ctx.batch, ctx.device, rows=kernels.DELTA_CHUNK_ROWS)
        kernels.gated_delta_scan(tok, o, state.state, ctx.batch, self.kv_heads, self.heads, self.key_dim,
                                 self.value_dim, chunks=chunks, scratch=ctx.scratch)
        gated = ctx.scratch("delta_rule.gated", (T, self.v_width))
        kernels.grouped_gated_rms_norm(o, self.norm_weight, self.eps, second[:, self.decay_width:], gated, self.heads)
        return _finish(ctx, self.out, gated, residual, "delta_rule.result")
