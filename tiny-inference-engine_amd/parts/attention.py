"""Grouped-query attention over the paged cache.

In the reference's order (``src/model/qwen3.cpp:219-231``): q, k, v projections
without bias; per-head RMSNorm of q and k (one weight vector of length
head_dim shared by all heads, the layer's eps) BEFORE the rotation; rotate-half
rotary on q and k; k (normalised, rotated) and raw v written to the cache at
the step's slots; causal attention of every new row over its sequence's cached
keys with ``score = scale * q.k``, query head h reading KV head
``h // (num_heads // num_kv_heads)``; output projection, added to the residual.

Parameters (all from the spec, none assumed): ``hidden``, ``num_heads``,
``num_kv_heads``, ``head_dim``, ``scale``, ``window`` (None = all keys),
``qk_norm`` (None or ``{"eps", "q_weight", "k_weight"}``), ``position`` (a
PartSpec of the position family), ``names`` (``q``, ``k``, ``v``, ``o``) and, for
architectures whose projections have one, ``bias`` (names of bias vectors under ``q``,
``k``, ``v`` - all three or none - and/or ``o``; the reference has none).

Further parameters, for architectures that have them (absent or None: not applied):

* ``softcap`` c: scores become ``c * tanh(scale * q.k / c)`` before the softmax.
* ``value_dim``: the size of a value head where it differs from ``head_dim``. Keys and values then live in the
  cache, and run through the attention kernels, at one common size (the larger of the two, in steps of 16):
  at load time the q, k and v weights get zero rows and the o weight zero columns for the dimensions a head
  lacks. Zero dimensions add nothing to a score, and zero values give zero outputs that meet zero columns,
  so the arithmetic is unchanged. Such heads take no per-head norm and no rotation.
* ``value_mix`` ``{"role", "weight", "share"}``: values blended across layers. The layer with role ``"keep"``
  keeps its values of the step's tokens (float32, in step scratch memory named by ``share``); a layer with role
  ``"blend"`` caches and attends to ``(1 - lam) * v + lam * v_kept`` with ``lam`` the one-element tensor
  ``weight``. Both declare the weight tensor (a checkpoint stores one per layer); the keeper does not read it.
  Only values of the same token and the same step meet, so nothing of this lives in the cache. The blend happens
  in the kernel that writes keys and values into the cache.

* ``chunk`` n: instead of a sliding window, a query at position p sees the keys ``j <= p`` of its own chunk,
  ``floor(j / n) = floor(p / n)``, chunks counted from the sequence's position 0 (not from where a prompt was cut).
  The cache gives back the pages of chunks a request has left behind.
* ``keep_first`` f (beside a ``window``): a query also sees the keys of positions below f, at their true positions
  (for the rotation and for distances), however far back they lie; the cache keeps their pages to the request's end.
* ``sink`` (a tensor name, one float per query head): ``exp(sink[h])`` is one more term of head h's softmax
  denominator; it has no key and no value and is not scaled.
* ``values_are_keys``: there is no value projection; the values are the keys as projected (with their bias), before
  the per-head norm and the rotation. ``names`` then has no ``v`` and ``bias`` none for it.

* ``conv`` ``{"taps", "q", "k", "v"}`` (tensor names, each ``[channels, taps]``): a short causal convolution over time
  on every channel of the projected q, k and v, directly behind the projection (before norm and rotation):
  ``y_t = sum_j w[:, j] * u_(t - taps + 1 + j)``, zeros before the sequence's start. The last ``taps - 1`` projected
  rows of a sequence are a state of fixed size, so the mixer then declares two needs (pages, state).
* ``qk_norm`` with ``"over": "projection"``: q and k are RMS-normed over their whole projection at once (all heads
  together, weights of that size) instead of head by head.
* ``output_scale``: a factor on the mixer's result, folded into the convolution's value weights (float32) where there
  is a convolution and into the output projection's weight otherwise.

``forward(..., residual=None)`` returns the mixer's output (float32 rows, or planes of partial sums) instead of
adding it to a stream: for arrangements that norm a sub-layer's output first.
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..cache.spec import FixedState, PagedKV
from ..errors import InvalidArgument
from .base import Mixer, Part, PartSpec, StepContext, TensorSpec, build_part, register_part
from .linear import Linear


@register_part("mixer", "paged_attention")
class PagedAttention(Mixer):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    takes_row_scale = True   # h goes into the QKV projection only, through Linear with the step context
    returns_result = True    # forward(..., residual=None) returns the output instead of adding it

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        self.scale = float(params["scale"])
        self.window: Optional[int] = params.get("window")
        self.chunk: Optional[int] = int(params["chunk"]) if params.get("chunk") else None
        if self.window and self.chunk:
            raise InvalidArgument("attention takes a sliding window or causal chunks, not both")
        self.keep_first = int(params.get("keep_first") or 0)
        if self.keep_first < 0 or (self.keep_first and not self.window):
            raise InvalidArgument("first positions are kept beside a sliding window only")
        self.sink_name: Optional[str] = params.get("sink")
        self.sinks: torch.Tensor = None
        self.values_are_keys = bool(params.get("values_are_keys", False))
        self.softcap: Optional[float] = float(params["softcap"]) if params.get("softcap") else None
        # What the checkpoint stores per head (keys, values) and what the cache and the kernels run at.
        self.stored_key_dim = self.head_dim
        self.stored_value_dim = int(params.get("value_dim") or self.head_dim)
        # Heads of unequal or odd size always; heads that nothing rotates or norms also where a size in steps of
        # 16 opens the matrix-core kernels.
        self.qk_norm = params.get("qk_norm")
        self.norm_over_projection = bool(self.qk_norm) and self.qk_norm.get("over") == "projection"
        self.conv = dict(params["conv"]) if params.get("conv") else None
        self.taps = int(self.conv["taps"]) if self.conv else 1
        if self.conv and not 1 <= self.taps <= kernels.CONV_MAX_TAPS:
            raise InvalidArgument(f"a convolution of {self.taps} taps: 1 to {kernels.CONV_MAX_TAPS} are supported")
        self.output_scale = float(params.get("output_scale", 1.0))
        self.conv_weight: torch.Tensor = None
        plain_heads = not params.get("qk_norm") and (params.get("position") or PartSpec("none")).kind == "none" \
            and not params.get("bias")
        self.padded = self.stored_value_dim != self.stored_key_dim or self.head_dim % 2 != 0 or \
            (plain_heads and self.head_dim % 16 != 0)
        if self.padded:
            self.head_dim = -(-max(self.stored_key_dim, self.stored_value_dim) // 16) * 16
        kernels.check_attention_sizes(self.num_heads, self.num_kv_heads, self.head_dim)
        names = params["names"]
        q_dim, kv_dim = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        self.q_dim, self.kv_dim = q_dim, kv_dim
        self.value_mix = dict(params["value_mix"]) if params.get("value_mix") else None
        if self.value_mix is not None and self.value_mix.get("role") not in ("keep", "blend"):
            raise InvalidArgument("value_mix needs a role, 'keep' or 'blend'")
        self.value_mix_weight: torch.Tensor = None
        bias = params.get("bias") or {}
        inputs = "qk" if self.values_are_keys else "qkv"
        if any(k in bias for k in inputs) and not all(k in bias for k in inputs):
            raise InvalidArgument("the q, k and v projections run as one product: a bias for all of them or for none")
        if self.padded and bias:
            raise InvalidArgument("heads padded to a common size take no bias")
        if (self.conv or self.norm_over_projection) and (self.values_are_keys or bias or self.value_mix is not None):
            raise InvalidArgument("a convolution or a norm over the whole projection goes with plain q, k and v "
                                  "projections: no bias, no blended values, no values that are the keys")
        if self.values_are_keys and (self.padded or self.value_mix is not None or "v" in names or "v" in bias):
            raise InvalidArgument("values that are the keys have the keys' size, no projection of their own and no blend")
        stored = [self.num_heads * self.stored_key_dim, self.num_kv_heads * self.stored_key_dim,
                  self.num_kv_heads * self.stored_value_dim]
        sizes = stored if self.padded else [q_dim, kv_dim, kv_dim]
        # The projection's bias is added by the kernel that reads its sums (per-head norm, rotation, cache write), so
        # the product stays free to run as planes of partial sums at decode sizes; an encoding that is no rotation
        # table changes the rows in place first and keeps the bias in the product.
        position_spec: PartSpec = params.get("position") or PartSpec("none")
        self.bias_in_kernel = "q" in bias and build_part("position", position_spec).rotary_table() is not None
        self.qkv_bias_names = [bias[k] for k in inputs] if self.bias_in_kernel else None
        self.qkv_bias: torch.Tensor = None
        self.qkv = Linear([names[k] for k in inputs], sizes[:len(inputs)], self.hidden,
                          bias=[bias[k] for k in inputs] if "q" in bias and not self.bias_in_kernel else None)
        self.out = Linear([names["o"]], [self.hidden], self.num_heads * self.stored_value_dim if self.padded else q_dim,
                          bias=[bias["o"]] if "o" in bias else None)
        self.q_norm_weight: torch.Tensor = None
        self.k_norm_weight: torch.Tensor = None
        position: PartSpec = params.get("position") or PartSpec("none")
        self.position = build_part("position", position)
        if self.values_are_keys and self.position.rotary_table() is None:
            raise InvalidArgument("values that are the keys need a position encoding the fused kernel applies: any "
                                  "other changes the projected keys in place before they are cached as values")
        table = self.position.rotary_table()
        rotates_only = table is not None and int(table[1] or 0) <= self.stored_key_dim
        if self.padded and ((self.qk_norm and not self.norm_over_projection) or
                            (position.kind != "none" and not rotates_only)):
            raise InvalidArgument("heads whose key and value sizes differ take no per-head norm, and a rotation only "
                                  "of dimensions the stored keys have")

    def children(self) -> List[Part]:
        return [self.position]

    def cache_need(self):
        pages = PagedKV(self.num_kv_heads, self.head_dim, self.window, self.chunk, self.keep_first)
        if self.taps > 1:
            return (pages, FixedState((self.taps - 1, self.q_dim + 2 * self.kv_dim)))
        return pages

    def tensors(self) -> List[TensorSpec]:
        specs = self.qkv.tensors() + self.out.tensors()
        if self.qkv_bias_names is not None:
            specs += [TensorSpec(b, (o,), "vector", ("normal", 0.02))
                      for b, o in zip(self.qkv_bias_names, self.qkv.out_features)]
        if self.qk_norm:
            init = ("one_plus_uniform", 0.1)
            sizes = (self.num_heads * self.stored_key_dim, self.num_kv_heads * self.stored_key_dim) \
                if self.norm_over_projection else (self.head_dim, self.head_dim)
            specs.append(TensorSpec(self.qk_norm["q_weight"], (sizes[0],), "vector", init))
            specs.append(TensorSpec(self.qk_norm["k_weight"], (sizes[1],), "vector", init))
        if self.conv:
            for key, heads, width in (("q", self.num_heads, self.stored_key_dim),
                                      ("k", self.num_kv_heads, self.stored_key_dim),
                                      ("v", self.num_kv_heads, self.stored_value_dim)):
                specs.append(TensorSpec(self.conv[key], (heads * width, self.taps), "vector", ("normal", 0.4)))
        if self.value_mix is not None and self.value_mix.get("weight"):
            specs.append(TensorSpec(self.value_mix["weight"], (1,), "vector", ("normal", 0.3)))   # a stored scalar reads as [1]
        if self.sink_name:
            specs.append(TensorSpec(self.sink_name, (self.num_heads,), "vector", ("normal", 1.0)))
        return specs

    def _load_padded(self, fetch) -> None:
        """Zero rows (q, k, v) and zero columns (o) for the dimensions a stored head lacks of the common size."""
        def rows(name, heads, stored):
            w = fetch(name, "matrix")
            out = w.new_zeros((heads, self.head_dim, self.hidden))
            out[:, :stored] = w.view(heads, stored, self.hidden)
            return out.view(heads * self.head_dim, self.hidden)

        q, k, v = self.qkv.names
        parts = [rows(q, self.num_heads, self.stored_key_dim), rows(k, self.num_kv_heads, self.stored_key_dim),
                 rows(v, self.num_kv_heads, self.stored_value_dim)]
        self.qkv.set_weight(torch.cat(parts, dim=0).contiguous())
        w = fetch(self.out.names[0], "matrix")
        o = w.new_zeros((self.hidden, self.num_heads, self.head_dim))
        o[:, :, :self.stored_value_dim] = w.view(self.hidden, self.num_heads, self.stored_value_dim)
        self.out.set_weight(o.view(self.hidden, self.q_dim).contiguous())

    def _per_channel(self, t: torch.Tensor, heads: int, stored: int) -> torch.Tensor:
        """A stored per-channel tensor ``[heads * stored, ...]`` at the heads' common size (zeros for what a head lacks)."""
        t = t.to(torch.float32).reshape(heads, stored, -1)
        if stored != self.head_dim:
            wide = t.new_zeros((heads, self.head_dim, t.shape[2]))
            wide[:, :stored] = t
            t = wide
        return t.reshape(heads * self.head_dim, -1)

    def load(self, fetch, mode, device) -> None:
        if self.padded:
            self._load_padded(fetch)
        else:
            self.qkv.load(fetch)
            self.out.load(fetch)
        H, KVH = self.num_heads, self.num_kv_heads
        if self.conv:
            parts = [self._per_channel(fetch(self.conv["q"], "vector"), H, self.stored_key_dim),
                     self._per_channel(fetch(self.conv["k"], "vector"), KVH, self.stored_key_dim),
                     self._per_channel(fetch(self.conv["v"], "vector"), KVH, self.stored_value_dim) * self.output_scale]
            self.conv_weight = torch.cat(parts).contiguous()
        elif self.output_scale != 1.0:
            w = self.out.weight
            if isinstance(w, kernels.PackedWeight):
                raise InvalidArgument("an output scale without a convolution must be folded before the weight is packed")
            self.out.set_weight((w.to(torch.float32) * self.output_scale).to(w.dtype))
        if self.value_mix is not None and self.value_mix.get("weight"):
            weight = fetch(self.value_mix["weight"], "vector")
            self.value_mix_weight = weight.reshape(1).contiguous() if self.value_mix["role"] == "blend" else None
        if self.qk_norm:
            self.q_norm_weight = fetch(self.qk_norm["q_weight"], "vector")
            self.k_norm_weight = fetch(self.qk_norm["k_weight"], "vector")
            if self.norm_over_projection:
                self.q_norm_weight = self._per_channel(self.q_norm_weight, H, self.stored_key_dim).reshape(-1).contiguous()
                self.k_norm_weight = self._per_channel(self.k_norm_weight, KVH, self.stored_key_dim).reshape(-1).contiguous()
        if self.sink_name:
            self.sinks = fetch(self.sink_name, "vector").to(torch.float32).contiguous()
        if self.qkv_bias_names is not None:
            self.qkv_bias = torch.cat([fetch(b, "vector").to(torch.float32) for b in self.qkv_bias_names]).contiguous()

    def _finish(self, ctx: StepContext, attn: torch.Tensor, residual: Optional[torch.Tensor]):
        """The output projection: added to ``residual``, or (``residual`` None) returned for the caller to place."""
        if residual is not None:
            self.out(attn, residual, accumulate=True, ctx=ctx)
            return None
        ctx.settle()
        planes = self.out.partial_planes(ctx, attn, "attention.result_planes")
        if planes is not None:
            return planes
        result = ctx.scratch("attention.result", (attn.shape[0], self.hidden), torch.float32)
        self.out(attn, result, accumulate=False, ctx=ctx)
        return result

    def _unit_conv(self, device) -> torch.Tensor:
        """The weights of a convolution of one tap that changes nothing (a norm over the projection without one)."""
        if self.conv_weight is None:
            self.conv_weight = torch.ones((self.q_dim + 2 * self.kv_dim, 1), dtype=torch.float32, device=device)
        return self.conv_weight

    def _kernel_bias(self, writes: bool) -> Optional[torch.Tensor]:
        """The bias as the cache-write kernel takes it: of the columns it reads (q alone where it writes no keys)."""
        if self.qkv_bias is None:
            return None
        return self.qkv_bias if writes else self.qkv_bias[:self.q_dim]

    def _value_mix(self, ctx: StepContext, T: int):
        if self.value_mix is None:
            return None
        kept = ctx.scratch("attention.kept_values:" + str(self.value_mix.get("share", "")),
                           (T, self.num_kv_heads * self.stored_value_dim), torch.float32)
        if self.value_mix["role"] == "keep":
            return ("keep", kept)
        return ("blend", kept, self.value_mix_weight)

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        H, KVH, Dh = self.num_heads, self.num_kv_heads, self.head_dim
        conv_state = None
        if isinstance(cache, tuple):          # pages, and the convolution's last inputs
            cache, conv_state = cache[0], cache[1].state
        step = cache.step
        eps = float(self.qk_norm["eps"]) if self.qk_norm else 0.0
        q_weight, k_weight = (self.q_norm_weight, self.k_norm_weight) if self.qk_norm else (None, None)

        width = self.q_dim + (1 if self.values_are_keys else 2) * self.kv_dim
        q = ctx.scratch("attention.q", (T, self.q_dim))
        table = self.position.rotary_table()
        # Decode-size steps: the projection comes as planes of partial sums, added by the kernel that reads them.
        rows_first = self.conv is not None or self.norm_over_projection
        planes = self.qkv.partial_planes(ctx, h, "attention.qkv") if table is not None and not rows_first else None
        if planes is not None:
            qkv = planes[0]
        else:
            qkv = ctx.scratch("attention.qkv", (T, width), torch.float32)
            self.qkv(h, qkv, ctx=ctx)
        if rows_first:
            # The convolution over time (from the rows as projected and the sequence's state) and the norms over a
            # whole projection, one kernel; the kernels below then neither norm nor see the raw rows.
            raw, qkv = qkv, ctx.scratch("attention.qkv_conv", (T, width), torch.float32)
            kernels.conv_qkv(raw, self.conv_weight if self.conv else self._unit_conv(raw.device), self.taps, conv_state,
                             ctx.batch, (self.q_dim, self.kv_dim, self.kv_dim), qkv,
                             q_weight if self.norm_over_projection else None,
                             k_weight if self.norm_over_projection else None,
                             (H * self.stored_key_dim, KVH * self.stored_key_dim), eps)
            if conv_state is not None and cache.writes:
                kernels.conv_state_update(raw, self.taps, conv_state, ctx.batch, width)
            if self.norm_over_projection:
                q_weight = k_weight = None
        if table is not None:
            inv_freq, rotary_dim, pairing = table
            if (inv_freq is not None and not rows_first and rotary_dim == Dh and pairing == "rotate_half" and self.softcap is None
                    and self.value_mix is None and not self.values_are_keys and not self.chunk and self.sinks is None
                    and self.qkv_bias is None and not self.keep_first
                    and kernels.decode_attention_prepares(ctx.batch, q.dtype, cache.k_cache, H)):
                # A step of single decoded tokens: the attention kernel sums the planes, norms and rotates its own
                # queries and writes the newest keys and values itself: one kernel less.
                attn = ctx.scratch("attention.out", (T, self.q_dim))
                kernels.paged_attention_prepared(
                    planes if planes is not None else qkv.unsqueeze(0),
                    q_weight, k_weight, eps, self.position.angles(ctx), cache.writes, cache.k_cache, cache.v_cache, attn, step, ctx.batch,
                    H, self.scale, self.window, ctx.scratch)
                return self._finish(ctx, attn, residual)
            if inv_freq is None:                      # an encoding that leaves queries and keys as they are
                rotary_dim, pairing = None, "rotate_half"
            kernels.qk_norm_rope_kv_write(
                qkv, q, q_weight, k_weight, eps, inv_freq, ctx.batch.positions,
                step.slot_mapping, cache.k_cache, cache.v_cache, H, KVH, Dh, cache.block_size,
                write_kv=cache.writes, planes=1 if planes is None else planes.shape[0], plane_stride=T * width,
                angles=self.position.angles(ctx) if inv_freq is not None else None,
                rotary_dim=rotary_dim, pairing=pairing, value_mix=self._value_mix(ctx, T) if cache.writes else None,
                values_are_keys=self.values_are_keys, bias=self._kernel_bias(cache.writes))
        else:
            # A position encoding that is no rotation table: normalise in place, let the part
            # change q and k (float32 views into the projection rows), then convert and store.
            q_view = qkv[:, :self.q_dim]
            k_view = qkv[:, self.q_dim:self.q_dim + self.kv_dim]
            if q_weight is not None:
                kernels.qk_norm_rope_kv_write(
                    qkv, q_view, q_weight, k_weight, eps, None, ctx.batch.positions,
                    None, None, None, H, KVH, Dh, cache.block_size, write_kv=False, k_dense=k_view)
            self.position.apply(ctx, q_view.unflatten(1, (H, Dh)), k_view.unflatten(1, (KVH, Dh)),
                                ctx.batch.positions)
            kernels.qk_norm_rope_kv_write(
                qkv, q, None, None, 0.0, None, ctx.batch.positions, step.slot_mapping, cache.k_cache,
                cache.v_cache, H, KVH, Dh, cache.block_size, write_kv=cache.writes,
                value_mix=self._value_mix(ctx, T) if cache.writes else None, values_are_keys=self.values_are_keys)

        attn = ctx.scratch("attention.out", (T, self.q_dim))
        kernels.paged_attention(q, cache.k_cache, cache.v_cache, attn, step, ctx.batch, H, self.scale, self.window,
                                scratch=ctx.scratch, softcap=self.softcap, chunk=self.chunk, sinks=self.sinks,
                                keep_first=self.keep_first)
        return self._finish(ctx, attn, residual)
