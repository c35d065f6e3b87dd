"""Grouped-query causal attention over the paged cache.

Per step (``fastgen/forward.py:421-472``): one product for q, k and v (the
three projections are stored as one matrix), rotation of q and k and the
write of k, v into the pages in one launch, attention of every new token
over all cached keys of its request, output projection.

Options beyond the reference's layer: ``value_from_key`` (there is no value
projection: a token's value is its key as projected, before the rotation),
``output_gate`` (the heads' outputs are multiplied by ``sigmoid(W_g x)`` before
the output projection; ``W_g`` rides in the same product as q and k),
``exact_weights`` (the softmax weights enter the product with the values in
more than bfloat16's digits), ``bias`` (q, k and v have biases, added in fp32
where the product's fp32 result is read), ``qk_norm`` (an RMS norm per head on
q and on k, one weight for all heads, before any rotation), ``sink`` (a learned
number per head whose exponential is one more term of the softmax's
denominator), ``v_head_dim`` (values of another width than keys: the cache
holds both padded with zeros to one width), ``has_kv`` = False (a layer that
reads another layer's keys and values has only its queries), ``cache_window``
(how long the cache keeps a key, where later layers read this layer's cache
through longer windows than its own).
"""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, skinny_ok, streamed
from .base import LayerStore, Mixer, PagedNeed, TensorSpec, build_part, place, register_part, MATRIX, VECTOR


class Attention(Mixer):
    folds_norms = True  # takes ScaledRows and the ``then`` request (see parts.block)

    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.dim = int(o["dim"])
        self.n_heads = int(o["n_heads"])
        self.n_kv_heads = int(o["n_kv_heads"])
        self.head_dim = int(o["head_dim"])
        self.scale = float(o.get("scale", self.head_dim**-0.5))
        self.window: Optional[int] = o.get("window") or None
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"n_heads={self.n_heads} is not a multiple of n_kv_heads={self.n_kv_heads}")
        if self.head_dim % 8 or self.head_dim > 512:
            raise ValueError(
                f"{self.prefix}: head size {self.head_dim} is not supported: the cache and the attention"
                " kernels work in chunks of 8 head dimensions, up to 512"
            )
        self.value_from_key = bool(o.get("value_from_key", False))
        self.output_gate = bool(o.get("output_gate", False))
        self.exact_weights = bool(o.get("exact_weights", False))
        self.bias = bool(o.get("bias", False))
        self.qk_norm = bool(o.get("qk_norm", False))
        self.qk_norm_eps = float(o.get("qk_norm_eps", 1e-6))
        self.sink = bool(o.get("sink", False))
        self.has_kv = bool(o.get("has_kv", True))
        self.v_head_dim = int(o.get("v_head_dim") or self.head_dim)
        self.cache_window: Optional[int] = o.get("cache_window", self.window) or None
        # the width of a head in the cache: keys and values of different widths are padded with zeros to one
        # width, a multiple of 16 (what the matrix-core kernels take)
        # the general form: what the product gives goes through a kernel of its own on its way to the attention
        self.prepared = self.bias or self.qk_norm or not self.has_kv or self.v_head_dim != self.head_dim
        self.cache_dim = -(-max(self.head_dim, self.v_head_dim) // 16) * 16 if self.prepared else self.head_dim
        if self.prepared and (self.value_from_key or self.output_gate):
            raise ValueError(f"{self.prefix}: value_from_key and output_gate do not go with bias, qk_norm, v_head_dim or has_kv")
        if self.v_head_dim % 2 or self.cache_dim > 512:
            raise ValueError(f"{self.prefix}: value size {self.v_head_dim} is not supported (even, at most 512)")
        self.position = build_part("position", o["position"])
        self.b_qkv = self.q_norm_w = self.k_norm_w = self.sinks = None
        self.wqkv: Optional[StreamedMatrix] = None
        self.wo: Optional[StreamedMatrix] = None
        self.freqs: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        q, kv = self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim
        vw = self.n_kv_heads * self.v_head_dim
        specs = [TensorSpec(self._name("q_proj.weight"), (q, self.dim))]
        if self.has_kv:
            specs.append(TensorSpec(self._name("k_proj.weight"), (kv, self.dim)))
            if not self.value_from_key:
                specs.append(TensorSpec(self._name("v_proj.weight"), (vw, self.dim)))
        if self.output_gate:
            specs.append(TensorSpec(self._name("gate_proj.weight"), (q, self.dim)))
        if self.bias:
            specs.append(TensorSpec(self._name("q_proj.bias"), (q,), VECTOR))
            if self.has_kv:
                specs += [TensorSpec(self._name("k_proj.bias"), (kv,), VECTOR),
                          TensorSpec(self._name("v_proj.bias"), (vw,), VECTOR)]
        if self.qk_norm:
            specs.append(TensorSpec(self._name("q_norm.weight"), (self.head_dim,), VECTOR, ("one_plus_normal", 0.01)))
            if self.has_kv:
                specs.append(TensorSpec(self._name("k_norm.weight"), (self.head_dim,), VECTOR, ("one_plus_normal", 0.01)))
        if self.sink:
            specs.append(TensorSpec(self._name("sinks"), (self.n_heads,), VECTOR, ("normal", 1.0)))
        return specs + [TensorSpec(self._name("o_proj.weight"), (self.dim, self.n_heads * self.v_head_dim))]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        # one matrix for everything that reads the mixer's input: q, k, then v (if it has a projection
        # of its own), then the output gate
        f32 = lambda name: tensors[self._name(name)].to(device=device, dtype=torch.float32).contiguous()
        mats = [self.position.arrange_rows(tensors[self._name("q_proj.weight")], self.n_heads)]
        if self.has_kv:
            mats.append(self.position.arrange_rows(tensors[self._name("k_proj.weight")], self.n_kv_heads))
            if not self.value_from_key:
                mats.append(tensors[self._name("v_proj.weight")])
        if self.output_gate:
            mats.append(tensors[self._name("gate_proj.weight")])
        self.wqkv = streamed(place(torch.cat(mats, dim=0), MATRIX, dtype, device))
        wo = tensors[self._name("o_proj.weight")]
        if self.cache_dim != self.v_head_dim:
            # the attention's output rows hold heads of the cache's width: zero columns meet the padding
            wide = wo.new_zeros(self.dim, self.n_heads, self.cache_dim)
            wide[:, :, : self.v_head_dim] = wo.view(self.dim, self.n_heads, self.v_head_dim)
            wo = wide.view(self.dim, self.n_heads * self.cache_dim)
        self.wo = streamed(place(wo, MATRIX, dtype, device))
        self.freqs = self.position.frequencies_on(device)
        if self.bias:
            names = ["q_proj.bias"] + (["k_proj.bias", "v_proj.bias"] if self.has_kv else [])
            if self.position.rotary_dim and getattr(self.position, "pairing", "") == "half":
                raise ValueError(f"{self.prefix}: biases with rows rearranged for the rotation are not supported")
            self.b_qkv = torch.cat([f32(n) for n in names])
        if self.qk_norm:
            self.q_norm_w = f32("q_norm.weight")
            self.k_norm_w = f32("k_norm.weight") if self.has_kv else None
        if self.sink:
            self.sinks = f32("sinks")

    def paged_need(self) -> PagedNeed:
        return PagedNeed(self.n_kv_heads, self.cache_dim, self.cache_window)

    def forward(self, x, ctx: Any, store: LayerStore, then=None):
        """``x``: the normed rows, or ``ScaledRows`` (a norm not yet finished, which the q/k/v product
        finishes).  ``then``: a norm's ``fold_request``; the output projection may fold the addition
        to the residual stream and that norm into its kernel and return ``ScaledRows``."""
        if self.prepared:
            return self._forward_prepared(x, ctx, store, then)
        group = ctx.groups[store.group]
        q_width = self.n_heads * self.head_dim
        kv_width = self.n_kv_heads * self.head_dim
        # columns of the product: q, k, v (or none: the values are the k columns), gate
        v_col = q_width if self.value_from_key else q_width + kv_width
        gate_col = v_col + kv_width
        table = None
        if self.freqs is not None:
            # sin and cos of the step's positions: computed by the first layer, shared by all layers
            # that rotate with the same frequencies
            key = ("rope_table", self.freqs.data_ptr())
            table = ctx.scratch.get(key)
            if table is None:
                table = ctx.scratch[key] = ops.rope_table(ctx.positions, self.freqs)
        rows = x.rows if isinstance(x, ops.ScaledRows) else x
        fused = store.owns and self.head_dim % 16 == 0 and skinny_ok(rows, self.wqkv)
        if not fused and rows is not x:
            x = x.materialize()
        if fused:
            # few rows (decode): rotation and cache write happen where the product is stored
            qkv = ops.gemm_skinny_qkv(x, self.wqkv.streaming, table, group.slots, store.k_pages, store.v_pages, self.n_heads,
                                      self.n_kv_heads, self.head_dim, self.position.rotary_dim,
                                      value_from_key=self.value_from_key, gate=self.output_gate)
            gate = qkv[:, q_width:] if self.output_gate else None  # sigmoid applied where it was stored
            gate_done = True
        else:
            # an entry that reads another entry's cache needs its queries only (and its gate)
            own_rows = self.wqkv if store.owns or self.output_gate else self.wqkv.first_rows(q_width)
            qkv = linear(x, own_rows)
            ops.rope_kv_write(
                qkv, ctx.positions, self.freqs, group.slots, store.k_pages, store.v_pages,
                self.n_heads, self.n_kv_heads, self.head_dim, self.position.rotary_dim, write_kv=store.owns,
                table=table, v_col=v_col,
            )
            gate = qkv[:, gate_col:] if self.output_gate else None
            gate_done = False
        out = torch.empty((rows.shape[0], q_width), dtype=rows.dtype, device=rows.device)
        ops.paged_attention(qkv, out, store.k_pages, store.v_pages, group, ctx, self.n_heads, self.scale,
                            self.window or 0, exact_weights=self.exact_weights, sinks=self.sinks)
        if gate is not None:
            ops.gate_mul(out, gate, sigmoid=not gate_done)
        return linear(out, self.wo, partials_ok=True, residual=then)

    def _rope_table(self, ctx: Any):
        if self.freqs is None:
            return None
        key = ("rope_table", self.freqs.data_ptr())
        table = ctx.scratch.get(key)
        if table is None:
            table = ctx.scratch[key] = ops.rope_table(ctx.positions, self.freqs)
        return table

    def _forward_prepared(self, x, ctx: Any, store: LayerStore, then=None):
        """The general form: the product's fp32 rows go through ``heads_prepare`` (bias, the norms per
        head, rotation, padding to the cache's head width, cache write), then attention and output
        projection."""
        if isinstance(x, ops.ScaledRows):
            x = x.materialize()
        group = ctx.groups[store.group]
        d, hc = self.head_dim, self.cache_dim
        q_width, kv_width = self.n_heads * d, self.n_kv_heads * d
        rows = linear(x, self.wqkv, out_dtype=torch.float32)
        q = torch.empty((x.shape[0], self.n_heads * hc), dtype=x.dtype, device=x.device)
        writes = store.owns and self.has_kv
        ops.heads_prepare(
            rows, self.b_qkv, self.qk_norm_eps, n_q=self.n_heads, q_col=0, q_width=d, q_norm=self.q_norm_w,
            q_norm_dims=d if self.qk_norm else 0, q_out=q, q_out_width=hc,
            n_kv=self.n_kv_heads if writes else 0, k_col=q_width, k_width=d, k_norm=self.k_norm_w,
            k_norm_dims=d if self.qk_norm else 0, v_col=q_width + kv_width, v_width=self.v_head_dim,
            table=self._rope_table(ctx), rot_start=0, rotary_dim=self.position.rotary_dim,
            slots=group.slots if writes else None, k_pages=store.k_pages if writes else None,
            v_pages=store.v_pages if writes else None)
        out = torch.empty_like(q)
        ops.paged_attention(q, out, store.k_pages, store.v_pages, group, ctx, self.n_heads, self.scale,
                            self.window or 0, exact_weights=self.exact_weights, sinks=self.sinks)
        return linear(out, self.wo, partials_ok=True)


register_part("mixer", "attention", Attention)
