"""Gated linear attention: a recurrence per head instead of a cache of keys.

Per head a state ``S [head_dim, v_head_dim]`` in fp32 lives in the request's state slot:
``S <- diag(a_t) S + k_t v_t^T``, ``o_t = S^T q_t`` with ``q`` scaled by ``head_dim^-1/2`` and a decay
per key channel ``a_t = sigmoid(z_t)^(1/tau)``, ``z = W_a2 (W_a1 x) + b`` (a projection through a
narrow middle).  Each head's output is RMS-normed (one weight for all heads), multiplied by
``silu(W_g x)`` and projected.  The recurrence runs token by token in fp32
(``csrc/recurrence.hip``): what it gives for a token does not depend on how the prompt was cut (beyond
rounding where a step brings hundreds of tokens of a sequence, which are scanned in chunks side by side).

Options: ``dim``, ``n_heads``, ``head_dim``, ``v_head_dim``, ``tau``, ``decay_rank``, ``eps``.
"""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, streamed
from .base import MATRIX, VECTOR, LayerStore, Mixer, StateNeed, TensorSpec, place, register_part


class GatedLinearAttention(Mixer):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.dim = int(o["dim"])
        self.n_heads = int(o["n_heads"])
        self.head_dim = int(o["head_dim"])
        self.v_head_dim = int(o["v_head_dim"])
        self.tau = float(o["tau"])
        self.decay_rank = int(o["decay_rank"])
        self.eps = float(o["eps"])
        if self.head_dim > 512 or self.v_head_dim > 1024:
            raise ValueError(f"{self.prefix}: heads of {self.head_dim} x {self.v_head_dim} are not supported"
                             " (at most 512 key channels and 1024 value channels)")
        if not self.tau > 0:
            raise ValueError(f"{self.prefix}: tau must be positive")
        self.w_in: Optional[StreamedMatrix] = None
        self.w_a2: Optional[StreamedMatrix] = None
        self.wo: Optional[StreamedMatrix] = None
        self.a2_bias = self.norm_w = None

    def tensor_specs(self) -> List[TensorSpec]:
        H, d, e, low = self.n_heads, self.head_dim, self.v_head_dim, self.decay_rank
        return [
            TensorSpec(self._name("q_proj.weight"), (H * d, self.dim)), TensorSpec(self._name("k_proj.weight"), (H * d, self.dim)),
            TensorSpec(self._name("v_proj.weight"), (H * e, self.dim)), TensorSpec(self._name("gate_proj.weight"), (H * e, self.dim)),
            TensorSpec(self._name("o_proj.weight"), (self.dim, H * e)),
            TensorSpec(self._name("out_norm.weight"), (e,), VECTOR, ("one_plus_normal", 0.01)),
            TensorSpec(self._name("decay_down.weight"), (low, self.dim)),
            TensorSpec(self._name("decay_up.weight"), (H * d, low)),
            TensorSpec(self._name("decay_up.bias"), (H * d,), VECTOR, ("one_plus_normal", 0.5)),
        ]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        t = lambda name: tensors[self._name(name)]
        f32 = lambda name: t(name).to(device=device, dtype=torch.float32).contiguous()
        # one matrix for everything that reads the mixer's input: q, k, v, the output gate, the decay's narrow middle
        mats = [t("q_proj.weight"), t("k_proj.weight"), t("v_proj.weight"), t("gate_proj.weight"), t("decay_down.weight")]
        self.w_in = streamed(place(torch.cat(mats, dim=0), MATRIX, dtype, device))
        self.w_a2 = streamed(place(t("decay_up.weight"), MATRIX, dtype, device))
        self.wo = streamed(place(t("o_proj.weight"), MATRIX, dtype, device))
        self.a2_bias, self.norm_w = f32("decay_up.bias"), f32("out_norm.weight")

    def state_need(self) -> StateNeed:
        return StateNeed((self.n_heads, self.head_dim, self.v_head_dim), torch.float32)

    def forward(self, x: torch.Tensor, ctx: Any, store: LayerStore) -> torch.Tensor:
        H, d, e, low = self.n_heads, self.head_dim, self.v_head_dim, self.decay_rank
        T = x.shape[0]
        k_col, v_col, g_col, a_col = H * d, 2 * H * d, 2 * H * d + H * e, 2 * H * d + 2 * H * e
        rows = linear(x, self.w_in)  # [T, q | k | v | gate | narrow]
        z = linear(rows[:, a_col : a_col + low], self.w_a2, out_dtype=torch.float32)
        o = torch.empty((T, H * e), dtype=torch.float32, device=x.device)
        ops.decay_scan(rows, 0, k_col, v_col, z, self.a2_bias, self.tau, d ** -0.5, store.state, ctx.slot_ids,
                       ctx.q_start, ctx.n_seqs, o, q_start_host=None if ctx.graph_capacity else ctx.q_start_host)
        out = torch.empty((T, H * e), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(o, self.norm_w, self.eps, rows[:, g_col:], H, out)
        return linear(out, self.wo, partials_ok=True)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
