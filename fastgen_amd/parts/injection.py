"""Parts that add to the residual stream between layers."""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from .base import VECTOR, Injection, TensorSpec, register_part


class LoopInput(Injection):
    """What enters the stream at the start of each pass of a looped stretch of layers: before every
    pass but the first the embedding's output is added again, and before every pass row ``t`` of a
    table ``[times, dim]``, ``t`` the number of the pass.  The sums are fp32, in that order."""

    needs_embedding = True

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.dim = int(spec.options["dim"])
        self.times = int(spec.options["times"])
        self.step: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self._name("step"), (self.times, self.dim), VECTOR, ("normal", 0.5))]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        # the rows are added to the fp32 stream: kept in fp32 (exact for values stored in bfloat16)
        self.step = tensors[self._name("step")].to(device=device, dtype=torch.float32).contiguous()

    def forward(self, h, pending, embedded, index: int) -> None:
        ops.stream_add(h, pending, embedded if index > 0 else None, self.step[index])


register_part("injection", "loop_input", LoopInput)
