"""Short causal convolutions over time that carry their last inputs from step to step."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .. import ops
from ..weights.loader import VECTOR, TensorSpec
from .base import CONVS, Part, PartSpec, StateNeed
from .context import StateCacheView, StepContext


@CONVS.register("causal_conv")
class CausalConv(Part):
    """out[t, c] = (x[t, c] if ``add_input``) + sum_j w[c, j] * x[t - (taps - 1) + j, c], then ``activation``:
    one filter of ``taps`` taps per channel, the last tap on the current token, zeros before a sequence's
    start, no bias.  A request's last ``taps - 1`` inputs are its state (float32), so that a portion cut
    anywhere, or a single decoded token, continues where the last step ended.

    Parameters: ``channels``, ``taps``, ``weights`` (tensor names, each ``[its channels, taps]``, laid side by
    side along the channels: projections that were fused into one product are convolved in one launch),
    ``add_input`` (the residual form x + conv(x)), ``activation`` (None, "silu", "sigmoid").
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        self.taps = int(spec["taps"])
        self.names: Sequence[str] = list(spec["weights"])
        self.widths: Sequence[int] = [int(c) for c in spec["channels"]] if isinstance(spec["channels"], (list, tuple)) \
            else [int(spec["channels"])]
        if len(self.names) != len(self.widths):
            raise ValueError("a causal convolution needs one channel count per weight")
        if self.taps < 2:
            raise ValueError(f"a causal convolution needs at least 2 taps, found {self.taps}")
        self.channels = sum(self.widths)
        self.add_input = bool(spec.get("add_input", False))
        self.activation = spec.get("activation")
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(name, (width, self.taps), VECTOR) for name, width in zip(self.names, self.widths)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        parts = [tensors.pop(name) for name in self.names]
        if len({p.dtype for p in parts}) > 1:
            parts = [p.float() for p in parts]
        self.weight = torch.cat(parts, dim=0).contiguous()

    def cache_need(self) -> StateNeed:
        return StateNeed((self.taps - 1, self.channels), torch.float32)

    def forward(self, x: torch.Tensor, step: StepContext, cache: StateCacheView, out_dtype: torch.dtype) -> torch.Tensor:
        """``x`` ``[rows, channels]`` (may be a column slice of wider rows) -> ``[rows, channels]`` in ``out_dtype``."""
        return ops.causal_conv(x, self.weight, cache.state, step, out_dtype, add_input=self.add_input,
                               activation=self.activation, write_state=cache.writes)
