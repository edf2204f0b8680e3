"""A short causal convolution over time, channel by channel, added to its input."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops.short_conv import short_conv_add
from .base import Filter, LayerSlot, ParamSpec, StateNeed, StepContext, register_part

__all__ = ["ShortConvolution"]


class ShortConvolution(Filter):
    """``x_t + sum_j w[:, j] x_(t - taps + 1 + j)`` for the float32 residual rows ``x`` of each request, zeros
    before its first token.  The last ``taps - 1`` rows a request has brought are its state (float32
    ``[taps - 1, channels]``, oldest first), so that a sequence may be cut into steps anywhere.

    params: ``channels``, ``taps``.  The weight is ``[channels, taps]`` in a checkpoint and is kept in float32 as
    ``[taps, channels]``, so that neighbouring channels' weights of a tap lie side by side.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.channels = int(params["channels"])
        self.taps = int(params["taps"])
        if self.taps < 1:
            raise ValueError("a convolution has at least one tap")
        self.weight: Optional[torch.Tensor] = None

    def state_need(self) -> Optional[StateNeed]:
        return StateNeed((self.taps - 1, self.channels), torch.float32) if self.taps > 1 else None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.channels, self.taps), "vector")}

    def load(self, tensors):
        self.weight = tensors["weight"].t().contiguous()

    def named_weights(self) -> Dict[str, torch.Tensor]:
        return {"weight": self.weight.t()}

    def forward(self, h: torch.Tensor, step: StepContext, slot: Optional[LayerSlot]) -> torch.Tensor:
        state = slot.state if slot is not None else None
        if self.taps > 1 and state is None:
            raise RuntimeError("a convolution with more than one tap needs a state slot")
        return short_conv_add(h, self.weight, state, step.cu_q, step.req_slots, step.token_req, self.dtype)


register_part("filter", "short_conv", ShortConvolution)
