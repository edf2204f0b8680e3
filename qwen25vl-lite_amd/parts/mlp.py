"""SwiGLU feed-forward (reference src/qwen25vl_lite/text.py:56-66)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops.linear import gate_up_swiglu, linear_into
from .base import FeedForward, ParamSpec, StepContext, register_part

__all__ = ["SwiGLU", "ClampedGatedFF", "PlainFF"]


class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))`` without biases.

    params: ``hidden_size``, ``intermediate_size``, ``names`` (local names of the gate, up and down matrices;
    default ``gate_proj``, ``up_proj``, ``down_proj``).
    """

    graph_safe = True
    takes_lazy_norm = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        # gate and up rows alternate in groups of 8 where the size allows: a 16-row tile of the
        # product then holds 8 features' gate and up and can apply the activation itself
        self.grouped = self.inter % 8 == 0
        names = dict(params.get("names") or {})
        self.names = {k: names.get(k, f"{k}_proj") for k in ("gate", "up", "down")}
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {
            f"{self.names['gate']}.weight": ParamSpec((self.inter, self.hidden)),
            f"{self.names['up']}.weight": ParamSpec((self.inter, self.hidden)),
            f"{self.names['down']}.weight": ParamSpec((self.hidden, self.inter)),
        }

    def load(self, tensors):
        # gate and up share their input: one product of [2 I, H]
        gate, up = tensors[f"{self.names['gate']}.weight"], tensors[f"{self.names['up']}.weight"]
        if self.grouped:
            both = torch.stack([gate.view(-1, 8, self.hidden), up.view(-1, 8, self.hidden)], dim=1)
            self.w_gate_up = both.reshape(2 * self.inter, self.hidden).contiguous()
        else:
            self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = tensors[f"{self.names['down']}.weight"]

    def named_weights(self) -> Dict[str, torch.Tensor]:
        if self.grouped:
            both = self.w_gate_up.view(-1, 2, 8, self.hidden)
            gate, up = both[:, 0].reshape(self.inter, self.hidden), both[:, 1].reshape(self.inter, self.hidden)
        else:
            gate, up = self.w_gate_up[:self.inter], self.w_gate_up[self.inter:]
        return {f"{self.names['gate']}.weight": gate, f"{self.names['up']}.weight": up,
                f"{self.names['down']}.weight": self.w_down}

    def forward(self, x, step: StepContext):
        act = gate_up_swiglu(x, self.w_gate_up, self.grouped)
        return linear_into(step.residual if step is not None else None, act, self.w_down)


class ClampedGatedFF(FeedForward):
    """``down(g sigmoid(alpha g) (u + shift))`` with ``g = min(gate(x), limit)`` and
    ``u = clamp(up(x), -limit, limit)``, no biases.

    params: ``hidden_size``, ``intermediate_size``, ``alpha`` (default 1), ``limit`` (None: no
    clamps), ``shift`` (default 0), ``names`` (local names of the gate, up and down matrices;
    default ``gate_proj``, ``up_proj``, ``down_proj``).
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        self.alpha = float(params.get("alpha", 1.0))
        limit = params.get("limit")
        self.limit = None if limit is None else float(limit)
        if self.limit is not None and not self.limit > 0:
            raise ValueError("the clamp limit of a feed-forward must be positive")
        self.shift = float(params.get("shift", 0.0))
        names = dict(params.get("names") or {})
        self.names = {k: names.get(k, f"{k}_proj") for k in ("gate", "up", "down")}
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {
            f"{self.names['gate']}.weight": ParamSpec((self.inter, self.hidden)),
            f"{self.names['up']}.weight": ParamSpec((self.inter, self.hidden)),
            f"{self.names['down']}.weight": ParamSpec((self.hidden, self.inter)),
        }

    def load(self, tensors):
        # gate and up share their input: one product of [2 I, H], gate rows first
        self.w_gate_up = torch.cat([tensors[f"{self.names['gate']}.weight"], tensors[f"{self.names['up']}.weight"]],
                                   dim=0).contiguous()
        self.w_down = tensors[f"{self.names['down']}.weight"]

    def named_weights(self) -> Dict[str, torch.Tensor]:
        return {f"{self.names['gate']}.weight": self.w_gate_up[:self.inter],
                f"{self.names['up']}.weight": self.w_gate_up[self.inter:],
                f"{self.names['down']}.weight": self.w_down}

    def forward(self, x, step: StepContext):
        from ..ops.gated import gated_act
        from ..ops.linear import linear

        both = linear(x, self.w_gate_up)
        act = gated_act(both if both.is_contiguous() else both.contiguous(), self.alpha, self.limit, self.shift)
        return linear_into(step.residual if step is not None else None, act, self.w_down)


class PlainFF(FeedForward):
    """``down(act(up(x)))`` without gate or biases.

    params: ``hidden_size``, ``intermediate_size``, ``activation``: ``"relu2"`` (the square of relu) or
    ``"normed_powers"`` (``a N(z) + b N(z^2) + c N(z^3) + e`` with powers taken element by element and ``N`` dividing
    a token's row by its root mean square, ``eps`` inside the root; the four numbers are a tensor of the part),
    ``eps`` (for the normed powers), ``names`` (local names of the up and down matrices and the activation's
    tensor; default ``up_proj``, ``down_proj``, ``act``).
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        self.activation = str(params["activation"])
        if self.activation not in ("relu2", "normed_powers"):
            raise ValueError(f"activation {self.activation!r}; known: relu2, normed_powers")
        self.eps = float(params.get("eps", 0.0))
        names = dict(params.get("names") or {})
        self.names = {"up": names.get("up", "up_proj"), "down": names.get("down", "down_proj"), "act": names.get("act", "act")}
        self.w_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None
        self.coeff: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {f"{self.names['up']}.weight": ParamSpec((self.inter, self.hidden)),
                 f"{self.names['down']}.weight": ParamSpec((self.hidden, self.inter))}
        if self.activation == "normed_powers":
            specs[f"{self.names['act']}.weight"] = ParamSpec((4,), "vector", init="around_one")
        return specs

    def load(self, tensors):
        self.w_up = tensors[f"{self.names['up']}.weight"]
        self.w_down = tensors[f"{self.names['down']}.weight"]
        self.coeff = tensors.get(f"{self.names['act']}.weight")

    def named_weights(self) -> Dict[str, torch.Tensor]:
        out = {f"{self.names['up']}.weight": self.w_up, f"{self.names['down']}.weight": self.w_down}
        if self.coeff is not None:
            out[f"{self.names['act']}.weight"] = self.coeff
        return out

    def forward(self, x, step: StepContext):
        from ..ops import rownorm
        from ..ops.linear import linear

        z = linear(x, self.w_up)
        z = z if z.is_contiguous() else z.contiguous()
        if self.activation == "relu2":
            act = rownorm.squared_relu_(z)
        else:
            act = rownorm.normed_powers(z, self.coeff, self.eps, self.dtype)
        return linear_into(step.residual if step is not None else None, act, self.w_down)


register_part("ffn", "swiglu", SwiGLU)
register_part("ffn", "plain", PlainFF)
register_part("ffn", "clamped_gated", ClampedGatedFF)
