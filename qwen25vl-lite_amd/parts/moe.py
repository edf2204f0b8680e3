"""A feed-forward made of many small experts of which every token uses a few, plus an optional
expert that every token uses.

The router's logits ``z = x Wr^T`` (``+ b`` for a router with a bias) are float32 sums.  Scores ``s`` are ``sigmoid(z)`` (or a softmax
over the experts).  Experts ``e`` with the same ``e // (E / groups)`` are one group, ranked by the sum of its
top two scores; the ``top`` experts with the highest scores are picked among the members of the
``keep`` highest-ranked groups.  A token's result is ``sum_k w_k expert_k(x)`` with ``w`` the chosen scores over
their sum, times ``scale``, plus ``shared(x)``.  Every expert is
``down(g sigmoid(alpha g) (u + shift))`` with ``g = min(gate(x), limit)``, ``u = clamp(up(x), +-limit)``.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import moe as moe_ops
from ..ops.linear import linear
from .base import FeedForward, ParamSpec, Part, PartSpec, StepContext, build_part, register_part

__all__ = ["RoutedExperts"]

FLOAT32_PAIRS = 512     # up to this many (token, expert) pairs the experts' results stay float32 until they are summed


class RoutedExperts(FeedForward):
    """params: ``hidden_size``, ``num_experts``, ``top``, ``intermediate_size`` (of one expert),
    ``alpha`` (default 1), ``limit`` (None: no clamps), ``shift`` (default 0), ``groups`` and ``keep``
    (default 1 and 1: no groups), ``scale`` (default 1), ``score`` (``"sigmoid"`` or ``"softmax"``),
    ``normalize`` (default True), ``floor`` (added to the sum the weights are divided by, default 1e-20),
    ``shared`` (a :class:`PartSpec` of category ``ffn`` that every token runs through, or None),
    ``expert_kind`` (``"gated"``, the default, or ``"plain"``: an expert is ``down(act(up(x)))`` with ``activation``
    ``"relu2"``, the square of relu, and has no gate matrix), ``router_bias`` (True: the router has a bias of
    ``[experts]``, added to the logits in float32), ``names``
    (``router``, ``expert`` with ``{}`` for the index, ``gate``, ``up``, ``down``, ``shared``; defaults
    ``router``, ``experts.{}``, ``gate_proj``, ``up_proj``, ``down_proj``, ``shared``).

    The experts' matrices are kept stacked: ``[E, 2 ff, hidden]`` (gate rows, then up rows) and
    ``[E, hidden, ff]``.  A step lists its (token, choice) pairs by expert on the device and runs
    two products over that list; no count ever comes to the host.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.experts = int(params["num_experts"])
        self.top = int(params["top"])
        self.inter = int(params["intermediate_size"])
        self.alpha = float(params.get("alpha", 1.0))
        limit = params.get("limit")
        self.limit = None if limit is None else float(limit)
        self.shift = float(params.get("shift", 0.0))
        self.groups = int(params.get("groups", 1))
        self.keep = int(params.get("keep", self.groups))
        self.scale = float(params.get("scale", 1.0))
        self.score = str(params.get("score", "sigmoid"))
        self.normalize = bool(params.get("normalize", True))
        self.floor = float(params.get("floor", 1e-20))
        self.router_bias = bool(params.get("router_bias", False))
        self.expert_kind = str(params.get("expert_kind", "gated"))
        self.activation = params.get("activation")
        if self.expert_kind not in ("gated", "plain"):
            raise ValueError(f"expert kind {self.expert_kind!r}; known: gated, plain")
        if self.expert_kind == "plain" and self.activation not in moe_ops.PLAIN_ACTS:
            raise ValueError(f"a plain expert's activation {self.activation!r}; known: {sorted(map(str, moe_ops.PLAIN_ACTS))}")
        if self.score not in moe_ops.SCORE_FUNCTIONS:
            raise ValueError(f"router score {self.score!r}; known: {sorted(moe_ops.SCORE_FUNCTIONS)}")
        if self.groups <= 0 or self.experts % self.groups:
            raise ValueError(f"{self.experts} experts do not divide into {self.groups} equal groups")
        if not 0 < self.keep <= self.groups:
            raise ValueError(f"{self.keep} of {self.groups} groups cannot be kept")
        if not 0 < self.top <= self.keep * (self.experts // self.groups):
            raise ValueError(f"{self.top} experts cannot be chosen from {self.keep} groups of "
                             f"{self.experts // self.groups}")
        if self.limit is not None and not self.limit > 0:
            raise ValueError("the clamp limit of an expert must be positive")
        names = dict(params.get("names") or {})
        self.names = {k: names.get(k, d) for k, d in (("router", "router"), ("expert", "experts.{}"), ("gate", "gate_proj"),
                                                      ("up", "up_proj"), ("down", "down_proj"), ("shared", "shared"))}
        shared: Optional[PartSpec] = params.get("shared")
        self.shared: Optional[Part] = None if shared is None else build_part("ffn", shared, dtype, device)
        self.w_router: Optional[torch.Tensor] = None
        self.b_router: Optional[torch.Tensor] = None
        self.w_gate_up: Optional[torch.Tensor] = None   # [E, 2 ff, hidden]; plain experts: [E, ff, hidden], up rows only
        self.w_down: Optional[torch.Tensor] = None      # [E, hidden, ff]

    def sub_parts(self) -> Dict[str, Part]:
        return {} if self.shared is None else {self.names["shared"]: self.shared}

    def _expert(self, e: int, which: str) -> str:
        return f"{self.names['expert'].format(e)}.{self.names[which]}.weight"

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {f"{self.names['router']}.weight": ParamSpec((self.experts, self.hidden))}
        if self.router_bias:
            specs[f"{self.names['router']}.bias"] = ParamSpec((self.experts,), "vector")
        for e in range(self.experts):
            if self.expert_kind == "gated":
                specs[self._expert(e, "gate")] = ParamSpec((self.inter, self.hidden))
            specs[self._expert(e, "up")] = ParamSpec((self.inter, self.hidden))
            specs[self._expert(e, "down")] = ParamSpec((self.hidden, self.inter))
        return specs

    def load(self, tensors):
        self.w_router = tensors[f"{self.names['router']}.weight"]
        self.b_router = tensors.get(f"{self.names['router']}.bias")
        if self.expert_kind == "gated":
            both = [torch.cat([tensors[self._expert(e, "gate")], tensors[self._expert(e, "up")]], dim=0)
                    for e in range(self.experts)]
        else:
            both = [tensors[self._expert(e, "up")] for e in range(self.experts)]
        self.w_gate_up = torch.stack(both).contiguous()
        self.w_down = torch.stack([tensors[self._expert(e, "down")] for e in range(self.experts)]).contiguous()

    def named_weights(self) -> Dict[str, torch.Tensor]:
        out = {f"{self.names['router']}.weight": self.w_router}
        if self.b_router is not None:
            out[f"{self.names['router']}.bias"] = self.b_router
        for e in range(self.experts):
            if self.expert_kind == "gated":
                out[self._expert(e, "gate")] = self.w_gate_up[e, :self.inter]
                out[self._expert(e, "up")] = self.w_gate_up[e, self.inter:]
            else:
                out[self._expert(e, "up")] = self.w_gate_up[e]
            out[self._expert(e, "down")] = self.w_down[e]
        return out

    def route(self, x: torch.Tensor):
        """``(chosen int32 [N, top], weights float32 [N, top])`` of the rows of ``x``."""
        z = linear(x, self.w_router, self.b_router, out_dtype=torch.float32)
        return moe_ops.route(z if z.is_contiguous() else z.contiguous(), self.top, self.groups, self.keep, self.scale,
                             self.score, self.normalize, self.floor)

    def forward(self, x, step: StepContext):
        n = x.shape[0]
        ids, weights = self.route(x)
        order, offsets = moe_ops.sort_pairs(ids, self.experts)
        pairs = n * self.top
        if self.expert_kind == "gated":
            how = dict(gated=(self.alpha, self.limit, self.shift))
        else:
            how = dict(act=self.activation)
        act = moe_ops.expert_products(x, self.w_gate_up, order, offsets, pairs, self.top, self.dtype, **how)
        # few pairs: the float32 sums as they are; many: one rounding, half the traffic
        y = moe_ops.expert_products(act, self.w_down, order, offsets, pairs, 1,
                                    torch.float32 if pairs <= FLOAT32_PAIRS else self.dtype)
        extra = None
        if self.shared is not None:
            residual, step.residual = step.residual, None      # the shared expert's result is an addend of this sum
            extra = self.shared.forward(x, step)
            step.residual = residual
        return moe_ops.combine(y, weights, extra)


register_part("ffn", "routed_experts", RoutedExperts)
