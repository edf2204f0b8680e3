"""Linear attention with a decayed outer-product state per request and head.

Per head, ``S_t = diag(a_t) S_(t-1) + k_t v_t^T`` and ``o_t = S_t^T q_t``; ``S`` is float32
``[dim, vdim]``, starts at zero and is carried from step to step in the request's state slot.
What varies between designs is a parameter: the decay (a constant per head, per key channel
and token from a low-rank projection, or a forget gate with a floor whose complement is the key), an
activation on q, k and v, a scale on q, whether the heads' outputs are normed together or one by one,
and the gate's activation (or no gate).
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import gated
from ..ops.linear import linear, linear_into
from ..ops.linear_attention import CHUNKED_FROM, chunked_scan, decayed_scan, plan_chunks, scan_groups
from .base import LayerSlot, Mixer, ParamSpec, StateNeed, StepContext, register_part

__all__ = ["LinearAttention"]


class LinearAttention(Mixer):
    """params: ``hidden_size``, ``num_heads``, ``key_dim``, ``value_dim``, ``eps`` (of the output norm),

    * ``decay``: ``{"kind": "head", "values": [a_0, ...]}``, one constant per head, or
      ``{"kind": "channel", "rank": r, "tau": tau}``: ``a = sigmoid(z)^(1/tau)`` with
      ``z = A2 (A1 x) + b``, ``A1 [r, hidden]``, ``A2 [heads * key_dim, r]``; or ``{"kind": "forget"}``:
      ``a = l + (1 - l) sigmoid(F x + b)`` with a floor ``l`` per key channel (a tensor), and the key is
      ``1 - a`` (there is no key projection);
    * ``activation``: None or ``"silu"``, applied to q, k and v, or only to those ``activation_on`` names
      (a string of the letters q, k, v; default all three); ``q_scale`` (default 1);
    * ``norm``: ``"all_heads"`` (one RMS norm over the concatenated heads, weight
      ``[heads * value_dim]``) or ``"per_head"`` (each head by itself, weight ``[value_dim]`` shared);
    * ``gate``: ``"sigmoid"`` or ``"silu"`` of a projection ``g [heads * value_dim, hidden]``, which
      multiplies the normed output before the output projection, or None: no gate;
    * ``names``: local names of the tensors' owners (default ``q``, ``k``, ``v``, ``g``, ``o``, ``norm``,
      ``a1``, ``a2``, ``f``, ``lower``).

    q, k, v, the gate and the decay's first factor come from one stacked product in the run
    dtype (with the forget gate's projection among them, the product is left in float32); decays, the
    state, the output of the recurrence and its norm are float32.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.heads = int(params["num_heads"])
        self.dim = int(params["key_dim"])
        self.vdim = int(params["value_dim"])
        self.eps = float(params["eps"])
        decay = dict(params["decay"])
        self.decay_kind = decay["kind"]
        self.head_decay: Optional[torch.Tensor] = None
        self.rank, self.tau = 0, 1.0
        if self.decay_kind == "head":
            values = [float(a) for a in decay["values"]]
            if len(values) != self.heads:
                raise ValueError(f"{len(values)} decay constants for {self.heads} heads")
            self.head_decay = torch.tensor(values, dtype=torch.float32, device=device)
        elif self.decay_kind == "channel":
            self.rank, self.tau = int(decay["rank"]), float(decay["tau"])
            if not self.tau > 0:
                raise ValueError("tau must be positive")
        elif self.decay_kind != "forget":
            raise ValueError(f"decay kind {self.decay_kind!r}; known: head, channel, forget")
        self.activation = params.get("activation")
        if self.activation not in (None, "silu"):
            raise ValueError(f"activation {self.activation!r}; known: None, silu")
        self.silu_on = (params.get("activation_on") or "qkv") if self.activation == "silu" else ""
        if not set(self.silu_on) <= set("qkv"):
            raise ValueError("activation_on names some of q, k and v")
        self.q_scale = float(params.get("q_scale", 1.0))
        self.norm_kind = params.get("norm", "per_head")
        if self.norm_kind not in ("all_heads", "per_head"):
            raise ValueError(f"norm {self.norm_kind!r}; known: all_heads, per_head")
        self.gate_act = params.get("gate", "sigmoid")
        if self.gate_act not in (None, "sigmoid", "silu"):
            raise ValueError(f"gate {self.gate_act!r}; known: None, sigmoid, silu")
        names = dict(params.get("names") or {})
        self.names = {k: names.get(k, k) for k in ("q", "k", "v", "g", "o", "norm", "a1", "a2", "f", "lower")}
        self.lower: Optional[torch.Tensor] = None
        self.b_forget: Optional[torch.Tensor] = None
        self.w_in: Optional[torch.Tensor] = None
        self.w_out: Optional[torch.Tensor] = None
        self.w_norm: Optional[torch.Tensor] = None
        self.w_a2: Optional[torch.Tensor] = None
        self.b_a2: Optional[torch.Tensor] = None

    def state_need(self) -> StateNeed:
        return StateNeed((self.heads, self.dim, self.vdim), torch.float32)

    def _stacked(self):
        """``(role, rows)`` of the matrices of the input product, in order."""
        hk, hv = self.heads * self.dim, self.heads * self.vdim
        out = [("q", hk)]
        if self.decay_kind != "forget":
            out.append(("k", hk))
        out.append(("v", hv))
        if self.gate_act is not None:
            out.append(("g", hv))
        if self.decay_kind == "channel":
            out.append(("a1", self.rank))
        if self.decay_kind == "forget":
            out.append(("f", hk))
        return out

    def _offset(self, role: str) -> int:
        at = 0
        for name, rows in self._stacked():
            if name == role:
                return at
            at += rows
        raise KeyError(role)

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        specs = {f"{n[role]}.weight": ParamSpec((rows, self.hidden)) for role, rows in self._stacked()}
        if self.decay_kind == "channel":
            specs[f"{n['a2']}.weight"] = ParamSpec((self.heads * self.dim, self.rank))
            specs[f"{n['a2']}.bias"] = ParamSpec((self.heads * self.dim,), "vector")
        if self.decay_kind == "forget":
            specs[f"{n['f']}.bias"] = ParamSpec((self.heads * self.dim,), "vector")
            specs[f"{n['lower']}.weight"] = ParamSpec((self.heads * self.dim,), "vector", init="unit_interval")
        width = self.heads * self.vdim if self.norm_kind == "all_heads" else self.vdim
        specs[f"{n['norm']}.weight"] = ParamSpec((width,), "vector", init="around_one")
        specs[f"{n['o']}.weight"] = ParamSpec((self.hidden, self.heads * self.vdim))
        return specs

    def load(self, tensors):
        n = self.names
        self.w_in = torch.cat([tensors[f"{n[role]}.weight"] for role, _ in self._stacked()], dim=0).contiguous()
        self.w_out = tensors[f"{n['o']}.weight"]
        self.w_norm = tensors[f"{n['norm']}.weight"]
        if self.decay_kind == "channel":
            self.w_a2, self.b_a2 = tensors[f"{n['a2']}.weight"], tensors[f"{n['a2']}.bias"]
        if self.decay_kind == "forget":
            self.b_forget, self.lower = tensors[f"{n['f']}.bias"], tensors[f"{n['lower']}.weight"]

    def named_weights(self) -> Dict[str, torch.Tensor]:
        n = self.names
        out, row = {}, 0
        for role, rows in self._stacked():
            out[f"{n[role]}.weight"] = self.w_in[row:row + rows]
            row += rows
        if self.decay_kind == "channel":
            out[f"{n['a2']}.weight"], out[f"{n['a2']}.bias"] = self.w_a2, self.b_a2
        if self.decay_kind == "forget":
            out[f"{n['f']}.bias"], out[f"{n['lower']}.weight"] = self.b_forget, self.lower
        out[f"{n['norm']}.weight"] = self.w_norm
        out[f"{n['o']}.weight"] = self.w_out
        return out

    def forward(self, x, step: StepContext, slot: LayerSlot):
        if slot.state is None:
            raise RuntimeError("linear attention needs a state slot")
        hk, hv = self.heads * self.dim, self.heads * self.vdim
        forget = self.decay_kind == "forget"
        # [N, q | (k) | v | (g) | (a1) | (f)] in the run dtype; with a forget gate's projection, which enters the
        # recurrence, in float32
        proj = linear(x, self.w_in, out_dtype=torch.float32 if forget else None)
        z = None
        if self.decay_kind == "channel":
            at = self._offset("a1")
            low = proj[:, at:at + self.rank].contiguous()      # a few columns: copied to rows of their own
            z = linear(low, self.w_a2, self.b_a2, out_dtype=torch.float32)
        elif forget:
            at = self._offset("f")
            z = proj[:, at:at + hk]
        how = dict(head_decay=self.head_decay, z=z, tau=self.tau, silu=self.silu_on, q_scale=self.q_scale,
                   lower=self.lower, z_bias=self.b_forget)
        q_at, k_at, v_at = 0, 0 if forget else hk, self._offset("v")
        if step.max_q_len >= CHUNKED_FROM and len(step.cu_q_host) == step.num_reqs + 1:
            # long runs (never a captured decode step): in chunks side by side; the plan is the step's, shared by layers
            plan = step.derived.get("la_chunks")
            if plan is None:
                plan = step.derived["la_chunks"] = plan_chunks(step.cu_q_host, self.device)
            o = chunked_scan(proj, q_at, k_at, v_at, self.heads, self.dim, self.vdim, slot.state, plan, step.req_slots, **how)
        else:
            o = decayed_scan(proj, q_at, k_at, v_at, self.heads, self.dim, self.vdim, slot.state, step.cu_q,
                             step.req_slots, groups=scan_groups(step.num_reqs, step.max_q_len, self.heads, self.dim,
                                                                self.vdim, self.device), **how)
        span = hv if self.norm_kind == "all_heads" else self.vdim
        gate = None
        if self.gate_act is not None:
            at = self._offset("g")
            gate = proj[:, at:at + hv]
        y = gated.group_norm_gate(o, self.w_norm, span, self.eps, self.dtype, gate=gate, gate_act=self.gate_act)
        return linear_into(step.residual, y, self.w_out)


register_part("mixer", "linear_attention", LinearAttention)
