"""Attention over the paged cache (reference src/qwen25vl_lite/text.py:69-185).

``q = x Wq^T + bq`` and likewise k, v; queries and keys are rotated by the position encoding;
keys (rotated) and values go into the request's pages; every token attends to the keys of its
request up to itself (``scale * q.k``, softmax in float32, GQA: query head h reads key head
``h // (heads / kv_heads)``), within ``window`` keys if the layer has one; then ``Wo``.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels, skinny
from ..ops.attention import paged_attention
from ..ops.linear import NormedRows, linear, linear_into
from .base import (CacheNeed, LayerSlot, Mixer, ParamSpec, PartSpec, StateNeed, StepContext, build_part,
                   register_part)

# 33 to 48 rows: the projection cut along its inner size (slabs) and the rotation's kernel behind it beat the
# fused kernel on teams of blocks (7B sizes: a step of 33 rows 4.14 ms against 4.24, of 48 rows 4.34 against 4.39,
# of 64 rows 4.68 against 4.67)
SPLIT_ROWS = (33, 48)

__all__ = ["PagedAttention"]


class PagedAttention(Mixer):
    """params: ``hidden_size``, ``num_heads``, ``num_kv_heads``, ``head_dim``, ``qkv_bias``,
    ``window`` (None: all keys), ``scale`` (None: ``head_dim ** -0.5``, reference text.py:78),
    ``position`` (a :class:`PartSpec` of category ``position``), ``kv_shared`` (True: the layer
    has no key/value projections and reads the cache another layer wrote).

    Optional: ``qk_norm_eps`` (a number: queries and keys are RMS-normed per head before the
    rotation, with weights ``q_norm`` / ``k_norm`` of ``[head_dim]`` shared by the heads),
    ``values_are_keys`` (there is no value projection: a key head as projected, before norm and
    rotation, is its own value), ``head_gate`` (each head's output is multiplied by the sigmoid of
    one number per head, a projection ``g`` of ``[heads, hidden]`` of the mixer's input), ``names``
    (local names of the tensors' owners, default ``q_proj`` ... ``o_proj``, ``g_proj``, ``q_norm``,
    ``k_norm``, ``v``).  A position encoding may ask for interleaved pairs (``interleaved``).
    ``qk_norm_where`` (``"before"``, the default, or ``"after"`` the rotation) and ``qk_norm_weights``
    (False: the norm has no gains and the mixer no such tensors), ``value_dim`` (values of another
    width than keys), ``keep_first`` (with a window: the first so many keys of a request stay visible
    to every later token; their rotation and their distance to a query are those of where they stand),
    ``element_gate`` (channel ``c`` of the heads' joined output is scaled by ``sigmoid(g_c)``, ``g`` a
    projection of ``[heads value_dim, hidden]``),
    ``out_bias`` (the output projection has a bias), ``qk_norm_scope`` (``"head"``, the default, or ``"whole"``: one
    RMS norm over all of a token's query heads together and one over all its key heads, before the rotation,
    with weights of ``[heads head_dim]``), ``conv_taps`` (a number: the projected queries and keys pass a causal
    convolution over time, ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)`` per channel with weights ``q_conv`` /
    ``k_conv`` of ``[channels, taps]``, before norm and rotation; keys that are their own values are taken behind
    it; a request's last ``taps - 1`` projected rows are its state), ``sinks`` (True: a tensor ``sink [heads]``
    whose ``exp`` joins each head's softmax denominator).  Any of these except the output bias and the sinks
    takes the projection through float32 and one kernel that norms, rotates and writes the cache."""

    graph_safe = True
    takes_lazy_norm = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.nq = int(params["num_heads"])
        self.nkv = int(params["num_kv_heads"])
        self.hd = int(params["head_dim"])
        self.qkv_bias = bool(params.get("qkv_bias", False))
        self.window: Optional[int] = params.get("window")
        scale = params.get("scale")
        self.scale = float(scale) if scale is not None else self.hd ** -0.5
        self.kv_shared = bool(params.get("kv_shared", False))
        eps = params.get("qk_norm_eps")
        self.qk_norm_eps: Optional[float] = None if eps is None else float(eps)
        self.qk_norm_where = str(params.get("qk_norm_where", "before"))
        self.qk_norm_weights = bool(params.get("qk_norm_weights", True))
        self.values_are_keys = bool(params.get("values_are_keys", False))
        self.head_gate = bool(params.get("head_gate", False))
        self.element_gate = bool(params.get("element_gate", False))
        self.out_bias = bool(params.get("out_bias", False))
        self.qk_norm_scope = str(params.get("qk_norm_scope", "head"))
        self.conv_taps = int(params.get("conv_taps") or 0)
        self.has_sinks = bool(params.get("sinks", False))
        self.vd = int(params.get("value_dim") or self.hd)
        self.keep_first = int(params.get("keep_first") or 0) if self.window else 0
        if self.qk_norm_where not in ("before", "after"):
            raise ValueError("qk_norm_where is 'before' or 'after' (the rotation)")
        if self.head_gate and self.element_gate:
            raise ValueError("an attention mixer has one kind of output gate at most")
        if self.values_are_keys and self.vd != self.hd:
            raise ValueError("keys that are their own values have the keys' width")
        if self.keep_first < 0:
            raise ValueError("keep_first cannot be negative")
        if self.qk_norm_scope not in ("head", "whole"):
            raise ValueError("qk_norm_scope is 'head' or 'whole'")
        if self.qk_norm_scope == "whole" and (self.qk_norm_eps is None or self.qk_norm_where != "before"
                                              or not self.qk_norm_weights):
            raise ValueError("a norm over the whole projection stands before the rotation and has weights")
        if self.conv_taps and not (self.values_are_keys and not self.qkv_bias):
            raise ValueError("the convolution on queries and keys is built for keys that are their own values, "
                             "without biases")
        names = dict(params.get("names") or {})
        self.names = {k: names.get(k, d) for k, d in (("q", "q_proj"), ("k", "k_proj"), ("v", "v_proj"), ("o", "o_proj"),
                                                      ("g", "g_proj"), ("q_norm", "q_norm"), ("k_norm", "k_norm"),
                                                      ("q_conv", "q_conv"), ("k_conv", "k_conv"), ("sink", "sink"))}
        self.q_norm: Optional[torch.Tensor] = None
        self.k_norm: Optional[torch.Tensor] = None
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} heads are not a multiple of {self.nkv} key/value heads")
        pos: PartSpec = params["position"]
        self.position = build_part("position", pos, dtype, device)
        self.interleaved = bool(getattr(self.position, "interleaved", False))
        self.normed_path = (self.qk_norm_eps is not None or self.values_are_keys or self.head_gate
                            or self.element_gate or self.interleaved or self.vd != self.hd or bool(self.conv_taps))
        self.gate_rows = self.nq if self.head_gate else (self.nq * self.vd if self.element_gate else 0)
        self.w_in: Optional[torch.Tensor] = None
        self.b_in: Optional[torch.Tensor] = None
        self.w_out: Optional[torch.Tensor] = None
        self.b_out: Optional[torch.Tensor] = None
        self.w_conv: Optional[torch.Tensor] = None      # float32 [taps, convolved channels]
        self.sink: Optional[torch.Tensor] = None

    def cache_need(self) -> CacheNeed:
        return CacheNeed(self.nkv, self.hd, self.window, self.keep_first, None if self.vd == self.hd else self.vd)

    @property
    def conv_channels(self) -> int:
        """Columns of the stacked projection that pass the convolution: the queries' and the keys'."""
        return (self.nq + (0 if self.kv_shared else self.nkv)) * self.hd if self.conv_taps else 0

    def state_need(self) -> Optional[StateNeed]:
        if self.conv_taps > 1:
            return StateNeed((self.conv_taps - 1, self.conv_channels), torch.float32)
        return None

    def _projections(self):
        """``(role, rows)`` of the matrices stacked into the input product, in order."""
        out = [("q", self.nq * self.hd)]
        if not self.kv_shared:
            out.append(("k", self.nkv * self.hd))
            if not self.values_are_keys:
                out.append(("v", self.nkv * self.vd))
        return out

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        specs = {}
        for role, rows in self._projections():
            specs[f"{n[role]}.weight"] = ParamSpec((rows, self.hidden))
        if self.qkv_bias:
            for role, rows in self._projections():
                specs[f"{n[role]}.bias"] = ParamSpec((rows,), "vector")
        if self.conv_taps:
            specs[f"{n['q_conv']}.weight"] = ParamSpec((self.nq * self.hd, self.conv_taps), "vector")
            if not self.kv_shared:
                specs[f"{n['k_conv']}.weight"] = ParamSpec((self.nkv * self.hd, self.conv_taps), "vector")
        if self.qk_norm_eps is not None and self.qk_norm_weights:
            whole = self.qk_norm_scope == "whole"
            specs[f"{n['q_norm']}.weight"] = ParamSpec((self.nq * self.hd if whole else self.hd,), "vector",
                                                       init="around_one")
            if not self.kv_shared:
                specs[f"{n['k_norm']}.weight"] = ParamSpec((self.nkv * self.hd if whole else self.hd,), "vector",
                                                           init="around_one")
        if self.has_sinks:
            specs[f"{n['sink']}.weight"] = ParamSpec((self.nq,), "vector")
        if self.gate_rows:
            specs[f"{n['g']}.weight"] = ParamSpec((self.gate_rows, self.hidden))
        specs[f"{n['o']}.weight"] = ParamSpec((self.hidden, self.nq * self.vd))
        if self.out_bias:
            specs[f"{n['o']}.bias"] = ParamSpec((self.hidden,), "vector")
        return specs

    def load(self, tensors):
        n = self.names
        roles = [role for role, _ in self._projections()]
        # One product for q, k and v (and the heads' gate): the matrices are stacked by rows.
        mats = [tensors[f"{n[r]}.weight"] for r in roles]
        bias = [tensors[f"{n[r]}.bias"] for r in roles] if self.qkv_bias else None
        if self.gate_rows:
            mats.append(tensors[f"{n['g']}.weight"])
            if bias is not None:
                bias.append(torch.zeros(self.gate_rows, dtype=bias[0].dtype, device=bias[0].device))
        self.w_in = torch.cat(mats, dim=0).contiguous()
        self.b_in = torch.cat(bias).contiguous() if bias is not None else None
        self.w_out = tensors[f"{n['o']}.weight"]
        self.b_out = tensors.get(f"{n['o']}.bias")
        if self.qk_norm_eps is not None and self.qk_norm_weights:
            self.q_norm = tensors[f"{n['q_norm']}.weight"]
            self.k_norm = tensors.get(f"{n['k_norm']}.weight")
        if self.conv_taps:
            # kept tap-major: neighbouring channels' weights of a tap lie side by side
            taps = [tensors[f"{n['q_conv']}.weight"]]
            if not self.kv_shared:
                taps.append(tensors[f"{n['k_conv']}.weight"])
            self.w_conv = torch.cat(taps, dim=0).t().contiguous()
        self.sink = tensors.get(f"{n['sink']}.weight")

    def named_weights(self) -> Dict[str, torch.Tensor]:
        """Views of the stacked tensors under their checkpoint names."""
        n = self.names
        out, row = {}, 0
        for role, rows in self._projections():
            out[f"{n[role]}.weight"] = self.w_in[row:row + rows]
            if self.b_in is not None:
                out[f"{n[role]}.bias"] = self.b_in[row:row + rows]
            row += rows
        if self.gate_rows:
            out[f"{n['g']}.weight"] = self.w_in[row:row + self.gate_rows]
        if self.b_out is not None:
            out[f"{n['o']}.bias"] = self.b_out
        if self.q_norm is not None:
            out[f"{n['q_norm']}.weight"] = self.q_norm
        if self.k_norm is not None:
            out[f"{n['k_norm']}.weight"] = self.k_norm
        if self.w_conv is not None:
            out[f"{n['q_conv']}.weight"] = self.w_conv[:, :self.nq * self.hd].t()
            if not self.kv_shared:
                out[f"{n['k_conv']}.weight"] = self.w_conv[:, self.nq * self.hd:].t()
        if self.sink is not None:
            out[f"{n['sink']}.weight"] = self.sink
        out[f"{n['o']}.weight"] = self.w_out
        return out

    def forward(self, x: torch.Tensor, step: StepContext, slot: LayerSlot) -> torch.Tensor:
        if slot.group is None or slot.k_cache is None:
            raise RuntimeError("attention needs a cache slot")
        group = step.groups[slot.group]
        write = slot.writes and not self.kv_shared
        if slot.writes == self.kv_shared:
            raise RuntimeError("a layer without key/value projections must read another layer's cache, "
                               "and a layer with them must write its own")
        inv_freq, freq_row = self.position.rotary_tables(self.hd)
        if self.normed_path:
            return self._forward_normed(x, step, group, slot, write, inv_freq, freq_row)
        q = self._project_few_rows(x, step, group, slot, write, inv_freq, freq_row)
        if q is None:
            q = self._project(x, step, group, slot, write, inv_freq, freq_row)
        o = paged_attention(q, slot.k_cache, slot.v_cache, group.block_table, step, self.nq, self.window, self.scale,
                            keep_first=self.keep_first, sinks=self.sink)
        return self._output(o, step)

    def _output(self, o: torch.Tensor, step: StepContext):
        """The output projection: into the residual where the block offers it and there is no bias."""
        if self.b_out is None:
            return linear_into(step.residual, o, self.w_out)
        return linear(o, self.w_out, self.b_out,
                      out_dtype=torch.float32 if o.shape[0] <= skinny.ONE_BLOCK_ROWS else None)

    def _forward_normed(self, x, step, group, slot, write, inv_freq, freq_row):
        """The path with a per-head norm, interleaved pairs, keys as values or a gate per head: the
        stacked projection leaves its product in float32, one kernel norms and rotates queries and
        keys and writes keys and values into the pages, and the gate multiplies the heads' outputs."""
        from ..ops import gated

        proj = linear(x, self.w_in, out_dtype=torch.float32)     # the bias is added by the kernel that norms
        cs = self._rotation_table(step, inv_freq, freq_row, proj.shape[0])
        heads_in = proj
        if self.conv_taps:
            from ..ops.short_conv import short_conv
            if self.conv_taps > 1 and slot.state is None:
                raise RuntimeError("a convolution with more than one tap needs a state slot")
            heads_in = short_conv(proj[:, :self.conv_channels], self.w_conv, slot.state, step.cu_q, step.req_slots,
                                  step.token_req, torch.float32)
        norm = None if self.qk_norm_eps is None else ("whole" if self.qk_norm_scope == "whole" else self.qk_norm_where)
        q = gated.qk_norm_rope_write(
            heads_in, self.q_norm, self.k_norm, self.qk_norm_eps if self.qk_norm_eps is not None else 0.0, cs,
            group.slot_mapping if write else None, slot.k_cache if write else None, slot.v_cache if write else None,
            self.nq, self.nkv, self.hd, group.page_size, self.dtype, interleaved=self.interleaved,
            values_are_keys=self.values_are_keys, norm=norm, bias=self.b_in, value_dim=self.vd)
        o = paged_attention(q, slot.k_cache, slot.v_cache, group.block_table, step, self.nq, self.window, self.scale,
                            keep_first=self.keep_first, sinks=self.sink)
        if self.gate_rows:
            # one gate per head, or one per element (a "head" of one channel)
            at = self.w_in.shape[0] - self.gate_rows
            gated.head_gate_(o, proj[:, at:at + self.gate_rows], self.gate_rows)
        return self._output(o, step)

    def _project(self, x, step, group, slot, write, inv_freq, freq_row) -> torch.Tensor:
        # Projections are written out in float32 (the accumulator, unrounded): bias, rotation and
        # the residual sum then happen in float32 and each stored value is rounded once.
        m, k = x.shape
        if (SPLIT_ROWS[0] <= m <= SPLIT_ROWS[1] and self.dtype == torch.bfloat16 and isinstance(x, torch.Tensor)
                and x.dtype == torch.bfloat16 and self.hd % 4 == 0 and inv_freq.shape[0] % 4 == 0
                and skinny.takes_split(m, k, self.w_in) and x.stride(1) == 1 and x.stride(0) % 8 == 0
                and x.data_ptr() % 16 == 0):
            qkv = skinny.split_product(self.w_in, x)   # slabs of partial sums: the rotation's kernel adds them
        else:
            qkv = linear(x, self.w_in, out_dtype=torch.float32)
        cs = self._rotation_table(step, inv_freq, freq_row, m)
        return kernels.rope_kv_write(
            qkv, self.b_in, step.positions, inv_freq, freq_row,
            group.slot_mapping if write else None, slot.k_cache if write else None, slot.v_cache if write else None,
            self.nq, self.nkv if write else 0, self.hd, group.page_size, out_dtype=self.dtype, cs=cs)

    def _rotation_table(self, step, inv_freq, freq_row, n: int) -> torch.Tensor:
        """Cosines and sines of the step's angles: computed once per pass and position encoding,
        by the first layer that needs them, and read by every head of every layer."""
        key = ("rope_cs", self.position.table_key(self.hd))
        cs = step.per_pass.get(key)
        if cs is None:
            cs = step.per_pass[key] = kernels.rope_table(step.positions, inv_freq, freq_row, n,
                                                         amplitude=float(getattr(self.position, "amplitude", 1.0)))
        return cs

    def _project_few_rows(self, x, step, group, slot, write, inv_freq, freq_row) -> Optional[torch.Tensor]:
        """A decode step's few bfloat16 rows: projection, bias, rotation and cache write in one
        kernel (the float32 sums never leave it)."""
        lazy = isinstance(x, NormedRows)
        m, k = x.shape
        if not lazy and SPLIT_ROWS[0] <= m <= SPLIT_ROWS[1]:
            return None
        if self.dtype != torch.bfloat16 or not skinny.takes_qkv_rope(
                m, k, self.w_in, self.hd, inv_freq.shape[0], slot.k_cache.dtype if write else None, norm=lazy):
            return None
        if not lazy and (x.dtype != torch.bfloat16 or x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16):
            return None
        cs = self._rotation_table(step, inv_freq, freq_row, m)
        src = dict(h=x.h, norm_weight=x.weight, eps=x.eps) if lazy else dict(x=x)
        return skinny.qkv_rope_product(
            self.w_in, cs, bias=self.b_in, slots=group.slot_mapping if write else None,
            k_cache=slot.k_cache if write else None, v_cache=slot.v_cache if write else None,
            num_q_heads=self.nq, num_kv_heads=self.nkv if write else 0, head_dim=self.hd,
            page_size=group.page_size, **src)


register_part("mixer", "paged_attention", PagedAttention)
