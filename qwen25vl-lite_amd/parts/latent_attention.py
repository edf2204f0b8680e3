"""Attention through a latent: queries, keys and values are projected down to a few channels, normed, and
projected up again per head; what a token leaves in the cache is its key/value latent and one rotated key
part that all heads share.

With ``c`` the normed key/value latent and ``r`` the rotated key part of a key, head ``h`` scores a query
``[q_plain | q_rot]`` as ``scale (q_plain . (Uk_h c) + q_rot . r)``.  Since ``q_plain . (Uk_h c) =
(Uk_h^T q_plain) . c``, the query is carried into the latent's space once per token and head, and attention
runs over one cached key ``[c | r]`` per token, shared by all heads, whose value is ``c`` itself; the
value up-projection ``Uv_h`` is applied to the attended latent.  The pages, block tables and attention
kernels are the engine's own (one key/value head, values narrower than keys).  The two products with a
matrix per head run through the kernels of the routed experts, a head taking an expert's place: they read
and write a head's slice of a token's row where it lies, so nothing is transposed or copied.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels, latent, moe as moe_ops
from ..ops.attention import paged_attention
from ..ops.linear import linear, linear_into
from .base import CacheNeed, LayerSlot, Mixer, ParamSpec, PartSpec, StepContext, build_part, register_part

__all__ = ["LatentAttention"]


class LatentAttention(Mixer):
    """params: ``hidden_size``, ``num_heads``, ``head_dim`` (a head's unrotated query/key channels), ``rot_dim``
    (its rotated ones), ``value_dim``, ``q_rank`` and ``kv_rank`` (the latents' sizes; ``q_rank`` None: the queries
    are one projection ``q`` of the mixer's input and pass no latent), ``scale`` (None:
    ``(head_dim + rot_dim) ** -0.5``), ``eps`` (of the latents' RMS norms), ``window`` (None: all keys; a number:
    a query at index i sees keys j with ``0 <= i - j < window``), ``retain`` (how many keys back pages are kept,
    None: all; default ``window``; a layer whose cache another layer with a longer window reads keeps more than
    it sees), ``sinks`` (True: a tensor ``sink [heads]`` whose ``exp`` joins each head's softmax denominator),
    ``position`` (a :class:`PartSpec` of category ``position`` for the ``rot_dim`` rotated channels), ``kv_shared``
    (True: no key/value down projection; the layer reads the latents another layer cached, with up projections
    of its own), ``names`` (``dq``, ``dq_norm``, ``uq``, ``q``, ``dkv``, ``dkv_norm``, ``uk``, ``uv``, ``sink``, ``o``).  The
    position encoding says whether rotated channels are paired in halves or as neighbours (``interleaved``).

    The down projections are one stacked product left in float32; the norms, the rotation's angles, the scores
    and the softmax are float32; the latents in the cache, the queries and the attended latents are in the run
    dtype."""

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.heads = int(params["num_heads"])
        self.dim = int(params["head_dim"])
        self.rot_dim = int(params["rot_dim"])
        self.vdim = int(params["value_dim"])
        self.q_rank = int(params["q_rank"]) if params.get("q_rank") is not None else 0   # 0: queries pass no latent
        self.kv_rank = int(params["kv_rank"])
        if min(self.heads, self.dim, self.vdim, self.kv_rank) <= 0 or self.rot_dim < 0 or self.q_rank < 0 \
                or (params.get("q_rank") is not None and self.q_rank == 0):
            raise ValueError("a latent attention's sizes must be positive (rot_dim may be 0)")
        scale = params.get("scale")
        self.scale = float(scale) if scale is not None else (self.dim + self.rot_dim) ** -0.5
        self.eps = float(params["eps"])
        self.window: Optional[int] = params.get("window")
        self.retain: Optional[int] = params.get("retain", self.window)
        if self.window is not None and self.retain is not None and self.retain < self.window:
            raise ValueError("pages must be kept at least as far back as the window reaches")
        if self.window is None and self.retain is not None:
            raise ValueError("a layer that sees all keys keeps all pages")
        self.kv_shared = bool(params.get("kv_shared", False))
        self.has_sinks = bool(params.get("sinks", False))
        names = dict(params.get("names") or {})
        self.names = {k: names.get(k, k) for k in ("dq", "dq_norm", "uq", "q", "dkv", "dkv_norm", "uk", "uv", "sink", "o")}
        pos: Optional[PartSpec] = params.get("position")
        self.position = build_part("position", pos, dtype, device) if pos is not None and self.rot_dim else None
        self.interleaved = bool(getattr(self.position, "interleaved", False))
        self.w_down: Optional[torch.Tensor] = None      # [q_rank (+ kv_rank + rot_dim), hidden]
        self.q_norm: Optional[torch.Tensor] = None
        self.kv_norm: Optional[torch.Tensor] = None
        self.w_uq: Optional[torch.Tensor] = None        # [heads (dim + rot_dim), q_rank]; without a query latent [.., hidden]
        self.w_uk_t: Optional[torch.Tensor] = None      # [heads, kv_rank, dim]: Uk_h^T, the matrix that carries a query over
        self.w_uv: Optional[torch.Tensor] = None        # [heads, vdim, kv_rank]
        self.sink: Optional[torch.Tensor] = None
        self.w_out: Optional[torch.Tensor] = None

    @property
    def key_dim(self) -> int:
        return self.kv_rank + self.rot_dim

    def cache_need(self) -> CacheNeed:
        return CacheNeed(1, self.key_dim, self.retain, 0, self.kv_rank)

    def param_specs(self) -> Dict[str, ParamSpec]:
        n, h = self.names, self.heads
        if self.q_rank:
            specs = {f"{n['dq']}.weight": ParamSpec((self.q_rank, self.hidden)),
                     f"{n['dq_norm']}.weight": ParamSpec((self.q_rank,), "vector", init="around_one"),
                     f"{n['uq']}.weight": ParamSpec((h * (self.dim + self.rot_dim), self.q_rank))}
        else:
            specs = {f"{n['q']}.weight": ParamSpec((h * (self.dim + self.rot_dim), self.hidden))}
        if not self.kv_shared:
            specs[f"{n['dkv']}.weight"] = ParamSpec((self.kv_rank + self.rot_dim, self.hidden))
            specs[f"{n['dkv_norm']}.weight"] = ParamSpec((self.kv_rank,), "vector", init="around_one")
        specs[f"{n['uk']}.weight"] = ParamSpec((h * self.dim, self.kv_rank))
        specs[f"{n['uv']}.weight"] = ParamSpec((h * self.vdim, self.kv_rank))
        if self.has_sinks:
            specs[f"{n['sink']}.weight"] = ParamSpec((h,), "vector")
        specs[f"{n['o']}.weight"] = ParamSpec((self.hidden, h * self.vdim))
        return specs

    def load(self, tensors):
        n = self.names
        mats = [tensors[f"{n['dq']}.weight"]] if self.q_rank else []
        if not self.kv_shared:
            mats.append(tensors[f"{n['dkv']}.weight"])
            self.kv_norm = tensors[f"{n['dkv_norm']}.weight"]
        self.w_down = torch.cat(mats, dim=0).contiguous() if mats else None
        self.q_norm = tensors.get(f"{n['dq_norm']}.weight")
        self.w_uq = tensors[f"{n['uq' if self.q_rank else 'q']}.weight"]
        self.w_uk_t = tensors[f"{n['uk']}.weight"].view(self.heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[f"{n['uv']}.weight"].view(self.heads, self.vdim, self.kv_rank)
        self.sink = tensors.get(f"{n['sink']}.weight")
        self.w_out = tensors[f"{n['o']}.weight"]

    def named_weights(self) -> Dict[str, torch.Tensor]:
        n = self.names
        out = {f"{n['uk']}.weight": self.w_uk_t.transpose(1, 2).reshape(-1, self.kv_rank),
               f"{n['uv']}.weight": self.w_uv.reshape(-1, self.kv_rank), f"{n['o']}.weight": self.w_out}
        if self.q_rank:
            out.update({f"{n['dq']}.weight": self.w_down[:self.q_rank], f"{n['dq_norm']}.weight": self.q_norm,
                        f"{n['uq']}.weight": self.w_uq})
        else:
            out[f"{n['q']}.weight"] = self.w_uq
        if not self.kv_shared:
            out[f"{n['dkv']}.weight"] = self.w_down[self.q_rank:]
            out[f"{n['dkv_norm']}.weight"] = self.kv_norm
        if self.sink is not None:
            out[f"{n['sink']}.weight"] = self.sink
        return out

    def _rotation_table(self, step: StepContext, n: int) -> Optional[torch.Tensor]:
        """Cosines and sines of the step's angles, shared by the layers whose rotations agree."""
        if self.position is None:
            return None
        key = ("rope_cs", self.position.table_key(self.rot_dim))
        cs = step.per_pass.get(key)
        if cs is None:
            inv_freq, freq_row = self.position.rotary_tables(self.rot_dim)
            cs = step.per_pass[key] = kernels.rope_table(step.positions, inv_freq, freq_row, n,
                                                         amplitude=float(getattr(self.position, "amplitude", 1.0)))
        return cs

    def forward(self, x: torch.Tensor, step: StepContext, slot: LayerSlot):
        if slot.group is None or slot.k_cache is None:
            raise RuntimeError("attention needs a cache slot")
        if slot.writes == self.kv_shared:
            raise RuntimeError("a layer without a key/value down projection must read another layer's cache, "
                               "and a layer with one must write its own")
        group = step.groups[slot.group]
        n, h, r, rot = x.shape[0], self.heads, self.kv_rank, self.rot_dim
        cs = self._rotation_table(step, n)
        cq = x
        if self.w_down is not None:
            down = linear(x, self.w_down, out_dtype=torch.float32)
            if self.kv_shared:
                cq = latent.latent_down(down, self.q_rank, self.q_norm, self.eps, self.dtype)
            else:
                cq = latent.latent_down(down, self.q_rank, self.q_norm, self.eps, self.dtype, kv_rank=r, rot_dim=rot,
                                        kv_norm=self.kv_norm, cs=cs, slots=group.slot_mapping, k_cache=slot.k_cache,
                                        v_cache=slot.v_cache, interleaved=self.interleaved)
            if not self.q_rank:
                cq = x                      # the queries are a projection of the mixer's input itself
        q = linear(cq, self.w_uq)
        q = q if q.is_contiguous() else q.contiguous()
        # the query in the latent's space, head by head: [N, heads, kv_rank | rot_dim]
        q_lat = torch.empty((n, h, r + rot), dtype=self.dtype, device=x.device)
        by_head = step.per_pass.get(("pairs_by_head", h))
        if by_head is None:
            by_head = step.per_pass[("pairs_by_head", h)] = moe_ops.pairs_by_column(n, h, x.device)
        moe_ops.expert_products(q.view(n * h, self.dim + rot)[:, :self.dim], self.w_uk_t, *by_head, n * h, 1, self.dtype,
                                out=q_lat.view(n * h, r + rot)[:, :r])
        latent.latent_query_rotate_(q, h, self.dim, rot, r, cs, q_lat, interleaved=self.interleaved)
        o_lat = paged_attention(q_lat.view(n, h * (r + rot)), slot.k_cache, slot.v_cache, group.block_table, step, h,
                                self.window, self.scale, sinks=self.sink)
        o = moe_ops.expert_products(o_lat.view(n * h, r), self.w_uv, *by_head, n * h, 1, self.dtype)
        return linear_into(step.residual, o.view(n, h * self.vdim), self.w_out)


register_part("mixer", "latent_attention", LatentAttention)
