"""The arrangement of parts in a layer (reference src/qwen25vl_lite/text.py:188-206)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Block, LayerSlot, Part, PartSpec, ResidualStream, StepContext, build_part, register_part

__all__ = ["PreNormBlock", "ParallelBlock", "SandwichBlock", "PostNormBlock"]


class PreNormBlock(Block):
    """``h += mixer(norm1(h)); h += ffn(norm2(h))``.

    params: ``norm1``, ``mixer``, ``norm2``, ``ffn`` (:class:`PartSpec` each) and ``names``,
    the checkpoint sub-name of each of the four.  Each sum into ``h`` happens in float32,
    inside the following norm's kernel or, in a decode step, inside the product that ends the
    mixer or the feed-forward.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.norm1 = build_part("norm", params["norm1"], dtype, device)
        self.mixer = build_part("mixer", params["mixer"], dtype, device)
        self.norm2 = build_part("norm", params["norm2"], dtype, device)
        self.ffn = build_part("ffn", params["ffn"], dtype, device)
        self.names: Dict[str, str] = dict(params["names"])

    def sub_parts(self) -> Dict[str, Part]:
        return {self.names["norm1"]: self.norm1, self.names["mixer"]: self.mixer,
                self.names["norm2"]: self.norm2, self.names["ffn"]: self.ffn}

    def forward(self, stream: ResidualStream, step: StepContext, slot: LayerSlot) -> ResidualStream:
        x = self.norm1.forward(stream, lazy=self.mixer.takes_lazy_norm)
        step.residual = stream.h            # the mixer may add its result in place and return None
        stream.pending = self.mixer.forward(x, step, slot)
        y = self.norm2.forward(stream, lazy=self.ffn.takes_lazy_norm)
        step.residual = stream.h
        stream.pending = self.ffn.forward(y, step)
        step.residual = None
        return stream


class ParallelBlock(Block):
    """``x = norm(h); h += mixer(x) + ffn(x)``: one norm, both sublayers read its output; or, with a second
    norm, ``h += mixer(norm(h)) + ffn(norm2(h))``, both norms of the same ``h``.

    params: ``norm``, ``mixer`` (:class:`PartSpec` each), ``ffn`` (a :class:`PartSpec`, or None
    for a layer without a feed-forward), ``norm2`` (a :class:`PartSpec` or absent: the feed-forward reads the
    first norm's rows) and ``names``, the checkpoint sub-name of each.  The
    normalised rows are computed before either sublayer runs, so a sublayer's last product may add
    into ``h`` in place; what a sublayer returns instead is added in float32, the first result by a
    kernel of its own, the last one by the next norm's kernel.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.norm = build_part("norm", params["norm"], dtype, device)
        self.mixer = build_part("mixer", params["mixer"], dtype, device)
        self.ffn: Optional[Part] = None if params.get("ffn") is None else build_part("ffn", params["ffn"], dtype, device)
        self.norm2: Optional[Part] = None
        if self.ffn is not None and params.get("norm2") is not None:
            self.norm2 = build_part("norm", params["norm2"], dtype, device)
        # two RMS norms of one sum with one eps differ in their gains only: one kernel forms both
        self._pair = (self.norm2 is not None and hasattr(self.norm, "forward_pair") and type(self.norm2) is type(self.norm)
                      and self.norm.eps == self.norm2.eps and self.norm.size == self.norm2.size)
        self.names: Dict[str, str] = dict(params["names"])

    def sub_parts(self) -> Dict[str, Part]:
        parts = {self.names["norm"]: self.norm, self.names["mixer"]: self.mixer}
        if self.ffn is not None:
            parts[self.names["ffn"]] = self.ffn
        if self.norm2 is not None:
            parts[self.names["norm2"]] = self.norm2
        return parts

    def forward(self, stream: ResidualStream, step: StepContext, slot: LayerSlot) -> ResidualStream:
        from ..ops.gated import residual_add

        if self._pair:
            x, x2 = self.norm.forward_pair(stream, self.norm2)     # one pass over the sum for both norms
        else:
            x = self.norm.forward(stream)    # never lazily: h changes before the second reader would look
            x2 = x if self.norm2 is None else self.norm2.forward(stream)   # the sum is folded: this one only norms
        step.residual = stream.h
        y = self.mixer.forward(x, step, slot)
        if self.ffn is None:
            stream.pending = y
        else:
            if y is not None:
                residual_add(stream.h, y)
            stream.pending = self.ffn.forward(x2, step)
        step.residual = None
        return stream


class SandwichBlock(Block):
    """``h += m * norm1b(mixer(norm1(h))); h += m * norm2b(ffn(norm2(h)))``: a norm before and one
    behind each sublayer, and a fixed factor ``m`` on what joins the sum.

    params: ``norm1``, ``mixer``, ``norm1b``, ``norm2``, ``ffn``, ``norm2b`` (:class:`PartSpec` each; ``ffn``
    None for a layer without a feed-forward, whose ``norm2`` and ``norm2b`` are then not built),
    ``residual_mult`` (``m``, default 1) and ``names``, the checkpoint sub-name of each part.  The
    norms behind the sublayers are RMS norms: a sublayer's result waits in the stream with that
    norm's gain, and the kernel of the next norm in line forms the normed addend, the float32 sum
    and its own output in one pass.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.names: Dict[str, str] = dict(params["names"])
        self.mult = float(params.get("residual_mult", 1.0))
        self.norm1 = build_part("norm", params["norm1"], dtype, device)
        self.mixer = build_part("mixer", params["mixer"], dtype, device)
        self.norm1b = build_part("norm", params["norm1b"], dtype, device)
        self.ffn: Optional[Part] = None
        if params.get("ffn") is not None:
            self.norm2 = build_part("norm", params["norm2"], dtype, device)
            self.ffn = build_part("ffn", params["ffn"], dtype, device)
            self.norm2b = build_part("norm", params["norm2b"], dtype, device)
        for post in (self.norm1b, getattr(self, "norm2b", None)):
            if post is not None and not (hasattr(post, "weight") and hasattr(post, "eps")):
                raise ValueError("the norm behind a sublayer must be an RMS norm")

    def sub_parts(self) -> Dict[str, Part]:
        parts = {self.names["norm1"]: self.norm1, self.names["mixer"]: self.mixer, self.names["norm1b"]: self.norm1b}
        if self.ffn is not None:
            parts.update({self.names["norm2"]: self.norm2, self.names["ffn"]: self.ffn,
                          self.names["norm2b"]: self.norm2b})
        return parts

    def forward(self, stream: ResidualStream, step: StepContext, slot: LayerSlot) -> ResidualStream:
        x = self.norm1.forward(stream)
        step.residual = None                 # a sublayer's result is normed before it joins the sum
        stream.pending = self.mixer.forward(x, step, slot)
        stream.pending_norm = (self.norm1b.weight, self.norm1b.eps, self.mult)
        if self.ffn is not None:
            y = self.norm2.forward(stream)
            stream.pending = self.ffn.forward(y, step)
            stream.pending_norm = (self.norm2b.weight, self.norm2b.eps, self.mult)
        return stream


class PostNormBlock(Block):
    """``h += norm1(mixer(f(h))); h += norm2(ffn(h))``: the sublayers read the residual sum itself and the
    norm stands on each sublayer's output only; ``f`` is an optional filter on what the mixer reads (a short
    convolution over time with a state per request).

    params: ``mixer``, ``norm1`` (:class:`PartSpec` each; the norm must offer ``add_normed``, as the layer
    norm does), ``ffn`` and ``norm2`` (or ``ffn`` None for a layer without a feed-forward, whose ``norm2`` is
    then not built), ``filter`` (a :class:`PartSpec` of category ``filter``, or None) and ``names``, the
    checkpoint sub-name of each.  The sum stays float32; a sublayer is handed its rounding to the run dtype.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.names: Dict[str, str] = dict(params["names"])
        self.mixer = build_part("mixer", params["mixer"], dtype, device)
        self.norm1 = build_part("norm", params["norm1"], dtype, device)
        self.filter: Optional[Part] = None
        if params.get("filter") is not None:
            self.filter = build_part("filter", params["filter"], dtype, device)
        self.ffn: Optional[Part] = None
        self.norm2: Optional[Part] = None
        if params.get("ffn") is not None:
            self.ffn = build_part("ffn", params["ffn"], dtype, device)
            self.norm2 = build_part("norm", params["norm2"], dtype, device)
        for norm in (self.norm1, self.norm2):
            if norm is not None and not hasattr(norm, "add_normed"):
                raise ValueError("the norm behind a sublayer must be able to add its result into the sum")

    def sub_parts(self) -> Dict[str, Part]:
        # the mixer first: an entry's own slot is its first part's
        parts = {self.names["mixer"]: self.mixer, self.names["norm1"]: self.norm1}
        if self.filter is not None:
            parts[self.names["filter"]] = self.filter
        if self.ffn is not None:
            parts.update({self.names["ffn"]: self.ffn, self.names["norm2"]: self.norm2})
        return parts

    def _rounded(self, h):
        return h if self.dtype == h.dtype else h.to(self.dtype)

    def forward(self, stream: ResidualStream, step: StepContext, slot: LayerSlot) -> ResidualStream:
        from ..ops.gated import residual_add

        if stream.pending_norm is not None or stream.row_addend is not None:
            raise RuntimeError("this block reads the sum itself: what is pending must be a plain addend")
        if stream.pending is not None:
            residual_add(stream.h, stream.pending)
            stream.pending = None
        h = stream.h
        step.residual = None                 # a sublayer's result is normed before it joins the sum
        mixer_slot = slot.by_part.get(self.names["mixer"], slot)
        if self.filter is not None:
            x = self.filter.forward(h, step, slot.by_part.get(self.names["filter"]))
        else:
            x = self._rounded(h)
        y = self.mixer.forward(x, step, mixer_slot)
        wants_copy = self.ffn is not None and self.dtype != torch.float32
        x = self.norm1.add_normed(h, y, self.dtype if wants_copy else None)
        if self.ffn is not None:
            y = self.ffn.forward(x if wants_copy else h, step)
            self.norm2.add_normed(h, y)
        return stream


register_part("block", "sandwich", SandwichBlock)
register_part("block", "post_norm", PostNormBlock)
register_part("block", "pre_norm", PreNormBlock)
register_part("block", "parallel", ParallelBlock)
