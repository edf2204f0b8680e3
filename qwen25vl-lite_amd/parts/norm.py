"""RMSNorm (reference src/qwen25vl_lite/layers.py:14-31)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels, skinny
from ..ops.linear import NormedRows
from .base import Norm, ParamSpec, ResidualStream, register_part

__all__ = ["RMSNorm", "LayerNorm"]


class RMSNorm(Norm):
    """``x * rsqrt(mean(x^2) + eps) * (offset + weight)`` with the statistics in float32 and
    ``eps`` inside the root.  ``offset`` 0 uses the weight as stored; ``offset`` 1 is a weight
    stored around zero (the gain is formed once, in float32, when the weight arrives).

    params: ``size`` (row width), ``eps``, ``offset`` (default 0).
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.offset = float(params.get("offset", 0.0))
        self.weight: Optional[torch.Tensor] = None    # the gain: offset + stored weight

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.size,), "vector", init="normal" if self.offset else "around_one")}

    def load(self, tensors):
        stored = tensors["weight"]
        self.weight = stored + self.offset if self.offset else stored

    def forward(self, stream: ResidualStream, rows: Optional[torch.Tensor] = None, lazy: bool = False):
        if stream.pending_norm is not None or stream.row_addend is not None:
            # an addend that is normed on its way into the sum, or a vector for every row: one kernel
            # forms the sum and this norm
            from ..ops.gated import sandwich_norm
            gain, eps_y, factor = stream.pending_norm or (None, 0.0, 1.0)
            out = sandwich_norm(stream.h, stream.pending, gain if stream.pending is not None else None, eps_y, factor,
                                stream.row_addend, self.weight, self.eps, self.dtype, rows=rows)
            if rows is None:
                stream.pending = stream.pending_norm = stream.row_addend = None
            return out
        if (lazy and rows is None and stream.pending is None and self.dtype == torch.bfloat16
                and self.size % 8 == 0 and skinny.folds_norm(stream.h.shape[0], self.size, stream.h.device)):
            # a decode step: the product that follows computes the norm on the way
            return NormedRows(stream.h, self.weight, self.eps, self.dtype)
        out = kernels.add_rmsnorm(stream.h, stream.pending, self.weight, self.eps, self.dtype, rows=rows)
        if rows is None:
            stream.pending = None  # folded into h
        return out


    def forward_pair(self, stream: ResidualStream, other: "RMSNorm"):
        """Fold what is pending into the sum and return its rows normed under this norm's gain and under
        ``other``'s: one pass for two sublayers that read the same sum (both norms have one ``eps``)."""
        from ..ops.gated import sandwich_norm
        gain, eps_y, factor = stream.pending_norm or (None, 0.0, 1.0)
        pair = sandwich_norm(stream.h, stream.pending, gain if stream.pending is not None else None, eps_y, factor,
                             stream.row_addend, self.weight, self.eps, self.dtype, weight2=other.weight)
        stream.pending = stream.pending_norm = stream.row_addend = None
        return pair


class LayerNorm(Norm):
    """``(x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * weight``: the mean is taken off, there is no
    bias; statistics in float32, the deviations formed from the mean (two passes).

    params: ``size`` (row width), ``eps``.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.size,), "vector", init="around_one")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, stream: ResidualStream, rows: Optional[torch.Tensor] = None, lazy: bool = False):
        from ..ops import rownorm
        from ..ops.gated import residual_add

        if stream.pending_norm is not None or stream.row_addend is not None:
            raise RuntimeError("a layer norm does not fold a normed addend or a pass vector into the sum")
        if stream.pending is not None:
            residual_add(stream.h, stream.pending)
            stream.pending = None
        return rownorm.layer_norm(stream.h, self.weight, self.eps, self.dtype, rows=rows)

    def add_normed(self, h: torch.Tensor, y: torch.Tensor, copy_dtype: Optional[torch.dtype] = None):
        """``h += norm(y)`` in float32, in place; with ``copy_dtype`` the new ``h`` is also returned in it."""
        from ..ops import rownorm

        return rownorm.layer_norm_add_(h, y, self.weight, self.eps, copy_dtype)


register_part("norm", "rms_norm", RMSNorm)
register_part("norm", "layer_norm", LayerNorm)
