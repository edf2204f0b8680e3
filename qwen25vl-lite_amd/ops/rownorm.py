"""Python entry points of the row-wise kernels in ``csrc/rownorm.hip``: a layer norm that may add its result
into the float32 residual, a sum of normed powers, and the square of relu.

As in :mod:`~qwen25vl_lite_amd.ops.kernels`, every function checks on the host what the kernel and
its grid assume and launches on the current stream; there is no CPU path.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .kernels import _check, _dev, _fn, _need, _ptr, _stream, dtype_code

__all__ = ["layer_norm", "layer_norm_add_", "normed_powers", "squared_relu_"]

_c_int, _c_float, _c_ptr, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong
_LN_ARGS = [_c_ptr, _c_int, _c_int, _c_ll, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr]


def _source(y: torch.Tensor, width: int):
    """``(rows, slabs, slab stride)`` of a norm's input: ``[N, H]``, or float32 slabs ``[slabs, N, H]``."""
    if y.dim() == 3:
        _need(y.dtype == torch.float32 and y.shape[2] == width and y.is_contiguous(),
              "slabs must be contiguous float32 [slabs, N, H]")
        return y.shape[1], y.shape[0], y.shape[1] * width
    _need(y.dim() == 2 and y.shape[1] == width and y.is_contiguous() and y.dtype in (torch.float32, torch.bfloat16),
          "the input must be contiguous [N, H], float32 or bfloat16")
    return y.shape[0], 1, 0


def layer_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
               rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``(x - mean) / sqrt(mean((x - mean)^2) + eps) * weight`` over each row (of ``x[rows]`` if given), in
    ``out_dtype``; statistics and arithmetic in float32."""
    _dev(x, weight, rows)
    width = x.shape[-1]
    _need(weight.dtype == torch.float32 and weight.shape == (width,) and weight.is_contiguous(),
          "the norm's weight must be float32 [H]")
    n, nslabs, stride = _source(x, width)
    m = n
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous() and nslabs == 1,
              "rows must be int32 [M] and pick rows of a plain input")
        m = rows.shape[0]
    out = torch.empty((m, width), dtype=out_dtype, device=x.device)
    fn = _fn("rownorm", "qvl_layer_norm", _LN_ARGS)
    _check(fn(_ptr(x), dtype_code(x.dtype), nslabs, stride, _ptr(weight), float(eps), None, _ptr(out),
              dtype_code(out_dtype), _ptr(rows), m, width, _stream()), "layer_norm")
    return out


def layer_norm_add_(h: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float,
                    copy_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """``h += layer_norm(y) * weight`` in float32, in place (``y``: ``[N, H]`` or float32 slabs of it, added in
    order).  With ``copy_dtype`` the new rows of ``h`` are also returned in that dtype."""
    _dev(h, y, weight)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "h must be contiguous float32 [N, H]")
    n, width = h.shape
    _need(weight.dtype == torch.float32 and weight.shape == (width,) and weight.is_contiguous(),
          "the norm's weight must be float32 [H]")
    rows, nslabs, stride = _source(y, width)
    _need(rows == n, "the addend must have h's rows")
    out = None if copy_dtype is None else torch.empty((n, width), dtype=copy_dtype, device=h.device)
    fn = _fn("rownorm", "qvl_layer_norm", _LN_ARGS)
    _check(fn(_ptr(y), dtype_code(y.dtype), nslabs, stride, _ptr(weight), float(eps), _ptr(h), _ptr(out),
              dtype_code(copy_dtype) if copy_dtype is not None else 0, None, n, width, _stream()), "layer_norm_add")
    return out


def normed_powers(z: torch.Tensor, coeff: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """``a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e`` over each row of ``z [N, I]``, powers element by
    element, ``rms(u) = sqrt(mean(u^2) + eps)``, ``coeff = (a, b, c, e)`` float32."""
    _dev(z, coeff)
    _need(z.dim() == 2 and z.is_contiguous() and z.dtype in (torch.float32, torch.bfloat16), "z must be contiguous [N, I]")
    _need(coeff.dtype == torch.float32 and coeff.shape == (4,) and coeff.is_contiguous(), "coeff must be float32 [4]")
    out = torch.empty(z.shape, dtype=out_dtype, device=z.device)
    fn = _fn("rownorm", "qvl_normed_powers", [_c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(z), dtype_code(z.dtype), _ptr(coeff), float(eps), _ptr(out), dtype_code(out_dtype), z.shape[0],
              z.shape[1], _stream()), "normed_powers")
    return out


def squared_relu_(z: torch.Tensor) -> torch.Tensor:
    """``z = max(z, 0)^2`` in place."""
    _dev(z)
    _need(z.is_contiguous(), "z must be contiguous")
    fn = _fn("rownorm", "qvl_squared_relu", [_c_ptr, _c_ptr, _c_ll, _c_int, _c_ptr])
    _check(fn(_ptr(z), _ptr(z), z.numel(), dtype_code(z.dtype), _stream()), "squared_relu")
    return z
