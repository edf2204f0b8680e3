"""Python entry point of the short causal convolution with a per-request state (``csrc/short_conv.hip``)."""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .kernels import _check, _dev, _fn, _need, _ptr, _stream, dtype_code

__all__ = ["short_conv_add", "short_conv"]

_c_int, _c_ptr = ctypes.c_int, ctypes.c_void_p


def short_conv_add(x: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor], cu_q: torch.Tensor,
                   req_slots: torch.Tensor, token_req: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """:func:`short_conv` with the input added to the result."""
    return short_conv(x, weight, state, cu_q, req_slots, token_req, out_dtype, add_input=True)


def short_conv(x: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor], cu_q: torch.Tensor,
               req_slots: torch.Tensor, token_req: torch.Tensor, out_dtype: torch.dtype, *,
               add_input: bool = False) -> torch.Tensor:
    """``out[t] = [x[t] +] sum_j weight[j] * x[t - taps + 1 + j]`` over each request's tokens (``cu_q [R + 1]``
    bounds its run, ``token_req [N]`` names the request of a token), the inputs before a run coming from row
    ``req_slots[r]`` of ``state`` (float32 ``[slots, taps - 1, C]``, oldest first; zeros for a new request), which
    the run's last inputs replace.  ``x`` float32 ``[N, C]`` (rows may lie further apart: columns of a wider tensor), ``weight`` float32 ``[taps, C]`` (a tap's weights of all channels side by side); with one tap there
    is no state.  Returns ``[N, C]`` in ``out_dtype``."""
    _dev(x, weight, state, cu_q, req_slots, token_req)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1 and (x.shape[0] <= 1 or x.stride(0) >= x.shape[1]),
          "x must be float32 [N, C] with contiguous rows")
    n, c = x.shape
    _need(weight.dtype == torch.float32 and weight.dim() == 2 and weight.shape[1] == c and weight.is_contiguous(),
          "the weight must be contiguous float32 [taps, C]")
    taps = weight.shape[0]
    for t in (cu_q, req_slots, token_req):
        _need(t.dtype == torch.int32 and t.dim() == 1 and t.is_contiguous(), "cu_q, req_slots and token_req must be int32")
    r = req_slots.shape[0]
    _need(cu_q.shape[0] == r + 1 and token_req.shape[0] == n, "cu_q has one entry more than requests, token_req one per token")
    if taps > 1:
        _need(state is not None and state.dtype == torch.float32 and state.dim() == 3 and state.is_contiguous()
              and tuple(state.shape[1:]) == (taps - 1, c), "state must be contiguous float32 [slots, taps - 1, C]")
    out = torch.empty((n, c), dtype=out_dtype, device=x.device)
    fn = _fn("short_conv", "qvl_short_conv", [_c_ptr] * 7 + [_c_int] * 5 + [ctypes.c_longlong, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(weight), _ptr(state) if taps > 1 else None, _ptr(cu_q), _ptr(req_slots), _ptr(token_req),
              _ptr(out), dtype_code(out_dtype), n, r, c, taps, x.stride(0) if n > 1 else c, int(bool(add_input)),
              _stream()), "short_conv")
    return out
