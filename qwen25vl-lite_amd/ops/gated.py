"""Python entry points of the row-wise kernels of gated and normed sublayers (``csrc/gated.hip``).

As in :mod:`~qwen25vl_lite_amd.ops.kernels`, every function checks on the host what the kernel and
its grid assume and launches on the current stream; there is no CPU path.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .kernels import _check, _dev, _fn, _need, _ptr, _stream, dtype_code

__all__ = ["residual_add", "gated_act", "softcap_", "group_norm_gate", "head_gate_", "qk_norm_rope_write", "sandwich_norm",
           "row_inv_rms"]

_c_int, _c_float, _c_ptr, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong
GATE_ACTS = {None: 0, "sigmoid": 1, "silu": 2}


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> None:
    """``h += delta`` in float32.  ``delta`` is ``[N, H]`` (float32 or bfloat16) or float32
    ``[slabs, N, H]``, partial sums that are added in slab order."""
    _dev(h, delta)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "h must be contiguous float32 [N, H]")
    nslabs, stride = 1, 0
    if delta.dim() == 3:
        _need(delta.dtype == torch.float32 and tuple(delta.shape[1:]) == tuple(h.shape) and delta.is_contiguous(),
              "slabs of delta must be contiguous float32 [slabs, N, H]")
        nslabs, stride = delta.shape[0], h.numel()
    else:
        _need(delta.shape == h.shape and delta.is_contiguous(), "delta must match h's shape")
    fn = _fn("gated", "qvl_residual_add", [_c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_ll, _c_ptr])
    _check(fn(_ptr(h), _ptr(delta), h.numel(), dtype_code(delta.dtype), nslabs, stride, _stream()), "residual_add")


def gated_act(x: torch.Tensor, alpha: float = 1.0, limit: Optional[float] = None, shift: float = 0.0) -> torch.Tensor:
    """``g sigmoid(alpha g) (u + shift)`` for ``x`` of ``[N, 2 I]``, gate branch ``g`` in the first
    ``I`` columns and linear branch ``u`` in the rest; with ``limit`` the gate is capped from above
    at it and the linear branch clamped to ``[-limit, limit]`` first."""
    _dev(x)
    _need(x.dim() == 2 and x.shape[1] % 2 == 0 and x.is_contiguous(), "x must be contiguous [N, 2 I]")
    _need(limit is None or limit > 0, "a limit must be positive")
    n, inter = x.shape[0], x.shape[1] // 2
    out = torch.empty((n, inter), dtype=x.dtype, device=x.device)
    fn = _fn("gated", "qvl_gated_act", [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float, _c_ptr])
    _check(fn(_ptr(x), _ptr(out), n, inter, dtype_code(x.dtype), float(alpha), float(limit or 0.0), float(shift),
              _stream()), "gated_act")
    return out


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x = cap * tanh(x / cap)`` in place on float32."""
    _dev(x)
    _need(x.dtype == torch.float32 and x.is_contiguous(), "x must be contiguous float32")
    fn = _fn("gated", "qvl_softcap", [_c_ptr, _c_ll, _c_float, _c_ptr])
    _check(fn(_ptr(x), x.numel(), float(cap), _stream()), "softcap")
    return x


def group_norm_gate(x: torch.Tensor, weight: torch.Tensor, span: int, eps: float, out_dtype: torch.dtype,
                    gate: Optional[torch.Tensor] = None, gate_act: Optional[str] = None) -> torch.Tensor:
    """Every group of ``span`` consecutive channels of float32 ``x [N, C]`` (or of the sum of the
    slabs of ``x [slabs, N, C]``, added in order) divided by its root
    mean square, times ``weight[c % len(weight)]``, times ``sigmoid`` or ``silu`` of ``gate[n, c]``
    (``gate`` may be a view of columns of a wider tensor)."""
    _dev(x, weight, gate)
    _need(x.dtype == torch.float32 and x.dim() in (2, 3) and x.is_contiguous(),
          "x must be contiguous float32 [N, C] or [slabs, N, C]")
    nslabs = x.shape[0] if x.dim() == 3 else 1
    n, c = x.shape[-2:]
    _need(span > 0 and c % span == 0, "the width must be a multiple of the span")
    _need(weight.dtype == torch.float32 and weight.dim() == 1 and weight.is_contiguous()
          and weight.shape[0] in (span, c), "the weight must be float32 of one group's or the row's width")
    act = GATE_ACTS[gate_act] if gate is not None else 0
    gstride, gdtype = 0, dtype_code(out_dtype)
    if gate is not None:
        _need(gate.shape == (n, c) and gate.stride(1) == 1, "the gate must be [N, C] with contiguous rows")
        _need(gate.dtype in (torch.float32, out_dtype), "the gate must be float32 or of the output's dtype")
        gstride, gdtype = gate.stride(0), dtype_code(gate.dtype)
    out = torch.empty((n, c), dtype=out_dtype, device=x.device)
    fn = _fn("gated", "qvl_group_norm_gate", [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ll, _c_int, _c_ptr, _c_int, _c_int,
                                               _c_int, _c_int, _c_float, _c_int, _c_int, _c_ll, _c_ptr])
    _check(fn(_ptr(x), _ptr(weight), weight.shape[0], _ptr(gate), gstride, gdtype, _ptr(out), dtype_code(out_dtype),
              n, c, int(span), float(eps), act, nslabs, n * c, _stream()), "group_norm_gate")
    return out


def head_gate_(o: torch.Tensor, gate: torch.Tensor, num_heads: int) -> torch.Tensor:
    """``o[n, h, :] *= sigmoid(gate[n, h])`` in place; ``gate`` float32 ``[N, heads]``, possibly a
    view of columns of a wider tensor."""
    _dev(o, gate)
    n = o.shape[0]
    _need(o.dim() == 2 and o.is_contiguous() and o.shape[1] % num_heads == 0, "o must be contiguous [N, heads hd]")
    _need(gate.dtype == torch.float32 and gate.shape == (n, num_heads) and gate.stride(1) == 1,
          "gate must be float32 [N, heads] with contiguous rows")
    fn = _fn("gated", "qvl_head_gate", [_c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(o), _ptr(gate), gate.stride(0), n, num_heads, o.shape[1] // num_heads, dtype_code(o.dtype),
              _stream()), "head_gate")
    return o


def row_inv_rms(x: torch.Tensor, first: int, second: int, eps: float, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 ``[N, 2]``: ``1 / sqrt(mean(x[n, :first]^2) + eps)`` and the same over the next ``second`` columns
    (1 if there are none) of float32 ``x [N, >= first + second]``, ``bias`` added to the columns first."""
    _dev(x, bias)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1 and first > 0 and second >= 0
          and x.shape[1] >= first + second, "x must be float32 [N, at least the two ranges' columns]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.dim() == 1 and bias.shape[0] >= first + second
                           and bias.is_contiguous()), "the bias must be float32 over the ranges' columns")
    out = torch.empty((x.shape[0], 2), dtype=torch.float32, device=x.device)
    fn = _fn("gated", "qvl_row_inv_rms", [_c_ptr, _c_ll, _c_ptr, _c_int, _c_int, _c_float, _c_ptr, _c_int, _c_ptr])
    _check(fn(_ptr(x), x.stride(0), _ptr(bias), int(first), int(second), float(eps), _ptr(out), x.shape[0], _stream()),
           "row_inv_rms")
    return out


def qk_norm_rope_write(x: torch.Tensor, q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor], eps: float,
                       cs: torch.Tensor, slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                       v_cache: Optional[torch.Tensor], num_q_heads: int, num_kv_heads: int, head_dim: int,
                       page_size: int, out_dtype: torch.dtype, *, interleaved: bool, values_are_keys: bool,
                       norm: Optional[str] = "before", bias: Optional[torch.Tensor] = None,
                       value_dim: Optional[int] = None) -> torch.Tensor:
    """Per head: ``bias`` (float32 over all columns, or None) is added; RMS norm over the head
    (``norm`` ``"before"`` or ``"after"`` the rotation, None: no norm; weights ``q_norm`` / ``k_norm``
    of ``[head_dim]``, None: a gain of one; ``norm`` ``"whole"``: before the rotation and over all query heads of a
    token at once, and over all its key heads at once, with weights of ``[heads head_dim]``); rotation by the angles whose ``(cos, sin)`` are
    ``cs [N, rot/2, 2]``: pairs ``(2f, 2f+1)`` if ``interleaved``, else ``(f, f + rot/2)``.  Rotated
    queries are returned; rotated keys and the values go into the page slots (``slots`` None:
    queries only).  ``x`` is float32 ``[N, >= nq hd + nkv hd (+ nkv vd)]``: query heads, key heads, and value
    heads of ``value_dim`` channels unless ``values_are_keys``, in which case a key head as projected
    (before norm and rotation) is its own value."""
    _dev(x, q_norm, k_norm, cs, slots, k_cache, v_cache, bias)
    nq, nkv, hd = int(num_q_heads), int(num_kv_heads), int(head_dim)
    vd = hd if value_dim is None else int(value_dim)
    write = slots is not None
    n = x.shape[0]
    cols = nq * hd + ((nkv * hd + (0 if values_are_keys else nkv * vd)) if write else 0)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.shape[1] >= cols and x.stride(1) == 1,
          "x must be float32 [N, at least the heads' columns]")
    _need(norm in (None, "before", "after", "whole"), "the norm stands before or after the rotation, spans the whole "
          "projection, or is None")
    _need(not (values_are_keys and vd != hd), "keys that are their own values have the keys' width")
    for w, heads in ((q_norm, nq), (k_norm, nkv)):
        _need(w is None or (w.dtype == torch.float32 and w.shape == ((heads * hd,) if norm == "whole" else (hd,))
                            and w.is_contiguous()),
              "a head norm's weight must be float32 [head_dim], a whole projection's [heads head_dim]")
    row_rs = None
    if norm == "whole":
        row_rs = row_inv_rms(x, nq * hd, nkv * hd if write else 0, eps, bias)
    _need(bias is None or (bias.dtype == torch.float32 and bias.dim() == 1 and bias.shape[0] >= cols
                           and bias.is_contiguous()), "the bias must be float32 over the heads' columns")
    _need(cs.dtype == torch.float32 and cs.dim() == 3 and cs.is_contiguous() and cs.shape[0] >= n
          and cs.shape[2] == 2 and 2 * cs.shape[1] <= hd, "cs must be float32 [N, rot/2, 2] with rot <= head_dim")
    if write:
        _need(slots.dtype == torch.int32 and slots.shape == (n,) and slots.is_contiguous(), "slots must be int32 [N]")
        _need(k_cache is not None and v_cache is not None and k_cache.dtype == v_cache.dtype == out_dtype,
              "the cache must have the activation dtype")
        _need(k_cache.is_contiguous() and k_cache.dim() == 4 and tuple(k_cache.shape[1:]) == (nkv, page_size, hd),
              "k_cache must be [pages, nkv, page_size, hd]")
        _need(v_cache.is_contiguous() and tuple(v_cache.shape) == (k_cache.shape[0], nkv, vd, page_size),
              "v_cache must be [pages, nkv, vd, page_size]")
    q_out = torch.empty((n, nq * hd), dtype=out_dtype, device=x.device)
    fn = _fn("gated", "qvl_qk_norm_rope_write",
             [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
              _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_ptr])
    _check(fn(_ptr(x), x.stride(0), _ptr(bias), _ptr(q_norm), _ptr(k_norm), _ptr(cs), _ptr(slots), _ptr(q_out),
              _ptr(k_cache) if write else None, _ptr(v_cache) if write else None, n, nq, nkv, hd, vd, cs.shape[1],
              int(page_size), float(eps), int(interleaved), int(values_are_keys), int(write),
              {None: 0, "before": 1, "after": 2, "whole": 3}[norm], _ptr(row_rs), dtype_code(out_dtype), _stream()),
           "qk_norm_rope_write")
    return q_out


def sandwich_norm(h: torch.Tensor, y: Optional[torch.Tensor], gain: Optional[torch.Tensor], eps_y: float, factor: float,
                  vec: Optional[torch.Tensor], weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype,
                  rows: Optional[torch.Tensor] = None, weight2: Optional[torch.Tensor] = None):
    """``h += factor * rmsnorm(y) * gain + vec`` in float32 (``gain`` None: ``y`` is added as it is;
    ``y`` None: nothing of it; ``vec`` None or one float32 vector for every row; ``y`` may be float32
    slabs ``[slabs, N, H]``, added in order), then, if ``weight`` is given, ``rmsnorm(h) * weight`` in
    ``out_dtype`` is returned.  With ``rows`` only those rows are formed and ``h`` is not written.  With ``weight2``
    the normed rows are also formed under that second gain and the pair ``(under weight, under weight2)`` is returned."""
    _dev(h, y, gain, vec, weight, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "h must be contiguous float32 [N, H]")
    n, width = h.shape
    nslabs, stride = 1, 0
    if y is not None and y.dim() == 3:
        _need(y.dtype == torch.float32 and tuple(y.shape[1:]) == (n, width) and y.is_contiguous(),
              "slabs of y must be contiguous float32 [slabs, N, H]")
        nslabs, stride = y.shape[0], n * width
    elif y is not None:
        _need(y.shape == h.shape and y.is_contiguous() and y.dtype in (torch.float32, torch.bfloat16),
              "y must match h's shape, float32 or bfloat16")
    _need(weight2 is None or weight is not None, "a second gain comes with a first")
    for v in (gain, vec, weight, weight2):
        _need(v is None or (v.dtype == torch.float32 and v.shape == (width,) and v.is_contiguous()),
              "gains and vectors must be float32 [H]")
    m = n
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous(), "rows must be int32 [M]")
        _need(weight is not None, "rows are chosen for a norm's output")
        m = rows.shape[0]
    out = None if weight is None else torch.empty((m, width), dtype=out_dtype, device=h.device)
    out2 = None if weight2 is None else torch.empty((m, width), dtype=out_dtype, device=h.device)
    fn = _fn("gated", "qvl_sandwich_norm",
             [_c_ptr, _c_ptr, _c_int, _c_int, _c_ll, _c_ptr, _c_float, _c_float, _c_ptr, _c_ptr, _c_float, _c_ptr,
              _c_int, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr])
    _check(fn(_ptr(h), _ptr(y), dtype_code(y.dtype) if y is not None else 0, nslabs, stride, _ptr(gain), float(eps_y),
              float(factor), _ptr(vec), _ptr(weight), float(eps), _ptr(out), dtype_code(out_dtype), _ptr(rows), m,
              width, _ptr(weight2), _ptr(out2), _stream()), "sandwich_norm")
    return out if weight2 is None else (out, out2)
