"""Python entry points of the kernels of a feed-forward with routed experts (``csrc/moe.hip``).

As in :mod:`~qwen25vl_lite_amd.ops.kernels`, every function checks on the host what the kernel and
its grid assume and launches on the current stream; there is no CPU path.  Nothing here reads
device data on the host: how many pairs an expert got stays on the device, and the grids are sized
for the worst case, so a step through these kernels may be captured in a HIP graph.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from .kernels import _check, _dev, _fn, _need, _ptr, _stream, dtype_code

__all__ = ["route", "sort_pairs", "pairs_by_column", "expert_products", "combine", "SCORE_FUNCTIONS", "BIG_TILE_PAIRS"]

_c_int, _c_float, _c_ptr, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong
SCORE_FUNCTIONS = {"sigmoid": 0, "softmax": 1}
PLAIN_ACTS = {None: 0, "relu2": 1}
# from this many pairs per expert on (on average) the matrix-core kernels with tiles of 128 pairs through LDS run
BIG_TILE_PAIRS = 32


def route(logits: torch.Tensor, top: int, groups: int = 1, keep: int = 1, scale: float = 1.0,
          score: str = "sigmoid", normalize: bool = True, floor: float = 1e-20) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(chosen int32 [N, top], weights float32 [N, top])`` from float32 router logits ``[N, E]``.

    Scores are ``sigmoid`` or ``softmax`` of the logits.  Experts ``e`` with the same ``e // (E / groups)`` are one
    group, ranked by the sum of its top two scores; the ``top`` experts with the highest scores are
    picked among the members of the ``keep`` highest-ranked groups.  The weights are the chosen
    scores, divided by their sum plus ``floor`` if ``normalize``, times ``scale``."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(),
          "router logits must be contiguous float32 [N, E]")
    n, e = logits.shape
    _need(score in SCORE_FUNCTIONS, f"score must be one of {sorted(SCORE_FUNCTIONS)}")
    _need(groups > 0 and e % groups == 0 and 0 < keep <= groups and 0 < top <= keep * (e // groups),
          "the experts must divide into the groups, and the kept groups must hold enough experts")
    ids = torch.empty((n, top), dtype=torch.int32, device=logits.device)
    wts = torch.empty((n, top), dtype=torch.float32, device=logits.device)
    fn = _fn("moe", "qvl_moe_route", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                                      _c_int, _c_float, _c_ptr])
    _check(fn(_ptr(logits), _ptr(ids), _ptr(wts), n, e, int(top), int(groups), int(keep), float(scale),
              SCORE_FUNCTIONS[score], int(bool(normalize)), float(floor), _stream()), "moe route")
    return ids, wts


def sort_pairs(ids: torch.Tensor, num_experts: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(sorted int32 [P], offsets int32 [E + 1])``: the pairs ``p = token * top + choice`` listed by
    the expert they chose; expert ``e`` has places ``offsets[e] .. offsets[e + 1]``."""
    _dev(ids)
    _need(ids.dtype == torch.int32 and ids.is_contiguous(), "ids must be contiguous int32")
    p = ids.numel()
    order = torch.empty(p, dtype=torch.int32, device=ids.device)
    offsets = torch.empty(num_experts + 1, dtype=torch.int32, device=ids.device)
    fn = _fn("moe", "qvl_moe_sort", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(ids), _ptr(order), _ptr(offsets), p, int(num_experts), _stream()), "moe sort")
    return order, offsets


def pairs_by_column(rows: int, columns: int, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(order, offsets)`` as :func:`sort_pairs` gives them for ``ids[row, c] = c``: pair ``row * columns + c``
    belongs to "expert" ``c``.  With it :func:`expert_products` multiplies slice ``c`` of every row of a
    ``[rows, columns, K]`` tensor by a matrix of its own (a product per head)."""
    order = torch.arange(rows * columns, dtype=torch.int32, device=device).view(rows, columns).t().contiguous().view(-1)
    offsets = torch.arange(columns + 1, dtype=torch.int32, device=device) * rows
    return order, offsets


def expert_products(x: torch.Tensor, weight: torch.Tensor, order: torch.Tensor, offsets: torch.Tensor, pairs: int,
                    div: int, out_dtype: torch.dtype, gated: Optional[Tuple[float, Optional[float], float]] = None,
                    act: Optional[str] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[p] = x[p // div] @ weight[e(p)].T`` for every pair ``p``, ``e(p)`` the expert whose range
    of ``order`` holds it; ``weight`` is ``[E, R, K]``.  With ``gated = (alpha, limit, shift)``,
    ``weight`` is ``[E, 2 R, K]`` (R gate rows, then R up rows) and
    ``out[p] = g sigmoid(alpha g) (u + shift)`` with ``g`` capped at ``limit`` and ``u`` clamped to
    ``[-limit, limit]`` (``limit`` None: no clamps).  Without ``gated``, ``act`` ``"relu2"`` squares the positive
    part of every value of the product.  Returns ``[pairs, R]`` in ``out_dtype``; with ``out`` (``[pairs, R]`` of
    that dtype, rows any number of values apart) the result goes there."""
    _dev(x, weight, order, offsets)
    _need(weight.dim() == 3 and weight.is_contiguous() and x.dim() == 2 and x.stride(1) == 1
          and x.dtype == weight.dtype and x.shape[1] == weight.shape[2], "x [M, K] and weight [E, rows, K] of one dtype")
    e, rows_w, k = weight.shape
    r = rows_w // 2 if gated else rows_w
    _need(not gated or rows_w % 2 == 0, "gate and up rows come in equal numbers")
    _need(act in PLAIN_ACTS and not (gated and act), "a plain product's activation is None or 'relu2'")
    _need(order.dtype == torch.int32 and order.shape == (pairs,) and offsets.dtype == torch.int32
          and offsets.shape == (e + 1,), "order must be int32 [pairs], offsets int32 [E + 1]")
    _need(pairs <= x.shape[0] * div, "a pair's row lies outside x")
    _need(out_dtype == x.dtype or (x.dtype == torch.bfloat16 and out_dtype == torch.float32),
          "float32 operands give float32; bfloat16 operands give either")
    if out is None:
        out = torch.empty((pairs, r), dtype=out_dtype, device=x.device)
    _dev(out)
    _need(out.dtype == out_dtype and tuple(out.shape) == (pairs, r) and out.stride(1) == 1 and out.stride(0) >= r,
          "out must be [pairs, R] of the output's dtype with contiguous rows")
    alpha, limit, shift = gated if gated else (1.0, None, 0.0)
    fn = _fn("moe", "qvl_moe_experts", [_c_ptr, _c_ll, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int,
                                        _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float, _c_int, _c_int,
                                        _c_ptr])
    _check(fn(_ptr(x), x.stride(0), dtype_code(x.dtype), _ptr(weight), _ptr(order), _ptr(offsets), _ptr(out),
              out.stride(0), dtype_code(out_dtype), int(pairs), e, r, k, int(div), int(bool(gated)), float(alpha), float(limit or 0.0),
              float(shift), PLAIN_ACTS[act], int(pairs >= BIG_TILE_PAIRS * e), _stream()), "moe experts")
    return out


def combine(y: torch.Tensor, weights: torch.Tensor, extra: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 ``[N, H]``: ``sum_k weights[n, k] * y[n top + k]`` in the order of ``k``, plus
    ``extra[n]`` (``[N, H]`` float32 or bfloat16, or float32 slabs ``[slabs, N, H]`` added in order)."""
    _dev(y, weights, extra)
    n, top = weights.shape
    _need(weights.dtype == torch.float32 and weights.is_contiguous(), "weights must be contiguous float32 [N, top]")
    _need(y.dim() == 2 and y.shape[0] == n * top and y.is_contiguous(), "y must be contiguous [N top, H]")
    h = y.shape[1]
    nslabs, stride, xdt = 1, 0, 0
    if extra is not None:
        if extra.dim() == 3:
            _need(extra.dtype == torch.float32 and tuple(extra.shape[1:]) == (n, h) and extra.is_contiguous(),
                  "slabs must be contiguous float32 [slabs, N, H]")
            nslabs, stride = extra.shape[0], n * h
        else:
            _need(tuple(extra.shape) == (n, h) and extra.is_contiguous(), "extra must be contiguous [N, H]")
        xdt = dtype_code(extra.dtype)
    out = torch.empty((n, h), dtype=torch.float32, device=y.device)
    fn = _fn("moe", "qvl_moe_combine", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_ll, _c_ptr, _c_int, _c_int,
                                        _c_int, _c_ptr])
    _check(fn(_ptr(y), dtype_code(y.dtype), _ptr(weights), _ptr(extra), xdt, nslabs, stride, _ptr(out), n, top, h,
              _stream()), "moe combine")
    return out
