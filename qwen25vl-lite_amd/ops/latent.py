"""Python entry points of the row-wise kernels of attention through a latent (``csrc/latent.hip``)."""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .kernels import _check, _dev, _fn, _need, _ptr, _stream, dtype_code

__all__ = ["latent_down", "latent_query_rotate_"]

_c_int, _c_float, _c_ptr, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong


def latent_down(proj: torch.Tensor, q_rank: int, q_norm: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype, *,
                kv_rank: int = 0, rot_dim: int = 0, kv_norm: Optional[torch.Tensor] = None,
                cs: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None,
                k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
                interleaved: bool = False) -> Optional[torch.Tensor]:
    """From the rows ``[query latent | key/value latent | rotated key part]`` of ``proj``: the RMS-normed query
    latent ``[N, q_rank]`` is returned; with ``k_cache`` the RMS-normed key/value latent and, behind it, the
    rotated key part go into the token's slot of ``k_cache [pages, 1, page_size, kv_rank + rot_dim]`` and the
    normed latent alone into ``v_cache [pages, 1, kv_rank, page_size]`` (``slots`` int32 ``[N]``, -1: nothing is
    written).  ``cs`` float32 ``[N, half, 2]`` holds (cos, sin) of the angles: channel i < half of the rotated
    part is paired with channel i + half (``interleaved``: channel 2i with channel 2i + 1), channels from ``2 half``
    on pass unchanged.  ``q_rank`` 0: the rows hold no query latent and nothing is returned."""
    _dev(proj, q_norm, kv_norm, cs, slots, k_cache, v_cache)
    n = proj.shape[0]
    write = k_cache is not None
    cols = q_rank + ((kv_rank + rot_dim) if write else 0)
    _need(proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= cols and proj.dtype in (torch.float32, out_dtype),
          "proj must be [N, at least the latents' columns], float32 or of the output's dtype")
    _need(q_rank >= 0 and (q_rank > 0 or write), "rows without a query latent hold a key/value latent")
    _need(q_rank == 0 or (q_norm is not None and q_norm.dtype == torch.float32 and q_norm.shape == (q_rank,)
                          and q_norm.is_contiguous()), "the query latent's norm weight must be float32 [q_rank]")
    half, ps = 0, 0
    if write:
        _need(kv_rank > 0 and rot_dim >= 0, "a cached latent has a size")
        _need(kv_norm is not None and kv_norm.dtype == torch.float32 and kv_norm.shape == (kv_rank,)
              and kv_norm.is_contiguous(), "the latent's norm weight must be float32 [kv_rank]")
        _need(slots is not None and slots.dtype == torch.int32 and slots.shape == (n,) and slots.is_contiguous(),
              "slots must be int32 [N]")
        ps = k_cache.shape[2]
        _need(k_cache.dtype == v_cache.dtype == out_dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
              and tuple(k_cache.shape[1:]) == (1, ps, kv_rank + rot_dim)
              and tuple(v_cache.shape) == (k_cache.shape[0], 1, kv_rank, ps),
              "the cache must be [pages, 1, page_size, kv_rank + rot_dim] and [pages, 1, kv_rank, page_size]")
        if cs is not None:
            half = cs.shape[1]
            _need(cs.dtype == torch.float32 and cs.dim() == 3 and cs.is_contiguous() and cs.shape[0] >= n
                  and cs.shape[2] == 2 and 2 * half <= rot_dim, "cs must be float32 [N, half, 2] with 2 half <= rot_dim")
    cq = torch.empty((n, q_rank), dtype=out_dtype, device=proj.device) if q_rank else None
    fn = _fn("latent", "qvl_latent_down", [_c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr,
                                           _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(proj), proj.stride(0), dtype_code(proj.dtype), int(q_rank), int(kv_rank), int(rot_dim),
              _ptr(q_norm) if q_rank else None,
              _ptr(kv_norm) if write else None, float(eps), _ptr(cs) if half else None, half,
              _ptr(slots) if write else None, _ptr(cq), _ptr(k_cache) if write else None,
              _ptr(v_cache) if write else None, ps, dtype_code(out_dtype), n, int(bool(interleaved)), _stream()),
           "latent_down")
    return cq


def latent_query_rotate_(q: torch.Tensor, heads: int, dim: int, rot_dim: int, kv_rank: int, cs: Optional[torch.Tensor],
                         out: torch.Tensor, interleaved: bool = False) -> torch.Tensor:
    """The rotated part of every head's query (columns ``[dim, dim + rot_dim)`` of its ``dim + rot_dim`` in ``q``)
    turned by ``cs`` and written into columns ``[kv_rank, kv_rank + rot_dim)`` of the head's slot of
    ``out [N, heads, kv_rank + rot_dim]``; the other columns of ``out`` are left as they are."""
    _dev(q, cs, out)
    n = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] == heads * (dim + rot_dim), "q must be [N, heads (dim + rot_dim)]")
    _need(out.is_contiguous() and tuple(out.shape) == (n, heads, kv_rank + rot_dim) and q.dtype in (torch.float32, out.dtype),
          "out must be contiguous [N, heads, kv_rank + rot_dim]; q float32 or of its dtype")
    half = 0
    if cs is not None:
        half = cs.shape[1]
        _need(cs.dtype == torch.float32 and cs.dim() == 3 and cs.is_contiguous() and cs.shape[0] >= n and cs.shape[2] == 2
              and 2 * half <= rot_dim, "cs must be float32 [N, half, 2] with 2 half <= rot_dim")
    fn = _fn("latent", "qvl_latent_query", [_c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_ptr,
                                            _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(q), q.stride(0), dtype_code(q.dtype), int(heads), int(dim), int(rot_dim), int(kv_rank),
              _ptr(cs) if half else None, half, _ptr(out), dtype_code(out.dtype), n, int(bool(interleaved)), _stream()),
           "latent_query")
    return out
