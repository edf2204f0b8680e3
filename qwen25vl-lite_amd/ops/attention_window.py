"""Dispatch to the matrix-core attention for windows that keep a request's first keys, for values
of another width than keys and for a softmax with one more term per head in its denominator
(bfloat16; key sizes in steps of 8 up to 256, value sizes up to 256).

The kernel is compiled per (key size, value size) at its first use.  Tiles are the other matrix-core
kernel's: 16 columns, a column being a (token, query head of one key/value group) pair.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .attention_mfma import _compute_units, _step_tiles, taken
from .kernels import _check, _fn, _need, _ptr, _stream

__all__ = ["try_attention", "supports"]

_c_int, _c_float, _c_ptr = ctypes.c_int, ctypes.c_float, ctypes.c_void_p
# below this many (tile, key/value head) pairs per compute unit the four waves of a block share a tile
SHARE_BELOW_PER_CU = 2


def supports(head_dim: int, value_dim: int, page_size: int, dtype: torch.dtype) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 8 == 0 and 0 < head_dim <= 256 and 0 < value_dim <= 256
            and page_size % 8 == 0)


def try_attention(q, k_cache, v_cache, block_table, step, num_q_heads: int, window: Optional[int], keep_first: int,
                  scale: float, share: Optional[bool] = None, sinks: Optional[torch.Tensor] = None
                  ) -> Optional[torch.Tensor]:
    """The attention through this kernel, or None if it does not take the shape.  ``share`` (tests):
    whether the waves of a block share a tile, else chosen by the number of tiles."""
    pages, nkv, ps, hd = k_cache.shape
    vd = v_cache.shape[2]
    if not supports(hd, vd, ps, q.dtype):
        return None
    n, nq = q.shape[0], int(num_q_heads)
    _need(q.is_cuda and q.shape == (n, nq * hd) and q.is_contiguous(), "q must be contiguous [N, nq hd] on the GPU")
    _need(k_cache.dtype == v_cache.dtype == torch.bfloat16 and k_cache.is_contiguous() and v_cache.is_contiguous()
          and tuple(v_cache.shape) == (pages, nkv, vd, ps), "cache must be bfloat16 [pages, nkv, ps, hd] / [.., vd, ps]")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
          and block_table.shape[0] == step.num_reqs, "block_table must be int32 [R, width]")
    _need(nq % nkv == 0, "query heads must be a multiple of key/value heads")
    _need(sinks is None or (sinks.is_cuda and sinks.dtype == torch.float32 and sinks.shape == (nq,)
                            and sinks.is_contiguous()), "sinks must be float32 [nq] on the GPU")
    group = nq // nkv
    defines = {"HD": hd, "VD": vd}
    tile_req, tile_ct, num_tiles = _step_tiles(step, group, 1, q.device)
    if share is None:
        share = num_tiles * nkv < SHARE_BELOW_PER_CU * _compute_units(q.device)
    cu_q = step.cu_q
    if share and step.max_q_len == 1 and num_tiles == step.num_reqs == len(step.cu_q_host) - 1 == step.cu_q_host[-1]:
        tile_req = tile_ct = cu_q = None     # decoded tokens only: request i brings token i and has tile i
    elif not share:
        # a wave owns an entry of several neighbouring column tiles
        wide = int(_fn("attention_window", "qvl_attn_window_entry_tiles", [], defines)())
        tile_req, tile_ct, num_tiles = _step_tiles(step, group, wide, q.device)
    out = torch.empty((n, nq * vd), dtype=q.dtype, device=q.device)
    fn = _fn("attention_window", "qvl_attn_window",
             [_c_ptr] * 4 + [_c_int] + [_c_ptr] * 4 + [_c_int, _c_ptr] + [_c_int] * 5 + [_c_float, _c_ptr, _c_int, _c_ptr],
             defines)
    _check(fn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(cu_q),
              _ptr(step.ctx_len), _ptr(tile_req), _ptr(tile_ct), num_tiles, _ptr(out), nq, nkv, ps, int(window or 0),
              int(keep_first) if window else 0, float(scale), _ptr(sinks), int(bool(share)), _stream()),
           "paged_attention (matrix cores, window with kept keys)")
    taken["window with kept keys, " + ("shared tiles" if share else "a wave per tile")] += 1
    return out
