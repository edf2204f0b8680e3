"""Dispatch to the linear-attention kernels (``csrc/linear_attention.hip``, compiled per key size).

``S_t = diag(a_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` per head, with the state of every
request in its slot's row of a float32 tensor ``[slots, heads, dim, vdim]``.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

import torch

from .kernels import _check, _dev, _fn, _need, _ptr, _stream, dtype_code

__all__ = ["decayed_scan", "scan_groups", "chunked_scan", "plan_chunks", "ChunkPlan", "MAX_KEY_SIZE", "CHUNK"]

_c_int, _c_float, _c_ptr, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong
MAX_KEY_SIZE = 512
LONG_RUN = 64
BLOCKS_PER_CU = 2
MIN_ROWS = 4
CHUNK = 64            # tokens of a chunk when long runs are scanned in chunks side by side
CHUNKED_FROM = 128    # a step whose longest run has this many tokens or more is scanned that way


def decayed_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, num_heads: int, dim: int, vdim: int,
                 state: torch.Tensor, cu_q: torch.Tensor, req_slots: torch.Tensor, *,
                 head_decay: Optional[torch.Tensor] = None, z: Optional[torch.Tensor] = None, tau: float = 1.0,
                 silu=False, q_scale: float = 1.0, groups: int = 1, out: Optional[torch.Tensor] = None,
                 lower: Optional[torch.Tensor] = None, z_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Run every request's tokens of the step through the recurrence, from and into ``state``.

    ``proj [N, cols]`` (float32 or bfloat16) holds, per token, ``heads * dim`` query columns from
    ``q_off``, as many key columns from ``k_off`` and ``heads * vdim`` value columns from ``v_off``;
    ``silu`` applies the activation as they are read (True: to all three; or a string naming which, e.g.
    ``"q"``), ``q_scale`` scales the queries.
    The decay is ``head_decay [heads]`` (float32, one constant per head) or, per token and key
    channel, ``sigmoid(z)^(1/tau)`` for float32 ``z [N, heads * dim]``, or, with ``lower`` (float32
    ``[heads * dim]``, and ``z_bias`` of the same shape or None), the floored forget gate
    ``lower + (1 - lower) sigmoid(z + z_bias)``, whose complement ``1 - decay`` is then the key (no key
    columns are read).  ``cu_q [R + 1]`` bounds each
    request's run of tokens, ``req_slots [R]`` names its row of ``state``.  Returns float32
    ``[groups, N, heads * vdim]``: with ``groups`` above 1 (2, 4 or 8; the key size must be a multiple
    of four times it) the key channels are cut into that many groups with blocks of their own, and the
    output is the sum of the slabs (see :func:`scan_groups`)."""
    _dev(proj, state, cu_q, req_slots, head_decay, z, lower, z_bias)
    h, d, v = int(num_heads), int(dim), int(vdim)
    n = proj.shape[0]
    _need(1 <= d <= MAX_KEY_SIZE, f"key sizes up to {MAX_KEY_SIZE} are built")
    _need(proj.dim() == 2 and proj.stride(1) == 1, "proj must be [N, cols] with contiguous rows")
    _check_forget(lower, z_bias, z, h * d)
    for off, width in ((q_off, h * d), (q_off if lower is not None else k_off, h * d), (v_off, h * v)):
        _need(0 <= off and off + width <= proj.shape[1], "q, k or v columns lie outside proj")
    _need(state.dtype == torch.float32 and state.dim() == 4 and tuple(state.shape[1:]) == (h, d, v)
          and state.is_contiguous(), "state must be contiguous float32 [slots, heads, dim, vdim]")
    for t in (cu_q, req_slots):
        _need(t.dtype == torch.int32 and t.dim() == 1 and t.is_contiguous(), "cu_q and req_slots must be int32")
    r = req_slots.shape[0]
    _need(cu_q.shape[0] == r + 1, "cu_q must have one more entry than there are requests")
    _need((head_decay is None) != (z is None), "exactly one of head_decay and z is needed")
    zstride = 0
    if head_decay is not None:
        _need(head_decay.dtype == torch.float32 and head_decay.shape == (h,) and head_decay.is_contiguous(),
              "head_decay must be float32 [heads]")
    else:
        _need(z.dtype == torch.float32 and z.shape == (n, h * d) and z.stride(1) == 1, "z must be float32 [N, heads dim]")
        _need(tau > 0, "tau must be positive")
        zstride = z.stride(0)
    _need(groups == 1 or (groups in (2, 4, 8) and d % (4 * groups) == 0),
          "groups must be 1, 2, 4 or 8 and divide a quarter of the key size")
    if out is None:
        out = torch.empty((groups, n, h * v), dtype=torch.float32, device=proj.device)
    _need(out.dtype == torch.float32 and out.shape == (groups, n, h * v) and out.is_contiguous() and out.is_cuda,
          "out must be contiguous float32 [groups, N, heads vdim]")
    fn = _fn("linear_attention", "qvl_la_scan",
             [_c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ll, _c_float, _c_ptr, _c_ptr, _c_ptr,
              _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr],
             {"LA_DIM": d})
    _check(fn(_ptr(proj), proj.stride(0), int(q_off), int(k_off), int(v_off), dtype_code(proj.dtype),
              _ptr(head_decay), _ptr(z), zstride, 1.0 / float(tau), _ptr(lower), _ptr(z_bias), _ptr(state), _ptr(cu_q),
              _ptr(req_slots), _ptr(out), out.stride(0), int(groups), r, h, d, v, silu_mask(silu), float(q_scale),
              _stream()), "decayed_scan")
    return out


def silu_mask(silu) -> int:
    """Which of q, k and v pass through silu as they are read, as the kernels' bit mask (1 q, 2 k, 4 v): True means
    all three, False or None none, a string names them (``"q"``, ``"qk"``, ...)."""
    if silu is True:
        return 7
    if not silu:
        return 0
    _need(set(silu) <= set("qkv"), "silu names some of q, k and v")
    return sum(bit for name, bit in (("q", 1), ("k", 2), ("v", 4)) if name in silu)


def _check_forget(lower, z_bias, z, width: int) -> None:
    if lower is None:
        _need(z_bias is None, "a bias on z belongs to the floored forget gate")
        return
    _need(z is not None, "the floored forget gate needs z")
    for t in (lower, z_bias):
        _need(t is None or (t.dtype == torch.float32 and t.shape == (width,) and t.is_contiguous()),
              "lower and z_bias must be float32 [heads dim]")


def scan_groups(num_reqs: int, max_run: int, num_heads: int, dim: int, vdim: int, device=None) -> int:
    """Into how many groups of key channels :func:`decayed_scan` is cut for a step.  A block walks its
    request's tokens one after the other, so the blocks, not the tokens, have to fill the device: runs
    of ``LONG_RUN`` tokens or more are cut until there are ``BLOCKS_PER_CU`` blocks a compute unit or
    a wave is down to ``MIN_ROWS`` rows of the state."""
    if max_run < LONG_RUN:
        return 1
    from .attention_mfma import _compute_units
    blocks = num_reqs * num_heads * ((vdim + 63) // 64)
    groups = 1
    while (groups < 8 and blocks * groups < BLOCKS_PER_CU * _compute_units(device)
           and dim % (8 * groups) == 0 and dim // (8 * groups) >= MIN_ROWS):
        groups *= 2
    return groups


@dataclass
class ChunkPlan:
    """A step's runs cut into chunks: ``chunk_cu [chunks + 1]`` (token bounds, chunks follow one another
    as the runs do), ``chunk_rows [chunks]`` (0, 1, ...: a chunk's row of the scratch state),
    ``req_first [R + 1]`` (the first chunk of each request), all int32 on the device."""

    chunks: int
    chunk_len: int
    chunk_cu: torch.Tensor
    chunk_rows: torch.Tensor
    req_first: torch.Tensor


def plan_chunks(cu_q_host: Sequence[int], device, chunk_len: int = CHUNK) -> ChunkPlan:
    bounds, first = [0], [0]
    for b, e in zip(cu_q_host[:-1], cu_q_host[1:]):
        at = b
        while at < e:
            at = min(at + chunk_len, e)
            bounds.append(at)
        first.append(len(bounds) - 1)
    n = len(bounds) - 1
    host = np.concatenate([np.asarray(bounds, np.int32), np.arange(n, dtype=np.int32), np.asarray(first, np.int32)])
    dev = torch.from_numpy(host).to(device)
    return ChunkPlan(n, chunk_len, dev[:n + 1], dev[n + 1:2 * n + 1], dev[2 * n + 1:])


def chunked_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, num_heads: int, dim: int, vdim: int,
                 state: torch.Tensor, plan: ChunkPlan, req_slots: torch.Tensor, *,
                 head_decay: Optional[torch.Tensor] = None, z: Optional[torch.Tensor] = None, tau: float = 1.0,
                 silu=False, q_scale: float = 1.0, lower: Optional[torch.Tensor] = None,
                 z_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """:func:`decayed_scan` for steps with long runs: the chunks of ``plan`` are scanned side by side
    from zero states, the states are carried from chunk to chunk, and what the state before a chunk
    adds to the chunk's outputs is one float32 matrix product per (chunk, head), ``(q_t P_t) S``
    with ``P_t`` the product of the decays from the chunk's first token to ``t``.  Returns float32
    ``[slabs, N, heads * vdim]`` whose sum over the slabs is the output (the last slab holds the
    second term)."""
    h, d, v = int(num_heads), int(dim), int(vdim)
    n = proj.shape[0]
    nch, clen = plan.chunks, plan.chunk_len
    scratch = torch.zeros((nch, h, d, v), dtype=torch.float32, device=proj.device)
    groups = scan_groups(nch, clen, h, d, v, proj.device)
    out = torch.empty((groups + 1, n, h * v), dtype=torch.float32, device=proj.device)
    decayed_scan(proj, q_off, k_off, v_off, h, d, v, scratch, plan.chunk_cu, plan.chunk_rows, head_decay=head_decay,
                 z=z, tau=tau, silu=silu, q_scale=q_scale, groups=groups, out=out[:groups], lower=lower, z_bias=z_bias)
    qp = torch.zeros((nch, h, clen, d), dtype=torch.float32, device=proj.device)
    last = torch.empty((nch, h, d), dtype=torch.float32, device=proj.device)
    defines = {"LA_DIM": d}
    fn = _fn("linear_attention", "qvl_la_prefix",
             [_c_ptr, _c_ll, _c_int, _c_int, _c_ptr, _c_ptr, _c_ll, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
              _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr], defines)
    _check(fn(_ptr(proj), proj.stride(0), int(q_off), dtype_code(proj.dtype), _ptr(head_decay), _ptr(z),
              z.stride(0) if z is not None else 0, 1.0 / float(tau), _ptr(lower), _ptr(z_bias), _ptr(plan.chunk_cu),
              _ptr(qp), _ptr(last), nch, h, d, clen, silu_mask(silu), float(q_scale), _stream()), "chunk prefix")
    r = req_slots.shape[0]
    _need(plan.req_first.shape[0] == r + 1, "the chunk plan belongs to another step")
    fn = _fn("linear_attention", "qvl_la_carry", [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                                                   _c_ptr], defines)
    _check(fn(_ptr(scratch), _ptr(last), _ptr(state), _ptr(plan.req_first), _ptr(req_slots), r, h, d, v, _stream()),
           "chunk carry")
    corr = torch.matmul(qp, scratch)          # [chunks, heads, chunk_len, vdim], true float32
    fn = _fn("linear_attention", "qvl_la_gather", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
             defines)
    _check(fn(_ptr(corr), _ptr(plan.chunk_cu), _ptr(out[groups]), nch, h, clen, v, _stream()), "chunk gather")
    return out
