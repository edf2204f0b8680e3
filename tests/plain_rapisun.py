"""A plain, slow implementation of the Rapisun decoder: whole sequences, no cache, dense masks,
token-by-token recurrences, one function per mechanism, on the CPU.  It reads config.json and the
safetensors file by itself and shares no code with the engine; the engine's logits are compared
with it.

Notation: ``x`` is ``[T, width]``, a linear weight is ``[out, in]`` and applied as ``x @ W.T``.
``store`` is applied to whatever the engine may keep in bfloat16 (matrix products, short convolutions
and their activations); norms, angles, scores, gates of the recurrence, the state, the router and the
residual sum stay in the working precision.
"""

from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional

import torch

WEIGHT_FLOOR = 1e-20   # added to the sum the routing weights are divided by


def _keep(x: torch.Tensor) -> torch.Tensor:
    return x


def to_bfloat16_and_back(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


def rapisun_read(model_dir: str, dtype=torch.float64):
    """``(config dict, {tensor name: tensor})`` with the names the file uses."""
    from safetensors import safe_open

    with open(os.path.join(model_dir, "config.json")) as fh:
        cfg = json.load(fh)
    tensors = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return cfg, tensors


# --------------------------------------------------------------------------------------------
# small pieces
# --------------------------------------------------------------------------------------------
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """Each row divided by its root mean square, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """Mean taken off, divided by the root of the mean squared deviation plus eps, times a weight; no bias."""
    centred = x - x.mean(dim=-1, keepdim=True)
    return centred / torch.sqrt((centred * centred).mean(dim=-1, keepdim=True) + eps) * w


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def causal_conv(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``h [T, C]``, ``w [C, taps]``: ``out_t = sum_j w[:, j] * h_(t - taps + 1 + j)``, zeros before the start."""
    t_len, taps = h.shape[0], w.shape[1]
    out = torch.zeros_like(h)
    for t in range(t_len):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


# --------------------------------------------------------------------------------------------
# rotation
# --------------------------------------------------------------------------------------------
def rotate_halves(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """``x [T, ..., n]``: of the first ``dims`` channels, channel i is paired with channel i + dims/2 and the
    pair turned by ``position * base^(-2i/dims)``; channels from ``dims`` on pass unchanged."""
    half = dims // 2
    if half == 0:
        return x
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = ang.cos().to(x.dtype).view(shape), ang.sin().to(x.dtype).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# --------------------------------------------------------------------------------------------
# mixers
# --------------------------------------------------------------------------------------------
def hgrn2(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
          store: Callable = _keep) -> torch.Tensor:
    """Linear attention whose forget gate also decides what is written: per head
    ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T q``, ``f = l + (1 - l) sigmoid(Wf h + b)``."""
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = store(silu(store(h @ t[p + "q"].T))).view(n, heads, dim)
    v = store(h @ t[p + "v"].T).view(n, heads, vdim)
    z = store(h @ t[p + "f"].T) + t[p + "f.b"]
    low = t[p + "lower"]
    f = (low + (1.0 - low) * torch.sigmoid(z)).view(n, heads, dim)
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    state = torch.zeros(heads, dim, vdim, dtype=h.dtype)
    for i in range(n):
        state = f[i][:, :, None] * state + (1.0 - f[i])[:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hdv,hd->hv", state, q[i])
    out = rms_norm(out, t[p + "norm"], eps)
    return store(out).reshape(n, heads * vdim) @ t[p + "o"].T


def latent_cache(h: torch.Tensor, positions: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                 store: Callable = _keep):
    """What a latent-attention layer keeps per token: ``(c [T, kv_rank], rotated key part [T, rot_dim])``."""
    rank = m["kv_rank"]
    down = store(h @ t[p + "dkv"].T)
    c = store(rms_norm(down[:, :rank], t[p + "dkv.norm"], eps))
    k_rot = store(rotate_halves(down[:, rank:], positions, m["rot"]["dims"], m["rot"]["base"]))
    return c, k_rot


def latent_attention(h: torch.Tensor, positions: torch.Tensor, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                     kept, store: Callable = _keep) -> torch.Tensor:
    """``kept``: ``(c, rotated key part)`` of this layer or of the layer it reads them from."""
    heads, dim, rot_dim, vdim = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    n = h.shape[0]
    c_q = store(rms_norm(store(h @ t[p + "dq"].T), t[p + "dq.norm"], eps))
    q = store(c_q @ t[p + "uq"].T).view(n, heads, dim + rot_dim)
    q_plain, q_rot = q[..., :dim], store(rotate_halves(q[..., dim:], positions, m["rot"]["dims"], m["rot"]["base"]))
    c, k_rot = kept
    k_plain = store(c @ t[p + "uk"].T).view(n, heads, dim)
    v = store(c @ t[p + "uv"].T).view(n, heads, vdim)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if m.get("mask"):
        seen = seen & (i - j < m["mask"]["size"])
    scores = scores.masked_fill(~seen[None], float("-inf"))
    sink = t[p + "sink"]
    top = torch.maximum(scores.max(dim=-1).values, sink[:, None])
    e = torch.exp(scores - top[..., None])
    w = e / (e.sum(dim=-1) + torch.exp(sink[:, None] - top))[..., None]
    o = torch.einsum("hij,jhv->ihv", w, v)
    return store(o).reshape(n, heads * vdim) @ t[p + "o"].T


# --------------------------------------------------------------------------------------------
# feed-forward
# --------------------------------------------------------------------------------------------
def poly_norm(z: torch.Tensor, coeff: torch.Tensor, eps: float) -> torch.Tensor:
    a, b, c, e = (coeff[i] for i in range(4))
    return a * unit_rms(z, eps) + b * unit_rms(z ** 2, eps) + c * unit_rms(z ** 3, eps) + e


def dense_ff(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, eps: float, store: Callable = _keep) -> torch.Tensor:
    return store(poly_norm(store(h @ t[p + "up"].T), t[p + "act"], eps)) @ t[p + "down"].T


def squared_relu_expert(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, store: Callable = _keep) -> torch.Tensor:
    return store(torch.relu(store(h @ t[p + "up"].T)) ** 2) @ t[p + "down"].T


def route(h: torch.Tensor, w_router: torch.Tensor, top: int):
    """``(chosen [T, top], weights [T, top])``: softmax over all experts, the ``top`` largest, their scores
    over their sum."""
    s = torch.softmax(h @ w_router.T, dim=-1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val / (val.sum(dim=-1, keepdim=True) + WEIGHT_FLOOR)


def moe_ff(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, mlp: dict, store: Callable = _keep) -> torch.Tensor:
    idx, w = route(h, t[p + "router"], mlp["router"]["top"])
    out = torch.zeros(h.shape[0], t[p + "e0.down"].shape[0], dtype=h.dtype)
    for n in range(h.shape[0]):
        for k in range(idx.shape[1]):
            e = int(idx[n, k])
            out[n] += w[n, k] * squared_relu_expert(h[n:n + 1], t, f"{p}e{e}.", store)[0]
    if mlp.get("shared"):
        out = out + squared_relu_expert(h, t, p + "shared.", store)
    return out


# --------------------------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------------------------
def rapisun_forward(cfg: dict, t: Dict[str, torch.Tensor], tokens: List[int], store: Callable = _keep,
                    layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence."""
    eps = cfg["norm"]["eps"]
    ids = torch.tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x = layer_norm(t["embed"][ids], t["embed.norm"], eps)
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = store(x)
        if cfg.get("canon"):
            h = store(h + causal_conv(h, t[p + "canon1"]))
        if layer["type"] == "hgrn2":
            y = hgrn2(h, t, p + "mix.", m, eps, store)
        else:
            src = m.get("kv_from")
            if src is None:
                kept[i] = latent_cache(h, positions, t, p + "mix.", m, eps, store)
            y = latent_attention(h, positions, t, p + "mix.", m, eps, kept[i if src is None else src], store)
        x = x + layer_norm(y, t[p + "norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = store(x)
            y = dense_ff(h, t, p + "mlp.", eps, store) if mlp["kind"] == "dense" else moe_ff(h, t, p + "mlp.", mlp, store)
            x = x + layer_norm(y, t[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return store(layer_norm(x, t["final.norm"], eps)) @ t["head"].T
