"""A plain, slow implementation of the Rofapel decoder: whole sequences, no cache, dense masks, one function
per mechanism, on the CPU.  It reads config.json and the safetensors file by itself and shares no code with
the engine; the engine's logits are compared with it.

Notation: ``x`` is ``[T, width]``, a linear weight is ``[out, in]`` and applied as ``x @ W.T``.  ``store`` is
applied to whatever the engine may keep in bfloat16 (what a matrix product reads and gives, the short
convolution's result); norms, angles, scores, softmax weights, the router and the residual sum stay in the
working precision.
"""

from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional

import torch


def _keep(x: torch.Tensor) -> torch.Tensor:
    return x


def to_bfloat16_and_back(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


def rofapel_read(model_dir: str, dtype=torch.float64):
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
    """The last axis divided by its root mean square, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """A layer's norm: the weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def frequencies(rot: dict) -> torch.Tensor:
    """``base^(-2i/dims)``, ``i < dims/2``, in float64."""
    dims = int(rot["dims"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    return float(rot["base"]) ** (-2.0 * i / dims)


def ramp_frequencies(rot: dict):
    """Frequencies stretched by a ramp over the pair index, and the factor on cosines and sines."""
    f, sc = frequencies(rot), rot.get("scaling")
    if not sc:
        return f, 1.0
    dims, base = int(rot["dims"]), float(rot["base"])

    def index_of(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(sc["fast"])), 0)
    hi = min(math.ceil(index_of(sc["slow"])), dims - 1)
    i = torch.arange(dims // 2, dtype=torch.float64)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def divided_frequencies(rot: dict):
    f, sc = frequencies(rot), rot.get("scaling")
    return (f / sc["factor"] if sc else f), 1.0


def scaled_frequencies(rot: dict):
    """``(frequencies, amplitude)`` by what ``rot.scaling`` holds: nothing, a factor alone, or the ramp's four numbers."""
    sc = rot.get("scaling")
    return ramp_frequencies(rot) if sc and "original" in sc else divided_frequencies(rot)


def window_of(m: dict) -> Optional[int]:
    return int(m["mask"]["size"]) if m.get("mask") else None


def rotate(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor, amplitude: float, pairs: str) -> torch.Tensor:
    """``x [T, heads, d]``: the first ``2 len(freqs)`` channels of every head turned by ``pos * freqs``;
    ``pairs`` ``"halves"`` (channel i with i + dims/2) or ``"neighbours"`` (2i with 2i + 1)."""
    dims = 2 * freqs.shape[0]
    if dims == 0:
        return x
    angle = pos.to(torch.float64)[:, None] * freqs[None, :]
    c = (torch.cos(angle) * amplitude).to(x.dtype)[:, None, :]
    s = (torch.sin(angle) * amplitude).to(x.dtype)[:, None, :]
    out = x.clone()
    if pairs == "halves":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    return out


def causal_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``y_t = sum_j w[:, j] u_(t - taps + 1 + j)`` per channel, zeros before the first row; ``w [C, taps]``."""
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], dim=0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + u.shape[0]] * w[:, j]
    return y


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: Optional[int] = None,
           sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]`` -> ``[T, H, dv]``.  Query i sees key j with
    ``0 <= i - j`` (``< window`` if there is one); ``sink[h]`` joins head h's denominator as ``exp(sink[h])``."""
    t, heads = q.shape[0], q.shape[1]
    per = heads // k.shape[1]
    i = torch.arange(t)
    seen = i[None, :] <= i[:, None]
    if window is not None:
        seen = seen & (i[:, None] - i[None, :] < window)
    out = torch.zeros(t, heads, v.shape[-1], dtype=q.dtype)
    for h in range(heads):
        g = h // per
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, -math.inf)
        top = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[h].expand_as(top))
        e = torch.exp(s - top)
        total = e.sum(dim=-1, keepdim=True)
        if sink is not None:
            total = total + torch.exp(sink[h] - top)
        out[:, h] = (e / total) @ v[:, g]
    return out


# --------------------------------------------------------------------------------------------
# mixers
# --------------------------------------------------------------------------------------------
def attention(x, pos, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float, store: Callable = _keep):
    """One norm over all query channels, one over all key channels; rotation in halves; a gate per head."""
    n, heads, groups, d, dv = x.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = store(x @ t[p + "q"].T), store(x @ t[p + "k"].T), store(x @ t[p + "v"].T)
    q = unit_rms(q, eps) * t[p + "q.norm"]
    k = unit_rms(k, eps) * t[p + "k.norm"]
    f, amp = scaled_frequencies(m["rot"])
    q = store(rotate(q.view(n, heads, d), pos, f, amp, "halves"))
    k = store(rotate(k.view(n, groups, d), pos, f, amp, "halves"))
    o = attend(q, k, v.view(n, groups, dv), m["scale"], window=window_of(m))
    o = store(o) * torch.sigmoid(x @ t[p + "g"].T)[:, :, None]
    return store(o).reshape(n, heads * dv) @ t[p + "o"].T


def attention_2(x, pos, t, p: str, m: dict, eps: float, store: Callable = _keep):
    """Queries and keys through a short convolution; values are the keys behind it; a norm per head; rotation
    in halves with divided frequencies; a window; a sink; a gate per head."""
    n, heads, groups, d = x.shape[0], m["heads"], m["kv_heads"], m["dim"]
    q = causal_conv(store(x @ t[p + "q"].T), t[p + "q.conv"])
    k = causal_conv(store(x @ t[p + "k"].T), t[p + "k.conv"])
    v = store(k).view(n, groups, d)
    qn = unit_rms(q.view(n, heads, d), eps) * t[p + "q.norm"]
    kn = unit_rms(k.view(n, groups, d), eps) * t[p + "k.norm"]
    f, amp = scaled_frequencies(m["rot"])
    qn, kn = store(rotate(qn, pos, f, amp, "halves")), store(rotate(kn, pos, f, amp, "halves"))
    o = attend(qn, kn, v, m["scale"], window=window_of(m), sink=t[p + "sink"])
    o = store(o) * torch.sigmoid(x @ t[p + "g"].T)[:, :, None]
    return store(o).reshape(n, heads * d) @ t[p + "o"].T


def latent_attention(x, pos, t, p: str, m: dict, eps: float, store: Callable = _keep):
    """Keys and values of every head from one normed latent per token, plus one rotated key part for all heads."""
    n, heads, d, dr, dv, r = x.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = store(x @ t[p + "q"].T).view(n, heads, d + dr)
    down = x @ t[p + "dkv"].T
    c = store(unit_rms(down[:, :r], eps) * t[p + "dkv.norm"])
    f, amp = scaled_frequencies(m["rot"])
    k_rot = store(rotate(down[:, r:].reshape(n, 1, dr), pos, f, amp, "neighbours"))
    q_rot = store(rotate(q[..., d:], pos, f, amp, "neighbours"))
    k_plain = (c @ t[p + "uk"].T).view(n, heads, d)
    v = (c @ t[p + "uv"].T).view(n, heads, dv)
    o = attend(torch.cat([q[..., :d], q_rot], dim=-1), torch.cat([k_plain, k_rot.expand(n, heads, dr)], dim=-1), v,
               m["scale"], window=window_of(m))
    return store(o).reshape(n, heads * dv) @ t[p + "o"].T


MIXERS = {"attention": attention, "attention_2": attention_2, "latent_attention": latent_attention}


# --------------------------------------------------------------------------------------------
# feed-forwards
# --------------------------------------------------------------------------------------------
def gated_ff(x, t, p: str, store: Callable = _keep):
    return store(silu(store(x @ t[p + "gate"].T)) * store(x @ t[p + "up"].T)) @ t[p + "down"].T


def route(z: torch.Tensor, top: int):
    """The ``top`` largest logits of every row and the softmax over just those."""
    values, chosen = z.topk(top, dim=-1)
    return chosen, torch.softmax(values, dim=-1)


def moe_ff(x, t, p: str, mlp: dict, store: Callable = _keep):
    z = x @ t[p + "router"].T + t[p + "router.b"]
    chosen, weights = route(z, int(mlp["router"]["top"]))
    out = torch.zeros_like(x)
    for e in range(int(mlp["router"]["experts"])):
        rows, place = (chosen == e).nonzero(as_tuple=True)
        if rows.numel():
            out[rows] += weights[rows, place][:, None] * gated_ff(x[rows], t, f"{p}e{e}.", store)
    if mlp.get("shared"):
        out = out + gated_ff(x, t, p + "shared.", store)
    return out


def feed_forward(x, t, p: str, mlp: dict, store: Callable = _keep):
    return gated_ff(x, t, p, store) if mlp["kind"] == "dense" else moe_ff(x, t, p, mlp, store)


# --------------------------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------------------------
def layer(cfg: dict, t, i: int, x, pos, store: Callable = _keep):
    lay, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}."
    y = MIXERS[lay["type"]](store(norm_one_plus(x, t[p + "norm1"], eps)), pos, t, p + "mix.", lay["mixer"], eps, store)
    if lay.get("mlp") is not None:
        y = y + feed_forward(store(norm_one_plus(x, t[p + "norm2"], eps)), t, p + "mlp.", lay["mlp"], store)
    return x + y


def run_order(cfg: dict) -> List[tuple]:
    """``(layer, pass or None)``: ``pass`` is the number of the pass that begins at this layer."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for k in range(loop["times"]):
        order += [(i, k if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def rofapel_forward(cfg: dict, t, tokens: List[int], store: Callable = _keep, trace: Optional[list] = None):
    """Logits ``[T, vocab]`` of a whole sequence."""
    pos = torch.arange(len(tokens))
    first = t["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    x = first
    for i, begins in run_order(cfg):
        if begins is not None:
            x = store(torch.cat([x, first], dim=-1)) @ t["loop.in"].T + t["loop.step"][begins]
        x = layer(cfg, t, i, x, pos, store)
        if trace is not None:
            trace.append(x)
    return store(norm_one_plus(x, t["final.norm"], cfg["norm"]["eps"])) @ t["head"].T
