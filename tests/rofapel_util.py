"""Small Rofapel configurations and model folders with random weights for the tests.  The weights
are drawn here (not by the engine) and written with the safetensors package."""

from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch


def attention(heads, kv_heads, dim, vdim, base=10000.0, dims=None, scale=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "scale": scale or dim ** -0.5,
                                           "rot": {"base": base, "dims": dim if dims is None else dims}}}


def attention_2(heads, kv_heads, dim, mask, conv=3, base=10000.0, dims=None, scale=None, factor=2.0):
    rot = {"base": base, "dims": dim if dims is None else dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return {"type": "attention_2", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "conv": conv,
                                             "mask": {"size": mask}, "scale": scale or dim ** -0.5, "rot": rot}}


def latent(heads, dim, rot_dim, vdim, kv_rank, base=10000.0, scale=None, ramp=(4.0, 64, 16.0, 2.0)):
    rot = {"base": base, "dims": rot_dim}
    if ramp is not None:
        rot["scaling"] = {"factor": ramp[0], "original": ramp[1], "fast": ramp[2], "slow": ramp[3]}
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                                                  "kv_rank": kv_rank, "scale": scale or (dim + rot_dim) ** -0.5,
                                                  "rot": rot}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        mlp["shared"] = {"ff": shared}
    return mlp


def layer(mixer, mlp=None):
    return {**mixer, "mlp": mlp}


def config(width, vocab, layers, eps=1e-5, scale=2.5, loop=None):
    cfg = {"architecture": "Rofapel", "width": width, "vocab": vocab, "norm": {"eps": eps},
           "embedding": {"scale": scale}, "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# Sizes that all differ from one another: a layer before the looped range, three passes over two layers, two
# layers behind it; key/value groups of 1, 2 and 3 heads; values wider and narrower than keys; partial and full
# rotation; windows of 9 and 37 tokens; two and four taps; experts with and without a shared one; a layer
# without a feed-forward.
MIXED = config(72, 203, [
    layer(attention_2(4, 2, 16, mask=9, conv=2, base=500.0, dims=8, scale=0.6, factor=3.0), dense(88)),
    layer(latent(3, 16, 8, 24, 40, base=300.0, scale=0.3, ramp=(4.0, 48, 8.0, 1.5)), moe(6, 2, 40, shared=56)),
    layer(attention(6, 2, 24, 16, base=80.0, dims=16, scale=0.25), moe(5, 3, 24)),
    layer(attention_2(3, 3, 24, mask=37, conv=4, base=200.0, scale=0.3, factor=None)),
    layer(latent(2, 8, 16, 8, 24, base=50.0, scale=0.4, ramp=None), dense(40)),
], eps=1e-5, scale=1.7, loop=(1, 3, 3))

# The same shapes with score scales so large that the softmax picks single keys: a key lost at a window's
# edge or a page's border moves the logits.
SHARP = json.loads(json.dumps(MIXED))
for _i, _s in ((0, 4.0), (1, 2.0), (2, 1.5), (3, 2.5), (4, 2.5)):
    SHARP["layers"][_i]["mixer"]["scale"] = _s

# Values that happen to be 1 or equal: one head, one expert chosen of one, every expert chosen, a window of
# one token, one tap (a convolution without a state), one pass, an embedding scale of 1, a loop over all
# layers.
ONES = config(32, 61, [
    layer(attention_2(1, 1, 16, mask=1, conv=1, base=100.0, scale=1.0, factor=1.0), moe(1, 1, 16, shared=16)),
    layer(latent(1, 16, 16, 16, 16, base=100.0, scale=0.25, ramp=(1.0, 32, 4.0, 1.0)), moe(2, 2, 8)),
    layer(attention(2, 2, 8, 8, base=9.0, dims=2), dense(32)),
], eps=1e-6, scale=1.0, loop=(0, 3, 1))

# Sizes that no vector width divides: an odd width and vocabulary, odd head, latent and expert sizes, five
# taps; no loop at all.
ODD = config(50, 101, [
    layer(latent(3, 10, 6, 7, 13, base=77.0, scale=0.4, ramp=(2.5, 40, 6.0, 1.2)), moe(9, 2, 11, shared=13)),
    layer(attention_2(3, 1, 10, mask=5, conv=5, base=77.0, dims=6, scale=0.5, factor=1.5), moe(2, 1, 7)),
    layer(attention(2, 1, 6, 9, base=77.0, dims=4, scale=0.6), dense(27)),
], eps=1e-5, scale=0.8, loop=None)

# The loop at the end of the stack, two passes over one layer.
TAIL_LOOP = config(40, 77, [
    layer(attention(2, 1, 8, 12, base=50.0), dense(24)),
    layer(attention_2(2, 2, 8, mask=6, conv=3, base=50.0), moe(3, 2, 16)),
], eps=1e-5, scale=3.0, loop=(1, 2, 2))


# Scalings and masks on the mixers that usually have none or another: attention on the ramp and with a window,
# the latent attention with divided frequencies and a window, attention_2 on the ramp.
CROSSED = config(48, 90, [
    layer(attention(4, 2, 16, 8, base=400.0, dims=8, scale=0.5), dense(40)),
    layer(latent(2, 8, 8, 16, 24, base=60.0, scale=0.6, ramp=None), moe(4, 2, 16, shared=8)),
    layer(attention_2(2, 1, 16, mask=11, conv=3, base=90.0, dims=8, scale=0.7, factor=None), dense(24)),
], eps=1e-5, scale=2.0, loop=(0, 2, 2))
CROSSED["layers"][0]["mixer"]["rot"]["scaling"] = {"factor": 4.0, "original": 32, "fast": 6.0, "slow": 1.0}
CROSSED["layers"][0]["mixer"]["mask"] = {"size": 13}
CROSSED["layers"][1]["mixer"]["rot"]["scaling"] = {"factor": 2.5}
CROSSED["layers"][1]["mixer"]["mask"] = {"size": 20}
CROSSED["layers"][2]["mixer"]["rot"]["scaling"] = {"factor": 3.0, "original": 24, "fast": 5.0, "slow": 1.0}


# No channel is rotated anywhere (a latent layer without a rotated key part), and a pass over the first layer alone.
NO_ROTATION = config(40, 70, [
    layer(latent(2, 8, 0, 8, 16, base=60.0, scale=0.6, ramp=None), dense(24)),
    layer(attention(2, 1, 8, 8, base=50.0, dims=0, scale=0.5), moe(3, 1, 16)),
    layer(attention_2(2, 2, 8, mask=7, conv=2, base=50.0, dims=0, scale=0.6, factor=None), dense(16)),
], eps=1e-5, scale=1.2, loop=(0, 1, 3))


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    w = cfg["width"]
    shapes = {"embed": (cfg["vocab"], w), "final.norm": (w,), "head": (cfg["vocab"], w)}
    if cfg.get("loop"):
        shapes.update({"loop.in": (w, 2 * w), "loop.step": (cfg["loop"]["times"], w)})
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        h, d, v = m["heads"], m["dim"], m["vdim"]
        shapes[p + "norm1"] = (w,)
        if lay["type"] == "latent_attention":
            r, rot = m["kv_rank"], m["rot_dim"]
            shapes.update({p + "mix.q": (h * (d + rot), w), p + "mix.dkv": (r + rot, w), p + "mix.dkv.norm": (r,),
                           p + "mix.uk": (h * d, r), p + "mix.uv": (h * v, r), p + "mix.o": (w, h * v)})
        elif lay["type"] == "attention":
            g = m["kv_heads"]
            shapes.update({p + "mix.q": (h * d, w), p + "mix.k": (g * d, w), p + "mix.v": (g * v, w),
                           p + "mix.q.norm": (h * d,), p + "mix.k.norm": (g * d,), p + "mix.g": (h, w),
                           p + "mix.o": (w, h * v)})
        else:
            g, taps = m["kv_heads"], m["conv"]
            shapes.update({p + "mix.q": (h * d, w), p + "mix.k": (g * d, w), p + "mix.q.conv": (h * d, taps),
                           p + "mix.k.conv": (g * d, taps), p + "mix.q.norm": (d,), p + "mix.k.norm": (d,),
                           p + "mix.sink": (h,), p + "mix.g": (h, w), p + "mix.o": (w, h * d)})
        mlp = lay.get("mlp")
        if mlp:
            shapes[p + "norm2"] = (w,)
            if mlp["kind"] == "dense":
                names = [("", mlp["ff"])]
            else:
                shapes[p + "mlp.router"] = (mlp["router"]["experts"], w)
                shapes[p + "mlp.router.b"] = (mlp["router"]["experts"],)
                names = [(f"e{e}.", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
                if mlp.get("shared"):
                    names.append(("shared.", mlp["shared"]["ff"]))
            for name, ff in names:
                shapes.update({f"{p}mlp.{name}gate": (ff, w), f"{p}mlp.{name}up": (ff, w), f"{p}mlp.{name}down": (w, ff)})
    return shapes


def random_tensors(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors.  Matrices N(0, 1/in) (the router's larger and its bias of order one, so that choices
    are clear and the bias decides some); layer norms' weights around zero, the mixers' norm weights around one;
    sinks of a few units; the convolution's taps of order 1/2; pass vectors of order 1/2."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(".sink"):
            t = 1.0 + 1.5 * torch.randn(shape, generator=g)
        elif name.endswith(".norm"):
            wide = ".mix." in name
            t = (1.0 if wide else 0.0) + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith("norm1") or name.endswith("norm2"):
            t = 0.2 * torch.randn(shape, generator=g)
        elif name.endswith(".conv") or name == "loop.step":
            t = 0.5 * torch.randn(shape, generator=g)
        elif name.endswith("router.b"):
            t = torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            boost = 3.0 if name.endswith("router") else 1.0
            t = torch.randn(shape, generator=g) * boost / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def write_model(folder: str, cfg: dict, seed: int, tensors: Optional[Dict[str, torch.Tensor]] = None) -> str:
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    save_file(tensors if tensors is not None else random_tensors(cfg, seed), os.path.join(folder, "model.safetensors"))
    return folder
