"""Small Rapisun configurations and model folders with random weights for the tests.  The weights
are drawn here (not by the engine) and written with the safetensors package."""

from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch


def hgrn2(heads, dim, vdim):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, dims=None, scale=None, mask=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale or (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if mask is not None:
        m["mask"] = {"size": mask}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        mlp["shared"] = {"ff": shared}
    return mlp


def layer(mixer, mlp=None):
    return {**mixer, "mlp": mlp}


def config(width, vocab, layers, eps=1e-5, taps=4):
    cfg = {"architecture": "Rapisun", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if taps is not None:
        cfg["canon"] = {"taps": taps}
    return cfg


# Sizes that all differ from one another: an attention layer first, a reader of its cache with a longer
# window two layers on, a recurrent layer between them, a second cache of another shape whose reader sees
# all keys, value heads wider and narrower than key heads, partial and full rotation, a layer without a
# feed-forward, experts with and without a shared one, three taps.
MIXED = config(72, 203, [
    layer(latent(3, 16, 8, 24, 40, 24, base=500.0, scale=0.6, mask=9), moe(6, 2, 40, shared=56)),
    layer(hgrn2(2, 12, 20), dense(88)),
    layer(latent(4, 8, 8, 12, 24, 24, base=500.0, scale=0.5, mask=21, kv_from=0), moe(5, 3, 24)),
    layer(latent(2, 24, 16, 16, 32, 40, base=80.0, dims=8, scale=0.4, mask=37)),
    layer(hgrn2(3, 20, 8), moe(4, 4, 32, shared=16)),
    layer(latent(5, 16, 16, 8, 16, 40, base=80.0, dims=8, scale=0.3, kv_from=3), dense(40)),
], eps=1e-5, taps=3)

# The same shapes with score scales so large that the softmax picks single keys: a key lost at a
# window's edge or a page's border moves the logits.
SHARP = json.loads(json.dumps(MIXED))
for _i, _s in ((0, 5.0), (2, 4.0), (3, 3.0), (5, 2.5)):
    SHARP["layers"][_i]["mixer"]["scale"] = _s

# Values that happen to be 1 or equal: one head, one expert chosen of one, every expert chosen, a window
# of one token, one tap (a convolution without a state), equal key and value sizes, equal latent sizes.
ONES = config(32, 61, [
    layer(hgrn2(1, 16, 16), moe(1, 1, 16, shared=16)),
    layer(latent(1, 16, 16, 16, 16, 16, base=100.0, scale=1.0, mask=1), moe(2, 2, 8)),
    layer(latent(2, 8, 2, 8, 8, 8, base=9.0, scale=0.25), dense(32)),
], eps=1e-6, taps=1)

# Sizes that no vector width divides: an odd width and vocabulary, odd head, latent and expert sizes, five
# taps, a model without a convolution is NO_CONV.
ODD = config(50, 101, [
    layer(latent(3, 10, 6, 7, 11, 13, base=77.0, scale=0.4, mask=5), moe(9, 2, 11, shared=13)),
    layer(hgrn2(3, 5, 7), moe(2, 1, 7)),
    layer(latent(2, 6, 6, 9, 9, 13, base=77.0, scale=0.6, kv_from=0), dense(27)),
], eps=1e-5, taps=5)

NO_CONV = config(40, 77, [
    layer(hgrn2(2, 8, 12), dense(24)),
    layer(latent(2, 8, 4, 8, 12, 12, base=50.0, mask=6), moe(3, 2, 16)),
], eps=1e-5, taps=None)


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    w = cfg["width"]
    shapes = {"embed": (cfg["vocab"], w), "embed.norm": (w,), "final.norm": (w,), "head": (cfg["vocab"], w)}
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        h, d, v = m["heads"], m["dim"], m["vdim"]
        shapes[p + "norm1"] = (w,)
        if cfg.get("canon"):
            shapes[p + "canon1"] = (w, cfg["canon"]["taps"])
        if lay["type"] == "hgrn2":
            shapes.update({p + "mix.q": (h * d, w), p + "mix.f": (h * d, w), p + "mix.f.b": (h * d,),
                           p + "mix.lower": (h * d,), p + "mix.v": (h * v, w), p + "mix.norm": (v,),
                           p + "mix.o": (w, h * v)})
        else:
            r, rot, qr = m["kv_rank"], m["rot_dim"], m["q_rank"]
            shapes.update({p + "mix.dq": (qr, w), p + "mix.dq.norm": (qr,), p + "mix.uq": (h * (d + rot), qr),
                           p + "mix.uk": (h * d, r), p + "mix.uv": (h * v, r), p + "mix.sink": (h,),
                           p + "mix.o": (w, h * v)})
            if m.get("kv_from") is None:
                shapes.update({p + "mix.dkv": (r + rot, w), p + "mix.dkv.norm": (r,)})
        mlp = lay.get("mlp")
        if mlp:
            shapes[p + "norm2"] = (w,)
            if mlp["kind"] == "dense":
                shapes.update({p + "mlp.up": (mlp["ff"], w), p + "mlp.down": (w, mlp["ff"]), p + "mlp.act": (4,)})
            else:
                shapes[p + "mlp.router"] = (mlp["router"]["experts"], w)
                names = [(f"e{e}", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
                if mlp.get("shared"):
                    names.append(("shared", mlp["shared"]["ff"]))
                for name, ff in names:
                    shapes.update({f"{p}mlp.{name}.up": (ff, w), f"{p}mlp.{name}.down": (w, ff)})
    return shapes


def random_tensors(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors.  Matrices N(0, 1/in) (the router's larger, so that choices are clear); norm weights
    around 1; the forget gate's floor uniform on [0, 0.9] and its bias positive on average (slow channels
    exist); sinks of a few units; the convolution's taps and the activation's four numbers of order 1/2."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(".lower"):
            t = 0.9 * torch.rand(shape, generator=g)
        elif name.endswith(".f.b"):
            t = 1.0 + 1.5 * torch.randn(shape, generator=g)
        elif name.endswith(".sink"):
            t = 1.0 + 1.5 * torch.randn(shape, generator=g)
        elif "norm" in name:
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith(".act") or name.endswith("canon1"):
            t = 0.5 * torch.randn(shape, generator=g)
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
