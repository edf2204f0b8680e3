"""The Rofapel decoder as a model spec.

The residual sum starts at ``s table[id]`` (``s`` = ``embedding.scale``).  A layer is parallel with a norm for each
sublayer, ``x += mixer(norm1(x)) + ff(norm2(x))``, both norms (RMS, weight stored around zero and used as
``1 + w``) of the same ``x``.  A range of the layers may run several times in a row with the same weights; each
pass has a cache and state of its own and starts from ``Win [x; x0] + step_t``, ``x0`` being the embedding's
output, ``Win`` the tensor ``loop.in`` and ``step_t`` row ``t`` of ``loop.step``.  Three mixers:

* ``attention``: grouped key/value heads without biases; one RMS norm over all of a token's query channels and one
  over all its key channels (weights of the projection's size) before the rotation; rotation of the first
  ``rot.dims`` channels of every head in halves; a fixed score scale; all earlier keys; each head's output times
  the sigmoid of one number per head, a projection ``g`` of the mixer's input.
* ``latent_attention``: queries a plain projection, head by head ``[dim unrotated | rot_dim rotated]``; keys and
  values from a normed latent ``c`` and one rotated key part shared by the heads, which are all a token leaves in
  the cache; rotation of neighbouring channel pairs with frequencies stretched by a ramp over the channel index and
  cosines and sines scaled (``rot.scaling``: ``factor``, ``original``, ``fast``, ``slow``); all earlier keys.
* ``attention_2``: grouped heads whose values are the keys; queries and keys pass a short causal convolution over
  time right behind their projection (the values are the keys as they leave it), then an RMS norm per head with
  one weight shared by the heads, then rotation in halves with every frequency divided by ``rot.scaling.factor``;
  a sliding window of ``mask.size`` keys; a learned term per head in the softmax's denominator; the gate per head.

Feed-forwards: ``dense``, ``down(silu(gate x) * up x)``; ``moe``, experts of the same form chosen by the largest
router logits ``Wr x + b`` and weighted by the softmax over the chosen logits, plus a shared expert.  The final
norm (``1 + w``), then an untied head.

``rot.scaling`` is read by its keys in every mixer (a ``factor`` alone divides the frequencies; with ``original``,
``fast`` and ``slow`` it is the ramp), and a mixer with a ``mask`` sees its last ``mask.size`` keys only.

``config.json``: ``architecture``, ``width``, ``vocab``, ``norm.eps``, ``embedding.scale``, ``loop`` (``start``,
``stop``, ``times``; optional) and ``layers``, a list of ``{"type", "mixer": {...}, "mlp": {...} | null}``.  Tensors
are named ``embed``, ``final.norm``, ``head``, ``loop.in``, ``loop.step``, ``l<i>.norm1|norm2``, ``l<i>.mix.<name>``,
``l<i>.mlp.<name>``, ``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.mlp.shared.gate|up|down``; a bias ends in ``.b``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .spec import LayerSpec, ModelSpec, RunEntry

__all__ = ["RofapelConfig", "rofapel_spec", "rofapel_run_list"]

MIXER_TYPES = ("attention", "latent_attention", "attention_2")
MLP_KINDS = ("dense", "moe")


def _need(block: Any, keys, where: str) -> None:
    if not isinstance(block, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    missing = [k for k in keys if k not in block]
    if missing:
        raise ConfigError(f"config.json: {where} lacks {', '.join(missing)}")


def _positive(block: Dict[str, Any], keys, where: str) -> None:
    for key in keys:
        if not (isinstance(block[key], (int, float)) and not isinstance(block[key], bool) and block[key] > 0):
            raise ConfigError(f"config.json: {where}.{key} must be positive")


def _check_rot(rot: Any, limit: int, where: str, limit_name: str) -> None:
    _need(rot, ("base", "dims"), where)
    dims = int(rot["dims"])
    if dims < 0 or dims % 2 or dims > limit:
        raise ConfigError(f"config.json: {where}.dims must be even and at most {limit_name}")
    if dims and not float(rot["base"]) > 0:
        raise ConfigError(f"config.json: {where}.base must be positive")


def _check_scaling(rot: Dict[str, Any], where: str) -> None:
    """``rot.scaling`` is absent or null, ``{factor}`` (every frequency divided by it) or ``{factor, original, fast,
    slow}`` (the ramp over the channel index, with scaled cosines and sines)."""
    sc = rot.get("scaling")
    if not sc:
        return
    keys = ("factor", "original", "fast", "slow") if any(k in sc for k in ("original", "fast", "slow")) else ("factor",)
    _need(sc, keys, f"{where}.scaling")
    _positive(sc, keys, f"{where}.scaling")


def _check_mask(m: Dict[str, Any], where: str) -> None:
    if m.get("mask") is not None:
        _need(m["mask"], ("size",), f"{where}.mask")
        _positive(m["mask"], ("size",), f"{where}.mask")


def _check_gated(block: Any, where: str) -> None:
    _need(block, ("ff",), where)
    _positive(block, ("ff",), where)


@dataclass
class RofapelConfig:
    """The parsed ``config.json``.  Sizes and constants have no defaults: what the file does not give is an
    error (``loop``, a layer's ``mlp``, an ``mlp``'s ``shared`` and, where a mixer may have none, ``rot.scaling``
    may be absent or null: then the model has none)."""

    width: int
    vocab: int
    eps: float
    embed_scale: float
    layers: List[Dict[str, Any]]
    loop: Optional[Dict[str, int]] = None
    architecture: str = "Rofapel"
    eos_token_id: Optional[int] = None
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "RofapelConfig":
        _need(raw, ("width", "vocab", "norm", "embedding", "layers"), "the top level")
        _need(raw["norm"], ("eps",), "norm")
        _need(raw["embedding"], ("scale",), "embedding")
        _positive(raw, ("width", "vocab"), "the top level")
        layers = raw["layers"]
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            kind, m = layer["type"], layer["mixer"]
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: {', '.join(MIXER_TYPES)}")
            _need(m, ("heads", "dim", "vdim", "scale", "rot"), f"{where}.mixer")
            _positive(m, ("heads", "dim", "vdim", "scale"), f"{where}.mixer")
            if kind == "latent_attention":
                _need(m, ("kv_rank", "rot_dim"), f"{where}.mixer")
                _positive(m, ("kv_rank",), f"{where}.mixer")
                if int(m["rot_dim"]) < 0:
                    raise ConfigError(f"config.json: {where}.mixer.rot_dim cannot be negative")
                _check_rot(m["rot"], int(m["rot_dim"]), f"{where}.mixer.rot", "rot_dim")
            else:
                _need(m, ("kv_heads",), f"{where}.mixer")
                _positive(m, ("kv_heads",), f"{where}.mixer")
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"config.json: {where}: heads must be a multiple of kv_heads")
                _check_rot(m["rot"], int(m["dim"]), f"{where}.mixer.rot", "dim")
            _check_scaling(m["rot"], f"{where}.mixer.rot")
            if kind == "attention_2":
                _need(m, ("conv", "mask"), f"{where}.mixer")
                _positive(m, ("conv",), f"{where}.mixer")
                _need(m["mask"], ("size",), f"{where}.mixer")
                if int(m["vdim"]) != int(m["dim"]):
                    raise ConfigError(f"config.json: {where}: the values are the keys, so vdim must equal dim")
            _check_mask(m, f"{where}.mixer")
            mlp = layer.get("mlp")
            if mlp is not None:
                _need(mlp, ("kind",), f"{where}.mlp")
                if mlp["kind"] not in MLP_KINDS:
                    raise ConfigError(f"config.json: {where}.mlp has kind {mlp['kind']!r}; known: {', '.join(MLP_KINDS)}")
                if mlp["kind"] == "dense":
                    _check_gated(mlp, f"{where}.mlp")
                else:
                    _need(mlp, ("expert", "router"), f"{where}.mlp")
                    _check_gated(mlp["expert"], f"{where}.mlp.expert")
                    _need(mlp["router"], ("experts", "top"), f"{where}.mlp.router")
                    e, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
                    if not 0 < top <= e:
                        raise ConfigError(f"config.json: {where}.mlp.router: {top} of {e} experts cannot be chosen")
                    if mlp.get("shared"):
                        _check_gated(mlp["shared"], f"{where}.mlp.shared")
        loop = raw.get("loop") or None
        if loop is not None:
            _need(loop, ("start", "stop", "times"), "loop")
            start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ConfigError("config.json: loop needs 0 <= start <= stop <= the number of layers and times >= 1")
            # an empty range loops over nothing: the layers run once, in order
            loop = {"start": start, "stop": stop, "times": times} if start < stop else None
        return cls(width=int(raw["width"]), vocab=int(raw["vocab"]), eps=float(raw["norm"]["eps"]),
                   embed_scale=float(raw["embedding"]["scale"]), layers=layers, loop=loop,
                   architecture=str(raw.get("architecture") or "Rofapel"), eos_token_id=raw.get("eos_token_id"),
                   raw=dict(raw))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def _store_name(name: str) -> str:
    """Canonical name (``l0.mix.q.weight``, ``l1.mlp.router.bias``) -> the file's (``l0.mix.q``, ``l1.mlp.router.b``)."""
    if name.endswith(".weight"):
        return name[:-len(".weight")]
    if name.endswith(".bias"):
        return name[:-len(".bias")] + ".b"
    return name


def _map_name(name: str) -> str:
    return name[:-2] + ".bias" if name.endswith(".b") else name + ".weight"


def _scaling(rot: Dict[str, Any]) -> Optional[Dict[str, Any]]:
    """The position part's ``scaling``: the ramp where the file gives its four numbers, else the plain division."""
    sc = rot.get("scaling") or None
    if sc is None:
        return None
    if "original" in sc:
        return {"kind": "ramp", "factor": float(sc["factor"]), "original": int(sc["original"]),
                "fast": float(sc["fast"]), "slow": float(sc["slow"])}
    return {"kind": "linear", "factor": float(sc["factor"])}


def _window(m: Dict[str, Any]) -> Optional[int]:
    return int(m["mask"]["size"]) if m.get("mask") is not None else None


def _mixer_spec(kind: str, m: Dict[str, Any], width: int, eps: float) -> PartSpec:
    heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    rot = m["rot"]
    if kind == "latent_attention":
        position = PartSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"]), "scaling": _scaling(rot),
                                     "interleaved": True})
        return PartSpec("latent_attention", {
            "hidden_size": width, "num_heads": heads, "head_dim": dim, "rot_dim": int(m["rot_dim"]), "value_dim": vdim,
            "q_rank": None, "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "eps": eps, "window": _window(m),
            "sinks": False, "position": position, "names": {"dkv_norm": "dkv.norm"}})
    common = {"hidden_size": width, "num_heads": heads, "num_kv_heads": int(m["kv_heads"]), "head_dim": dim,
              "value_dim": vdim, "qkv_bias": False, "scale": float(m["scale"]), "qk_norm_eps": eps, "head_gate": True}
    names = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_norm": "q.norm", "k_norm": "k.norm",
             "q_conv": "q.conv", "k_conv": "k.conv", "sink": "sink"}
    position = PartSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"]), "scaling": _scaling(rot)})
    if kind == "attention":
        return PartSpec("paged_attention", {**common, "window": _window(m), "position": position, "qk_norm_scope": "whole",
                                            "names": names})
    return PartSpec("paged_attention", {**common, "window": _window(m), "position": position,
                                        "values_are_keys": True, "conv_taps": int(m["conv"]), "sinks": True,
                                        "names": names})


def _gated_ff(width: int, ff: int) -> PartSpec:
    return PartSpec("swiglu", {"hidden_size": width, "intermediate_size": int(ff),
                               "names": {"gate": "gate", "up": "up", "down": "down"}})


def _ffn_spec(mlp: Dict[str, Any], width: int) -> PartSpec:
    if mlp["kind"] == "dense":
        return _gated_ff(width, mlp["ff"])
    return PartSpec("routed_experts", {
        "hidden_size": width, "num_experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
        "intermediate_size": int(mlp["expert"]["ff"]), "expert_kind": "gated", "alpha": 1.0, "limit": None, "shift": 0.0,
        "groups": 1, "keep": 1, "scale": 1.0,
        # the softmax over the chosen logits: every expert's share of the softmax over all, over the chosen shares' sum
        "score": "softmax", "normalize": True, "floor": 0.0, "router_bias": True,
        "shared": _gated_ff(width, mlp["shared"]["ff"]) if mlp.get("shared") else None,
        "names": {"router": "router", "expert": "e{}", "gate": "gate", "up": "up", "down": "down", "shared": "shared"}})


def rofapel_run_list(num_layers: int, loop: Optional[Dict[str, int]]) -> List[RunEntry]:
    """The layers in the order they run: those before the looped range, the range ``times`` times (the first
    layer of pass t mixes the embedding's output in and adds pass vector t), those after it."""
    if loop is None:
        return [RunEntry(i) for i in range(num_layers)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    run = [RunEntry(i) for i in range(start)]
    for t in range(times):
        run += [RunEntry(i, add_vector=t if i == start else None, mix_input=i == start) for i in range(start, stop)]
    return run + [RunEntry(i) for i in range(stop, num_layers)]


def rofapel_spec(config: RofapelConfig) -> ModelSpec:
    width, eps = config.width, config.eps
    norm = PartSpec("rms_norm", {"size": width, "eps": eps, "offset": 1.0})
    layers: List[LayerSpec] = []
    for i, layer in enumerate(config.layers):
        mlp = layer.get("mlp")
        block = PartSpec("parallel", {
            "norm": norm, "mixer": _mixer_spec(layer["type"], layer["mixer"], width, eps),
            "ffn": None if mlp is None else _ffn_spec(mlp, width), "norm2": None if mlp is None else norm,
            "names": {"norm": "norm1", "mixer": "mix", "ffn": "mlp", "norm2": "norm2"}})
        layers.append(LayerSpec(block, f"l{i}."))
    sizes = {"vocab_size": config.vocab, "hidden_size": width}
    # a layer without a feed-forward has no use for a second norm: a file that stores one all the same is read
    unused = {f"l{i}.norm2" for i, layer in enumerate(config.layers) if layer.get("mlp") is None}
    if config.loop is None:
        unused |= {"loop.in", "loop.step"}     # of a loop over an empty range
    return ModelSpec(
        hidden_size=width, vocab_size=config.vocab, layers=layers, run=rofapel_run_list(len(layers), config.loop),
        final_norm=norm, tie_word_embeddings=False, position_rows=1,
        embed_name="embed.weight", final_norm_prefix="final.norm.", head_name="head.weight",
        map_name=lambda name: None if name in unused else _map_name(name), store_name=_store_name, eos_token_id=config.eos_token_id,
        embed=PartSpec("token_table", {**sizes, "scale": config.embed_scale}),
        pass_vectors_name=None if config.loop is None else "loop.step.weight",
        pass_vectors_rows=0 if config.loop is None else config.loop["times"],
        pass_mix_name=None if config.loop is None else "loop.in.weight",
    )


register_architecture("Rofapel", rofapel_spec, RofapelConfig.from_dict)
