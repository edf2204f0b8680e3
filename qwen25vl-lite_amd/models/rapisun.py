"""The Rapisun decoder as a model spec.

The token table's rows are layer-normed; a layer is ``x += norm1(mixer(f(x)))``, ``x += norm2(ff(x))``: the
sublayers read the residual sum itself, the norm (a layer norm with a weight and no bias) stands on their
outputs, and what the mixer reads first passes a short causal convolution over time that is added to it
(``f(x)_t = x_t + sum_j w_j x_(t - taps + 1 + j)``, per channel).  Two mixers:

* ``hgrn2``: linear attention whose forget gate also decides what is written: per head
  ``S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T``, ``o_t = S_t^T q_t`` with ``q = silu(Wq x)``, ``v = Wv x`` and
  ``f = l + (1 - l) sigmoid(Wf x + b)``, ``l`` a floor per key channel; each head's output RMS-normed, then ``Wo``.
* ``latent_attention``: queries through a normed latent; keys and values from a normed latent ``c`` and one
  rotated key part shared by the heads, which are all a token leaves in the cache; a head's query and key are
  ``[dim unrotated | rot_dim rotated]`` (rotation in halves); a sliding window; a learned term per head in the
  softmax's denominator.  A layer with ``kv_from: j`` has no key/value down projection and reads what layer ``j``
  cached, with up projections, window and everything else of its own.

Feed-forwards: ``dense``, ``down(P(up x))`` with ``P(z) = a N(z) + b N(z^2) + c N(z^3) + e`` (``N`` divides a row by its
root mean square); ``moe``, experts ``down(relu(up x)^2)`` chosen by the largest softmax scores, weighted by the
chosen scores over their sum, plus a shared expert of the same form.  The final layer norm, then an untied head.

``config.json``: ``architecture``, ``width``, ``vocab``, ``norm.eps``, ``canon.taps`` and ``layers``, a list of
``{"type", "mixer": {...}, "mlp": {...} | null}``.  Tensors are named ``embed``, ``embed.norm``, ``final.norm``, ``head``,
``l<i>.norm1|norm2``, ``l<i>.canon1``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``, ``l<i>.mlp.e<j>.up|down``,
``l<i>.mlp.shared.up|down``; a bias ends in ``.b``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .spec import LayerSpec, ModelSpec, RunEntry

__all__ = ["RapisunConfig", "rapisun_spec"]

# constants the design fixes
WEIGHT_SUM_FLOOR = 1e-20        # added to the sum the routing weights are divided by
MIXER_TYPES = ("hgrn2", "latent_attention")
MLP_KINDS = ("dense", "moe")


def _need(block: Any, keys, where: str) -> None:
    if not isinstance(block, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    missing = [k for k in keys if k not in block]
    if missing:
        raise ConfigError(f"config.json: {where} lacks {', '.join(missing)}")


def _positive(block: Dict[str, Any], keys, where: str) -> None:
    for key in keys:
        if not (isinstance(block[key], (int, float)) and block[key] > 0):
            raise ConfigError(f"config.json: {where}.{key} must be positive")


@dataclass
class RapisunConfig:
    """The parsed ``config.json``.  Sizes and constants have no defaults: what the file does not give is an
    error (``canon``, a mixer's ``mask``, a layer's ``mlp`` and an ``mlp``'s ``shared`` may be absent or null: then
    the model has none)."""

    width: int
    vocab: int
    eps: float
    layers: List[Dict[str, Any]]
    taps: Optional[int] = None
    architecture: str = "Rapisun"
    eos_token_id: Optional[int] = None
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "RapisunConfig":
        _need(raw, ("width", "vocab", "norm", "layers"), "the top level")
        _need(raw["norm"], ("eps",), "norm")
        _positive(raw, ("width", "vocab"), "the top level")
        taps = None
        if raw.get("canon"):
            _need(raw["canon"], ("taps",), "canon")
            taps = int(raw["canon"]["taps"])
            if taps < 1:
                raise ConfigError("config.json: canon.taps must be at least 1")
        layers = raw["layers"]
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            kind, m = layer["type"], layer["mixer"]
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: {', '.join(MIXER_TYPES)}")
            _need(m, ("heads", "dim", "vdim"), f"{where}.mixer")
            _positive(m, ("heads", "dim", "vdim"), f"{where}.mixer")
            if kind == "latent_attention":
                _need(m, ("q_rank", "kv_rank", "rot_dim", "scale", "rot"), f"{where}.mixer")
                _positive(m, ("q_rank", "kv_rank", "scale"), f"{where}.mixer")
                _need(m["rot"], ("base", "dims"), f"{where}.mixer.rot")
                dims, rot_dim = int(m["rot"]["dims"]), int(m["rot_dim"])
                if rot_dim < 0 or dims < 0 or dims % 2 or dims > rot_dim:
                    raise ConfigError(f"config.json: {where}.mixer.rot.dims must be even and at most rot_dim")
                if m.get("mask") is not None:
                    _need(m["mask"], ("size",), f"{where}.mixer.mask")
                    _positive(m["mask"], ("size",), f"{where}.mixer.mask")
                src = m.get("kv_from")
                if src is not None:
                    if not (isinstance(src, int) and 0 <= src < i and layers[src].get("type") == "latent_attention"
                            and layers[src]["mixer"].get("kv_from") is None):
                        raise ConfigError(f"config.json: {where}.mixer.kv_from must name an earlier latent_attention "
                                          "layer that has a cache of its own")
                    theirs = layers[src]["mixer"]
                    same = (int(theirs["kv_rank"]) == int(m["kv_rank"]) and int(theirs["rot_dim"]) == rot_dim
                            and int(theirs["rot"]["dims"]) == dims and float(theirs["rot"]["base"]) == float(m["rot"]["base"]))
                    if not same:
                        raise ConfigError(f"config.json: {where}.mixer reads layer {src}'s cache, whose kv_rank, rot_dim "
                                          "or rotation differs")
            mlp = layer.get("mlp")
            if mlp is not None:
                _need(mlp, ("kind",), f"{where}.mlp")
                if mlp["kind"] not in MLP_KINDS:
                    raise ConfigError(f"config.json: {where}.mlp has kind {mlp['kind']!r}; known: {', '.join(MLP_KINDS)}")
                if mlp["kind"] == "dense":
                    _need(mlp, ("ff",), f"{where}.mlp")
                    _positive(mlp, ("ff",), f"{where}.mlp")
                else:
                    _need(mlp, ("expert", "router"), f"{where}.mlp")
                    _need(mlp["expert"], ("ff",), f"{where}.mlp.expert")
                    _need(mlp["router"], ("experts", "top"), f"{where}.mlp.router")
                    e, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
                    if not 0 < top <= e:
                        raise ConfigError(f"config.json: {where}.mlp.router: {top} of {e} experts cannot be chosen")
                    if mlp.get("shared"):
                        _need(mlp["shared"], ("ff",), f"{where}.mlp.shared")
        return cls(width=int(raw["width"]), vocab=int(raw["vocab"]), eps=float(raw["norm"]["eps"]), layers=layers,
                   taps=taps, architecture=str(raw.get("architecture") or "Rapisun"),
                   eos_token_id=raw.get("eos_token_id"), raw=dict(raw))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def _store_name(name: str) -> str:
    """Canonical name (``l0.mix.q.weight``, ``l0.mix.f.bias``) -> the file's (``l0.mix.q``, ``l0.mix.f.b``)."""
    if name.endswith(".weight"):
        return name[:-len(".weight")]
    if name.endswith(".bias"):
        return name[:-len(".bias")] + ".b"
    return name


def _map_name(name: str) -> str:
    return name[:-2] + ".bias" if name.endswith(".b") else name + ".weight"


def _window(m: Dict[str, Any]) -> Optional[int]:
    return int(m["mask"]["size"]) if m.get("mask") is not None else None


def retained_keys(layers: List[Dict[str, Any]]) -> Dict[int, Optional[int]]:
    """For every latent-attention layer that owns a cache: how many keys back its pages must stay, the
    longest window among itself and the layers that read its cache (None: one of them sees all keys)."""
    keep: Dict[int, Optional[int]] = {}
    for i, layer in enumerate(layers):
        if layer["type"] != "latent_attention":
            continue
        owner = layer["mixer"].get("kv_from")
        owner = i if owner is None else int(owner)
        window = _window(layer["mixer"])
        if owner not in keep:
            keep[owner] = window
        elif keep[owner] is not None:
            keep[owner] = None if window is None else max(keep[owner], window)
    return keep


def _mixer_spec(kind: str, m: Dict[str, Any], width: int, eps: float, retain: Optional[int]) -> PartSpec:
    heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    if kind == "hgrn2":
        return PartSpec("linear_attention", {
            "hidden_size": width, "num_heads": heads, "key_dim": dim, "value_dim": vdim, "eps": eps,
            "decay": {"kind": "forget"}, "activation": "silu", "activation_on": "q", "q_scale": 1.0,
            "norm": "per_head", "gate": None})
    rot = m["rot"]
    position = PartSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"])})
    return PartSpec("latent_attention", {
        "hidden_size": width, "num_heads": heads, "head_dim": dim, "rot_dim": int(m["rot_dim"]), "value_dim": vdim,
        "q_rank": int(m["q_rank"]), "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "eps": eps,
        "window": _window(m), "retain": retain, "sinks": True, "position": position,
        "kv_shared": m.get("kv_from") is not None,
        "names": {"dq_norm": "dq.norm", "dkv_norm": "dkv.norm"}})


def _ffn_spec(mlp: Dict[str, Any], width: int, eps: float) -> PartSpec:
    names = {"up": "up", "down": "down", "act": "act"}
    if mlp["kind"] == "dense":
        return PartSpec("plain", {"hidden_size": width, "intermediate_size": int(mlp["ff"]),
                                  "activation": "normed_powers", "eps": eps, "names": names})
    shared = None
    if mlp.get("shared"):
        shared = PartSpec("plain", {"hidden_size": width, "intermediate_size": int(mlp["shared"]["ff"]),
                                    "activation": "relu2", "names": names})
    return PartSpec("routed_experts", {
        "hidden_size": width, "num_experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
        "intermediate_size": int(mlp["expert"]["ff"]), "expert_kind": "plain", "activation": "relu2",
        "groups": 1, "keep": 1, "scale": 1.0, "score": "softmax", "normalize": True, "floor": WEIGHT_SUM_FLOOR,
        "shared": shared,
        "names": {"router": "router", "expert": "e{}", "up": "up", "down": "down", "shared": "shared"}})


def rapisun_spec(config: RapisunConfig) -> ModelSpec:
    width, eps = config.width, config.eps
    norm = PartSpec("layer_norm", {"size": width, "eps": eps})
    keep = retained_keys(config.layers)
    layers: List[LayerSpec] = []
    run: List[RunEntry] = []
    for i, layer in enumerate(config.layers):
        m = layer["mixer"]
        owner = m.get("kv_from") if layer["type"] == "latent_attention" else None
        retain = keep.get(i if owner is None else int(owner))
        mlp = layer.get("mlp")
        block = PartSpec("post_norm", {
            "mixer": _mixer_spec(layer["type"], m, width, eps, retain), "norm1": norm,
            "ffn": None if mlp is None else _ffn_spec(mlp, width, eps), "norm2": norm,
            "filter": None if config.taps is None else PartSpec("short_conv", {"channels": width, "taps": config.taps}),
            "names": {"mixer": "mix", "norm1": "norm1", "ffn": "mlp", "norm2": "norm2", "filter": "canon1"}})
        layers.append(LayerSpec(block, f"l{i}."))
        run.append(RunEntry(i, cache_from=None if owner is None else int(owner)))   # one entry a layer: indices agree
    sizes = {"vocab_size": config.vocab, "hidden_size": width}
    return ModelSpec(
        hidden_size=width, vocab_size=config.vocab, layers=layers, run=run,
        final_norm=norm, tie_word_embeddings=False, position_rows=1,
        embed_name="embed.weight", final_norm_prefix="final.norm.", head_name="head.weight",
        map_name=_map_name, store_name=_store_name, eos_token_id=config.eos_token_id,
        embed=PartSpec("normed_table", {**sizes, "norm": norm, "norm_name": "norm"}),
    )


register_architecture("Rapisun", rapisun_spec, RapisunConfig.from_dict)
