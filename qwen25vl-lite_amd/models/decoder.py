"""A decoder built from a :class:`ModelSpec`: embedding, the run list of layers, the final
norm and the output head (reference src/qwen25vl_lite/text.py:209-279, model.py:84-86, 200-202).
"""

from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..cache.manager import CacheGroupSpec
from ..parts.base import (Block, CacheNeed, LayerSlot, Mixer, ParamSpec, Part, PartSpec, ResidualStream, StateNeed,
                          StepContext, build_part)
from .spec import ModelSpec

__all__ = ["DecoderModel"]


def _collect(part: Part, prefix: str, out: Dict[str, Tuple[Part, str, ParamSpec]]) -> None:
    for local, spec in part.param_specs().items():
        out[prefix + local] = (part, local, spec)
    for name, sub in part.sub_parts().items():
        _collect(sub, f"{prefix}{name}.", out)


def _prefix_of(name: str) -> str:
    """``"a.b.weight"`` -> ``"a.b."``: where the tensors of the part behind a named tensor go."""
    return name[:name.rfind(".") + 1]


def _mixers_of(block: Part, prefix: str = "") -> List[Tuple[str, Part]]:
    """Every mixer inside a block, however deep, and every other part that keeps a cache or a per-request
    state (a short convolution), with its dotted sub-part name."""
    found: List[Tuple[str, Part]] = []
    for name, sub in block.sub_parts().items():
        if isinstance(sub, Mixer) or sub.state_need() is not None or sub.cache_need() is not None:
            found.append((prefix + name, sub))
        else:
            found.extend(_mixers_of(sub, f"{prefix}{name}."))
    return found


class PassVectors(Part):
    """Vectors ``[rows, hidden]`` in float32, one of which a run entry may add to every token's residual sum."""

    graph_safe = True

    def __init__(self, rows: int, hidden: int, dtype, device):
        super().__init__(dtype, device)
        self.rows, self.hidden = int(rows), int(hidden)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.rows, self.hidden), "vector")}

    def load(self, tensors):
        self.weight = tensors["weight"]


class PassMix(Part):
    """``x <- W [x; x0]`` for a matrix ``W [hidden, 2 hidden]``: the running residual sum and the embedding's output
    of every token, mixed into the sum a pass starts from.  The two halves of ``W`` are kept apart, so nothing is
    laid side by side at run time, and the half that reads the embedding's output is applied once per step."""

    graph_safe = True

    def __init__(self, hidden: int, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(hidden)
        self.w_sum: Optional[torch.Tensor] = None     # [hidden, hidden]: the columns that read the running sum
        self.w_first: Optional[torch.Tensor] = None   # [hidden, hidden]: the columns that read the embedding's output

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.hidden, 2 * self.hidden), "matrix")}

    def load(self, tensors):
        w = tensors["weight"]
        self.w_sum = w[:, :self.hidden].contiguous()
        self.w_first = w[:, self.hidden:].contiguous()

    def named_weights(self) -> Dict[str, torch.Tensor]:
        return {"weight": torch.cat([self.w_sum, self.w_first], dim=1)}

    def _rounded(self, h: torch.Tensor) -> torch.Tensor:
        return h if h.dtype == self.dtype else h.to(self.dtype)

    def from_first(self, x0: torch.Tensor) -> torch.Tensor:
        """float32 ``[N, hidden]``: the embedding's share of every pass's start."""
        from ..ops.linear import linear
        return linear(self._rounded(x0), self.w_first, out_dtype=torch.float32)

    def forward(self, stream: ResidualStream, first_share: torch.Tensor) -> ResidualStream:
        """The stream whose sum is ``w_sum x`` with ``first_share`` waiting to be added (by the next norm)."""
        from ..ops.gated import residual_add, sandwich_norm
        from ..ops.linear import linear

        if stream.pending_norm is not None or stream.row_addend is not None:
            gain, eps_y, factor = stream.pending_norm or (None, 0.0, 1.0)
            sandwich_norm(stream.h, stream.pending, gain if stream.pending is not None else None, eps_y, factor,
                          stream.row_addend, None, 0.0, self.dtype)
        elif stream.pending is not None:
            residual_add(stream.h, stream.pending)
        h = linear(self._rounded(stream.h), self.w_sum, out_dtype=torch.float32)
        return ResidualStream(h if h.is_contiguous() else h.contiguous(), pending=first_share)


class DecoderModel:
    """Holds the parts and runs a step over them.  Tensors arrive through :meth:`load_part`."""

    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.blocks: List[Block] = [build_part("block", ls.block, dtype, self.device) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, dtype, self.device)
        sizes = {"vocab_size": spec.vocab_size, "hidden_size": spec.hidden_size}
        self.embedding = build_part("embedding", spec.embed or PartSpec("token_table", sizes), dtype, self.device)
        self.head_part = build_part("head", spec.head or PartSpec("linear", sizes), dtype, self.device)
        self._has_weights = False
        self.pass_vectors: Optional[PassVectors] = None
        if spec.pass_vectors_name is not None:
            if not spec.pass_vectors_name.endswith(".weight") or spec.pass_vectors_rows <= 0:
                raise ValueError("pass vectors are a tensor '<name>.weight' with at least one row")
            self.pass_vectors = PassVectors(spec.pass_vectors_rows, spec.hidden_size, dtype, self.device)
        self.pass_mix: Optional[PassMix] = None
        if spec.pass_mix_name is not None:
            if not spec.pass_mix_name.endswith(".weight"):
                raise ValueError("the pass-mix matrix is a tensor '<name>.weight'")
            self.pass_mix = PassMix(spec.hidden_size, dtype, self.device)
        for i, entry in enumerate(spec.run):
            if entry.add_vector is not None and not (self.pass_vectors is not None
                                                     and 0 <= entry.add_vector < spec.pass_vectors_rows):
                raise ValueError(f"run entry {i} adds pass vector {entry.add_vector}, which the model does not have")
            if entry.mix_input and self.pass_mix is None:
                raise ValueError(f"run entry {i} mixes the embedding's output in, but the model has no matrix for it")

        # The run list: which cache layer and state every mixer of every entry owns.  The lists
        # below have one element per (run entry, mixer of its block), in run order ("places");
        # entry_places[i] names the places of entry i by the mixer's sub-part name.  A block with
        # one mixer, the usual case, has one place.
        self.group_needs: List[CacheNeed] = []
        self.group_layers: List[int] = []
        self.entry_places: List[Dict[str, int]] = []
        self.entry_group: List[Optional[int]] = []
        self.entry_cache_layer: List[Optional[int]] = []
        self.entry_writes: List[bool] = []
        self.entry_state: List[Optional[StateNeed]] = []
        for i, entry in enumerate(spec.run):
            if not 0 <= entry.layer < len(self.blocks):
                raise ValueError(f"run entry {i} names layer {entry.layer}, which does not exist")
            mixers = _mixers_of(self.blocks[entry.layer])
            if entry.cache_from is not None:
                src = entry.cache_from
                if not 0 <= src < i:
                    raise ValueError(f"run entry {i} must read the cache of an earlier entry that writes one")
                if not any(m.cache_need() is not None for _, m in mixers):
                    raise ValueError(f"run entry {i} reads a cache but its mixer keeps none")
            places: Dict[str, int] = {}
            for name, mixer in mixers:
                need = mixer.cache_need()
                places[name] = len(self.entry_state)
                self.entry_state.append(mixer.state_need())
                if need is None:
                    self.entry_group.append(None)
                    self.entry_cache_layer.append(None)
                    self.entry_writes.append(False)
                    continue
                if entry.cache_from is not None:
                    src_place = self.entry_places[entry.cache_from].get(name)
                    if src_place is None or self.entry_group[src_place] is None or not self.entry_writes[src_place]:
                        raise ValueError(f"run entry {i} must read the cache of an earlier entry that writes one")
                    if self.group_needs[self.entry_group[src_place]] != need:
                        raise ValueError(
                            f"run entry {i} reads the cache of entry {entry.cache_from}, whose shape or window differs")
                    self.entry_group.append(self.entry_group[src_place])
                    self.entry_cache_layer.append(self.entry_cache_layer[src_place])
                    self.entry_writes.append(False)
                    continue
                if need not in self.group_needs:
                    self.group_needs.append(need)
                    self.group_layers.append(0)
                g = self.group_needs.index(need)
                self.entry_group.append(g)
                self.entry_cache_layer.append(self.group_layers[g])
                self.entry_writes.append(True)
                self.group_layers[g] += 1
            self.entry_places.append(places)

        self.params: Dict[str, Tuple[Optional[Part], str, ParamSpec]] = {}
        _collect(self.embedding, _prefix_of(spec.embed_name), self.params)
        if self.pass_vectors is not None:
            _collect(self.pass_vectors, _prefix_of(spec.pass_vectors_name), self.params)
        if self.pass_mix is not None:
            _collect(self.pass_mix, _prefix_of(spec.pass_mix_name), self.params)
        for ls, block in zip(spec.layers, self.blocks):
            _collect(block, ls.prefix, self.params)
        _collect(self.final_norm, spec.final_norm_prefix, self.params)
        _collect(self.head_part, _prefix_of(spec.head_name), self.params)
        for name in (spec.embed_name, spec.head_name):
            if name not in self.params:
                raise ValueError(f"the spec names the tensor {name}, which neither end of the model declares")

    # ------------------------------------------------------------------ structure
    @property
    def graph_safe(self) -> bool:
        """True if every part may run under HIP graph capture."""
        def safe(part) -> bool:
            return part.graph_safe and all(safe(s) for s in part.sub_parts().values())
        return (all(safe(b) for b in self.blocks) and safe(self.final_norm) and safe(self.embedding)
                and safe(self.head_part))


    def cache_groups(self) -> List[CacheGroupSpec]:
        return [CacheGroupSpec(need, n) for need, n in zip(self.group_needs, self.group_layers)]

    def expected_tensors(self) -> Dict[str, ParamSpec]:
        """Canonical tensor name -> what is expected under it."""
        return {name: spec for name, (_, _, spec) in self.params.items()}

    def part_groups(self) -> List[Tuple[Optional[Part], Dict[str, str]]]:
        """Tensors grouped by the part that takes them: ``(part, {local: canonical})``."""
        groups: Dict[int, Tuple[Optional[Part], Dict[str, str]]] = {}
        for name, (part, local, _) in self.params.items():
            key = id(part) if part is not None else hash(name)
            groups.setdefault(key, (part, {}))[1][local] = name
        return list(groups.values())

    def load_part(self, part: Part, tensors: Dict[str, torch.Tensor]) -> None:
        part.load(tensors)
        self._has_weights = True

    def tie_head(self) -> None:
        self.head_part.tie(self.embedding)

    @property
    def embed(self) -> Optional[torch.Tensor]:
        """The token table (what a tied head shares)."""
        return self.embedding.table

    @property
    def head(self) -> Optional[torch.Tensor]:
        """The built-in head's matrix (None for a head of another kind)."""
        return getattr(self.head_part, "weight", None)

    def make_slots(self, storage, state_tensors: List[Optional[torch.Tensor]]) -> List[LayerSlot]:
        """One slot per run entry.  ``state_tensors`` has one element per place (see
        ``entry_state``).  The slot of an entry is its first mixer's; a block with several
        mixers finds each one's under the mixer's sub-part name in ``slot.by_part``."""
        def place_slot(p: int) -> LayerSlot:
            g, layer = self.entry_group[p], self.entry_cache_layer[p]
            return LayerSlot(
                group=g,
                k_cache=storage.k[g][layer] if g is not None else None,
                v_cache=storage.v[g][layer] if g is not None else None,
                writes=self.entry_writes[p],
                state=state_tensors[p],
            )

        slots = []
        for places in self.entry_places:
            by_part = {name: place_slot(p) for name, p in places.items()}
            first = next(iter(by_part.values()), LayerSlot(writes=False))
            first.by_part = by_part
            slots.append(first)
        return slots

    # ------------------------------------------------------------------ the step
    def forward(self, step: StepContext, slots: List[LayerSlot]) -> torch.Tensor:
        """Run the step's tokens through the run list; float32 logits ``[M, vocab]`` at
        ``step.logit_rows``."""
        if not self._has_weights:
            raise RuntimeError("the model has no weights yet")
        stream = ResidualStream(self.embedding.forward(step.token_ids, step))
        first_share = None
        if self.pass_mix is not None and any(e.mix_input for e in self.spec.run):
            first_share = self.pass_mix.from_first(stream.h)     # before any layer changes the sum in place
        for entry, slot in zip(self.spec.run, slots):
            if entry.mix_input:
                stream = self.pass_mix.forward(stream, first_share)
            if entry.add_vector is not None:
                if stream.row_addend is not None:
                    raise RuntimeError("a block left a pass vector unadded: its first norm must fold the stream")
                stream.row_addend = self.pass_vectors.weight[entry.add_vector]   # the layer's first norm adds it
            stream = self.blocks[entry.layer].forward(stream, step, slot)
        if step.logit_rows.shape[0] == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        x = self.final_norm.forward(stream, rows=step.logit_rows)
        return self.head_part.forward(x, step)
