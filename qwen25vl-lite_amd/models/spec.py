"""The description of a model as data: its layers, the parts of each, the run list.

An architecture is a function from a parsed configuration to a :class:`ModelSpec`.  The
generic :class:`~qwen25vl_lite_amd.models.decoder.DecoderModel` builds any spec; it never
looks at the architecture's name.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, List, Optional

from ..parts.base import PartSpec

__all__ = ["LayerSpec", "RunEntry", "ModelSpec"]


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block part (which names its norms, mixer and feed-forward) and the
    checkpoint prefix of its tensors, e.g. ``layers.3.``."""

    block: PartSpec
    prefix: str


@dataclass(frozen=True)
class RunEntry:
    """One step of the run list: run ``layer``.  ``cache_from`` names an earlier entry of the
    run list whose cache this entry reads instead of writing its own.  A layer that is named by
    several entries runs with the same weights each time; every entry has a cache layer and a
    state of its own unless it says ``cache_from``."""

    layer: int
    cache_from: Optional[int] = None
    # a row of the model's pass vectors that is added to every token's residual sum right before
    # this entry's layer runs
    add_vector: Optional[int] = None
    # True: right before this entry's layer runs (and before ``add_vector``), every token's residual sum x
    # becomes ``W [x; x0]``, ``x0`` being what the embedding gave for the token and ``W`` the model's pass-mix matrix
    mix_input: bool = False


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    layers: List[LayerSpec]
    run: List[RunEntry]
    final_norm: PartSpec
    tie_word_embeddings: bool
    position_rows: int = 3
    embed_name: str = "embed_tokens.weight"
    final_norm_prefix: str = "norm."
    head_name: str = "lm_head.weight"
    # checkpoint tensor name -> canonical name, or None for a tensor this model ignores
    map_name: Callable[[str], Optional[str]] = field(default=lambda name: name)
    # canonical name -> the name a written model folder stores the tensor under
    store_name: Callable[[str], str] = field(default=lambda name: name)
    eos_token_id: Optional[int] = None
    # the parts at the two ends; None: a plain token table and a plain linear head of [vocab, hidden].
    # Their tensors go by ``embed_name`` / ``head_name`` with the last component replaced by the part's own names.
    embed: Optional[PartSpec] = None
    head: Optional[PartSpec] = None
    # vectors that run entries add to the residual sum (``RunEntry.add_vector``): the canonical name
    # of a tensor ``[rows, hidden]`` and its number of rows; None: the model has none
    pass_vectors_name: Optional[str] = None
    pass_vectors_rows: int = 0
    # the matrix ``[hidden, 2 hidden]`` of the run entries with ``mix_input`` (columns of the running sum first,
    # then those of the embedding's output): the canonical name of the tensor; None: the model has none
    pass_mix_name: Optional[str] = None
