"""The two ends of the decoder that touch the vocabulary: the token table and the output head
(reference src/qwen25vl_lite/text.py:209-213, 275-279; model.py:84-86 for the tied head)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels
from ..ops.linear import linear
from .base import Embedding, Head, ParamSpec, Part, PartSpec, build_part, register_part

__all__ = ["TokenTable", "NormedTokenTable", "LinearHead"]


class TokenTable(Embedding):
    """Row ``id`` of a ``[vocab, hidden]`` table, widened to float32 and multiplied by ``scale``.

    params: ``vocab_size``, ``hidden_size``, optional ``scale`` (default 1).
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.vocab, self.hidden = int(params["vocab_size"]), int(params["hidden_size"])
        self.scale = float(params.get("scale", 1.0))
        self.table: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab, self.hidden), "table")}

    def load(self, tensors):
        self.table = tensors["weight"]

    def forward(self, token_ids, step):
        return kernels.embed_gather(token_ids, self.table, scale=self.scale)


class NormedTokenTable(TokenTable):
    """A token's row of the table, normed: the residual sum starts at ``norm(table[id])`` in float32.

    params: ``vocab_size``, ``hidden_size``, ``norm`` (a :class:`PartSpec` of a norm that has a ``weight`` and an
    ``eps``: a layer norm), ``norm_name`` (the norm's checkpoint sub-name, default ``norm``).
    """

    def __init__(self, params, dtype, device):
        super().__init__(params, dtype, device)
        spec: PartSpec = params["norm"]
        if spec.kind != "layer_norm":
            raise ValueError("the norm on the token table is a layer norm")
        self.norm = build_part("norm", spec, dtype, device)
        self.norm_name = str(params.get("norm_name", "norm"))

    def sub_parts(self) -> Dict[str, Part]:
        return {self.norm_name: self.norm}

    def forward(self, token_ids, step):
        from ..ops import rownorm

        rows = kernels.embed_gather(token_ids, self.table, scale=self.scale)
        return rownorm.layer_norm(rows, self.norm.weight, self.norm.eps, torch.float32)


class LinearHead(Head):
    """``x @ weight.T`` in float32, ``weight`` being ``[vocab, hidden]`` or the tied token table;
    with ``softcap`` c the logits become ``c tanh(logits / c)``.

    params: ``vocab_size``, ``hidden_size``, optional ``softcap``.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.vocab, self.hidden = int(params["vocab_size"]), int(params["hidden_size"])
        cap = params.get("softcap")
        self.softcap = float(cap) if cap else None
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab, self.hidden), "matrix")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def tie(self, embedding):
        if embedding.table is None or tuple(embedding.table.shape) != (self.vocab, self.hidden):
            raise ValueError("a tied head needs the embedding's table of [vocab, hidden]")
        self.weight = embedding.table

    def forward(self, x, step):
        logits = linear(x, self.weight, out_dtype=torch.float32)
        if self.softcap is not None:
            from ..ops.gated import softcap_
            logits = softcap_(logits if logits.is_contiguous() else logits.contiguous(), self.softcap)
        return logits


register_part("embedding", "token_table", TokenTable)
register_part("embedding", "normed_table", NormedTokenTable)
register_part("head", "linear", LinearHead)
