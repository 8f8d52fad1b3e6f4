"""Token embedding: a row gather into the float32 residual stream."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import Part, StreamAddend, UnscaledRows


@register_part("embedding", "token")
class TokenEmbedding(Part):
    """x[t] = E[ids[t]] * scale, no padding row; `scale` is 1 unless the architecture says otherwise
    (src/qwen3_from_scratch/models/qwen3.py:17-19,45). With `copies` the residual starts as
    that many equal streams, (T, copies, hidden_size), for blocks that keep several."""

    graph_safe = True

    def __init__(self, prefix, precision, device, vocab_size, hidden_size, leaf="weight", copies=0, scale=1.0):
        super().__init__(prefix, precision, device)
        self.copies = int(copies)
        self.scale = float(scale)
        if self.copies and self.scale != 1.0:
            raise ValueError("a residual that starts as several streams has no scale on its embedding")
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.leaf = leaf
        self.weight = None

    def tensors(self):
        return {self._name(self.leaf): (self.vocab_size, self.hidden_size)}

    def load(self, fetch):
        self.weight = fetch(self._name(self.leaf), self.precision.act)

    def forward(self, token_ids):
        if self.copies:
            return ops.embed_streams(token_ids, self.weight, self.copies)
        return ops.embed_rows(token_ids, self.weight, scale=self.scale)


@register_part("embedding", "pass_vectors")
class PassVectors(Part):
    """One vector per pass of a run of layers that a model goes through several times with the
    same weights: a table (passes, hidden_size), of which row t is added to every row of the
    residual stream before pass t begins. The addition itself is left to the norm that reads the
    stream next (`join` hands it on as part of a `StreamAddend`), in float32."""

    graph_safe = True

    def __init__(self, prefix, precision, device, passes, hidden_size, leaf="weight"):
        super().__init__(prefix, precision, device)
        self.passes, self.hidden_size, self.leaf = passes, hidden_size, leaf
        self.table = None

    def tensors(self):
        return {self._name(self.leaf): (self.passes, self.hidden_size)}

    def load(self, fetch):
        self.table = fetch(self._name(self.leaf), torch.float32).contiguous()

    def join(self, pending, number):
        """`pending` (what the stream still lacks: None, a tensor or a StreamAddend) with pass
        `number`'s vector added to it."""
        row = self.table[number]
        if pending is None:
            return StreamAddend(bias=row)
        if isinstance(pending, UnscaledRows):
            raise ValueError("a pass cannot begin behind rows whose addition is already done")
        if isinstance(pending, StreamAddend):
            if pending.bias is not None:
                raise ValueError("two vectors wait for the same place of the stream")
            return StreamAddend(values=pending.values, weight=pending.weight, eps=pending.eps, bias=row,
                                values_bias=pending.values_bias)
        return StreamAddend(values=pending, bias=row)
