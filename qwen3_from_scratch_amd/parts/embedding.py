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
    stream next (`join` hands it on as part of a `StreamAddend`), in float32. With `restart` every
    pass but the first also begins with the embedding's output added to the stream once more, rows
    that the model keeps for this (`wants_start`) and that travel the same way."""

    graph_safe = True

    def __init__(self, prefix, precision, device, passes, hidden_size, leaf="weight", restart=False):
        super().__init__(prefix, precision, device)
        self.passes, self.hidden_size, self.leaf = passes, hidden_size, leaf
        self.restart = bool(restart)
        self.table = None

    @property
    def wants_start(self):
        """Whether `join` needs the stream as the embedding left it (a copy: the stream itself moves on)."""
        return self.restart and self.passes > 1

    def tensors(self):
        return {self._name(self.leaf): (self.passes, self.hidden_size)}

    def load(self, fetch):
        self.table = fetch(self._name(self.leaf), torch.float32).contiguous()

    def join(self, pending, number, start=None):
        """`pending` (what the stream still lacks: None, a tensor or a StreamAddend) with pass
        `number`'s vector added to it and, with `restart`, for every pass but the first also `start`,
        the float32 rows the embedding gave."""
        row = self.table[number]
        extra = None
        if self.restart and number > 0:
            if start is None:
                raise ValueError("pass %d begins with the embedding's output once more, which was not kept" % number)
            extra = start
        if pending is None:
            return StreamAddend(bias=row, extra=extra)
        if isinstance(pending, UnscaledRows):
            raise ValueError("a pass cannot begin behind rows whose addition is already done")
        if isinstance(pending, StreamAddend):
            if pending.bias is not None or pending.extra is not None:
                raise ValueError("two vectors wait for the same place of the stream")
            return StreamAddend(values=pending.values, weight=pending.weight, eps=pending.eps, bias=row,
                                values_bias=pending.values_bias, extra=extra)
        return StreamAddend(values=pending, bias=row, extra=extra)
