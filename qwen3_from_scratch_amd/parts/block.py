"""How a layer's parts are arranged around the residual stream."""

from ..config.registry import register_part
import torch

from .base import BiasedRows, HyperAddend, Part, TensorShape, UnscaledRows


def _says(part, what):
    return bool(getattr(part, what, False))


@register_part("block", "pre_norm")
class PreNormBlock(Part):
    """x = x + mixer(norm_1(x)); x = x + feed_forward(norm_2(x))
    (src/qwen3_from_scratch/models/transformer_block.py:38-46); a layer may lack the second half.

    The residual stream x is float32. The second addition is handed to whoever
    normalises next, so that each addition is fused with the norm that follows
    it: `forward` takes the stream and a pending delta and returns the same
    pair. In steps of few rows the addition and the norm move further, into
    the products on either side (NormSink, UnscaledRows), where the parts on
    both sides say they can; the stand-alone norm kernel serves all other cases.
    """

    graph_safe = True

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)
        self.mixer = self.feed_forward = self.mixer_norm = self.feed_forward_norm = None

    def attach(self, mixer, feed_forward=None, mixer_norm=None, feed_forward_norm=None):
        """The layer's parts, under the names its LayerSpec gave them: a block's `attach` names
        the parts it arranges as its keywords, and a layer that brings others does not build. A
        layer without a feed-forward attaches the mixer and its norm only."""
        if mixer_norm is None:
            raise ValueError("a mixer comes with the norm before it")
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a feed-forward comes with its norm, or not at all")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def entry_norm(self):
        """The norm a preceding block may fuse into its last product (see
        NormSink), or None if this block's mixer wants finished rows."""
        return self.mixer_norm if _says(self.mixer, "takes_unscaled") and hasattr(self.mixer_norm, "sink_for") else None

    def forward(self, x, pending, batch, cache, next_norm=None):
        """`pending`: None, the addend the stream still lacks, or UnscaledRows
        (then the addition is done and `mixer_norm` all but applied).
        `next_norm`: the norm that reads the stream after this block, if its
        reader takes UnscaledRows. Returns the stream and the next `pending`."""
        h = pending if isinstance(pending, UnscaledRows) else self.mixer_norm.forward(x, delta=pending)
        sink = None
        if (self.feed_forward is not None and _says(self.mixer, "feeds_sink") and _says(self.feed_forward, "takes_unscaled")
                and hasattr(self.feed_forward_norm, "sink_for")):
            sink = self.feed_forward_norm.sink_for(x)
        d = self.mixer.forward(h, batch, cache, sink=sink) if sink is not None else self.mixer.forward(h, batch, cache)
        if self.feed_forward is None:
            return x, d
        h = d if isinstance(d, UnscaledRows) else self.feed_forward_norm.forward(x, delta=d)
        sink = next_norm.sink_for(x) if next_norm is not None and _says(self.feed_forward, "feeds_sink") else None
        if sink is not None:
            return x, self.feed_forward.forward(h, batch, sink=sink)
        return x, self.feed_forward.forward(h, batch)


@register_part("block", "sandwich")
class SandwichBlock(Part):
    """x = x + norm_1b(mixer(norm_1(x))); x = x + norm_2b(feed_forward(norm_2(x))): a norm before
    and a norm behind each part. A layer without a feed-forward attaches the mixer and its two
    norms only. What a part returns is not normalised by a kernel of its own: it travels as a
    `StreamAddend` to the norm that reads the stream next (this block's second, or the next
    block's first, or the model's last), which normalises it, adds it into the float32 stream and
    normalises the stream in one pass; a norm that cannot take that (no `as_addend`) is applied
    on the spot."""

    graph_safe = True

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)
        self.mixer = self.feed_forward = None
        self.mixer_norm = self.mixer_out_norm = self.feed_forward_norm = self.feed_forward_out_norm = None

    def attach(self, mixer, mixer_norm, mixer_out_norm, feed_forward=None, feed_forward_norm=None,
               feed_forward_out_norm=None):
        if (feed_forward is None) != (feed_forward_norm is None) or (feed_forward is None) != (feed_forward_out_norm is None):
            raise ValueError("a feed-forward comes with a norm before and a norm behind it, or not at all")
        self.mixer, self.mixer_norm, self.mixer_out_norm = mixer, mixer_norm, mixer_out_norm
        self.feed_forward, self.feed_forward_norm = feed_forward, feed_forward_norm
        self.feed_forward_out_norm = feed_forward_out_norm

    @staticmethod
    def _behind(norm, values):
        if hasattr(norm, "as_addend"):
            return norm.as_addend(values)
        if isinstance(values, BiasedRows):
            values = values.finished()
        return norm.forward(values.float())

    def forward(self, x, pending, batch, cache, next_norm=None):
        mixed = self.mixer.forward(self.mixer_norm.forward(x, delta=pending), batch, cache)
        pending = self._behind(self.mixer_out_norm, mixed)
        if self.feed_forward is None:
            return x, pending
        fed = self.feed_forward.forward(self.feed_forward_norm.forward(x, delta=pending), batch)
        return x, self._behind(self.feed_forward_out_norm, fed)


@register_part("block", "hyper_connections")
class HyperConnectionBlock(Part):
    """A pre-norm layer over a residual that is held in `streams` copies x_1 .. x_n, (T, streams,
    width) float32. Sublayer q (1: the mixer, 2: the feed-forward, which a layer may lack) has
    three small tensors `hc<q>.in` (n), `hc<q>.out` (n) and `hc<q>.mix` (n, n), indexed [from, to]:

        u = sum_s in[s] x_s,   y = sublayer(norm_q(u)),   x_t <- sum_s mix[s, t] x_s + mult out[t] y

    for all t at once from the old streams. With `streams` 0 the layer has no such tensors and the
    residual is the ordinary one, x <- x + mult y, which is the same computation with one stream,
    in = out = mix = 1. The update of one sublayer and the read of the next are one kernel: what a
    sublayer returns travels as a `HyperAddend` to the norm that reads the streams next (this
    block's second, the next block's first, or the model's last, which reads their plain sum)."""

    graph_safe = True

    def __init__(self, prefix, precision, device, streams, mult=1.0):
        super().__init__(prefix, precision, device)
        self.streams, self.mult = int(streams), float(mult)
        if not 0 <= self.streams <= 8:
            raise ValueError("the kernel that updates and reads the streams takes up to 8 of them, not %d" % self.streams)
        self.mixer = self.feed_forward = self.mixer_norm = self.feed_forward_norm = None
        self.tables = {}

    def attach(self, mixer, mixer_norm, feed_forward=None, feed_forward_norm=None):
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a feed-forward comes with its norm, or not at all")
        self.mixer, self.mixer_norm = mixer, mixer_norm
        self.feed_forward, self.feed_forward_norm = feed_forward, feed_forward_norm

    def _sublayers(self):
        return (1, 2) if self.feed_forward is not None else (1,)

    def tensors(self):
        names, n = {}, self.streams
        if n:
            for q in self._sublayers():
                names[self._name("hc%d.in" % q)] = TensorShape((n,), "scale")
                names[self._name("hc%d.out" % q)] = TensorShape((n,), "scale")
                names[self._name("hc%d.mix" % q)] = TensorShape((n, n), "matrix")
        return names

    def load(self, fetch):
        for q in self._sublayers():
            if self.streams:
                read = fetch(self._name("hc%d.in" % q), torch.float32).contiguous()
                write = (fetch(self._name("hc%d.out" % q), torch.float32) * self.mult).contiguous()
                mix = fetch(self._name("hc%d.mix" % q), torch.float32).contiguous()
            else:
                read = torch.ones(1, dtype=torch.float32, device=self.device)
                write = torch.full((1,), self.mult, dtype=torch.float32, device=self.device)
                mix = torch.ones((1, 1), dtype=torch.float32, device=self.device)
            self.tables[q] = (read, write, mix)

    def forward(self, x, pending, batch, cache, next_norm=None):
        read, write, mix = self.tables[1]
        y = self.mixer.forward(self.mixer_norm.forward(x, delta=pending, read=read), batch, cache)
        pending = HyperAddend(y, mix, write)
        if self.feed_forward is not None:
            read, write, mix = self.tables[2]
            y = self.feed_forward.forward(self.feed_forward_norm.forward(x, delta=pending, read=read), batch)
            pending = HyperAddend(y, mix, write)
        return x, pending
