"""Norms over the last dimension."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import BiasedRows, HyperAddend, NormSink, Part, StreamAddend, TensorShape


def _no_extra_rows(addend, norm):
    if addend.extra is not None:
        raise ValueError("%s takes no rows of their own among what the stream still lacks; the norm "
                         "'layer_bias' does" % type(norm).__name__)


@register_part("norm", "rms")
class RMSNorm(Part):
    """y = x * rsqrt(mean(x^2) + eps) * weight, eps inside the root, plain weight
    (src/qwen3_from_scratch/models/norm.py:18-22,51-53). It reads the float32
    residual stream and can fold the pending addition `x += delta` into the
    same pass; the sum, the mean and the products are float32 and the result
    is rounded once."""

    graph_safe = True

    def __init__(self, prefix, precision, device, size, eps, leaf="weight"):
        super().__init__(prefix, precision, device)
        self.size = size
        self.eps = float(eps)
        self.leaf = leaf            # the tensor's name below the prefix; "" if it is the prefix itself
        self.weight = None

    def tensors(self):
        return {self._name(self.leaf): TensorShape((self.size,), "scale")}

    def load(self, fetch):
        self.weight = fetch(self._name(self.leaf))

    def forward(self, x, delta=None, rows=None):
        """Normalised rows in the activation dtype. With `delta`, x += delta
        first (in place, unless `rows` selects a subset: then x is left alone)."""
        if isinstance(delta, StreamAddend):
            _no_extra_rows(delta, self)
            return ops.rmsnorm_addend(x, self.weight, self.eps, self.precision.act, delta=delta.values,
                                      delta_weight=delta.weight, delta_eps=delta.eps, bias=delta.bias, rows=rows,
                                      write_back=rows is None, delta_bias=delta.values_bias)
        return ops.rmsnorm(x, self.weight, self.eps, self.precision.act, delta=delta,
                           rows=rows, write_back=rows is None)

    def as_addend(self, values):
        """`values` (a part's result, a tensor or `BiasedRows`) as what the stream still lacks, to be
        normalised by this norm on its way in: the norm that reads the stream next does both in one
        kernel."""
        if isinstance(values, BiasedRows):
            return StreamAddend(values=values.values, weight=self.weight, eps=self.eps, values_bias=values.bias)
        return StreamAddend(values=values, weight=self.weight, eps=self.eps)

    def sink_for(self, x):
        """A NormSink for the residual `x` if this step may have the addition
        and this norm fused into the neighbouring products (bfloat16 with
        tiled matrices; at most 16 rows and a width in steps of 16, or up to
        128 rows and a width in steps of 64), else None."""
        rows = x.shape[0]
        if self.precision.act != torch.bfloat16 or not self.precision.tiled or self.weight is None:
            return None
        if not 1 <= rows <= ops.FUSED_ROWS_MOST or self.size % (16 if rows <= ops.FUSED_ROWS_FEW else 64):
            return None
        return NormSink(x, self.weight, self.eps, self.size)


@register_part("norm", "none")
class StreamReader(Part):
    """No norm at all, in a norm's place: y = x, the float32 residual stream rounded once to the
    activation dtype, for sublayers that read the stream as it is (a layer that normalises only
    what its parts return). Like the norms it folds the pending addition into its pass: a
    `StreamAddend` is normalised, added into the stream and the sum read in one kernel. It has no
    tensors; `size` is the stream's width."""

    graph_safe = True

    def __init__(self, prefix, precision, device, size):
        super().__init__(prefix, precision, device)
        self.size = size

    def forward(self, x, delta=None, rows=None):
        if not isinstance(delta, StreamAddend):
            delta = StreamAddend(values=delta)
        _no_extra_rows(delta, self)
        return ops.rmsnorm_addend(x, None, 0.0, self.precision.act, delta=delta.values, delta_weight=delta.weight,
                                  delta_eps=delta.eps, bias=delta.bias, rows=rows, write_back=rows is None,
                                  delta_bias=delta.values_bias, plain=True)


@register_part("norm", "layer")
class LayerNorm(Part):
    """y = (u - mean(u)) * rsqrt(var(u) + eps) * weight, var the mean of the squared deviations,
    a weight and no bias. u is read from a float32 residual that is held in one or several
    streams, (T, width) or (T, streams, width): u = sum_s read[s] x_s (`read` None: the plain sum,
    which is also what the model's last norm wants). A `HyperAddend` given as `delta` first enters
    all streams at once (x_t <- sum_s mix[s, t] x_s + write[t] y), a plain tensor is added to the
    only stream; all of it float32 in one kernel, the result rounded once."""

    graph_safe = True

    def __init__(self, prefix, precision, device, size, eps, leaf="weight"):
        super().__init__(prefix, precision, device)
        self.size, self.eps, self.leaf = size, float(eps), leaf
        self.weight = None
        self._one = None

    def tensors(self):
        return {self._name(self.leaf): TensorShape((self.size,), "scale")}

    def load(self, fetch):
        self.weight = fetch(self._name(self.leaf), torch.float32)

    def forward(self, x, delta=None, rows=None, read=None):
        streams = x if x.dim() == 3 else x.unsqueeze(1)
        mix = write = values = None
        if isinstance(delta, HyperAddend):
            values, mix, write = delta.values, delta.mix, delta.write
        elif delta is not None:
            if streams.shape[1] != 1:
                raise ValueError("a plain addend joins a residual of one stream, not %d" % streams.shape[1])
            if self._one is None:
                self._one = torch.ones((1, 1), dtype=torch.float32, device=x.device)
            values, mix, write = delta, self._one, self._one[0]
        return ops.hyper_norm(streams, self.weight, self.eps, self.precision.act, read=read, delta=values, mix=mix,
                              write=write, rows=rows, write_back=rows is None)


@register_part("norm", "layer_bias")
class BiasedLayerNorm(Part):
    """y = (x - mean(x)) * rsqrt(var(x) + eps) * weight + bias, var the mean of the squared deviations
    (the mean is taken out first), over the float32 residual stream (T, width). Like the other norms it
    folds what the stream still lacks into its pass: a part's result (a tensor in the activation
    dtype), or a `StreamAddend` whose result, vector for every row and float32 rows of their own all
    join in float32 in the one kernel, before the norm; a result that is itself to be normalised
    first is not taken. The weight is the tensor `leaf` under the prefix ("" for the prefix itself),
    the bias the same name with `bias_suffix` added; both are used as float32."""

    graph_safe = True

    def __init__(self, prefix, precision, device, size, eps, leaf="weight", bias_suffix=".b"):
        super().__init__(prefix, precision, device)
        self.size, self.eps, self.leaf, self.bias_suffix = size, float(eps), leaf, bias_suffix
        self.weight = self.bias = None

    def tensors(self):
        name = self._name(self.leaf)
        return {name: TensorShape((self.size,), "scale"), name + self.bias_suffix: TensorShape((self.size,), "bias")}

    def load(self, fetch):
        name = self._name(self.leaf)
        self.weight = fetch(name, torch.float32).contiguous()
        self.bias = fetch(name + self.bias_suffix, torch.float32).contiguous()

    def forward(self, x, delta=None, rows=None):
        """Normalised rows in the activation dtype. With `delta`, the stream is brought up to date first
        (in place, unless `rows` selects a subset: then x is left alone)."""
        values = extra = vec = None
        if isinstance(delta, StreamAddend):
            if delta.weight is not None or delta.values_bias is not None:
                raise ValueError("BiasedLayerNorm adds a result as it is: it neither normalises it first nor "
                                 "carries a bias of its last product")
            values, extra, vec = delta.values, delta.extra, delta.bias
        elif isinstance(delta, BiasedRows):
            values = delta.finished()
        elif delta is not None:
            values = delta
        return ops.layernorm_addend(x, self.weight, self.bias, self.eps, self.precision.act, delta=values, extra=extra,
                                    vec=vec, rows=rows, write_back=rows is None)
