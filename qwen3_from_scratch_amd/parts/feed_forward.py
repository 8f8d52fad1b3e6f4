"""Feed-forward parts."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import BiasedRows, Part, TensorShape
from .linear import LinearWeight


@register_part("feed_forward", "swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)), no biases
    (src/qwen3_from_scratch/models/feedback.py:28-34). gate and up are kept as
    one matrix with their rows interleaved (row 2i gate's, row 2i + 1 up's), so
    that one product feeds the activation, which for few rows is the product
    kernel's epilogue (the reference's fused variant concatenates them,
    feedback.py:52-54). `activation`: what the gate passes, "silu" or one of the other kinds of
    `ops.GATE_KINDS` (the tanh form of gelu, the exact gelu), which run as the plain product and an
    activation kernel behind it."""

    graph_safe = True
    feeds_sink = True

    def __init__(self, prefix, precision, device, hidden_size, intermediate_size,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight"), activation="silu"):
        super().__init__(prefix, precision, device)
        if activation not in ops.GATE_KINDS:
            raise ValueError("activation is one of %s" % ", ".join(sorted(ops.GATE_KINDS)))
        self.activation = activation
        self.names = tuple(names)         # the tensors' names below the prefix: gate, up, down
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up = None
        self.down = None

    def tensors(self):
        H, I = self.hidden_size, self.intermediate_size
        gate, up, down = self.names
        return {self._name(gate): (I, H), self._name(up): (I, H), self._name(down): (H, I)}

    def load(self, fetch):
        act = self.precision.act
        I, H = self.intermediate_size, self.hidden_size
        gate_up = torch.empty((2 * I, H), dtype=act, device=self.device)
        gate, up, down = self.names
        gate_up[0::2].copy_(fetch(self._name(gate), act, keep=False))
        gate_up[1::2].copy_(fetch(self._name(up), act, keep=False))
        self.gate_up = LinearWeight(gate_up, self.precision)
        self.down = LinearWeight(fetch(self._name(down), act), self.precision)

    @property
    def takes_unscaled(self):
        return self.activation == "silu" and self.gate_up is not None and self.gate_up.fuses

    def forward(self, x, batch=None, sink=None):
        if self.activation == "silu":
            h = self.gate_up.forward_swiglu(x)
        else:
            h = ops.gated_act(self.gate_up.forward(x), self.activation)
        return self.down.forward(h) if sink is None else self.down.forward_into(h, sink)


@register_part("feed_forward", "clamped_glu")
class ClampedGLU(Part):
    """g = min(W_gate h + b_gate, limit), u = clamp(W_up h + b_up, -limit, limit);
    y = g sigmoid(slope g) (u + 1); the result is W_down y + b_down. Tensors: gate, gate.b, up, up.b,
    down, down.b. gate and up are kept as one matrix with their rows interleaved (row 2i gate's, row
    2i + 1 up's) and their product leaves float32 rows, so biases, clamps and the activation see
    unrounded numbers. The last bias is not added here: it travels with the result (`BiasedRows`)
    and joins it in float32 where the result enters the residual stream."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, intermediate_size, limit, slope=1.702):
        super().__init__(prefix, precision, device)
        if not limit > 0:
            raise ValueError("limit must be positive")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.limit, self.slope = float(limit), float(slope)
        self.gate_up = self.down = self.bias_in = self.bias_out = None

    def tensors(self):
        H, I = self.hidden_size, self.intermediate_size
        return {self._name("gate"): (I, H), self._name("gate.b"): TensorShape((I,), "bias"),
                self._name("up"): (I, H), self._name("up.b"): TensorShape((I,), "bias"),
                self._name("down"): (H, I), self._name("down.b"): TensorShape((H,), "bias")}

    def load(self, fetch):
        act = self.precision.act
        I, H = self.intermediate_size, self.hidden_size
        gate_up = torch.empty((2 * I, H), dtype=act, device=self.device)
        gate_up[0::2].copy_(fetch(self._name("gate"), act, keep=False))
        gate_up[1::2].copy_(fetch(self._name("up"), act, keep=False))
        self.gate_up = LinearWeight(gate_up, self.precision)
        self.down = LinearWeight(fetch(self._name("down"), act), self.precision)
        bias = torch.empty((2 * I,), dtype=torch.float32, device=self.device)
        bias[0::2].copy_(fetch(self._name("gate.b"), torch.float32))
        bias[1::2].copy_(fetch(self._name("up.b"), torch.float32))
        self.bias_in = bias
        self.bias_out = fetch(self._name("down.b"), torch.float32).contiguous()

    def forward(self, x, batch=None):
        both = self.gate_up.forward(x, out_dtype=torch.float32)
        hidden = ops.glu_clamped(both, self.limit, self.slope, bias=self.bias_in, out_dtype=self.precision.act)
        return BiasedRows(self.down.forward(hidden), self.bias_out)
