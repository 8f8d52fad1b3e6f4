"""A feed-forward of many small experts, of which a router gives each token a few."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import Part, TensorShape
from .linear import LinearWeight


@register_part("feed_forward", "routed_experts")
class RoutedExperts(Part):
    """z = W_router h (float32), s = softmax(z) over all experts; a token's `top` experts are
    those with the largest scores, weighted by s / (their sum + 1e-20); each expert is
    W_down act(W_up h) without biases; an optional shared expert of the same form (its own inner
    size) serves every token and is added. `activation`: "erf" (the exact gelu) or "tanh".

    Tensors: router (experts, hidden), e<i>.up (expert_ff, hidden), e<i>.down (hidden, expert_ff),
    shared.up (shared_ff, hidden), shared.down (hidden, shared_ff). The experts' matrices are kept
    stacked, (experts, ff, hidden) and (experts, hidden, ff); tokens are never counted on the
    host, so a step is launches only.
    """

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, experts, top, expert_ff, shared_ff=0, activation="erf"):
        super().__init__(prefix, precision, device)
        if not 1 <= top <= experts:
            raise ValueError("top (%d) must lie in 1..experts (%d)" % (top, experts))
        if activation not in ops.GELU_KINDS:
            raise ValueError("activation is one of %s" % ", ".join(sorted(ops.GELU_KINDS)))
        self.hidden_size, self.experts, self.top = hidden_size, experts, top
        self.expert_ff, self.shared_ff, self.activation = expert_ff, shared_ff, activation
        self.router = self.up = self.down = self.shared_up = self.shared_down = None

    def tensors(self):
        W = self.hidden_size
        names = {self._name("router"): (self.experts, W)}
        for e in range(self.experts):
            names[self._name("e%d.up" % e)] = (self.expert_ff, W)
            names[self._name("e%d.down" % e)] = (W, self.expert_ff)
        if self.shared_ff:
            names[self._name("shared.up")] = (self.shared_ff, W)
            names[self._name("shared.down")] = (W, self.shared_ff)
        return names

    def load(self, fetch):
        act, E = self.precision.act, self.experts
        self.router = LinearWeight(fetch(self._name("router"), act), self.precision)
        self.up = torch.stack([fetch(self._name("e%d.up" % e), act, keep=False) for e in range(E)]).contiguous()
        self.down = torch.stack([fetch(self._name("e%d.down" % e), act, keep=False) for e in range(E)]).contiguous()
        if self.shared_ff:
            self.shared_up = LinearWeight(fetch(self._name("shared.up"), act), self.precision)
            self.shared_down = LinearWeight(fetch(self._name("shared.down"), act), self.precision)

    def forward(self, x, batch=None):
        chosen, weights = ops.moe_route(x, self.router.weight, self.top, tiled=self.router.tiled)
        shared = None
        if self.shared_ff:
            shared = self.shared_down.forward(ops.gelu(self.shared_up.forward(x), self.activation))
        return ops.moe_experts(x, chosen, weights, self.up, self.down, shared=shared, activation=self.activation)


@register_part("feed_forward", "gated_experts")
class GatedExperts(Part):
    """z = W_router h (float32), s = sigmoid(z), every expert for itself; a token's `top` experts are
    those with the largest scores (the lowest index among equals) and their weights are those
    scores as they are. Each expert is a gated unit with clamped branches and no biases,
    g = min(W_gate x, limit), u = clamp(W_up x, -limit, limit), W_down (g sigmoid(slope g) (u + 1)),
    and its weight multiplies its input, not its result: the layer's result is the sum of
    expert_e(s_e h) over the chosen e.

    Tensors: router (experts, hidden), e<i>.gate and e<i>.up (expert_ff, hidden), e<i>.down (hidden,
    expert_ff). The experts' matrices are kept stacked, gate and up as one with their rows
    interleaved, (experts, 2 ff, hidden), and (experts, hidden, ff); tokens are never counted on
    the host, so a step is launches only."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, experts, top, expert_ff, limit, slope=1.702):
        super().__init__(prefix, precision, device)
        if not 1 <= top <= experts:
            raise ValueError("top (%d) must lie in 1..experts (%d)" % (top, experts))
        if not limit > 0:
            raise ValueError("limit must be positive")
        self.hidden_size, self.experts, self.top, self.expert_ff = hidden_size, experts, top, expert_ff
        self.limit, self.slope = float(limit), float(slope)
        self.router = self.gate_up = self.down = None

    def tensors(self):
        W = self.hidden_size
        names = {self._name("router"): (self.experts, W)}
        for e in range(self.experts):
            names[self._name("e%d.gate" % e)] = (self.expert_ff, W)
            names[self._name("e%d.up" % e)] = (self.expert_ff, W)
            names[self._name("e%d.down" % e)] = (W, self.expert_ff)
        return names

    def load(self, fetch):
        act, E, ff, W = self.precision.act, self.experts, self.expert_ff, self.hidden_size
        self.router = LinearWeight(fetch(self._name("router"), act), self.precision)
        gate_up = torch.empty((E, 2 * ff, W), dtype=act, device=self.device)
        for e in range(E):
            gate_up[e, 0::2].copy_(fetch(self._name("e%d.gate" % e), act, keep=False))
            gate_up[e, 1::2].copy_(fetch(self._name("e%d.up" % e), act, keep=False))
        self.gate_up = gate_up
        self.down = torch.stack([fetch(self._name("e%d.down" % e), act, keep=False) for e in range(E)]).contiguous()

    def forward(self, x, batch=None):
        chosen, weights = ops.moe_route(x, self.router.weight, self.top, tiled=self.router.tiled, scoring="sigmoid")
        return ops.moe_gated_experts(x, chosen, weights, self.gate_up, self.down, self.limit, self.slope)


@register_part("feed_forward", "grouped_experts")
class GroupedExperts(Part):
    """z = W_router h (float32), s = sigmoid(z), every expert for itself. A token's `top` experts are
    those with the largest s + correction (`correction`, a number per expert that enters the choice
    only), taken from `keep` of the `groups` equal groups of neighbouring experts: a group's score is
    the sum of its two largest s + correction, the best groups are kept, and an expert of another
    group cannot be chosen whatever its score. The weights are the chosen experts' s as they are.
    Each expert is a gated unit without biases, W_down (act(W_gate h) * (W_up h)), and the layer's
    result is the weighted sum of the chosen experts' results. A shared expert of the same form
    (inner size `shared_ff`, 0: none) serves every token and is added, multiplied by sigmoid(w_sg . h),
    one number per token.

    Tensors: router (experts, hidden), correction (experts), e<i>.gate and e<i>.up (expert_ff, hidden),
    e<i>.down (hidden, expert_ff), shared.gate, shared.up (shared_ff, hidden), shared.down (hidden,
    shared_ff), shared.sg (1, hidden). The experts' matrices are kept stacked, gate and up as one with
    their rows interleaved; the shared expert's gate vector is one more row of the router's matrix, so
    that one product with float32 sums gives the experts' logits and the gate's. Tokens are never
    counted on the host, so a step is launches only."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, experts, top, expert_ff, groups=1, keep=1, shared_ff=0,
                 activation="silu"):
        super().__init__(prefix, precision, device)
        if not 1 <= top <= experts:
            raise ValueError("top (%d) must lie in 1..experts (%d)" % (top, experts))
        if groups < 1 or experts % groups or not 1 <= keep <= groups or top > keep * (experts // groups):
            raise ValueError("groups (%d) must divide the experts (%d), keep (%d) lie in 1..groups, and the kept groups "
                             "hold at least top (%d) experts" % (groups, experts, keep, top))
        if activation not in ops.GATE_KINDS:
            raise ValueError("activation is one of %s" % ", ".join(sorted(ops.GATE_KINDS)))
        self.hidden_size, self.experts, self.top, self.expert_ff = hidden_size, experts, top, expert_ff
        self.groups, self.keep, self.shared_ff, self.activation = groups, keep, shared_ff, activation
        self.router = self.correction = self.gate_up = self.down = self.shared_gate_up = self.shared_down = None

    def tensors(self):
        W = self.hidden_size
        names = {self._name("router"): (self.experts, W), self._name("correction"): TensorShape((self.experts,), "bias")}
        for e in range(self.experts):
            names[self._name("e%d.gate" % e)] = (self.expert_ff, W)
            names[self._name("e%d.up" % e)] = (self.expert_ff, W)
            names[self._name("e%d.down" % e)] = (W, self.expert_ff)
        if self.shared_ff:
            names[self._name("shared.gate")] = (self.shared_ff, W)
            names[self._name("shared.up")] = (self.shared_ff, W)
            names[self._name("shared.down")] = (W, self.shared_ff)
            names[self._name("shared.sg")] = (1, W)
        return names

    @staticmethod
    def _interleaved(gate, up):
        both = torch.empty((2 * gate.shape[0], gate.shape[1]), dtype=gate.dtype, device=gate.device)
        both[0::2].copy_(gate)
        both[1::2].copy_(up)
        return both

    def load(self, fetch):
        act, E = self.precision.act, self.experts
        rows = [fetch(self._name("router"), act, keep=False)]
        if self.shared_ff:
            rows.append(fetch(self._name("shared.sg"), act, keep=False))
        self.router = LinearWeight(torch.cat(rows, dim=0).contiguous(), self.precision)
        self.correction = fetch(self._name("correction"), torch.float32).contiguous()
        self.gate_up = torch.stack([self._interleaved(fetch(self._name("e%d.gate" % e), act, keep=False),
                                                      fetch(self._name("e%d.up" % e), act, keep=False))
                                    for e in range(E)]).contiguous()
        self.down = torch.stack([fetch(self._name("e%d.down" % e), act, keep=False) for e in range(E)]).contiguous()
        if self.shared_ff:
            self.shared_gate_up = LinearWeight(self._interleaved(fetch(self._name("shared.gate"), act, keep=False),
                                                                 fetch(self._name("shared.up"), act, keep=False)),
                                               self.precision)
            self.shared_down = LinearWeight(fetch(self._name("shared.down"), act), self.precision)

    def forward(self, x, batch=None):
        chosen, weights, rest = ops.moe_route(x, self.router.weight, self.top, tiled=self.router.tiled,
                                              scoring="sigmoid_groups", correction=self.correction, groups=self.groups,
                                              keep=self.keep, experts=self.experts)
        shared = shared_gate = None
        if self.shared_ff:
            if self.activation == "silu":
                hidden = self.shared_gate_up.forward_swiglu(x)
            else:
                hidden = ops.gated_act(self.shared_gate_up.forward(x), self.activation)
            shared, shared_gate = self.shared_down.forward(hidden), rest
        return ops.moe_glu_experts(x, chosen, weights, self.gate_up, self.down, activation=self.activation,
                                   shared=shared, shared_gate=shared_gate)
