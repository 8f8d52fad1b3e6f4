"""The gated delta rule with a decay per head and key channel, behind short convolutions."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import AnySize, CacheNeed, Part, TensorShape
from .linear import LinearWeight


@register_part("mixer", "channel_delta")
class ChannelDelta(Part):
    """q = W_q h and k = W_k h (kv_heads x dim), v = W_v h (heads x vdim), no biases; head a reads q
    and k of group a // (heads / kv_heads). Each of the three passes a causal convolution per channel
    (`conv` taps, the last tap the current token's, zeros before the start, no bias) and silu; q and
    k then become unit vectors per head, x / sqrt(sum(x^2) + unit_eps), q also times dim^(-1/2). With
    beta = sigmoid(W_b h), a number per head, and one decay per head and key channel,
    g = exp(-exp(A_log_a) softplus(W_a2 (W_a1 h) + dt_bias)), per head

        S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q     (S: dim x vdim)

    in this order, so the read-out sees the current token's write. Each head's o is divided by its
    root mean square (eps inside the root), multiplied by `norm` (vdim numbers the heads share) and
    by sigmoid(W_g2 (W_g1 h)), and goes through the output product. The two products through a
    narrow middle take their middle's size from the stored tensors (`rank`: what random weights
    are made with).

    Products: [q | k | v | b] from h in one, leaving float32 rows; [a1 | g1] from h in one; [a2 | g2]
    on that as one product with a matrix that is zero where the two do not meet, leaving float32
    rows. Convolutions, unit norms, softplus, exponentials, beta, g, S and the norm are float32.
    Per request the mixer keeps the convolutions' last taps - 1 inputs and S, one float32 vector;
    S lies (head, column, row), a column's numbers side by side."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, heads, kv_heads, dim, vdim, conv, eps, unit_eps=1e-6,
                 rank=0):
        super().__init__(prefix, precision, device)
        if heads % kv_heads:
            raise ValueError("heads (%d) must be a multiple of kv_heads (%d)" % (heads, kv_heads))
        if dim > 256 or not 1 <= conv <= 8:
            raise ValueError("the delta rule's kernels take keys of up to 256 numbers and 1 to 8 taps, not %d and %d"
                             % (dim, conv))
        self.hidden_size, self.heads, self.kv_heads, self.dim, self.vdim = hidden_size, heads, kv_heads, dim, vdim
        self.taps, self.eps, self.unit_eps = int(conv), float(eps), float(unit_eps)
        self.rank = AnySize(rank if rank else max(8, dim // 2))
        self.channels = 2 * kv_heads * dim + heads * vdim
        self.w_in = self.w_low = self.w_up = self.w_out = None
        self.conv = self.no_bias = self.dt_bias = self.a_log = self.norm = None

    def _tail(self):
        return (self.taps - 1) * self.channels

    def cache_need(self):
        return CacheNeed(state_shape=(self._tail() + self.heads * self.dim * self.vdim,), state_dtype=torch.float32)

    def tensors(self):
        H, G, d, dv, W, r = self.heads, self.kv_heads, self.dim, self.vdim, self.hidden_size, self.rank
        names = {self._name("b"): (H, W), self._name("A_log"): TensorShape((H,), "bias"),
                 self._name("dt_bias"): TensorShape((H * d,), "bias"), self._name("norm"): TensorShape((dv,), "scale"),
                 self._name("a1"): (r, W), self._name("a2"): (H * d, r), self._name("g1"): (r, W),
                 self._name("g2"): (H * dv, r), self._name("o"): (W, H * dv)}
        for name, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
            names[self._name(name)] = (n, W)
            names[self._name(name + ".conv")] = (n, self.taps)
        return names

    def load(self, fetch):
        act, H, d, dv = self.precision.act, self.heads, self.dim, self.vdim
        joined = torch.cat([fetch(self._name(n), act, keep=False) for n in ("q", "k", "v", "b")], dim=0)
        self.w_in = LinearWeight(joined.contiguous(), self.precision)
        a1, g1 = fetch(self._name("a1"), act, keep=False), fetch(self._name("g1"), act, keep=False)
        a2, g2 = fetch(self._name("a2"), act, keep=False), fetch(self._name("g2"), act, keep=False)
        ra, rg = a1.shape[0], g1.shape[0]
        if a2.shape[1] != ra or g2.shape[1] != rg:
            raise ValueError("%s: the two halves of a product through a narrow middle disagree about its size" % self.prefix)
        self.w_low = LinearWeight(torch.cat((a1, g1), dim=0).contiguous(), self.precision)
        up = torch.zeros((H * d + H * dv, ra + rg), dtype=act, device=self.device)
        up[:H * d, :ra].copy_(a2)
        up[H * d:, ra:].copy_(g2)
        self.w_up = LinearWeight(up, self.precision)
        self.w_out = LinearWeight(fetch(self._name("o"), act), self.precision)
        self.conv = torch.cat([fetch(self._name(n + ".conv"), torch.float32) for n in ("q", "k", "v")], dim=0).contiguous()
        self.no_bias = torch.zeros(self.channels, dtype=torch.float32, device=self.device)
        self.dt_bias = fetch(self._name("dt_bias"), torch.float32)
        self.a_log = fetch(self._name("A_log"), torch.float32)
        self.norm = fetch(self._name("norm"), torch.float32)

    def forward(self, x, batch, cache):
        H, d, C, tail = self.heads, self.dim, self.channels, self._tail()
        rows = self.w_in.forward(x, out_dtype=torch.float32)
        wide = self.w_up.forward(self.w_low.forward(x), out_dtype=torch.float32)
        qkv = ops.causal_conv(rows[:, :C], self.conv, self.no_bias, cache.state[:, :tail], batch.state_slots,
                              batch.cu_seqlens_q, batch.seq_index, activation="silu", out_dtype=torch.float32,
                              max_q_len=batch.max_q_len)
        mixed = ops.channel_delta(qkv, rows[:, C:], wide[:, :H * d], wide[:, H * d:], self.dt_bias, self.a_log, self.norm,
                                  self.eps, self.unit_eps, cache.state[:, tail:], batch.state_slots, batch.cu_seqlens_q,
                                  H, self.kv_heads, d, self.vdim, self.precision.act)
        return self.w_out.forward(mixed)
