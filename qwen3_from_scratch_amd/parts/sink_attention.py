"""Softmax attention with a sink per head, a norm per head on queries and keys, no rotation and a
gate per head; a layer may read another layer's keys and values."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import CacheNeed, PagedTensor, Part, TensorShape
from .linear import LinearWeight


@register_part("mixer", "sink_attention")
class SinkAttention(Part):
    """q = W_q h (heads x dim), k = W_k h (kv_heads x dim), v = W_v h (kv_heads x vdim), no biases;
    query head a reads key head a // (heads / kv_heads). Every head of q and of k is divided by its
    own root mean square and multiplied by a weight of dim numbers that the heads share (`q.norm`,
    `k.norm`). Positions do not enter the scores: score = (q . k) scale over the keys at positions
    j <= i (the last `window` of them, 0: all). The softmax's denominator also holds exp(sink_a), a
    learned number per head that has no key and no value and is not scaled; head a's result is
    multiplied by sigmoid(W_g h)_a before the output product.

    With `own_keys` false the layer has no W_k, W_v and k.norm: its run-order entry reads the cache
    of the layer that made the keys (after their norm) and values, with queries, sink, gate and
    output product of its own. All products of a layer are one and leave float32 rows; norms,
    scores and the softmax are float32. Keys and values are paged as the matrix-core attention
    kernels read them, a page of keys (kv_heads, page, dim) and a page of values (kv_heads, vdim,
    page): bfloat16 with equal key and value sizes of 64 or 128 runs on those kernels, everything
    else on a general one."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, heads, kv_heads, dim, vdim, scale, eps, own_keys=True,
                 window=0):
        super().__init__(prefix, precision, device)
        if heads % kv_heads:
            raise ValueError("heads (%d) must be a multiple of kv_heads (%d)" % (heads, kv_heads))
        if dim > 512 or vdim > 512:
            raise ValueError("the attention kernels take keys and values of up to 512 numbers, not %d and %d" % (dim, vdim))
        self.hidden_size, self.heads, self.kv_heads, self.dim, self.vdim = hidden_size, heads, kv_heads, dim, vdim
        self.scale, self.eps, self.window, self.own_keys = float(scale), float(eps), int(window), bool(own_keys)
        self.w_in = self.w_out = self.q_norm = self.k_norm = self.sink = None

    def cache_need(self):
        return CacheNeed(paged=(PagedTensor("keys", (self.kv_heads, self.dim), token_axis=1),
                                PagedTensor("values", (self.kv_heads, self.vdim), token_axis=2)), window=self.window)

    def _projections(self):
        return ("q", "k", "v", "g") if self.own_keys else ("q", "g")

    def tensors(self):
        H, G, d, dv, W = self.heads, self.kv_heads, self.dim, self.vdim, self.hidden_size
        names = {self._name("q"): (H * d, W), self._name("q.norm"): TensorShape((d,), "scale"),
                 self._name("sink"): TensorShape((H,), "bias"), self._name("g"): (H, W), self._name("o"): (W, H * dv)}
        if self.own_keys:
            names.update({self._name("k"): (G * d, W), self._name("v"): (G * dv, W),
                          self._name("k.norm"): TensorShape((d,), "scale")})
        return names

    def load(self, fetch):
        act = self.precision.act
        joined = torch.cat([fetch(self._name(n), act, keep=False) for n in self._projections()], dim=0)
        self.w_in = LinearWeight(joined.contiguous(), self.precision)
        self.w_out = LinearWeight(fetch(self._name("o"), act), self.precision)
        self.q_norm = fetch(self._name("q.norm"), torch.float32)
        self.k_norm = fetch(self._name("k.norm"), torch.float32) if self.own_keys else None
        self.sink = fetch(self._name("sink"), torch.float32)

    def forward(self, x, batch, cache):
        H, d, dv = self.heads, self.dim, self.vdim
        if cache.writes != self.own_keys:
            raise ValueError("%s: a layer with keys of its own writes its cache, one without reads another's" % self.prefix)
        G = self.kv_heads if self.own_keys else 0
        rows = self.w_in.forward(x, out_dtype=torch.float32)
        keys, values = cache.paged["keys"], cache.paged["values"]
        q = ops.headnorm_prepare(rows, H, G, d, dv, self.q_norm, self.k_norm, self.eps, batch.positions, batch.seq_index,
                                 self.precision.act, block_table=cache.block_table, k_cache=keys, v_cache=values,
                                 values_transposed=True)
        mixed = ops.softcap_attention(q, keys, values, cache.block_table, batch.cu_seqlens_q, batch.kv_lens,
                                      batch.seq_index, batch.positions, batch.max_q_len, batch.max_kv_len, self.scale,
                                      0.0, window=self.window, gate=rows[:, H * d + G * (d + dv):], sink=self.sink,
                                      values_transposed=True, min_q_len=batch.min_q_len,
                                      max_kv_len_of_many=getattr(batch, "max_kv_len_portions", None))
        return self.w_out.forward(mixed)
