"""Softmax attention with biased projections, a norm over the whole query and key projections,
capped scores and a gate per head."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import CacheNeed, PagedTensor, Part, TensorShape
from .linear import LinearWeight
from .position import rotation_frequencies


@register_part("mixer", "softcap_attention")
class SoftcapAttention(Part):
    """q = W_q h + b_q (heads x dim), k = W_k h + b_k (kv_heads x dim), v = W_v h + b_v (kv_heads x
    vdim); query head a reads key head a // (heads / kv_heads). q and k are each divided by the
    root mean square of the whole projection (all heads at once) and multiplied by a weight of
    that size, then turn by the position over the first `rot_dims` numbers of every head, pairs
    (2i, 2i + 1), frequency rot_base^(-2i / rot_dims). score = (q . k) scale, then
    softcap * tanh(score / softcap) (softcap 0: as it is); softmax over the keys at positions
    j <= i (the last `window` of them, 0: all); head a's result is multiplied by sigmoid(W_g h)_a
    before the output product. `biases` false: the three projections have no biases (no `.b` tensors);
    `gated` false: no gate (no `g`). The products are one and leave float32 rows, so biases and
    norms see unrounded numbers; norms, angles, scores and the softmax are float32. Keys (rotated)
    and values are paged, a page of keys (kv_heads, page, dim) and a page of values (kv_heads, vdim,
    page), transposed within the page as the matrix-core attention kernels read them: bfloat16 with
    equal key and value sizes of 64 or 128 runs on those kernels, everything else on a general one."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, heads, kv_heads, dim, vdim, scale, eps, softcap=0.0,
                 rot_dims=0, rot_base=1.0, window=0, biases=True, gated=True):
        super().__init__(prefix, precision, device)
        if heads % kv_heads:
            raise ValueError("heads (%d) must be a multiple of kv_heads (%d)" % (heads, kv_heads))
        if dim > 512 or vdim > 512 or rot_dims > dim or rot_dims % 2:
            raise ValueError("the attention kernels take keys and values of up to 512 numbers and an even rotation within "
                             "the keys, not %d, %d and %d" % (dim, vdim, rot_dims))
        self.hidden_size, self.heads, self.kv_heads, self.dim, self.vdim = hidden_size, heads, kv_heads, dim, vdim
        self.scale, self.eps, self.softcap, self.window = float(scale), float(eps), float(softcap), int(window)
        self.rot_dims, self.rot_base = int(rot_dims), float(rot_base)
        self.biases, self.gated = bool(biases), bool(gated)
        self.w_in = self.w_out = self.bias = self.q_norm = self.k_norm = self.inv_freq = None

    def cache_need(self):
        return CacheNeed(paged=(PagedTensor("keys", (self.kv_heads, self.dim), token_axis=1),
                                PagedTensor("values", (self.kv_heads, self.vdim), token_axis=2)), window=self.window)

    def tensors(self):
        H, G, d, dv, W = self.heads, self.kv_heads, self.dim, self.vdim, self.hidden_size
        names = {self._name("q"): (H * d, W), self._name("k"): (G * d, W), self._name("v"): (G * dv, W),
                 self._name("q.norm"): TensorShape((H * d,), "scale"), self._name("k.norm"): TensorShape((G * d,), "scale"),
                 self._name("o"): (W, H * dv)}
        if self.biases:
            names.update({self._name("q.b"): TensorShape((H * d,), "bias"), self._name("k.b"): TensorShape((G * d,), "bias"),
                          self._name("v.b"): TensorShape((G * dv,), "bias")})
        if self.gated:
            names[self._name("g")] = (H, W)
        return names

    def load(self, fetch):
        act = self.precision.act
        joined = torch.cat([fetch(self._name(n), act, keep=False)
                            for n in (("q", "k", "v", "g") if self.gated else ("q", "k", "v"))], dim=0)
        self.w_in = LinearWeight(joined.contiguous(), self.precision)
        self.w_out = LinearWeight(fetch(self._name("o"), act), self.precision)
        if self.biases:
            self.bias = torch.cat([fetch(self._name(n + ".b"), torch.float32) for n in ("q", "k", "v")]).contiguous()
        self.q_norm = fetch(self._name("q.norm"), torch.float32)
        self.k_norm = fetch(self._name("k.norm"), torch.float32)
        self.inv_freq = rotation_frequencies(self.rot_dims, self.rot_base, self.device)

    def forward(self, x, batch, cache):
        H, G, d, dv = self.heads, self.kv_heads, self.dim, self.vdim
        rows = self.w_in.forward(x, out_dtype=torch.float32)
        keys, values = cache.paged["keys"], cache.paged["values"]
        q = ops.softcap_prepare(rows, self.bias, H, G, d, dv, self.q_norm, self.k_norm, self.eps, self.inv_freq,
                                batch.positions, batch.seq_index, self.precision.act,
                                block_table=cache.block_table if cache.writes else None,
                                k_cache=keys if cache.writes else None, v_cache=values if cache.writes else None,
                                values_transposed=True)
        mixed = ops.softcap_attention(q, keys, values, cache.block_table, batch.cu_seqlens_q, batch.kv_lens,
                                      batch.seq_index, batch.positions, batch.max_q_len, batch.max_kv_len, self.scale,
                                      self.softcap, window=self.window,
                                      gate=rows[:, (H + G) * d + G * dv:] if self.gated else None,
                                      values_transposed=True, min_q_len=batch.min_q_len,
                                      max_kv_len_of_many=getattr(batch, "max_kv_len_portions", None))
        return self.w_out.forward(mixed)
