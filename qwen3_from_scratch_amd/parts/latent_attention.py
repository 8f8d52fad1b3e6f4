"""Attention whose keys and values are made from one narrow cached vector per token."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import CacheNeed, PagedTensor, Part, TensorShape
from .linear import LinearWeight


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    """Queries, keys and values pass through latents:

        c_q = rms_norm(W_dq h) * g_q            q_h = [W_uq c_q]_h = [q_h^n | q_h^r]   (dim | rot_dim)
        [a | b] = W_dkv h,  c = rms_norm(a) * g_kv (kv_rank),  k^r = rotate(b)  (rot_dim, one for all heads)
        k_h^n = [W_uk c]_h,  v_h = [W_uv c]_h
        score_h(i, j) = (q_h^n(i) . k_h^n(j) + rotate(q_h^r(i)) . k^r(j)) * scale,   softmax over the
        positions j <= i that lie fewer than `window` behind i (all of them with window = 0),
        out = W_o [sum_j p_h(i, j) v_h(j)]_h.

    Only [c | k^r] is cached, one row of kv_rank + rot_dim numbers per token. The per-head key
    and value matrices are applied on the query's side: q_h^n . (U_h c) = (U_h^T q_h^n) . c, so
    the attention kernel reads the cached rows as keys for every head, sums their first kv_rank
    numbers with the softmax weights, and the head's value matrix multiplies that sum. The two
    down-projections are one matrix. Norms, rotation, scores and sums are float32.

    With `rot_dim` 0 keys have no rotated part, positions do not enter the scores and the layer needs
    no position part. With `sink` the softmax's denominator of head a also holds exp(sink_a), a
    learned number per head (`sink`, (heads,)) that has no key and no value and is not scaled. With
    `gated` head a's result is multiplied by sigmoid(W_g h)_a (`g`, (heads, hidden)), a gate that reads
    the mixer's own input and rides on the down-projections' product.

    Tensors (under the part's prefix): dq (q_rank, hidden), dq.norm (q_rank), uq (heads (dim +
    rot_dim), q_rank), dkv (kv_rank + rot_dim, hidden), dkv.norm (kv_rank), uk (heads dim,
    kv_rank), uv (heads vdim, kv_rank), o (hidden, heads vdim). The rotation's frequencies come
    from the layer's position part (`frequencies()`).
    """

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, heads, dim, rot_dim, vdim, q_rank, kv_rank, scale,
                 eps, window=0, sink=False, gated=False):
        super().__init__(prefix, precision, device)
        self.hidden_size, self.heads, self.dim, self.rot_dim, self.vdim = hidden_size, heads, dim, rot_dim, vdim
        self.q_rank, self.kv_rank = q_rank, kv_rank
        self.scale, self.eps, self.window = float(scale), float(eps), int(window)
        self.has_sink, self.gated = bool(sink), bool(gated)
        self.sink = None
        self.position = None
        self.down = self.uq = self.uk = self.uv = self.out = self.q_norm = self.kv_norm = None

    def attach_position(self, position):
        if not self.rot_dim:
            return
        if not hasattr(position, "frequencies"):
            raise ValueError("latent attention rotates by frequencies; the position part %s has none"
                             % type(position).__name__)
        self.position = position

    def cache_need(self):
        return CacheNeed(paged=(PagedTensor("latent", (self.kv_rank + self.rot_dim,), token_axis=0),),
                         window=self.window)

    def tensors(self):
        H, W = self.heads, self.hidden_size
        names = {
            self._name("dq"): (self.q_rank, W),
            self._name("dq.norm"): TensorShape((self.q_rank,), "scale"),
            self._name("uq"): (H * (self.dim + self.rot_dim), self.q_rank),
            self._name("dkv"): (self.kv_rank + self.rot_dim, W),
            self._name("dkv.norm"): TensorShape((self.kv_rank,), "scale"),
            self._name("uk"): (H * self.dim, self.kv_rank),
            self._name("uv"): (H * self.vdim, self.kv_rank),
            self._name("o"): (W, H * self.vdim),
        }
        if self.has_sink:
            names[self._name("sink")] = TensorShape((H,), "bias")
        if self.gated:
            names[self._name("g")] = (H, W)
        return names

    def load(self, fetch):
        act, H = self.precision.act, self.heads
        down = torch.cat([fetch(self._name(n), act, keep=False) for n in (("dq", "dkv", "g") if self.gated else ("dq", "dkv"))],
                         dim=0)
        self.down = LinearWeight(down.contiguous(), self.precision)
        self.uq = LinearWeight(fetch(self._name("uq"), act), self.precision)
        # per head (result index, summed index): uk transposed (it is applied to the query), uv as stored
        self.uk = fetch(self._name("uk"), act, keep=False).view(H, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.uv = fetch(self._name("uv"), act).view(H, self.vdim, self.kv_rank).contiguous()
        self.out = LinearWeight(fetch(self._name("o"), act), self.precision)
        self.q_norm = fetch(self._name("dq.norm"))
        self.kv_norm = fetch(self._name("dkv.norm"))
        if self.has_sink:
            self.sink = fetch(self._name("sink"), torch.float32).contiguous()

    def forward(self, x, batch, cache):
        H, dn, dr, rank = self.heads, self.dim, self.rot_dim, self.kv_rank
        inv_freq, factor = self.position.frequencies() if dr else (None, 1.0)
        latent = cache.paged["latent"]
        down = self.down.forward(x)
        cq = ops.latent_prepare(down, self.q_rank, rank, dr, self.q_norm, self.kv_norm, self.eps, inv_freq, factor,
                                batch.positions, batch.seq_index,
                                block_table=cache.block_table if cache.writes else None,
                                cache=latent if cache.writes else None)
        q = self.uq.forward(cq).view(-1, H, dn + dr)
        rows = torch.empty((q.shape[0], H, rank + dr), dtype=q.dtype, device=q.device)
        ops.headwise_linear(q[:, :, :dn], self.uk, out=rows[:, :, :rank])
        if dr:
            ops.rotate_heads(q[:, :, dn:], rows[:, :, rank:], inv_freq, factor, batch.positions)
        at = self.q_rank + rank + dr
        mixed = ops.latent_attention(rows, latent, rank, cache.block_table, batch.cu_seqlens_q, batch.kv_lens,
                                     batch.max_q_len, self.scale, window=self.window, max_kv_len=batch.max_kv_len,
                                     sink=self.sink, gate=down[:, at:at + H] if self.gated else None)
        o = ops.headwise_linear(mixed, self.uv)
        return self.out.forward(o.view(-1, H * self.vdim))
