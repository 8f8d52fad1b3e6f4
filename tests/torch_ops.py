"""Plain PyTorch twins of the HIP operations, with the same signatures.

They serve two purposes: each GPU kernel test compares a kernel with its twin
here, at float32; and the tests that have no GPU substitute these functions for
the package's operations (see conftest.py, fixture `cpu_ops`) so that the cache,
the step function and the scheduler can be exercised on the CPU. They are not
part of the product, which has no host implementation.
"""

import math

import torch


def embed_rows(ids, table, out=None, scale=1.0):
    res = table[ids.long()].float() * scale
    if out is not None:
        out.copy_(res)
        return out
    return res


GATE_KINDS = {"silu": 0, "gelu_tanh": 1, "gelu_erf": 2}


def gated_act(gate_up, kind="silu", out=None):
    g = gate_up[:, 0::2].float()          # gate and up interleaved
    u = gate_up[:, 1::2].float()
    if kind == "silu":
        a = g / (1.0 + torch.exp(-g))
    elif kind == "gelu_tanh":
        a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g ** 3)))
    else:
        a = 0.5 * g * (1.0 + torch.erf(g / math.sqrt(2.0)))
    res = (a * u).to(gate_up.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def swiglu(gate_up, out=None):
    return gated_act(gate_up, "silu", out=out)


def layernorm_addend(x, weight, bias, eps, out_dtype, delta=None, extra=None, vec=None, rows=None, write_back=True):
    src = x if rows is None else x[rows.long()]
    if delta is not None:
        src = src + (delta if rows is None else delta[rows.long()]).float()
    if extra is not None:
        src = src + (extra if rows is None else extra[rows.long()])
    if vec is not None:
        src = src + vec
    if write_back and rows is None and (delta is not None or extra is not None or vec is not None):
        x.copy_(src)
    if weight is None:
        return None
    dev = src - src.mean(dim=-1, keepdim=True)
    res = dev * torch.rsqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * weight
    if bias is not None:
        res = res + bias
    return res.to(out_dtype)


def rmsnorm(x, weight, eps, out_dtype, delta=None, rows=None, write_back=True, out=None):
    src = x if rows is None else x[rows.long()]
    if delta is not None:
        d = delta if rows is None else delta[rows.long()]
        src = src + d.float()
        if write_back and rows is None:
            x.copy_(src)
    ms = (src * src).mean(dim=-1, keepdim=True)
    res = (src * torch.rsqrt(ms + eps) * weight.float()).to(out_dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def rope_table(inv_freq, max_positions):
    p = torch.arange(max_positions, dtype=torch.float32, device=inv_freq.device)
    ang = p[:, None] * inv_freq[None, :]
    return torch.cat((ang.cos(), ang.sin()), dim=-1)


def qk_norm_rope_store(qkv, num_q_heads, num_kv_heads, head_dim, positions, seq_index,
                       q_weight=None, k_weight=None, eps=0.0, table=None,
                       block_table=None, k_cache=None, v_cache=None,
                       cu_seqlens_q=None, kv_lens=None, max_q_len=0, max_kv_len=0):
    Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
    T = qkv.shape[0]
    if table is not None and max_kv_len > table.shape[0]:
        raise ValueError("the step reaches position %d, the rotation table ends at %d"
                         % (max_kv_len - 1, table.shape[0] - 1))
    x = qkv.view(T, Hq + 2 * Hkv, D).float()
    q, k, v = x[:, :Hq], x[:, Hq:Hq + Hkv], x[:, Hq + Hkv:]

    def norm(t, w):
        if w is None:
            return t
        ms = (t * t).mean(dim=-1, keepdim=True)
        return t * torch.rsqrt(ms + eps) * w.float()

    def rotate(t):
        if table is None:
            return t
        R = table.shape[1]
        half = R // 2
        cs = table[positions.long()]
        cos, sin = cs[:, None, :half], cs[:, None, half:]
        a, b = t[..., :half], t[..., half:R]
        return torch.cat((a * cos - b * sin, b * cos + a * sin, t[..., R:]), dim=-1)

    q = rotate(norm(q, q_weight))
    k = rotate(norm(k, k_weight))
    qkv.view(T, Hq + 2 * Hkv, D)[:, :Hq] = q.to(qkv.dtype)
    if k_cache is not None:
        page = k_cache.shape[2]
        pos = positions.long()
        pages = block_table[seq_index.long(), pos // page].long()
        ok = pages >= 0
        k_cache[pages[ok], :, (pos % page)[ok]] = k[ok].to(k_cache.dtype)
        v_cache[pages[ok], :, :, (pos % page)[ok]] = v[ok].to(v_cache.dtype)     # values: (pages, Hkv, D, page)
    return qkv


def paged_attention(q, num_q_heads, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens,
                    max_q_len, max_kv_len, scale, window=0, out=None, min_q_len=1, max_kv_len_of_many=None):
    T, Hq, D = q.shape
    Hkv, page = k_cache.shape[1], k_cache.shape[2]
    G = Hq // Hkv
    res = torch.zeros((T, Hq * D), dtype=torch.float32, device=q.device)
    cu = cu_seqlens_q.tolist()
    kvl = kv_lens.tolist()
    for b in range(len(kvl)):
        q0, q1 = cu[b], cu[b + 1]
        n, L = q1 - q0, kvl[b]
        if n == 0:
            continue
        nblk = -(-L // page)
        pages = block_table[b, :nblk].long().clamp(min=0)
        K = k_cache[pages].float().permute(1, 0, 2, 3).reshape(Hkv, nblk * page, D)[:, :L]
        V = v_cache[pages].float().permute(1, 0, 3, 2).reshape(Hkv, nblk * page, D)[:, :L]
        qpos = torch.arange(L - n, L, device=q.device)[:, None]
        kpos = torch.arange(L, device=q.device)[None, :]
        hidden = kpos > qpos
        if window > 0:
            hidden = hidden | (qpos - kpos >= window)
        qq = q[q0:q1].float()
        for h in range(Hq):
            s = (qq[:, h] @ K[h // G].T) * scale
            s = s.masked_fill(hidden, float("-inf"))
            p = torch.softmax(s, dim=-1)
            res[q0:q1, h * D:(h + 1) * D] = p @ V[h // G]
    res = res.to(q.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def decode_attention_takes(*args, **kwargs):
    return False            # the fused decoding kernel has no twin: its two halves above are the reference


def tile_weight(weight):
    return None


def linear(x, weight, out_dtype=None, out=None, tiled=None):
    res = (x.float() @ weight.float().T).to(out_dtype or x.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def linear_swiglu(x, weight, tiled=None):
    return swiglu(linear(x, weight))


def _uniform(seed, counter, n, device):
    # any fixed stream will do for the stand-in; the kernel's generator is tested on the GPU
    g = torch.Generator(device="cpu")
    g.manual_seed((int(seed) * 1000003 + int(counter)) & 0x7FFFFFFFFFFFFFFF)
    return torch.rand(n, generator=g).to(device)


def sample(logits, temperature, top_k, seed, counter, out=None, any_top_k=True):
    R, V = logits.shape
    res = torch.empty(R, dtype=torch.int32, device=logits.device)
    for r in range(R):
        row = logits[r]
        t = float(temperature[r])
        if t <= 0:
            res[r] = int(torch.argmax(row))
            continue
        z = row / t
        k = int(top_k[r])
        if 0 < k < V:
            kth = torch.topk(row, k).values[-1]
            z = z.masked_fill(row < kth, float("-inf"))
        u = _uniform(seed[r], counter[r], V, logits.device).clamp(1e-12, 1 - 1e-7)
        res[r] = int(torch.argmax(z - torch.log(-torch.log(u))))
    if out is not None:
        out.copy_(res)
        return out
    return res


def rmsnorm_addend(x, weight, eps, out_dtype, delta=None, delta_weight=None, delta_eps=0.0, bias=None, rows=None,
                   write_back=True, out=None, delta_bias=None, plain=False):
    src = x if rows is None else x[rows.long()]
    if delta is not None:
        d = (delta if rows is None else delta[rows.long()]).float()
        if delta_bias is not None:
            d = d + delta_bias
        if delta_weight is not None:
            d = d * torch.rsqrt((d * d).mean(dim=-1, keepdim=True) + delta_eps) * delta_weight.float()
        src = src + d
    if bias is not None:
        src = src + bias
    if write_back and rows is None and (delta is not None or bias is not None):
        x.copy_(src)
    if weight is None and not plain:
        return None
    if plain:
        res = src.to(out_dtype)
    else:
        res = (src * torch.rsqrt((src * src).mean(dim=-1, keepdim=True) + eps) * weight.float()).to(out_dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def glu_clamped(gate_up, limit, slope, bias=None, scale=None, scale_index=None, out_dtype=None):
    a = gate_up.float()
    if scale is not None:
        w = scale[scale_index.long()] if scale_index is not None else scale
        a = a * w[:, None]
    if bias is not None:
        a = a + bias
    g = torch.clamp(a[:, 0::2], max=limit)
    u = torch.clamp(a[:, 1::2], min=-limit, max=limit)
    return (g * torch.sigmoid(slope * g) * (u + 1.0)).to(out_dtype or gate_up.dtype)


GELU_KINDS = {"erf": 0, "tanh": 1}


def gelu(x, kind="erf", out=None):
    z = x.float()
    if kind == "erf":
        res = 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))
    else:
        res = 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
    res = res.to(x.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def _turn_pairs(t, positions, inv_freq, rot_factor):
    """t (T, ..., n): pairs (2i, 2i + 1), i < len(inv_freq), turned by float32(position) * inv_freq[i]."""
    n2 = 2 * inv_freq.shape[0]
    angle = positions.float()[:, None] * inv_freq[None, :]
    shape = (t.shape[0],) + (1,) * (t.dim() - 2) + (inv_freq.shape[0],)
    cos, sin = (angle.cos() * rot_factor).view(shape), (angle.sin() * rot_factor).view(shape)
    u, v = t[..., 0:n2:2], t[..., 1:n2:2]
    turned = torch.stack((u * cos - v * sin, v * cos + u * sin), dim=-1).flatten(-2)
    return torch.cat((turned, t[..., n2:]), dim=-1)


def latent_prepare(down, q_rank, kv_rank, rot_dim, q_weight, kv_weight, eps, inv_freq, rot_factor, positions, seq_index,
                   block_table=None, cache=None):
    x = down.float()
    a, b, tail = x[:, :q_rank], x[:, q_rank:q_rank + kv_rank], x[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim]
    cq = a * torch.rsqrt((a * a).mean(dim=-1, keepdim=True) + eps) * q_weight.float()
    if cache is not None:
        c = b * torch.rsqrt((b * b).mean(dim=-1, keepdim=True) + eps) * kv_weight.float()
        row = torch.cat((c, _turn_pairs(tail, positions, inv_freq, rot_factor)), dim=-1) if inv_freq is not None \
            else torch.cat((c, tail), dim=-1)
        page = cache.shape[1]
        pos = positions.long()
        pages = block_table[seq_index.long(), pos // page].long()
        ok = pages >= 0
        cache[pages[ok], (pos % page)[ok]] = row[ok].to(cache.dtype)
    return cq.to(down.dtype)


def headwise_linear(x, weight, out=None):
    res = torch.einsum("thi,hoi->tho", x.float(), weight.float()).to(x.dtype).contiguous()
    if out is not None:
        out.copy_(res)
        return out
    return res


def rotate_heads(x, out, inv_freq, rot_factor, positions):
    out.copy_(_turn_pairs(x.float(), positions, inv_freq, rot_factor).to(x.dtype))
    return out


def latent_attention(q, cache, value_dim, block_table, cu_seqlens_q, kv_lens, max_q_len, scale, window=0, general=False,
                     max_kv_len=0, sink=None, gate=None):
    T, H, Dk = q.shape
    page = cache.shape[1]
    res = torch.zeros((T, H, value_dim), dtype=torch.float32, device=q.device)
    cu, kvl = cu_seqlens_q.tolist(), kv_lens.tolist()
    for b in range(len(kvl)):
        q0, q1 = cu[b], cu[b + 1]
        n, L = q1 - q0, kvl[b]
        if n == 0:
            continue
        nblk = -(-L // page)
        pages = block_table[b, :nblk].long().clamp(min=0)
        rows = cache[pages].float().reshape(nblk * page, Dk)[:L]
        qpos = torch.arange(L - n, L, device=q.device)[:, None]
        kpos = torch.arange(L, device=q.device)[None, :]
        hidden = kpos > qpos
        if window > 0:
            hidden = hidden | (qpos - kpos >= window)
        s = torch.einsum("thd,sd->hts", q[q0:q1].float(), rows) * scale
        s = s.masked_fill(hidden[None], float("-inf"))
        if sink is not None:
            s = torch.cat((s, sink.float()[:, None, None].expand(H, n, 1)), dim=-1)
        p = torch.softmax(s, dim=-1)[..., :L]
        res[q0:q1] = torch.einsum("hts,sd->thd", p, rows[:, :value_dim])
    if gate is not None:
        res = res * torch.sigmoid(gate.float())[:, :, None]
    return res.to(q.dtype)


def moe_route(h, router, top, tiled=None, scoring="softmax", correction=None, groups=1, keep=1, experts=None):
    z = h.float() @ router.float().T
    if experts is not None:
        chosen, weights = moe_route(h, router[:experts], top, scoring=scoring, correction=correction, groups=groups, keep=keep)
        return chosen, weights, z[:, experts:]
    if scoring == "sigmoid_groups":
        T, E = z.shape
        score = torch.sigmoid(z)
        choice = score + correction
        if keep < groups:
            size = E // groups
            grouped = choice.view(T, groups, size)
            of_group = grouped.topk(min(2, size), dim=-1).values.sum(dim=-1)
            kept = torch.zeros((T, groups), dtype=torch.bool)
            kept[torch.arange(T)[:, None], of_group.topk(keep, dim=-1).indices] = True
            choice = grouped.masked_fill(~kept[:, :, None], float("-inf")).reshape(T, E)
        chosen = choice.topk(top, dim=-1).indices
        return chosen.to(torch.int32), score.gather(1, chosen)
    if scoring == "sigmoid":
        best, chosen = torch.topk(z, top, dim=-1)
        return chosen.to(torch.int32), torch.sigmoid(best)
    s = torch.softmax(z, dim=-1)
    best, chosen = torch.topk(s, top, dim=-1)
    return chosen.to(torch.int32), best / (best.sum(dim=-1, keepdim=True) + 1e-20)


def moe_gated_experts(h, chosen, weights, gate_up, down, limit, slope):
    T, top = chosen.shape
    out = torch.zeros((T, h.shape[1]), dtype=torch.float32, device=h.device)
    for k in range(top):
        e = chosen[:, k].long()
        both = torch.einsum("ti,tfi->tf", h.float(), gate_up[e].float()).to(h.dtype)
        hidden = glu_clamped(both, limit, slope, scale=weights[:, k].contiguous())
        out += torch.einsum("tf,twf->tw", hidden.float(), down[e].float()).to(h.dtype).float()
    return out.to(h.dtype)


def moe_glu_experts(h, chosen, weights, gate_up, down, activation="silu", shared=None, shared_gate=None):
    T, top = chosen.shape
    out = torch.zeros((T, h.shape[1]), dtype=torch.float32, device=h.device)
    for k in range(top):
        e = chosen[:, k].long()
        both = torch.einsum("ti,tfi->tf", h.float(), gate_up[e].float())       # the gated unit sees unrounded sums
        y = torch.einsum("tf,twf->tw", gated_act(both, activation).to(h.dtype).float(), down[e].float()).to(h.dtype)
        out += weights[:, k, None] * y.float()
    if shared is not None:
        out += shared.float() * (torch.sigmoid(shared_gate.reshape(T, 1)) if shared_gate is not None else 1.0)
    return out.to(h.dtype)


def moe_experts(h, chosen, weights, up, down, shared=None, activation="erf"):
    T, top = chosen.shape
    out = torch.zeros((T, h.shape[1]), dtype=torch.float32, device=h.device)
    for k in range(top):
        e = chosen[:, k].long()
        hidden = gelu(torch.einsum("ti,tfi->tf", h.float(), up[e].float()).to(h.dtype), activation)
        y = torch.einsum("tf,twf->tw", hidden.float(), down[e].float()).to(h.dtype)
        out += weights[:, k, None] * y.float()
    if shared is not None:
        out += shared.float()
    return out.to(h.dtype)


# ---- the recurrent mixers, the residual in several streams, attention with capped scores ----

def embed_streams(ids, table, copies):
    return table[ids.long()].float()[:, None, :].repeat(1, copies, 1).contiguous()


def hyper_norm(x, weight, eps, out_dtype, read=None, delta=None, mix=None, write=None, rows=None, write_back=True):
    src = x if rows is None else x[rows.long()]
    if delta is not None:
        d = (delta if rows is None else delta[rows.long()]).float()
        src = torch.einsum("st,nsw->ntw", mix.float(), src) + write.float()[None, :, None] * d[:, None, :]
        if write_back and rows is None:
            x.copy_(src)
    u = src.sum(dim=1) if read is None else torch.einsum("s,nsw->nw", read.float(), src)
    if weight is None:
        return None
    dev = u - u.mean(dim=-1, keepdim=True)
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return (dev * torch.rsqrt(var + eps) * weight.float()).to(out_dtype)


def _sequences(cu_seqlens_q, slots):
    cu = cu_seqlens_q.tolist()
    return [(cu[b], cu[b + 1], int(slot)) for b, slot in enumerate(slots.tolist())]


def causal_conv(x, weight, bias, state, slots, cu_seqlens_q, seq_index, activation=None, out_dtype=None, in_bias=None,
                max_q_len=0):
    T, C = x.shape
    taps = weight.shape[1]
    out = torch.empty((T, C), dtype=torch.float32, device=x.device)
    for first, last, slot in _sequences(cu_seqlens_q, slots):
        if last == first:
            continue
        rows = x[first:last].float()
        if in_bias is not None:
            rows = rows + in_bias.float()
        seen = torch.cat((state[slot].view(taps - 1, C), rows), dim=0)
        acc = bias.float().expand(last - first, C).clone()
        for j in range(taps):
            acc += weight[:, taps - 1 - j].float() * seen[taps - 1 - j: taps - 1 - j + last - first]
        out[first:last] = acc
        state[slot] = seen[seen.shape[0] - (taps - 1):].reshape(-1)
    if activation == "silu":
        out = out * torch.sigmoid(out)
    return out.to(out_dtype or x.dtype)


def mamba2_scan(xbc, dt, dt_bias, a_log, d_skip, state, slots, cu_seqlens_q, heads, vdim, n_state, groups, max_q_len=1):
    T = xbc.shape[0]
    inner, gn = heads * vdim, groups * n_state
    x = xbc[:, :inner].float().view(T, heads, vdim)
    B = xbc[:, inner:inner + gn].float().view(T, groups, n_state).repeat_interleave(heads // groups, dim=1)
    C = xbc[:, inner + gn:].float().view(T, groups, n_state).repeat_interleave(heads // groups, dim=1)
    step = torch.nn.functional.softplus(dt.float() + dt_bias.float())
    decay = torch.exp(-torch.exp(a_log.float()) * step)
    y = torch.empty((T, heads, vdim), dtype=torch.float32, device=xbc.device)
    for first, last, slot in _sequences(cu_seqlens_q, slots):
        S = state[slot].view(heads, n_state, vdim).clone()
        for t in range(first, last):
            S = decay[t][:, None, None] * S + step[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
            y[t] = torch.einsum("hnp,hn->hp", S, C[t]) + d_skip.float()[:, None] * x[t]
        state[slot] = S.reshape(-1)
    return y.view(T, inner)


def gated_rmsnorm(y, gate, weight, groups, eps, out_dtype):
    T, inner = y.shape
    g = gate.float()
    v = (y.float() * g * torch.sigmoid(g)).view(T, groups, inner // groups)
    v = v * torch.rsqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return (v.view(T, inner) * weight.float()).to(out_dtype)


def block_gates(u, weights, biases):
    T, width = u.shape
    blocks = weights.shape[1]
    ub = u.float().view(T, blocks, width // blocks)
    z = torch.einsum("tbi,gbio->gtbo", ub, weights.float()) + biases.float()[:, None]
    return torch.sigmoid(z).reshape(2, T, width)


def rglru_scan(u, gates, rate, y, y_bias, state, slots, cu_seqlens_q, out_dtype, max_q_len=1):
    T, width = u.shape
    a = torch.exp(-rate.float() * gates[0])
    push = torch.sqrt(1.0 - a * a) * gates[1] * u.float()
    z = y.float() + y_bias.float()
    branch = 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
    out = torch.empty((T, width), dtype=torch.float32, device=u.device)
    for first, last, slot in _sequences(cu_seqlens_q, slots):
        S = state[slot].clone()
        for t in range(first, last):
            S = a[t] * S + push[t]
            out[t] = S * branch[t]
        state[slot] = S
    return out.to(out_dtype)


def _turn(v, positions, inv_freq, neighbours):
    """v (T, heads, dim): the first 2 * len(inv_freq) numbers of each head turn by position * frequency,
    pairs (2i, 2i + 1) or (i, i + half)."""
    if inv_freq is None:
        return v
    half = inv_freq.shape[0]
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    out = v.clone()
    if neighbours:
        a, b = v[..., 0:2 * half:2], v[..., 1:2 * half:2]
        out[..., 0:2 * half:2] = a * c - b * s
        out[..., 1:2 * half:2] = b * c + a * s
    else:
        a, b = v[..., :half], v[..., half:2 * half]
        out[..., :half] = a * c - b * s
        out[..., half:2 * half] = b * c + a * s
    return out


def retention_scan(qkvg, heads, dim, vdim, inv_freq, positions, decay, k_scale, eps, state, slots, cu_seqlens_q, out_dtype,
                   max_q_len=1, log_decay=None):
    T = qkvg.shape[0]
    hd, hv = heads * dim, heads * vdim
    rows = qkvg.float()
    q = _turn(rows[:, :hd].view(T, heads, dim), positions, inv_freq, False)
    k = _turn(rows[:, hd:2 * hd].view(T, heads, dim), positions, inv_freq, False) * k_scale
    v = rows[:, 2 * hd:2 * hd + hv].view(T, heads, vdim)
    g = rows[:, 2 * hd + hv:]
    o = torch.empty((T, heads, vdim), dtype=torch.float32, device=qkvg.device)
    for first, last, slot in _sequences(cu_seqlens_q, slots):
        S = state[slot].view(heads, dim, vdim).clone()
        for t in range(first, last):
            S = decay.float()[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S.reshape(-1)
    o = o * torch.rsqrt((o * o).mean(dim=-1, keepdim=True) + eps)
    return (o.reshape(T, hv) * g * torch.sigmoid(g)).to(out_dtype)


def softcap_prepare(rows, bias, heads, kv_heads, dim, vdim, q_weight, k_weight, eps, inv_freq, positions, seq_index,
                    out_dtype, block_table=None, k_cache=None, v_cache=None, values_transposed=False):
    T = rows.shape[0]
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    z = rows[:, :nq + nk + nv].float()
    if bias is not None:
        z = z + bias.float()
    q, k, v = z[:, :nq], z[:, nq:nq + nk], z[:, nq + nk:]
    q = q * torch.rsqrt((q * q).mean(dim=-1, keepdim=True) + eps) * q_weight.float()
    k = k * torch.rsqrt((k * k).mean(dim=-1, keepdim=True) + eps) * k_weight.float()
    q = _turn(q.view(T, heads, dim), positions, inv_freq, True)
    k = _turn(k.view(T, kv_heads, dim), positions, inv_freq, True)
    if k_cache is not None:
        page = k_cache.shape[2]
        pos = positions.long()
        pages = block_table[seq_index.long(), pos // page].long()
        k_cache[pages, :, pos % page] = k.to(k_cache.dtype)
        if values_transposed:
            v_cache[pages, :, :, pos % page] = v.reshape(T, kv_heads, vdim).to(v_cache.dtype)
        else:
            v_cache[pages, :, pos % page] = v.reshape(T, kv_heads, vdim).to(v_cache.dtype)
    return q.to(out_dtype).contiguous()


def headnorm_prepare(rows, heads, kv_heads, dim, vdim, q_weight, k_weight, eps, positions, seq_index, out_dtype,
                     block_table=None, k_cache=None, v_cache=None, values_transposed=False):
    T = rows.shape[0]
    nq, nk = heads * dim, kv_heads * dim
    q = rows[:, :nq].float().view(T, heads, dim)
    q = q * torch.rsqrt((q * q).mean(dim=-1, keepdim=True) + eps) * q_weight.float()
    if kv_heads:
        k = rows[:, nq:nq + nk].float().view(T, kv_heads, dim)
        k = k * torch.rsqrt((k * k).mean(dim=-1, keepdim=True) + eps) * k_weight.float()
        v = rows[:, nq + nk:nq + nk + kv_heads * vdim].float().reshape(T, kv_heads, vdim)
        page = k_cache.shape[2]
        pos = positions.long()
        pages = block_table[seq_index.long(), pos // page].long()
        k_cache[pages, :, pos % page] = k.to(k_cache.dtype)
        if values_transposed:
            v_cache[pages, :, :, pos % page] = v.to(v_cache.dtype)
        else:
            v_cache[pages, :, pos % page] = v.to(v_cache.dtype)
    return q.to(out_dtype).contiguous()


def channel_delta(conv, b_logits, a_logits, gate, dt_bias, a_log, norm_weight, eps, unit_eps, state, slots, cu_seqlens_q,
                  heads, kv_heads, dim, vdim, out_dtype):
    T = conv.shape[0]
    H, G, d, dv = heads, kv_heads, dim, vdim
    q = conv[:, :G * d].view(T, G, d)
    k = conv[:, G * d:2 * G * d].view(T, G, d)
    v = conv[:, 2 * G * d:].view(T, H, dv)
    q = q * torch.rsqrt((q * q).sum(dim=-1, keepdim=True) + unit_eps) * d ** -0.5
    k = k * torch.rsqrt((k * k).sum(dim=-1, keepdim=True) + unit_eps)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(b_logits)
    decay = torch.exp(-torch.exp(a_log)[None, :, None] * torch.nn.functional.softplus((a_logits + dt_bias).view(T, H, d)))
    o = torch.empty((T, H, dv), dtype=torch.float32, device=conv.device)
    for first, last, slot in _sequences(cu_seqlens_q, slots):
        S = state[slot].view(H, dv, d).transpose(1, 2).clone()       # kept (head, column, row)
        for t in range(first, last):
            S = decay[t][:, :, None] * S
            u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
            S = S + k[t][:, :, None] * u[:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S.transpose(1, 2).reshape(-1)
    o = o * torch.rsqrt((o * o).mean(dim=-1, keepdim=True) + eps) * norm_weight * torch.sigmoid(gate.view(T, H, dv))
    return o.reshape(T, H * dv).to(out_dtype)


def softcap_attention(q, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens, seq_index, positions, max_q_len,
                      max_kv_len, scale, softcap, window=0, gate=None, values_transposed=False, min_q_len=1,
                      max_kv_len_of_many=None, sink=None):
    T, H, dim = q.shape
    if values_transposed:
        v_cache = v_cache.transpose(2, 3)
    G, page, vdim = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    res = torch.zeros((T, H, vdim), dtype=torch.float32, device=q.device)
    cu, kvl = cu_seqlens_q.tolist(), kv_lens.tolist()
    for b in range(len(kvl)):
        q0, q1, L = cu[b], cu[b + 1], kvl[b]
        n = q1 - q0
        if n == 0:
            continue
        blocks = -(-L // page)
        pages = block_table[b, :blocks].long().clamp(min=0)
        K = k_cache[pages].float().permute(1, 0, 2, 3).reshape(G, blocks * page, dim)[:, :L]
        V = v_cache[pages].float().permute(1, 0, 2, 3).reshape(G, blocks * page, vdim)[:, :L]
        qpos = torch.arange(L - n, L, device=q.device)[:, None]
        kpos = torch.arange(L, device=q.device)[None, :]
        hidden = kpos > qpos
        if window > 0:
            hidden = hidden | (qpos - kpos >= window)
        for h in range(H):
            s = (q[q0:q1, h].float() @ K[h // (H // G)].T) * scale
            if softcap > 0:
                s = softcap * torch.tanh(s / softcap)
            s = s.masked_fill(hidden, float("-inf"))
            if sink is not None:
                s = torch.cat((s, sink[h].float().expand(n, 1)), dim=-1)
                res[q0:q1, h] = torch.softmax(s, dim=-1)[:, :-1] @ V[h // (H // G)]
            else:
                res[q0:q1, h] = torch.softmax(s, dim=-1) @ V[h // (H // G)]
    if gate is not None:
        res = res * torch.sigmoid(gate.float())[:, :, None]
    return res.reshape(T, H * vdim).to(q.dtype)


def scaled_sum(a, alpha, b, beta):
    return (alpha * a.float() + beta * b.float()).to(a.dtype)


ALL = ("gated_act", "GATE_KINDS", "layernorm_addend", "moe_glu_experts", "glu_clamped", "moe_gated_experts", "headnorm_prepare", "channel_delta", "embed_rows", "swiglu", "rmsnorm", "rope_table", "qk_norm_rope_store",
       "paged_attention", "decode_attention_takes", "linear", "linear_swiglu", "tile_weight", "sample",
       "rmsnorm_addend", "gelu", "GELU_KINDS", "latent_prepare", "headwise_linear", "rotate_heads", "latent_attention",
       "moe_route", "moe_experts", "embed_streams", "hyper_norm", "causal_conv", "mamba2_scan", "gated_rmsnorm",
       "block_gates", "rglru_scan", "retention_scan", "softcap_prepare", "softcap_attention", "scaled_sum")
