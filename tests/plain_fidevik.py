"""The Fidevik decoder on one whole sequence with elementary tensor operations, one function per
mechanism, in the dtype of the weights it is given (float64 for a truth, float32 to see what
rounding does). It shares no code with the package: the tests compare the engine with this.

`config` is config.json as a dict, `w` maps tensor names to tensors.
"""

import math

import torch


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def layer_norm(x, weight, bias, eps):
    """Mean out, divided by the root of the mean squared deviation (eps inside), weight and bias."""
    centred = x - x.mean(dim=-1, keepdim=True)
    return centred / torch.sqrt((centred * centred).mean(dim=-1, keepdim=True) + eps) * weight + bias


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_pairs(x, positions, rot):
    """x (T, heads, n): the first rot.dims numbers of every head turn, (2i, 2i + 1) together, by
    position * base^(-2i / dims); the rest pass."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64).to(torch.float32)
    angle = positions.to(torch.float32)[:, None] * f[None, :]          # 32-bit angles, as the design forms them
    cos = angle.to(torch.float64).cos().to(x.dtype)[:, None, :]
    sin = angle.to(torch.float64).sin().to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack((u * cos - v * sin, v * cos + u * sin), dim=-1).flatten(-2)
    return torch.cat((turned, x[..., dims:]), dim=-1)


def causal_softmax(scores, sink=None):
    """scores (heads, T, T) -> weights; position i sees j <= i. With `sink` (heads,) the
    denominator of head a also holds exp(sink_a), which belongs to no key."""
    T = scores.shape[-1]
    hidden = torch.arange(T)[None, :] > torch.arange(T)[:, None]
    scores = scores.masked_fill(hidden[None], float("-inf"))
    if sink is None:
        return torch.softmax(scores, dim=-1)
    column = sink.to(scores.dtype)[:, None, None].expand(-1, T, 1)
    return torch.softmax(torch.cat((scores, column), dim=-1), dim=-1)[..., :T]


def attention(h, w, p, m, eps):
    """Grouped heads; q and k are each normalised over the whole projection (all heads at once),
    then turned by the position; plain causal softmax."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = rms_norm(h @ w[p + ".q"].T, w[p + ".q.norm"], eps).view(T, H, d)
    k = rms_norm(h @ w[p + ".k"].T, w[p + ".k.norm"], eps).view(T, G, d)
    v = (h @ w[p + ".v"].T).view(T, G, dv)
    if m.get("rot"):
        q, k = rotate_pairs(q, pos, m["rot"]), rotate_pairs(k, pos, m["rot"])
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) * float(m["scale"])
    o = torch.einsum("hts,shd->thd", causal_softmax(scores), v)
    return o.reshape(T, H * dv) @ w[p + ".o"].T


def latent_attention(h, w, p, m, eps):
    """Queries through a normalised narrow vector; keys and values per head from one normalised
    narrow vector per token; no positions; a sink in the softmax; a gate per head from the
    mixer's input."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    cq = rms_norm(h @ w[p + ".dq"].T, w[p + ".dq.norm"], eps)
    q = (cq @ w[p + ".uq"].T).view(T, H, d)
    c = rms_norm(h @ w[p + ".dkv"].T, w[p + ".dkv.norm"], eps)
    k = (c @ w[p + ".uk"].T).view(T, H, d)
    v = (c @ w[p + ".uv"].T).view(T, H, dv)
    scores = torch.einsum("thd,shd->hts", q, k) * float(m["scale"])
    o = torch.einsum("hts,shd->thd", causal_softmax(scores, w[p + ".sink"]), v)
    o = o * torch.sigmoid(h @ w[p + ".g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w[p + ".o"].T


def gated_unit(h, w, p, act):
    return (act(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def choose_experts(z, correction, top, groups, keep):
    """z (T, E) router logits -> (chosen (T, top), their weights). The choice goes by
    sigmoid(z) + correction among the experts of the `keep` groups whose two largest such
    scores sum highest; the weights are sigmoid(z) of the chosen, as they are."""
    T, E = z.shape
    s = torch.sigmoid(z)
    choice = s + correction
    size = E // groups
    grouped = choice.view(T, groups, size)
    group_score = grouped.topk(min(2, size), dim=-1).values.sum(dim=-1)
    kept = group_score.topk(keep, dim=-1).indices
    allowed = torch.zeros((T, groups), dtype=torch.bool)
    allowed[torch.arange(T)[:, None], kept] = True
    choice = grouped.masked_fill(~allowed[:, :, None], float("-inf")).view(T, E)
    chosen = choice.topk(top, dim=-1).indices
    return chosen, s.gather(1, chosen)


def routed_feed_forward(h, w, p, f):
    E, top = int(f["router"]["experts"]), int(f["router"]["top"])
    groups = f["router"].get("groups") or {"count": 1, "keep": 1}
    z = h @ w[p + ".router"].T
    chosen, share = choose_experts(z, w[p + ".correction"], top, int(groups["count"]), int(groups["keep"]))
    out = torch.zeros_like(h)
    for e in range(E):
        for k in range(top):
            rows = (chosen[:, k] == e).nonzero()[:, 0]
            if rows.numel():
                out[rows] += share[rows, k, None] * gated_unit(h[rows], w, "%s.e%d" % (p, e), silu)
    if f.get("shared"):
        out = out + torch.sigmoid(h @ w[p + ".shared.sg"].T) * gated_unit(h, w, p + ".shared", silu)
    return out


def run_order(config):
    """[(layer, number of the pass that starts here or None)]"""
    n = len(config["layers"])
    loop = config.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    if b <= a:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def logits_of_sequence(config, w, tokens, layers_out=None):
    eps = float(config["norm"]["eps"])
    embedded = w["embed"][torch.tensor(tokens)]
    x = embedded
    for i, enters in run_order(config):
        layer, p = config["layers"][i], "l%d" % i
        if enters is not None:
            if enters > 0:
                x = x + embedded
            x = x + w["loop.step"][enters]
        h = layer_norm(x, w[p + ".norm1"], w[p + ".norm1.b"], eps)
        if layer["type"] == "attention":
            x = x + attention(h, w, p + ".mix", layer["mixer"], eps)
        else:
            assert layer["type"] == "latent_attention"
            x = x + latent_attention(h, w, p + ".mix", layer["mixer"], eps)
        if layer.get("mlp"):
            h = layer_norm(x, w[p + ".norm2"], w[p + ".norm2.b"], eps)
            if layer["mlp"]["kind"] == "dense":
                x = x + gated_unit(h, w, p + ".mlp", gelu_tanh)
            else:
                assert layer["mlp"]["kind"] == "moe"
                x = x + routed_feed_forward(h, w, p + ".mlp", layer["mlp"])
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return (x @ w["head"].T) * float(config.get("logit_scale", 1.0))
