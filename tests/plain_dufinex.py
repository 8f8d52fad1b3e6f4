"""A plain, slow implementation of the Dufinex decoder, one function per mechanism, in float64 and
token by token wherever a recurrence is involved. It takes a config.json's dict and a dict of
tensors (name -> torch tensor) and shares no code with the engine: it is what the engine's
results are compared with.

Notation: h is a sublayer's input (tokens, width); `w` is the tensor dict; `p` a tensor name prefix
ending in "."; positions count from 0.
"""

import math

import torch

F = torch.float64


def _t(w, name):
    return w[name].to(F)


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def clamped_glu(gate, up, limit):
    """g = min(gate, limit), u = clamp(up, -limit, limit); g sigmoid(1.702 g) (u + 1)."""
    g = torch.clamp(gate, max=limit)
    u = torch.clamp(up, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def short_conv(x, taps):
    """out[t, c] = sum_j taps[c, K - 1 - j] x[t - j, c]; what lies before the first token is zero."""
    T, C = x.shape
    K = taps.shape[1]
    out = torch.zeros(T, C, dtype=F)
    for t in range(T):
        for j in range(K):
            if t - j >= 0:
                out[t] += taps[:, K - 1 - j] * x[t - j]
    return out


def keys_and_values(h, w, p, m, eps):
    """What an attention layer with projections of its own keeps: keys after their norm, values."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = rms_norm((h @ _t(w, p + "k").T).reshape(T, G, d), _t(w, p + "k.norm"), eps)
    v = (h @ _t(w, p + "v").T).reshape(T, G, dv)
    return k, v


def sink_attention(h, w, p, m, eps, k, v):
    """Causal softmax attention whose denominator also holds exp(sink) per head, with a gate per
    head on the result. k (T, G, dim) and v (T, G, vdim) are this layer's or another layer's."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ _t(w, p + "q").T).reshape(T, H, d), _t(w, p + "q.norm"), eps)
    gate = torch.sigmoid(h @ _t(w, p + "g").T)           # (T, H)
    sink = _t(w, p + "sink")
    out = torch.zeros(T, H, dv, dtype=F)
    hidden = torch.triu(torch.ones(T, T, dtype=torch.bool), diagonal=1)      # key j > query i
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(hidden, float("-inf"))
        top = torch.maximum(s.max(dim=-1).values, sink[a])
        e = torch.exp(s - top[:, None])
        out[:, a] = (e @ v[:, g]) / (e.sum(dim=-1) + torch.exp(sink[a] - top))[:, None]
    out = out * gate[:, :, None]
    return out.reshape(T, H * dv) @ _t(w, p + "o").T


def channel_delta(h, w, p, m, eps):
    """The gated delta rule with one decay per head and key channel."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ _t(w, p + "q").T, _t(w, p + "q.conv"))).reshape(T, G, d)
    k = silu(short_conv(h @ _t(w, p + "k").T, _t(w, p + "k.conv"))).reshape(T, G, d)
    v = silu(short_conv(h @ _t(w, p + "v").T, _t(w, p + "v.conv"))).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(dim=-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(dim=-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ _t(w, p + "b").T)           # (T, H)
    step = softplus((h @ _t(w, p + "a1").T) @ _t(w, p + "a2").T + _t(w, p + "dt_bias")).reshape(T, H, d)
    decay = torch.exp(-torch.exp(_t(w, p + "A_log"))[None, :, None] * step)
    gate = torch.sigmoid((h @ _t(w, p + "g1").T) @ _t(w, p + "g2").T).reshape(T, H, dv)
    S = torch.zeros(H, d, dv, dtype=F)
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        for a in range(H):
            g = a // (H // G)
            S[a] = decay[t, a][:, None] * S[a]
            u = beta[t, a] * (v[t, a] - S[a].T @ k[t, g])
            S[a] = S[a] + torch.outer(k[t, g], u)
            o[t, a] = S[a].T @ q[t, g]
    o = rms_norm(o, _t(w, p + "norm"), eps) * gate
    return o.reshape(T, H * dv) @ _t(w, p + "o").T


def dense_ff(h, w, p, f):
    gate = h @ _t(w, p + "gate").T + _t(w, p + "gate.b")
    up = h @ _t(w, p + "up").T + _t(w, p + "up.b")
    return clamped_glu(gate, up, f["limit"]) @ _t(w, p + "down").T + _t(w, p + "down.b")


def routed_ff(h, w, p, f):
    """Each token's `top` experts by sigmoid score; the score multiplies the expert's input."""
    T = h.shape[0]
    E, top, limit = f["router"]["experts"], f["router"]["top"], f["expert"]["limit"]
    scores = torch.sigmoid(h @ _t(w, p + "router").T)
    out = torch.zeros_like(h)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(scores[t, e]), e))[:top]
        for e in order:
            x = scores[t, e] * h[t]
            q = "%se%d." % (p, e)
            y = clamped_glu(_t(w, q + "gate") @ x, _t(w, q + "up") @ x, limit)
            out[t] += _t(w, q + "down") @ y
    return out


def forward(config, w, tokens, streams=None):
    """Logits (T, vocab) of one sequence; `streams`, a list, receives the residual behind every layer."""
    eps = config["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = _t(w, "embed")[ids] * config["embedding"]["scale"]
    kept = {}
    for i, layer in enumerate(config["layers"]):
        p, m = "l%d." % i, layer["mixer"]
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = keys_and_values(x, w, p + "mix.", m, eps)
                k, v = kept[i]
            else:
                k, v = kept[m["kv_from"]]
            y = sink_attention(x, w, p + "mix.", m, eps, k, v)
        elif layer["type"] == "channel_delta":
            y = channel_delta(x, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, _t(w, p + "norm1"), eps)
        f = layer.get("mlp")
        if f is not None:
            y = dense_ff(x, w, p + "mlp.", f) if f["kind"] == "dense" else routed_ff(x, w, p + "mlp.", f)
            x = x + rms_norm(y, _t(w, p + "norm2"), eps)
        if streams is not None:
            streams.append(x.clone())
    return rms_norm(x, _t(w, "final.norm"), eps) @ _t(w, "embed").T


def greedy(config, w, prompt, new_tokens):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(forward(config, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]
