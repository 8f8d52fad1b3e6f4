"""The kernels that came with the Dufinex parts against their plain PyTorch twins (tests/torch_ops.py),
at sizes of their own: the clamped gated unit, the experts chosen by sigmoid scores, the norm per head
in front of attention, attention with a sink (on the general kernel and on the matrix cores, over
prompts, single tokens and both in one step, with key splits and without), and the gated delta rule
over packed steps of unequal sequences with states that are continued. Where random numbers would hide
a fault the inputs are made so that it shows: a sink that carries nearly all of a softmax, one far key
that carries the rest, a decay of nearly nothing next to one of nearly one."""

import pytest
import torch

import torch_ops as twin
from qwen3_from_scratch_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _rand(g, *shape, scale=1.0, dtype=torch.float32):
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def _int(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def _close(got, want, tol):
    got, want = got.float(), want.float()
    bound = tol * max(1.0, float(want.abs().max()))
    assert float((got - want).abs().max()) <= bound, (float((got - want).abs().max()), bound)


def _tol(dtype):
    return 2e-5 if dtype == torch.float32 else 1.2e-2


# ---- feed-forwards ----

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(1, 24), (37, 96), (300, 1000)])
def test_glu_clamped(dtype, T, I):
    g = _gen(T + I)
    x = _rand(g, T, 2 * I, scale=2.0, dtype=dtype)
    bias, scale = _rand(g, 2 * I), torch.rand(T + 9, generator=g).to(DEV)
    index = torch.randint(0, T + 9, (T,), generator=g).to(torch.int32).to(DEV)
    for kwargs in (dict(), dict(bias=bias), dict(scale=scale[:T].contiguous()), dict(scale=scale, scale_index=index),
                   dict(bias=bias, out_dtype=torch.float32 if dtype == torch.float32 else torch.bfloat16)):
        _close(ops.glu_clamped(x, 1.5, 1.702, **kwargs), twin.glu_clamped(x, 1.5, 1.702, **kwargs), _tol(dtype))
    wide = _rand(g, T, 2 * I, scale=2.0)
    _close(ops.glu_clamped(wide, 0.7, 1.1, bias=bias, out_dtype=dtype), twin.glu_clamped(wide, 0.7, 1.1, bias=bias, out_dtype=dtype),
           _tol(dtype))
    # the clamps: a gate far above the limit is the limit, the other branch is held on both sides
    big = torch.tensor([[9.0, 9.0, 9.0, -9.0, -9.0, 0.3]], device=DEV)
    got = ops.glu_clamped(big, 2.0, 1.702)
    s = lambda z: z / (1.0 + torch.exp(torch.tensor(-1.702 * z)))
    want = torch.tensor([[s(2.0) * 3.0, s(2.0) * -1.0, s(-9.0) * 1.3]])
    _close(got.cpu(), want, 1e-6)


@pytest.mark.parametrize("dtype,W,ff,E,top,T", [
    (torch.float32, 48, 40, 6, 2, 29), (torch.float32, 40, 10, 3, 3, 7), (torch.bfloat16, 64, 96, 16, 1, 300),
    (torch.bfloat16, 128, 64, 8, 3, 2000), (torch.bfloat16, 64, 32, 4, 2, 5), (torch.bfloat16, 48, 24, 70, 4, 130),
    (torch.bfloat16, 160, 96, 8, 2, 1500), (torch.float32, 160, 96, 8, 2, 1500)])
def test_experts_by_sigmoid_scores(dtype, W, ff, E, top, T):
    g = _gen(W + E + T)
    h = _rand(g, T, W, dtype=dtype)
    router = _rand(g, E, W, scale=0.3, dtype=dtype)
    gate_up, down = _rand(g, E, 2 * ff, W, scale=0.2, dtype=dtype), _rand(g, E, W, ff, scale=0.2, dtype=dtype)
    chosen, weights = ops.moe_route(h, router, top, scoring="sigmoid")
    chosen2, weights2 = twin.moe_route(h, router, top, scoring="sigmoid")
    same = (chosen == chosen2).all(dim=1)
    assert float(same.float().mean()) >= (1.0 if dtype == torch.float32 else 0.97)      # close calls may fall either way
    _close(weights[same], weights2[same], 1e-5 if dtype == torch.float32 else 2e-2)
    assert float(weights.min()) > 0.0 and float(weights.max()) <= 1.0
    assert top == 1 or float(weights.sum(dim=1).max()) > 1.0          # the chosen scores as they are, not shares of one
    _close(ops.moe_gated_experts(h, chosen, weights, gate_up, down, 2.0, 1.702),
           twin.moe_gated_experts(h, chosen, weights, gate_up, down, 2.0, 1.702), _tol(dtype) * 2)


def test_sigmoid_scores_that_have_run_into_one_still_tell_experts_apart():
    h = torch.zeros(1, 4, device=DEV)
    h[0, 0] = 1.0
    router = torch.zeros(4, 4, device=DEV)
    router[:, 0] = torch.tensor([40.0, 30.0, 50.0, -5.0])          # the logits of the one token
    chosen, weights = ops.moe_route(h, router, 2, scoring="sigmoid")
    assert chosen.tolist() == [[2, 0]] and weights.tolist() == [[1.0, 1.0]]


# ---- attention ----

def _paged_step(g, lens, H, G, d, dv, page, dtype, own=True):
    """A packed step of sequences (rows, keys after the step) over a cache whose pages are handed
    out in a random order, filled with random keys and values."""
    B = len(lens)
    T = sum(q for q, _ in lens)
    n = (H + (G if own else 0)) * d + (G * dv if own else 0) + H
    rows = _rand(g, T, n)
    width = max(-(-k // page) for _, k in lens)
    table = torch.full((B, width), -1, dtype=torch.int32)
    perm = torch.randperm(B * width + 3, generator=g)
    pos, seq, cu, kv, at = [], [], [0], [], 0
    for b, (q, k) in enumerate(lens):
        pos += list(range(k - q, k))
        seq += [b] * q
        cu.append(cu[-1] + q)
        kv.append(k)
        for j in range(-(-k // page)):
            table[b, j] = perm[at]
            at += 1
    P = B * width + 3
    keys, values = _rand(g, P, G, page, d, dtype=dtype), _rand(g, P, G, dv, page, dtype=dtype)
    return rows, keys, values, table.to(DEV), _int(pos), _int(seq), _int(cu), _int(kv)


ATTENTION_CASES = [
    (torch.float32, 6, 2, 24, 40, 16, [(5, 5), (1, 70), (33, 100)]),
    (torch.float32, 3, 3, 10, 6, 8, [(2, 2), (1, 1), (1, 17)]),
    (torch.bfloat16, 8, 1, 64, 64, 16, [(5, 5), (1, 70), (33, 100)]),          # prompts beside single tokens
    (torch.bfloat16, 8, 1, 64, 64, 16, [(1, 1), (1, 700), (1, 3000), (1, 17)]),  # single tokens, keys split over blocks
    (torch.bfloat16, 8, 2, 128, 128, 16, [(300, 3000), (1, 50), (2, 9)]),       # a portion over many keys, split
    (torch.bfloat16, 4, 4, 64, 64, 32, [(600, 600)]),
    (torch.bfloat16, 4, 2, 32, 64, 16, [(7, 40), (1, 33)]),                    # key and value sizes differ: the general kernel
    (torch.bfloat16, 16, 1, 64, 64, 16, [(3, 40), (1, 33), (1, 900)]),          # as many heads on a key head as a block of rows
    (torch.bfloat16, 32, 1, 64, 64, 16, [(3, 40), (1, 33)]),                   # more heads on a key head than a block of rows
]


@pytest.mark.parametrize("dtype,H,G,d,dv,page,lens", ATTENTION_CASES)
@pytest.mark.parametrize("own", [True, False])
def test_norm_per_head_and_attention_with_a_sink(dtype, H, G, d, dv, page, lens, own):
    g = _gen(H * d + len(lens))
    rows, keys, values, table, pos, seq, cu, kv = _paged_step(g, lens, H, G, d, dv, page, dtype, own)
    q_w, k_w = torch.rand(d, generator=g).to(DEV) + 0.5, torch.rand(d, generator=g).to(DEV) + 0.5
    keys2, values2 = keys.clone(), values.clone()
    Gp = G if own else 0
    q = ops.headnorm_prepare(rows, H, Gp, d, dv, q_w, k_w, 1e-5, pos, seq, dtype, block_table=table, k_cache=keys,
                             v_cache=values, values_transposed=True)
    q2 = twin.headnorm_prepare(rows, H, Gp, d, dv, q_w, k_w, 1e-5, pos, seq, dtype, block_table=table, k_cache=keys2,
                               v_cache=values2, values_transposed=True)
    _close(q, q2, _tol(dtype))
    _close(keys, keys2, _tol(dtype))
    _close(values, values2, 0.0)
    sink = _rand(g, H, scale=2.0)
    gate = rows[:, rows.shape[1] - H:]
    sizes = dict(max_q_len=max(n for n, _ in lens), max_kv_len=max(k for _, k in lens))
    for kwargs in (dict(sink=sink, gate=gate), dict(sink=sink), dict(gate=gate)):
        got = ops.softcap_attention(q2, keys2, values2, table, cu, kv, seq, pos, sizes["max_q_len"], sizes["max_kv_len"], 0.3,
                                    0.0, values_transposed=True, min_q_len=min(n for n, _ in lens), **kwargs)
        want = twin.softcap_attention(q2, keys2, values2, table, cu, kv, seq, pos, sizes["max_q_len"], sizes["max_kv_len"],
                                      0.3, 0.0, values_transposed=True, **kwargs)
        _close(got, want, _tol(dtype))


@pytest.mark.parametrize("dtype,d,page", [(torch.float32, 24, 16), (torch.bfloat16, 64, 16), (torch.bfloat16, 128, 64)])
def test_a_sink_that_carries_the_softmax_and_one_far_key(dtype, d, page):
    """Scores of nearly nothing everywhere, so that a large sink takes nearly the whole denominator
    (the result is then exp(score - sink) times the values' sum, and a sink that is left out or
    counted per block of keys is off by orders of magnitude), except that every query's direction is
    the key's at position 3 (or the last of a page, or the first of the next), scaled so that this
    score stands level with the sink: half of the result is that one value, hundreds of keys back."""
    H, G = 4, 2
    for far in (3, page - 1, page, 2 * page):
        g = _gen(d + far)
        lens = [(40, 1000), (1, 1000), (1, 3 * page)]
        rows, keys, values, table, pos, seq, cu, kv = _paged_step(g, lens, H, G, d, d, page, dtype)
        keys.mul_(1e-3)
        direction = torch.nn.functional.normalize(_rand(g, G, d), dim=-1)
        q = direction.repeat_interleave(H // G, dim=0)[None].repeat(rows.shape[0], 1, 1).to(dtype).contiguous()
        for b in range(len(lens)):
            keys[table[b, far // page].long(), :, far % page] = (direction * 8.0).to(dtype)
        sink = torch.full((H,), 8.0, device=DEV) + _rand(g, H, scale=0.3)
        got = ops.softcap_attention(q, keys, values, table, cu, kv, seq, pos, 40, 1000, 1.0, 0.0, sink=sink,
                                    values_transposed=True, min_q_len=1)
        want = twin.softcap_attention(q, keys, values, table, cu, kv, seq, pos, 40, 1000, 1.0, 0.0, sink=sink,
                                      values_transposed=True)
        without = twin.softcap_attention(q, keys, values, table, cu, kv, seq, pos, 40, 1000, 1.0, 0.0, values_transposed=True)
        assert float((want - without).abs().max()) > 0.2            # the sink matters here
        _close(got, want, _tol(dtype))


# ---- the gated delta rule ----

DELTA_CASES = [
    (torch.float32, 4, 4, 32, 64, [5, 1, 40]), (torch.float32, 6, 2, 24, 20, [3, 1, 1, 17]),
    (torch.bfloat16, 4, 2, 128, 128, [100, 1]), (torch.float32, 2, 1, 200, 48, [9, 2]),
    (torch.float32, 3, 3, 64, 100, [33]), (torch.float32, 1, 1, 4, 70, [1, 1, 1]), (torch.bfloat16, 2, 1, 256, 36, [2, 50]),
]


def _delta_inputs(g, H, G, d, dv, lens, slots_n=5, pad=7):
    T = sum(lens)
    conv = _rand(g, T, 2 * G * d + H * dv)
    wide = _rand(g, T, H + H * d + H * dv + 3)           # the three inputs as stretches of wider rows
    parts = wide[:, :H], wide[:, H:H + H * d], wide[:, H + H * d:H + H * d + H * dv]
    consts = _rand(g, H * d), _rand(g, H, scale=0.5), torch.rand(dv, generator=g).to(DEV) + 0.5
    state = _rand(g, slots_n, pad + H * d * dv, scale=0.1)
    slots = torch.randperm(slots_n, generator=g)[:len(lens)].to(torch.int32).to(DEV)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    return conv, parts, consts, state, slots, _int(cu)


@pytest.mark.parametrize("dtype,H,G,d,dv,lens", DELTA_CASES)
def test_channel_delta(dtype, H, G, d, dv, lens):
    g = _gen(H * d + dv)
    conv, (b, a, gate), (dt_bias, a_log, norm), state, slots, cu = _delta_inputs(g, H, G, d, dv, lens)
    s1, s2 = state.clone(), state.clone()
    got = ops.channel_delta(conv, b, a, gate, dt_bias, a_log, norm, 1e-5, 1e-6, s1[:, 7:], slots, cu, H, G, d, dv, dtype)
    want = twin.channel_delta(conv, b, a, gate, dt_bias, a_log, norm, 1e-5, 1e-6, s2[:, 7:], slots, cu, H, G, d, dv, dtype)
    _close(got, want, _tol(dtype))
    _close(s1, s2, 2e-5)              # the states, and what lies beside them and in other slots untouched
    # the same tokens one step at a time give the same numbers: a column's arithmetic has one order
    s3 = state.clone()
    pieces = []
    offsets = cu.tolist()
    longest = max(lens)
    out = torch.zeros_like(got)
    for i in range(longest):
        rows = [offsets[j] + i for j, n in enumerate(lens) if i < n]
        who = [j for j, n in enumerate(lens) if i < n]
        index = torch.tensor(rows, device=DEV)
        step = ops.channel_delta(conv[index].contiguous(), b[index], a[index], gate[index], dt_bias, a_log, norm, 1e-5, 1e-6,
                                 s3[:, 7:], slots[torch.tensor(who, device=DEV)].contiguous(), _int(list(range(len(rows) + 1))),
                                 H, G, d, dv, dtype)
        out[index] = step
    assert torch.equal(out, got) and torch.equal(s3, s1)


def test_decays_of_nothing_and_of_everything():
    """A head whose decay is nearly zero forgets all but the current token (its result is beta (v . ) of
    that token alone), a head whose decay is nearly one keeps everything: both beside each other."""
    H, G, d, dv, lens = 2, 1, 32, 16, [60]
    g = _gen(11)
    conv, (b, a, gate), (dt_bias, a_log, norm), state, slots, cu = _delta_inputs(g, H, G, d, dv, lens)
    state.zero_()
    a_log = torch.tensor([11.0, -12.0], device=DEV)
    args = (dt_bias, a_log, norm, 1e-5, 1e-6)
    s1, s2 = state.clone(), state.clone()
    got = ops.channel_delta(conv, b, a, gate, *args, s1[:, 7:], slots, cu, H, G, d, dv, torch.float32)
    want = twin.channel_delta(conv, b, a, gate, *args, s2[:, 7:], slots, cu, H, G, d, dv, torch.float32)
    _close(got, want, 2e-5)
    # head 0 alone on the last token from an empty state: the same result, since nothing was kept
    s3 = state.clone()
    last = ops.channel_delta(conv[-1:].contiguous(), b[-1:], a[-1:], gate[-1:], *args, s3[:, 7:], slots, _int([0, 1]), H, G, d,
                             dv, torch.float32)
    _close(last[:, :dv], got[-1:, :dv], 1e-4)
    assert float((last[:, dv:] - got[-1:, dv:]).abs().max()) > 1e-2
