"""The Fidevik architecture through the engine against tests/plain_fidevik.py: each mechanism alone,
whole prompts against token-by-token decoding, portions down to two tokens, mixed batches with pages
that are used again, keys far back and at page borders, the first tokens, long decoding, and greedy
generation through the engine. The configurations are made here; their sizes differ from layer to
layer and avoid values that hide a fault (equal key and value sizes, one key head per query head, a
rotation over the whole head, one pass, groups that are all kept, a logit scale of one)."""

import copy
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import plain_fidevik as plain
from helpers import max_live_tokens, random_tokens, run_trace, trace_mixed, trace_portions, trace_tail_decoded, trace_whole
from qwen3_from_scratch_amd.config import load_model_config
from qwen3_from_scratch_amd.config.fidevik_config import FidevikConfig
from qwen3_from_scratch_amd.config.model_config import ConfigError
from qwen3_from_scratch_amd.engine import StepEntry, SyncEngine, load_runner
from qwen3_from_scratch_amd.weights import write_random_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _attention(heads, kv_heads, dim, vdim, dims=None, base=10000.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or 1.0 / math.sqrt(dim)}
    if dims:
        m["rot"] = {"dims": dims, "base": base}
    return {"type": "attention", "mixer": m}


def _latent(heads, dim, vdim, q_rank, kv_rank, scale=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank,
                                                  "kv_rank": kv_rank, "scale": scale or 1.0 / math.sqrt(dim)}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, groups=None, keep=None, shared=0):
    f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if groups:
        f["router"]["groups"] = {"count": groups, "keep": keep}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def _layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


# a layer before the loop and one behind it, three passes; a layer without a feed-forward; heads that share
# key heads two and three to one; a rotation over part of the head and over all of it
MIXED = {
    "architecture": "Fidevik", "vocab": 131, "width": 48, "norm": {"eps": 1e-5}, "logit_scale": 0.7,
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        _layer(_attention(4, 2, 16, 24, dims=8, base=500.0), _dense(56)),
        _layer(_latent(3, 8, 12, 20, 24), _moe(6, 2, 20, groups=3, keep=2, shared=28)),
        _layer(_attention(6, 2, 8, 8, dims=8), None),
        _layer(_latent(5, 12, 20, 28, 40, scale=0.4), _moe(8, 3, 24, groups=4, keep=3)),
    ]}
# sizes in steps that the matrix-core kernels take; the loop from the first layer on, two passes
CORES = {
    "architecture": "Fidevik", "vocab": 257, "width": 128, "norm": {"eps": 1e-6}, "logit_scale": 1.5,
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        _layer(_latent(4, 32, 48, 64, 96), _moe(8, 3, 64, groups=4, keep=2, shared=96)),
        _layer(_attention(4, 1, 64, 64, dims=32, base=20000.0), _dense(192)),
        _layer(_attention(8, 4, 128, 128, dims=128), _moe(4, 2, 128, groups=2, keep=1, shared=64)),
    ]}
# sizes that no vector access and no matrix instruction takes; one head, one expert a token, groups of one
# expert, a loop of one pass, no rotation, no logit scale
ODD = {
    "architecture": "Fidevik", "vocab": 53, "width": 40, "norm": {"eps": 1e-5},
    "loop": {"start": 0, "stop": 2, "times": 1},
    "layers": [
        _layer(_attention(3, 1, 10, 14, dims=4), _moe(3, 1, 18, groups=3, keep=1)),
        _layer(_latent(1, 6, 3, 5, 7), _moe(4, 4, 9, shared=10)),
        _layer(_attention(2, 2, 6, 10), _dense(22)),
    ]}
# no loop at all, and the two mixers the other way round
STRAIGHT = {
    "architecture": "Fidevik", "vocab": 97, "width": 64, "norm": {"eps": 1e-6}, "logit_scale": 0.25,
    "layers": [
        _layer(_latent(2, 16, 24, 24, 32), _dense(96)),
        _layer(_attention(4, 4, 16, 32, dims=12, base=30000.0), _moe(6, 2, 32, groups=2, keep=1, shared=32)),
    ]}
CONFIGS = {"mixed": MIXED, "cores": CORES, "odd": ODD, "straight": STRAIGHT}


def _write(folder, data, seed=5, std=0.2, peak=None):
    write_random_model(str(folder), FidevikConfig.from_dict(data), seed=seed, std=std, norm_jitter=0.3)
    if peak:                              # larger queries: every softmax then stands on a few keys
        path = os.path.join(str(folder), "model.safetensors")
        tensors = load_file(path)
        for key in tensors:
            if key.endswith("dq.norm") or key.endswith("mix.q.norm"):
                tensors[key] = (tensors[key].float() * peak).to(tensors[key].dtype)
        save_file(tensors, path, metadata={"format": "pt"})
    return str(folder)


def _every_expert(data):
    """The configuration with every expert chosen for every token. In bfloat16 a router's score moves
    by a few thousandths, and with random weights some token in a hundred then changes an expert, which
    no bound on rounding covers; the choice itself is float32 in both precisions and is tested there and
    on the router kernel. With all experts chosen the weights still matter."""
    data = copy.deepcopy(data)
    for layer in data["layers"]:
        if layer["mlp"] and layer["mlp"]["kind"] == "moe":
            router = layer["mlp"]["router"]
            router["top"] = router["experts"]
            if "groups" in router:
                router["groups"]["keep"] = router["groups"]["count"]
    return data


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def folder(request, tmp_path_factory):
    return _write(tmp_path_factory.mktemp(request.param), CONFIGS[request.param], peak=3.0)


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def folders(request, tmp_path_factory):
    """{dtype: folder}: the configuration as it is for float32, with every expert chosen for bfloat16."""
    return {"float32": _write(tmp_path_factory.mktemp(request.param), CONFIGS[request.param], peak=3.0),
            "bfloat16": _write(tmp_path_factory.mktemp(request.param + "_all"), _every_expert(CONFIGS[request.param]))}


def _truth(folder, requests, dtype=torch.float64):
    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    w = {k: v.to(dtype) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, w, {rid: plain.logits_of_sequence(config, w, toks) for rid, toks in requests.items()}


def _requests(folder, lengths=(70, 9, 41, 130, 25, 2, 1)):
    vocab = load_model_config(folder).vocab
    return {"f%d" % i: random_tokens(n, vocab, 260 + i) for i, n in enumerate(lengths)}


def _off(got, want, dtype):
    """The worst row: its difference (mean taken off, root mean square) over the spread of the true
    row, in units of what the dtype may be off by."""
    worst = 0.0
    for rid, logits in want.items():
        for p in range(logits.shape[0]):
            d = got[(rid, p)].double() - logits[p].double()
            err = float((d - d.mean()).pow(2).mean().sqrt() / logits[p].double().std())
            worst = max(worst, err / (5e-5 if dtype == "float32" else 5e-2))
    return worst


# ---- configuration and weights ----

def test_config_is_read_by_its_own_keys_and_written_back(folder):
    config = load_model_config(folder)
    assert isinstance(config, FidevikConfig) and config.architecture == "Fidevik"
    with open(os.path.join(folder, "config.json")) as fh:
        raw = json.load(fh)
    assert config.to_dict() == raw and len(config.layers) == len(raw["layers"])
    assert config.logit_scale == raw.get("logit_scale", 1.0)
    names = set(load_file(os.path.join(folder, "model.safetensors")))
    assert {"embed", "head", "final.norm", "final.norm.b", "l0.norm1", "l0.norm1.b"} <= names
    assert ("loop.step" in names) == ("loop" in raw)
    for i, (layer, entry) in enumerate(zip(config.layers, raw["layers"])):
        p = "l%d." % i
        assert layer.type == entry["type"] and (layer.mlp is None) == (entry["mlp"] is None)
        assert (p + "norm2.b" in names) == (entry["mlp"] is not None)
        if entry["type"] == "attention":
            assert {p + "mix.q.norm", p + "mix.k.norm", p + "mix.o"} <= names and p + "mix.q.b" not in names
            assert p + "mix.g" not in names
            assert (layer.mixer.rot is None) == ("rot" not in entry["mixer"])
        else:
            assert {p + "mix.dq.norm", p + "mix.uk", p + "mix.sink", p + "mix.g"} <= names
        if entry["mlp"] and entry["mlp"]["kind"] == "moe":
            assert {p + "mlp.router", p + "mlp.correction", p + "mlp.e0.gate"} <= names
            assert (p + "mlp.shared.sg" in names) == ("shared" in entry["mlp"])
            groups = entry["mlp"]["router"].get("groups", {"count": 1, "keep": 1})
            assert (layer.mlp.groups, layer.mlp.keep) == (groups["count"], groups["keep"])
        elif entry["mlp"]:
            assert {p + "mlp.gate", p + "mlp.up", p + "mlp.down"} <= names


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="other"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "divide"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "kind"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=99), "top"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "kept"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "divide"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=7), "keep"),
    (lambda c: c.update(loop={"start": 2, "stop": 9, "times": 2}), "loop"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "exceeds"),
    (lambda c: c.pop("width"), "width"),
])
def test_config_errors_name_the_key(change, word):
    data = copy.deepcopy(MIXED)
    change(data)
    with pytest.raises(ConfigError, match=word):
        FidevikConfig.from_dict(data)


def test_run_order_and_cache_planes(cpu_ops, tmp_path):
    """The loop's layers appear once per pass, each appearance with a cache plane of its own; planes
    of equal needs share a group."""
    folder = _write(tmp_path / "m", MIXED)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=256, max_requests=4)
    order = [(s.layer, s.enters) for s in runner.model.spec.order]
    assert order == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None)]
    assert order == [(i, t) for i, t in plain.run_order(MIXED)]
    assert len(runner.model.plane_needs) == 8 and len(set(runner.model.plane_of_step)) == 8
    groups = sorted((tuple(t.shape for t in g.tensors), len(g.planes)) for g in runner.manager.groups)
    assert groups == sorted([(((2, 16), (2, 24)), 1), (((24,),), 3), (((2, 8), (2, 8)), 3), (((40,),), 1)])
    assert runner.model.pass_vectors.wants_start
    # a loop of one pass never asks for the embedding's output again; a model without a loop has no pass vectors
    one = load_runner(_write(tmp_path / "o", ODD), dtype="float32", device="cpu", page_size=8, max_tokens=64, max_requests=1)
    assert one.model.pass_vectors is not None and not one.model.pass_vectors.wants_start
    none = load_runner(_write(tmp_path / "s", STRAIGHT), dtype="float32", device="cpu", page_size=8, max_tokens=64,
                       max_requests=1)
    assert none.model.pass_vectors is None


def test_a_loop_over_no_layers_is_no_loop(cpu_ops, tmp_path):
    """start == stop: the layers run once, no pass begins, and the table of vectors that such a file may
    still hold is left unread."""
    data = dict(copy.deepcopy(STRAIGHT), loop={"start": 1, "stop": 1, "times": 2})
    folder = _write(tmp_path / "m", data)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    assert "loop.step" not in tensors
    tensors["loop.step"] = torch.ones((2, data["width"]), dtype=torch.bfloat16)
    save_file(tensors, path, metadata={"format": "pt"})
    requests = {"a": random_tokens(20, data["vocab"], 3)}
    _, _, want = _truth(folder, requests)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=32, max_requests=1)
    assert [(s.layer, s.enters) for s in runner.model.spec.order] == [(0, None), (1, None)]
    assert _off(run_trace(runner, trace_whole(requests)), want, "float32") <= 1.0


# ---- each mechanism alone, on the host twins and against the plain functions ----

def test_layer_norm_twin_takes_every_addend(cpu_ops):
    g = torch.Generator().manual_seed(2)
    x, delta, extra = (torch.randn(9, 20, generator=g) for _ in range(3))
    vec, w, b = (torch.randn(20, generator=g) for _ in range(3))
    want = plain.layer_norm((x + delta + extra + vec).double(), w.double(), b.double(), 1e-5)
    stream = x.clone()
    got = cpu_ops.layernorm_addend(stream, w, b, 1e-5, torch.float32, delta=delta, extra=extra, vec=vec)
    assert torch.allclose(got.double(), want, atol=1e-5) and torch.allclose(stream, x + delta + extra + vec)
    rows = torch.tensor([8, 0], dtype=torch.int32)
    stream = x.clone()
    got = cpu_ops.layernorm_addend(stream, w, b, 1e-5, torch.float32, delta=delta, rows=rows)
    assert torch.equal(stream, x)
    assert torch.allclose(got.double(), plain.layer_norm((x + delta).double(), w.double(), b.double(), 1e-5)[[8, 0]], atol=1e-5)
    # the mean comes out before the squares: a row that is constant plus a small wave
    row = (1000.0 + torch.sin(torch.arange(20.0)))[None, :]
    got = cpu_ops.layernorm_addend(row.clone(), torch.ones(20), torch.zeros(20), 0.0, torch.float32)
    wave = torch.sin(torch.arange(20.0, dtype=torch.float64))
    wave = wave - wave.mean()
    assert torch.allclose(got[0].double(), wave / wave.pow(2).mean().sqrt(), atol=1e-3)


def test_router_twin_and_plain_agree(cpu_ops):
    g = torch.Generator().manual_seed(1)
    for E, top, groups, keep in ((12, 3, 4, 2), (6, 2, 3, 2), (8, 8, 4, 4), (5, 1, 5, 1), (9, 2, 1, 1), (6, 4, 2, 2)):
        h, router = torch.randn(60, 24, generator=g), torch.randn(E, 24, generator=g)
        correction = torch.randn(E, generator=g) * 0.5
        chosen, weights = cpu_ops.moe_route(h, router, top, scoring="sigmoid_groups", correction=correction,
                                            groups=groups, keep=keep)
        z = h.double() @ router.double().T
        at, share = plain.choose_experts(z, correction.double(), top, groups, keep)
        assert torch.equal(chosen.long().sort(dim=-1).values, at.sort(dim=-1).values)
        assert torch.allclose(weights.double().sort(dim=-1).values, share.sort(dim=-1).values, atol=1e-6)


def test_choice_goes_by_the_corrected_score_within_the_best_groups():
    """Made by hand: the correction decides the choice and never the weight; a group is judged by its
    two best; an expert outside the kept groups is not chosen however good it is, also when every
    corrected score is negative (what is left out counts as minus infinity, not as nothing)."""
    z = torch.tensor([[2.0, -3.0, 1.0, 0.9, -1.0, -1.1]], dtype=torch.float64)        # groups (0,1) (2,3) (4,5)
    none = torch.zeros(6, dtype=torch.float64)
    at, share = plain.choose_experts(z, none, 2, 3, 1)
    # group 0 has the single best expert, but group 1's two best sum higher
    assert sorted(at[0].tolist()) == [2, 3]
    assert torch.allclose(share[0].sort().values, torch.sigmoid(torch.tensor([0.9, 1.0], dtype=torch.float64)))
    at, share = plain.choose_experts(z, torch.tensor([0.0, 0.0, 0.0, 0.0, 0.6, 0.6], dtype=torch.float64), 2, 3, 1)
    assert sorted(at[0].tolist()) == [4, 5]
    assert torch.allclose(share[0].sort().values, torch.sigmoid(torch.tensor([-1.1, -1.0], dtype=torch.float64)))
    at, _ = plain.choose_experts(z, torch.full((6,), -5.0, dtype=torch.float64), 3, 3, 2)
    assert sorted(at[0].tolist()) == [0, 2, 3]            # all negative: experts 4 and 5 still never come up


def test_sink_and_gate_twin_against_plain(cpu_ops):
    """The latent attention of one layer through the twins, a sink of +4 on one head and -30 on
    another: the first head's result shrinks, the second's is what it is without a sink."""
    data = copy.deepcopy(STRAIGHT)
    config = FidevikConfig.from_dict(data)
    m = data["layers"][0]["mixer"]
    g = torch.Generator().manual_seed(3)
    names = {"dq": (m["q_rank"], 64), "uq": (m["heads"] * m["dim"], m["q_rank"]), "dkv": (m["kv_rank"], 64),
             "uk": (m["heads"] * m["dim"], m["kv_rank"]), "uv": (m["heads"] * m["vdim"], m["kv_rank"]), "g": (m["heads"], 64),
             "o": (64, m["heads"] * m["vdim"])}
    w = {"x." + k: torch.randn(s, generator=g, dtype=torch.float64) * 0.3 for k, s in names.items()}
    w["x.dq.norm"] = torch.ones(m["q_rank"], dtype=torch.float64)
    w["x.dkv.norm"] = torch.ones(m["kv_rank"], dtype=torch.float64)
    h = torch.randn(11, 64, generator=g, dtype=torch.float64)
    w["x.sink"] = torch.tensor([4.0, -30.0], dtype=torch.float64)
    with_sink = plain.latent_attention(h, w, "x", m, config.eps)
    w["x.sink"] = torch.tensor([-30.0, -30.0], dtype=torch.float64)
    without = plain.latent_attention(h, w, "x", m, config.eps)
    w["x.o"] = torch.eye(64, dtype=torch.float64)[:, :m["heads"] * m["vdim"]]       # heads side by side in the result
    w["x.sink"] = torch.tensor([4.0, -30.0], dtype=torch.float64)
    a = plain.latent_attention(h, w, "x", m, config.eps)
    w["x.sink"] = torch.tensor([-30.0, -30.0], dtype=torch.float64)
    b = plain.latent_attention(h, w, "x", m, config.eps)
    dv = m["vdim"]
    assert float((a[:, :dv].abs() / b[:, :dv].abs().clamp(min=1e-12)).max()) < 1.0          # the sink takes weight away
    assert torch.allclose(a[:, dv:2 * dv], b[:, dv:2 * dv], atol=1e-12)
    assert not torch.allclose(with_sink, without)
    # the first token sees itself and the sink only: its weight is 1 / (1 + exp(sink - score))
    cq = plain.rms_norm(h[:1] @ w["x.dq"].T, w["x.dq.norm"], config.eps)
    c = plain.rms_norm(h[:1] @ w["x.dkv"].T, w["x.dkv.norm"], config.eps)
    q0, k0 = (cq @ w["x.uq"].T)[0, :m["dim"]], (c @ w["x.uk"].T)[0, :m["dim"]]
    v0 = (c @ w["x.uv"].T)[0, :dv]
    share = 1.0 / (1.0 + torch.exp(4.0 - (q0 @ k0) * m["scale"]))
    gate = torch.sigmoid(h[:1] @ w["x.g"].T)[0, 0]
    assert torch.allclose(a[0, :dv], share * gate * v0, atol=1e-12)


def test_logits_on_the_host_under_every_cutting(cpu_ops, folder):
    requests = _requests(folder)
    _, _, want = _truth(folder, requests)
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype="float32", device="cpu", page_size=8,
                             max_tokens=max_live_tokens(steps, page=8), max_requests=4)
        assert _off(run_trace(runner, steps), want, "float32") <= 1.0, make.__name__
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.groups)


def test_layer_streams_on_the_host(cpu_ops, tmp_path):
    """The residual stream behind every run of a layer, what it still lacks included: the passes'
    vectors and, from the second pass on, the embedding's output once more are in it."""
    folder = _write(tmp_path / "m", MIXED)
    tokens = random_tokens(37, MIXED["vocab"], 4)
    config, w, _ = _truth(folder, {})
    streams = []
    plain.logits_of_sequence(config, w, tokens, streams)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=64, max_requests=1)
    seen = []
    runner.model.observer = lambda i, x, pending: seen.append(x.double() + pending.double())
    runner.step([StepEntry("r", tokens, [])])
    assert len(seen) == len(streams) == 8
    for got, want in zip(seen, streams):
        assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max())
    # without the embedding's second entry the third run already differs
    left_out = dict(config, loop=dict(config["loop"], times=1))
    short = []
    plain.logits_of_sequence(left_out, w, tokens, short)
    assert float((short[2] - streams[2]).abs().max()) == 0 and len(short) == 4


def test_greedy_generation_through_the_engine_on_the_host(cpu_ops, folder):
    requests = _requests(folder)
    config, w, _ = _truth(folder, {})
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=256, block_size=8, num_blocks=60,
                        max_num_seqs=3, max_num_tokens=24, chunked_prefill_size=16)
    prompts = [toks[:n] for toks, n in zip(requests.values(), (30, 9, 41, 2))]
    got = engine.generate_ids(prompts, max_new_tokens=5, temperature=0.0, ignore_eos=True)
    for prompt, new in zip(prompts, got):
        seq = list(prompt)
        for _ in range(5):
            seq.append(int(torch.argmax(plain.logits_of_sequence(config, w, seq)[-1])))
        assert new == seq[len(prompt):]
    assert engine.runner.manager.num_free() == 60


def test_requests_share_a_prefix(cpu_ops, tmp_path):
    """No layer has a window or a state, so the pages of a shared beginning serve a second request, in
    every pass's plane, and it generates what it would have alone."""
    folder = _write(tmp_path / "m", MIXED, peak=3.0)
    config, w, _ = _truth(folder, {})
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=128, block_size=8, num_blocks=40,
                        max_num_seqs=2, max_num_tokens=32, chunked_prefill_size=16, enable_prefix_cache=True)
    assert engine.runner.manager.prefix_cache
    stem = random_tokens(29, MIXED["vocab"], 21)
    prompts = [stem + random_tokens(5, MIXED["vocab"], 22), stem + random_tokens(9, MIXED["vocab"], 23)]
    got = [engine.generate_ids([p], max_new_tokens=4, temperature=0.0, ignore_eos=True)[0] for p in prompts]
    assert engine.runner.manager.prefix_hits == 24            # three blocks of eight
    for prompt, new in zip(prompts, got):
        seq = list(prompt)
        for _ in range(4):
            seq.append(int(torch.argmax(plain.logits_of_sequence(config, w, seq)[-1])))
        assert new == seq[len(prompt):]


def test_command_line_writes_a_folder_from_the_nested_config(tmp_path):
    from qwen3_from_scratch_amd.engine.cli import main

    source = tmp_path / "config.json"
    source.write_text(json.dumps(STRAIGHT))
    assert main(["--write_random", str(tmp_path / "m"), "--from_config", str(source), "--seed", "3"]) == 0
    assert load_model_config(str(tmp_path / "m")).to_dict() == STRAIGHT
    names = set(load_file(str(tmp_path / "m" / "model.safetensors")))
    assert "l1.mlp.e2.down" in names and "l1.mlp.shared.sg" in names and "loop.step" not in names


# ---- kernels against their twins ----

def _rand(shape, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H", [(5, 48), (130, 260), (3, 1031), (1, 4096)])
def test_layer_norm_kernel(dtype, T, H):
    import torch_ops
    from qwen3_from_scratch_amd import ops

    w, b = _rand((H,), 1, torch.float32) + 1, _rand((H,), 2, torch.float32)
    delta, extra, vec = _rand((T, H), 3, dtype, 3.0), _rand((T, H), 4, torch.float32), _rand((H,), 6, torch.float32)
    rows = torch.tensor([T - 1, 0], dtype=torch.int32).cuda()
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    for kw in (dict(delta=delta, extra=extra, vec=vec), dict(delta=delta), dict(vec=vec), dict(extra=extra), dict(),
               dict(delta=delta, vec=vec, rows=rows), dict(rows=rows)):
        x1 = _rand((T, H), 5, torch.float32, 2.0) + 3.0               # a mean that is not small beside the spread
        x2 = x1.clone()
        a = ops.layernorm_addend(x1, w, b, 1e-5, dtype, **kw)
        c = torch_ops.layernorm_addend(x2, w, b, 1e-5, dtype, **kw)
        assert torch.allclose(x1, x2, atol=1e-5, rtol=1e-5) and float((a.float() - c.float()).abs().max()) <= tol
        if "rows" in kw:
            assert torch.equal(x1, _rand((T, H), 5, torch.float32, 2.0) + 3.0)      # a selection leaves the stream alone
    x1 = _rand((T, H), 5, torch.float32)
    x2 = x1.clone()
    assert ops.layernorm_addend(x1, None, None, 0.0, dtype, delta=delta, vec=vec) is None
    torch_ops.layernorm_addend(x2, None, None, 0.0, dtype, delta=delta, vec=vec)
    assert torch.allclose(x1, x2, atol=1e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,I", [(37, 53), (4, 256), (300, 24)])
def test_gated_activation_kernel(dtype, T, I):
    import torch_ops
    from qwen3_from_scratch_amd import ops

    x = _rand((T, 2 * I), 1, dtype, 3.0)
    for kind in ("silu", "gelu_tanh", "gelu_erf"):
        a, b = ops.gated_act(x, kind), torch_ops.gated_act(x, kind)
        assert float((a.float() - b.float()).abs().max()) <= (1e-5 if dtype == torch.float32 else 6e-2), kind
    assert torch.equal(ops.swiglu(x), ops.gated_act(x, "silu"))
    pair = torch.tensor([[1.0, 2.0]]).cuda()
    assert abs(float(ops.gated_act(pair, "gelu_tanh")) - 2 * 0.8411920) < 1e-6
    assert abs(float(ops.gated_act(pair, "gelu_erf")) - 2 * 0.8413447) < 1e-6
    assert abs(float(ops.gated_act(pair, "silu")) - 2 * 0.7310586) < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_rank,kv_rank,more", [(20, 40, 3), (80, 128, 4), (33, 7, 0)])
def test_latent_prepare_without_a_rotated_part(dtype, q_rank, kv_rank, more):
    """Rows that carry further columns behind the two latents (a gate's), keys without a rotated part."""
    import torch_ops
    from qwen3_from_scratch_amd import ops

    T, page = 45, 8
    wide = _rand((T, q_rank + kv_rank + more), 1, dtype, 2.0)
    qw, kw = _rand((q_rank,), 2, torch.bfloat16) + 1, _rand((kv_rank,), 3, torch.bfloat16) + 1
    positions = torch.cat((torch.arange(30), torch.arange(7, 22))).int().cuda()
    seq = torch.cat((torch.zeros(30), torch.ones(15))).int().cuda()
    table = torch.tensor([[5, 2, 7, 0], [1, 6, 3, -1]], dtype=torch.int32).cuda()
    c1 = torch.zeros((9, page, kv_rank), dtype=dtype).cuda()
    c2 = c1.clone()
    a = ops.latent_prepare(wide, q_rank, kv_rank, 0, qw, kw, 1e-5, None, 1.0, positions, seq, table, c1)
    b = torch_ops.latent_prepare(wide, q_rank, kv_rank, 0, qw, kw, 1e-5, None, 1.0, positions, seq, table, c2)
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    assert float((a.float() - b.float()).abs().max()) <= tol * 4 and float((c1.float() - c2.float()).abs().max()) <= tol * 4
    assert float(c1[8].abs().max()) == 0 and float(c1[4].abs().max()) == 0     # untouched pages


def _paged(rows_per_seq, page, Dk, dtype, seed):
    """Sequences' cached rows scattered over pages in a shuffled order; returns cache, table, rows."""
    blocks = [-(-n // page) for n in rows_per_seq]
    order = torch.randperm(sum(blocks) + 3, generator=torch.Generator().manual_seed(seed)).tolist()
    cache = torch.zeros((sum(blocks) + 3, page, Dk), dtype=dtype)
    table = torch.full((len(rows_per_seq), max(blocks)), -1, dtype=torch.int32)
    rows = []
    for b, n in enumerate(rows_per_seq):
        r = (torch.randn((n, Dk), generator=torch.Generator().manual_seed(seed + 1 + b))).to(dtype)
        rows.append(r)
        for j in range(blocks[b]):
            pg = order.pop()
            table[b, j] = pg
            part = r[j * page:(j + 1) * page]
            cache[pg, :part.shape[0]] = part
    return cache.cuda(), table.cuda(), rows


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("general", [False, True])
@pytest.mark.parametrize("H,D,page", [(3, 40, 8), (5, 128, 16), (4, 96, 16), (1, 7, 16), (16, 64, 32), (6, 256, 16)])
def test_latent_attention_with_sink_and_gate(dtype, H, D, page, general):
    """Keys that are values whole (no rotated part), a sink per head and a gate per (token, head) that lies
    in a wider tensor: prompts' portions beside single tokens, over scattered pages, against the twin; then
    one key made to carry the whole softmax, far back and at a page's first and last place, against a
    sink that is out of reach and a sink that takes half."""
    import torch_ops
    from qwen3_from_scratch_amd import ops

    if general and not (dtype == torch.bfloat16 and D % 32 == 0):
        pytest.skip("these sizes take the general kernel anyway")
    kv = [150, 33, 1, 257, 64]
    q_lens = [37, 1, 1, 2, 64]
    cache, table, rows = _paged(kv, page, D, dtype, 11)
    cu = torch.tensor([0] + list(np.cumsum(q_lens)), dtype=torch.int32).cuda()
    kvl = torch.tensor(kv, dtype=torch.int32).cuda()
    T = sum(q_lens)
    q = _rand((T, H, D), 3, dtype, 1.5)
    sink = _rand((H,), 4, torch.float32, 2.0)
    wide = _rand((T, H + 5), 5, dtype, 2.0)
    gate = wide[:, 2:2 + H]
    scale = D ** -0.5
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for kw in (dict(sink=sink, gate=gate), dict(sink=sink), dict(gate=gate)):
        a = ops.latent_attention(q, cache, D, table, cu, kvl, max(q_lens), scale, general=general, max_kv_len=max(kv), **kw)
        b = torch_ops.latent_attention(q, cache, D, table, cu, kvl, max(q_lens), scale, **kw)
        assert float((a.float() - b.float()).abs().max()) <= tol, sorted(kw)
    seq, L = 3, kv[3]
    at = int(cu[seq]) + 1                               # the sequence's last token
    for back in sorted({0, 1, page - 1, page, 2 * page, L - 1}) if D >= 32 else ():      # few numbers tell no key apart
        target = L - 1 - back
        peaked = q.clone()
        peaked[at] = (rows[seq][target] * 8.0).to(dtype).cuda()[None, :]
        want = rows[seq][target].float().cuda()
        score = float((rows[seq][target].to(dtype).float() * 8.0) @ rows[seq][target].float())
        for value, share in ((-1e4, 1.0), (score, 0.5)):
            s = torch.full((H,), value, dtype=torch.float32).cuda()
            got = ops.latent_attention(peaked, cache, D, table, cu, kvl, max(q_lens), 1.0, general=general, sink=s)[at].float()
            assert float((got - share * want[None, :]).abs().max()) <= 0.05, (back, share)


@pytest.mark.gpu
@pytest.mark.parametrize("H,D", [(5, 128), (16, 512), (3, 64)])
def test_latent_attention_of_single_tokens_with_sink_and_gate(H, D):
    """Steps of one token a sequence over many keys: the keys go over several blocks, and the sink and
    the gate join where the shares are merged."""
    import torch_ops
    from qwen3_from_scratch_amd import ops

    kv = [1000, 1, 513, 37, 2048]
    cache, table, rows = _paged(kv, 16, D, torch.bfloat16, 5)
    cu = torch.arange(len(kv) + 1, dtype=torch.int32).cuda()
    kvl = torch.tensor(kv, dtype=torch.int32).cuda()
    q = _rand((len(kv), H, D), 3, torch.bfloat16, 1.5)
    sink = _rand((H,), 4, torch.float32, 2.0) + 2.0
    gate = _rand((len(kv), H), 5, torch.bfloat16, 2.0)
    assert ops._latent_splits(len(kv), len(kv), H, 1, max(kv), 0) > 1
    a = ops.latent_attention(q, cache, D, table, cu, kvl, 1, D ** -0.5, max_kv_len=max(kv), sink=sink, gate=gate)
    b = torch_ops.latent_attention(q, cache, D, table, cu, kvl, 1, D ** -0.5, sink=sink, gate=gate)
    c = torch_ops.latent_attention(q, cache, D, table, cu, kvl, 1, D ** -0.5)
    assert float((a.float() - b.float()).abs().max()) <= 3e-2
    assert float((b.float() - c.float()).abs().max()) > 0.1           # sink and gate are not small here
    for back in (0, 31, 32, 500, 2047):
        peaked = q.clone()
        peaked[4] = (rows[4][2047 - back] * 8.0).to(torch.bfloat16).cuda()[None, :]
        far = torch.full((H,), -1e4, dtype=torch.float32).cuda()
        got = ops.latent_attention(peaked, cache, D, table, cu, kvl, 1, 1.0, max_kv_len=max(kv), sink=far)[4].float()
        assert float((got - rows[4][2047 - back].float().cuda()[None, :]).abs().max()) <= 0.05, back


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,width,E,top,groups,keep,more", [
    (1, 64, 12, 4, 4, 3, 1), (77, 48, 6, 2, 3, 2, 0), (300, 192, 72, 6, 8, 3, 1), (9, 33, 3, 1, 3, 1, 2),
    (50, 40, 8, 8, 4, 4, 1), (40, 32, 10, 3, 1, 1, 0), (33, 64, 130, 5, 65, 4, 1)])
def test_grouped_router_kernel(dtype, T, width, E, top, groups, keep, more):
    """The choice by corrected scores within the best groups against the plain function, from the logits
    the kernel's own product leaves (a close call between two experts is the product's rounding, not the
    choice's); `more` further rows of the router's matrix come back as they are."""
    from qwen3_from_scratch_amd import ops

    h, router = _rand((T, width), 1, dtype), _rand((E + more, width), 2, dtype, 0.5)
    correction = _rand((E,), 3, torch.float32, 0.7) - 0.3
    chosen, weights, rest = ops.moe_route(h, router, top, scoring="sigmoid_groups", correction=correction, groups=groups,
                                          keep=keep, experts=E)
    z = ops.linear(h, router, out_dtype=torch.float32).double().cpu()
    assert rest.shape == (T, more) and torch.equal(rest.cpu().double(), z[:, E:])
    at, share = plain.choose_experts(z[:, :E], correction.double().cpu(), top, groups, keep)
    choice = torch.sigmoid(z[:, :E]) + correction.double().cpu()
    for t in range(T):
        got, want = sorted(chosen[t].tolist()), sorted(at[t].tolist())
        if got != want:                                  # only where two scores all but tie
            odd = set(got) ^ set(want)
            assert max(choice[t, list(odd)]) - min(choice[t, list(odd)]) < 1e-5, t
        else:
            order = chosen[t].long().cpu()
            assert bool((choice[t, order][:-1] >= choice[t, order][1:] - 1e-6).all())       # in falling order
            assert torch.allclose(weights[t].double().cpu(), torch.sigmoid(z[t, order]), atol=2e-6)
    assert all(len(set(row)) == top for row in chosen.tolist())
    # every chosen expert lies in one of at most `keep` groups
    size = E // groups
    assert all(len({e // size for e in row}) <= keep for row in chosen.tolist())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,width,ff,E,top,shared", [(1, 64, 32, 7, 3, True), (50, 48, 24, 5, 2, False),
                                                      (333, 128, 96, 6, 3, True), (17, 40, 20, 4, 4, True),
                                                      (700, 96, 160, 3, 2, True), (900, 64, 64, 2, 2, False)])
def test_gated_experts_with_a_gated_shared_expert(dtype, T, width, ff, E, top, shared):
    import torch_ops
    from qwen3_from_scratch_amd import ops

    h = _rand((T, width), 1, dtype)
    gate_up, down = _rand((E, 2 * ff, width), 2, dtype, width ** -0.5), _rand((E, width, ff), 3, dtype, ff ** -0.5)
    chosen, weights = torch_ops.moe_route(h, _rand((E, width), 4, dtype), top, scoring="sigmoid")
    if T > 20:
        chosen[:, 0] = 1                                # one expert takes a row of every token, others few or none
    extra = _rand((T, width), 5, dtype) if shared else None
    logits = _rand((T, 3), 6, torch.float32, 2.0)
    for act in ("silu", "gelu_tanh"):
        for sg in ((logits[:, 1:2], None) if shared else (None,)):
            a = ops.moe_glu_experts(h, chosen, weights, gate_up, down, activation=act, shared=extra, shared_gate=sg)
            b = torch_ops.moe_glu_experts(h, chosen, weights, gate_up, down, activation=act, shared=extra, shared_gate=sg)
            assert float((a.float() - b.float()).abs().max()) <= (3e-5 if dtype == torch.float32 else 5e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_projection_norms_without_biases(dtype):
    """The attention layer's preparation (norms over whole projections, the rotation of pairs, the cache
    write) with no bias vector at all."""
    import torch_ops
    from qwen3_from_scratch_amd import ops

    T, H, G, d, dv, page = 21, 6, 2, 24, 40, 8
    rows = _rand((T, H * d + G * (d + dv)), 1, torch.float32, 2.0)
    qw, kw = _rand((H * d,), 2, torch.float32) + 1, _rand((G * d,), 3, torch.float32) + 1
    inv_freq = (torch.rand(5, generator=torch.Generator().manual_seed(4)) + 0.01).cuda()
    positions = torch.arange(100, 100 + T).int().cuda()
    seq = torch.zeros(T, dtype=torch.int32).cuda()
    table = torch.arange(20, dtype=torch.int32).flip(0)[None, :].contiguous().cuda()
    caches = [(torch.zeros((20, G, page, d), dtype=dtype).cuda(), torch.zeros((20, G, dv, page), dtype=dtype).cuda())
              for _ in range(2)]
    a = ops.softcap_prepare(rows, None, H, G, d, dv, qw, kw, 1e-5, inv_freq, positions, seq, dtype, table, *caches[0],
                            values_transposed=True)
    b = torch_ops.softcap_prepare(rows, None, H, G, d, dv, qw, kw, 1e-5, inv_freq, positions, seq, dtype, table, *caches[1],
                                  values_transposed=True)
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    assert float((a.float() - b.float()).abs().max()) <= tol
    for got, want in zip(caches[0], caches[1]):
        assert float((got.float() - want.float()).abs().max()) <= tol


# ---- the model on the GPU ----

@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logits_under_every_cutting(folders, dtype):
    folder = folders[dtype]
    requests = _requests(folder, lengths=(70, 9, 141, 330, 25, 2, 1))
    _, _, want = _truth(folder, requests)
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16,
                             max_tokens=max_live_tokens(steps, page=16), max_requests=4)
        assert _off(run_trace(runner, steps), want, dtype) <= 1.0, make.__name__
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.groups)


@pytest.mark.gpu
def test_layer_streams(tmp_path):
    """The float32 engine's residual stream behind every run of a layer against the plain one's."""
    folder = _write(tmp_path / "m", MIXED, peak=3.0)
    tokens = random_tokens(45, MIXED["vocab"], 4)
    config, w, _ = _truth(folder, {})
    streams = []
    plain.logits_of_sequence(config, w, tokens, streams)
    runner = load_runner(folder, dtype="float32", device="cuda", page_size=16, max_tokens=64, max_requests=1)
    seen = []
    runner.model.observer = lambda i, x, pending: seen.append((x.double() + pending.double()).cpu())
    runner.step([StepEntry("r", tokens, [])])
    assert len(seen) == len(streams)
    for got, want in zip(seen, streams):
        assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max())


@pytest.mark.gpu
def test_long_decoding_and_first_tokens(folders):
    """A request decoded token by token from its second token on, through graph replays and page ends,
    beside a request that is decoded from its very first."""
    for dtype in ("float32", "bfloat16"):
        folder = folders[dtype]
        vocab = load_model_config(folder).vocab
        requests = {"long": random_tokens(200, vocab, 7), "short": random_tokens(3, vocab, 8)}
        _, _, want = _truth(folder, requests)
        runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16, max_tokens=256, max_requests=2)
        steps = [([(rid, toks[:1], [0]) for rid, toks in requests.items()], [])]
        for i in range(1, 200):
            entries = [(rid, [toks[i]], [0]) for rid, toks in requests.items() if i < len(toks)]
            steps.append((entries, [rid for rid, toks in requests.items() if i == len(toks) - 1]))
        assert _off(run_trace(runner, steps), want, dtype) <= 1.0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_carries_the_last_row(tmp_path, dtype):
    """A prompt of 700 tokens in which one early token returns at the end, with weights made so that in
    both kinds of attention a query stands on the keys of its own token: the last rows then lean on a key
    hundreds of positions back, in a whole prompt, in portions whose ends fall anywhere, and decoded."""
    data = _every_expert(CORES) if dtype == "bfloat16" else CORES
    folder = _write(tmp_path / "m", data, std=0.15)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for i, layer in enumerate(data["layers"]):
        p, m = "l%d.mix." % i, layer["mixer"]
        if layer["type"] == "attention":                # queries of a group of heads are their key head's keys
            per = m["heads"] // m["kv_heads"]
            k = tensors[p + "k"].view(m["kv_heads"], m["dim"], -1)
            tensors[p + "q"] = k.repeat_interleave(per, dim=0).reshape(m["heads"] * m["dim"], -1).contiguous()
            tensors[p + "q.norm"] = (tensors[p + "k.norm"].view(m["kv_heads"], m["dim"]).repeat_interleave(per, dim=0)
                                     .reshape(-1).float() * 6.0).to(torch.bfloat16)
        else:                                           # the two latents and their per-head matrices coincide
            tensors[p + "dq"] = tensors[p + "dkv"][:m["q_rank"]].clone()
            tensors[p + "uq"] = tensors[p + "uk"][:, :m["q_rank"]].contiguous()
            tensors[p + "dq.norm"] = (tensors[p + "dkv.norm"][:m["q_rank"]].float() * 6.0).to(torch.bfloat16)
    save_file(tensors, path, metadata={"format": "pt"})
    vocab = data["vocab"]
    tokens = random_tokens(700, vocab, 31)
    rare = vocab - 1
    tokens = [t if t != rare else 0 for t in tokens]
    tokens[37] = rare
    tokens[-2] = rare
    config, w, want = _truth(folder, {"far": tokens})
    # the truth itself leans on the far key: without it the last rows change
    cut = plain.logits_of_sequence(config, w, tokens[38:])
    assert float((cut[-2] - want["far"][-2]).abs().max()) > 0.05 * float(want["far"][-2].std())
    for steps in (trace_whole({"far": tokens}), trace_tail_decoded({"far": tokens}, tail=4),
                  trace_portions({"far": tokens}, sizes=(130, 37, 2, 261, 64, 3))):
        runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16, max_tokens=704, max_requests=1)
        got = run_trace(runner, steps)
        worst = 0.0
        for p in range(690, 700):
            d = got[("far", p)].double() - want["far"][p]
            worst = max(worst, float((d - d.mean()).pow(2).mean().sqrt() / want["far"][p].std()))
        assert worst <= (5e-5 if dtype == "float32" else 5e-2)


@pytest.mark.gpu
def test_greedy_generation_through_the_engine(folders):
    for dtype in ("float32", "bfloat16"):
        folder = folders[dtype]
        requests = _requests(folder)
        config, w, _ = _truth(folder, {})
        engine = SyncEngine(path=folder, dtype=dtype, device="cuda", max_len=256, block_size=16, num_blocks=30,
                            max_num_seqs=3, max_num_tokens=48, chunked_prefill_size=32)
        prompts = [toks[:n] for toks, n in zip(requests.values(), (60, 9, 41, 2))]
        got = engine.generate_ids(prompts, max_new_tokens=8, temperature=0.0, ignore_eos=True)
        for prompt, new in zip(prompts, got):
            logits = plain.logits_of_sequence(config, w, prompt + new)
            for i, token in enumerate(new):
                row = logits[len(prompt) + i - 1]
                slack = 0.0 if dtype == "float32" else 0.02 * float(row.max() - row.min())
                assert float(row[token]) >= float(row.max()) - slack - 1e-9
        assert engine.runner.manager.num_free() == 30


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_program(folders, tmp_path, dtype):
    folder = folders[dtype]
    requests = _requests(folder)
    _, _, want = _truth(folder, requests)
    steps = trace_mixed(requests, seed=3)
    lines = [json.dumps({"step": i, "entries": [{"id": r, "tokens": t, "want": ws} for r, t, ws in entries],
                         "end": ends}) for i, (entries, ends) in enumerate(steps)]
    out = str(tmp_path / dtype)
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out,
         "--max-tokens", str(max_live_tokens(steps, page=64))],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done %d" % i for i in range(len(steps))]
    got, lengths = {}, {}
    for i, (entries, _) in enumerate(steps):
        wanted = [(r, lengths.get(r, 0) + p) for r, t, ws in entries for p in ws]
        for r, t, _ in entries:
            lengths[r] = lengths.get(r, 0) + len(t)
        if wanted:
            data = np.fromfile(os.path.join(out, "%d.f32" % i), dtype="<f4").reshape(len(wanted), -1)
            for key, row in zip(wanted, data):
                got[key] = torch.from_numpy(row.copy())
    assert _off(got, want, dtype) <= 1.0


@pytest.mark.gpu
def test_command_line_generates(tmp_path):
    folder = _write(tmp_path / "m", CORES, peak=3.0)
    config, w, _ = _truth(folder, {})
    prompt = random_tokens(50, CORES["vocab"], 12)
    proc = subprocess.run(
        [sys.executable, "-m", "qwen3_from_scratch_amd", "--path", folder, "--dtype", "float32", "--prompt_ids",
         ",".join(map(str, prompt)), "--max_new_tokens", "6", "--temperature", "0", "--ignore_eos", "--max_len", "128",
         "--block_size", "16", "--num_blocks", "16", "--max_num_seqs", "2"],
        capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [int(t) for t in proc.stdout.split()]
    seq = list(prompt)
    for _ in range(6):
        seq.append(int(torch.argmax(plain.logits_of_sequence(config, w, seq)[-1])))
    assert got == seq[len(prompt):]
