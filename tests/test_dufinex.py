"""The Dufinex architecture through the engine against tests/plain_dufinex.py: each mixer and each
feed-forward alone in a model of one layer, whole prompts against token-by-token decoding, portions
down to two tokens, mixed batches in which pages and state slots are used again, the residual behind
every layer, long decoding from the first token, keys far back and at page borders, a sink that
carries most of a softmax, and greedy generation through the engine, the command line and the replay
program. The configurations are made here; their sizes differ from layer to layer and avoid values
that hide a fault (one key head, one expert per token, as many key heads as heads in the delta rule,
equal key and value sizes everywhere, every layer with a feed-forward)."""

import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import plain_dufinex as plain
from helpers import max_live_tokens, random_tokens, run_trace, trace_mixed, trace_portions, trace_tail_decoded, trace_whole
from qwen3_from_scratch_amd.config import load_model_config
from qwen3_from_scratch_amd.config.dufinex_config import DufinexConfig
from qwen3_from_scratch_amd.config.model_config import ConfigError
from qwen3_from_scratch_amd.engine import StepEntry, SyncEngine, load_runner
from qwen3_from_scratch_amd.weights import write_random_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _attention(heads, kv_heads, dim, vdim, scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return ("attention", m)


def _delta(heads, kv_heads, dim, vdim, conv):
    return ("channel_delta", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv})


def _dense(ff, limit=2.0):
    return {"kind": "dense", "ff": ff, "limit": limit}


def _moe(experts, top, ff, limit=2.0):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def _layer(mixer, mlp=None):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def _model(vocab, width, layers, eps=1e-5, scale=2.5):
    return {"architecture": "Dufinex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": layers}


# every kind of layer, with either feed-forward and with none; two layers that read another's keys
MIXED = _model(131, 48, [
    _layer(_attention(6, 2, 24, 16, scale=0.3), _dense(40, 1.5)),
    _layer(_delta(4, 2, 12, 20, 3), _moe(6, 2, 24, 2.5)),
    _layer(_attention(6, 2, 24, 16, scale=0.25, kv_from=0)),
    _layer(_attention(4, 4, 8, 40), _moe(5, 1, 20)),
    _layer(_delta(2, 2, 40, 8, 5), _dense(56)),
    _layer(_attention(4, 4, 8, 40, kv_from=3), _dense(24, 0.7)),
])
# the delta rule first, attention last, a reader right behind its owner
PLAIN = _model(97, 64, [
    _layer(_delta(3, 1, 16, 24, 2)),
    _layer(_attention(4, 1, 16, 24), _moe(4, 4, 16)),
    _layer(_attention(4, 1, 16, 24, kv_from=1), _dense(48)),
], eps=1e-6, scale=1.0)
# sizes in steps of 64: the matrix-core attention kernels in bfloat16, the experts' matrix-core kernels
WIDE = _model(257, 128, [
    _layer(_attention(8, 2, 64, 64, scale=0.125), _moe(8, 2, 64)),
    _layer(_delta(4, 2, 64, 64, 4), _dense(192)),
    _layer(_attention(8, 2, 64, 64, scale=0.2, kv_from=0), _dense(128)),
    _layer(_attention(4, 1, 128, 128), _moe(16, 1, 96)),
    _layer(_delta(2, 2, 128, 128, 4)),
], scale=3.0)
# odd sizes everywhere
ODD = _model(53, 40, [
    _layer(_attention(3, 3, 10, 6), _moe(3, 3, 10, 1.2)),
    _layer(_delta(3, 1, 20, 12, 2), _dense(28)),
    _layer(_attention(3, 3, 10, 6, kv_from=0), _moe(7, 2, 12)),
], scale=0.7)
# sizes at the kernels' ends: thirty-two query heads on one key head, keys of 256 in the delta rule with values that
# are no multiple of its sixteen columns, eight taps, many experts with several a token
EDGES = _model(70, 64, [
    _layer(_attention(32, 1, 8, 4), _moe(70, 4, 8)),
    _layer(_delta(2, 1, 256, 36, 8), _dense(24)),
    _layer(_attention(2, 1, 64, 64), _dense(24)),
    _layer(_delta(1, 1, 4, 70, 2)),
    _layer(_attention(32, 1, 8, 4, kv_from=0)),
], eps=1e-6)
CONFIGS = {"mixed": MIXED, "plain": PLAIN, "wide": WIDE, "odd": ODD, "edges": EDGES}
# one layer of each kind alone: a mixer without a feed-forward, or a feed-forward behind the cheapest mixer
ALONE = {
    "attention": _model(61, 32, [_layer(_attention(4, 2, 12, 20))]),
    "channel_delta": _model(61, 32, [_layer(_delta(4, 2, 12, 10, 4))]),
    "dense": _model(61, 32, [_layer(_attention(1, 1, 8, 8), _dense(40, 1.0))]),
    "moe": _model(61, 32, [_layer(_attention(1, 1, 8, 8), _moe(6, 3, 12, 1.0))]),
}


def _write(folder, data, seed=5, peak=None, std=0.2, ranks=None):
    """Random weights of the configuration with what a trained model has and small random numbers
    hide: sinks of a size that carries a good part of a softmax, decays between nothing and all,
    biases that matter and, with `peak`, query norms so large that a softmax stands on few keys.
    `ranks`: other middle sizes for the delta rule's two narrow products."""
    folder = str(folder)
    write_random_model(folder, DufinexConfig.from_dict(data), seed=seed, std=std, norm_jitter=0.3)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(seed)

    def normal(shape, sigma, mean=0.0):
        return (mean + sigma * torch.randn(tuple(shape), generator=g)).to(torch.bfloat16)

    for key in sorted(tensors):
        t = tensors[key]
        if key.endswith(".sink"):
            tensors[key] = normal(t.shape, 1.5, 1.0)
        elif key.endswith(".A_log") or key.endswith(".dt_bias"):
            tensors[key] = normal(t.shape, 1.0)
        elif key.endswith(".b") and t.dim() == 1:
            tensors[key] = normal(t.shape, 0.5)
        elif peak and key.endswith("q.norm"):
            tensors[key] = (t.float() * peak).to(torch.bfloat16)
        elif key == "embed":
            tensors[key] = (t.float() * (0.2 / std)).to(torch.bfloat16)      # logits that span a few units
        elif ranks and key.rsplit(".", 1)[-1] in ("a1", "g1", "a2", "g2"):
            r = ranks[0] if key.endswith(("a1", "a2")) else ranks[1]
            tensors[key] = normal((r, t.shape[1]) if key.endswith("1") else (t.shape[0], r), std)
    save_file(tensors, path, metadata={"format": "pt"})
    return folder


# In bfloat16 the choice among experts of random weights is a close call for some token of every prompt (the gap
# between two neighbouring scores and the rounding of the router's input shrink and grow together, whatever the
# weights' size), and the plain implementation, which rounds nothing, then chooses otherwise. The bfloat16 folders
# therefore give every token all experts of a layer: the experts' kernels run as they do otherwise, and the choice
# itself is compared in float32 here and in bfloat16 against its twin in the kernels' tests.
def _all_chosen(data):
    data = copy.deepcopy(data)
    for layer in data["layers"]:
        if layer["mlp"] and layer["mlp"]["kind"] == "moe":
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return data


ROUNDED = {name: _all_chosen(data) for name, data in CONFIGS.items()}
ROUNDED["edges"]["layers"][0]["mlp"]["router"]["experts"] = ROUNDED["edges"]["layers"][0]["mlp"]["router"]["top"] = 9
# and unit vectors of four numbers, which carry a rounding of their inputs on many times larger, are left to float32
del ROUNDED["edges"]["layers"][3]
# how the float32 folders are written: large weights and peaked queries
SHARP = {name: dict(peak=3.0) for name in CONFIGS}
SHARP["plain"] = dict(peak=3.0, ranks=(5, 9))
SHARP["edges"] = dict(peak=2.0, std=0.1)


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def folder(request, tmp_path_factory):
    return _write(tmp_path_factory.mktemp(request.param), CONFIGS[request.param], **SHARP[request.param])


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def folders(request, tmp_path_factory):
    """{dtype: folder}. float32 gets large weights and peaked queries, where a key, a tap, a sink or a
    state left out stands far above float32's rounding; bfloat16 gets weights under which its own
    rounding, which the recurrences carry on, stays well below the bound."""
    return {"float32": _write(tmp_path_factory.mktemp(request.param), CONFIGS[request.param], **SHARP[request.param]),
            "bfloat16": _write(tmp_path_factory.mktemp(request.param + "_b"), ROUNDED[request.param],
                               std=0.06)}


def _truth(folder, requests):
    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    w = load_file(os.path.join(folder, "model.safetensors"))
    return config, w, {rid: plain.forward(config, w, toks) for rid, toks in requests.items()}


def _requests(folder, lengths=(70, 9, 41, 130, 25, 2, 1)):
    vocab = load_model_config(folder).vocab
    return {"s%d" % i: random_tokens(n, vocab, 260 + i) for i, n in enumerate(lengths)}


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


def _all_cuttings(folder, requests, want, dtype, device, page):
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype=dtype, device=device, page_size=page,
                             max_tokens=max_live_tokens(steps, page=page), max_requests=4)
        assert _off(run_trace(runner, steps), want, dtype) <= 1.0, make.__name__
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.groups)


# ---- configuration, weights, cache ----

def test_config_is_read_by_its_own_keys_and_written_back(folder):
    config = load_model_config(folder)
    with open(os.path.join(folder, "config.json")) as fh:
        data = json.load(fh)
    assert config.architecture == "Dufinex" and config.to_dict() == data
    assert config.vocab == data["vocab"] and config.width == data["width"]
    assert config.eps == data["norm"]["eps"] and config.embedding_scale == data["embedding"]["scale"]
    assert [layer.type for layer in config.layers] == [layer["type"] for layer in data["layers"]]
    assert [layer.mlp_kind for layer in config.layers] == [(layer["mlp"] or {}).get("kind") for layer in data["layers"]]


@pytest.mark.parametrize("change,word", [
    (lambda d: d["layers"][0].__setitem__("type", "convolution"), "type"),
    (lambda d: d["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda d: d["layers"][0]["mixer"].__setitem__("kv_heads", 4), "kv_heads"),
    (lambda d: d["layers"][1]["mixer"].pop("conv"), "conv"),
    (lambda d: d["layers"][1]["mlp"]["router"].__setitem__("top", 9), "top"),
    (lambda d: d["layers"][0]["mlp"].__setitem__("limit", 0.0), "limit"),
    (lambda d: d["layers"][0]["mlp"].__setitem__("kind", "wide"), "kind"),
    (lambda d: d["layers"][2]["mixer"].__setitem__("kv_from", 1), "kv_from"),
    (lambda d: d["layers"][2]["mixer"].__setitem__("kv_from", 2), "kv_from"),
    (lambda d: d["layers"][5]["mixer"].__setitem__("kv_from", 0), "kv_from"),
    (lambda d: d.pop("embedding"), "embedding"),
    (lambda d: d["norm"].pop("eps"), "eps"),
])
def test_config_errors_name_the_key(change, word):
    data = copy.deepcopy(MIXED)
    change(data)
    with pytest.raises(ConfigError, match=word):
        DufinexConfig.from_dict(data)


def test_cache_planes_hold_what_each_mixer_keeps(cpu_ops, tmp_path):
    """Attention layers with keys of their own own a plane of pages, the delta rule a state of its own
    size (the convolutions' tails and S); a layer that reads another's keys has no plane but that one's."""
    runner = load_runner(_write(tmp_path / "m", MIXED), dtype="float32", device="cpu", page_size=8, max_tokens=128,
                         max_requests=3)
    model = runner.model
    assert model.plane_of_step == [0, 1, 0, 2, 3, 2]
    needs = model.plane_needs
    assert [bool(n.paged) for n in needs] == [True, False, True, False]
    assert [n.state_shape[0] for n in needs if n.has_state] == [2 * (48 + 80) + 4 * 12 * 20, 4 * (160 + 16) + 2 * 40 * 8]
    assert len(runner.manager.groups) == 2 and len(runner.manager.state_groups) == 2
    assert not runner.manager.prefix_cache and model.graph_safe()
    names = set(model.tensors())
    assert "l0.mix.k" in names and "l2.mix.k" not in names and "l2.mix.k.norm" not in names and "l2.mix.sink" in names
    assert "l2.norm2" not in names and "l1.mlp.e5.gate" in names and "l0.mlp.down.b" in names


def test_the_narrow_products_take_their_middle_from_the_tensors(cpu_ops, tmp_path):
    """No configuration key names the middle size of the decays' and the gate's products: whatever the
    stored tensors have is loaded, also two different sizes; halves that disagree are refused."""
    folder = _write(tmp_path / "m", ALONE["channel_delta"], ranks=(3, 11))
    requests = _requests(folder, lengths=(20, 3))
    _, w, want = _truth(folder, requests)
    assert w["l0.mix.a1"].shape[0] == 3 and w["l0.mix.g2"].shape[1] == 11
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=64, max_requests=2)
    assert _off(run_trace(runner, trace_whole(requests)), want, "float32") <= 1.0
    w["l0.mix.a2"] = w["l0.mix.a2"][:, :2].contiguous()
    save_file(w, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    with pytest.raises(ValueError, match="middle"):
        load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=64, max_requests=2)


# ---- what the plain implementation is sensitive to (so that a comparison with it means something) ----

def test_a_mechanism_that_is_left_out_shows(tmp_path):
    """With these weights the sink, the gates, the embedding's scale, the last bias, the clamp, the
    decays and the other layer's keys each move the logits by far more than rounding: a model that
    ignored one of them would not pass the comparisons below."""
    folder = _write(tmp_path / "m", MIXED, peak=3.0)
    tokens = random_tokens(40, MIXED["vocab"], 3)
    config, w, _ = _truth(folder, {})
    base = plain.forward(config, w, tokens)
    spread = float(base.std())

    def moved(**changes):
        other = dict(w)
        other.update(changes)
        return float((plain.forward(config, other, tokens) - base).abs().max()) / spread

    assert moved(**{"l0.mix.sink": w["l0.mix.sink"] - 30.0}) > 0.05                  # no sink at all
    assert moved(**{"l2.mix.sink": w["l2.mix.sink"] - 30.0}) > 0.05
    assert moved(**{"l0.mix.g": w["l0.mix.g"] * 0}) > 0.05                           # every gate one half
    assert moved(**{"l0.mlp.down.b": w["l0.mlp.down.b"] * 0}) > 0.05
    assert moved(**{"l4.mix.A_log": w["l4.mix.A_log"] - 30.0}) > 0.05                # no decay
    assert moved(**{"l1.mix.dt_bias": w["l1.mix.dt_bias"] + 3.0}) > 0.05
    assert moved(**{"l1.mix.q.conv": w["l1.mix.q.conv"].flip(1)}) > 0.05             # the taps' order
    assert moved(**{"l0.mix.k": w["l0.mix.k"].flip(0)}) > 0.05                       # layer 2 reads layer 0's keys
    wider = copy.deepcopy(config)
    wider["layers"][0]["mlp"]["limit"] = 50.0
    assert float((plain.forward(wider, w, tokens) - base).abs().max()) / spread > 0.05
    unscaled = copy.deepcopy(config)
    unscaled["embedding"]["scale"] = 1.0
    assert float((plain.forward(unscaled, w, tokens) - base).abs().max()) / spread > 0.05
    renormed = dict(w)
    for e in range(6):                                                               # the weight on the input, not the output
        renormed["l1.mlp.e%d.gate" % e] = w["l1.mlp.e%d.gate" % e] * 0.5
    assert moved(**{k: v for k, v in renormed.items() if ".mlp.e" in k}) > 0.02


# ---- each mixer and feed-forward alone, and the stream behind every layer ----

@pytest.mark.parametrize("kind", sorted(ALONE))
def test_one_part_alone_on_the_host(cpu_ops, tmp_path, kind):
    folder = _write(tmp_path / kind, ALONE[kind], seed=9, peak=2.0)
    requests = _requests(folder, lengths=(45, 3, 1, 20))
    _, _, want = _truth(folder, requests)
    _all_cuttings(folder, requests, want, "float32", "cpu", 8)


def _stream_behind(folder, tokens, device, dtype):
    runner = load_runner(folder, dtype=dtype, device=device, page_size=8 if device == "cpu" else 16, max_tokens=64,
                         max_requests=1)
    seen = []

    def observe(i, x, pending):
        a = pending.values.double().cpu()
        if pending.values_bias is not None:
            a = a + pending.values_bias.double().cpu()
        a = a / torch.sqrt((a * a).mean(dim=-1, keepdim=True) + pending.eps) * pending.weight.double().cpu()
        seen.append(x.double().cpu() + a)

    runner.model.observer = observe
    runner.step([StepEntry("r", tokens, [])])
    return seen


@pytest.mark.parametrize("name", ["mixed", "plain", "odd", "edges"])
def test_stream_behind_every_layer_on_the_host(cpu_ops, tmp_path, name):
    """The residual behind every layer, what the last sublayer still owes it included."""
    folder = _write(tmp_path / "m", CONFIGS[name])
    tokens = random_tokens(37, CONFIGS[name]["vocab"], 4)
    config, w, _ = _truth(folder, {})
    want = []
    plain.forward(config, w, tokens, want)
    seen = _stream_behind(folder, tokens, "cpu", "float32")
    assert len(seen) == len(want) == len(config["layers"])
    for got, truth in zip(seen, want):
        assert float((got - truth).abs().max()) <= 2e-5 * float(truth.abs().max())


# ---- the whole model ----

def test_logits_on_the_host_under_every_cutting(cpu_ops, folder):
    requests = _requests(folder)
    _, _, want = _truth(folder, requests)
    _all_cuttings(folder, requests, want, "float32", "cpu", 8)


def test_a_slot_that_is_used_again_starts_from_nothing(cpu_ops, tmp_path):
    """One state slot and a pool of a few pages: every request takes the slot and the pages the
    last one left, and must not see what that one kept there."""
    folder = _write(tmp_path / "m", MIXED)
    requests = _requests(folder, lengths=(33, 40, 5, 17))
    _, _, want = _truth(folder, requests)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=40, max_requests=1)
    got = run_trace(runner, trace_portions(requests, sizes=(7, 2, 13)))
    assert _off(got, want, "float32") <= 1.0


def test_greedy_generation_through_the_engine_on_the_host(cpu_ops, folder):
    requests = _requests(folder)
    config, w, _ = _truth(folder, {})
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=256, block_size=8, num_blocks=60,
                        max_num_seqs=3, max_num_tokens=24, chunked_prefill_size=16)
    prompts = [toks[:n] for toks, n in zip(requests.values(), (30, 9, 41, 2))]
    got = engine.generate_ids(prompts, max_new_tokens=5, temperature=0.0, ignore_eos=True)
    for prompt, new in zip(prompts, got):
        assert new == plain.greedy(config, w, prompt, 5)
    assert engine.runner.manager.num_free() == 60


def test_a_preempted_request_builds_its_state_again_on_the_host(cpu_ops, tmp_path):
    """Too few pages for three requests at once: one is preempted, gives pages and state slot back, and
    later goes through its prompt and its generated tokens again from an empty state. What it generates
    is what it would have generated alone."""
    folder = _write(tmp_path / "m", MIXED, peak=3.0)
    config, w, _ = _truth(folder, {})
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=128, block_size=8, num_blocks=12,
                        max_num_seqs=3, max_num_tokens=24, chunked_prefill_size=16)
    prompts = [random_tokens(n, MIXED["vocab"], 300 + n) for n in (30, 9, 41)]
    requests = [engine.add_request(p, engine.default_params(10, temperature=0.0, ignore_eos=True)) for p in prompts]
    steps = 0
    while engine.scheduler.has_work() and steps < 500:
        engine.step()
        engine.runner.manager.audit()
        steps += 1
    assert not engine.scheduler.has_work() and sum(r.preemptions for r in requests) >= 1
    for prompt, request in zip(prompts, requests):
        assert list(request.generated) == plain.greedy(config, w, prompt, 10)
    assert engine.runner.manager.num_free() == 12


def test_command_line_writes_a_folder_from_the_nested_config(tmp_path):
    from qwen3_from_scratch_amd.engine.cli import main

    source = tmp_path / "config.json"
    source.write_text(json.dumps(PLAIN))
    assert main(["--write_random", str(tmp_path / "m"), "--from_config", str(source), "--seed", "3"]) == 0
    assert load_model_config(str(tmp_path / "m")).to_dict() == PLAIN
    names = set(load_file(str(tmp_path / "m" / "model.safetensors")))
    assert "l0.mix.v.conv" in names and "l2.mix.v" not in names and "l0.norm2" not in names


# ---- the model on the GPU ----

@pytest.mark.gpu
@pytest.mark.parametrize("kind", sorted(ALONE))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_part_alone(tmp_path, kind, dtype):
    folder = (_write(tmp_path / kind, ALONE[kind], seed=9, peak=2.0) if dtype == "float32"
              else _write(tmp_path / kind, _all_chosen(ALONE[kind]), seed=9, std=0.06))
    requests = _requests(folder, lengths=(45, 3, 1, 200))
    _, _, want = _truth(folder, requests)
    _all_cuttings(folder, requests, want, dtype, "cuda", 16)


ONES = _model(61, 32, [_layer(_delta(4, 2, 12, 10, 1)), _layer(_delta(2, 1, 8, 10, 3), _moe(1, 1, 8))])


def test_sizes_of_one_on_the_host(cpu_ops, tmp_path):
    """A convolution of one tap (no tail in the state), one expert, and a model without attention (no pages at all)."""
    folder = _write(tmp_path / "m", ONES)
    requests = _requests(folder, lengths=(20, 3, 1))
    _, _, want = _truth(folder, requests)
    _all_cuttings(folder, requests, want, "float32", "cpu", 8)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_of_one(tmp_path, dtype):
    folder = _write(tmp_path / "m", ONES, **(dict(peak=2.0) if dtype == "float32" else dict(std=0.06)))
    requests = _requests(folder, lengths=(45, 3, 1, 100))
    _, _, want = _truth(folder, requests)
    _all_cuttings(folder, requests, want, dtype, "cuda", 16)


@pytest.mark.gpu
def test_stream_behind_every_layer(tmp_path):
    folder = _write(tmp_path / "m", WIDE)
    tokens = random_tokens(50, WIDE["vocab"], 4)
    config, w, _ = _truth(folder, {})
    want = []
    plain.forward(config, w, tokens, want)
    for got, truth in zip(_stream_behind(folder, tokens, "cuda", "float32"), want):
        assert float((got - truth).abs().max()) <= 5e-5 * float(truth.abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logits_under_every_cutting(folders, dtype):
    folder = folders[dtype]
    requests = _requests(folder, lengths=(70, 9, 141, 330, 25, 2, 1))
    _, _, want = _truth(folder, requests)
    _all_cuttings(folder, requests, want, dtype, "cuda", 16)


@pytest.mark.gpu
def test_long_decoding_and_first_tokens(folders):
    """A request decoded token by token from its second token on, through graph replays and page
    ends, beside a request that is decoded from its very first and one that joins later into a slot
    that was used before."""
    for dtype in ("float32", "bfloat16"):
        folder = folders[dtype]
        vocab = load_model_config(folder).vocab
        requests = {"long": random_tokens(200, vocab, 7), "short": random_tokens(3, vocab, 8),
                    "late": random_tokens(150, vocab, 10)}
        _, _, want = _truth(folder, requests)
        runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16, max_tokens=416, max_requests=2)
        steps = []
        for i in range(200):
            entries = [(rid, [requests[rid][i]], [0]) for rid in ("long", "short") if i < len(requests[rid])]
            if i >= 50:
                entries.append(("late", [requests["late"][i - 50]], [0]))
            steps.append((entries, [rid for rid, _, _ in entries
                                    if (i - 50 if rid == "late" else i) == len(requests[rid]) - 1]))
        assert _off(run_trace(runner, steps), want, dtype) <= 1.0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_far_back_carries_the_softmax(tmp_path, dtype):
    """A prompt of some hundred tokens with weights under which a query finds the key of its own token:
    queries and keys are the same projection. Two tokens differ only in a coordinate that queries and
    keys do not see and values do; one stands early in the prompt, once, the other at its end. The
    last rows, in the prompt and decoded, then have two scores far above all others, their own and
    the early key's, hundreds of positions and dozens of pages back, and the early token's value is
    half of what attention returns: a table entry, a split or a tile that loses it gives other logits."""
    data = _model(90, 128, [_layer(_attention(4, 2, 64, 64, scale=0.05), _dense(64)),
                            _layer(_attention(4, 2, 64, 64, scale=0.05, kv_from=0))], scale=1.0)
    folder = _write(tmp_path / "m", data, std=0.1)
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    w["l0.mix.q"][:, 0] = 0.0                                          # coordinate 0: unseen by queries and keys
    w["l0.mix.k"] = w["l0.mix.q"].view(2, 2, 64, 128)[:, 0].reshape(128, 128).clone()   # a key head = its first query head
    w["l1.mix.q"] = w["l0.mix.q"].clone()
    w["l0.mix.v"][:, 0] = 1.0                                          # and seen by every value
    for name in ("l0.mix.q.norm", "l0.mix.k.norm", "l1.mix.q.norm"):
        w[name] = torch.full_like(w[name], 2.0)
    w["embed"][88] = w["embed"][89]
    w["embed"][88, 0] += 4.0
    save_file(w, path, metadata={"format": "pt"})
    tokens = random_tokens(700, 88, 5)                                 # tokens 88 and 89 nowhere else
    tokens[5] = 88
    tokens += [89, 3, 89, 89]
    config, w, _ = _truth(folder, {})
    want = plain.forward(config, w, tokens)
    without = plain.forward(config, w, tokens[:5] + [7] + tokens[6:])
    for p in (700, 702, 703):
        assert float((want[p] - without[p]).abs().max()) > 0.2 * float(want[p].std())      # the early key matters
    runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16, max_tokens=768, max_requests=1)
    got = {}
    logits = runner.step([StepEntry("r", tokens[:701], [699, 700])]).float().cpu()
    got[("r", 699)], got[("r", 700)] = logits[0], logits[1]
    for i in range(701, len(tokens)):
        got[("r", i)] = runner.step([StepEntry("r", [tokens[i]], [0])]).float().cpu()[0]
    worst = 0.0
    for (_, p), row in got.items():
        d = row.double() - want[p]
        worst = max(worst, float((d - d.mean()).pow(2).mean().sqrt() / want[p].std()) / (5e-5 if dtype == "float32" else 5e-2))
    assert worst <= 1.0


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
            logits = plain.forward(config, w, prompt + new)
            for i, token in enumerate(new):
                row = logits[len(prompt) + i - 1]
                slack = 1e-4 if dtype == "float32" else 0.02 * float(row.max() - row.min())
                assert float(row[token]) >= float(row.max()) - slack
        assert engine.runner.manager.num_free() == 30


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_program(tmp_path, dtype):
    folder = (_write(tmp_path / "m", MIXED, peak=3.0) if dtype == "float32"
              else _write(tmp_path / "m", ROUNDED["mixed"], std=0.06))
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
    folder = _write(tmp_path / "m", WIDE, peak=3.0)
    config, w, _ = _truth(folder, {})
    prompt = random_tokens(50, WIDE["vocab"], 12)
    proc = subprocess.run(
        [sys.executable, "-m", "qwen3_from_scratch_amd", "--path", folder, "--dtype", "float32", "--prompt_ids",
         ",".join(map(str, prompt)), "--max_new_tokens", "6", "--temperature", "0", "--ignore_eos", "--max_len", "128",
         "--block_size", "16", "--num_blocks", "16", "--max_num_seqs", "2"],
        capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == plain.greedy(config, w, prompt, 6)
