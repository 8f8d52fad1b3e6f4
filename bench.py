"""Decode and prefill throughput of the Qwen3-8B-shaped model on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
                    [--shape 8b|14b|32b|0.6b] [--prompt P] [--context C]
                    [--workload decode|continuous|served|prefix|products|kodisun|surasun|dufinex|fidevik]

Random bfloat16 weights, uniform-random prompts of 2,048 tokens, greedy decoding
through the engine's own step loop (scheduler, step function, sampling). A
"step" is one decode step of the whole batch. One JSON line is printed:
`value` is decoded tokens per second at the default batch; `prefill` is one
2,048-token prompt in one step (the median of three); `roofline` prices the decode step against HBM
bandwidth, the published peak and the rate a plain read kernel reaches on this GPU (`measured_peak`);
`points` holds decoding at batch 1 and 64 and a prompt of 8,192 tokens in one step (tokens a second), `points_roofline` their fractions of the published peaks. The default run is the
8B shape with prompts of 2,048 in a context of 8,192; `--shape`, `--prompt` and
`--context` move the decode measurement to the larger shapes and to longer
contexts (the prefill measurement stays at 2,048 tokens).
"""

import argparse
import json
import sys
import time

PEAK_HBM = 8.0e12            # bytes/s, MI355X HBM3E
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}   # dense MFMA peaks

QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=4096, hidden_act="silu",
                num_hidden_layers=36, max_position_embeddings=40960, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, intermediate_size=12288, rms_norm_eps=1e-6,
                rope_theta=1000000.0, tie_word_embeddings=False)
QWEN3_14B = dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=40, num_attention_heads=40, intermediate_size=17408)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=64, num_attention_heads=64, intermediate_size=25600)
# the model the reference's own measurements are of, by the sizes its configuration defaults to
# (src/qwen3_from_scratch/factory/config.py:19-42)
QWEN3_06B = dict(QWEN3_8B, hidden_size=1024, num_hidden_layers=28, num_attention_heads=16, intermediate_size=4096,
                 rms_norm_eps=1e-5, rope_theta=100000.0)
SHAPES = {"8b": ("Qwen3-8B", QWEN3_8B), "14b": ("Qwen3-14B", QWEN3_14B), "32b": ("Qwen3-32B", QWEN3_32B),
          "0.6b": ("Qwen3-0.6B", QWEN3_06B)}
PREFILL = 2048
LONG_PREFILL = 8192          # a second prompt length, reported under `points`
BLOCK = 16


def layer_params(c):
    qkv = (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim * c.hidden_size
    o = c.hidden_size * c.num_attention_heads * c.head_dim
    mlp = 3 * c.hidden_size * c.intermediate_size
    return qkv + o + mlp


def decode_bytes(c, contexts, itemsize):
    """Bytes one decode step has to read: every weight it uses once, and the
    keys and values of the live requests."""
    weights = (c.num_hidden_layers * layer_params(c) + c.vocab_size * c.hidden_size) * itemsize
    kv_per_token = 2 * c.num_hidden_layers * c.num_key_value_heads * c.head_dim * itemsize
    return weights + kv_per_token * sum(contexts)


def prefill_flops(c, tokens):
    gemm = 2.0 * tokens * c.num_hidden_layers * layer_params(c) + 2.0 * c.vocab_size * c.hidden_size
    attn = 4.0 * (tokens * (tokens + 1) / 2) * c.head_dim * c.num_attention_heads * c.num_hidden_layers
    return gemm + attn


def _model_tensors(model):
    """Every tensor a loaded model keeps on the device, each once."""
    import torch

    seen, found, stack = set(), [], [model]
    while stack:
        obj = stack.pop()
        if id(obj) in seen:
            continue
        seen.add(id(obj))
        if isinstance(obj, torch.Tensor):
            if obj.is_cuda and obj.untyped_storage().data_ptr() not in seen:
                seen.add(obj.untyped_storage().data_ptr())
                found.append(obj)
        elif isinstance(obj, (list, tuple)):
            stack.extend(obj)
        elif isinstance(obj, dict):
            stack.extend(obj.values())
        elif hasattr(obj, "__dict__") and type(obj).__module__.startswith("qwen3_from_scratch_amd"):
            stack.extend(vars(obj).values())
    return found


def continuous(args, config, model, shape_name, gen, sync):
    """64 requests admitted at once and served by continuous batching: prompt lengths uniform in
    [128, 4096], generated tokens uniform in [64, 512], prompts cut into portions of 512 beside
    the decoding requests, a budget of 576 tokens a step. Run twice; the second run (graphs
    captured, library kernels chosen) is the one reported."""
    import random

    import torch

    from qwen3_from_scratch_amd.engine import SyncEngine

    requests, portion, context = 64, 512, 8192
    rng = random.Random(0)
    sizes = [(rng.randint(128, 4096), rng.randint(64, 512)) for _ in range(requests)]
    engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context, block_size=BLOCK,
                        num_blocks=requests * context // BLOCK // 2, max_num_seqs=requests,
                        max_num_tokens=portion + requests, chunked_prefill_size=portion,
                        enable_prefix_cache=False)         # the second pass computes every prompt again
    for _ in range(2):
        for prompt, generated in sizes:
            engine.add_request(torch.randint(0, config.vocab_size, (prompt,), generator=gen).tolist(),
                               engine.default_params(generated, temperature=0.0, ignore_eos=True))
        sync()
        t0 = time.perf_counter()
        steps = 0
        while engine.scheduler.has_work():
            engine.step()
            steps += 1
        sync()
        seconds = time.perf_counter() - t0
    tokens_in, tokens_out = sum(p for p, _ in sizes), sum(g for _, g in sizes)
    print(json.dumps({
        "metric": "continuous batching, tokens/s in and out, %s %s"
                  % (shape_name, "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round((tokens_in + tokens_out) / seconds, 1), "unit": "tokens/s", "n_gpus": 1,
        "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "seconds": round(seconds, 3), "steps": steps, "generated_tokens_per_s": round(tokens_out / seconds, 1),
        "config": {"model": "%s-shaped, random weights N(0, 0.02)" % shape_name, "requests": requests,
                   "prompt_tokens": tokens_in, "generated_tokens": tokens_out, "prefill_portion": portion,
                   "step_token_budget": portion + requests, "context_len": context, "kv_block_size": BLOCK,
                   "layers": config.num_hidden_layers, "sampling": "greedy"},
    }))
    return 0


def served(args, config, model, shape_name, gen, sync):
    """The load of the reference's own benchmark (docs/benchmark.md:40-68, exps/run_eval_scope_bench.sh):
    200 requests, 20 in flight at any time, 512 prompt tokens and 512 generated tokens each (end-of-sequence
    ignored), a new request admitted when one ends; without its HTTP server: requests enter and tokens leave
    through the engine's own loop. Sampling as the engine defaults to (temperature 1.0, as the reference).
    Run twice; the second run is the one reported."""
    import torch

    from qwen3_from_scratch_amd.engine import SyncEngine
    from qwen3_from_scratch_amd.engine.scheduler import RequestStatus

    number, parallel, prompt_tokens, new_tokens = 200, 20, 512, 512
    context = prompt_tokens + new_tokens
    engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context, block_size=BLOCK,
                        num_blocks=(parallel + 1) * (context // BLOCK + 1), max_num_seqs=parallel,
                        max_num_tokens=512 + parallel, chunked_prefill_size=512, enable_prefix_cache=False)
    for _ in range(2):
        prompts = [torch.randint(0, config.vocab_size, (prompt_tokens,), generator=gen).tolist() for _ in range(number)]
        admitted, first, ended, live, queued = {}, {}, {}, {}, 0
        sync()
        t0 = time.perf_counter()
        steps = 0
        while queued < number or live:
            while queued < number and len(live) < parallel:
                request = engine.add_request(prompts[queued], engine.default_params(new_tokens, ignore_eos=True))
                admitted[request.request_id] = time.perf_counter()
                live[request.request_id] = request
                queued += 1
            engine.step()
            steps += 1
            now = time.perf_counter()
            for rid, request in list(live.items()):
                if request.generated and rid not in first:
                    first[rid] = now
                if request.status == RequestStatus.FINISHED:
                    ended[rid] = now
                    del live[rid]
        sync()
        seconds = time.perf_counter() - t0
    latency = [ended[r] - admitted[r] for r in ended]
    ttft = [first[r] - admitted[r] for r in ended]
    tpot = [(ended[r] - first[r]) / (new_tokens - 1) for r in ended]
    mean = lambda xs: sum(xs) / len(xs)
    print(json.dumps({
        "metric": "output tokens/s, %d requests, %d in flight, %d in + %d out, %s %s"
                  % (number, parallel, prompt_tokens, new_tokens, shape_name,
                     "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round(number * new_tokens / seconds, 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic", "seconds": round(seconds, 3),
        "steps": steps, "requests_per_s": round(number / seconds, 2), "latency_avg_s": round(mean(latency), 3),
        "ttft_avg_ms": round(1e3 * mean(ttft), 1), "tpot_avg_ms": round(1e3 * mean(tpot), 2),
        "config": {"model": "%s-shaped, random weights N(0, 0.02)" % shape_name, "requests": number,
                   "in_flight": parallel, "prompt_tokens": prompt_tokens, "generated_tokens": new_tokens,
                   "prefill_portion": 512, "kv_block_size": BLOCK, "layers": config.num_hidden_layers,
                   "sampling": "temperature 1.0", "server": "none: the engine's own loop"},
    }))
    return 0


def products(args, config, shape_name, sync):
    """The four products of a layer at 2,048, 576 and 64 rows: the kernel that the contest
    chose (library candidates and the hand-written tiled kernel, timed with cold caches) beside
    every tile shape of the hand-written kernel, microseconds with the weight coming from
    memory (as many weights in turn as exceed the last-level cache; the calls are captured in a
    graph, so the time is the GPU's)."""
    import torch

    from qwen3_from_scratch_amd import ops

    c = config
    shapes = [("qkv", (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim, c.hidden_size),
              ("o", c.hidden_size, c.num_attention_heads * c.head_dim),
              ("gate_up", 2 * c.intermediate_size, c.hidden_size), ("down", c.hidden_size, c.intermediate_size)]

    def timed(f, calls, replays=5):
        """Microseconds of one call on the GPU: `calls` of them captured in a graph (no host
        time between them), the graph replayed."""
        for _ in range(2):
            f()                                  # sizes are met, and timed, outside the capture
        sync()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for _ in range(calls):
                    f()
        torch.cuda.current_stream().wait_stream(side)
        graph.replay()
        sync()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        sync()
        return (time.perf_counter() - t0) / (replays * calls) * 1e6

    rows = {}
    for M in [int(m) for m in __import__("os").environ.get("Q3_ROWS", "2048,576,64").split(",")]:
        for name, N, K in shapes:
            x = torch.randn(M, K, device="cuda:0").to(torch.bfloat16)
            copies = max(3, -(-600_000_000 // (N * K * 2)))    # more than the 256 MB cache holds, in turn
            ws = [(torch.randn(N, K, device="cuda:0") * 0.02).to(torch.bfloat16) for _ in range(copies)]
            out = torch.empty(M, N, device="cuda:0", dtype=torch.bfloat16)
            turn = [0]

            def chosen():
                turn[0] = (turn[0] + 1) % copies
                ops.linear(x, ws[turn[0]], out=out)

            entry = {"chosen_us": round(min(timed(chosen, copies), timed(chosen, copies)), 1), "plan": ops.matmul_plan(M, N, K),
                     "us_at_1_pflops": round(2.0 * M * N * K / 1e9, 1)}
            for shape in range(ops.gemm_tiles_configs()):
                def own():
                    turn[0] = (turn[0] + 1) % copies
                    ops.gemm_tiles(x, ws[turn[0]], shape, out=out)
                entry["tiles_%d_us" % shape] = round(min(timed(own, copies), timed(own, copies)), 1)
                splits = ops.gemm_tiles_splits(shape, M, N, K)
                if splits > 1:
                    def shared():
                        turn[0] = (turn[0] + 1) % copies
                        ops.gemm_tiles(x, ws[turn[0]], shape, out=out, splits=splits)
                    entry["tiles_%d_in_%d_us" % (shape, splits)] = round(min(timed(shared, copies), timed(shared, copies)), 1)
            rows["%s_%d" % (name, M)] = entry
            del ws
    print(json.dumps({"metric": "products of a layer, microseconds, %s bf16" % shape_name, "unit": "us", "n_gpus": 1,
                      "higher_is_better": False, "dtype": "bf16", "data": "synthetic", "products": rows}))
    return 0


def shared_prefix(args, config, model, shape_name, gen, sync):
    """64 requests that begin with the same 2,048 tokens (a system prompt, say) and go on with 32
    to 256 tokens of their own, 64 generated tokens each, with the prefix index on and off. Each
    engine serves such a load twice, with new tokens behind the shared ones each time; the second
    pass is the one reported (with the index on it finds the shared blocks of the first pass, as
    a server that has seen the system prompt before would)."""
    import random

    import torch

    from qwen3_from_scratch_amd.engine import SyncEngine

    requests, stem_len, context = 64, 2048, 4096
    rng = random.Random(0)
    stem = torch.randint(0, config.vocab_size, (stem_len,), generator=gen).tolist()
    tails = [rng.randint(32, 256) for _ in range(requests)]
    seconds, hits = {}, {}
    for on in (False, True):
        engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context, block_size=BLOCK,
                            num_blocks=requests * context // BLOCK // 2, max_num_seqs=requests,
                            max_num_tokens=512 + requests, chunked_prefill_size=512, enable_prefix_cache=on)
        for _ in range(2):
            before = engine.runner.manager.prefix_hits
            # every pass has new tokens behind the shared ones: only those can be found again
            prompts = [stem + torch.randint(0, config.vocab_size, (n,), generator=gen).tolist() for n in tails]
            for p in prompts:
                engine.add_request(p, engine.default_params(64, temperature=0.0, ignore_eos=True))
            sync()
            t0 = time.perf_counter()
            while engine.scheduler.has_work():
                engine.step()
            sync()
            seconds[on] = time.perf_counter() - t0
            hits[on] = engine.runner.manager.prefix_hits - before
        del engine
    tokens_in = sum(len(p) for p in prompts)
    print(json.dumps({
        "metric": "shared-prefix load, seconds, %s %s" % (shape_name, "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round(seconds[True], 3), "unit": "s", "n_gpus": 1, "higher_is_better": False,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "seconds_without_prefix_index": round(seconds[False], 3), "prompt_tokens": tokens_in,
        "prompt_tokens_taken_over": hits[True], "generated_tokens": 64 * requests,
        "config": {"model": "%s-shaped, random weights N(0, 0.02)" % shape_name, "requests": requests,
                   "shared_tokens": stem_len, "prefill_portion": 512, "context_len": context, "kv_block_size": BLOCK,
                   "layers": config.num_hidden_layers, "sampling": "greedy"},
    }))
    return 0


KODISUN_SHAPES = {
    # (width, heads, dim, rot_dim, vdim, q_rank, kv_rank, window, experts, top, expert_ff, shared_ff, layers)
    "lite": (2048, 16, 128, 64, 128, 768, 512, 1024, 64, 6, 1408, 2816, 4),
    "mid": (4096, 32, 128, 64, 128, 1536, 512, 2048, 32, 4, 2048, 4096, 2),
}


def kodisun(args, sync):
    """Prefill and decode throughput of the Kodisun design at sizes that resemble a real model's
    layers (random weights, a few layers, a vocabulary of 32,768), beside the Qwen3 dense decoder
    at equal size: the same width, head count and layer count, grouped heads of 128, and an inner
    size equal to what a Kodisun token passes through (its chosen experts and the shared one).
    Both go through the engine's own loop: one prompt of 2,048 tokens in one step, then greedy
    decoding at batch 8 and 64 behind prompts of 1,024 tokens. `frac` prices a prompt's
    multiply-adds against the bfloat16 matrix peak and a decode step's bytes (the weights it
    touches once, the cached rows its requests see) against the HBM peak."""
    import torch

    from qwen3_from_scratch_amd.config import ModelConfig
    from qwen3_from_scratch_amd.config.kodisun_config import KodisunConfig
    from qwen3_from_scratch_amd.engine import SyncEngine, random_model

    vocab, prompt_len, decode_prompt, context = 32768, args.prefill_tokens, 1024, 4096
    results = {}
    for shape in ([args.kodisun_shape] if args.kodisun_shape != "all" else sorted(KODISUN_SHAPES)):
        W, H, dn, dr, dv, qr, kr, window, E, top, ff, sff, layers = KODISUN_SHAPES[shape]
        if args.layers:
            layers = args.layers
        mixer = {"heads": H, "dim": dn, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": kr, "mask": {"size": window},
                 "scale": (dn + dr) ** -0.5,
                 "rot": {"dims": dr, "base": 10000.0, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
        mlp = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": ff}, "shared": {"ff": sff}}
        new = KodisunConfig.from_dict({"architecture": "Kodisun", "vocab": vocab, "width": W, "norm": {"eps": 1e-5},
                                       "layers": [{"type": "latent_attention", "mixer": mixer, "mlp": mlp}] * layers})
        dense = ModelConfig.from_dict(dict(QWEN3_8B, vocab_size=vocab, hidden_size=W, num_hidden_layers=layers,
                                           num_attention_heads=H, num_key_value_heads=max(1, H // 4), head_dim=128,
                                           intermediate_size=top * ff + sff, max_position_embeddings=context))
        # what a token multiplies with, per layer, and what a decode step reads
        new_active = ((qr + kr + dr) * W + H * (dn + dr) * qr + H * dn * kr + H * dv * kr + W * H * dv + E * W
                      + 2 * top * ff * W + 2 * sff * W)
        for name, config in (("kodisun", new), ("qwen3_dense", dense)):
            if args.kodisun_only and name != args.kodisun_only:
                continue
            model = random_model(config, dtype=args.dtype, device="cuda:0", seed=0, std=0.02)
            gen = torch.Generator().manual_seed(1)
            entry = {}
            if "prefill" in args.phases:
                room = prompt_len + 64
                engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=room, block_size=BLOCK,
                                    num_blocks=-(-room // BLOCK), max_num_seqs=1, max_num_tokens=prompt_len,
                                    chunked_prefill_size=prompt_len, enable_prefix_cache=False)
                timings = []
                for _ in range(4):
                    engine.add_request(torch.randint(0, vocab, (prompt_len,), generator=gen).tolist(),
                                       engine.default_params(1, temperature=0.0, ignore_eos=True))
                    sync()
                    t0 = time.perf_counter()
                    engine.step()
                    sync()
                    timings.append(time.perf_counter() - t0)
                    while engine.scheduler.has_work():
                        engine.step()
                seconds = sorted(timings[1:])[1]
                if name == "kodisun":
                    pairs = sum(min(i + 1, window) for i in range(prompt_len))
                    flops = layers * (2.0 * prompt_len * new_active + 2.0 * pairs * H * ((kr + dr) + kr)) + 2.0 * prompt_len * vocab * W
                else:
                    flops = prefill_flops(config, prompt_len)
                entry["prefill"] = {"tokens": prompt_len, "tokens_per_s": round(prompt_len / seconds, 1),
                                    "ms": round(seconds * 1e3, 3), "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
                del engine
            for batch in ((8, 64) if "decode" in args.phases else ()):
                engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context,
                                    block_size=BLOCK, num_blocks=batch * (context // BLOCK), max_num_seqs=batch,
                                    max_num_tokens=max(2048, batch), chunked_prefill_size=2048, enable_prefix_cache=False)
                params = engine.default_params(context - decode_prompt - 1, temperature=0.0, ignore_eos=True)
                requests = [engine.add_request(torch.randint(0, vocab, (decode_prompt,), generator=gen).tolist(), params)
                            for _ in range(batch)]
                while any(r.is_prefill for r in requests) or len(engine.scheduler.waiting):
                    engine.step()
                for _ in range(args.warmup):
                    engine.step()
                sync()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    engine.step()
                sync()
                step_s = (time.perf_counter() - t0) / args.steps
                seen = decode_prompt + args.warmup + args.steps // 2
                if name == "kodisun":
                    touched = min(E, batch * top)                      # experts a step can touch at most
                    weights = layers * (new_active - 2 * top * ff * W + 2 * touched * ff * W) + vocab * W
                    need = 2 * (weights + layers * batch * min(seen, window) * (kr + dr))
                else:
                    need = decode_bytes(config, [seen] * batch, 2)
                entry["decode_b%d" % batch] = {"tokens_per_s": round(batch / step_s, 1), "ms_per_step": round(step_s * 1e3, 3),
                                               "frac_hbm": round(need / step_s / PEAK_HBM, 4)}
                del engine
            results.setdefault(shape, {})[name] = entry
            del model
            torch.cuda.empty_cache()
        results[shape]["sizes"] = {"width": W, "heads": H, "dim": dn, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": kr,
                                   "window": window, "experts": E, "top": top, "expert_ff": ff, "shared_ff": sff,
                                   "layers": layers, "dense_intermediate": top * ff + sff, "vocab": vocab}
    print(json.dumps({"metric": "Kodisun beside the Qwen3 dense decoder at equal size: prefill and decode tokens/s",
                      "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
                      "steps": args.steps, "warmup": args.warmup, "shapes": results}))
    return 0


SURASUN_SHAPES = {
    # (width, streams, feed-forward inner size, layers as (type, with a feed-forward)); the mixers' sizes follow below
    "base": (2048, 4, 6144, (("mamba2", False), ("rglru", True), ("parallel", True), ("mamba2", False))),
    "wide": (4096, 2, 12288, (("rglru", True), ("parallel", True))),
}


def surasun_layers(W, ff, kinds):
    """Layers of real proportions: Mamba-2 with an inner size of twice the width in heads of 64 and a
    state of 128; the recurrent unit as wide as the model in blocks of 256; softmax attention in
    heads of 128, four query heads a key head, beside retention in heads of 128 with values of 256."""
    mixers = {
        "mamba2": {"heads": 2 * W // 64, "vdim": 64, "state": 128, "groups": 1, "conv": 4, "norm_groups": 1},
        "rglru": {"width": W, "blocks": W // 256, "conv": 4},
        "parallel": {"left": {"heads": W // 128, "kv_heads": W // 512, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                              "softcap": 50.0, "rot": {"dims": 64, "base": 10000.0}},
                     "right": {"heads": W // 256, "dim": 128, "vdim": 256, "rot": {"dims": 128, "base": 10000.0},
                               "decay": [1.0 - 2.0 ** (-5 - i % 8) for i in range(W // 256)]},
                     "left_scale": 0.5, "right_scale": 0.5},
    }
    return [{"type": kind, "mixer": mixers[kind], "mlp": {"kind": "dense", "ff": ff} if fed else None} for kind, fed in kinds]


def surasun(args, sync):
    """Prefill and decode throughput of the Surasun design at sizes that resemble a real model's
    layers (random weights, a few layers, a vocabulary of 32,768), beside the Qwen3 dense decoder of
    the same width and layer count (heads of 128, four query heads a key head, the same feed-forward
    inner size in every layer). Both go through the engine's own loop: one prompt in one step, then
    greedy decoding at batch 8 and 64 behind prompts of 1,024 tokens. `frac` prices a prompt's
    multiply-adds (the products, the recurrences' updates and reads, the attention's pairs) against
    the bfloat16 matrix peak, and a decode step's bytes (the weights once, the states read and
    written, the cached keys and values) against the HBM peak."""
    import torch

    from qwen3_from_scratch_amd.config import ModelConfig
    from qwen3_from_scratch_amd.config.surasun_config import SurasunConfig
    from qwen3_from_scratch_amd.engine import SyncEngine, random_model

    vocab, prompt_len, decode_prompt, context = 32768, args.prefill_tokens, 1024, 4096
    results = {}
    for shape in ([args.surasun_shape] if args.surasun_shape != "all" else sorted(SURASUN_SHAPES)):
        W, streams, ff, kinds = SURASUN_SHAPES[shape]
        if args.layers:
            kinds = (kinds * args.layers)[:args.layers]
        listed = surasun_layers(W, ff, kinds)
        new = SurasunConfig.from_dict({"architecture": "Surasun", "vocab": vocab, "width": W, "norm": {"eps": 1e-5},
                                       "residual_mult": 1.0, "streams": streams, "layers": listed})
        dense = ModelConfig.from_dict(dict(QWEN3_8B, vocab_size=vocab, hidden_size=W, num_hidden_layers=len(listed),
                                           num_attention_heads=W // 128, num_key_value_heads=W // 512, head_dim=128,
                                           intermediate_size=ff, max_position_embeddings=context))
        for name, config in (("surasun", new), ("qwen3_dense", dense)):
            if args.surasun_only and name != args.surasun_only:
                continue
            model = random_model(config, dtype=args.dtype, device="cuda:0", seed=0, std=0.02)
            gen = torch.Generator().manual_seed(1)
            entry = {}
            if name == "surasun":
                matrices = sum(shape_[0] * shape_[1] for key, shape_ in model.tensors().items()
                               if len(shape_) == 2 and key != "embed" and ".hc" not in key and not key.endswith("conv"))
                gates = sum(shape_[0] * shape_[1] * shape_[2] for shape_ in model.tensors().values() if len(shape_) == 3)
                scans = pairs_each = state = cached = 0        # per token: recurrences' multiply-adds; per (query, key) pair; floats of state; cached numbers
                for layer in listed:
                    m = layer["mixer"]
                    if layer["type"] == "mamba2":
                        scans += 3 * m["heads"] * m["state"] * m["vdim"]
                        state += m["heads"] * m["state"] * m["vdim"] + 3 * (m["heads"] * m["vdim"] + 2 * m["state"])
                    elif layer["type"] == "rglru":
                        state += 4 * m["width"]
                    else:
                        scans += 3 * m["right"]["heads"] * m["right"]["dim"] * m["right"]["vdim"]
                        state += m["right"]["heads"] * m["right"]["dim"] * m["right"]["vdim"]
                        pairs_each += m["left"]["heads"] * (m["left"]["dim"] + m["left"]["vdim"])
                        cached += m["left"]["kv_heads"] * (m["left"]["dim"] + m["left"]["vdim"])
            if "prefill" in args.phases:
                room = prompt_len + 64
                engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=room, block_size=BLOCK,
                                    num_blocks=-(-room // BLOCK), max_num_seqs=1, max_num_tokens=prompt_len,
                                    chunked_prefill_size=prompt_len, enable_prefix_cache=False)
                timings = []
                for _ in range(4):
                    engine.add_request(torch.randint(0, vocab, (prompt_len,), generator=gen).tolist(),
                                       engine.default_params(1, temperature=0.0, ignore_eos=True))
                    sync()
                    t0 = time.perf_counter()
                    engine.step()
                    sync()
                    timings.append(time.perf_counter() - t0)
                    while engine.scheduler.has_work():
                        engine.step()
                seconds = sorted(timings[1:])[1]
                if name == "surasun":
                    flops = (2.0 * prompt_len * (matrices + gates + scans) + 2.0 * vocab * W
                             + 2.0 * (prompt_len * (prompt_len + 1) / 2) * pairs_each)
                else:
                    flops = prefill_flops(config, prompt_len)
                entry["prefill"] = {"tokens": prompt_len, "tokens_per_s": round(prompt_len / seconds, 1),
                                    "ms": round(seconds * 1e3, 3), "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
                del engine
            for batch in ((8, 64) if "decode" in args.phases else ()):
                engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context,
                                    block_size=BLOCK, num_blocks=batch * (context // BLOCK), max_num_seqs=batch,
                                    max_num_tokens=max(2048, batch), chunked_prefill_size=2048, enable_prefix_cache=False)
                params = engine.default_params(context - decode_prompt - 1, temperature=0.0, ignore_eos=True)
                requests = [engine.add_request(torch.randint(0, vocab, (decode_prompt,), generator=gen).tolist(), params)
                            for _ in range(batch)]
                while any(r.is_prefill for r in requests) or len(engine.scheduler.waiting):
                    engine.step()
                for _ in range(args.warmup):
                    engine.step()
                sync()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    engine.step()
                sync()
                step_s = (time.perf_counter() - t0) / args.steps
                seen = decode_prompt + args.warmup + args.steps // 2
                if name == "surasun":
                    need = 2 * (matrices + vocab * W) + 4 * gates + batch * (8 * state + 2 * cached * seen)
                else:
                    need = decode_bytes(config, [seen] * batch, 2)
                entry["decode_b%d" % batch] = {"tokens_per_s": round(batch / step_s, 1), "ms_per_step": round(step_s * 1e3, 3),
                                               "frac_hbm": round(need / step_s / PEAK_HBM, 4)}
                del engine
            results.setdefault(shape, {})[name] = entry
            del model
            torch.cuda.empty_cache()
        results[shape]["sizes"] = {"width": W, "streams": streams, "ff": ff, "layers": [k + ("+ff" if f else "") for k, f in kinds],
                                   "vocab": vocab}
    print(json.dumps({"metric": "Surasun beside the Qwen3 dense decoder at equal size: prefill and decode tokens/s",
                      "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
                      "steps": args.steps, "warmup": args.warmup, "shapes": results}))
    return 0


DUFINEX_SHAPES = {
    # (width, dense feed-forward inner size, experts, experts a token, layers as (mixer, reads the keys of, feed-forward))
    "base": (2048, 6144, 32, 4, (("attention", None, "dense"), ("attention", 0, "moe"), ("channel_delta", None, "dense"),
                                 ("attention", None, "moe"))),
    "wide": (4096, 12288, 64, 8, (("channel_delta", None, "moe"), ("attention", None, "dense"))),
}


def dufinex_layers(W, ff, experts, top, kinds):
    """Layers of real proportions: attention in heads of 128, four query heads a key head; the delta rule in
    heads of 128 with values of 128, a key head per head, four taps; experts whose inner sizes add up, over a
    token's choices, to the dense feed-forward's."""
    mixers = {"attention": {"heads": W // 128, "kv_heads": W // 512, "dim": 128, "vdim": 128, "scale": 128 ** -0.5},
              "channel_delta": {"heads": W // 128, "kv_heads": W // 128, "dim": 128, "vdim": 128, "conv": 4}}
    feeds = {"dense": {"kind": "dense", "ff": ff, "limit": 7.0},
             "moe": {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff // top, "limit": 7.0}}}
    listed = []
    for kind, source, feed in kinds:
        mixer = dict(mixers[kind])
        if source is not None:
            mixer["kv_from"] = source
        listed.append({"type": kind, "mixer": mixer, "mlp": feeds[feed]})
    return listed


def dufinex(args, sync):
    """Prefill and decode throughput of the Dufinex design at sizes that resemble a real model's layers
    (random weights, a few layers, a vocabulary of 32,768), beside the Surasun design, the closest of the
    others (softmax attention with a gate per head through the same kernels, recurrences with a state per
    head), at the same width, layer count and feed-forward inner size, a layer of attention beside
    retention where this one has attention and Mamba-2 where it has the delta rule. Both go through the
    engine's own loop: one prompt in one step, then greedy decoding at batch 8 and 64 behind prompts of
    1,024 tokens. `frac` prices a prompt's multiply-adds (the products with a token's share of the
    experts, the recurrences' updates and reads, the attention's pairs) against the bfloat16 matrix peak,
    and a decode step's bytes (the weights once, of the experts those a batch can reach, the states read
    and written, the cached keys and values) against the HBM peak."""
    import torch

    from qwen3_from_scratch_amd.config.dufinex_config import DufinexConfig
    from qwen3_from_scratch_amd.config.surasun_config import SurasunConfig
    from qwen3_from_scratch_amd.engine import SyncEngine, random_model

    vocab, prompt_len, decode_prompt, context = 32768, args.prefill_tokens, 1024, 4096
    results = {}
    for shape in ([args.dufinex_shape] if args.dufinex_shape != "all" else sorted(DUFINEX_SHAPES)):
        W, ff, experts, top, kinds = DUFINEX_SHAPES[shape]
        if args.layers:
            kinds = tuple((k, None, f) for k, _, f in (kinds * args.layers)[:args.layers])
        listed = dufinex_layers(W, ff, experts, top, kinds)
        new = DufinexConfig.from_dict({"architecture": "Dufinex", "vocab": vocab, "width": W, "norm": {"eps": 1e-5},
                                       "embedding": {"scale": 1.0}, "layers": listed})
        other = SurasunConfig.from_dict({"architecture": "Surasun", "vocab": vocab, "width": W, "norm": {"eps": 1e-5},
                                         "residual_mult": 1.0,
                                         "layers": surasun_layers(W, ff, [("parallel" if k == "attention" else "mamba2", True)
                                                                          for k, _, _ in kinds])})
        for name, config in (("dufinex", new), ("surasun", other)):
            if args.dufinex_only and name != args.dufinex_only:
                continue
            model = random_model(config, dtype=args.dtype, device="cuda:0", seed=0, std=0.02)
            gen = torch.Generator().manual_seed(1)
            entry = {}
            tensors = model.tensors()
            # per token: matrix numbers every token meets, those of one expert's share, the recurrences' multiply-adds;
            # per (query, key) pair; floats of state; cached numbers
            matrices = sum(t[0] * t[1] for key, t in tensors.items()
                           if len(t) == 2 and key != "embed" and ".hc" not in key and not key.endswith("conv") and ".mlp.e" not in key)
            expert_numbers = sum(t[0] * t[1] for key, t in tensors.items() if ".mlp.e" in key)
            scans = pairs_each = state = cached = 0
            for layer in (listed if name == "dufinex" else config.to_dict()["layers"]):
                m = layer["mixer"]
                if layer["type"] == "channel_delta":
                    scans += 4 * m["heads"] * m["dim"] * m["vdim"]
                    state += m["heads"] * m["dim"] * m["vdim"] + 3 * (2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"])
                elif layer["type"] == "attention":
                    pairs_each += m["heads"] * (m["dim"] + m["vdim"])
                    cached += 0 if m.get("kv_from") is not None else m["kv_heads"] * (m["dim"] + m["vdim"])
                elif layer["type"] == "mamba2":
                    scans += 3 * m["heads"] * m["state"] * m["vdim"]
                    state += m["heads"] * m["state"] * m["vdim"] + 3 * (m["heads"] * m["vdim"] + 2 * m["state"])
                else:
                    scans += 3 * m["right"]["heads"] * m["right"]["dim"] * m["right"]["vdim"]
                    state += m["right"]["heads"] * m["right"]["dim"] * m["right"]["vdim"]
                    pairs_each += m["left"]["heads"] * (m["left"]["dim"] + m["left"]["vdim"])
                    cached += m["left"]["kv_heads"] * (m["left"]["dim"] + m["left"]["vdim"])
            share = top / experts
            if "prefill" in args.phases:
                room = prompt_len + 64
                engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=room, block_size=BLOCK,
                                    num_blocks=-(-room // BLOCK), max_num_seqs=1, max_num_tokens=prompt_len,
                                    chunked_prefill_size=prompt_len, enable_prefix_cache=False)
                timings = []
                for _ in range(4):
                    engine.add_request(torch.randint(0, vocab, (prompt_len,), generator=gen).tolist(),
                                       engine.default_params(1, temperature=0.0, ignore_eos=True))
                    sync()
                    t0 = time.perf_counter()
                    engine.step()
                    sync()
                    timings.append(time.perf_counter() - t0)
                    while engine.scheduler.has_work():
                        engine.step()
                seconds = sorted(timings[1:])[1]
                flops = (2.0 * prompt_len * (matrices + share * expert_numbers + scans) + 2.0 * vocab * W
                         + 2.0 * (prompt_len * (prompt_len + 1) / 2) * pairs_each)
                entry["prefill"] = {"tokens": prompt_len, "tokens_per_s": round(prompt_len / seconds, 1),
                                    "ms": round(seconds * 1e3, 3), "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
                del engine
            for batch in ((8, 64) if "decode" in args.phases else ()):
                engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context,
                                    block_size=BLOCK, num_blocks=batch * (context // BLOCK), max_num_seqs=batch,
                                    max_num_tokens=max(2048, batch), chunked_prefill_size=2048, enable_prefix_cache=False)
                params = engine.default_params(context - decode_prompt - 1, temperature=0.0, ignore_eos=True)
                requests = [engine.add_request(torch.randint(0, vocab, (decode_prompt,), generator=gen).tolist(), params)
                            for _ in range(batch)]
                while any(r.is_prefill for r in requests) or len(engine.scheduler.waiting):
                    engine.step()
                for _ in range(args.warmup):
                    engine.step()
                sync()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    engine.step()
                sync()
                step_s = (time.perf_counter() - t0) / args.steps
                seen = decode_prompt + args.warmup + args.steps // 2
                reached = min(1.0, batch * share)
                need = 2 * (matrices + reached * expert_numbers + vocab * W) + batch * (8 * state + 2 * cached * seen)
                entry["decode_b%d" % batch] = {"tokens_per_s": round(batch / step_s, 1), "ms_per_step": round(step_s * 1e3, 3),
                                               "frac_hbm": round(need / step_s / PEAK_HBM, 4)}
                del engine
            results.setdefault(shape, {})[name] = entry
            del model
            torch.cuda.empty_cache()
        results[shape]["sizes"] = {"width": W, "ff": ff, "experts": experts, "top": top, "vocab": vocab,
                                   "layers": ["%s%s+%s" % (k, "" if src is None else "(keys of %d)" % src, f) for k, src, f in kinds]}
    print(json.dumps({"metric": "Dufinex beside Surasun at equal size: prefill and decode tokens/s",
                      "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
                      "steps": args.steps, "warmup": args.warmup, "shapes": results}))
    return 0


FIDEVIK_SHAPES = {
    # (width, query heads, key heads, q_rank, kv_rank, dense inner size, experts, top, groups, keep, expert_ff, shared_ff,
    #  layers as (mixer, feed-forward), loop or None)
    "base": (2048, 16, 4, 768, 512, 6144, 64, 6, 8, 4, 768, 1536,
             (("attention", "dense"), ("latent_attention", "moe"), ("latent_attention", "moe"), ("attention", "moe")),
             {"start": 1, "stop": 3, "times": 2}),
    "wide": (4096, 32, 8, 1536, 512, 12288, 32, 4, 4, 2, 2048, 4096,
             (("latent_attention", "moe"), ("attention", "dense")), None),
}


def fidevik(args, sync):
    """Prefill and decode throughput of the Fidevik design at sizes that resemble a real model's layers
    (random weights, a few layers, a vocabulary of 32,768), beside Kodisun, the closest of the other designs
    (latent attention, a choice among small experts beside a shared one, a run of layers passed several
    times), at the same width, head count, latent sizes, cached numbers per token, experts and run order,
    with latent attention in every layer (64 of a head's 128 query numbers rotated) and the experts in
    every layer. Both go through the engine's own loop: one prompt in one step, then greedy decoding at
    batch 8 and 64 behind prompts of 1,024 tokens. `frac` prices a prompt's multiply-adds (the products
    with a token's share of the experts, the attention's pairs in the form each design computes them)
    against the bfloat16 matrix peak, and a decode step's bytes (the weights once, of the experts those a
    batch can reach, the cached numbers its requests see) against the HBM peak."""
    import torch

    from qwen3_from_scratch_amd.config.fidevik_config import FidevikConfig
    from qwen3_from_scratch_amd.config.kodisun_config import KodisunConfig
    from qwen3_from_scratch_amd.engine import SyncEngine, random_model

    vocab, prompt_len, decode_prompt, context = 32768, args.prefill_tokens, 1024, 4096
    results = {}
    for shape in ([args.fidevik_shape] if args.fidevik_shape != "all" else sorted(FIDEVIK_SHAPES)):
        W, H, G, qr, kr, dense_ff, E, top, groups, keep, ff, sff, kinds, loop = FIDEVIK_SHAPES[shape]
        if args.layers:
            kinds, loop = (kinds * args.layers)[:args.layers], None
        mixers = {"attention": {"heads": H, "kv_heads": G, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                                "rot": {"dims": 64, "base": 10000.0}},
                  "latent_attention": {"heads": H, "dim": 128, "vdim": 128, "q_rank": qr, "kv_rank": kr, "scale": 128 ** -0.5}}
        feeds = {"dense": {"kind": "dense", "ff": dense_ff},
                 "moe": {"kind": "moe", "router": {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}},
                         "expert": {"ff": ff}, "shared": {"ff": sff}}}
        listed = [{"type": m, "mixer": mixers[m], "mlp": feeds[f]} for m, f in kinds]
        data = {"architecture": "Fidevik", "vocab": vocab, "width": W, "norm": {"eps": 1e-5}, "logit_scale": 1.0, "layers": listed}
        like = {"type": "latent_attention",
                "mixer": {"heads": H, "dim": 64, "rot_dim": 64, "vdim": 128, "q_rank": qr, "kv_rank": kr - 64, "scale": 128 ** -0.5,
                          "rot": {"dims": 64, "base": 10000.0}},
                "mlp": {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": ff}, "shared": {"ff": sff}}}
        other = {"architecture": "Kodisun", "vocab": vocab, "width": W, "norm": {"eps": 1e-5}, "layers": [like] * len(kinds)}
        if loop:
            data["loop"] = other["loop"] = loop
        for name, config in (("fidevik", FidevikConfig.from_dict(data)), ("kodisun", KodisunConfig.from_dict(other))):
            if args.fidevik_only and name != args.fidevik_only:
                continue
            model = random_model(config, dtype=args.dtype, device="cuda:0", seed=0, std=0.02)
            gen = torch.Generator().manual_seed(1)
            entry = {}
            tensors = model.tensors()
            # per run of a layer: matrix numbers every token meets, those of the experts (a token meets its share);
            # multiply-adds per (query, key) pair in the form the design computes; numbers cached per token
            matrices = expert_numbers = pairs_each = cached = 0
            runs = [step.layer for step in model.spec.order]
            for i in runs:
                own = {key: t for key, t in tensors.items() if key.startswith("l%d." % i) and len(t) == 2}
                expert_numbers += sum(t[0] * t[1] for key, t in own.items() if ".mlp.e" in key)
                matrices += sum(t[0] * t[1] for key, t in own.items() if ".mlp.e" not in key)
                layer = config.to_dict()["layers"][i]
                m = layer["mixer"]
                if layer["type"] == "attention":
                    pairs_each += m["heads"] * (m["dim"] + m["vdim"])
                    cached += m["kv_heads"] * (m["dim"] + m["vdim"])
                else:                                    # in the latent's space: the cached row is key and value
                    row = m["kv_rank"] + m.get("rot_dim", 0)
                    pairs_each += m["heads"] * (row + m["kv_rank"])
                    cached += row
            share = top / E
            if "prefill" in args.phases:
                room = prompt_len + 64
                engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=room, block_size=BLOCK,
                                    num_blocks=-(-room // BLOCK), max_num_seqs=1, max_num_tokens=prompt_len,
                                    chunked_prefill_size=prompt_len, enable_prefix_cache=False)
                timings = []
                for _ in range(4):
                    engine.add_request(torch.randint(0, vocab, (prompt_len,), generator=gen).tolist(),
                                       engine.default_params(1, temperature=0.0, ignore_eos=True))
                    sync()
                    t0 = time.perf_counter()
                    engine.step()
                    sync()
                    timings.append(time.perf_counter() - t0)
                    while engine.scheduler.has_work():
                        engine.step()
                seconds = sorted(timings[1:])[1]
                flops = (2.0 * prompt_len * (matrices + share * expert_numbers) + 2.0 * vocab * W
                         + 2.0 * (prompt_len * (prompt_len + 1) / 2) * pairs_each)
                entry["prefill"] = {"tokens": prompt_len, "tokens_per_s": round(prompt_len / seconds, 1),
                                    "ms": round(seconds * 1e3, 3), "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
                del engine
            for batch in ((8, 64) if "decode" in args.phases else ()):
                engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context,
                                    block_size=BLOCK, num_blocks=batch * (context // BLOCK), max_num_seqs=batch,
                                    max_num_tokens=max(2048, batch), chunked_prefill_size=2048, enable_prefix_cache=False)
                params = engine.default_params(context - decode_prompt - 1, temperature=0.0, ignore_eos=True)
                requests = [engine.add_request(torch.randint(0, vocab, (decode_prompt,), generator=gen).tolist(), params)
                            for _ in range(batch)]
                while any(r.is_prefill for r in requests) or len(engine.scheduler.waiting):
                    engine.step()
                for _ in range(args.warmup):
                    engine.step()
                sync()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    engine.step()
                sync()
                step_s = (time.perf_counter() - t0) / args.steps
                seen = decode_prompt + args.warmup + args.steps // 2
                reached = min(1.0, batch * share)
                # a layer's weights are read once per run of it: a pass finds little of the last pass's in the caches
                need = 2 * (matrices + reached * expert_numbers + vocab * W) + batch * 2 * cached * seen
                entry["decode_b%d" % batch] = {"tokens_per_s": round(batch / step_s, 1), "ms_per_step": round(step_s * 1e3, 3),
                                               "frac_hbm": round(need / step_s / PEAK_HBM, 4)}
                del engine
            results.setdefault(shape, {})[name] = entry
            del model
            torch.cuda.empty_cache()
        results[shape]["sizes"] = {"width": W, "heads": H, "kv_heads": G, "q_rank": qr, "kv_rank": kr, "dense_ff": dense_ff,
                                   "experts": E, "top": top, "groups": groups, "keep": keep, "expert_ff": ff, "shared_ff": sff,
                                   "vocab": vocab, "layers": ["%s+%s" % k for k in kinds], "loop": loop}
    print(json.dumps({"metric": "Fidevik beside Kodisun at equal size: prefill and decode tokens/s",
                      "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
                      "steps": args.steps, "warmup": args.warmup, "shapes": results}))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0 = all)")
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES))
    ap.add_argument("--prompt", type=int, default=2048, help="tokens every request holds when decoding starts")
    ap.add_argument("--context", type=int, default=8192, help="tokens of cache per request")
    ap.add_argument("--workload", default="decode", choices=["decode", "continuous", "served", "prefix", "products", "kodisun", "surasun", "dufinex", "fidevik"],
                    help="continuous: 64 requests at once, prompts of 128 to 4,096 tokens, 64 to 512 generated "
                         "tokens each, prompts in portions of 512 (its own JSON line; --steps and --warmup unused); "
                         "prefix: 64 requests that share their first 2,048 tokens, with the prefix index on and off; "
                         "products: a layer's four products by the chosen kernel and by each tile shape of the "
                         "hand-written one; kodisun, surasun: that design beside the dense decoder at equal size; dufinex: "
                         "that design beside Surasun at equal size")
    ap.add_argument("--kodisun-shape", default="all", choices=["all"] + sorted(KODISUN_SHAPES))
    ap.add_argument("--kodisun-only", default="", choices=["", "kodisun", "qwen3_dense"], help="one of the two models")
    ap.add_argument("--surasun-shape", default="all", choices=["all"] + sorted(SURASUN_SHAPES))
    ap.add_argument("--surasun-only", default="", choices=["", "surasun", "qwen3_dense"], help="one of the two models")
    ap.add_argument("--dufinex-shape", default="all", choices=["all"] + sorted(DUFINEX_SHAPES))
    ap.add_argument("--dufinex-only", default="", choices=["", "dufinex", "surasun"], help="one of the two models")
    ap.add_argument("--fidevik-shape", default="all", choices=["all"] + sorted(FIDEVIK_SHAPES))
    ap.add_argument("--fidevik-only", default="", choices=["", "fidevik", "kodisun"], help="one of the two models")
    ap.add_argument("--phases", default="prefill,decode",
                    help="of --workload kodisun, surasun, dufinex or fidevik: prefill, decode or both")
    ap.add_argument("--single-copy", action="store_true",
                    help="hold the matrices once (no tile-ordered copy for steps of few rows): half the weights' memory, slower decoding")
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 points")
    ap.add_argument("--no-probes", action="store_true",
                    help="skip the measurement of this GPU's read and matrix rates (for profiles of the engine alone)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL,
                    help="length of the prompt whose one step is the prefill measurement (2,048 in the default line)")
    ap.add_argument("--skip-prefill", action="store_true",
                    help="skip the prefill measurement (for profiles of decoding alone; the line then has no value for it)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported" % args.gpus)
        return 2

    import torch

    from qwen3_from_scratch_amd.config import ModelConfig
    from qwen3_from_scratch_amd.engine import SyncEngine, random_model

    if args.workload == "kodisun":
        torch.cuda.set_device(0)
        args.steps, args.warmup = min(args.steps, 32), min(args.warmup, 8)
        return kodisun(args, torch.cuda.synchronize)
    if args.workload == "surasun":
        torch.cuda.set_device(0)
        args.steps, args.warmup = min(args.steps, 32), min(args.warmup, 8)
        return surasun(args, torch.cuda.synchronize)
    if args.workload == "dufinex":
        torch.cuda.set_device(0)
        args.steps, args.warmup = min(args.steps, 32), min(args.warmup, 8)
        return dufinex(args, torch.cuda.synchronize)
    if args.workload == "fidevik":
        torch.cuda.set_device(0)
        args.steps, args.warmup = min(args.steps, 32), min(args.warmup, 8)
        return fidevik(args, torch.cuda.synchronize)
    shape_name, raw = SHAPES[args.shape]
    raw = dict(raw)
    prompt_len, context = args.prompt, args.context
    if not 0 < prompt_len + args.warmup + args.steps < context <= raw["max_position_embeddings"]:
        print("bench.py: --prompt, --warmup and --steps must fit in --context, and that in the model's positions")
        return 2
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    config = ModelConfig.from_dict(raw)
    itemsize = 2 if args.dtype == "bfloat16" else 4
    torch.cuda.set_device(0)
    if args.workload == "products":
        return products(args, config, shape_name, torch.cuda.synchronize)
    model = random_model(config, dtype=args.dtype, device="cuda:0", seed=0, std=0.02, tiled_weights=not args.single_copy)
    gen = torch.Generator().manual_seed(1)

    def prompts(n, length):
        return [torch.randint(0, config.vocab_size, (length,), generator=gen).tolist() for _ in range(n)]

    def engine_for(batch):
        pages = batch * (context // BLOCK)
        return SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context,
                          block_size=BLOCK, num_blocks=pages, max_num_seqs=batch,
                          max_num_tokens=max(PREFILL, batch), chunked_prefill_size=PREFILL,
                          enable_prefix_cache=False)       # every token of every prompt is computed

    def sync():
        torch.cuda.synchronize()

    if args.workload == "continuous":
        return continuous(args, config, model, shape_name, gen, sync)
    if args.workload == "served":
        return served(args, config, model, shape_name, gen, sync)
    if args.workload == "prefix":
        return shared_prefix(args, config, model, shape_name, gen, sync)

    # ---- prefill: one prompt of 2,048 tokens in one step (and of 8,192 for `points`) ----
    def prefill_of(tokens, timed=3):
        """Seconds of one step that is one whole prompt of `tokens` tokens: a warm-up, then the
        median of `timed` runs, each a new prompt."""
        room = tokens + 64
        engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=room,
                            block_size=BLOCK, num_blocks=-(-room // BLOCK), max_num_seqs=1,
                            max_num_tokens=tokens, chunked_prefill_size=tokens, enable_prefix_cache=False)
        timings = []
        for _ in range(1 + timed):
            engine.add_request(prompts(1, tokens)[0], engine.default_params(1, temperature=0.0, ignore_eos=True))
            sync()
            t0 = time.perf_counter()
            plan = engine.step()
            sync()
            timings.append(time.perf_counter() - t0)
            assert len(plan) == 1 and plan[0].num_tokens == tokens
            while engine.scheduler.has_work():
                engine.step()
        return sorted(timings[1:])[timed // 2]

    prefill = None
    prefill_s = None if args.skip_prefill else prefill_of(args.prefill_tokens)
    if prefill_s is not None:
        prefill = {"value": round(args.prefill_tokens / prefill_s, 1), "tokens": args.prefill_tokens,
                   "ms": round(prefill_s * 1e3, 3),
                   "frac": round(prefill_flops(config, args.prefill_tokens) / prefill_s / PEAK_FLOPS[args.dtype], 4)}

    # ---- decode ----
    def decode(batch, steps, warmup):
        engine = engine_for(batch)
        params = engine.default_params(context - prompt_len - 1, temperature=0.0, ignore_eos=True)
        requests = [engine.add_request(p, params) for p in prompts(batch, prompt_len)]
        while any(r.is_prefill for r in requests) or len(engine.scheduler.waiting):
            engine.step()
        for _ in range(warmup):
            engine.step()
        contexts = [r.num_tokens for r in requests]
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            plan = engine.step()
        sync()
        dt = time.perf_counter() - t0
        assert len(plan) == batch and all(s.num_tokens == 1 for s in plan)
        mean_contexts = [n + steps / 2 for n in contexts]
        return batch * steps / dt, dt / steps, mean_contexts

    tps, step_s, contexts = decode(args.batch, args.steps, args.warmup)
    need = decode_bytes(config, contexts, itemsize)
    roofline = {"bound": "hbm", "achieved": round(need / step_s / 1e9, 1), "peak": PEAK_HBM / 1e9,
                "unit": "GB/s", "frac": round(need / step_s / PEAK_HBM, 4)}
    points, points_roofline = {}, {}
    if not args.no_points and not args.skip_prefill and config.max_position_embeddings > LONG_PREFILL + 64:
        long_s = prefill_of(LONG_PREFILL, timed=1)          # one more step of a tenth of a second
        points["prefill_%d" % LONG_PREFILL] = round(LONG_PREFILL / long_s, 1)
        points_roofline["prefill_%d" % LONG_PREFILL] = round(
            prefill_flops(config, LONG_PREFILL) / long_s / PEAK_FLOPS[args.dtype], 4)
    if not args.no_points:
        for b in (1, 64):
            if b == args.batch:
                points["decode_b%d" % b] = round(tps, 1)
                points_roofline["decode_b%d" % b] = roofline["frac"]
                continue
            p_tps, p_step_s, p_contexts = decode(b, max(16, args.steps // 4), max(4, args.warmup // 2))
            points["decode_b%d" % b] = round(p_tps, 1)
            points_roofline["decode_b%d" % b] = round(decode_bytes(config, p_contexts, itemsize) / p_step_s / PEAK_HBM, 4)
    resident = sum(t.untyped_storage().nbytes() for t in _model_tensors(model))
    # what this GPU delivers, measured here: a plain read of 4 GB, the matrix instruction from registers
    from qwen3_from_scratch_amd import ops
    read_rate = matrix_rate = None
    if not args.no_probes:
        read_rate, matrix_rate = ops.measured_read_rate(), ops.measured_matrix_rate()
        roofline["measured_peak"] = round(read_rate / 1e9, 1)
        roofline["frac_of_measured"] = round(need / step_s / read_rate, 4)
    if prefill is not None and args.dtype == "bfloat16" and matrix_rate:
        prefill["measured_peak_tflops"] = round(matrix_rate / 1e12, 1)
        prefill["frac_of_measured"] = round(prefill_flops(config, args.prefill_tokens) / prefill_s / matrix_rate, 4)

    line = {
        "metric": "decode tok/s at batch 1/8/64 + prefill tok/s at 2048 tokens, %s %s"
                  % (shape_name, "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round(tps, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": "%s-shaped, random weights N(0, 0.02)" % shape_name, "global_batch": args.batch,
            "seq_len": prompt_len, "parallelism": "single-gpu", "context_len": context,
            "layers": config.num_hidden_layers, "layers_full": full_layers, "hidden_size": config.hidden_size,
            "num_attention_heads": config.num_attention_heads, "num_key_value_heads": config.num_key_value_heads,
            "head_dim": config.head_dim, "intermediate_size": config.intermediate_size,
            "vocab_size": config.vocab_size, "rope_theta": config.rope_theta, "rms_norm_eps": config.rms_norm_eps,
            "tie_word_embeddings": config.tie_word_embeddings, "kv_block_size": BLOCK, "sampling": "greedy",
        },
        "prefill": prefill, "roofline": roofline, "points": points,
        # the same fraction of the HBM peak for the other batch sizes; what the weights hold on the GPU (bfloat16
        # matrices are kept twice, row-major and in the few-row kernel's order); how many-row products get their kernels
        "points_roofline": points_roofline, "resident_weight_gb": round(resident / 1e9, 2),
        "matmul_choice": "table and rule, no timing",
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
