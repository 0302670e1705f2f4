#!/usr/bin/env python3
"""Throughput of the engine on one MI355X: decode tokens per second at batch 8 (the headline value),
at batch 1 and 64, and prefill tokens per second at 2,048 tokens, each with its roofline fraction.

    python bench.py --gpus 1 --steps K --warmup W

The model has the layer sizes of Qwen2.5-7B (28 layers, hidden 3584, 28 heads over 4 KV heads of
width 128, feed-forward 18944, vocabulary 152064, rotary base 1e6, untied output matrix) with seeded
random weights N(0, 0.02) in bfloat16; token ids are seeded uniform-random.  Every request is
prefilled for real and then decoded up to a context of 4,096 tokens; the timed steps are the last K
decode steps of that run, through the engine's scheduler, captured step and greedy sampler.  A step
is one decode step of the whole batch.  The engine launches a step before the tokens of the step
before have reached the host (`pipelined=True`; `--in-turn` switches that off): every timed call of
`step()` launches one decode step and takes in the tokens of the one before.

Bytes a decode step has to read: every weight it uses once (all layer matrices, norms and the output
matrix; of the embedding table only the batch's rows) and the keys and values of the live requests.
Peaks are MI355X's published ones: HBM 8 TB/s; dense bfloat16 matrix cores 2.5 PFLOP/s.
"""
import argparse
import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN25_7B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 32768, "hidden_act": "silu",
    "use_sliding_window": False, "sliding_window": 131072, "max_window_layers": 28, "torch_dtype": "bfloat16",
}


# the other Qwen2.5 shapes, for measurements beside the headline one (--shape); the sizes are those of the published
# config.json of each model
SHAPES = {
    "7b": ("Qwen2.5-7B shape", QWEN25_7B),
    "0.5b": ("Qwen2.5-0.5B shape", dict(QWEN25_7B, num_hidden_layers=24, hidden_size=896, num_attention_heads=14,
                                        num_key_value_heads=2, intermediate_size=4864, vocab_size=151936,
                                        tie_word_embeddings=True, max_window_layers=21)),
    "3b": ("Qwen2.5-3B shape", dict(QWEN25_7B, num_hidden_layers=36, hidden_size=2048, num_attention_heads=16,
                                    num_key_value_heads=2, intermediate_size=11008, vocab_size=151936,
                                    tie_word_embeddings=True, max_window_layers=70)),
    "14b": ("Qwen2.5-14B shape", dict(QWEN25_7B, num_hidden_layers=48, hidden_size=5120, num_attention_heads=40,
                                      num_key_value_heads=8, intermediate_size=13824, max_window_layers=48)),
    "72b": ("Qwen2.5-72B shape", dict(QWEN25_7B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                                      num_key_value_heads=8, intermediate_size=29568, max_window_layers=70)),
    "1.5b": ("Qwen2.5-1.5B shape", dict(QWEN25_7B, num_hidden_layers=28, hidden_size=1536, num_attention_heads=12,
                                        num_key_value_heads=2, intermediate_size=8960, vocab_size=151936,
                                        tie_word_embeddings=True, max_window_layers=21)),
    "32b": ("Qwen2.5-32B shape", dict(QWEN25_7B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=40,
                                      num_key_value_heads=8, intermediate_size=27648, max_window_layers=64)),
}


SETTLE_STEPS = 96   # untimed decode steps between the prompts and the warm-up steps (see decode())


def log(text):
    print(f"[bench] {text}", file=sys.stderr, flush=True)


def still_running(every_seconds: float = 60.0) -> None:
    """A line on stderr every minute for as long as the program runs: a 32-bit step over the prompts of a large
    batch takes minutes, and a run that prints nothing for long looks hung to whoever watches it."""
    started = time.perf_counter()

    def beat():
        while True:
            time.sleep(every_seconds)
            log(f"  still running, {time.perf_counter() - started:.0f} s")

    threading.Thread(target=beat, daemon=True).start()


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8, help="batch of the headline decode measurement")
    parser.add_argument("--ctx", type=int, default=4096, help="context length the decode steps end at")
    parser.add_argument("--shape", default="7b", choices=sorted(SHAPES), help="layer sizes; the headline run is 7b")
    parser.add_argument("--layers", type=int, default=0,
                        help="fewer layers than the shape has, only where memory or time needs it (0: all)")
    parser.add_argument("--points", default="1,64", help="further decode batch sizes to report")
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--block-size", type=int, default=16)
    parser.add_argument("--serving", action="store_true",
                        help="instead of the headline measurement: a continuous batch of 64 requests, prompts of 128 to "
                             "8,192 random tokens in portions of 512, 256 new tokens each (the 1.5B workload; use with "
                             "--shape 1.5b --ctx 32768)")
    parser.add_argument("--cache-share", type=float, default=1.0,
                        help="with --serving: the cache pool as a share of the pages that all requests need together "
                             "(below 1 the scheduler has to hold requests back, and preempts when pages run out)")
    parser.add_argument("--split", action="store_true",
                        help="also run one decode step (of --batch requests at --ctx) and one prefill eagerly with a "
                             "pair of GPU events around every kernel launch, and add the microseconds of each class of "
                             "kernel to the line (split_decode_us, split_prefill_us)")
    parser.add_argument("--in-turn", action="store_true",
                        help="wait for a step's tokens on the host before the next step is launched")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine runs on a single MI355X, so --gpus {args.gpus} is not run")
        return 2

    still_running()

    import torch

    import vipera_rs_amd  # noqa: F401
    from vipera_rs_amd import Engine
    from vipera_rs_amd.config import config_from_dict
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    from vipera_rs_amd.models import build_model
    from vipera_rs_amd.runtime import Runtime
    from vipera_rs_amd.weights import random_device_tensors

    dtype_key = "bf16" if args.dtype == "bfloat16" else "fp32"
    element = 2 if dtype_key == "bf16" else 4
    shape_name, shape = SHAPES[args.shape]
    layers_full = shape["num_hidden_layers"]
    args.layers = args.layers or layers_full
    data = dict(shape, num_hidden_layers=args.layers)
    config = config_from_dict(data)
    runtime = Runtime("cuda:0", args.dtype)
    model = build_model(config, runtime)
    started = time.perf_counter()
    model.load(random_device_tensors(model.tensor_specs(), 0, runtime.dtype, runtime.device))
    torch.cuda.synchronize()
    log(f"random weights for {args.layers} layers on the device in {time.perf_counter() - started:.1f} s")

    if args.serving:
        return serving(args, config, runtime, model, shape_name, layers_full, dtype_key)
    batches = [args.batch] + [int(b) for b in args.points.split(",") if b.strip()]
    largest = max(batches)
    ctx = args.ctx
    pages_per_request = (ctx + args.block_size - 1) // args.block_size
    num_blocks = largest * pages_per_request + (args.prefill_tokens + args.block_size - 1) // args.block_size + 8
    runner = ModelRunner(model, runtime, args.block_size, num_blocks, largest + 1, use_graphs=True, max_context=ctx)

    H, L, V = config.hidden_size, args.layers, config.vocab_size
    Q, KV, I = config.num_attention_heads * config.head_dim, config.num_key_value_heads * config.head_dim, \
        config.intermediate_size
    layer_matrix = H * (Q + 2 * KV) + Q * H + 2 * I * H + I * H
    layer_vectors = (Q + 2 * KV) + 2 * H
    kv_per_token = 2 * KV * element * L
    weight_bytes = L * (layer_matrix * element + layer_vectors * 4) + V * H * element + H * 4  # output matrix (tied or not)

    gen = torch.Generator().manual_seed(0)

    def tokens(n):
        return torch.randint(0, V, (n,), generator=gen).tolist()

    # --- prefill of 2,048 tokens -----------------------------------------------------------------------
    T = args.prefill_tokens
    prompt = tokens(T)

    def prefill_once(request):
        runner.cache.reserve(request, 0, T)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry(request, 0, prompt, [T - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        runner.cache.release(request)
        return dt

    prefill_once(10_000)
    PREFILL_RUNS = 3     # the best of this many timed runs is reported (named in `config`)
    prefill_s = min(prefill_once(10_001 + k) for k in range(PREFILL_RUNS))
    prefill_flops = 2.0 * T * L * layer_matrix + 2.0 * V * H + L * 4.0 * config.num_attention_heads * config.head_dim \
        * (T * (T + 1) / 2)
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops / prefill_s / MFMA_PEAK[dtype_key], 4)}
    log(f"prefill {T} tokens: {prefill['ms']} ms, {prefill['value']} tok/s, {prefill['frac']:.3f} of peak")

    # --- decode ---------------------------------------------------------------------------------------------
    def decode(batch, steps, warmup):
        # every prompt gets a portion in every prefill step, so that all requests start decoding together
        engine = Engine(None, runner=runner, max_num_seqs=batch, max_num_batched_tokens=batch * 2048, chunk_size=2048,
                        max_model_len=ctx + 8, pipelined=not args.in_turn)
        prompt_len = ctx - steps - warmup - SETTLE_STEPS - 1
        for _ in range(batch):
            engine.add_request(tokens(prompt_len), max_new_tokens=steps + warmup + SETTLE_STEPS + 4)
        last = time.perf_counter()
        for guard in range(10_000):  # prefill, until every request has its first token and the next step is all decode
            if guard == 9_999 or not engine.has_work():
                raise RuntimeError("the requests ended before a step of decode tokens only was reached")
            report = engine.step()
            if time.perf_counter() - last > 20:
                log(f"  prefilling batch {batch}: {engine.scheduler.num_waiting} requests still waiting")
                last = time.perf_counter()
            if engine.scheduler.num_waiting == 0 and report.num_batched_tokens == batch:
                break
        # The GPU's power management takes about 0.2 s to settle after the change from prompts to decoding: for
        # that long every decode step takes 3.5 % longer (3.885 then 3.745 ms at batch 8, from one step to the
        # next). These untimed steps let it settle; the warm-up steps asked for follow them.
        for _ in range(SETTLE_STEPS):
            engine.step()
        for _ in range(warmup - 1):
            engine.step()
        torch.cuda.synchronize()
        engine.micros = {key: 0 for key in engine.micros}
        t0 = time.perf_counter()
        for _ in range(steps):
            report = engine.step()
            assert report.num_batched_tokens == batch and len(report.tokens) == batch
        torch.cuda.synchronize()
        seconds = time.perf_counter() - t0
        log(f"  host microseconds per step: " + ", ".join(f"{k} {v // steps}" for k, v in engine.micros.items()))
        # the same captured step replayed back to back, nothing else in the stream: what the GPU alone needs for it
        graphs = getattr(runner, "graphs", None)
        if graphs is not None and graphs.graphs:
            captured = list(graphs.graphs.values())[-1]
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(8):
                captured.graph.replay()
            torch.cuda.synchronize()
            log(f"  the step's graph alone, replayed back to back: {(time.perf_counter() - t1) / 8 * 1e3:.3f} ms "
                f"(the engine's step: {seconds / steps * 1e3:.3f} ms)")
        mean_ctx = ctx - steps / 2.0
        for request in list(engine._live):
            engine.cancel(request)
        assert runner.cache.check() == "" and runner.cache.live_requests() == 0
        step_bytes = weight_bytes + batch * H * element + batch * mean_ctx * kv_per_token
        return seconds, step_bytes

    results = {}
    for batch in batches:
        steps = args.steps if batch == args.batch else max(16, args.steps // 2)
        seconds, step_bytes = decode(batch, steps, args.warmup)
        ms = seconds / steps * 1e3
        results[batch] = {"tok_s": batch * steps / seconds, "ms": ms, "bytes": step_bytes,
                          "gbs": step_bytes / (seconds / steps) / 1e9}
        log(f"decode batch {batch}: {ms:.3f} ms/step, {results[batch]['tok_s']:.1f} tok/s, "
            f"{results[batch]['gbs']:.0f} GB/s of {HBM_PEAK / 1e9:.0f}")

    head = results[args.batch]
    line = {
        "metric": f"decode tokens per second at batch {args.batch}, context {ctx}",
        "value": round(head["tok_s"], 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_key,
        "data": "synthetic: seeded random weights N(0, 0.02) and uniform-random token ids",
        "config": {
            "model": shape_name, "layers": args.layers, "layers_full": layers_full, "hidden": H,
            "heads": config.num_attention_heads, "kv_heads": config.num_key_value_heads,
            "head_dim": config.head_dim, "intermediate": I, "vocab": V, "global_batch": args.batch,
            "seq_len": ctx, "prefill_tokens": T, "block_size": args.block_size, "parallelism": "single GPU",
            "sampling": "greedy", "weights_gb": round(weight_bytes / 1e9, 2), "steps_launched_ahead": not args.in_turn,
            "untimed_decode_steps_before_warmup": SETTLE_STEPS, "prefill_is_best_of_runs": PREFILL_RUNS,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(head["gbs"], 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(head["gbs"] * 1e9 / HBM_PEAK, 4)},
        "points": {f"decode_b{b}": round(r["tok_s"], 1) for b, r in results.items() if b != args.batch},
        "points_ms": {f"decode_b{b}": round(r["ms"], 4) for b, r in results.items() if b != args.batch},
    }
    if args.split:
        line.update(kernel_split(args, config, runner, tokens, ctx, T))
    print(json.dumps(line), flush=True)
    return 0


def kernel_split(args, config, runner, tokens, ctx, T):
    """Microseconds per class of kernel for one decode step of ``--batch`` requests at context ``ctx`` and for one
    prefill of ``T`` tokens, each the mean of five eager runs with a pair of GPU events around every launch
    (``vipera_rs_amd.ops.profile``; the reference prints such a split as its PROFILE lines,
    crates/vipera-backend-cpu/src/profile.rs:226-275).  The decode step reads a cache of ``ctx - 1`` positions per
    request that no prompt has filled: its kernels' times do not depend on what the pages hold."""
    import torch

    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.ops.profile import KernelTimer, weight_shape
    from vipera_rs_amd.sampling import BatchSampler, RowRequest, SamplingParams

    H, V, I = config.hidden_size, config.vocab_size, config.intermediate_size
    Q, KV = config.num_attention_heads * config.head_dim, config.num_key_value_heads * config.head_dim
    products = {(Q + 2 * KV, H): "qkv", (H, Q): "output", (2 * I, H): "gate_up", (H, I): "down", (V, H): "head"}
    other = {"attn_bf16_prefill": "attention", "attn_bf16_decode": "attention", "attn_generic": "attention", "attn_decode_f32": "attention", "attn_prefill_f32": "attention",
             "rmsnorm": "norms", "rope_kvwrite": "rope_kvwrite", "rope_angles": "rope_kvwrite",
             "embed_gather": "embedding", "sample": "sampler", "swiglu": "swiglu", "fetch_words": "metadata"}

    def label(name, call_args, kwargs):
        shape = weight_shape(name, call_args)
        if shape is not None:
            return products.get(shape, f"product_{shape[0]}x{shape[1]}")
        return other.get(name, name)

    sampler = BatchSampler(runner.runtime.device, slots=max(64, args.batch))
    runs = 5

    def measure(entries_of, rows):
        timer = KernelTimer(label)
        wall = 0.0
        for run in range(runs + 1):          # the first run loads what is not loaded yet and is not counted
            entries = entries_of(run)
            batch = runner.prepare(entries)
            torch.cuda.synchronize()
            if run == 0:
                logits = runner.run(batch)
                sampler.sample(logits, rows)
                continue
            with timer:
                timer.hold_back()
                start = torch.cuda.Event(enable_timing=True)
                end = torch.cuda.Event(enable_timing=True)
                start.record()
                logits = runner.run(batch)
                sampler.launch(logits, rows)
                end.record()
            torch.cuda.synchronize()
            wall += start.elapsed_time(end) * 1e3
        split = {key: round(value / runs, 1) for key, value in timer.microseconds().items()}
        split["kernels_sum"] = round(sum(v for k, v in split.items() if k != "launches"), 1)
        split["eager_step"] = round(wall / runs, 1)
        return split

    batch = args.batch
    for request in range(batch):
        runner.cache.reserve(20_000 + request, 0, ctx)
    greedy = [RowRequest(SamplingParams(), slot=k, position=ctx) for k in range(batch)]
    ids = tokens(batch)
    decode = measure(lambda run: [StepEntry(20_000 + r, ctx - 1, [ids[r]], [0]) for r in range(batch)], greedy)
    for request in range(batch):
        runner.cache.release(20_000 + request)
    prompt = tokens(T)
    runner.cache.reserve(30_000, 0, T)
    prefill = measure(lambda run: [StepEntry(30_000, 0, prompt, [T - 1])], greedy[:1])
    runner.cache.release(30_000)
    log("split of one decode step (us): " + ", ".join(f"{k} {v}" for k, v in decode.items()))
    log("split of one prefill (us): " + ", ".join(f"{k} {v}" for k, v in prefill.items()))
    return {"split_decode_us": decode, "split_prefill_us": prefill}


def serving(args, config, runtime, model, shape_name, layers_full, dtype_key) -> int:
    """Continuous batching under load: every request is queued at once, prompts run in portions of 512 beside the
    decode tokens of the requests that are further on, and the run ends when all have their 256 new tokens."""
    import torch

    from vipera_rs_amd import Engine
    from vipera_rs_amd.engine.runner import ModelRunner

    requests, new_tokens, chunk, budget = 64, 256, 512, 2048
    gen = torch.Generator().manual_seed(1)
    lengths = torch.randint(128, 8193, (requests,), generator=gen).tolist()
    prompts = [torch.randint(0, config.vocab_size, (n,), generator=gen).tolist() for n in lengths]
    needed = [(n + new_tokens + args.block_size - 1) // args.block_size + 1 for n in lengths]
    pages = max(int(sum(needed) * args.cache_share), max(needed) + 1)   # the longest request has to fit
    context = max(args.ctx, max(lengths) + new_tokens)
    runner = ModelRunner(model, runtime, args.block_size, pages, requests + 1, use_graphs=True, max_context=context)
    engine = Engine(None, runner=runner, max_num_seqs=requests, max_num_batched_tokens=budget, chunk_size=chunk,
                    max_model_len=context, pipelined=not args.in_turn)
    # a short run first: kernel modules are compiled and loaded; then the decode steps of every size are captured,
    # as a server does before it takes requests
    engine.generate([prompts[0][:600], prompts[1][:300]], 8)
    started = time.perf_counter()
    captured = engine.warm_up()
    log(f"{captured} decode steps captured ahead in {time.perf_counter() - started:.1f} s")
    for prompt in prompts:
        engine.add_request(prompt, new_tokens)
    torch.cuda.synchronize()
    started = time.perf_counter()
    steps = generated = 0
    last = started
    while engine.has_work():
        report = engine.step()
        steps += 1
        generated += len(report.tokens)
        if time.perf_counter() - last > 20:
            log(f"  serving: {steps} steps, {generated} tokens generated, {engine.scheduler.num_waiting} requests waiting")
            last = time.perf_counter()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - started
    assert generated == requests * new_tokens and runner.cache.live_requests() == 0
    prompt_tokens = sum(lengths)
    log(f"serving: {requests} requests, {prompt_tokens} prompt tokens and {generated} new tokens in {seconds:.2f} s "
        f"over {steps} steps; {engine.stats()['preemptions']} preemptions")
    print(json.dumps({
        "metric": "tokens per second (prompt and generated) of a continuous batch of 64 requests",
        "value": round((prompt_tokens + generated) / seconds, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
        "warmup": 0, "ms_per_step": round(seconds / steps * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype_key,
        "data": "synthetic: seeded random weights N(0, 0.02) and uniform-random token ids",
        "config": {"model": shape_name, "layers": args.layers, "layers_full": layers_full, "requests": requests,
                   "prompt_tokens": prompt_tokens, "new_tokens_each": new_tokens, "chunk_size": chunk,
                   "max_num_batched_tokens": budget, "seq_len": context, "block_size": args.block_size,
                   "steps_launched_ahead": not args.in_turn, "decode_steps_captured_ahead": captured,
                   "cache_pages": pages, "cache_share": args.cache_share,
                   "preemptions": engine.stats()["preemptions"]},
        "generated_per_second": round(generated / seconds, 1), "seconds": round(seconds, 3),
    }), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
