"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model qwen3-4b|qwen3-8b|qwen3-14b|qwen3-32b|qwen3-0.6b|qwen3-1.7b]

The default run has the layer sizes of Qwen3-4B with random weights (bfloat16),
eight requests decoding from 1,024-token random prompts in a cache pool sized
for the benchmark context, and prints ONE JSON line: decoded tokens a second
at batch 8 (``value``), the same at batch 1 and 64 (``points``), the prefill of
one 2,048-token prompt, and the decode step's memory roofline.  A "step" is one
decode step: every request's last token through the model, and the next token
sampled (greedy) and read back.  The sampled tokens are fed to the next step on
the device and read by the host while that step runs (``--no-overlap`` reads
them before the next step is launched).  Everything goes through the engine's
own step function, cache and kernels.

Protocol (after tools/validate_l4.py:136-183 of the reference): W untimed steps,
then K steps each bracketed by a pair of device events; the line reports their
minimum, 10th percentile, median, 90th percentile and maximum, ``value`` is
batch / median, and ``ms_per_step_wall`` is the host's clock over the same K
steps (synchronised on both sides).  The roofline is given against the
published peak and against a streaming read measured when the program starts.

``--through scheduler`` decodes through ``ConcurrentGenerationEngine.step()``
(admission, selection, sampling and finishing included) instead of calling the
step function directly.  ``--workload mixed`` runs requests with prompts of
random lengths to completion through the scheduler and reports the whole job.
``--phase check`` times nothing: it feeds one prompt of ``--prefill-tokens`` whole
and eight more tokens one by one through the chosen model in bfloat16 and in
32-bit, built from the same seed, and prints how far the logits lie apart.
"""

from __future__ import annotations

import argparse
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def _qwen3(**sizes) -> dict:
    base = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu",
            "vocab_size": 151936, "num_key_value_heads": 8, "head_dim": 128, "max_position_embeddings": 262144,
            "rms_norm_eps": 1e-6, "attention_bias": False, "eos_token_id": 151645}
    base.update(sizes)
    return base


# Sizes and workloads of the three models the benchmark names (and one between them); the first is the default.
MODELS = {
    "qwen3-4b": {
        "label": "Qwen3-4B",
        "config": _qwen3(hidden_size=2560, intermediate_size=9728, num_hidden_layers=36, num_attention_heads=32,
                         rope_theta=5000000.0, tie_word_embeddings=True),
        "batch": 8, "points": "1,64", "prompt_len": 1024, "context": 8192,
    },
    "qwen3-8b": {
        "label": "Qwen3-8B",
        "config": _qwen3(hidden_size=4096, intermediate_size=12288, num_hidden_layers=36, num_attention_heads=32,
                         rope_theta=1000000.0, tie_word_embeddings=False),
        "batch": 8, "points": "1,64", "prompt_len": 1024, "context": 8192,
    },
    # beside the three: the sizes between them, so that choices measured at those are checked at one more width
    "qwen3-14b": {
        "label": "Qwen3-14B",
        "config": _qwen3(hidden_size=5120, intermediate_size=17408, num_hidden_layers=40, num_attention_heads=40,
                         rope_theta=1000000.0, tie_word_embeddings=False),
        "batch": 8, "points": "1,64", "prompt_len": 1024, "context": 8192,
    },
    # ... and the two smallest of the family, whose products have fewer blocks than the chip has CUs
    "qwen3-0.6b": {
        "label": "Qwen3-0.6B",
        "config": _qwen3(hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16,
                         rope_theta=1000000.0, tie_word_embeddings=True),
        "batch": 8, "points": "1,64", "prompt_len": 1024, "context": 8192,
    },
    "qwen3-1.7b": {
        "label": "Qwen3-1.7B",
        "config": _qwen3(hidden_size=2048, intermediate_size=6144, num_hidden_layers=28, num_attention_heads=16,
                         rope_theta=1000000.0, tie_word_embeddings=True),
        "batch": 8, "points": "1,64", "prompt_len": 1024, "context": 8192,
    },
    "qwen3-32b": {
        "label": "Qwen3-32B",
        "config": _qwen3(hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64,
                         rope_theta=1000000.0, tie_word_embeddings=False),
        "batch": 8, "points": "1,32", "prompt_len": 2048, "context": 16384,
    },
}


def parse_args():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=10)
    parser.add_argument("--model", choices=sorted(MODELS), default="qwen3-4b")
    parser.add_argument("--batch", type=int, default=None)
    parser.add_argument("--prompt-len", type=int, default=None)
    parser.add_argument("--context", type=int, default=None)
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--block-size", type=int, default=16)
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the model has")
    parser.add_argument("--dtype", choices=("bf16", "fp32"), default="bf16")
    parser.add_argument("--points", default=None, help="other decode batch sizes to report")
    parser.add_argument("--phase", choices=("all", "decode", "prefill", "micro", "check"), default="all",
                        help="run one phase only (for profiles); the record then holds that phase alone")
    parser.add_argument("--through", choices=("step", "scheduler"), default="step",
                        help="decode by calling the step function, or through the scheduler's step()")
    parser.add_argument("--workload", choices=("steady", "mixed"), default="steady",
                        help="mixed: requests with prompts of random lengths run to completion through the scheduler")
    parser.add_argument("--requests", type=int, default=64, help="mixed workload: number of requests")
    parser.add_argument("--prompt-range", default="128,4096", help="mixed workload: prompt lengths, uniform")
    parser.add_argument("--new-tokens", type=int, default=256, help="mixed workload: tokens generated per request")
    parser.add_argument("--token-budget", type=int, default=2048, help="scheduler: tokens a step")
    parser.add_argument("--sampled", action="store_true",
                        help="through the scheduler: draw with temperature 0.8, top-k 50, top-p 0.9 instead of the arg-max")
    parser.add_argument("--no-overlap", dest="overlap", action="store_false",
                        help="read every step's tokens back before the next step is launched")
    parser.add_argument("--seed", type=int, default=0)
    args = parser.parse_args()
    chosen = MODELS[args.model]
    for name in ("batch", "prompt_len", "context", "points"):
        if getattr(args, name) is None:
            setattr(args, name, chosen[name])
    return args


def weight_bytes(model) -> int:
    """Bytes of every tensor a decode step reads once (the embedding matrix
    counts once: as the head of a tied model, or as the head's own matrix)."""
    seen, total = set(), 0
    for part in model.parts():
        for value in vars(part).values():
            if hasattr(value, "data_ptr") and hasattr(value, "element_size") and value.data_ptr() not in seen:
                seen.add(value.data_ptr())
                total += value.numel() * value.element_size()
    if not getattr(model.head, "tied", False):
        total -= model.embedding.weight.numel() * model.embedding.weight.element_size()
    return total


def percentile(ordered: list[float], fraction: float) -> float:
    """Linear interpolation between the two nearest of the sorted values."""
    at = fraction * (len(ordered) - 1)
    low = int(at)
    high = min(low + 1, len(ordered) - 1)
    return ordered[low] + (ordered[high] - ordered[low]) * (at - low)


def spread(times_ms: list[float]) -> dict:
    ordered = sorted(times_ms)
    return {"min": round(ordered[0], 4), "p10": round(percentile(ordered, 0.1), 4),
            "median": round(percentile(ordered, 0.5), 4), "p90": round(percentile(ordered, 0.9), 4),
            "max": round(ordered[-1], 4)}


def micro_benchmarks() -> int:
    """The three kernel measurements that the reference publishes (docs/benchmarks.md:27-29,
    results/l4-v0.1.0.json:51-65; one NVIDIA L4), with its shapes and its protocol
    (tools/validate_l4.py:136-183: 10 warm-up calls, 50 timed ones, a pair of device events around
    each call, the median), on this engine's kernels.  A call is timed as the reference times it,
    from the host, so a few microseconds of every figure are the launch."""
    import torch

    from forge_engine_amd.kernels import ops

    device = torch.device("cuda:0")
    generator = torch.Generator(device=device).manual_seed(0)

    def rand(*shape, dtype=torch.bfloat16):
        return torch.randn(*shape, generator=generator, device=device, dtype=torch.float32).to(dtype)

    def measure(fn):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(50)]
        for begin, end in events:
            begin.record()
            fn()
            end.record()
        torch.cuda.synchronize()
        return spread([begin.elapsed_time(end) for begin, end in events])

    record = {"phase": "micro", "protocol": "10 warm-up, 50 timed, device events around each call, milliseconds"}

    # residual add + RMSNorm, [512, 2560]: the stream is float32 here, the update and the result bfloat16
    stream, update = rand(512, 2560, dtype=torch.float32), rand(512, 2560)
    weight, normed = rand(2560, dtype=torch.float32), torch.empty(512, 2560, dtype=torch.bfloat16, device=device)
    record["residual_add_rms_norm_512x2560"] = dict(measure(lambda: ops.add_rmsnorm(stream, update, weight, 1e-6, normed)),
                                                    reference_l4_ms=0.0850)

    def paged(context, q_tokens, q_heads, kv_heads):
        pages = -(-context // 16)
        keys, values = rand(pages + 1, kv_heads, 16, 128), rand(pages + 1, kv_heads, 128, 16)
        q = rand(q_tokens, q_heads * 128)
        out = torch.empty(q_tokens, q_heads * 128, dtype=torch.bfloat16, device=device)
        cu = torch.tensor([0, q_tokens], dtype=torch.int32, device=device)
        ctx = torch.tensor([context], dtype=torch.int32, device=device)
        table = torch.arange(pages, dtype=torch.int32, device=device).view(1, pages)
        return lambda: ops.paged_attention(q, keys, values, out, cu, ctx, table, num_seqs=1, max_q_len=q_tokens,
                                           q_heads=q_heads, kv_heads=kv_heads, head_dim=128, scale=128 ** -0.5,
                                           num_decode=1 if q_tokens == 1 else 0, max_ctx=context)

    # causal attention of a 128-token prompt, 8 heads of 128 (the reference's [1, 8, 128, 128]), over the paged cache
    record["causal_prefill_1x8x128x128"] = dict(measure(paged(128, 128, 8, 8)), reference_l4_ms=0.0891)
    # one decoded token over 127 cached keys and its own, 32 query heads, 8 kv heads of 128, pages of 16
    record["paged_gqa_decode_past127_q32_kv8"] = dict(measure(paged(128, 1, 32, 8)), reference_l4_ms=0.1004)

    # beside the reference's three: a sampling call for 8 and 64 rows of a 151,936-token vocabulary with
    # temperature, top-k, top-p and min-p (parameters packed and sent, the kernel's launches, tokens read back)
    from forge_engine_amd.sampling import SamplingParams
    from forge_engine_amd.sampling.sampler import Sampler

    sampler = Sampler(device)
    for rows in (8, 64):
        logits = rand(rows, 151936, dtype=torch.float32) * 3
        params = [SamplingParams(temperature=0.8, top_k=50, top_p=0.9, min_p=0.05, seed=1)] * rows
        seeds, draws = list(range(rows)), [3] * rows
        record[f"sample_top_k_top_p_min_p_{rows}x151936"] = measure(lambda: sampler.sample(logits, params, seeds, draws))
    print(json.dumps(record))
    return 0


def cross_check(args) -> int:
    """The model at the benchmark's sizes in bfloat16 against the same weights in 32-bit: a
    prompt whole (logits at a place in its middle and at its end), then eight single tokens.
    Rounding grows slowly with the number of layers; a kernel that is wrong at these sizes
    only (a width, a head count, a cache of this length) shows as a jump."""
    import torch

    from forge_engine_amd.config import load_model_config
    from forge_engine_amd.engine import ModelRunner, StepEntry, random_model

    chosen = MODELS[args.model]
    raw = dict(chosen["config"])
    full_layers = raw["num_hidden_layers"]
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    config = load_model_config(raw)
    prompt = args.prefill_tokens
    generator = torch.Generator().manual_seed(args.seed)
    tokens = torch.randint(0, config.vocab_size, (prompt + 8,), generator=generator).tolist()
    rows = {}
    for dtype in ("bfloat16", "float32"):
        model = random_model(config, args.seed, dtype=dtype, device=torch.device("cuda:0"))
        runner = ModelRunner(model, block_size=args.block_size,
                             block_capacity=-(-(prompt + 8) // args.block_size) + 1, num_state_slots=2)
        runner.begin("a")
        got = [runner.step([StepEntry("a", tokens[:prompt], [prompt // 2, prompt - 1])]).float().cpu()]
        for token in tokens[prompt:]:
            got.append(runner.step([StepEntry("a", [token], [0])]).float().cpu())
        rows[dtype] = torch.cat(got)
        del runner, model
        torch.cuda.empty_cache()
    want, got = rows["float32"], rows["bfloat16"]
    scale = float(want.abs().max())
    apart = (got - want).abs().max(dim=1).values
    print(json.dumps({
        "check": "bfloat16 against float32", "model": chosen["label"], "layers_run": config.num_hidden_layers,
        "layers_model": full_layers, "prompt_tokens": prompt, "rows": len(apart), "largest_logit": round(scale, 3),
        "largest_difference": round(float(apart.max()), 4), "fraction": round(float(apart.max()) / scale, 4),
        "argmax_agree": int((got.argmax(1) == want.argmax(1)).sum()),
    }))
    return 0


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2
    if args.phase == "micro":
        return micro_benchmarks()
    if args.phase == "check":
        return cross_check(args)
    import torch

    from forge_engine_amd.config import SchedulerConfig, load_model_config
    from forge_engine_amd.engine import ModelRunner, StepEntry, random_model
    from forge_engine_amd.engine.scheduler import ConcurrentGenerationEngine
    from forge_engine_amd.sampling import SamplingParams
    from forge_engine_amd.sampling.sampler import Sampler

    chosen = MODELS[args.model]
    raw = dict(chosen["config"])
    full_layers = raw["num_hidden_layers"]
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    config = load_model_config(raw)
    device = torch.device("cuda:0")
    dtype = {"bf16": "bfloat16", "fp32": "float32"}[args.dtype]

    def timed(fn, warmup, steps):
        """Per-step device times (ms) of ``steps`` calls after ``warmup`` untimed ones, and the
        host's mean over the same calls."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        start = time.perf_counter()
        for begin, end in events:
            begin.record()
            fn()
            end.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - start) / steps
        return [begin.elapsed_time(end) for begin, end in events], wall * 1e3

    def measured_read_bandwidth() -> float:
        """Bytes a second of a plain streaming read: a kernel that only reads, over four 400 MB
        buffers in turn so that no cache holds what it reads, twenty times between one pair of
        device events."""
        from forge_engine_amd.kernels import ops

        buffers = [torch.zeros(100_000_000, dtype=torch.float32, device=device) for _ in range(4)]
        sink = torch.zeros(1, dtype=torch.float32, device=device)
        for data in buffers:
            ops.stream_read(data, sink)
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        for index in range(20):
            ops.stream_read(buffers[index % 4], sink)
        end.record()
        torch.cuda.synchronize()
        seconds = begin.elapsed_time(end) * 1e-3 / 20
        return 400_000_000 / seconds

    read_peak = measured_read_bandwidth()
    model = random_model(config, args.seed, dtype=dtype, device=device)
    sampler = Sampler(device)
    greedy = SamplingParams()
    generator = torch.Generator().manual_seed(args.seed)

    def random_tokens(n):
        return torch.randint(0, config.vocab_size, (n,), generator=generator).tolist()

    element = 2 if args.dtype == "bf16" else 4
    layers = config.num_hidden_layers
    kv_bytes_per_token = 2 * layers * config.kv_size * element

    if args.workload == "mixed":
        low, high = (int(v) for v in args.prompt_range.split(","))
        lengths = torch.randint(low, high + 1, (args.requests,), generator=generator).tolist()
        pages = sum(-(-(n + args.new_tokens) // args.block_size) for n in lengths)
        runner = ModelRunner(model, block_size=args.block_size, block_capacity=pages, num_state_slots=args.requests)
        scheduler = SchedulerConfig(max_requests=args.requests, max_batch_size=min(64, args.requests),
                                    token_budget=args.token_budget, block_size=args.block_size, block_capacity=pages,
                                    max_context=args.context)
        engine = ConcurrentGenerationEngine(runner, sampler, greedy, scheduler, eos_token_ids=())
        for round_index in range(2):        # the first round warms up (graphs are captured), the second is timed
            ids = [engine.submit(random_tokens(n), sampling_params=SamplingParams(max_new_tokens=args.new_tokens))
                   for n in lengths]
            torch.cuda.synchronize()
            start = time.perf_counter()
            steps = 0
            while not engine.idle:
                engine.step()
                steps += 1
            torch.cuda.synchronize()
            seconds = time.perf_counter() - start
            for request_id in ids:
                engine.forget(request_id)
        generated = args.requests * args.new_tokens
        print(json.dumps({
            "workload": "mixed", "through": "scheduler", "model": chosen["label"], "dtype": args.dtype,
            "requests": args.requests, "prompt_tokens": sum(lengths), "generated_tokens": generated,
            "token_budget": args.token_budget, "steps": steps, "seconds": round(seconds, 3),
            "generated_tokens_per_s": round(generated / seconds, 1),
            "all_tokens_per_s": round((generated + sum(lengths)) / seconds, 1),
            "layers_run": layers, "layers_model": full_layers,
        }))
        return 0

    batches = sorted({args.batch, *[int(b) for b in args.points.split(",") if b]})
    if args.phase == "decode" or args.through == "scheduler":
        batches = [args.batch]
    spare = args.steps + args.warmup + 8
    # through the scheduler the first requests already decode while the last prompts are still fed
    joining = max(batches) * args.prompt_len // max(args.token_budget, 1) + 2 if args.through == "scheduler" else 0
    spare += joining
    per_request = -(-(args.prompt_len + spare) // args.block_size)
    capacity = max(args.batch * -(-args.context // args.block_size), max(batches) * per_request,
                   -(-(args.prefill_tokens + 1) // args.block_size))
    runner = ModelRunner(model, block_size=args.block_size, block_capacity=capacity,
                         num_state_slots=max(batches) + 1, eager_sightings=1)   # the timed loops repeat one shape

    def decode_run(batch):
        names = [f"d{batch}_{i}" for i in range(batch)]
        state = {}
        for name in names:
            runner.begin(name)
            prompt = random_tokens(args.prompt_len)
            for at in range(0, len(prompt), 2048):      # untimed: fill the cache
                portion = prompt[at:at + 2048]
                last = at + 2048 >= len(prompt)
                logits = runner.step([StepEntry(name, portion, [len(portion) - 1] if last else [])])
            state[name] = sampler.sample(logits, [greedy], [0], [0])[0]

        def one_step():
            logits = runner.step([StepEntry(n, [state[n]], [0]) for n in names])
            tokens = sampler.sample(logits, [greedy] * batch, [0] * batch, [0] * batch)
            for n, t in zip(names, tokens):
                state[n] = t

        # The sampled tokens go into the next step on the device, and the host reads them while
        # that step runs (a step late): the GPU does not wait for the host between two steps.
        placeholders = [StepEntry(n, [0], [0]) for n in names]
        flight = {"feed": torch.tensor([state[n] for n in names], dtype=torch.int32, device=device), "unread": None}

        def one_overlapped_step():
            logits = runner.step(placeholders, device_tokens=flight["feed"])
            both = sampler.sample_greedy_on_device(logits)
            if flight["unread"] is not None:
                sampler.read(flight["unread"])
            flight["unread"], flight["feed"] = both, both[0]

        overlapped = args.overlap and runner.feeds_from_device(placeholders)
        times, wall = timed(one_overlapped_step if overlapped else one_step, args.warmup, args.steps)
        contexts = [runner.length(n) for n in names]
        for name in names:
            runner.end(name)
        return times, wall, sum(contexts) / batch - args.steps / 2.0

    def scheduler_run(batch):
        """The same decode steps through the scheduler: requests are admitted with their prompts,
        stepped until every one decodes, then K calls of step() are timed."""
        scheduler = SchedulerConfig(max_requests=batch, max_batch_size=batch, token_budget=max(args.token_budget, batch),
                                    block_size=args.block_size, block_capacity=capacity, overlap_decode=args.overlap)
        engine = ConcurrentGenerationEngine(runner, sampler, greedy, scheduler, eos_token_ids=())
        limit = args.steps + args.warmup + 4 + joining
        drawn = dict(temperature=0.8, top_k=50, top_p=0.9) if args.sampled else {}
        ids = [engine.submit(random_tokens(args.prompt_len), sampling_params=SamplingParams(max_new_tokens=limit, seed=i, **drawn))
               for i in range(batch)]
        while any(n != 1 for n in engine.snapshot().last_batch_tokens) or len(engine.snapshot().last_batch) != batch:
            engine.step()
        times, wall = timed(engine.step, args.warmup, args.steps)
        mean_ctx = sum(runner.length(request_id) for request_id in ids) / batch - args.steps / 2.0
        for request_id in ids:
            engine.cancel(request_id)
        return times, wall, mean_ctx

    run = scheduler_run if args.through == "scheduler" else decode_run
    results = {} if args.phase == "prefill" else {b: run(b) for b in batches}

    # prefill: one whole prompt in one step, logits at its last token
    prompt = random_tokens(args.prefill_tokens)
    counter = [0]

    def prefill_once():
        name = f"p{counter[0]}"
        counter[0] += 1
        runner.begin(name)
        logits = runner.step([StepEntry(name, prompt, [len(prompt) - 1])])
        sampler.sample(logits, [greedy], [0], [0])
        runner.end(name)

    def roofline(batch, times, mean_ctx):
        seconds = spread(times)["median"] * 1e-3
        step_bytes = weight_bytes(model) + batch * mean_ctx * kv_bytes_per_token
        achieved = step_bytes / seconds
        return {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                "frac": round(achieved / HBM_BYTES_PER_S, 4), "measured_peak": round(read_peak / 1e9, 1),
                "frac_measured": round(achieved / read_peak, 4)}

    if args.phase == "decode" or args.through == "scheduler":
        times, wall, mean_ctx = results[args.batch]
        median = spread(times)["median"]
        print(json.dumps({"phase": "decode", "through": args.through, "model": chosen["label"], "batch": args.batch,
                          "ms_per_step": median, "ms_per_step_wall": round(wall, 4), "step_ms": spread(times),
                          "value": round(args.batch / median * 1e3, 2), "unit": "tokens/s",
                          "roofline": roofline(args.batch, times, mean_ctx),
                          "layers_run": layers, "layers_model": full_layers}))
        return 0
    prefill_times, _ = timed(prefill_once, 2, max(3, min(10, args.steps)))
    prefill_ms = spread(prefill_times)["median"]
    matrix_params = layers * (config.hidden_size * (config.q_size + 2 * config.kv_size)
                              + config.q_size * config.hidden_size
                              + 3 * config.hidden_size * config.intermediate_size)
    t = args.prefill_tokens
    prefill_flops = 2.0 * t * matrix_params + 2.0 * t * t * config.q_size * layers \
        + 2.0 * config.vocab_size * config.hidden_size
    if args.phase == "prefill":
        print(json.dumps({"phase": "prefill", "model": chosen["label"], "dtype": args.dtype, "tokens": t, "ms": prefill_ms,
                          "step_ms": spread(prefill_times),
                          "value": round(t / prefill_ms * 1e3, 1), "unit": "tokens/s",
                          "frac": round(prefill_flops / (prefill_ms * 1e-3) / PEAK_FLOPS[args.dtype], 4),
                          "peak_tflops": PEAK_FLOPS[args.dtype] / 1e12,
                          "layers_run": layers, "layers_model": full_layers}))
        return 0

    times, wall, mean_ctx = results[args.batch]
    median = spread(times)["median"]
    record = {
        "metric": f"decode tok/s at batch {args.batch} ({chosen['label']} sizes, {args.prompt_len}-token prompts)",
        "value": round(args.batch / median * 1e3, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": median,
        "ms_per_step_wall": round(wall, 4),
        "step_ms": spread(times),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic: random weights drawn on the device, uniform-random token ids",
        "config": {
            "model": f"{chosen['label']} sizes (Qwen3ForCausalLM)", "global_batch": args.batch,
            "seq_len": args.prompt_len, "parallelism": "single GPU", "context": args.context,
            "block_size": args.block_size, "layers_run": layers, "layers_model": full_layers,
            "hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size,
            "q_heads": config.num_attention_heads, "kv_heads": config.num_key_value_heads,
            "head_dim": config.head_dim, "vocab_size": config.vocab_size,
            "tied_embeddings": config.tie_word_embeddings, "rope_theta": config.rope_theta,
            "prefill_tokens": args.prefill_tokens, "sampling": "greedy",
        },
        "prefill": {
            "value": round(t / prefill_ms * 1e3, 1), "tokens": t, "ms": prefill_ms,
            "frac": round(prefill_flops / (prefill_ms * 1e-3) / PEAK_FLOPS[args.dtype], 4),
        },
        "roofline": roofline(args.batch, times, mean_ctx),
        "points": {f"decode_b{b}": round(b / spread(results[b][0])["median"] * 1e3, 2) for b in batches if b != args.batch},
    }
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
