"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run has the layer sizes of Qwen3-4B with random weights (bfloat16),
eight requests decoding from 1,024-token random prompts in a cache pool sized
for the benchmark context, and prints ONE JSON line: decoded tokens a second
at batch 8 (``value``), the same at batch 1 and 64 (``points``), the prefill of
one 2,048-token prompt, and the decode step's memory roofline.  A "step" is one
decode step: every request's last token through the model, and the next token
sampled (greedy) and read back.  Everything goes through the engine's own step
function, cache and kernels.
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

QWEN3_4B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu",
    "vocab_size": 151936, "hidden_size": 2560, "intermediate_size": 9728, "num_hidden_layers": 36,
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "max_position_embeddings": 262144, "rms_norm_eps": 1e-6, "rope_theta": 5000000.0,
    "tie_word_embeddings": True, "attention_bias": False, "eos_token_id": 151645,
}


def parse_args():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=10)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--prompt-len", type=int, default=1024)
    parser.add_argument("--context", type=int, default=8192)
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--block-size", type=int, default=16)
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the model has")
    parser.add_argument("--dtype", choices=("bf16", "fp32"), default="bf16")
    parser.add_argument("--points", default="1,64", help="other decode batch sizes to report")
    parser.add_argument("--phase", choices=("all", "decode", "prefill"), default="all",
                        help="run one phase only (for profiles); the record then holds that phase alone")
    parser.add_argument("--seed", type=int, default=0)
    return parser.parse_args()


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


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2
    import torch

    from forge_engine_amd.config import load_model_config
    from forge_engine_amd.engine import ModelRunner, StepEntry, random_model
    from forge_engine_amd.sampling import SamplingParams
    from forge_engine_amd.sampling.sampler import Sampler

    raw = dict(QWEN3_4B)
    full_layers = raw["num_hidden_layers"]
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    config = load_model_config(raw)
    device = torch.device("cuda:0")
    dtype = {"bf16": "bfloat16", "fp32": "float32"}[args.dtype]
    model = random_model(config, args.seed, dtype=dtype, device=device)
    batches = sorted({args.batch, *[int(b) for b in args.points.split(",") if b]})
    if args.phase == "decode":
        batches = [args.batch]
    spare = args.steps + args.warmup + 8
    per_request = -(-(args.prompt_len + spare) // args.block_size)
    capacity = max(args.batch * -(-args.context // args.block_size), max(batches) * per_request,
                   -(-(args.prefill_tokens + 1) // args.block_size))
    runner = ModelRunner(model, block_size=args.block_size, block_capacity=capacity,
                         num_state_slots=max(batches) + 1)
    sampler = Sampler(device)
    greedy = SamplingParams()
    generator = torch.Generator().manual_seed(args.seed)

    def random_tokens(n):
        return torch.randint(0, config.vocab_size, (n,), generator=generator).tolist()

    def timed(fn, warmup, steps):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        start = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - start) / steps

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

        seconds = timed(one_step, args.warmup, args.steps)
        contexts = [runner.length(n) for n in names]
        for name in names:
            runner.end(name)
        return seconds, sum(contexts) / batch - args.steps / 2.0

    if args.phase == "prefill":
        results = {}
    else:
        results = {b: decode_run(b) for b in batches}

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

    if args.phase == "decode":
        seconds = results[args.batch][0]
        print(json.dumps({"phase": "decode", "batch": args.batch, "ms_per_step": round(seconds * 1e3, 4),
                          "value": round(args.batch / seconds, 2), "unit": "tokens/s"}))
        return 0
    prefill_seconds = timed(prefill_once, 2, max(3, min(10, args.steps)))
    if args.phase == "prefill":
        print(json.dumps({"phase": "prefill", "tokens": args.prefill_tokens, "ms": round(prefill_seconds * 1e3, 3),
                          "value": round(args.prefill_tokens / prefill_seconds, 1), "unit": "tokens/s"}))
        return 0

    layers = config.num_hidden_layers
    matrix_params = layers * (config.hidden_size * (config.q_size + 2 * config.kv_size)
                              + config.q_size * config.hidden_size
                              + 3 * config.hidden_size * config.intermediate_size)
    t = args.prefill_tokens
    prefill_flops = 2.0 * t * matrix_params + 2.0 * t * t * config.q_size * layers \
        + 2.0 * config.vocab_size * config.hidden_size
    element = 2 if args.dtype == "bf16" else 4
    kv_bytes_per_token = 2 * layers * config.kv_size * element
    seconds, mean_ctx = results[args.batch]
    step_bytes = weight_bytes(model) + args.batch * mean_ctx * kv_bytes_per_token
    achieved = step_bytes / seconds / 1e9
    record = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen3-4B sizes, {args.prompt_len}-token prompts)",
        "value": round(args.batch / seconds, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(seconds * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic: random weights drawn on the device, uniform-random token ids",
        "config": {
            "model": "Qwen3-4B sizes (Qwen3ForCausalLM)", "global_batch": args.batch,
            "seq_len": args.prompt_len, "parallelism": "single GPU", "context": args.context,
            "block_size": args.block_size, "layers_run": layers, "layers_model": full_layers,
            "hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size,
            "q_heads": config.num_attention_heads, "kv_heads": config.num_key_value_heads,
            "head_dim": config.head_dim, "vocab_size": config.vocab_size,
            "tied_embeddings": config.tie_word_embeddings, "rope_theta": config.rope_theta,
            "prefill_tokens": args.prefill_tokens, "sampling": "greedy",
        },
        "prefill": {
            "value": round(t / prefill_seconds, 1), "tokens": t, "ms": round(prefill_seconds * 1e3, 3),
            "frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS[args.dtype], 4),
        },
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
            "frac": round(achieved / (HBM_BYTES_PER_S / 1e9), 4),
        },
        "points": {f"decode_b{b}": round(b / results[b][0], 2) for b in batches if b != args.batch},
    }
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
