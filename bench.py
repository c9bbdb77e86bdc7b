"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The default run has the layer sizes of Qwen2.5-1.5B (configs/qwen2.5-1.5b.json) with seeded
random bfloat16 weights: 8 requests with 512-token prompts are prefilled, then decoded
through the engine's own iteration loop (scheduler, step function, sampling, one token per
request per step).  W untimed decode steps, then exactly K timed ones between device
synchronisations.  One JSON line is printed: decoded tokens a second, the prefill of a
2,048-token prompt, the decode step's share of the HBM roofline, and decoding at batch 1 and 64.
"""

from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}  # dense MFMA, published


def parse() -> argparse.Namespace:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--prompt-len", type=int, default=512)
    parser.add_argument("--prefill-len", type=int, default=2048)
    parser.add_argument("--config", default=str(ROOT / "configs" / "qwen2.5-1.5b.json"))
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--seed", type=int, default=7)
    parser.add_argument("--skip-points", action="store_true", help="leave out batch 1 and 64")
    return parser.parse_args()


def main() -> int:
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not measured")
        return 2

    import dataclasses

    import torch

    from llmserve_amd import CacheConfig, EngineCore, GenerationConfig, ModelRunner, Qwen2Config, SchedulerConfig, StepEntry
    from llmserve_amd.engine import RequestState
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.weights import random_model, run_dtype

    full = Qwen2Config.from_json_file(args.config)
    config = dataclasses.replace(full, num_layers=args.layers) if args.layers else full
    dtype = run_dtype(args.dtype)
    device = torch.device("cuda:0")
    loaded = random_model(config, args.seed, dtype=dtype, device=device)
    tensors, spec = loaded.tensors, loaded.spec
    kernels = HipKernels(dtype, device)
    page = 16
    most = max(64, args.batch)
    per_request = args.prompt_len + 256 + page
    pages = most * (-(-per_request // page)) + args.prefill_len // page + 8
    runner = ModelRunner(loaded, kernels, CacheConfig(block_size=page, num_blocks=pages, max_sequences=most + 1))
    weight_bytes = sum(t.numel() * t.element_size() for t in tensors.values())
    element = 2 if dtype == torch.bfloat16 else 4
    kv_bytes_per_token = 2 * config.num_layers * config.num_key_value_heads * config.head_dim * element
    generator = torch.Generator().manual_seed(args.seed)

    def tokens(count: int) -> list[int]:
        return torch.randint(4, config.vocab_size, (count,), generator=generator).tolist()

    def decode(batch: int, steps: int, warmup: int) -> tuple[float, float]:
        """(seconds for `steps` decode steps, mean context length during them)"""
        core = EngineCore(runner, SchedulerConfig(batch, max(2048, batch)), prefill_chunk_size=512)
        requests = []
        for index in range(batch):
            request = RequestState(f"b{batch}-{index}", tokens(args.prompt_len), warmup + steps + 1)
            core.submit(request, GenerationConfig(max_new_tokens=warmup + steps + 1))
            requests.append(request)
        while any(not r.generated_token_ids for r in requests):
            core.step()
        for _ in range(warmup):
            core.step()
        torch.cuda.synchronize()
        started = time.perf_counter()
        for _ in range(steps):
            core.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        assert all(len(r.generated_token_ids) == 1 + warmup + steps for r in requests)
        for request in requests:
            core.finish(request)
        return elapsed, args.prompt_len + 1 + warmup + (steps - 1) / 2.0

    def prefill(length: int, repeats: int = 5) -> float:
        times = []
        for repeat in range(repeats + 1):
            prompt = tokens(length)
            torch.cuda.synchronize()
            started = time.perf_counter()
            runner.step([StepEntry(f"p{repeat}", prompt, [length - 1])], create_missing=True)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - started)
            runner.end_request(f"p{repeat}")
        return statistics.median(times[1:])

    steps = min(args.steps, 250 - args.warmup)
    elapsed, context = decode(args.batch, steps, args.warmup)
    value = args.batch * steps / elapsed
    step_bytes = weight_bytes + args.batch * context * kv_bytes_per_token
    achieved = step_bytes / (elapsed / steps) / 1e9

    prefill_seconds = prefill(args.prefill_len)
    layer_weights = sum(
        t.numel() for name, t in tensors.items() if t.ndim == 2 and name != spec.embedding_name and name != spec.head_name
    )
    t = args.prefill_len
    flops = 2.0 * t * layer_weights + 2.0 * config.vocab_size * config.hidden_size
    flops += config.num_layers * 4.0 * config.num_attention_heads * config.head_dim * t * (t + 1) / 2
    peak = PEAK_FLOPS["bf16" if dtype == torch.bfloat16 else "fp32"]

    points = {}
    if not args.skip_points:
        for batch in (1, 64):
            short = min(steps, 64)
            seconds, _ = decode(batch, short, min(args.warmup, 8))
            points[f"decode_b{batch}"] = round(batch * short / seconds, 1)

    label = Path(args.config).stem.replace("qwen", "Qwen").replace("b", "B")
    record = {
        "metric": f"decode tok/s at batch {args.batch}, {args.prompt_len}-token prompts ({label} shape)",
        "value": round(value, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": args.warmup,
        "ms_per_step": round(1000 * elapsed / steps, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "fp32",
        "data": "synthetic: seeded random weights, uniform random token ids",
        "config": {
            "model": f"{label} layer sizes, random weights",
            "layers": config.num_layers,
            "layers_full": full.num_layers,
            "hidden": config.hidden_size,
            "heads": config.num_attention_heads,
            "kv_heads": config.num_key_value_heads,
            "head_dim": config.head_dim,
            "intermediate": config.intermediate_size,
            "vocab": config.vocab_size,
            "rope_theta": config.rope_theta,
            "rms_norm_eps": config.rms_norm_eps,
            "tied_embeddings": config.tie_word_embeddings,
            "max_context": config.max_position_embeddings,
            "page_size": page,
            "global_batch": args.batch,
            "seq_len": args.prompt_len,
            "decode_context": round(context, 1),
            "output_tokens": 256,
            "parallelism": "none (1 GPU)",
        },
        "prefill": {
            "value": round(t / prefill_seconds, 1),
            "tokens": t,
            "ms": round(1000 * prefill_seconds, 3),
            "frac": round(flops / prefill_seconds / peak, 4),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
        },
        "points": points,
    }
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
