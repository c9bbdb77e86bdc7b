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
    parser.add_argument("--skip-context-points", action="store_true",
                        help="leave out decoding at contexts of 8k and 30k (batch 8) and 4k (batch 64)")
    return parser.parse_args()


def main() -> int:
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not measured")
        return 2

    import dataclasses

    import torch

    from llmserve_amd import CacheConfig, EngineCore, GenerationConfig, ModelRunner, SchedulerConfig, StepEntry
    from llmserve_amd.engine import Request
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.weights import random_model, read_config, run_dtype

    _, full = read_config(args.config)  # the architecture is whatever the file names
    config = dataclasses.replace(full, num_layers=args.layers) if args.layers else full
    dtype = run_dtype(args.dtype)
    device = torch.device("cuda:0")
    loaded = random_model(config, args.seed, dtype=dtype, device=device)
    tensors, spec = loaded.tensors, loaded.spec
    kernels = HipKernels(dtype, device)
    page = 16
    # (batch, prompt length) of every decode measurement: the headline, batch 1 and 64, and longer contexts
    headline = (args.batch, args.prompt_len)
    extra = {} if args.skip_points else {"decode_b1": (1, args.prompt_len), "decode_b64": (64, args.prompt_len)}
    if not args.skip_points and not args.skip_context_points:
        extra.update({"decode_b8_ctx8k": (8, 8192), "decode_b8_ctx30k": (8, 30000), "decode_b64_ctx4k": (64, 4096)})
    longest = getattr(config, "max_position_embeddings", 32768)
    steps = min(args.steps, 250 - args.warmup)

    def budget(batch: int) -> int:
        return max(2048, batch)  # tokens a step

    def output_tokens(batch: int, prompt: int) -> int:
        """How many tokens a request of a decode measurement may generate.  Prompts come in portions under
        the step's token budget, so the requests finish their prompts in different steps and those that
        finish first decode meanwhile: with this many tokens none of them ends before the timed steps do."""
        steps_of_prompts = -(-batch * prompt // budget(batch)) + batch
        return steps_of_prompts + args.warmup + steps + 1

    extra = {name: shape for name, shape in extra.items() if shape[1] + output_tokens(*shape) <= longest}
    most = max(batch for batch, _ in [headline, *extra.values()])
    pages = max(
        batch * (-(-(prompt + output_tokens(batch, prompt) + page) // page)) for batch, prompt in [headline, *extra.values()]
    )
    pages += args.prefill_len // page + 8
    runner = ModelRunner(loaded, kernels, CacheConfig(block_size=page, num_blocks=pages, max_sequences=most + 1))
    # What a decode step has to read: every weight it uses once (of an untied embedding table only the
    # rows of the step's tokens) and the cache of the live requests.
    weight_bytes = sum(t.numel() * t.element_size() for t in tensors.values())
    embedding_bytes = 0
    if not spec.tie_embeddings:
        table = tensors[spec.embedding_name]
        embedding_bytes = table.numel() * table.element_size()
        weight_bytes -= embedding_bytes
    embedding_row_bytes = spec.hidden_size * tensors[spec.embedding_name].element_size() if embedding_bytes else 0
    kv_bytes_per_token = runner.cache.bytes_per_token
    generator = torch.Generator().manual_seed(args.seed)

    def tokens(count: int) -> list[int]:
        return torch.randint(4, spec.vocab_size, (count,), generator=generator).tolist()

    def decode(batch: int, prompt_len: int, steps: int, warmup: int) -> dict:
        """`steps` timed decode steps of `batch` requests after prompts of `prompt_len` tokens.  Every timed
        step decodes one token of every request (checked): a request that finished its prompt earlier than
        the others is further on by then, and the context is the mean over requests and timed steps."""
        core = EngineCore(runner, SchedulerConfig(batch, budget(batch)), prefill_chunk_size=min(2048, prompt_len))
        settings = GenerationConfig(max_new_tokens=output_tokens(batch, prompt_len))
        requests = [Request(f"b{batch}-{prompt_len}-{index}", tokens(prompt_len), settings) for index in range(batch)]
        for request in requests:
            core.submit(request)
        while any(not request.output for request in requests):
            core.step()
        for _ in range(warmup):
            core.step()
        before = [len(request.output) for request in requests]
        torch.cuda.synchronize()
        started = time.perf_counter()
        for _ in range(steps):
            produced = core.step()
            if len(produced) != batch:
                raise RuntimeError(f"a timed step decoded {len(produced)} tokens, not one of each of the {batch} requests")
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        assert all(len(request.output) == had + steps and not request.done for request, had in zip(requests, before))
        for request in requests:
            core.finish(request)
        # keys a request's token sees in timed step j: its prompt, what it had generated before, and j
        context = prompt_len + sum(before) / batch + (steps - 1) / 2.0
        step_bytes = weight_bytes + batch * embedding_row_bytes + batch * context * kv_bytes_per_token
        seconds = elapsed / steps
        return {
            "tokens_per_s": batch * steps / elapsed,
            "ms_per_step": 1000 * seconds,
            "context": context,
            "achieved_gbs": step_bytes / seconds / 1e9,
            "generated": settings.max_new_tokens,
        }

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

    main_run = decode(*headline, steps, args.warmup)

    prefill_seconds = prefill(args.prefill_len)
    layer_weights = sum(
        t.numel() for name, t in tensors.items() if t.ndim == 2 and name != spec.embedding_name and name != spec.head_name
    )
    t = args.prefill_len
    flops = 2.0 * t * layer_weights + 2.0 * spec.vocab_size * spec.hidden_size
    # attention: scores and weighted values, 2 flops each for every (query, key, head, dimension) below the diagonal
    score_width = sum(
        need.num_kv_heads * need.head_dim * heads_per_kv
        for need, heads_per_kv in attention_widths(spec)
    )
    flops += 4.0 * score_width * t * (t + 1) / 2
    peak = PEAK_FLOPS["bf16" if dtype == torch.bfloat16 else "fp32"]

    points = {}
    for name, (batch, prompt_len) in extra.items():
        short = min(steps, 64 if prompt_len <= 4096 else 32)
        run = decode(batch, prompt_len, short, min(args.warmup, 8))
        points[name] = round(run["tokens_per_s"], 1)
        points[name + "_ms_per_step"] = round(run["ms_per_step"], 4)
        points[name + "_hbm_frac"] = round(run["achieved_gbs"] / HBM_PEAK_GBS, 4)

    label = Path(args.config).stem.replace("qwen", "Qwen").replace("b", "B")
    sizes = {
        key: getattr(config, key)
        for key in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size",
                    "rope_theta", "rms_norm_eps", "max_position_embeddings")
        if hasattr(config, key)
    }
    record = {
        "metric": f"decode tok/s at batch {args.batch}, {args.prompt_len}-token prompts ({label} shape)",
        "value": round(main_run["tokens_per_s"], 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_run["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "fp32",
        "data": "synthetic: seeded random weights, uniform random token ids",
        "config": {
            "model": f"{label} layer sizes, random weights",
            "layers": len(spec.run_order),
            "layers_full": full.num_layers,
            **sizes,
            "vocab_size": spec.vocab_size,
            "tied_embeddings": spec.tie_embeddings,
            "page_size": page,
            "global_batch": args.batch,
            "seq_len": args.prompt_len,
            "decode_context": round(main_run["context"], 1),
            "output_tokens": main_run["generated"],
            "kv_bytes_per_token": kv_bytes_per_token,
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
            "achieved": round(main_run["achieved_gbs"], 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(main_run["achieved_gbs"] / HBM_PEAK_GBS, 4),
        },
        "points": points,
    }
    print(json.dumps(record))
    return 0


def attention_widths(spec):
    """(cache need, query heads per kv head) of every run of the run order whose mixer attends over pages."""
    from llmserve_amd.parts.base import PagedKeyValue

    found = []
    for index, run in enumerate(spec.run_order):
        need = spec.cell_need(index)
        mixer = getattr(spec.layers[run.layer].block, "mixer", None)
        if isinstance(need, PagedKeyValue) and hasattr(mixer, "num_heads"):
            found.append((need, mixer.num_heads // need.num_kv_heads))
    return found


if __name__ == "__main__":
    sys.exit(main())
