"""The `llmserve` command line, in the reference's manner (`src/llmserve/cli.py:244-328`):
argparse subcommands, with the reference's option names and meanings where it has them.

    llmserve benchmark   run the synthetic open-loop workload through the engine
    llmserve generate    generate tokens for one prompt
    llmserve replay      feed token ids step by step and write logits (bin/trace_run)
    llmserve random-model  write a model folder with seeded random weights

The reference's `serve`, `quantize-eval` and `speculative-eval` have no counterpart here:
servers, quantized weights and speculative decoding are outside this engine.  Nor have its
switches between back ends (`--paged-attention-backend`, `--linear-backend`,
`--rebuild-device-metadata`, `cli.py:263-271`): there is one attention path and one product
path here, and an option that chose nothing would only pretend.
"""

from __future__ import annotations

import argparse
import asyncio
import json
import sys
import tempfile
from dataclasses import replace
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def _load_runtime(args):
    """A model folder; or weights drawn from --seed at the sizes of a config.json
    (--random-weights, made on the device: no folder is written); or without either the
    bundled tiny configuration with such weights and the byte tokenizer (`cli.py:22-45`)."""
    from .engine.tokenizer import ByteTokenizer, FileTokenizer
    from .weights import load_model_folder, random_model, read_config, write_model_folder

    if args.model and getattr(args, "random_weights", None):
        raise SystemExit("give --model or --random-weights, not both")
    if getattr(args, "random_weights", None):
        device = args.device if args.device != "auto" else "cuda:0"
        return random_model(args.random_weights, args.seed, dtype=args.dtype, device=device), ByteTokenizer()
    if args.model:
        loaded = load_model_folder(args.model, args.dtype)
        try:
            tokenizer = FileTokenizer(args.model)
        except FileNotFoundError:
            tokenizer = ByteTokenizer()
        return loaded, tokenizer
    _, config = read_config(ROOT / "configs" / "tiny.json")  # whatever architecture that file names
    folder = write_model_folder(Path(tempfile.mkdtemp(prefix="llmserve-tiny-")), config, seed=args.seed)
    return load_model_folder(folder, args.dtype), ByteTokenizer()


def _engine(args, loaded, tokenizer, *, batch_size: int, mode: str):
    from .config import CacheConfig, SchedulerConfig
    from .engine import LLMEngine

    kernels = None
    if getattr(args, "own_products", False):  # every product on the hand-written kernels, none sent to the BLAS library
        from .kernels import HipKernels
        from .weights import run_dtype

        kernels = HipKernels(run_dtype(args.dtype), args.device if args.device != "auto" else "cuda:0", library_products=False)
    return LLMEngine(
        loaded,
        tokenizer,
        cache_config=CacheConfig(args.block_size, args.num_blocks, max(batch_size, 1)),
        scheduler_config=SchedulerConfig(batch_size, max(args.max_tokens_per_step, batch_size), args.policy),
        scheduler_mode=mode,
        prefill_chunk_size=args.prefill_chunk_size,
        collect_iteration_metrics=True,
        device=args.device if args.device != "auto" else "cuda:0",
        dtype=args.dtype,
        kernels=kernels,
    )


async def _benchmark(args) -> None:
    """`cli.py:48-125`: naive = one request at a time, the whole prefix again for every token;
    paged = the engine with batch size 1; static and continuous = the two admission modes."""
    from .benchmark import BenchmarkHarness, LoadProfile
    from .sampling import GenerationConfig

    loaded, tokenizer = _load_runtime(args)
    profile = LoadProfile.from_yaml(args.profile)
    if args.requests and profile.groups:
        raise SystemExit("--requests cannot change a profile made of groups")
    batch_size = 1 if args.config in ("naive", "paged") else args.batch_size
    engine = _engine(args, loaded, tokenizer, batch_size=batch_size, mode="static" if args.config == "static" else "continuous")
    profile = replace(
        profile,
        requests=args.requests or profile.requests,
        arrival_rate=args.arrival_rate or profile.arrival_rate,
        vocabulary_size=engine.runner.vocab_size,
    ).fitted(engine.cache.max_sequence_length)
    harness = BenchmarkHarness(profile)

    def settings(count: int) -> GenerationConfig:
        return GenerationConfig(max_new_tokens=count, temperature=0.0, seed=args.seed, stop_token_ids=())

    if args.config == "naive":
        lock = asyncio.Lock()

        async def generate(arrival, callback):
            async with lock:  # reference engine.py:83-105: no cache is kept between tokens
                sequence = list(arrival.prompt)
                for _ in range(arrival.max_new_tokens):
                    sequence += await engine.generate(sequence, settings(1))
                    callback(sequence[-1])
                return sequence[len(arrival.prompt):]

        facts = None
    else:

        async def generate(arrival, callback):
            return await engine.generate(
                list(arrival.prompt), settings(arrival.max_new_tokens), callback, request_id=arrival.request_id
            )

        facts = engine.request_facts

    report = await harness.run(f"{args.config}-{args.policy}", generate, facts)
    report.cache = engine.cache_stats
    report.metadata["engine"] = engine.iteration_stats
    await engine.close()
    output = Path(args.output)
    output.parent.mkdir(parents=True, exist_ok=True)
    report.write_json(output)
    report.write_csv(output.with_suffix(".csv"))
    print(json.dumps(report.summary, indent=2))


async def _generate(args) -> None:
    from .sampling import GenerationConfig

    loaded, tokenizer = _load_runtime(args)
    engine = _engine(args, loaded, tokenizer, batch_size=1, mode="continuous")
    prompt = [int(t) for t in args.prompt_tokens.split(",")] if args.prompt_tokens else args.prompt
    stops = tuple(args.stop_token_id or ())
    if not stops and args.model and not args.ignore_eos:
        # as the reference's service does (`service/app.py:88`): generation ends at the model's own
        # end-of-sequence token unless the caller says where it ends
        from .engine.tokenizer import folder_eos_token_ids

        stops = folder_eos_token_ids(args.model)
    settings = GenerationConfig(args.max_tokens, args.temperature, args.top_p, args.seed, stops)
    tokens = await engine.generate(prompt, settings)
    await engine.close()
    print(json.dumps({"token_ids": tokens, "text": tokenizer.decode(tokens)}))


def _replay(args) -> int:
    import subprocess

    command = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", args.model, "--dtype", args.dtype, "--out",
               args.out, "--max-tokens", str(args.max_tokens), "--block-size", str(args.block_size),
               "--max-requests", str(args.max_requests)]
    if args.own_products:
        command.append("--own-products")
    return subprocess.call(command)


def _random_model(args) -> None:
    import torch

    from .weights import read_config, write_model_folder

    _, config = read_config(args.config)
    folder = write_model_folder(args.output, config, args.seed, dtype=torch.bfloat16, norm_std=args.norm_std,
                                bias_std=args.bias_std, std=args.std)
    print(folder)


def _engine_options(parser: argparse.ArgumentParser) -> None:
    parser.add_argument("--model", help="model folder with config.json and safetensors files")
    parser.add_argument("--random-weights", metavar="CONFIG_JSON",
                        help="instead of --model: weights drawn from --seed at the sizes of this config.json")
    parser.add_argument("--device", default="auto")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--block-size", type=int, default=16)
    parser.add_argument("--num-blocks", type=int, default=1024)
    parser.add_argument("--prefill-chunk-size", type=int, default=16)
    parser.add_argument("--max-tokens-per-step", type=int, default=2048)
    parser.add_argument("--policy", choices=("fcfs", "sjf", "priority"), default="fcfs")
    parser.add_argument("--seed", type=int, default=7)
    parser.add_argument("--own-products", action="store_true",
                        help="every matrix product on the engine's own kernels, none sent to the BLAS library")


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="llmserve")
    commands = parser.add_subparsers(dest="command", required=True)

    benchmark = commands.add_parser("benchmark", help="run the synthetic workload")
    benchmark.add_argument("--config", choices=("naive", "paged", "static", "continuous"), default="continuous")
    benchmark.add_argument("--profile", default=str(ROOT / "configs" / "benchmark-sharegpt.yaml"))
    benchmark.add_argument("--requests", type=int)
    benchmark.add_argument("--arrival-rate", type=float)
    benchmark.add_argument("--batch-size", type=int, default=16)
    benchmark.add_argument("--output", default="artifacts/benchmark.json")
    _engine_options(benchmark)

    generate = commands.add_parser("generate", help="generate tokens for one prompt")
    generate.add_argument("--prompt", default="Explain paged attention in one paragraph.")
    generate.add_argument("--prompt-tokens", help="comma-separated token ids instead of --prompt")
    generate.add_argument("--max-tokens", type=int, default=32)
    generate.add_argument("--temperature", type=float, default=0.0)
    generate.add_argument("--top-p", type=float, default=1.0)
    generate.add_argument("--stop-token-id", type=int, action="append",
                          help="default: the eos_token_id that the model folder names (generation_config.json, config.json)")
    generate.add_argument("--ignore-eos", action="store_true", help="run to --max-tokens whatever the model folder names")
    _engine_options(generate)

    replay = commands.add_parser("replay", help="feed token ids step by step (stdin) and write logits")
    replay.add_argument("--model", required=True)
    replay.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    replay.add_argument("--out", required=True)
    replay.add_argument("--max-tokens", type=int, required=True)
    replay.add_argument("--block-size", type=int, default=16)
    replay.add_argument("--max-requests", type=int, default=8, help="most requests alive at a time")
    replay.add_argument("--own-products", action="store_true",
                        help="every matrix product on the engine's own kernels, none sent to the BLAS library")

    random_model = commands.add_parser("random-model", help="write a model folder with seeded random weights")
    random_model.add_argument("--config", required=True, help="a config.json")
    random_model.add_argument("--output", required=True)
    random_model.add_argument("--seed", type=int, default=7)
    random_model.add_argument("--std", type=float, default=0.02)
    random_model.add_argument("--bias-std", type=float, default=0.02)
    random_model.add_argument("--norm-std", type=float, default=0.0)
    return parser


def main(argv: list[str] | None = None) -> int:
    args = build_parser().parse_args(argv)
    if args.command == "benchmark":
        asyncio.run(_benchmark(args))
    elif args.command == "generate":
        asyncio.run(_generate(args))
    elif args.command == "replay":
        return _replay(args)
    else:
        _random_model(args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
