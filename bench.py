"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The default run has the layer sizes of Qwen2.5-1.5B (configs/qwen2.5-1.5b.json) with seeded
random bfloat16 weights: 8 requests with 512-token prompts are prefilled, then decoded
through the engine's own iteration loop (scheduler, step function, sampling, one token per
request per step).  The timed window is K decode steps placed so that its mean context is 640
keys (512-token prompts, 256 outputs: the middle of the stated workload) whatever K is, after at
least W untimed steps.  The measurement is repeated with fresh requests (five times by default);
`ms_per_step` is the median over the repeats of the wall clock between two device
synchronisations, with the smallest and largest beside it and the same window by device events.
One JSON line is printed: decoded tokens a second, the prefill of a 2,048-token prompt, the decode
step's share of the HBM roofline, and in `points` batch 1 and 64, longer contexts, longer prompts,
the same model in float32, and the 7B and 32B layer sizes.

    python bench.py --op decode-attention

prints the reference's own kernel-level table instead (one attention layer, context 128, batch
1/2/4/8, its protocol: scripts/benchmark_triton_paged_attention.py:60-107).

    python bench.py --op prefill-attention

times the paged attention of prompt portions alone (the configuration's heads; whole prompts of 2,048
and 8,192 tokens, a 2,048-token portion behind 8,192 to 32,704 keys, sixteen prompts of 512) and prints
microseconds and PFLOP/s, counting the causal half only.
"""

from __future__ import annotations

import argparse
import dataclasses
import json
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}  # dense MFMA, published
PAGE = 16
STATED_CONTEXT = 640  # 512-token prompts and 256 outputs: the mean context of the stated workload


def parse() -> argparse.Namespace:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=128)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--repeats", type=int, default=5, help="how often the timed window is measured, with fresh requests")
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--prompt-len", type=int, default=512)
    parser.add_argument("--prefill-len", type=int, default=2048)
    parser.add_argument("--config", default=str(ROOT / "configs" / "qwen2.5-1.5b.json"))
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--seed", type=int, default=7)
    parser.add_argument("--own-products", action="store_true",
                        help="every product on the hand-written kernels, none sent to the BLAS library")
    parser.add_argument("--skip-points", action="store_true", help="the headline and the prefill only")
    parser.add_argument("--skip-context-points", action="store_true",
                        help="leave out decoding at contexts of 8k and 30k (batch 8) and 4k (batch 64), and the long prompts")
    parser.add_argument("--skip-other-models", action="store_true",
                        help="leave out the float32 run and the 7B and 32B layer sizes")
    parser.add_argument("--op", choices=("decode-attention", "prefill-attention"), default=None,
                        help="measure one operation alone instead, as the reference's kernel benchmark does")
    return parser.parse_args()


def budget(batch: int) -> int:
    return max(2048, batch)  # tokens a step


def generated_before(prompt: int, steps: int, warmup: int) -> int:
    """How many tokens each request has generated, on average, when the timed window begins: enough
    that the window's mean context is the stated one where the prompt allows it, and at least `warmup`."""
    return max(warmup, STATED_CONTEXT - prompt - steps // 2) if prompt < STATED_CONTEXT else warmup


def output_tokens(batch: int, prompt: int, steps: int, warmup: int, windows: int = 1) -> int:
    """How many tokens a request of a decode measurement may generate.  Prompts come in portions under
    the step's token budget, so the requests finish their prompts in different steps and those that
    finish first decode meanwhile: with this many tokens none of them ends before the timed steps do."""
    steps_of_prompts = -(-batch * prompt // budget(batch)) + batch
    return steps_of_prompts + generated_before(prompt, steps, warmup) + windows * steps + 2


class Bench:
    """One model on the device with a runner, and the measurements over it."""

    def __init__(self, config_path: str, dtype_name: str, seed: int, *, layers: int | None = None, library_products: bool = True,
                 shapes: list[tuple[int, int, int]], prefill_tokens: int, longest_prompt: int = 0) -> None:
        import torch

        from llmserve_amd import CacheConfig, ModelRunner
        from llmserve_amd.kernels import HipKernels
        from llmserve_amd.weights import random_model, read_config, run_dtype

        self.torch = torch
        _, self.full = read_config(config_path)  # the architecture is whatever the file names
        self.config = dataclasses.replace(self.full, num_layers=layers) if layers else self.full
        self.dtype = run_dtype(dtype_name)
        self.dtype_name = "bf16" if self.dtype == torch.bfloat16 else "fp32"
        self.device = torch.device("cuda:0")
        self.loaded = random_model(self.config, seed, dtype=self.dtype, device=self.device)
        self.spec, self.tensors = self.loaded.spec, self.loaded.tensors
        self.kernels = HipKernels(self.dtype, self.device, library_products=library_products)
        self.longest = getattr(self.config, "max_position_embeddings", 32768)
        # pages for the largest measurement: (batch, prompt, tokens generated) each, and the prefill beside it
        pages = max(batch * (-(-(prompt + generated + PAGE) // PAGE)) for batch, prompt, generated in shapes)
        pages = max(pages, -(-max(prefill_tokens, longest_prompt) // PAGE)) + prefill_tokens // PAGE + 8
        most = max(batch for batch, _, _ in shapes)
        self.runner = ModelRunner(self.loaded, self.kernels, CacheConfig(block_size=PAGE, num_blocks=pages, max_sequences=most + 1))
        # What a decode step has to read: every weight it uses once (of an untied embedding table only the
        # rows of the step's tokens) and the cache of the live requests.
        self.weight_bytes = sum(t.numel() * t.element_size() for t in self.tensors.values())
        self.embedding_row_bytes = 0
        if not self.spec.tie_embeddings:
            table = self.tensors[self.spec.embedding_name]
            self.weight_bytes -= table.numel() * table.element_size()
            self.embedding_row_bytes = self.spec.hidden_size * table.element_size()
        self.kv_bytes_per_token = self.runner.cache.bytes_per_token
        self.generator = torch.Generator().manual_seed(seed)
        self.serial = 0

    def close(self) -> None:
        self.runner.close()
        self.torch.cuda.synchronize()

    def tokens(self, count: int) -> list[int]:
        return self.torch.randint(4, self.spec.vocab_size, (count,), generator=self.generator).tolist()

    def decode(self, batch: int, prompt_len: int, steps: int, warmup: int, repeats: int, fresh: bool = True) -> dict:
        """`repeats` timed windows of `steps` decode steps of `batch` requests after prompts of `prompt_len`
        tokens.  Every timed step decodes one token of every request (checked).  `fresh`: each window has
        requests of its own, prefilled and decoded up to the window's place (the same contexts every time);
        else the windows follow each other over the same requests (long prompts, whose prefill would take
        longer than everything else), and the context is the mean over all of them."""
        from llmserve_amd import EngineCore, GenerationConfig, SchedulerConfig
        from llmserve_amd.engine import Request

        torch = self.torch
        before = generated_before(prompt_len, steps, warmup)
        wall, device, contexts = [], [], []
        runs = repeats if fresh else 1
        for run in range(runs):
            windows = 1 if fresh else repeats
            core = EngineCore(self.runner, SchedulerConfig(batch, budget(batch)), prefill_chunk_size=min(2048, prompt_len))
            settings = GenerationConfig(max_new_tokens=output_tokens(batch, prompt_len, steps, warmup, windows))
            self.serial += 1
            requests = [Request(f"m{self.serial}-{index}", self.tokens(prompt_len), settings) for index in range(batch)]
            for request in requests:
                core.submit(request)
            while any(not request.output for request in requests):
                core.step()
            untimed = 0
            while sum(len(request.output) for request in requests) < before * batch or untimed < warmup:
                core.step()
                untimed += 1
            for _ in range(windows):
                had = [len(request.output) for request in requests]
                began, ended = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                started = time.perf_counter()
                began.record()
                for _ in range(steps):
                    produced = core.step()
                    if len(produced) != batch:
                        raise RuntimeError(f"a timed step decoded {len(produced)} tokens, not one of each of the {batch} requests")
                ended.record()
                torch.cuda.synchronize()
                wall.append((time.perf_counter() - started) / steps)
                device.append(began.elapsed_time(ended) / 1000.0 / steps)
                assert all(len(request.output) == count + steps and not request.done for request, count in zip(requests, had))
                # keys a request's token sees in timed step j: its prompt, what it had generated before, and j
                contexts.append(prompt_len + sum(had) / batch + (steps - 1) / 2.0)
            for request in requests:
                core.finish(request)
        seconds = statistics.median(wall)
        context = statistics.mean(contexts)
        step_bytes = self.weight_bytes + batch * self.embedding_row_bytes + batch * context * self.kv_bytes_per_token
        return {
            "tokens_per_s": batch / seconds,
            "ms_per_step": 1000 * seconds,
            "ms_min": 1000 * min(wall),
            "ms_max": 1000 * max(wall),
            "ms_device": 1000 * statistics.median(device),
            "context": context,
            "achieved_gbs": step_bytes / seconds / 1e9,
            "generated": settings.max_new_tokens,
            "repeats": len(wall),
        }

    def prefill_flops(self, tokens: int) -> float:
        """Products: two flops for every weight of the layers and every token, and the head on one row.  Attention:
        scores and weighted values, two flops each for every (query, key, head, dimension) at or below the diagonal."""
        spec = self.spec
        layer_weights = sum(
            t.numel() for name, t in self.tensors.items() if t.ndim == 2 and name != spec.embedding_name and name != spec.head_name
        )
        flops = 2.0 * tokens * layer_weights + 2.0 * spec.vocab_size * spec.hidden_size
        score_width = sum(need.num_kv_heads * need.head_dim * heads_per_kv for need, heads_per_kv in attention_widths(spec))
        return flops + 4.0 * score_width * tokens * (tokens + 1) / 2

    def prefill(self, length: int, portion: int | None = None, repeats: int = 5) -> dict:
        """A prompt of `length` tokens through the step function, whole or in portions of `portion`, the last
        token's logits wanted: median, smallest and largest of `repeats` after one untimed run."""
        from llmserve_amd import StepEntry

        torch = self.torch
        portion = portion or length
        times = []
        for repeat in range(repeats + 1):
            prompt = self.tokens(length)
            name = f"p{self.serial}-{repeat}"
            torch.cuda.synchronize()
            started = time.perf_counter()
            for at in range(0, length, portion):
                piece = prompt[at : at + portion]
                last = at + portion >= length
                self.runner.step([StepEntry(name, piece, [len(piece) - 1] if last else [])], create_missing=True)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - started)
            self.runner.end_request(name)
        self.serial += 1
        seconds = statistics.median(times[1:])
        peak = PEAK_FLOPS[self.dtype_name]
        return {
            "value": round(length / seconds, 1),
            "tokens": length,
            "ms": round(1000 * seconds, 3),
            "frac": round(self.prefill_flops(length) / seconds / peak, 4),
            "ms_min": round(1000 * min(times[1:]), 3),
            "ms_max": round(1000 * max(times[1:]), 3),
        }

    def sizes(self) -> str:
        c = self.config
        return (f"L{len(self.spec.run_order)} of {self.full.num_layers} H{c.hidden_size} Hq{c.num_attention_heads} Hkv{c.num_key_value_heads} "
                f"D{c.head_dim} I{c.intermediate_size} V{c.vocab_size} {'tied' if self.spec.tie_embeddings else 'untied'} {self.dtype_name}")


def put(points: dict, name: str, run: dict) -> None:
    points[name] = round(run["tokens_per_s"], 1)
    points[name + "_ms_per_step"] = round(run["ms_per_step"], 4)
    points[name + "_ms_min_max"] = f"{run['ms_min']:.4f}-{run['ms_max']:.4f}"
    points[name + "_hbm_frac"] = round(run["achieved_gbs"] / HBM_PEAK_GBS, 4)
    points[name + "_context"] = round(run["context"], 1)


def put_prefill(points: dict, name: str, run: dict) -> None:
    points[name] = run["value"]
    points[name + "_ms"] = run["ms"]
    points[name + "_ms_min_max"] = f"{run['ms_min']:.3f}-{run['ms_max']:.3f}"
    points[name + "_mfma_frac"] = run["frac"]


def decode_attention_table(args) -> int:
    """The reference's kernel-level measurement (scripts/benchmark_triton_paged_attention.py:60-107, artifacts/
    checkpoint2-t4.json): the attention part of one layer at the 1.5B sizes (12 query heads, 2 kv heads, head size
    128: projections, rotation, cache write, paged attention, output projection) for batch 1/2/4/8 decoded tokens
    over a context of 128, five untimed calls, then five repeats of twenty calls between device events."""
    import torch

    from llmserve_amd import CacheConfig, ModelRunner, StepEntry
    from llmserve_amd.engine.runner import build_step_batch
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.weights import random_model, read_config, run_dtype

    _, full = read_config(args.config)
    config = dataclasses.replace(full, num_layers=1)
    dtype = run_dtype(args.dtype)
    device = torch.device("cuda:0")
    loaded = random_model(config, args.seed, dtype=dtype, device=device)
    kernels = HipKernels(dtype, device)
    runner = ModelRunner(loaded, kernels, CacheConfig(block_size=PAGE, num_blocks=256, max_sequences=9), use_graphs=False)
    generator = torch.Generator().manual_seed(args.seed)
    context, repeats, iterations = 128, 5, 20
    block = runner.model.layers[0]
    rows = []
    for batch_size in (1, 2, 4, 8):
        names = [f"a{batch_size}-{index}" for index in range(batch_size)]
        prompts = [torch.randint(4, config.vocab_size, (context - 1,), generator=generator).tolist() for _ in names]
        runner.step([StepEntry(name, prompt, []) for name, prompt in zip(names, prompts)], create_missing=True)
        reservations = [runner.cache.reserve(name, 1) for name in names]
        entries = [StepEntry(name, [5], [0]) for name in names]
        batch = build_step_batch(reservations, entries, runner.cache, device)
        hidden = torch.randn((batch_size, config.hidden_size), generator=torch.Generator(device=device).manual_seed(101 + batch_size),
                             device=device, dtype=dtype)

        def run_once() -> None:  # the token's key and value are written again to the same place every time
            batch.computed.clear()  # the angles are computed anew, as the reference computes them in every call
            block.mixer.forward(hidden, batch, runner.cells[0])

        with torch.inference_mode():
            for _ in range(5):
                run_once()
            torch.cuda.synchronize()
            times = []
            for _ in range(repeats):
                began, ended = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                began.record()
                for _ in range(iterations):
                    run_once()
                ended.record()
                ended.synchronize()
                times.append(began.elapsed_time(ended) / iterations)
        for name in names:
            runner.end_request(name)
        rows.append({"kind": "micro", "batch_size": batch_size, "sequence_length": context, "metric": "attention_ms",
                     "median": round(statistics.median(times), 5), "min": round(min(times), 5), "max": round(max(times), 5),
                     "stdev": round(statistics.stdev(times), 6)})
    print(json.dumps({
        "op": "decode-attention", "dtype": args.dtype, "repeats": repeats, "micro_iterations": iterations,
        "launch": "kernel by kernel from the host, as the reference's (a step of the engine replays a graph instead)",
        "sizes": "H1536 Hq12 Hkv2 D128, page 16, one layer", "summaries": rows,
    }))
    return 0


def prefill_attention_table(args) -> int:
    """The engine's paged attention for prompt portions alone, through the call the layers make
    (`HipKernels.paged_attention`), over pages of random keys and values laid out as the cache manager lays them
    out: per shape five untimed calls, then five repeats of ten calls between device events.  Flops count the
    keys a query sees (the causal half of a whole prompt), 4 * head size a (query, key, head)."""
    import torch

    from llmserve_amd.cache import CacheCell
    from llmserve_amd.engine.batch import GroupBatch, SequenceChunk, StepBatch
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.parts import HeadLayout, PagedKeyValue
    from llmserve_amd.weights import read_config, run_dtype

    _, config = read_config(args.config)
    dtype = run_dtype(args.dtype)
    device = torch.device("cuda:0")
    kernels = HipKernels(dtype, device)
    heads, kv_heads, dim = config.num_attention_heads, config.num_key_value_heads, config.head_dim
    layout = HeadLayout(heads, kv_heads, dim)
    need = PagedKeyValue(kv_heads, dim)
    generator = torch.Generator(device=device).manual_seed(args.seed)
    shapes = [([2048], [2048]), ([8192], [8192]), ([8192], [2048]), ([16384], [2048]), ([32704], [2048]), ([512] * 16, [512] * 16)]
    repeats, iterations = 5, 10
    rows = []
    for contexts, portions in shapes:
        blocks = [-(-context // PAGE) for context in contexts]
        pages, width = sum(blocks) + 1, max(blocks)
        tables = torch.zeros((len(contexts), width), dtype=torch.int32)
        positions, sequence, slots, chunks, first_page = [], [], [], [], 0
        for index, (context, count) in enumerate(zip(contexts, portions)):
            tables[index, : blocks[index]] = torch.arange(first_page, first_page + blocks[index], dtype=torch.int32)
            mine = torch.arange(context - count, context)
            positions.append(mine)
            sequence.append(torch.full((count,), index))
            slots.append(first_page * PAGE + mine)
            chunks.append(SequenceChunk(f"r{index}", index, context - count, count))
            first_page += blocks[index]
        ints = lambda values: torch.as_tensor(values, dtype=torch.int32, device=device)
        starts = [0]
        for count in portions:
            starts.append(starts[-1] + count)
        tokens = sum(portions)
        group = GroupBatch(PAGE, tables.to(device), ints(torch.cat(slots)), width)
        batch = StepBatch(
            num_tokens=tokens, chunks=chunks, token_ids=ints([0] * tokens), positions=ints(torch.cat(positions)),
            token_sequence=ints(torch.cat(sequence)), query_start=ints(starts), context_lengths=ints(contexts),
            state_slots=ints(list(range(len(contexts)))), groups=[group], logit_rows=ints([]), num_logit_rows=0,
            max_query_length=max(portions), max_context_length=max(contexts),
        )
        fields = {name: torch.randn((pages, *shape), generator=generator, device=device).to(dtype)
                  for name, shape in need.page_fields(PAGE).items()}
        cell = CacheCell(need, True, 0, fields=fields)
        qkv = torch.randn((tokens, layout.width), generator=generator, device=device).to(dtype)
        scale = dim ** -0.5

        def run_once() -> None:
            kernels.paged_attention(qkv, layout, batch, cell, scale, None)

        with torch.inference_mode():
            for _ in range(5):
                run_once()
            torch.cuda.synchronize()
            times = []
            for _ in range(repeats):
                began, ended = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                began.record()
                for _ in range(iterations):
                    run_once()
                ended.record()
                ended.synchronize()
                times.append(began.elapsed_time(ended) / iterations * 1e3)
        flops = sum(4.0 * heads * dim * (count * (context - count) + count * (count + 1) / 2) for context, count in zip(contexts, portions))
        median = statistics.median(times)
        rows.append({"contexts": f"{len(contexts)} x {contexts[0]}", "portion": portions[0], "us": round(median, 1),
                     "us_min": round(min(times), 1), "us_max": round(max(times), 1),
                     "pflops": round(flops / median / 1e9, 3), "frac": round(flops / median / 1e9 / (PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"] / 1e15), 3)})
        del fields, cell, qkv
    print(json.dumps({
        "op": "prefill-attention", "dtype": args.dtype, "repeats": repeats, "micro_iterations": iterations,
        "sizes": f"Hq{heads} Hkv{kv_heads} D{dim}, page {PAGE}", "summaries": rows,
    }))
    return 0


def main() -> int:
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not measured")
        return 2
    if args.op == "decode-attention":
        return decode_attention_table(args)
    if args.op == "prefill-attention":
        return prefill_attention_table(args)

    import torch

    began = time.monotonic()
    steps = max(1, min(args.steps, 250 - args.warmup))
    warmup, repeats = args.warmup, max(1, args.repeats)
    headline = (args.batch, args.prompt_len)
    extra = {} if args.skip_points else {"decode_b1": (1, args.prompt_len), "decode_b64": (64, args.prompt_len)}
    long_context = {}
    if not args.skip_points and not args.skip_context_points:
        long_context = {"decode_b8_ctx8k": (8, 8192), "decode_b8_ctx30k": (8, 30000), "decode_b64_ctx4k": (64, 4096)}
    long_steps, long_windows = min(steps, 32), 3

    # every decode measurement as (batch, prompt, tokens generated), for the cache's size
    shapes = [(batch, prompt, output_tokens(batch, prompt, steps, warmup)) for batch, prompt in [headline, *extra.values()]]
    shapes += [(batch, prompt, output_tokens(batch, prompt, long_steps, min(warmup, 8), long_windows))
               for batch, prompt in long_context.values()]
    long_prompts = not args.skip_points and not args.skip_context_points
    bench = Bench(args.config, args.dtype, args.seed, layers=args.layers, library_products=not args.own_products, shapes=shapes,
                  prefill_tokens=args.prefill_len, longest_prompt=32768 if long_prompts else 0)
    long_context = {name: shape for name, shape in long_context.items()
                    if shape[1] + output_tokens(*shape, long_steps, min(warmup, 8), long_windows) <= bench.longest}

    main_run = bench.decode(*headline, steps, warmup, repeats)
    prefill = bench.prefill(args.prefill_len)

    points: dict = {}
    for name, (batch, prompt_len) in extra.items():
        put(points, name, bench.decode(batch, prompt_len, steps, warmup, repeats))
    for name, (batch, prompt_len) in long_context.items():
        # three windows one after the other over the same requests: their prompts take longer than all the rest
        put(points, name, bench.decode(batch, prompt_len, long_steps, min(warmup, 8), long_windows, fresh=False))
    if long_prompts:
        # longer prompts, where the engine's own attention kernel decides: in portions of 2,048 tokens
        put_prefill(points, "prefill_8k", bench.prefill(8192, 2048, repeats=3))
        if bench.longest >= 32768:
            put_prefill(points, "prefill_32k", bench.prefill(32768 - 64, 2048, repeats=3))
    label = Path(args.config).stem.replace("qwen", "Qwen").replace("b", "B")
    spec, config, full = bench.spec, bench.config, bench.full
    sizes = {
        key: getattr(config, key)
        for key in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size",
                    "rope_theta", "rms_norm_eps", "max_position_embeddings")
        if hasattr(config, key)
    }
    dtype_name, kv_bytes = bench.dtype_name, bench.kv_bytes_per_token
    layers_run = len(spec.run_order)
    vocab, tied = spec.vocab_size, spec.tie_embeddings

    if not args.skip_points and not args.skip_other_models and not args.own_products:
        if args.dtype == "bfloat16":
            # every product of a prefill on the hand-written kernels, none sent to the BLAS library
            own = Bench(args.config, args.dtype, args.seed, layers=args.layers, library_products=False, shapes=[(1, 64, 64)],
                        prefill_tokens=args.prefill_len)
            put_prefill(points, "prefill_own_products", own.prefill(args.prefill_len, repeats=3))
            own.close()
            del own
        bench.close()
        del bench
        torch.cuda.empty_cache()
        others = []
        if args.dtype == "bfloat16":
            others.append(("fp32", args.config, "float32", min(steps, 64), repeats))
        stem = Path(args.config).stem
        if stem == "qwen2.5-1.5b":
            others.append(("7b", str(ROOT / "configs" / "qwen2.5-7b.json"), args.dtype, min(steps, 64), repeats))
            others.append(("32b", str(ROOT / "configs" / "qwen2.5-32b.json"), args.dtype, min(steps, 32), 3))
        for tag, path, dtype, few, times in others:
            if time.monotonic() - began > 150:  # the whole run stays within minutes
                points[f"decode_b8_{tag}"] = None
                continue
            shape = (args.batch, args.prompt_len, output_tokens(args.batch, args.prompt_len, few, warmup))
            other = Bench(path, dtype, args.seed, shapes=[shape], prefill_tokens=args.prefill_len)
            put(points, f"decode_b{args.batch}_{tag}", other.decode(args.batch, args.prompt_len, few, warmup, times))
            put_prefill(points, f"prefill_{tag}", other.prefill(args.prefill_len, repeats=3))
            points[f"sizes_{tag}"] = other.sizes()
            other.close()
            del other
            torch.cuda.empty_cache()

    record = {
        "metric": f"decode tok/s at batch {args.batch}, {args.prompt_len}-token prompts ({label} shape)",
        "value": round(main_run["tokens_per_s"], 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(main_run["ms_per_step"], 4),
        "ms_per_step_min": round(main_run["ms_min"], 4),
        "ms_per_step_max": round(main_run["ms_max"], 4),
        "ms_per_step_device_events": round(main_run["ms_device"], 4),
        "repeats": main_run["repeats"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_name,
        "data": "synthetic: seeded random weights, uniform random token ids",
        "config": {
            "model": f"{label} layer sizes, random weights" + (", every product on the engine's own kernels" if args.own_products else ""),
            "layers": layers_run,
            "layers_full": full.num_layers,
            **sizes,
            "vocab_size": vocab,
            "tied_embeddings": tied,
            "page_size": PAGE,
            "global_batch": args.batch,
            "seq_len": args.prompt_len,
            "decode_context": round(main_run["context"], 1),
            "decode_window": f"{steps} steps centred on context {STATED_CONTEXT} of 512 + 256 tokens, median of {main_run['repeats']} runs",
            "output_tokens": main_run["generated"],
            "parallelism": "none (1 GPU)",
        },
        "prefill": {key: prefill[key] for key in ("value", "tokens", "ms", "frac")},
        "prefill_ms_min_max": f"{prefill['ms_min']:.3f}-{prefill['ms_max']:.3f}",
        "roofline": {
            "bound": "hbm",
            "achieved": round(main_run["achieved_gbs"], 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(main_run["achieved_gbs"] / HBM_PEAK_GBS, 4),
        },
        "kv_bytes_per_token": kv_bytes,
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
