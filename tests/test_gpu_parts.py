"""Each part of a layer alone on the GPU against the plain functions, the toy architecture
with a mixer that has state of its own, and generation through the entry points."""

from __future__ import annotations

import asyncio
import json
import math
import subprocess
import sys

import pytest
import torch

from llmserve_amd import CacheConfig, EngineCore, GenerationConfig, LLMEngine, ModelRunner, SchedulerConfig, StepEntry
from llmserve_amd.parts import (
    BLOCKS, FEED_FORWARDS, MIXERS, NORMS, AttentionSpec, GatedMLPSpec, PreNormBlockSpec, RMSNormSpec, RotarySpec,
)
from llmserve_amd.weights import load_model_folder, random_tensor
from tests import toy
from tests.gpu_helpers import ROOT
from tests.plain import qwen2_plain as plain
from tests.test_gpu_kernels import paged_case
from tests.tiny import CONFIGS, random_tokens

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
TOLERANCE = {torch.float32: dict(atol=3e-5, rtol=1e-4), torch.bfloat16: dict(atol=3e-2, rtol=3e-2)}


@pytest.fixture(scope="module")
def kernels():
    from llmserve_amd.kernels import HipKernels

    return {dtype: HipKernels(dtype) for dtype in DTYPES}


def draw(registry, spec, dtype, seed=1, **scales):
    """Random tensors of a part: what the kernel gets (on the GPU) and what the plain function gets."""
    on_gpu, exact = {}, {}
    for name, tensor_spec in registry.tensors(spec).items():
        value = random_tensor(name, tensor_spec, seed, std=0.08, norm_std=0.2, **scales).to(dtype)
        on_gpu[name] = value.cuda()
        exact[name] = value.double()
    return on_gpu, exact


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(kernels, dtype):
    spec = RMSNormSpec(136, 3e-4)
    tensors, exact = draw(NORMS, spec, dtype)
    part = NORMS.build(spec, tensors, kernels[dtype])
    hidden, delta = torch.randn(5, 136), torch.randn(5, 136)
    device_hidden = hidden.cuda()
    out = part.forward(device_hidden, delta.cuda())
    expected = plain.rms_norm((hidden + delta).double(), exact["weight"], 3e-4)
    torch.testing.assert_close(out.cpu().double(), expected, **TOLERANCE[dtype])
    torch.testing.assert_close(device_hidden.cpu(), hidden + delta)


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_part(kernels, dtype):
    spec = GatedMLPSpec(96, 208)
    tensors, exact = draw(FEED_FORWARDS, spec, dtype)
    part = FEED_FORWARDS.build(spec, tensors, kernels[dtype])
    for rows in (3, 80):  # the decoding kernel and the one for long portions
        x = torch.randn(rows, 96).to(dtype)
        out = part.forward(x.cuda(), None)
        assert out.dtype == torch.float32
        expected = plain.swiglu(x.double(), exact["gate_proj.weight"], exact["up_proj.weight"], exact["down_proj.weight"])
        torch.testing.assert_close(out.cpu().double(), expected, **TOLERANCE[dtype])


def attention_reference(spec, exact, xs, pairing, theta):
    outs = []
    config = plain.PlainConfig(
        vocab_size=1, hidden_size=spec.hidden_size, intermediate_size=1, num_layers=1, num_heads=spec.num_heads,
        num_kv_heads=spec.num_kv_heads, head_dim=spec.head_dim, rope_theta=theta, rms_norm_eps=0.0,
        attention_bias=spec.qkv_bias, tie_word_embeddings=True, rope_pairing=pairing,
    )
    for x in xs:
        outs.append(plain.attention_layer(x, exact, "", config, torch.arange(x.shape[0]), spec.window))
    return outs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,window,pairing", [(6, 2, 32, None, "half"), (5, 1, 48, 9, "adjacent"), (4, 4, 64, None, "adjacent")])
def test_attention_part(kernels, dtype, heads, kv_heads, dim, window, pairing):
    hidden, page, theta = 72, 8, 3000.0
    spec = AttentionSpec(hidden, heads, kv_heads, dim, 1 / math.sqrt(dim), RotarySpec(dim, theta, pairing), True, False, window)
    tensors, exact = draw(MIXERS, spec, dtype, bias_std=0.1)
    part = MIXERS.build(spec, tensors, kernels[dtype])
    lengths = [21, 40, 1]
    xs = [torch.randn(n, hidden).to(dtype) for n in lengths]
    expected = attention_reference(spec, exact, [x.double() for x in xs], pairing, theta)
    # first everything but each request's last three tokens, then those three: the second call reads the cache
    batch, cell, _, _ = paged_case(lengths, lengths, heads, kv_heads, dim, page, dtype)
    cell.keys.zero_()
    cell.values.zero_()
    whole = part.forward(torch.cat(xs).cuda(), batch, cell)
    torch.testing.assert_close(whole.cpu().double(), torch.cat(expected), **TOLERANCE[dtype])
    counts = [min(3, n) for n in lengths]
    tail_batch, _, _, _ = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype)
    tail = part.forward(torch.cat([x[-c:] for x, c in zip(xs, counts)]).cuda(), tail_batch, cell)
    torch.testing.assert_close(tail.cpu().double(), torch.cat([e[-c:] for e, c in zip(expected, counts)]), **TOLERANCE[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_part(kernels, dtype):
    hidden, heads, kv_heads, dim, page = 64, 4, 2, 16, 16
    norm = RMSNormSpec(hidden, 1e-5)
    attention = AttentionSpec(hidden, heads, kv_heads, dim, 0.25, RotarySpec(dim, 10000.0, "adjacent"))
    spec = PreNormBlockSpec(norm, attention, norm, GatedMLPSpec(hidden, 96))
    tensors, exact = draw(BLOCKS, spec, dtype)
    part = BLOCKS.build(spec, tensors, kernels[dtype])
    lengths = [33, 6]
    batch, cell, _, _ = paged_case(lengths, lengths, heads, kv_heads, dim, page, dtype)
    h = [torch.randn(n, hidden) for n in lengths]
    device_hidden = torch.cat(h).cuda()
    delta = part.forward(device_hidden, None, batch, cell)
    config = plain.PlainConfig(1, hidden, 96, 1, heads, kv_heads, dim, 10000.0, 1e-5, True, True, "adjacent")
    weights = {"layers.0." + name: value for name, value in exact.items()}
    expected = torch.cat([plain.decoder_layer(x.double(), weights, 0, config, torch.arange(x.shape[0])) for x in h])
    torch.testing.assert_close((device_hidden + delta).cpu().double(), expected, **TOLERANCE[dtype])


@pytest.mark.parametrize("dtype,page", [(torch.float32, 4), (torch.bfloat16, 8)])
def test_toy_architecture_on_the_gpu(tmp_path, kernels, dtype, page):
    """(pages of 8 in bfloat16: the attention whose scores carry a distance bias and a soft cap then runs on the
    matrix cores, as it does in float32)"""
    toy.register_toy()
    try:
        folder = toy.write_toy_folder(tmp_path / "toy")
        loaded = load_model_folder(folder, "float32" if dtype == torch.float32 else "bfloat16")
        runner = ModelRunner(loaded, kernels[dtype], CacheConfig(block_size=page, num_blocks=40, max_sequences=3))
        tokens = random_tokens(30, toy.TOY.vocab_size, seed=8)
        expected = toy.plain_toy_forward(folder, tokens)
        rows, at = [], 0
        for count in (7, 1, 1, 2, 19):
            rows.append(runner.step([StepEntry("t", tokens[at : at + count], range(count))], create_missing=True).clone())
            at += count
        bound = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=0.06 * float(expected.std()), rtol=3e-2)
        torch.testing.assert_close(torch.cat(rows).cpu().double(), expected, **bound)
        runner.close()
    finally:
        toy.unregister_toy()


def test_a_stateful_architecture_is_captured_and_replayed(tmp_path, kernels):
    """The toy architecture whose mixer keeps a state slot per request and runs on the device alone, with
    attention whose scores carry a distance bias and a soft cap: its decode steps and its mixed steps are
    replayed from graphs (the requests that pad a captured step write to a spare state slot, not to a
    request's), a request that ends hands its slot to the next with the state zeroed, and every logit is the
    plain forward's, in float32 and in bfloat16."""
    toy.register_toy()
    try:
        folder = toy.write_toy_folder(tmp_path / "sum", config=toy.SUM)
        sequences = [random_tokens(n, toy.SUM.vocab_size, seed=40 + n) for n in (33, 18, 26)]
        expected = [toy.plain_toy_forward(folder, tokens) for tokens in sequences]
        for dtype in DTYPES:
            loaded = load_model_folder(folder, "float32" if dtype == torch.float32 else "bfloat16")
            runner = ModelRunner(loaded, kernels[dtype], CacheConfig(block_size=4, num_blocks=40, max_sequences=3))
            assert runner.use_graphs and runner.cache.states
            bound = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=0.06 * float(expected[0].std()), rtol=3e-2)
            fed = [0, 0, 0]
            for turn in range(12):
                # request 0 decodes from the start; 1 and 2 bring portions of three tokens, then decode
                entries = []
                for index, tokens in enumerate(sequences):
                    count = 1 if index == 0 or turn >= 5 else 3
                    if fed[index] + count <= len(tokens):
                        entries.append((index, StepEntry(f"r{index}", tokens[fed[index] : fed[index] + count], [count - 1])))
                logits = runner.step([entry for _, entry in entries], create_missing=True).clone()
                for row, (index, entry) in enumerate(entries):
                    fed[index] += len(entry.tokens)
                    torch.testing.assert_close(logits[row].cpu().double(), expected[index][fed[index] - 1], **bound,
                                               msg=lambda m: f"{dtype} turn {turn} request {index}: {m}")
            assert runner.step_counts["replayed"] >= 4 and runner.step_counts["captured"] >= 2, runner.step_counts  # mixed and decode steps came from graphs
            runner.end_request("r1")  # its slot, state zeroed, goes to a new request
            again = runner.step([StepEntry("new", sequences[1], [len(sequences[1]) - 1])], create_missing=True)
            torch.testing.assert_close(again[0].cpu().double(), expected[1][-1], **bound)
            runner.close()
    finally:
        toy.unregister_toy()


def test_cache_needs_of_a_kind_of_their_own_on_the_gpu(tmp_path, kernels):
    """The third toy architecture on the GPU, in both precisions: pages of a kind of need that the cache manager
    has never heard of (a narrow key row and a wider value row per token), a run that holds pages and a state
    slot at once, and a feed-forward whose gate is a gelu (a plain product and the activation kernel behind
    it); three requests in changing portions against the plain forward, and the pages against its rows."""
    from tests.test_toy_parts import step_in_portions

    toy.register_toy()
    try:
        folder = toy.write_toy_folder(tmp_path / "latent", config=toy.LATENT)
        prompts = {name: random_tokens(n, toy.LATENT.vocab_size, seed=n) for name, n in (("a", 37), ("b", 9), ("c", 22))}
        expected = {name: toy.plain_toy_forward(folder, tokens, with_cached_rows=True) for name, tokens in prompts.items()}
        spread = float(torch.cat([logits for logits, _ in expected.values()]).std())
        for dtype in DTYPES:
            loaded = load_model_folder(folder, "float32" if dtype == torch.float32 else "bfloat16")
            runner = ModelRunner(loaded, kernels[dtype], CacheConfig(block_size=4, num_blocks=20, max_sequences=3))
            assert not runner.use_graphs and len(runner.cache.groups) == 2 and len(runner.cache.states) == 1
            got = step_in_portions(runner, prompts, {"a": [5, 1, 1, 9, 2, 19], "b": [2, 7], "c": [1, 1, 1, 1, 18]})
            bound = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=0.06 * spread, rtol=3e-2)
            for name in prompts:
                torch.testing.assert_close(got[name].cpu().double(), expected[name][0], **bound)
                first, rows = runner.cache.gather_fields(name, 0)
                stored = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
                torch.testing.assert_close(rows["key_rows"].cpu().double(), expected[name][1][0], **stored)
                torch.testing.assert_close(rows["value_rows"].cpu().double(), expected[name][1][1], **stored)
            for name in prompts:
                runner.end_request(name)
            runner.cache.check_invariants()
            assert runner.cache.used_pages == 0
            runner.close()
    finally:
        toy.unregister_toy()


# ------------------------------------------------------------------------------- entry points


@pytest.mark.parametrize("name", ["B", "B-loud"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(model_folders, dtype, name):
    config, page = CONFIGS[name]
    plain_config, weights = plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])
    prompts = [random_tokens(n, config.vocab_size, seed=n) for n in (2, 9, 23, 40, 64, 100)]
    expected = [plain.generate(weights, plain_config, prompt, 12) for prompt in prompts]

    async def run():
        async with LLMEngine(str(model_folders[name]), cache_config=CacheConfig(page, 96, 8),
                             scheduler_config=SchedulerConfig(4, 64), prefill_chunk_size=16, dtype=dtype) as engine:
            streamed = [[] for _ in prompts]
            outputs = await asyncio.gather(*[
                engine.generate(prompt, GenerationConfig(max_new_tokens=12), streamed[index].append)
                for index, prompt in enumerate(prompts)
            ])
            assert engine.cache.used_pages == 0
            return outputs, streamed

    outputs, streamed = asyncio.run(run())
    assert streamed == outputs
    if dtype == "float32":
        assert outputs == expected
    else:  # bfloat16 may turn a near-tie: every token must be the plain decoder's choice, or within rounding of it
        from tests.tiny import unjustified_greedy_tokens

        for prompt, got in zip(prompts, outputs):
            assert len(got) == 12 and not unjustified_greedy_tokens(plain, weights, plain_config, prompt, got)
        agreeing = sum(a == b for got, want in zip(outputs, expected) for a, b in zip(got, want))
        print(f"{name}: {agreeing} of {12 * len(prompts)} tokens equal the plain decoder's")


def test_sampled_generation_is_the_plain_decoders(model_folders):
    config, page = CONFIGS["B"]
    plain_config, weights = plain.PlainConfig.from_folder(model_folders["B"]), plain.read_weights(model_folders["B"])
    prompts = [random_tokens(n, config.vocab_size, seed=50 + n) for n in (9, 40)]
    settings = [GenerationConfig(12, 0.8, 1.0, seed=5), GenerationConfig(12, 0.8, 0.9, seed=6)]
    expected = [plain.generate(weights, plain_config, p, 12, s.temperature, s.top_p, s.seed) for p, s in zip(prompts, settings)]
    from llmserve_amd.kernels import HipKernels

    loaded = load_model_folder(model_folders["B"], "float32")
    runner = ModelRunner(loaded, HipKernels(torch.float32), CacheConfig(page, 64, 4))
    assert EngineCore(runner, SchedulerConfig(2, 64), prefill_chunk_size=16).generate(prompts, settings) == expected
    runner.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(model_folders, dtype):
    """300 tokens decoded one by one after a one-token prompt (the first tokens of a sequence,
    then many captured steps, page after page), each step's logits against the plain forward."""
    from tests.tiny import BF16_LARGEST, BF16_MEAN

    name = "A-loud"  # weights wide enough that attention decides the logits
    config, page = CONFIGS[name]
    plain_config, weights = plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])
    tokens = random_tokens(300, config.vocab_size, seed=4)
    expected = plain.forward(weights, plain_config, tokens)
    from llmserve_amd.kernels import HipKernels

    loaded = load_model_folder(model_folders[name], dtype)
    runner = ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(page, 24, 2))
    rows = [runner.step([StepEntry("r", [token], [0])], create_missing=True).clone() for token in tokens]
    got = torch.cat(rows).cpu().double()
    spread = float(expected.std())
    tolerance = dict(atol=2e-5 * max(1.0, spread / 0.3), rtol=1e-4) if dtype == "float32" else dict(atol=BF16_LARGEST * spread, rtol=3e-2)
    torch.testing.assert_close(got, expected, **tolerance)
    if dtype == "bfloat16":
        assert float((got - expected).abs().mean()) < BF16_MEAN * spread
    runner.close()


def test_command_line_generates(model_folders, tmp_path):
    common = ["--model", str(model_folders["A"]), "--dtype", "float32", "--block-size", "16", "--num-blocks", "64"]
    done = subprocess.run([sys.executable, str(ROOT / "bin" / "llmserve"), "generate", "--prompt-tokens", "5,17,3,200",
                           "--max-tokens", "6", *common], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    plain_config, weights = plain.PlainConfig.from_folder(model_folders["A"]), plain.read_weights(model_folders["A"])
    expected = plain.generate(weights, plain_config, [5, 17, 3, 200], 6)
    assert json.loads(done.stdout.strip().splitlines()[-1])["token_ids"] == expected
    # a folder that names its end-of-sequence token: generation stops there unless told otherwise
    import shutil

    named = tmp_path / "named"
    shutil.copytree(model_folders["A"], named)
    (named / "generation_config.json").write_text(json.dumps({"eos_token_id": [expected[2], 999999]}))
    for extra, wanted in (([], expected[: expected.index(expected[2]) + 1]), (["--ignore-eos"], expected)):
        done = subprocess.run([sys.executable, str(ROOT / "bin" / "llmserve"), "generate", "--prompt-tokens", "5,17,3,200",
                               "--max-tokens", "6", "--model", str(named), *common[2:], *extra], capture_output=True, text=True, timeout=300)
        assert done.returncode == 0, done.stderr[-2000:]
        assert json.loads(done.stdout.strip().splitlines()[-1])["token_ids"] == wanted
    output = tmp_path / "bench.json"
    done = subprocess.run([sys.executable, str(ROOT / "bin" / "llmserve"), "benchmark", "--config", "continuous",
                           "--requests", "6", "--arrival-rate", "200", "--batch-size", "4", "--output", str(output),
                           *common, "--num-blocks", "512"], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    summary = json.loads(output.read_text())["summary"]
    assert summary["successful_requests"] == 6 and summary["throughput_tokens_per_s"] > 0


def test_first_step_of_a_process_may_be_a_captured_one_of_many_rows(model_folders):
    """A fresh process whose prompts are short: no step before the first decode step has more than 16
    rows, so that step, captured into a graph, is the first to meet the BLAS library (which takes the
    products of 17 to 64 rows inside a capture).  The library must be set up by then."""
    script = f"""
import sys
sys.path.insert(0, {str(ROOT)!r})
from llmserve_amd import CacheConfig, EngineCore, GenerationConfig, ModelRunner, SchedulerConfig
from llmserve_amd.kernels import HipKernels
from llmserve_amd.weights import load_model_folder
loaded = load_model_folder({str(model_folders["B"])!r}, "bfloat16")
runner = ModelRunner(loaded, HipKernels(loaded.dtype, "cuda:0"), CacheConfig(8, 256, 32))
core = EngineCore(runner, SchedulerConfig(24, 64), prefill_chunk_size=16)
produced = core.generate([[7 + i, 3] for i in range(20)], GenerationConfig(max_new_tokens=4))
assert len(produced) == 20 and all(len(tokens) == 4 for tokens in produced), produced
runner.close()
print("ok")
"""
    done = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0 and done.stdout.strip().endswith("ok"), done.stderr[-2000:]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_everything_at_once_matches_the_plain_decoder(model_folders, dtype):
    """Twelve requests through the engine on the GPU with all it has switched on (captured decode steps,
    the next step prepared and queued ahead): greedy and sampled requests side by side, some with stop
    tokens, late arrivals, and so few pages that requests give way and replay.  In float32 every
    request's tokens are the plain decoder's.  In bfloat16 (the fused decode kernel that stores keys and
    values itself, key splits merged by the output projection, captured graphs whose padded rows read
    page 0, a stopped request's row in a step queued ahead writing into pages that were given back) a
    near-tie may turn, so every token is checked against the plain decoder fed the run's own prefix: a
    greedy token must be its choice or within rounding of it, a sampled one must be what its rule gives at
    the request's own draw once the probabilities may move by the bfloat16 bound.  The cache's books are
    checked after every step."""
    from llmserve_amd.engine import Request
    from llmserve_amd.kernels import HipKernels
    from tests.tiny import unjustified_tokens

    name = "B" if dtype == "float32" else "B-loud"  # wide weights: attention decides the logits (tests/tiny.py)
    config, page = CONFIGS[name]
    plain_config, weights = plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])
    lengths = [3, 30, 17, 1, 44, 9, 25, 2, 38, 12, 21, 5]
    prompts = [random_tokens(n, config.vocab_size, seed=100 + n) for n in lengths]
    settings = []
    for index in range(len(prompts)):
        sampled = index % 3 == 1
        # stop tokens: a tenth of the vocabulary, so that some requests stop early
        stops = tuple(range(index, config.vocab_size, 10)) if index % 4 == 0 else ()
        settings.append(GenerationConfig(10 + index, 0.9 if sampled else 0.0, 0.85 if index % 2 else 1.0, seed=index, stop_token_ids=stops))
    loaded = load_model_folder(model_folders[name], dtype)
    runner = ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(page, 14, 6))  # 14 pages of 8: 112 tokens
    core = EngineCore(runner, SchedulerConfig(5, 48), prefill_chunk_size=16)
    queued_ahead = 0
    step_from_device = runner.step_from_device

    def counted(*args, **kwargs):
        nonlocal queued_ahead
        queued_ahead += 1
        return step_from_device(*args, **kwargs)

    runner.step_from_device = counted
    requests = [Request(f"r{index}", prompt, s) for index, (prompt, s) in enumerate(zip(prompts, settings))]
    for request in requests[:5]:
        core.submit(request)
    waiting = requests[5:]
    turn = 0
    while core.has_work or waiting:
        if waiting and turn % 3 == 0:  # the others arrive one by one while the engine runs
            core.submit(waiting.pop(0))
        core.step()
        runner.cache.check_invariants()
        turn += 1
        assert turn < 2000
    torch.cuda.synchronize()
    assert runner.cache.used_pages == 0
    assert all(request.error is None for request in requests)
    assert sum(r.evictions for r in requests) > 0, "the pool was meant to be too small"
    assert any(len(r.output) < s.max_new_tokens for r, s in zip(requests, settings)), "nobody stopped early"
    assert runner.step_counts["replayed"] > 0 and queued_ahead > 0, (runner.step_counts, queued_ahead)
    if dtype == "float32":
        expected = [
            plain.generate(weights, plain_config, p, s.max_new_tokens, s.temperature, s.top_p, s.seed, s.stop_token_ids)
            for p, s in zip(prompts, settings)
        ]
        assert [r.output for r in requests] == expected
    else:
        for request, prompt, chosen in zip(requests, prompts, settings):
            assert not unjustified_tokens(plain, weights, plain_config, prompt, request.output, chosen), request.request_id
    runner.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_workloads_on_the_gpu(model_folders, dtype):
    """The whole runs drawn at random that the CPU tests put through the torch stand-in (tests/random_runs.py:
    pool, batch, budget, portion size, policy, who gives way, greedy and sampled requests with stop tokens, late
    arrivals), here through the kernels, captured steps and steps queued ahead: in float32 the plain decoder's
    tokens exactly, in bfloat16 (the loud folders) tokens that its rule can give for the run's own prefix."""
    from llmserve_amd.kernels import HipKernels
    from tests.random_runs import run_random_workload

    def make(name, blocks, batch):
        loaded = load_model_folder(model_folders[name], dtype)
        return ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(CONFIGS[name][1], blocks, batch))

    names = ("A", "B") if dtype == "float32" else ("A-loud", "B-loud")
    gave_way = [run_random_workload(3000 + case, model_folders, make, names, exact=dtype == "float32") for case in range(16)]
    torch.cuda.synchronize()
    assert sum(1 for count in gave_way if count > 0) >= 2, gave_way


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_second_tiny_workload_as_stated(model_folders, dtype):
    """Six requests with prompts of 2, 9, 23, 40, 64 and 100 tokens, fed in portions of 16 beside the
    decoded tokens of those that are ahead, twelve tokens each at temperature 0.8 from one seed: in
    float32 the plain decoder's tokens, in bfloat16 tokens that its rule can give for the run's own prefix."""
    from llmserve_amd.kernels import HipKernels
    from tests.tiny import unjustified_tokens

    name = "B" if dtype == "float32" else "B-loud"
    config, page = CONFIGS[name]
    plain_config, weights = plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])
    prompts = [random_tokens(n, config.vocab_size, seed=n) for n in (2, 9, 23, 40, 64, 100)]
    chosen = GenerationConfig(12, 0.8, 1.0, seed=1234)
    loaded = load_model_folder(model_folders[name], dtype)
    runner = ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(page, 64, 8))
    core = EngineCore(runner, SchedulerConfig(6, 64), prefill_chunk_size=16)
    core.step_log = []
    produced = core.generate(prompts, chosen)
    torch.cuda.synchronize()
    assert any(len({count for _, count in plan}) > 1 and 16 in {count for _, count in plan} for plan in core.step_log), \
        "portions of 16 were meant to run beside decoded tokens"
    if dtype == "float32":
        assert produced == [plain.generate(weights, plain_config, p, 12, 0.8, 1.0, 1234) for p in prompts]
    else:
        for prompt, got in zip(prompts, produced):
            assert not unjustified_tokens(plain, weights, plain_config, prompt, got, chosen)
    assert runner.cache.used_pages == 0
    runner.close()


@pytest.mark.parametrize("case", range(16))
def test_random_configurations_against_the_plain_forward(tmp_path, kernels, case):
    """Configurations drawn at random: head sizes in steps of 16 up to 256, one to five kv heads with
    one to seventeen query heads each, widths and vocabularies that are no power of two (some no
    multiple of 32, which the MFMA kernels refuse and the generic ones take), pages of 4 to 64, windows,
    with and without bias and tied head, both pairings.  Three requests go through the step function in
    portions of changing size side by side, then decode; every row's logits against the plain forward."""
    import random

    from llmserve_amd import Qwen2Config
    from llmserve_amd.weights import write_model_folder

    rng = random.Random(1000 + case)
    kv_heads, group = rng.choice([1, 2, 3, 5]), rng.choice([1, 2, 3, 5, 6, 7, 17])
    window = rng.choice([None, None, 5, 19, 40])
    config = Qwen2Config(
        vocab_size=rng.choice([61, 128, 257, 1000, 1031]), hidden_size=rng.choice([40, 64, 72, 96, 100, 128, 136, 160, 256, 264]),
        intermediate_size=rng.choice([48, 56, 96, 100, 128, 160, 256, 384, 392]), num_layers=rng.choice([1, 2, 3]),
        num_attention_heads=kv_heads * group, num_key_value_heads=kv_heads,
        head_dim=16 * rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 12, 16]), max_position_embeddings=512,
        rope_theta=rng.choice([100.0, 10000.0, 1e6]), rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-3]),
        attention_bias=rng.random() < 0.7, tie_word_embeddings=rng.random() < 0.5, rope_pairing=rng.choice(["adjacent", "half"]),
        use_sliding_window=window is not None, sliding_window=window or 0, max_window_layers=rng.choice([0, 1]) if window else 0,
    )
    page = rng.choice([4, 8, 16, 24, 32, 64])
    folder = write_model_folder(tmp_path / "model", config, seed=case, norm_std=0.1, std=0.08)
    plain_config, weights = plain.PlainConfig.from_folder(folder), plain.read_weights(folder)
    lengths = [rng.choice([1, 2, 7, 33, 70, 130]), rng.choice([3, 17, 64, 65, 97]), rng.choice([5, 40])]
    sequences = [[rng.randrange(config.vocab_size) for _ in range(n + 6)] for n in lengths]
    expected = [plain.forward(weights, plain_config, tokens) for tokens in sequences]
    for dtype in DTYPES:
        loaded = load_model_folder(folder, "float32" if dtype == torch.float32 else "bfloat16")
        pages = sum(-(-len(tokens) // page) for tokens in sequences) + 2
        runner = ModelRunner(loaded, kernels[dtype], CacheConfig(page, pages, 4))
        got, fed = [[] for _ in sequences], [0] * len(sequences)
        while any(fed[i] < lengths[i] for i in range(len(sequences))):
            entries = []
            for i, tokens in enumerate(sequences):
                if fed[i] < lengths[i]:
                    count = min(rng.choice([1, 2, 5, 16, 50]), lengths[i] - fed[i])
                    entries.append((i, StepEntry(f"r{i}", tokens[fed[i] : fed[i] + count], list(range(count)))))
                    fed[i] += count
            logits, at = runner.step([entry for _, entry in entries], create_missing=True), 0
            for i, entry in entries:
                got[i].append(logits[at : at + len(entry.tokens)].clone())
                at += len(entry.tokens)
        for step in range(6):
            logits = runner.step([StepEntry(f"r{i}", [tokens[lengths[i] + step]], [0]) for i, tokens in enumerate(sequences)])
            for i in range(len(sequences)):
                got[i].append(logits[i : i + 1].clone())
        for i in range(len(sequences)):
            spread = float(expected[i].std())  # bounds in units of the logits' spread, as these models' scales differ
            bound = dict(atol=1e-4 * spread, rtol=1e-4) if dtype == torch.float32 else dict(atol=0.2 * spread, rtol=5e-2)
            torch.testing.assert_close(torch.cat(got[i]).cpu().double(), expected[i], **bound, msg=lambda m: f"{config} page {page} request {i}: {m}")
        runner.close()


def test_captured_graphs_are_dropped_by_last_use_and_captured_again(model_folders):
    """More shapes of decode steps than the runner keeps graphs for: the graph used longest ago goes (after
    the device has finished with it), a shape that comes back is captured again, and every step's logits
    are the plain forward's whatever was dropped in between."""
    from llmserve_amd.kernels import HipKernels

    name = "A-loud"
    config, page = CONFIGS[name]
    plain_config, weights = plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])
    sequences = [random_tokens(40, config.vocab_size, seed=900 + index) for index in range(5)]
    expected = [plain.forward(weights, plain_config, tokens) for tokens in sequences]
    loaded = load_model_folder(model_folders[name], "float32")
    runner = ModelRunner(loaded, HipKernels(torch.float32), CacheConfig(page, 32, 8))
    runner.max_graphs = 2
    runner.step([StepEntry(f"r{index}", tokens[:8], []) for index, tokens in enumerate(sequences)], create_missing=True)
    fed = [8] * 5
    seen = []
    # batches of 1, 2, 3 (padded to 4), 5 (padded to 8) requests, coming back to earlier shapes
    for group in ([0], [0, 1], [0, 1, 2], [0], [0, 1, 2, 3, 4], [0, 1], [2, 3, 4], [0], [1, 2, 3, 4, 0], [3]):
        logits = runner.step([StepEntry(f"r{index}", [sequences[index][fed[index]]], [0]) for index in group])
        for row, index in enumerate(group):
            torch.testing.assert_close(logits[row].cpu().double(), expected[index][fed[index]], atol=5e-5, rtol=1e-4)
            fed[index] += 1
        seen.append(list(runner._graphs))
        assert len(runner._graphs) <= 2
    assert seen[0] == [(1, 1)] and seen[1] == [(1, 1), (2, 1)]
    assert seen[2] == [(2, 1), (4, 1)]  # the third shape pushed out the one used longest ago
    assert seen[3] == [(4, 1), (1, 1)]  # which was captured again when it came back
    assert seen[5][-1] == (2, 1) and seen[-1][-1] == (1, 1)
    runner.close()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_host_reads_the_pages_as_the_kernels_wrote_them(model_folders, dtype, name):
    """The cache manager's host-side read path (`gather`) and the kernels agree on where a key and a
    value lie in a page: after a prompt fed in portions and three tokens decoded one by one (these are
    stored by the fused decode attention in bfloat16), the first layer's pages hold, position by position,
    the rotated keys and the values the plain implementation computes."""
    from llmserve_amd.kernels import HipKernels

    config, page = CONFIGS[name]
    plain_config, weights = plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])
    tokens = random_tokens(3 * page + 8, config.vocab_size, seed=9)
    loaded = load_model_folder(model_folders[name], dtype)
    runner = ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(page, 16, 2))
    cut = len(tokens) - 3
    for start, end in ((0, page + 3), (page + 3, page + 4), (page + 4, cut)):
        runner.step([StepEntry("r", tokens[start:end], [])], create_missing=True)
    for token in tokens[cut:]:
        runner.step([StepEntry("r", [token], [0])])
    count = len(tokens)
    hidden = weights["embed_tokens.weight"][torch.tensor(tokens)]
    normed = plain.rms_norm(hidden, weights["layers.0.input_layernorm.weight"], plain_config.rms_norm_eps)
    prefix = "layers.0.self_attn."
    shape = (count, plain_config.num_kv_heads, plain_config.head_dim)
    bias = lambda which: weights.get(prefix + which + "_proj.bias", 0.0)  # C has no q/k/v biases
    keys = (normed @ weights[prefix + "k_proj.weight"].T + bias("k")).view(shape)
    values = (normed @ weights[prefix + "v_proj.weight"].T + bias("v")).view(shape)
    rotate = plain.rope_half if plain_config.rope_pairing == "half" else plain.rope_adjacent
    keys = rotate(keys, plain.rope_angles(plain_config.head_dim, plain_config.rope_theta, torch.arange(count)))
    first, cached_keys, cached_values = runner.cache.gather("r", 0)
    assert first == 0 and cached_keys.shape == shape
    tolerance = dict(atol=1e-5, rtol=1e-5) if dtype == "float32" else dict(atol=3e-2, rtol=3e-2)
    torch.testing.assert_close(cached_keys.cpu().double(), keys, **tolerance)
    torch.testing.assert_close(cached_values.cpu().double(), values, **tolerance)
    runner.close()
