"""Replays the same requests through bin/trace_run whole, with the last 32 tokens one by
one, in portions of changing size, and mixed with other requests in a pool so small that
pages are used again; in 32-bit and in bfloat16; against the plain implementation."""

from __future__ import annotations

import math

import pytest
import torch

from tests.gpu_helpers import TraceBuilder, replay
from tests.plain import qwen2_plain as plain
from tests.tiny import BF16_LARGEST, BF16_MEAN, CONFIGS, PAGE_WIDE, WIDE_CONFIGS, random_tokens, write_wide_folder

pytestmark = pytest.mark.gpu

# float32: rounding only.  bfloat16: activations are rounded to 8 bits of mantissa between kernels; the
# bound is stated in units of the logits' spread (tests/tiny.py), the same for every way of cutting.
TOLERANCE = {"float32": dict(atol=2e-5, rtol=1e-4)}
LENGTHS = {"A": [1, 5, 17, 33, 70, 100], "B": [2, 9, 23, 40, 64, 100], "C": [3, 48, 65]}


def build_trace(prompts: dict[str, list[int]], page: int, budget: int = 4 * 64):
    trace = TraceBuilder()
    # 1. each request alone and whole
    for name, tokens in prompts.items():
        trace.step([(f"whole-{name}", tokens)], end=[f"whole-{name}"])
    # 2. most of it in one step, the last 32 tokens one by one
    for name, tokens in prompts.items():
        if len(tokens) <= 33:
            continue
        head = len(tokens) - 32
        trace.step([(f"tail-{name}", tokens[:head])], want="last")
        for index in range(head, len(tokens)):
            trace.step([(f"tail-{name}", tokens[index : index + 1])], end=[f"tail-{name}"] if index == len(tokens) - 1 else [])
    # 3. portions of changing size, down to two tokens (and one at the end where it remains)
    sizes = [7, 2, 16, 3, 2, 31, 5, 2, 64]
    for name, tokens in prompts.items():
        at, turn = 0, 0
        while at < len(tokens):
            count = min(sizes[turn % len(sizes)], len(tokens) - at)
            last = at + count == len(tokens)
            trace.step([(f"cut-{name}", tokens[at : at + count])], end=[f"cut-{name}"] if last else [])
            at, turn = at + count, turn + 1
    # 4. mixed: up to four live requests, portions of some beside decoded tokens of others
    names = list(prompts)
    rng = torch.Generator().manual_seed(9)
    done = {name: 0 for name in names}
    waiting, live = list(names) + [], []
    # `budget`: tokens the pool holds; each live request counts rounded up to 64
    while waiting or live:
        while waiting and len(live) < 4 and sum(-(-len(prompts[n]) // 64) * 64 for n in live + [waiting[0]]) <= budget:
            live.append(waiting.pop(0))
        entries, ended = [], []
        for name in live:
            left = len(prompts[name]) - done[name]
            count = 1 if done[name] >= len(prompts[name]) // 2 else min(left, int(torch.randint(2, 14, (1,), generator=rng)))
            entries.append((f"mix-{name}", prompts[name][done[name] : done[name] + count]))
            done[name] += count
            if done[name] == len(prompts[name]):
                ended.append(name)
        trace.step(entries, end=[f"mix-{name}" for name in ended])
        for name in ended:
            live.remove(name)
    return trace


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "A-loud", "B-loud", "C-loud"])
def test_replay_matches_plain_under_every_cut(model_folders, tmp_path, name, dtype):
    """The "loud" folders hold the same configurations with weights wide enough that attention decides the
    logits: there the bfloat16 bound can see a wrong rotation or a lost bias (test_plain.py shows it does)."""
    config, page = CONFIGS[name]
    folder = model_folders[name]
    plain_config, weights = plain.PlainConfig.from_folder(folder), plain.read_weights(folder)
    prompts = {f"p{n}": random_tokens(n, config.vocab_size, seed=100 + n) for n in LENGTHS[name[0]]}
    expected = {key: plain.forward(weights, plain_config, tokens) for key, tokens in prompts.items()}
    trace = build_trace(prompts, page)
    results = replay(folder, dtype, trace.steps, tmp_path / "out", max_tokens=4 * 64, block_size=page,
                     vocab=config.vocab_size)
    rows = trace.collect(results)
    spread = float(torch.cat(list(expected.values())).std())
    # float32: 2e-5 where the logits spread by up to 0.3 (the quiet folders); rounding grows with the size of
    # the sums, so in proportion to the spread above that (the loud folders' is three to five times wider)
    bound = dict(atol=2e-5 * max(1.0, spread / 0.3), rtol=1e-4) if dtype == "float32" else dict(atol=BF16_LARGEST * spread, rtol=3e-2)
    checked, total, count = 0, 0.0, 0
    for (request, position), logits in rows.items():
        mode, key = request.split("-", 1)
        torch.testing.assert_close(
            logits.double(), expected[key][position], **bound,
            msg=lambda m: f"{mode} {key} position {position}: {m}",
        )
        total += float((logits.double() - expected[key][position]).abs().sum())
        count += logits.numel()
        checked += 1
    whole = sum(len(t) for t in prompts.values())
    assert checked >= 3 * whole  # whole, cut and mixed give every position; tails add theirs
    print(f"{name} {dtype}: mean error {total / count / spread:.2e} of the spread {spread:.3f}")
    if dtype == "bfloat16":  # a fault that stays under the bound for the largest element still moves the mean
        assert total / count < BF16_MEAN * spread


def test_float32_cuts_agree_with_each_other_to_rounding(model_folders, tmp_path):
    """How the tokens are cut must not matter beyond rounding: compare the cuts with each other,
    tighter than with the plain implementation."""
    config, page = CONFIGS["B"]
    prompts = {"p90": random_tokens(90, config.vocab_size, seed=77)}
    trace = build_trace(prompts, page)
    rows = trace.collect(replay(model_folders["B"], "float32", trace.steps, tmp_path / "out", 256, page, config.vocab_size))
    for position in range(90):
        whole = rows[("whole-p90", position)]
        for mode in ("cut", "mix"):
            torch.testing.assert_close(rows[(f"{mode}-p90", position)], whole, atol=3e-6, rtol=1e-5)


@pytest.fixture(scope="module")
def wide_models(tmp_path_factory):
    """Model folders at the 1.5B, 7B and 32B layer widths, each written once and read once for the plain
    implementation (the 32B widths hold half a billion weights a layer)."""
    made = {}

    def get(sizes: str):
        if sizes not in made:
            folder = write_wide_folder(tmp_path_factory.mktemp("wide"), sizes)
            made[sizes] = (folder, plain.PlainConfig.from_folder(folder), plain.read_weights(folder))
        return made[sizes]

    return get


@pytest.mark.parametrize("sizes,dtype,own", [(sizes, dtype, False) for sizes in ("1.5B", "7B", "32B") for dtype in ("float32", "bfloat16")]
                         + [("1.5B", "bfloat16", True)])
def test_replay_at_benchmark_layer_sizes(wide_models, tmp_path, sizes, dtype, own):
    """The layer widths of the 1.5B, 7B and 32B configurations (head size 128; six, seven and five query
    heads a kv head), one or two layers of them: the same four ways of cutting, with prompts that cross many
    pages and a pool that the three do not fit into together.  `own`: with every product on the engine's own
    kernels (--own-products), none sent to the BLAS library."""
    WIDE = WIDE_CONFIGS[sizes][0]
    folder, plain_config, weights = wide_models(sizes)
    prompts = {f"p{n}": random_tokens(n, WIDE.vocab_size, seed=300 + n) for n in (3, 130, 290)}
    expected = {key: plain.forward(weights, plain_config, tokens) for key, tokens in prompts.items()}
    trace = build_trace(prompts, PAGE_WIDE, budget=512)
    results = replay(folder, dtype, trace.steps, tmp_path / "out", max_tokens=512, block_size=PAGE_WIDE,
                     vocab=WIDE.vocab_size, extra=("--own-products",) if own else ())
    # These logits spread five to ten times wider than the tiny models' (std 0.78 at width 1536, 1.4 at 5120), so
    # both bounds are stated in units of that spread.  bfloat16: each of the ten or so roundings of an activation
    # between kernels adds about 2^-9 of it, 0.6 % together; the largest of 1.7 million elements lies near five times
    # that.  float32: a sum over K terms in another order than the plain implementation's differs by about
    # sqrt(K) * 2^-24 of its size (a random walk of roundings); the longest sum is the down projection's, and the
    # largest element again lies near five times the typical one.
    spread = float(torch.cat(list(expected.values())).std())
    walk = math.sqrt(WIDE.intermediate_size) * 2.0 ** -24 * spread
    bound = dict(atol=5 * walk, rtol=1e-4) if dtype == "float32" else dict(atol=BF16_LARGEST * spread, rtol=3e-2)
    total, count = 0.0, 0
    for (request, position), logits in trace.collect(results).items():
        mode, key = request.split("-", 1)
        torch.testing.assert_close(
            logits.double(), expected[key][position], **bound,
            msg=lambda m: f"{mode} {key} position {position}: {m}",
        )
        total += float((logits.double() - expected[key][position]).abs().sum())
        count += logits.numel()
    print(f"{dtype}: mean error {total / count:.3e}, spread {spread:.3f}")
    # a systematic fault that stays under the bound for the largest element still moves the mean
    assert total / count < (walk if dtype == "float32" else BF16_MEAN * spread)


@pytest.mark.parametrize("sizes,requests", [("1.5B", 20), ("1.5B", 40), ("7B", 20), ("7B", 40), ("32B", 20), ("32B", 8),
                                            ("1.5B", 100), ("7B", 70), ("1.5B", 150)])
def test_captured_steps_of_many_rows_at_benchmark_layer_sizes(wide_models, sizes, requests):
    """Decode steps of 17 rows and more are replayed from a graph in which the products go other ways than
    in every other step (up to 64 rows the kernel that streams a weight through a ring in LDS, the BLAS
    library or the weight-streaming kernel for small weights; 65 to 128 rows the ring kernel with eight tiles
    of x; beyond that the library, in a graph of a multiple of 64 rows).
    So many requests decode side by side through the step function; every step's logits are
    compared with the plain forward over each request's whole sequence."""
    from llmserve_amd import CacheConfig, ModelRunner, StepEntry
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.weights import load_model_folder

    WIDE = WIDE_CONFIGS[sizes][0]
    folder, plain_config, weights = wide_models(sizes)
    decoded = 5
    sequences = [random_tokens(3 + (7 * index) % 40 + decoded, WIDE.vocab_size, seed=500 + index) for index in range(requests)]
    loaded = load_model_folder(folder, "bfloat16")
    runner = ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(PAGE_WIDE, 4 * requests + 8, requests + 1))
    # prompts first, a few requests a step; then `decoded` steps of one token per request
    for first in range(0, requests, 8):
        group = range(first, min(first + 8, requests))
        runner.step([StepEntry(f"r{index}", sequences[index][:-decoded], []) for index in group], create_missing=True)
    rows = []
    for step in range(decoded):
        at = [len(tokens) - decoded + step for tokens in sequences]
        logits = runner.step([StepEntry(f"r{index}", [sequences[index][at[index]]], [0]) for index in range(requests)])
        rows.append((at, logits.clone()))
        # between two replays of the graph: a step launched kernel by kernel (another request's prompt, then gone),
        # and the host waits for the device
        runner.step([StepEntry("between", random_tokens(9 + step, WIDE.vocab_size, seed=step), [0])], create_missing=True)
        runner.end_request("between")
        torch.cuda.synchronize()
    assert len(runner._graphs) == 1, "these steps were meant to be replays of one graph"
    expected = [plain.forward(weights, plain_config, tokens) for tokens in sequences]
    spread = float(torch.cat(expected).std())
    for at, logits in rows:
        for index in range(requests):
            torch.testing.assert_close(
                logits[index].cpu().double(), expected[index][at[index]], atol=BF16_LARGEST * spread, rtol=3e-2,
                msg=lambda m: f"request {index} position {at[index]}: {m}",
            )
    runner.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", ["1.5B", "7B", "32B"])
def test_captured_mixed_steps_at_benchmark_layer_sizes(wide_models, dtype, sizes):
    """Steps that are not single tokens are replayed from graphs of their padded shape once a shape has come
    twice: portions of prompts beside decoded tokens at the 1.5B, 7B and 32B widths (at the wider ones the padded
    step's products go other ways: library products cut over K, four tiles of weight rows a wave), the same
    shape over and over with other requests, lengths and pages in it, steps launched kernel by kernel and waits
    between the replays (a library call that records a memory clear into a graph shows on replays after the
    first).  Every step's logits against the plain forward."""
    from llmserve_amd import CacheConfig, ModelRunner, StepEntry
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.weights import load_model_folder

    WIDE = WIDE_CONFIGS[sizes][0]
    folder, plain_config, weights = wide_models(sizes)
    sequences = [random_tokens(150 + 13 * index, WIDE.vocab_size, seed=700 + index) for index in range(5)]
    expected = [plain.forward(weights, plain_config, tokens) for tokens in sequences]
    spread = float(torch.cat(expected).std())
    walk = math.sqrt(WIDE.intermediate_size) * 2.0 ** -24 * spread
    bound = dict(atol=5 * walk, rtol=1e-4) if dtype == "float32" else dict(atol=BF16_LARGEST * spread, rtol=3e-2)
    loaded = load_model_folder(folder, dtype)
    runner = ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(PAGE_WIDE, 80, 8))
    fed = [0] * 5
    # requests 0 and 1 are ahead and decode; 2 to 4 bring portions of 16 tokens (the reference's default chunk)
    runner.step([StepEntry(f"r{index}", sequences[index][:40], []) for index in (0, 1)], create_missing=True)
    fed[0] = fed[1] = 40
    for turn in range(9):
        group = [0, 1] + [2 + (turn + offset) % 3 for offset in range(2)]  # two decoding, two of the three others
        entries = []
        for index in group:
            count = 1 if index < 2 else 16
            entries.append(StepEntry(f"r{index}", sequences[index][fed[index] : fed[index] + count], [count - 1]))
        logits = runner.step(entries, create_missing=True).clone()
        for row, (index, entry) in enumerate(zip(group, entries)):
            fed[index] += len(entry.tokens)
            torch.testing.assert_close(logits[row].cpu().double(), expected[index][fed[index] - 1], **bound,
                                       msg=lambda m: f"turn {turn} request {index} position {fed[index] - 1}: {m}")
        # between two replays: a step of another shape launched kernel by kernel, and the host waits
        runner.step([StepEntry("between", random_tokens(40 + turn, WIDE.vocab_size, seed=turn), [0])], create_missing=True)
        runner.end_request("between")
        torch.cuda.synchronize()
    assert any(key[:2] == (64, 8) for key in runner._step_graphs) and runner.step_counts["replayed"] >= 8, runner.step_counts
    runner.close()


_long_expected = {}


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_a_long_context_through_the_whole_engine(wide_models, dtype):
    """Over thousands of keys a prompt portion's waves walk hundreds of steps and pages, and a decoded token's
    keys are cut into splits (merged by the output projection, or by the merging kernel): the whole engine at
    the 1.5B widths over 4,400 keys, a prompt in portions of changing size, a portion beside decoded tokens
    of another long request, then single tokens; against the plain forward, in both precisions."""
    from llmserve_amd import CacheConfig, ModelRunner, StepEntry
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.weights import load_model_folder

    WIDE = WIDE_CONFIGS["1.5B"][0]
    folder, plain_config, weights = wide_models("1.5B")
    config = WIDE
    sequences = [random_tokens(4400, config.vocab_size, seed=811), random_tokens(4250, config.vocab_size, seed=812)]
    if not _long_expected:
        _long_expected["logits"] = [plain.forward(weights, plain_config, tokens) for tokens in sequences]
    expected = _long_expected["logits"]
    spread = float(expected[0].std())
    walk = math.sqrt(WIDE.intermediate_size) * 2.0 ** -24 * spread
    bound = dict(atol=BF16_LARGEST * spread, rtol=3e-2) if dtype == "bfloat16" else dict(atol=5 * walk, rtol=1e-4)
    loaded = load_model_folder(folder, dtype)
    runner = ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(PAGE_WIDE, 2 * 280, 4), max_sequence_length=4608)
    checked, total = 0, 0.0

    def check(logits, index, positions):
        nonlocal checked, total
        for row, position in enumerate(positions):
            torch.testing.assert_close(logits[row].cpu().double(), expected[index][position], **bound,
                                       msg=lambda m: f"request {index} position {position}: {m}")
            total += float((logits[row].cpu().double() - expected[index][position]).abs().mean())
            checked += 1

    # request 0: 2,048 + 2,000 + 300 tokens; the last portion's queries look back over more than 4,096 keys
    fed = 0
    for count in (2048, 2000, 300):
        want = [0, count // 2, count - 1]
        logits = runner.step([StepEntry("r0", sequences[0][fed : fed + count], want)], create_missing=True)
        check(logits, 0, [fed + place for place in want])
        fed += count
    # request 1 catches up to 4,200 while request 0 decodes beside its portions
    at = 0
    for count in (2048, 2048, 104):
        entries = [StepEntry("r0", [sequences[0][fed]], [0]), StepEntry("r1", sequences[1][at : at + count], [count - 1])]
        logits = runner.step(entries, create_missing=True)
        check(logits[:1], 0, [fed])
        check(logits[1:], 1, [at + count - 1])
        fed, at = fed + 1, at + count
    # both decode: steps of two single tokens over 4,350 and 4,200 keys (captured, keys cut into splits)
    for _ in range(6):
        logits = runner.step([StepEntry("r0", [sequences[0][fed]], [0]), StepEntry("r1", [sequences[1][at]], [0])])
        check(logits[:1], 0, [fed])
        check(logits[1:], 1, [at])
        fed, at = fed + 1, at + 1
    assert checked == 9 + 6 + 12 and total / checked < (BF16_MEAN * spread if dtype == "bfloat16" else walk)
    runner.close()


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_nine_thousand_keys_through_the_whole_engine(tmp_path_factory, dtype):
    """A context of more than 9,000 keys through the step function, in both precisions: a prompt in portions of
    2,048 tokens (each portion's queries behind thousands of cached keys), then single tokens decoded from captured
    steps whose keys are cut into splits and merged by the merging kernel, beside a short request; a key planted
    far back must decide the last logits.  Against the plain forward of a narrow model with the benchmark's head
    size."""
    from llmserve_amd import CacheConfig, ModelRunner, StepEntry
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.weights import load_model_folder, write_model_folder
    from tests.tiny import LONG, LOUD

    folder = write_model_folder(tmp_path_factory.mktemp("long") / "long", LONG, seed=77, norm_std=0.1, **LOUD)
    plain_config, weights = plain.PlainConfig.from_folder(folder), plain.read_weights(folder)
    sequences = [random_tokens(9100, LONG.vocab_size, seed=821), random_tokens(40, LONG.vocab_size, seed=822)]
    expected = [plain.forward(weights, plain_config, tokens) for tokens in sequences]
    spread = float(expected[0].std())
    walk = math.sqrt(9100) * 2.0 ** -24 * spread
    bound = dict(atol=BF16_LARGEST * spread, rtol=3e-2) if dtype == "bfloat16" else dict(atol=8 * walk, rtol=1e-4)
    loaded = load_model_folder(folder, dtype)
    runner = ModelRunner(loaded, HipKernels(loaded.dtype), CacheConfig(PAGE_WIDE, 600, 4))
    fed, checked = 0, 0
    for count in (2048, 2048, 2048, 2048, 900):
        want = [0, count - 1]
        logits = runner.step([StepEntry("long", sequences[0][fed : fed + count], want)], create_missing=True)
        for row, place in enumerate(want):
            torch.testing.assert_close(logits[row].cpu().double(), expected[0][fed + place], **bound,
                                       msg=lambda m: f"position {fed + place}: {m}")
        fed, checked = fed + count, checked + 2
    runner.step([StepEntry("short", sequences[1][:30], [])], create_missing=True)
    for step in range(8):  # two requests decode side by side: 9,092 + step keys and 30 + step
        entries = [StepEntry("long", [sequences[0][fed + step]], [0]), StepEntry("short", [sequences[1][30 + step]], [0])]
        logits = runner.step(entries)
        torch.testing.assert_close(logits[0].cpu().double(), expected[0][fed + step], **bound,
                                   msg=lambda m: f"decoded position {fed + step}: {m}")
        torch.testing.assert_close(logits[1].cpu().double(), expected[1][30 + step], **bound)
        checked += 2
    assert checked == 26 and runner.step_counts["replayed"] >= 6
    runner.close()


def test_long_portions_at_many_heads_beside_a_decoded_token(tmp_path_factory):
    """Portions of 2,048 tokens at 28 / 4 heads of 128 go to the attention kernel that shares K and V through LDS
    unsplit (448 workgroups), the second one behind 2,048 cached keys and beside another request's decoded token
    whose 2,100 keys are cut into runs in a launch of its own; then both requests decode.  Against the plain
    forward of a narrow model."""
    from llmserve_amd import CacheConfig, ModelRunner, StepEntry
    from llmserve_amd.kernels import HipKernels
    from llmserve_amd.weights import load_model_folder, write_model_folder
    from tests.tiny import LOUD, MANY_HEADS

    folder = write_model_folder(tmp_path_factory.mktemp("heads") / "heads", MANY_HEADS, seed=78, norm_std=0.1, **LOUD)
    plain_config, weights = plain.PlainConfig.from_folder(folder), plain.read_weights(folder)
    sequences = [random_tokens(4206, MANY_HEADS.vocab_size, seed=823), random_tokens(2106, MANY_HEADS.vocab_size, seed=824)]
    expected = [plain.forward(weights, plain_config, tokens) for tokens in sequences]
    spread = float(expected[0].std())
    bound = dict(atol=BF16_LARGEST * spread, rtol=3e-2)
    loaded = load_model_folder(folder, "bfloat16")
    kernels = HipKernels(loaded.dtype)
    library = kernels._attention_library(MANY_HEADS.head_dim)  # count which launches the steps below make
    calls = {"shared": 0, "by item": 0}
    shared_entry, tiles_entry = library.llmserve_attention_portions, library.llmserve_attention_tiles

    def counted_shared(*arguments):
        calls["shared"] += 1
        return shared_entry(*arguments)

    def counted_tiles(*arguments):
        calls["by item"] += 1 if arguments[20] & 4 and arguments[19] > 1 else 0  # (fuse, splits)
        return tiles_entry(*arguments)

    library.llmserve_attention_portions, library.llmserve_attention_tiles = counted_shared, counted_tiles
    runner = ModelRunner(loaded, kernels, CacheConfig(PAGE_WIDE, 420, 4))

    def check(logits, row, sequence, position):
        torch.testing.assert_close(logits[row].cpu().double(), expected[sequence][position], **bound,
                                   msg=lambda m: f"sequence {sequence} position {position}: {m}")

    logits = runner.step([StepEntry("other", sequences[1][:2100], [2099])], create_missing=True)
    check(logits, 0, 1, 2099)
    logits = runner.step([StepEntry("long", sequences[0][:2048], [0, 1000, 2047])], create_missing=True)
    for row, position in enumerate((0, 1000, 2047)):
        check(logits, row, 0, position)
    logits = runner.step([StepEntry("long", sequences[0][2048:4096], [0, 700, 2047]), StepEntry("other", [sequences[1][2100]], [0])])
    for row, position in enumerate((2048, 2748, 4095)):
        check(logits, row, 0, position)
    check(logits, 3, 1, 2100)
    logits = runner.step([StepEntry("long", sequences[0][4096:4200], [103]), StepEntry("other", [sequences[1][2101]], [0])])
    check(logits, 0, 0, 4199)
    check(logits, 1, 1, 2101)
    for step in range(4):
        entries = [StepEntry("long", [sequences[0][4200 + step]], [0]), StepEntry("other", [sequences[1][2102 + step]], [0])]
        logits = runner.step(entries)
        check(logits, 0, 0, 4200 + step)
        check(logits, 1, 1, 2102 + step)
    library.llmserve_attention_portions, library.llmserve_attention_tiles = shared_entry, tiles_entry
    assert calls == {"shared": 3, "by item": 1}, calls  # the prompts' three long portions; the token beside the second
    runner.close()
