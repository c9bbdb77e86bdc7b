"""Step function, scheduler and entry point without a GPU.  The kernel library
is replaced by the torch stand-in of tests/torch_kernels.py, so what is tested
here is the engine's own logic: batching, cache use, planning, giving way."""

from __future__ import annotations

import asyncio

import pytest
import torch

from llmserve_amd import CacheConfig, CacheFullError, GenerationConfig, LLMEngine, SchedulerConfig, StepEntry
from llmserve_amd.engine import EngineCore, IterationScheduler, ModelRunner, RequestState, plan_iteration
from llmserve_amd.sampling import uniform_for
from llmserve_amd.weights import load_model_folder
from tests.plain import qwen2_plain as plain
from tests.tiny import CONFIGS, random_tokens
from tests.torch_kernels import TorchKernels


def make_runner(model_folders, name, num_blocks=64, max_sequences=8, dtype="float32"):
    loaded = load_model_folder(model_folders[name], dtype)
    cache = CacheConfig(block_size=CONFIGS[name][1], num_blocks=num_blocks, max_sequences=max_sequences)
    return ModelRunner(loaded, TorchKernels(loaded.dtype), cache)


def oracle(model_folders, name):
    return plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])


def close(actual, expected):
    torch.testing.assert_close(actual.double(), expected, atol=1e-5, rtol=1e-5)


# --------------------------------------------------------------------------- the step function


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_then_one_by_one_then_portions(model_folders, name):
    config, weights = oracle(model_folders, name)
    tokens = random_tokens(70, config.vocab_size, seed=3)
    expected = plain.forward(weights, config, tokens)
    runner = make_runner(model_folders, name)
    close(runner.step([StepEntry("whole", tokens, range(70))], create_missing=True), expected)
    rows = [runner.step([StepEntry("tail", tokens[:38], [37])], create_missing=True)]
    rows += [runner.step([StepEntry("tail", [token], [0])]) for token in tokens[38:]]
    close(torch.cat(rows), expected[37:])
    rows, at = [], 0
    for count in (7, 2, 16, 3, 2, 25, 1, 14):
        rows.append(runner.step([StepEntry("cut", tokens[at : at + count], range(count))], create_missing=True))
        at += count
    close(torch.cat(rows), expected)
    runner.cache.check_invariants()


@pytest.mark.parametrize("name", ["A", "B"])
def test_mixed_batches_with_pages_used_again(model_folders, name):
    config, weights = oracle(model_folders, name)
    page = CONFIGS[name][1]
    lengths = [45, 9, 30, 61, 17, 26]
    prompts = [random_tokens(n, config.vocab_size, seed=10 + i) for i, n in enumerate(lengths)]
    expected = [plain.forward(weights, config, prompt) for prompt in prompts]
    runner = make_runner(model_folders, name, num_blocks=-(-160 // page), max_sequences=4)
    rng = torch.Generator().manual_seed(5)
    done = [0] * len(prompts)
    got = [[] for _ in prompts]
    waiting, live = list(range(len(prompts))), []
    while waiting or live:
        while waiting and len(live) < 4 and sum(-(-lengths[i] // page) for i in live + [waiting[0]]) * page <= 160:
            live.append(waiting.pop(0))
        entries, ended = [], []
        for index in live:
            left = lengths[index] - done[index]
            count = min(left, int(torch.randint(1, 12, (1,), generator=rng)))
            if done[index] > lengths[index] // 2:
                count = 1  # the second half is "decoded" token by token beside the others' portions
            entries.append((index, StepEntry(f"r{index}", prompts[index][done[index] : done[index] + count], range(count))))
            done[index] += count
            if done[index] == lengths[index]:
                ended.append(index)
        logits = runner.step([entry for _, entry in entries], create_missing=True)
        at = 0
        for index, entry in entries:
            got[index].append(logits[at : at + len(entry.tokens)])
            at += len(entry.tokens)
        for index in ended:
            runner.end_request(f"r{index}")
            live.remove(index)
        runner.cache.check_invariants()
    assert runner.cache.used_pages == 0
    for index in range(len(prompts)):
        close(torch.cat(got[index]), expected[index])


def test_a_step_that_does_not_fit_changes_nothing(model_folders):
    runner = make_runner(model_folders, "A", num_blocks=2)
    with pytest.raises(CacheFullError):
        runner.step([StepEntry("a", [1] * 20, []), StepEntry("b", [2] * 20, [])], create_missing=True)
    assert not runner.cache.sequences and runner.cache.used_pages == 0
    for bad in ([StepEntry("a", [], [])], [StepEntry("a", [1], [1])], [StepEntry("a", [999], [0])],
                [StepEntry("a", [1], []), StepEntry("a", [2], [])]):
        with pytest.raises(ValueError):
            runner.step(bad, create_missing=True)
    with pytest.raises(KeyError):
        runner.step([StepEntry("unknown", [1], [])])
    assert runner.step([StepEntry("a", [1, 2, 3], [])], create_missing=True).shape == (0, 256)


# --------------------------------------------------------------------------- scheduler decisions


def test_policies_and_the_static_barrier():
    """reference tests/test_engine.py:323-334"""
    scheduler = IterationScheduler(2, policy="sjf", mode="static")
    long, short, later = RequestState("long", [1], 20), RequestState("short", [1], 2), RequestState("later", [1], 1)
    scheduler.add(long)
    scheduler.add(short)
    assert [r.request_id for r in scheduler.admit()] == ["short", "long"]
    scheduler.add(later)
    assert scheduler.admit() == []
    scheduler.finish(short)
    assert scheduler.admit() == []
    scheduler.finish(long)
    assert scheduler.admit() == [later]

    by_priority = IterationScheduler(2, policy="priority")
    for name, priority in (("low", 0), ("high", 5), ("mid", 2)):
        by_priority.add(RequestState(name, [1], 4, priority=priority))
    assert [r.request_id for r in by_priority.admit()] == ["high", "mid"]

    first_come = IterationScheduler(1, policy="fcfs")
    a, b = RequestState("a", [1, 2], 4), RequestState("b", [1], 4)
    first_come.add(a)
    first_come.add(b)
    assert first_come.admit() == [a]
    a.processed_tokens = 2
    first_come.preempt(a)  # scheduler.py:88-93
    assert (a.processed_tokens, a.recomputed_tokens, a.preemptions) == (0, 2, 1)
    assert first_come.admit() == [a]  # it keeps its place in arrival order
    with pytest.raises(ValueError):
        IterationScheduler(2, policy="random")


def test_plan_gives_everyone_one_token_then_tops_up():
    """reference engine.py:372-391"""
    decoding = RequestState("d", [1, 2], 8, generated_token_ids=[3], processed_tokens=2)
    long = RequestState("l", list(range(40)), 8)
    short = RequestState("s", list(range(5)), 8)
    plan = plan_iteration([decoding, long, short], 2048, 16)
    assert [count for _, count in plan] == [1, 16, 5]
    assert [count for _, count in plan_iteration([decoding, long, short], 10, 16)] == [1, 8, 1]
    assert [count for _, count in plan_iteration([long, short], 2, 16)] == [1, 1]
    done = RequestState("x", [1], 8, processed_tokens=1)
    with pytest.raises(RuntimeError):
        plan_iteration([done], 8, 4)


def core_for(model_folders, name="A", num_blocks=64, batch=4, budget=64, chunk=16, mode="continuous", policy="fcfs"):
    runner = make_runner(model_folders, name, num_blocks=num_blocks)
    core = EngineCore(runner, SchedulerConfig(batch, budget, policy), scheduler_mode=mode, prefill_chunk_size=chunk,
                      collect_iteration_metrics=True)
    core.step_log = []
    return core


def test_generation_equals_the_plain_decoder(model_folders):
    config, weights = oracle(model_folders, "A")
    prompts = [random_tokens(n, config.vocab_size, seed=40 + n) for n in (1, 5, 17, 33)]
    expected = [plain.generate(weights, config, prompt, 8) for prompt in prompts]
    core = core_for(model_folders, "A")
    assert core.generate(prompts, GenerationConfig(max_new_tokens=8)) == expected
    assert core.runner.cache.used_pages == 0 and core.cache_stats["peak_blocks_used"] > 0


def test_temperature_sampling_equals_the_plain_decoder_whatever_the_batch(model_folders):
    config, weights = oracle(model_folders, "B")
    prompts = [random_tokens(n, config.vocab_size, seed=60 + n) for n in (2, 9, 23, 40)]
    settings = [GenerationConfig(max_new_tokens=6, temperature=0.8, seed=100 + i, top_p=1.0 if i % 2 else 0.9)
                for i in range(4)]
    expected = [plain.generate(weights, config, p, 6, s.temperature, s.top_p, s.seed) for p, s in zip(prompts, settings)]
    together = core_for(model_folders, "B", chunk=16).generate(prompts, settings)
    alone = [core_for(model_folders, "B", batch=1, chunk=3).generate([p], [s])[0] for p, s in zip(prompts, settings)]
    assert together == expected and alone == expected
    assert uniform_for(7, 3) == plain.uniform_for(7, 3)


def test_chunked_prefill_equals_token_at_a_time(model_folders):
    """reference tests/test_engine.py:210-247"""
    prompt = list(range(1, 24))
    config = GenerationConfig(max_new_tokens=4, seed=29)
    one = core_for(model_folders, "A", batch=1, chunk=1)
    many = core_for(model_folders, "A", batch=1, chunk=16)
    assert one.generate([prompt], config) == many.generate([prompt], config)
    stats = one.iteration_stats
    assert stats["prefill_iterations"] == len(prompt) and stats["decode_iterations"] == config.max_new_tokens - 1
    assert [plan[0][1] for plan in many.step_log[:2]] == [16, 7]


def test_late_prompt_portions_run_beside_decoding(model_folders):
    """reference tests/test_engine.py:105-143"""
    core = core_for(model_folders, "A", batch=2, budget=32, chunk=16)
    long = RequestState("long", list(range(1, 41)), 5)
    core.submit(long, GenerationConfig(max_new_tokens=5))
    while not long.generated_token_ids:
        core.step()
    core.submit(RequestState("short", [7, 8, 9, 10], 2), GenerationConfig(max_new_tokens=2))
    while core.has_work:
        core.step()
    assert any(dict(plan).get("long") == 1 and dict(plan).get("short", 0) > 1 for plan in core.step_log)


def test_static_mode_keeps_a_late_request_behind_the_barrier(model_folders):
    """reference tests/test_engine.py:146-185"""
    core = core_for(model_folders, "A", batch=2, budget=32, mode="static")
    first = RequestState("first", list(range(1, 25)), 4)
    core.submit(first, GenerationConfig(max_new_tokens=4))
    core.step()
    core.submit(RequestState("late", [9, 10], 2), GenerationConfig(max_new_tokens=2))
    while core.has_work:
        core.step()
    assert not any({"first", "late"} <= set(dict(plan)) for plan in core.step_log)


def test_pages_run_out_the_largest_gives_way_and_replays(model_folders):
    """reference tests/test_engine.py:280-320: page 16, 3 pages, two prompts that cannot both grow"""
    config, weights = oracle(model_folders, "A")
    prompts = [random_tokens(20, config.vocab_size, seed=1), random_tokens(20, config.vocab_size, seed=2)]
    expected = [plain.generate(weights, config, prompt, 14) for prompt in prompts]
    core = core_for(model_folders, "A", num_blocks=3, batch=2, budget=8, chunk=4)
    streamed = {"request-000000": [], "request-000001": []}
    requests = []
    for index, prompt in enumerate(prompts):
        request = RequestState(f"request-{index:06d}", prompt, 14)
        core.submit(request, GenerationConfig(max_new_tokens=14))
        requests.append(request)
    while core.has_work:
        for event in core.step():
            streamed[event.request.request_id].append(event.token)
        core.runner.cache.check_invariants()
    assert sum(r.preemptions for r in requests) > 0 and sum(r.recomputed_tokens for r in requests) > 0
    assert [r.generated_token_ids for r in requests] == expected  # replay changes nothing
    assert [streamed[r.request_id] for r in requests] == expected  # and no token is streamed twice
    assert core.iteration_stats["preemptions"] == sum(r.preemptions for r in requests)
    assert core.runner.cache.used_pages == 0


def test_looking_ahead_changes_no_decision(model_folders):
    """While a decode step runs, the engine has the runner reserve and pack the next one, and queues
    it before this one's tokens have reached the host.  With requests that arrive late, stop early
    (a stop token is seen only after the next step was queued) and give way for want of pages,
    every plan and every token is what it is without either, and nothing stays reserved."""
    config, weights = oracle(model_folders, "A")
    prompts = [random_tokens(n, config.vocab_size, seed=70 + n) for n in (20, 9, 26, 3)]
    free_run = [plain.generate(weights, config, prompt, 12) for prompt in prompts]
    stops = [(), (free_run[1][9],), (free_run[2][2],), ()]  # two requests stop on a token of their own
    outcomes, queued_ahead = [], []
    # (prepare the next step while this one runs, and queue it before this one's tokens are read)
    for look_ahead, run_ahead in ((True, True), (True, False), (False, False)):
        core = core_for(model_folders, "A", num_blocks=3, batch=3, budget=12, chunk=8)
        core.look_ahead, core.run_ahead = look_ahead, run_ahead
        queued_ahead.append(0)
        from_device = core.runner.step_from_device

        def counted(*args, _inner=from_device, **kwargs):
            queued_ahead[-1] += 1
            return _inner(*args, **kwargs)

        core.runner.step_from_device = counted
        requests = [RequestState(f"r{i}", prompt, 12) for i, prompt in enumerate(prompts)]
        for request, stop in zip(requests[:2], stops):
            core.submit(request, GenerationConfig(max_new_tokens=12, stop_token_ids=stop))
        steps = 0
        while core.has_work or steps < 8:
            if steps == 4:
                core.submit(requests[2], GenerationConfig(max_new_tokens=12, stop_token_ids=stops[2]))
            if steps == 7:
                core.submit(requests[3], GenerationConfig(max_new_tokens=12))
            core.step()
            core.runner.cache.check_invariants()
            steps += 1
        assert not core.runner._ahead and core.runner.cache.used_pages == 0
        assert all(request.error is None for request in requests)
        outcomes.append((core.step_log, [r.generated_token_ids for r in requests], [r.preemptions for r in requests]))
    assert outcomes[0] == outcomes[1] == outcomes[2]
    assert queued_ahead[0] > 5 and queued_ahead[1:] == [0, 0]
    assert sum(outcomes[0][2]) > 0  # pages did run out
    for tokens, whole, stop in zip(outcomes[0][1], free_run, stops):
        cut = whole.index(stop[0]) + 1 if stop else len(whole)
        assert tokens == whole[:cut]


def test_a_request_that_can_never_fit_fails_alone(model_folders):
    """reference tests/test_engine.py:261-277"""
    core = core_for(model_folders, "A", num_blocks=2, batch=2)
    small = RequestState("small", [1, 2, 3], 2)
    huge = RequestState("huge", list(range(1, 60)), 2)
    core.submit(small, GenerationConfig(max_new_tokens=2))
    core.submit(huge, GenerationConfig(max_new_tokens=2))
    while core.has_work:
        core.step()
    assert isinstance(huge.error, CacheFullError) and small.error is None and len(small.generated_token_ids) == 2
    assert core.runner.cache.used_pages == 0 and not core.runner.cache.sequences
    with pytest.raises(ValueError):
        core.submit(RequestState("empty", [], 2), GenerationConfig(max_new_tokens=2))
    with pytest.raises(ValueError):
        EngineCore(core.runner, SchedulerConfig(max_batch_size=8, max_tokens_per_step=4))


# --------------------------------------------------------------------------- the asynchronous entry point


def test_async_entry_point_streams_each_token_once(model_folders):
    """reference tests/test_engine.py:85-102, :188-207"""
    config, weights = oracle(model_folders, "A")

    async def run():
        loaded = load_model_folder(model_folders["A"], "float32")
        async with LLMEngine(loaded, cache_config=CacheConfig(16, 32, 8), scheduler_config=SchedulerConfig(3, 64),
                             dtype="float32", kernels=TorchKernels(torch.float32)) as engine:
            streamed = []
            texts = ["a", "medium", "third"]
            outputs = await asyncio.gather(
                engine.generate(texts[0], GenerationConfig(max_new_tokens=3), streamed.append, request_id="r0"),
                engine.generate(texts[1], GenerationConfig(max_new_tokens=3), request_id="r1"),
                engine.generate(texts[2], GenerationConfig(max_new_tokens=3), priority=2),
            )
            with pytest.raises(ValueError):
                await engine.generate([], GenerationConfig())
            with pytest.raises(ValueError):
                await engine.generate([1], GenerationConfig(max_new_tokens=0))
            assert engine.cache.used_pages == 0 and engine.cache_stats["peak_blocks_used"] > 0
            prompts = [engine.tokenizer.encode(text) for text in texts]
        with pytest.raises(RuntimeError):
            await engine.generate([1, 2])
        return prompts, outputs, streamed

    prompts, outputs, streamed = asyncio.run(run())
    assert outputs == [plain.generate(weights, config, prompt, 3) for prompt in prompts]
    assert streamed == outputs[0]
