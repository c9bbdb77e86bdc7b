"""Step function, scheduler and entry point without a GPU.  The kernel library
is replaced by the torch stand-in of tests/torch_kernels.py, so what is tested
here is the engine's own logic: batching, cache use, planning, giving way."""

from __future__ import annotations

import asyncio

import pytest
import torch

from llmserve_amd import CacheConfig, CacheFullError, GenerationConfig, LLMEngine, SchedulerConfig, StepEntry
from llmserve_amd.engine import EngineCore, ModelRunner, Request, RequestTooLongError, Scheduler
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


def test_the_pages_of_one_layer_hold_the_rotated_keys_and_the_values(model_folders):
    """The host-side read paths (reference kv_cache.py:268-342): after a prompt was fed in portions, the
    first layer's pages hold, position by position, the keys the plain implementation computes (bias added,
    rotated) and the values; in B's windowed layers the pages a window has passed are gone."""
    for name in ("A", "B"):
        config, weights = oracle(model_folders, name)
        tokens = random_tokens(61, config.vocab_size, seed=4)
        runner = make_runner(model_folders, name)
        for start, end in ((0, 23), (23, 24), (24, 61)):
            runner.step([StepEntry("r", tokens[start:end], [])], create_missing=True)
        h = weights["embed_tokens.weight"][torch.tensor(tokens)]
        normed = plain.rms_norm(h, weights["layers.0.input_layernorm.weight"], config.rms_norm_eps)
        prefix = "layers.0.self_attn."
        keys = (normed @ weights[prefix + "k_proj.weight"].T + weights[prefix + "k_proj.bias"]).view(61, config.num_kv_heads, config.head_dim)
        values = (normed @ weights[prefix + "v_proj.weight"].T + weights[prefix + "v_proj.bias"]).view(61, config.num_kv_heads, config.head_dim)
        rotate = plain.rope_half if config.rope_pairing == "half" else plain.rope_adjacent
        keys = rotate(keys, plain.rope_angles(config.head_dim, config.rope_theta, torch.arange(61)))
        first, cached_keys, cached_values = runner.cache.gather("r", 0)
        assert first == 0 and cached_keys.shape == (61, config.num_kv_heads, config.head_dim)
        close(cached_keys, keys)
        close(cached_values, values)
        page = CONFIGS[name][1]
        starts = [start for start, _, _ in runner.cache.iter_pages("r", 0)]
        assert starts == list(range(0, 61, page))
        tables, lengths = runner.cache.block_table_tensors(["r"])
        assert lengths.tolist() == [61] and tables.shape == (1, -(-61 // page)) and (tables >= 0).all()
        if name == "B":  # layers 1 and 2 see 24 keys: pages wholly before them go when the next token is reserved
            assert runner.cache.gather("r", 1)[0] == 0
            runner.step([StepEntry("r", [5], [])])
            first, windowed, _ = runner.cache.gather("r", 1)  # the query at 61 reads keys 38 to 61
            assert first == (38 // page) * page and windowed.shape[0] == 62 - first
            assert runner.cache.gather("r", 0)[0] == 0  # the first layer sees everything
        with pytest.raises(ValueError):
            runner.cache.gather("r", 99)


# --------------------------------------------------------------------------- scheduler decisions


def request(name, prompt, max_new_tokens=4, **fields):
    return Request(name, list(prompt), GenerationConfig(max_new_tokens=max_new_tokens), **fields)


def test_policies_and_the_static_barrier():
    """reference tests/test_engine.py:323-334"""
    scheduler = Scheduler(SchedulerConfig(2, policy="sjf"), mode="static")
    long, short, later = request("long", [1], 20), request("short", [1], 2), request("later", [1], 1)
    scheduler.enqueue(long)
    scheduler.enqueue(short)
    assert [r.request_id for r in scheduler.waiting] == ["short", "long"]
    assert [r.request_id for r in scheduler.admit()] == ["short", "long"]
    assert short.admitted_at is not None
    scheduler.enqueue(later)
    assert scheduler.admit() == []
    scheduler.retire(short)
    assert scheduler.admit() == []
    scheduler.retire(long)
    assert scheduler.admit() == [later] and not scheduler.idle
    scheduler.retire(later)
    assert scheduler.idle

    by_priority = Scheduler(SchedulerConfig(2, policy="priority"))
    for name, priority in (("low", 0), ("high", 5), ("mid", 2), ("mid-too", 2)):
        by_priority.enqueue(request(name, [1], priority=priority))
    assert [r.request_id for r in by_priority.admit()] == ["high", "mid"]
    assert [r.request_id for r in by_priority.waiting] == ["mid-too", "low"] and by_priority.num_waiting == 2
    by_priority.retire(by_priority.waiting[0])  # a request may leave the line too
    assert [r.request_id for r in by_priority.waiting] == ["low"]

    first_come = Scheduler(SchedulerConfig(1, policy="fcfs"))
    a, b = request("a", [1, 2]), request("b", [1])
    first_come.enqueue(a)
    first_come.enqueue(b)
    assert first_come.admit() == [a]
    a.cached = 2
    first_admission = a.admitted_at
    first_come.evict(a)  # scheduler.py:88-93
    assert (a.cached, a.replayed_tokens, a.evictions) == (0, 2, 1)
    assert first_come.admit() == [a] and a.admitted_at == first_admission  # it keeps its place in arrival order
    with pytest.raises(ValueError):
        Scheduler(SchedulerConfig(2, policy="random"))
    with pytest.raises(ValueError):
        Scheduler(SchedulerConfig(2), mode="sometimes")


def test_shortest_job_counts_what_is_left_when_a_request_rejoins_the_line():
    scheduler = Scheduler(SchedulerConfig(1, policy="sjf"))
    long, short = request("long", [1], 10), request("short", [1], 4)
    scheduler.enqueue(long)
    assert scheduler.admit() == [long]
    scheduler.enqueue(short)
    long.output = [5] * 8  # two tokens left: fewer than the short one's four
    long.cached = 9
    scheduler.evict(long)
    assert [r.request_id for r in scheduler.waiting] == ["long", "short"]


def test_plan_gives_everyone_one_token_then_tops_up():
    """reference engine.py:372-391"""
    decoding = request("d", [1, 2], 8, output=[3], cached=2)
    long = request("l", range(40), 8)
    short = request("s", range(5), 8)

    def counts(batch, budget, chunk):
        scheduler = Scheduler(SchedulerConfig(max_batch_size=8, max_tokens_per_step=budget))
        scheduler.running = list(batch)
        return [share.count for share in scheduler.plan(chunk)]

    assert counts([decoding, long, short], 2048, 16) == [1, 16, 5]
    assert counts([decoding, long, short], 10, 16) == [1, 8, 1]
    assert counts([long, short], 2, 16) == [1, 1]
    assert counts([long, short], 1, 16) == [1, 1]  # everybody brings a token whatever the budget says
    assert long.next_tokens(3) == [0, 1, 2] and decoding.next_tokens(1) == [3]
    straddling = request("x", [1, 2, 3], 8, output=[7, 8], cached=2)
    assert straddling.next_tokens(3) == [3, 7, 8] and straddling.owed == 3 and straddling.in_prompt
    done = request("x", [1], 8, cached=1)
    with pytest.raises(RuntimeError):
        counts([done], 8, 4)


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
    long = request("long", range(1, 41), 5)
    core.submit(long)
    while not long.output:
        core.step()
    core.submit(request("short", [7, 8, 9, 10], 2))
    while core.has_work:
        core.step()
    assert any(dict(plan).get("long") == 1 and dict(plan).get("short", 0) > 1 for plan in core.step_log)


def test_static_mode_keeps_a_late_request_behind_the_barrier(model_folders):
    """reference tests/test_engine.py:146-185"""
    core = core_for(model_folders, "A", batch=2, budget=32, mode="static")
    first = request("first", range(1, 25), 4)
    core.submit(first)
    core.step()
    core.submit(request("late", [9, 10], 2))
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
        requests.append(request(f"request-{index:06d}", prompt, 14))
        core.submit(requests[-1])
    while core.has_work:
        for event in core.step():
            streamed[event.request.request_id].append(event.token)
        core.runner.cache.check_invariants()
    assert sum(r.evictions for r in requests) > 0 and sum(r.replayed_tokens for r in requests) > 0
    assert [r.output for r in requests] == expected  # replay changes nothing
    assert [streamed[r.request_id] for r in requests] == expected  # and no token is streamed twice
    assert core.iteration_stats["preemptions"] == sum(r.evictions for r in requests)
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
        requests = [Request(f"r{i}", prompt, GenerationConfig(max_new_tokens=12, stop_token_ids=stop))
                    for i, (prompt, stop) in enumerate(zip(prompts, stops))]
        for each in requests[:2]:
            core.submit(each)
        steps = 0
        while core.has_work or steps < 8:
            if steps == 4:
                core.submit(requests[2])
            if steps == 7:
                core.submit(requests[3])
            core.step()
            core.runner.cache.check_invariants()
            steps += 1
        assert not core.runner._ahead and core.runner.cache.used_pages == 0
        assert all(each.error is None for each in requests)
        outcomes.append((core.step_log, [r.output for r in requests], [r.evictions for r in requests]))
    assert outcomes[0] == outcomes[1] == outcomes[2]
    assert queued_ahead[0] > 5 and queued_ahead[1:] == [0, 0]
    assert sum(outcomes[0][2]) > 0  # pages did run out
    for tokens, whole, stop in zip(outcomes[0][1], free_run, stops):
        cut = whole.index(stop[0]) + 1 if stop else len(whole)
        assert tokens == whole[:cut]


def test_a_request_that_can_never_fit_fails_alone(model_folders):
    """reference tests/test_engine.py:261-277"""
    core = core_for(model_folders, "A", num_blocks=2, batch=2)
    small = request("small", [1, 2, 3], 2)
    huge = request("huge", range(1, 60), 2)
    core.submit(small)
    core.submit(huge)
    while core.has_work:
        core.step()
    assert isinstance(huge.error, CacheFullError) and small.error is None and len(small.output) == 2
    assert core.runner.cache.used_pages == 0 and not core.runner.cache.sequences
    with pytest.raises(ValueError):
        core.submit(request("empty", [], 2))
    with pytest.raises(ValueError):
        EngineCore(core.runner, SchedulerConfig(max_batch_size=8, max_tokens_per_step=4))


def test_a_request_that_outgrows_the_longest_sequence_costs_nobody_else(model_folders):
    """Prompt plus new tokens beyond the longest sequence the cache can describe is not a shortage of
    pages: such a request is refused when it is submitted, and one that slipped into the batch ends
    alone with an error of its own, while nobody gives way for it."""
    config, weights = oracle(model_folders, "C")  # max_position_embeddings 256
    core = core_for(model_folders, "C", num_blocks=64, batch=3, budget=64)
    assert core.runner.cache.max_sequence_length == 256
    with pytest.raises(RequestTooLongError):
        core.submit(request("long", random_tokens(199, config.vocab_size, seed=1), 100))
    with pytest.raises(ValueError, match="vocabulary"):
        core.submit(request("alien", [1, 2, config.vocab_size], 4))
    with pytest.raises(ValueError, match="vocabulary"):
        core.submit(request("negative", [1, -2], 4))
    prompts = [random_tokens(n, config.vocab_size, seed=n) for n in (30, 41)]
    others = [request(f"ok{index}", prompt, 6) for index, prompt in enumerate(prompts)]
    for each in others:
        core.submit(each)
    smuggled = request("smuggled", random_tokens(250, config.vocab_size, seed=3), 20)
    core.scheduler.enqueue(smuggled)  # past the check, as if the limit had changed under it
    while core.has_work:
        core.step()
        core.runner.cache.check_invariants()
    assert isinstance(smuggled.error, RequestTooLongError) and len(smuggled.output) == 7  # 256 cached tokens give the seventh; it cannot be fed
    assert [each.evictions for each in others] == [0, 0] and all(each.error is None for each in others)
    assert [each.output for each in others] == [plain.generate(weights, config, prompt, 6) for prompt in prompts]
    assert core.iteration_stats["preemptions"] == 0 and core.runner.cache.used_pages == 0


def test_a_full_batch_decodes_ahead_while_others_wait(model_folders):
    """Requests in the line do not stop the engine from preparing (and queueing) the next decode step
    as long as none of them can be admitted: the batch is full and stays so."""
    config, weights = oracle(model_folders, "A")
    prompts = [random_tokens(n, config.vocab_size, seed=80 + n) for n in (5, 9, 4, 7)]
    expected = [plain.generate(weights, config, prompt, 9) for prompt in prompts]
    core = core_for(model_folders, "A", batch=2, budget=32, chunk=16)
    queued = []
    inner = core.runner.step_from_device
    core.runner.step_from_device = lambda ids, tokens: (queued.append((list(ids), core.scheduler.num_waiting)), inner(ids, tokens))[1]
    assert core.generate(prompts, GenerationConfig(max_new_tokens=9)) == expected
    assert any(waiting > 0 for _, waiting in queued), "no step was queued ahead while requests waited"
    assert core.runner.cache.used_pages == 0 and not core.runner._ahead


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


def test_the_entry_point_closes_its_runner_forgets_old_facts_and_serves_again_after_a_failure(model_folders):
    """`close` drops what the runner holds (a caller of `async with` need not know the runner); the facts of
    finished requests that nobody asks for are bounded; after a step has failed and everybody was told, the
    next request is served by a new task rather than waiting for one that has ended."""
    config, weights = oracle(model_folders, "A")

    async def run():
        loaded = load_model_folder(model_folders["A"], "float32")
        engine = LLMEngine(loaded, cache_config=CacheConfig(16, 32, 8), scheduler_config=SchedulerConfig(3, 64),
                           dtype="float32", kernels=TorchKernels(torch.float32))
        closed = []
        engine.runner.close = lambda: closed.append(True)
        engine.facts_kept = 2
        for index in range(4):
            await engine.generate([5 + index, 9], GenerationConfig(max_new_tokens=2), request_id=f"r{index}")
        assert list(engine._facts) == ["r2", "r3"] and engine.request_facts("r3")["preemptions"] == 0
        step, failing = engine.runner.step, [True]

        def broken(*args, **kwargs):
            if failing[0]:
                raise RuntimeError("the device went away")
            return step(*args, **kwargs)

        engine.runner.step = broken
        with pytest.raises(RuntimeError, match="went away"):
            await engine.generate([1, 2, 3], GenerationConfig(max_new_tokens=2))
        failing[0] = False
        again = await asyncio.wait_for(engine.generate([1, 2, 3], GenerationConfig(max_new_tokens=3)), timeout=60)
        assert engine.cache.used_pages == 0
        await engine.close()
        assert closed == [True]
        return again

    assert asyncio.run(run()) == plain.generate(weights, config, [1, 2, 3], 3)


@pytest.mark.parametrize("case", range(12))
def test_random_workloads_end_as_the_plain_decoder_says(model_folders, case):
    """Whole runs drawn at random (tests/random_runs.py) on the torch stand-in: every request ends with exactly
    the tokens the plain decoder gives it alone."""
    from tests.random_runs import run_random_workload

    _RANDOM_RUNS[case] = run_random_workload(1000 + case, model_folders, lambda name, blocks, batch: make_runner(model_folders, name, num_blocks=blocks, max_sequences=batch))


_RANDOM_RUNS: dict[int, int] = {}


def test_some_random_workloads_ran_out_of_pages():
    """(after the runs above) the draw is such that several of them had requests give way and replay"""
    if len(_RANDOM_RUNS) < 12:
        pytest.skip("the random runs did not all run in this process")
    assert sum(1 for evictions in _RANDOM_RUNS.values() if evictions > 0) >= 3, _RANDOM_RUNS


def test_the_sampler_says_whether_a_row_has_top_p():
    """The kernels may leave the top-p stages out when told that no row needs them: the sampler says so
    only if no row with a temperature has top_p < 1 (a greedy row's top_p does not count)."""
    from llmserve_amd.sampling.sampler import GenerationConfig, Sampler

    class Recording(TorchKernels):
        def sample(self, logits, temperatures, top_ps, uniforms, with_top_p=True):
            self.said = with_top_p
            return super().sample(logits, temperatures, top_ps, uniforms, with_top_p)

    kernels = Recording(torch.float32)
    sampler = Sampler(kernels)
    logits = torch.randn(3, 50)
    cases = [
        ([GenerationConfig(4, 0.7, 1.0), GenerationConfig(4, 0.0, 0.5), GenerationConfig(4, 1.2, 1.0)], False),
        ([GenerationConfig(4, 0.7, 1.0), GenerationConfig(4, 0.0, 1.0), GenerationConfig(4, 1.2, 0.9)], True),
    ]
    for configs, expected in cases:
        tokens = sampler.sample(logits, configs, [0, 1, 2])
        assert kernels.said is expected
        want = [plain.sample(logits[row], c.temperature, c.top_p, plain.uniform_for(c.seed, row)) for row, c in enumerate(configs)]
        assert tokens == want


def test_the_rows_of_a_decode_graph_by_the_number_of_requests():
    """A step of single tokens replays the graph of its padded shape: a power of two up to 128 requests,
    a multiple of 64 beyond, never fewer rows than requests and never more than twice as many."""
    rows = [ModelRunner._request_bucket(requests) for requests in range(1, 1025)]
    assert rows[:5] == [1, 2, 4, 4, 8] and rows[127] == 128 and rows[128] == 192 and rows[192] == 256
    assert all(later >= earlier for earlier, later in zip(rows, rows[1:]))
    for requests, padded in enumerate(rows, start=1):
        assert requests <= padded < 2 * requests or requests == 1
        assert padded & (padded - 1) == 0 if requests <= 128 else padded % 64 == 0
