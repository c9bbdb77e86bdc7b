"""Whole runs of the engine drawn at random, for the CPU stand-in and for the GPU."""

from __future__ import annotations

import random

from llmserve_amd import GenerationConfig, SchedulerConfig
from llmserve_amd.engine import EngineCore, Request
from tests.plain import qwen2_plain as plain
from tests.tiny import CONFIGS, random_tokens


def run_random_workload(seed, model_folders, make_runner, names=("A", "B"), exact=True):
    """One run: model (A, or B with its windowed layers), pool size, batch size, token budget, portion size,
    policy, who gives way, requests of random lengths with greedy or seeded sampling and stop tokens, some
    arriving while others run.  `make_runner(name, num_blocks, max_sequences)` builds the runner.  After every
    step the cache's books must balance; at the end every request has exactly the tokens the plain decoder gives
    it alone, however often it gave way and replayed (`exact`; else, for a precision in which a near-tie may turn,
    tokens that the plain decoder's rule can give for the run's own prefix), nothing was streamed twice, and every
    page is free again.  Returns how many times requests gave way."""
    from tests.tiny import unjustified_tokens

    rng = random.Random(seed)
    name = rng.choice(list(names))
    config, weights = plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])
    page = CONFIGS[name][1]
    count = rng.randint(3, 7)
    specs = []
    for index in range(count):
        prompt = random_tokens(rng.randint(1, 45), config.vocab_size, seed=rng.randrange(10_000))
        sampled = rng.random() < 0.5
        settings = GenerationConfig(
            max_new_tokens=rng.randint(1, 12), temperature=0.9 if sampled else 0.0,
            top_p=rng.choice([1.0, 0.8]) if sampled else 1.0, seed=rng.randrange(1000),
        )
        alone = plain.generate(weights, config, prompt, settings.max_new_tokens, settings.temperature, settings.top_p, settings.seed)
        if rng.random() < 0.3 and len(alone) > 2:  # a stop token that does come: the request ends there, stop token included
            stop = alone[rng.randrange(1, len(alone))]
            settings = GenerationConfig(settings.max_new_tokens, settings.temperature, settings.top_p, settings.seed, (stop,))
            alone = alone[: alone.index(stop) + 1]
        specs.append((f"r{index}", prompt, settings, alone, rng.randint(0, 3), rng.randint(0, 12)))
    longest = max(len(prompt) + settings.max_new_tokens for _, prompt, settings, _, _, _ in specs)
    # at least the pages of the longest request, so that everyone can finish; often too few for all at once
    num_blocks = -(-longest // page) + rng.randint(0, 6)
    batch = rng.randint(1, 4)
    budget = max(batch, rng.choice([4, 8, 16, 64]))
    runner = make_runner(name, num_blocks, batch)
    limits = SchedulerConfig(batch, budget, rng.choice(["fcfs", "sjf", "priority"]), rng.choice(["largest", "latest"]))
    core = EngineCore(runner, limits, scheduler_mode=rng.choice(["continuous", "continuous", "static"]),
                      prefill_chunk_size=rng.choice([1, 3, 16, 64]), collect_iteration_metrics=True)
    streamed = {request_id: [] for request_id, *_ in specs}
    requests = {}
    pending = sorted(specs, key=lambda spec: spec[5])  # by the step at which they arrive
    step = 0
    while pending or core.has_work:
        while pending and pending[0][5] <= step:
            request_id, prompt, settings, _, priority, _ = pending.pop(0)
            requests[request_id] = Request(request_id, list(prompt), settings, priority=priority)
            core.submit(requests[request_id])
        for event in core.step():
            streamed[event.request.request_id].append(event.token)
        runner.cache.check_invariants()
        step += 1
        assert step < 2000, "the run does not end"
    said = f"seed {seed}, model {name}"
    for request_id, prompt, settings, alone, _, _ in specs:
        assert requests[request_id].error is None, requests[request_id].error
        assert streamed[request_id] == requests[request_id].output, (said, request_id)
        if exact:
            assert requests[request_id].output == alone, (said, request_id)
        else:
            output = requests[request_id].output
            assert not unjustified_tokens(plain, weights, config, prompt, output, settings), (said, request_id)
            stopped = [index for index, token in enumerate(output) if token in settings.stop_token_ids]
            assert stopped == [len(output) - 1] if stopped else len(output) == settings.max_new_tokens, (said, request_id)
    assert runner.cache.used_pages == 0
    if hasattr(runner, "close"):
        runner.close()
    return sum(r.evictions for r in requests.values())
