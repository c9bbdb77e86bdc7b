"""The command line's options, the synthetic workload and the latency metrics (no GPU)."""

from __future__ import annotations

import asyncio

import pytest

from llmserve_amd.benchmark import (
    BenchmarkHarness, BenchmarkReport, LengthDistribution, LoadProfile, RequestMetrics, generate_workload, percentile,
)
from llmserve_amd.cli import ROOT, build_parser
from llmserve_amd import GenerationConfig, SchedulerConfig
from llmserve_amd.engine import Request, Scheduler, Share
from llmserve_amd.engine.tokenizer import ByteTokenizer


def test_benchmark_options_are_the_references():
    """reference cli.py:248-273: the same names, choices and defaults where the engine has them"""
    args = build_parser().parse_args(["benchmark"])
    assert (args.config, args.policy, args.batch_size, args.block_size, args.num_blocks) == ("continuous", "fcfs", 16, 16, 1024)
    assert (args.prefill_chunk_size, args.max_tokens_per_step, args.seed, args.device) == (16, 2048, 7, "auto")
    assert args.output == "artifacts/benchmark.json" and args.requests is None and args.arrival_rate is None
    for config in ("naive", "paged", "static", "continuous"):
        assert build_parser().parse_args(["benchmark", "--config", config]).config == config
    with pytest.raises(SystemExit):
        build_parser().parse_args(["benchmark", "--policy", "random"])
    with pytest.raises(SystemExit):
        build_parser().parse_args(["serve"])  # servers are outside this engine
    # the reference's switches between back ends it alone has (cli.py:263-271) are not options here
    for switch in (["--rebuild-device-metadata"], ["--paged-attention-backend", "triton"], ["--linear-backend", "fp16"]):
        with pytest.raises(SystemExit):
            build_parser().parse_args(["benchmark", *switch])
    generate = build_parser().parse_args(["generate", "--prompt-tokens", "1,2,3", "--temperature", "0.8", "--top-p", "0.9"])
    assert (generate.max_tokens, generate.temperature, generate.top_p) == (32, 0.8, 0.9)
    replay = build_parser().parse_args(["replay", "--model", "m", "--out", "o", "--max-tokens", "256"])
    assert replay.dtype == "bfloat16" and replay.block_size == 16


def test_workload_is_fixed_by_its_seed():
    """reference benchmark/workload.py:60-79 and configs/benchmark-sharegpt.yaml"""
    profile = LoadProfile.from_yaml(ROOT / "configs" / "benchmark-sharegpt.yaml")
    assert (profile.requests, profile.arrival_rate, profile.seed) == (100, 2.0, 7)
    assert profile.prompt == LengthDistribution(128, 0.9, 8, 1024) and profile.output == LengthDistribution(64, 0.7, 4, 256)
    first, again = generate_workload(profile), generate_workload(profile)
    assert first == again and len(first) == 100
    assert first[0].at_s == 0.0 and all(a.at_s <= b.at_s for a, b in zip(first, first[1:]))
    assert all(8 <= len(spec.prompt) <= 1024 and 4 <= spec.max_new_tokens <= 256 for spec in first)
    assert all(4 <= token < 32000 for spec in first for token in spec.prompt)  # reserved ids 0-3 avoided
    lengths = sorted(len(spec.prompt) for spec in first)
    assert 60 <= lengths[50] <= 260  # the median is near 128, the tail is long
    assert lengths[-1] > 3 * lengths[50]


def test_latency_metrics():
    """reference benchmark/metrics.py:11-58,71-94"""
    assert percentile([], 0.5) == 0.0 and percentile([1.0, 3.0], 0.5) == 2.0 and percentile([1, 2, 3, 4], 0.95) == pytest.approx(3.85)
    record = RequestMetrics("r", arrival_s=10.0, prompt_tokens=5, requested_output_tokens=4, first_token_s=10.5,
                            finished_s=12.0, output_tokens=4, preemptions=2, recomputed_tokens=30)
    assert (record.ttft_ms, record.tpot_ms, record.e2e_ms) == (500.0, 500.0, 2000.0)
    failed = RequestMetrics("f", 10.0, 5, 4, error="CacheFullError: x")
    assert failed.ttft_ms is None and failed.tpot_ms is None and RequestMetrics("one", 1.0, 2, 1, None, 2.0, 2.0, 1).tpot_ms is None
    report = BenchmarkReport("continuous-fcfs", 10.0, 12.0, [record, failed], cache={"blocks_used": 0.0})
    summary = report.summary
    assert summary["successful_requests"] == 1 and summary["throughput_tokens_per_s"] == 2.0
    assert summary["ttft_ms_p50"] == 500.0 and summary["cache_blocks_used"] == 0.0
    assert (summary["preemptions"], summary["recomputed_tokens"]) == (2, 30)
    assert {"admitted_s", "preemptions", "recomputed_tokens", "ttft_ms"} <= set(record.to_dict())  # reference metrics.py:29,33-34


def test_harness_sends_requests_at_their_arrival_times(tmp_path):
    profile = LoadProfile(requests=5, arrival_rate=500.0, prompt=LengthDistribution(6, 0.2, 2, 12),
                          output=LengthDistribution(3, 0.2, 2, 4), seed=3, vocabulary_size=100)

    async def generate(spec, callback):
        for token in range(spec.max_new_tokens):
            await asyncio.sleep(0)
            callback(token)
        return list(range(spec.max_new_tokens))

    facts = lambda request_id: {"admitted_s": 1.5, "preemptions": 1, "recomputed_tokens": 7}
    report = asyncio.run(BenchmarkHarness(profile).run("stub", generate, facts))
    assert [(r.admitted_s, r.preemptions, r.recomputed_tokens) for r in report.requests] == [(1.5, 1, 7)] * 5
    assert [r.output_tokens for r in report.requests] == [spec.max_new_tokens for spec in generate_workload(profile)]
    report.write_json(tmp_path / "r.json")
    report.write_csv(tmp_path / "r.csv")
    assert (tmp_path / "r.csv").read_text().count("\n") == 6


def test_who_gives_way():
    requests = [Request(name, [1], GenerationConfig(max_new_tokens=4), ticket=order, cached=done)
                for name, order, done in (("old", 0, 90), ("big", 1, 70), ("young", 2, 10))]
    shares = [Share(request, 1) for request in requests]
    largest, latest = Scheduler(SchedulerConfig(preemption="largest")), Scheduler(SchedulerConfig(preemption="latest"))
    assert largest.victim(shares).request_id == "big"  # most tokens cached, but never the oldest
    assert latest.victim(shares).request_id == "young"
    assert largest.victim(shares[:2]).request_id == "big"
    with pytest.raises(ValueError):
        largest.victim(shares[:1])
    with pytest.raises(ValueError):
        Scheduler(SchedulerConfig(preemption="random"))


def test_byte_tokenizer_round_trip():
    """reference tokenizer.py:15-29"""
    tokenizer = ByteTokenizer()
    ids = tokenizer.encode("héllo")
    assert min(ids) >= 4 and max(ids) < 260 and tokenizer.vocab_size == 260 and tokenizer.eos_token_id == 2
    assert tokenizer.decode(ids + [0, 1, 2]) == "héllo"


def test_bench_measures_one_gpu_only():
    import subprocess
    import sys

    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 2 and len(done.stdout.strip().splitlines()) == 1 and "one GPU" in done.stdout


def test_workload_groups_arrive_in_order_and_fit_the_context():
    """A profile made of groups: the groups' requests come one group after the other on the one
    arrival process, lengths from each group's own distributions; `fitted` clips prompts so that
    prompt plus output stay within the longest sequence."""
    from llmserve_amd.benchmark import LengthDistribution, LoadProfile, RequestGroup, generate_workload

    short = RequestGroup(5, LengthDistribution(20, 0.5, 4, 40), LengthDistribution(100, 0.1, 90, 110))
    long = RequestGroup(3, LengthDistribution(600, 0.0, 600, 600), LengthDistribution(8, 0.0, 8, 8))
    profile = LoadProfile(requests=8, arrival_rate=10.0, groups=(short, long), vocabulary_size=50)
    specs = generate_workload(profile)
    assert [len(spec.prompt) <= 40 for spec in specs] == [True] * 5 + [False] * 3
    assert [len(spec.prompt) for spec in specs[5:]] == [600] * 3
    assert all(90 <= spec.max_new_tokens <= 110 for spec in specs[:5]) and all(spec.max_new_tokens == 8 for spec in specs[5:])
    assert [spec.at_s for spec in specs] == sorted(spec.at_s for spec in specs)
    assert specs == generate_workload(profile)
    fitted = generate_workload(profile.fitted(500))
    assert [len(spec.prompt) for spec in fitted[5:]] == [492] * 3
    with pytest.raises(ValueError):
        LoadProfile(requests=7, groups=(short, long))
    mix = LoadProfile.from_yaml(ROOT / "configs" / "workload-long-context-mix.yaml")
    assert mix.requests == 64 and [group.requests for group in mix.groups] == [48, 16]


def test_the_end_of_sequence_ids_a_model_folder_names(tmp_path):
    """generation_config.json first (a number or a list), then config.json, else none: what `llmserve generate
    --model` stops at unless told otherwise (reference service/app.py:88 stops at the tokenizer's id)."""
    import json

    from llmserve_amd.engine.tokenizer import folder_eos_token_ids

    assert folder_eos_token_ids(tmp_path) == ()
    (tmp_path / "config.json").write_text(json.dumps({"eos_token_id": 7}))
    assert folder_eos_token_ids(tmp_path) == (7,)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [11, 12]}))
    assert folder_eos_token_ids(tmp_path) == (11, 12)
    (tmp_path / "generation_config.json").write_text(json.dumps({"temperature": 0.7}))
    assert folder_eos_token_ids(tmp_path) == (7,)


def test_replay_and_generate_options():
    from llmserve_amd.cli import build_parser

    args = build_parser().parse_args(["replay", "--model", "m", "--out", "o", "--max-tokens", "64", "--max-requests", "3"])
    assert args.max_requests == 3
    args = build_parser().parse_args(["generate", "--ignore-eos"])
    assert args.ignore_eos and args.stop_token_id is None
