"""The command line's options, the synthetic workload and the latency metrics (no GPU)."""

from __future__ import annotations

import asyncio

import pytest

from llmserve_amd.benchmark import (
    BenchmarkHarness, BenchmarkReport, LengthDistribution, LoadProfile, RequestMetrics, generate_workload, percentile,
)
from llmserve_amd.cli import ROOT, build_parser
from llmserve_amd.engine import RequestState, choose_victim
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
    # the reference's switches between its back ends (cli.py:263-271) parse, so its command lines carry over
    carried = build_parser().parse_args(["benchmark", "--rebuild-device-metadata", "--paged-attention-backend", "triton",
                                         "--linear-backend", "fp16"])
    assert carried.rebuild_device_metadata and carried.paged_attention_backend == "triton" and carried.linear_backend == "fp16"
    quantized = build_parser().parse_args(["benchmark", "--linear-backend", "triton-int8"])
    with pytest.raises(SystemExit, match="int8"):  # refused before anything is loaded
        import asyncio

        from llmserve_amd.cli import _benchmark

        asyncio.run(_benchmark(quantized))
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
    assert first[0].arrival_offset_s == 0.0 and all(a.arrival_offset_s <= b.arrival_offset_s for a, b in zip(first, first[1:]))
    assert all(8 <= len(spec.prompt_token_ids) <= 1024 and 4 <= spec.max_new_tokens <= 256 for spec in first)
    assert all(4 <= token < 32000 for spec in first for token in spec.prompt_token_ids)  # reserved ids 0-3 avoided
    lengths = sorted(len(spec.prompt_token_ids) for spec in first)
    assert 60 <= lengths[50] <= 260  # the median is near 128, the tail is long
    assert lengths[-1] > 3 * lengths[50]


def test_latency_metrics():
    """reference benchmark/metrics.py:11-58,71-94"""
    assert percentile([], 0.5) == 0.0 and percentile([1.0, 3.0], 0.5) == 2.0 and percentile([1, 2, 3, 4], 0.95) == pytest.approx(3.85)
    record = RequestMetrics("r", arrival_s=10.0, prompt_tokens=5, requested_output_tokens=4, first_token_s=10.5,
                            finished_s=12.0, output_tokens=4)
    assert (record.ttft_ms, record.tpot_ms, record.e2e_ms) == (500.0, 500.0, 2000.0)
    failed = RequestMetrics("f", 10.0, 5, 4, error="CacheFullError: x")
    report = BenchmarkReport("continuous-fcfs", 10.0, 12.0, [record, failed], cache={"blocks_used": 0.0})
    summary = report.summary
    assert summary["successful_requests"] == 1 and summary["throughput_tokens_per_s"] == 2.0
    assert summary["ttft_ms_p50"] == 500.0 and summary["cache_blocks_used"] == 0.0


def test_harness_sends_requests_at_their_arrival_times(tmp_path):
    profile = LoadProfile(requests=5, arrival_rate=500.0, prompt=LengthDistribution(6, 0.2, 2, 12),
                          output=LengthDistribution(3, 0.2, 2, 4), seed=3, vocabulary_size=100)

    async def generate(spec, callback):
        for token in range(spec.max_new_tokens):
            await asyncio.sleep(0)
            callback(token)
        return list(range(spec.max_new_tokens))

    report = asyncio.run(BenchmarkHarness(profile).run("stub", generate))
    assert [r.output_tokens for r in report.requests] == [spec.max_new_tokens for spec in generate_workload(profile)]
    report.write_json(tmp_path / "r.json")
    report.write_csv(tmp_path / "r.csv")
    assert (tmp_path / "r.csv").read_text().count("\n") == 6


def test_who_gives_way():
    requests = [RequestState(name, [1], 4, arrival_order=order, processed_tokens=done)
                for name, order, done in (("old", 0, 90), ("big", 1, 70), ("young", 2, 10))]
    planned = [(request, 1) for request in requests]
    assert choose_victim(planned, "largest").request_id == "big"  # most processed, but never the oldest
    assert choose_victim(planned, "latest").request_id == "young"
    assert choose_victim(planned[:2], "largest").request_id == "big"
    with pytest.raises(ValueError):
        choose_victim(planned[:1])
    with pytest.raises(ValueError):
        choose_victim(planned, "random")


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
    assert [len(spec.prompt_token_ids) <= 40 for spec in specs] == [True] * 5 + [False] * 3
    assert [len(spec.prompt_token_ids) for spec in specs[5:]] == [600] * 3
    assert all(90 <= spec.max_new_tokens <= 110 for spec in specs[:5]) and all(spec.max_new_tokens == 8 for spec in specs[5:])
    assert [spec.arrival_offset_s for spec in specs] == sorted(spec.arrival_offset_s for spec in specs)
    assert specs == generate_workload(profile)
    fitted = generate_workload(profile.fitted(500))
    assert [len(spec.prompt_token_ids) for spec in fitted[5:]] == [492] * 3
    with pytest.raises(ValueError):
        LoadProfile(requests=7, groups=(short, long))
    mix = LoadProfile.from_yaml(ROOT / "configs" / "workload-long-context-mix.yaml")
    assert mix.requests == 64 and [group.requests for group in mix.groups] == [48, 16]
