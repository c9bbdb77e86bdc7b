"""A toy mixer with state of its own, and a toy architecture around it, are registered,
built and stepped without a change to the framework's files (here with the torch stand-in
for the kernels; tests/test_gpu_parts.py does the same on the GPU)."""

from __future__ import annotations

import pytest
import torch

from llmserve_amd import CacheConfig, ModelRunner, StepEntry
from llmserve_amd.parts import FixedState, PagedKeyValue
from llmserve_amd.weights import load_model_folder
from tests import toy
from tests.tiny import random_tokens
from tests.torch_kernels import TorchKernels


@pytest.fixture()
def toy_folder(tmp_path):
    toy.register_toy()
    yield toy.write_toy_folder(tmp_path / "toy")
    toy.unregister_toy()


def test_toy_architecture_steps_like_its_plain_forward(toy_folder):
    loaded = load_model_folder(toy_folder, "float32")
    assert loaded.architecture.name == "ToyStateForCausalLM"
    runner = ModelRunner(loaded, TorchKernels(torch.float32), CacheConfig(block_size=4, num_blocks=40, max_sequences=3))
    cache = runner.cache
    # two state cells (layer 0 runs twice), two paged groups (rotated and unrotated attention need the same pages:
    # one group), the last run owns nothing and reads run 1's pages
    assert [type(cell.need) for cell in runner.cells] == [FixedState, PagedKeyValue, PagedKeyValue, FixedState, PagedKeyValue, PagedKeyValue]
    assert len(cache.states) == 2 and len(cache.groups) == 1 and [run for run, _ in cache.groups[0].cells] == [1, 2, 5]
    # the routed feed-forward and the decaying mixer look at values on the host: no step of this model is replayed from a graph
    assert not runner.model.replayable and not runner.use_graphs
    assert "layers.0.mlp.router.weight" in loaded.tensors and "layers.2.mixer.position.table" in loaded.tensors
    assert runner.cells[4].keys.data_ptr() == runner.cells[1].keys.data_ptr() and not runner.cells[4].writable

    prompts = {name: random_tokens(n, toy.TOY.vocab_size, seed=n) for name, n in (("a", 37), ("b", 9), ("c", 22))}
    expected = {name: toy.plain_toy_forward(toy_folder, tokens) for name, tokens in prompts.items()}
    got = {name: [] for name in prompts}
    fed = {name: 0 for name in prompts}
    sizes = {"a": [5, 1, 1, 9, 2, 19], "b": [2, 7], "c": [1, 1, 1, 1, 18]}
    for turn in range(6):
        entries = []
        for name, tokens in prompts.items():
            if turn < len(sizes[name]):
                count = sizes[name][turn]
                entries.append(StepEntry(name, tokens[fed[name] : fed[name] + count], range(count)))
                fed[name] += count
        logits = runner.step(entries, create_missing=True)
        at = 0
        for entry in entries:
            got[entry.request_id].append(logits[at : at + len(entry.tokens)])
            at += len(entry.tokens)
    for name in prompts:
        torch.testing.assert_close(torch.cat(got[name]).double(), expected[name], atol=1e-5, rtol=1e-5)
    # a freed slot's state is zeroed for the next request
    runner.end_request("b")
    again = runner.step([StepEntry("b2", prompts["b"], range(9))], create_missing=True)
    torch.testing.assert_close(again.double(), expected["b"], atol=1e-5, rtol=1e-5)
    cache.check_invariants()


def test_an_architecture_whose_state_runs_on_the_device_alone(toy_folder, tmp_path):
    """The second toy architecture: a mixer with a state slot per request that nothing on the host looks at, and
    attention whose scores carry a distance bias and a soft cap.  It is replayable (on the GPU its steps are
    captured; tests/test_gpu_parts.py), and steps like its plain forward whatever the cut."""
    folder = toy.write_toy_folder(tmp_path / "sum", config=toy.SUM)
    loaded = load_model_folder(folder, "float32")
    assert loaded.architecture.name == "ToySumForCausalLM"
    runner = ModelRunner(loaded, TorchKernels(torch.float32), CacheConfig(block_size=4, num_blocks=40, max_sequences=3))
    assert runner.model.replayable and len(runner.cache.states) == 2 and runner.cache.states[0].shape[0] == 4  # a spare slot
    prompts = {name: random_tokens(n, toy.SUM.vocab_size, seed=n) for name, n in (("a", 30), ("b", 11))}
    expected = {name: toy.plain_toy_forward(folder, tokens) for name, tokens in prompts.items()}
    got = {name: [] for name in prompts}
    fed = {name: 0 for name in prompts}
    sizes = {"a": [5, 1, 1, 9, 14], "b": [2, 1, 8]}
    for turn in range(5):
        entries = []
        for name, tokens in prompts.items():
            if turn < len(sizes[name]):
                count = sizes[name][turn]
                entries.append(StepEntry(name, tokens[fed[name] : fed[name] + count], range(count)))
                fed[name] += count
        logits = runner.step(entries, create_missing=True)
        at = 0
        for entry in entries:
            got[entry.request_id].append(logits[at : at + len(entry.tokens)])
            at += len(entry.tokens)
    for name in prompts:
        torch.testing.assert_close(torch.cat(got[name]).double(), expected[name], atol=1e-5, rtol=1e-5)
    runner.end_request("b")
    again = runner.step([StepEntry("b2", prompts["b"], range(11))], create_missing=True)
    torch.testing.assert_close(again.double(), expected["b"], atol=1e-5, rtol=1e-5)


def test_unregistered_parts_are_refused(tmp_path):
    toy.register_toy()
    folder = toy.write_toy_folder(tmp_path / "toy")
    toy.unregister_toy()
    with pytest.raises(Exception, match="ToyStateForCausalLM"):
        load_model_folder(folder, "float32")


def step_in_portions(runner, prompts, sizes):
    """Feeds the prompts through the step function, request `name` bringing sizes[name][turn] tokens in turn `turn`
    beside the others'; returns every position's logits per request."""
    got = {name: [] for name in prompts}
    fed = {name: 0 for name in prompts}
    for turn in range(max(len(cuts) for cuts in sizes.values())):
        entries = []
        for name, tokens in prompts.items():
            if turn < len(sizes[name]):
                count = sizes[name][turn]
                entries.append(StepEntry(name, tokens[fed[name] : fed[name] + count], range(count)))
                fed[name] += count
        logits = runner.step(entries, create_missing=True)
        at = 0
        for entry in entries:
            got[entry.request_id].append(logits[at : at + len(entry.tokens)].clone())
            at += len(entry.tokens)
        runner.cache.check_invariants()
    return {name: torch.cat(rows) for name, rows in got.items()}


def test_cache_needs_of_a_kind_of_their_own_and_two_needs_for_one_run(toy_folder, tmp_path):
    """The third toy architecture brings a kind of cache need that the cache manager has never heard of (per token
    a narrow key row and a wider value row, in pages of its own layout), a block whose two mixers need pages *and*
    a state slot for the same run, and a gate activation other than SiLU.  Registered from the test, built and
    stepped in changing portions, three requests side by side in a pool they fill; every logit is the plain
    forward's, the pages hold the plain forward's rows, and everything is given back at the end."""
    from llmserve_amd.cache import CacheCell
    from llmserve_amd.parts import PagedKeyValue

    folder = toy.write_toy_folder(tmp_path / "latent", config=toy.LATENT)
    loaded = load_model_folder(folder, "float32")
    assert loaded.architecture.name == "ToyLatentForCausalLM"
    runner = ModelRunner(loaded, TorchKernels(torch.float32), CacheConfig(block_size=4, num_blocks=20, max_sequences=3))
    cache = runner.cache
    # two groups of pages (the latent mixer's two runs share one, attention has the other) and one state
    assert [type(group.need) for group in cache.groups] == [toy.PagedRows, PagedKeyValue] and len(cache.states) == 1
    assert cache.groups[0].cells == [(0, None), (2, None)] and cache.groups[1].cells == [(1, "attention")]
    assert cache.groups[0].storage["key_rows"].shape == (2, 20, 4, 12) and cache.groups[0].storage["value_rows"].shape == (2, 20, 4, 28)
    assert isinstance(runner.cells[0], CacheCell) and set(runner.cells[1]) == {"attention", "decay"}
    assert runner.cells[1]["decay"].state.shape == (4, toy.LATENT.state_size)
    # a token costs its rows in both latent cells and its keys and values
    assert cache.bytes_per_token == 4 * (2 * (12 + 28) + 2 * toy.LATENT.num_heads * toy.LATENT.head_dim)

    prompts = {name: random_tokens(n, toy.LATENT.vocab_size, seed=n) for name, n in (("a", 37), ("b", 9), ("c", 22))}
    expected = {name: toy.plain_toy_forward(folder, tokens, with_cached_rows=True) for name, tokens in prompts.items()}
    got = step_in_portions(runner, prompts, {"a": [5, 1, 1, 9, 2, 19], "b": [2, 7], "c": [1, 1, 1, 1, 18]})
    for name in prompts:
        torch.testing.assert_close(got[name].double(), expected[name][0], atol=1e-5, rtol=1e-5)
        first, rows = cache.gather_fields(name, 0)
        assert first == 0
        torch.testing.assert_close(rows["key_rows"].double(), expected[name][1][0], atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(rows["value_rows"].double(), expected[name][1][1], atol=1e-5, rtol=1e-5)
    assert cache.groups[0].pool.used_pages == cache.groups[1].pool.used_pages == 10 + 3 + 6
    # a request that ends gives its pages and its slot back; the next one finds the state zeroed
    runner.end_request("b")
    again = runner.step([StepEntry("b2", prompts["b"], range(9))], create_missing=True)
    torch.testing.assert_close(again.double(), expected["b"][0], atol=1e-5, rtol=1e-5)
    for name in ("a", "c", "b2"):
        runner.end_request(name)
    cache.check_invariants()
    assert cache.used_pages == 0


def test_a_gate_activation_without_a_kernel_is_refused_by_name():
    from llmserve_amd.parts import FEED_FORWARDS, GatedMLPSpec

    spec = GatedMLPSpec(8, 16, activation="swish7")
    tensors = {name: torch.zeros(shape.shape) for name, shape in FEED_FORWARDS.tensors(spec).items()}
    with pytest.raises(ValueError, match="swish7"):
        FEED_FORWARDS.build(spec, tensors, TorchKernels(torch.float32))
