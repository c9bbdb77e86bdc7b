"""Pins the plain implementation by what fixes it beside the reference's text:
special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, a
swapped gate) fails it."""

from __future__ import annotations

import math

import pytest
import torch
import torch.nn.functional as F

from tests.plain import qwen2_plain as plain

torch.manual_seed(0)
DOUBLE = torch.float64


def test_rms_norm_is_the_library_routine():
    x = torch.randn(5, 48, dtype=DOUBLE)
    w = 1 + 0.1 * torch.randn(48, dtype=DOUBLE)
    for eps in (1e-6, 1e-2):
        torch.testing.assert_close(plain.rms_norm(x, w, eps), F.rms_norm(x, (48,), w, eps))


def test_rms_norm_scale_and_eps():
    x = torch.randn(3, 64, dtype=DOUBLE)
    ones = torch.ones(64, dtype=DOUBLE)
    y = plain.rms_norm(x, ones, 1e-12)
    torch.testing.assert_close(y.norm(dim=-1), torch.full((3,), 8.0, dtype=DOUBLE))  # sqrt(H)
    torch.testing.assert_close(plain.rms_norm(7 * x, ones, 1e-12), y)  # no mean subtraction, scale-free
    tiny = 1e-4 * x
    assert (plain.rms_norm(tiny, ones, 1e-6).norm(dim=-1) < 7.0).all()  # eps matters near zero
    shifted = x + 3.0
    assert not torch.allclose(plain.rms_norm(shifted, ones, 1e-12), plain.rms_norm(x, ones, 1e-12))


def _heads(length=6, heads=3, dim=8):
    return torch.randn(length, heads, dim, dtype=DOUBLE)


def test_rope_adjacent_is_complex_multiplication():
    x = _heads()
    positions = torch.tensor([0, 1, 2, 5, 9, 30])
    angles = plain.rope_angles(8, 10000.0, positions)
    as_complex = torch.view_as_complex(x.reshape(6, 3, 4, 2).contiguous())
    rotated = as_complex * torch.polar(torch.ones_like(angles, dtype=DOUBLE), angles.double())[:, None, :]
    expected = torch.view_as_real(rotated).reshape(6, 3, 8)
    torch.testing.assert_close(plain.rope_adjacent(x, angles), expected)


def test_rope_angles_follow_theta():
    angles = plain.rope_angles(8, 100.0, torch.tensor([0, 3]))
    torch.testing.assert_close(angles[0], torch.zeros(4))
    expected = 3.0 * torch.tensor([1.0, 100 ** -0.25, 100 ** -0.5, 100 ** -0.75])
    torch.testing.assert_close(angles[1], expected)


@pytest.mark.parametrize("rotate", [plain.rope_adjacent, plain.rope_half])
def test_rope_invariants(rotate):
    q, k = _heads(), _heads()
    zero = plain.rope_angles(8, 10000.0, torch.zeros(6, dtype=torch.long))
    torch.testing.assert_close(rotate(q, zero), q)  # position 0 is the identity
    positions = torch.arange(6)
    a = plain.rope_angles(8, 10000.0, positions)
    b = plain.rope_angles(8, 10000.0, positions + 17)
    torch.testing.assert_close(rotate(q, a).norm(dim=-1), q.norm(dim=-1))  # a rotation
    # scores depend on distances only: shift all positions
    near = torch.einsum("shd,thd->hst", rotate(q, a), rotate(k, a))
    far = torch.einsum("shd,thd->hst", rotate(q, b), rotate(k, b))
    torch.testing.assert_close(near, far, atol=1e-4, rtol=1e-4)  # angles are float32
    # and on their sign: swapping the roles of query and key positions changes them
    swapped = torch.einsum("shd,thd->hst", rotate(q, a), rotate(k, a.flip(0)))
    assert not torch.allclose(near, swapped, atol=1e-3)


def test_rope_half_is_adjacent_on_permuted_rows():
    x = _heads()
    angles = plain.rope_angles(8, 10000.0, torch.arange(6) + 2)
    permutation = torch.tensor([0, 2, 4, 6, 1, 3, 5, 7])
    torch.testing.assert_close(plain.rope_half(x[..., permutation], angles), plain.rope_adjacent(x, angles)[..., permutation])
    assert not torch.allclose(plain.rope_half(x, angles), plain.rope_adjacent(x, angles))


def test_attention_is_the_library_routine():
    q, k, v = _heads(7, 6, 8), _heads(7, 2, 8), _heads(7, 2, 8)
    scale = 1 / math.sqrt(8)
    ours = plain.causal_attention(q, k, v, scale)
    expanded_k = k.repeat_interleave(3, dim=1).transpose(0, 1)
    expanded_v = v.repeat_interleave(3, dim=1).transpose(0, 1)
    library = F.scaled_dot_product_attention(q.transpose(0, 1), expanded_k, expanded_v, is_causal=True)
    torch.testing.assert_close(ours, library.transpose(0, 1))
    # a different grouping of heads (h % Hkv instead of h // G) gives something else
    wrong_k = k.repeat(1, 3, 1).transpose(0, 1)
    wrong_v = v.repeat(1, 3, 1).transpose(0, 1)
    wrong = F.scaled_dot_product_attention(q.transpose(0, 1), wrong_k, wrong_v, is_causal=True)
    assert not torch.allclose(ours, wrong.transpose(0, 1))


def test_attention_special_cases():
    q, k, v = _heads(5, 2, 4), _heads(5, 2, 4), _heads(5, 2, 4)
    out = plain.causal_attention(q, k, v, 0.5)
    torch.testing.assert_close(out[0], v[0])  # one key: the value itself
    flat = plain.causal_attention(q, torch.zeros_like(k), v, 0.5)
    torch.testing.assert_close(flat[3], v[:4].mean(dim=0))  # equal scores: the mean of the values
    # one head, no rotation, no mask on the last row: plain softmax attention
    last = torch.softmax(q[4, 0] @ k[:, 0].T * 0.5, dim=0) @ v[:, 0]
    torch.testing.assert_close(out[4, 0], last)
    # the scale matters
    assert not torch.allclose(plain.causal_attention(q, k, v, 1.0), out)


def test_attention_window_keeps_the_last_keys():
    q, k, v = _heads(9, 2, 4), _heads(9, 1, 4), _heads(9, 1, 4)
    windowed = plain.causal_attention(q, k, v, 0.5, window=3)
    full = plain.causal_attention(q, k, v, 0.5)
    torch.testing.assert_close(windowed[:3], full[:3])  # the window is not yet full
    tail = plain.causal_attention(q[4:7], k[4:7], v[4:7], 0.5)
    torch.testing.assert_close(windowed[6], tail[2])  # position 6 sees keys 4, 5, 6 only
    assert not torch.allclose(windowed[6], full[6])
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.5, window=9), full)


def test_swiglu_is_the_library_routine():
    x = torch.randn(4, 10, dtype=DOUBLE)
    gate, up, down = (torch.randn(*s, dtype=DOUBLE) for s in ((14, 10), (14, 10), (10, 14)))
    expected = F.linear(F.silu(F.linear(x, gate)) * F.linear(x, up), down)
    torch.testing.assert_close(plain.swiglu(x, gate, up, down), expected)
    assert not torch.allclose(plain.swiglu(x, up, gate, down), expected)  # gate and up are not symmetric
    torch.testing.assert_close(plain.swiglu(x, torch.zeros_like(gate), up, down), torch.zeros(4, 10, dtype=DOUBLE))


def _tiny(folder_name, model_folders):
    folder = model_folders[folder_name]
    return plain.PlainConfig.from_folder(folder), plain.read_weights(folder)


def test_zeroed_output_projections_leave_the_embedding(model_folders):
    config, weights = _tiny("B", model_folders)
    for name in list(weights):
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            weights[name] = torch.zeros_like(weights[name])
    tokens = [3, 1, 4, 1, 5]
    embedded = weights["embed_tokens.weight"][tokens]
    expected = plain.rms_norm(embedded, weights["norm.weight"], config.rms_norm_eps) @ weights["lm_head.weight"].T
    torch.testing.assert_close(plain.forward(weights, config, tokens), expected)


def test_model_is_causal_and_uses_distances_only(model_folders):
    config, weights = _tiny("A", model_folders)
    tokens = [7, 200, 13, 13, 91, 5, 64, 33]
    whole = plain.forward(weights, config, tokens)
    torch.testing.assert_close(plain.forward(weights, config, tokens[:5]), whole[:5])  # no look-ahead
    shifted = plain.forward(weights, config, tokens, first_position=40)
    torch.testing.assert_close(shifted, whole, atol=1e-5, rtol=1e-5)  # only distances count
    assert whole.shape == (8, config.vocab_size)


def test_tied_head_is_the_embedding(model_folders):
    config, weights = _tiny("A", model_folders)
    assert config.tie_word_embeddings and "lm_head.weight" not in weights
    config_b, weights_b = _tiny("B", model_folders)
    assert not config_b.tie_word_embeddings
    assert not torch.equal(weights_b["lm_head.weight"], weights_b["embed_tokens.weight"])


def test_biases_and_norm_weights_take_part(model_folders):
    config, weights = _tiny("B", model_folders)
    tokens = [5, 9, 300, 2]
    base = plain.forward(weights, config, tokens)
    for suffix in ("q_proj.bias", "v_proj.bias", "post_attention_layernorm.weight"):
        changed = dict(weights)
        name = f"layers.1.self_attn.{suffix}" if "proj" in suffix else f"layers.1.{suffix}"
        changed[name] = weights[name] + 0.5
        assert not torch.allclose(plain.forward(changed, config, tokens), base, atol=1e-6), name


def test_window_of_config_b_reaches_the_model(model_folders):
    config, weights = _tiny("B", model_folders)
    assert config.windows == (None, 24, 24)
    tokens = list(range(1, 41))
    full = plain.forward(weights, plain.PlainConfig(**{**config.__dict__, "windows": ()}), tokens)
    windowed = plain.forward(weights, config, tokens)
    torch.testing.assert_close(windowed[:24], full[:24])
    assert not torch.allclose(windowed[30:], full[30:], atol=1e-6)


def test_sampling_rules():
    logits = torch.tensor([0.1, 2.0, -1.0, 2.0, 0.5])
    assert plain.sample(logits, 0.0, 1.0, 0.3) == 1  # greedy: the first maximum
    p = torch.softmax(logits / 0.7, dim=-1).double()
    cdf = p.cumsum(0)
    for u in (0.0, 0.2, 0.5, 0.77, 0.999):
        assert plain.sample(logits, 0.7, 1.0, u) == int((cdf > u).nonzero()[0])
    # top-p keeps entries whose preceding mass (descending) is below top_p
    order = sorted(range(5), key=lambda i: (-float(p[i]), i))
    assert order[:2] == [1, 3]
    assert plain.sample(logits, 0.7, 0.3, 0.99) == 1  # only the first survives
    assert plain.sample(logits, 0.7, 0.5, 0.49) == 1 and plain.sample(logits, 0.7, 0.5, 0.51) == 3
    draws = {plain.sample(logits, 0.7, 1.0, plain.uniform_for(11, step)) for step in range(200)}
    assert draws == {0, 1, 2, 3, 4}
    values = [plain.uniform_for(3, step) for step in range(1000)]
    assert 0.0 <= min(values) and max(values) < 1.0 and 0.45 < sum(values) / 1000 < 0.55


def test_generate_stops_and_keeps_the_stop_token(model_folders):
    config, weights = _tiny("A", model_folders)
    free = plain.generate(weights, config, [1, 2, 3], 6)
    assert len(free) == 6
    stopped = plain.generate(weights, config, [1, 2, 3], 6, stop_token_ids=(free[2],))
    assert stopped == free[: free.index(free[2]) + 1]


@pytest.mark.parametrize("name", ["A-loud", "B-loud", "C-loud"])
def test_the_bfloat16_bounds_can_see_a_wrong_rotation_and_a_lost_bias(model_folders, name):
    """The GPU tests allow a bfloat16 run BF16_LARGEST of the logits' spread at the largest element and
    BF16_MEAN of it on average.  At the "loud" folders both plausible mistakes of the attention part exceed
    that, by the plain implementation's own account: pairing the rotation the other way, and dropping the key
    bias (which matters only through the rotation: an unrotated bias adds the same to every score of a query)."""
    import dataclasses

    from tests.tiny import BF16_LARGEST, BF16_MEAN, random_tokens

    config, weights = plain.PlainConfig.from_folder(model_folders[name]), plain.read_weights(model_folders[name])
    prompts = [random_tokens(n, config.vocab_size, seed=100 + n) for n in (17, 33, 70)]
    right = torch.cat([plain.forward(weights, config, prompt) for prompt in prompts])
    spread = float(right.std())

    def visible(other: torch.Tensor) -> bool:
        error = (other - right).abs()
        return float(error.max()) > 2 * BF16_LARGEST * spread and float(error.mean()) > 2 * BF16_MEAN * spread

    swapped = dataclasses.replace(config, rope_pairing="adjacent" if config.rope_pairing == "half" else "half")
    assert visible(torch.cat([plain.forward(weights, swapped, prompt) for prompt in prompts]))
    if config.attention_bias:
        without = {key: torch.zeros_like(value) if key.endswith("k_proj.bias") else value for key, value in weights.items()}
        assert visible(torch.cat([plain.forward(without, config, prompt) for prompt in prompts]))
    quiet = name.split("-")[0]  # the reference's own initialisation hides both: that is why the loud folders exist
    config, weights = plain.PlainConfig.from_folder(model_folders[quiet]), plain.read_weights(model_folders[quiet])
    if config.attention_bias:
        right = torch.cat([plain.forward(weights, config, prompt) for prompt in prompts])
        without = {key: torch.zeros_like(value) if key.endswith("k_proj.bias") else value for key, value in weights.items()}
        lost = torch.cat([plain.forward(without, config, prompt) for prompt in prompts])
        assert float((lost - right).abs().max()) < BF16_LARGEST * float(right.std())


def test_the_token_by_token_check_of_a_reduced_precision_run(model_folders):
    """`unjustified_tokens` is what the GPU tests hold bfloat16 generation against.  It must pass the plain
    decoder's own tokens even with no allowance at all (greedy, sampled, top-p, stop tokens), and it must see a
    run whose tokens were drawn with another seed, with the draws of another step, or that went on after a
    stop token, at the allowance the GPU tests use."""
    from llmserve_amd import GenerationConfig
    from tests.tiny import random_tokens, unjustified_tokens

    config, weights = _tiny("B-loud", model_folders)
    prompt = random_tokens(23, config.vocab_size, seed=3)
    for chosen in (GenerationConfig(10), GenerationConfig(10, 0.8, 1.0, seed=5), GenerationConfig(10, 0.9, 0.85, seed=6)):
        own = plain.generate(weights, config, prompt, 10, chosen.temperature, chosen.top_p, chosen.seed)
        assert not unjustified_tokens(plain, weights, config, prompt, own, chosen, largest=1e-9)
        assert not unjustified_tokens(plain, weights, config, prompt, own, chosen)
        if chosen.temperature > 0:  # tokens drawn with another seed are not this request's
            other = plain.generate(weights, config, prompt, 10, chosen.temperature, chosen.top_p, chosen.seed + 1)
            assert other != own and unjustified_tokens(plain, weights, config, prompt, other, chosen)
            shifted = GenerationConfig(10, chosen.temperature, chosen.top_p, seed=chosen.seed)
            late = own[1:]  # every token one draw too early
            assert unjustified_tokens(plain, weights, config, prompt, late + own[:1], shifted)
        else:
            wrong = list(own)
            wrong[4] = (own[4] + 1) % config.vocab_size
            assert [index for index, _, _ in unjustified_tokens(plain, weights, config, prompt, wrong, chosen)][0] == 4
    own = plain.generate(weights, config, prompt, 10)
    stopping = GenerationConfig(10, stop_token_ids=(own[3],))
    first = own.index(own[3])
    assert not unjustified_tokens(plain, weights, config, prompt, own[: first + 1], stopping)
    assert unjustified_tokens(plain, weights, config, prompt, own[: first + 2], stopping)  # went on after the stop token
    assert unjustified_tokens(plain, weights, config, prompt, own[:first], stopping)  # ended early without one
