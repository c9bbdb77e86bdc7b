"""The tests' own small configurations.  They differ in every size and option:
head counts and group size, head size, widths that are no power of two, number
of layers, vocabulary, eps, theta, rotary pairing, tied or untied head, window,
page size, how norm weights are drawn and stored."""

from __future__ import annotations

from pathlib import Path

import torch

from llmserve_amd import Qwen2Config
from llmserve_amd.weights import write_model_folder

# A: 2 layers, G = 2, head size 16, tied, no window, reference pairing, page 16.
TINY_A = Qwen2Config(
    vocab_size=256,
    hidden_size=64,
    intermediate_size=128,
    num_layers=2,
    num_attention_heads=4,
    num_key_value_heads=2,
    head_dim=16,
    max_position_embeddings=512,
    rope_theta=10000.0,
    rms_norm_eps=1e-6,
    attention_bias=True,
    tie_word_embeddings=True,
    rope_pairing="adjacent",
)
PAGE_A = 16

# B: 3 layers, one kv head (G = 6), head size 32, untied, widths 192/320/384,
# layers 1 and 2 see a window of 24 keys, checkpoint pairing, page 8.
TINY_B = Qwen2Config(
    vocab_size=384,
    hidden_size=192,
    intermediate_size=320,
    num_layers=3,
    num_attention_heads=6,
    num_key_value_heads=1,
    head_dim=32,
    max_position_embeddings=1024,
    rope_theta=1e6,
    rms_norm_eps=1e-5,
    attention_bias=True,
    tie_word_embeddings=False,
    rope_pairing="half",
    use_sliding_window=True,
    sliding_window=24,
    max_window_layers=1,
)
PAGE_B = 8

# C: hidden size differs from heads * head_dim, 5 heads over 5 kv heads (G = 1),
# head size 48, no bias; used where a third shape helps.
TINY_C = Qwen2Config(
    vocab_size=131,
    hidden_size=80,
    intermediate_size=112,
    num_layers=2,
    num_attention_heads=5,
    num_key_value_heads=5,
    head_dim=48,
    max_position_embeddings=256,
    rope_theta=500.0,
    rms_norm_eps=1e-4,
    attention_bias=False,
    tie_word_embeddings=False,
    rope_pairing="half",
)
PAGE_C = 32


# W: the layer sizes of the 1.5B benchmark configuration (head size 128, G = 6, widths 1536 and 8960)
# with two layers and a small vocabulary that is no power of two: the kernels that serving picks at
# real widths, inside a whole model.
WIDE = Qwen2Config(
    vocab_size=1031,
    hidden_size=1536,
    intermediate_size=8960,
    num_layers=2,
    num_attention_heads=12,
    num_key_value_heads=2,
    head_dim=128,
    max_position_embeddings=4096,
    rope_theta=1e6,
    rms_norm_eps=1e-6,
    attention_bias=True,
    tie_word_embeddings=True,
    rope_pairing="half",
)
PAGE_WIDE = 16


# The 7B layer sizes (seven query heads a kv head, widths 3584 and 18944, untied head), two layers.
WIDE_7B = Qwen2Config(
    vocab_size=1019,
    hidden_size=3584,
    intermediate_size=18944,
    num_layers=2,
    num_attention_heads=28,
    num_key_value_heads=4,
    head_dim=128,
    max_position_embeddings=4096,
    rope_theta=1e6,
    rms_norm_eps=1e-6,
    attention_bias=True,
    tie_word_embeddings=False,
    rope_pairing="half",
)

# The 32B layer sizes (five query heads a kv head, widths 5120 and 27648, eps 1e-5, untied head), one layer:
# a layer holds 488 million weights, and the plain forward runs on the CPU.
WIDE_32B = Qwen2Config(
    vocab_size=1013,
    hidden_size=5120,
    intermediate_size=27648,
    num_layers=1,
    num_attention_heads=40,
    num_key_value_heads=8,
    head_dim=128,
    max_position_embeddings=4096,
    rope_theta=1e6,
    rms_norm_eps=1e-5,
    attention_bias=True,
    tie_word_embeddings=False,
    rope_pairing="half",
)

# A narrow model with the benchmark's head size, for contexts of thousands of keys through the whole engine: six
# query heads over one kv head of 128, so that decoding takes the kernels that serving takes there (the fused
# decode attention, its key splits, the kernel that merges them).
LONG = Qwen2Config(
    vocab_size=517,
    hidden_size=384,
    intermediate_size=640,
    num_layers=2,
    num_attention_heads=6,
    num_key_value_heads=1,
    head_dim=128,
    max_position_embeddings=16384,
    rope_theta=1e6,
    rms_norm_eps=1e-6,
    attention_bias=True,
    tie_word_embeddings=True,
    rope_pairing="half",
)

MANY_HEADS = Qwen2Config(  # narrow, with the 7B sizes' heads: a 2,048-token portion is 448 workgroups of 128 columns
    vocab_size=517,
    hidden_size=256,
    intermediate_size=384,
    num_layers=1,
    num_attention_heads=28,
    num_key_value_heads=4,
    head_dim=128,
    max_position_embeddings=8192,
    rope_theta=1e6,
    rms_norm_eps=1e-6,
    attention_bias=True,
    tie_word_embeddings=True,
    rope_pairing="half",
)

WIDE_CONFIGS = {"1.5B": (WIDE, 31), "7B": (WIDE_7B, 37), "32B": (WIDE_32B, 41)}


def write_wide_folder(root: Path, sizes: str = "1.5B") -> Path:
    config, seed = WIDE_CONFIGS[sizes]
    return write_model_folder(root / f"W{sizes}", config, seed=seed, norm_std=0.1)


# How the "loud" folders are drawn.  At N(0, 0.02) a model this narrow barely attends: every score is
# near zero, and a wrong rotation or a lost bias moves the logits by less than bfloat16 rounding does.
# Four times wider weights and biases of 0.3 make attention decide the logits, so that the bfloat16
# bounds below can see such faults (test_plain.py shows that they do).
LOUD = dict(std=0.08, bias_std=0.3)

# What a bfloat16 run may differ from the plain implementation by, in units of the logits' spread (their
# standard deviation): the largest element, and the mean over all elements.  Each of the ten or so roundings
# of an activation between kernels adds about 2^-9 of the spread.
BF16_LARGEST, BF16_MEAN = 0.06, 0.01


def write_tiny_folders(root: Path) -> dict[str, Path]:
    return {
        # norm weights 1.0 as the reference initialises them, biases drawn
        "A": write_model_folder(root / "A", TINY_A, seed=11, norm_std=0.0),
        # norm weights N(1, 0.1), stored in 32-bit so that they stay so in a bfloat16 run
        "B": write_model_folder(root / "B", TINY_B, seed=23, norm_std=0.1, wide_roles=("norm",)),
        "C": write_model_folder(root / "C", TINY_C, seed=5, norm_std=0.1, std=0.05),
        "A-loud": write_model_folder(root / "A-loud", TINY_A, seed=12, norm_std=0.0, **LOUD),
        "B-loud": write_model_folder(root / "B-loud", TINY_B, seed=24, norm_std=0.1, wide_roles=("norm",), **LOUD),
        "C-loud": write_model_folder(root / "C-loud", TINY_C, seed=6, norm_std=0.1, **LOUD),
    }


CONFIGS = {"A": (TINY_A, PAGE_A), "B": (TINY_B, PAGE_B), "C": (TINY_C, PAGE_C)}
CONFIGS.update({f"{name}-loud": CONFIGS[name] for name in ("A", "B", "C")})


def unjustified_greedy_tokens(plain, weights, config, prompt: list[int], generated: list[int], largest: float = BF16_LARGEST):
    """Checks greedy tokens of a reduced-precision run one by one: token j must be, for the plain
    implementation fed the run's own prefix, the best token or within rounding of it (two logits, each
    off by at most `largest` of the spread).  Returns [(j, token, how far below the best, allowed)] of
    those that are not; an exact run returns none because it equals the plain decoder."""
    bad = []
    for index, token in enumerate(generated):
        logits = plain.forward(weights, config, list(prompt) + list(generated[:index]))[-1]
        allowed = 2 * largest * float(logits.std())
        short = float(logits.max() - logits[token])
        if short > allowed:
            bad.append((index, token, short, allowed))
    return bad


def _mass_bounds(mass: float, stretch: float) -> tuple[float, float]:
    """What the summed probability of a fixed set of tokens can become when every normalised probability moves
    by a factor between 1 / stretch and stretch (the set's complement moves the same way)."""
    low = max(mass / stretch, 1.0 - (1.0 - mass) * stretch, 0.0)
    high = min(mass * stretch, 1.0 - (1.0 - mass) / stretch, 1.0)
    return low, high


def unjustified_tokens(plain, weights, config, prompt: list[int], generated: list[int], settings, largest: float = BF16_LARGEST):
    """Checks the tokens of a reduced-precision run one by one against the plain implementation fed the run's
    own prefix.  A greedy token must be the best or within rounding of it (`unjustified_greedy_tokens`).  A
    sampled token must be one that the plain sampler's rule could give at the request's own draw u =
    uniform_for(seed, j) once every logit may be off by `largest` of the spread: every probability then moves
    by a factor of at most exp(2 * that / temperature), and u (times the kept mass, for top-p) must fall into
    the token's interval of the cumulated probabilities widened by that much; under top-p the token must also
    be one that can be kept, and tokens whose probabilities are within the factor of the chosen one's may
    stand before or behind it.  Also: nothing follows a stop token, and a run that ends early ends in one.
    Returns the offending (index, token, why)."""
    import math

    bad = []
    stops = set(settings.stop_token_ids)
    if len(generated) > settings.max_new_tokens or (len(generated) < settings.max_new_tokens and (not generated or generated[-1] not in stops)):
        bad.append((len(generated), None, "wrong number of tokens"))
    for index, token in enumerate(generated):
        if index < len(generated) - 1 and token in stops:
            bad.append((index, token, "a stop token is not the last"))
        logits = plain.forward(weights, config, list(prompt) + list(generated[:index]))[-1].double()
        off = largest * float(logits.std())
        if settings.temperature <= 0:
            if float(logits.max() - logits[token]) > 2 * off:
                bad.append((index, token, f"{float(logits.max() - logits[token]):.4f} below the best, {2 * off:.4f} allowed"))
            continue
        u = plain.uniform_for(settings.seed, index)
        p = torch.softmax(logits / settings.temperature, dim=-1)
        stretch = math.exp(2 * off / settings.temperature)
        if settings.top_p >= 1.0:
            before, upto = float(p[:token].sum()), float(p[: token + 1].sum())
            kept_low = kept_high = 1.0
        else:
            mine = float(p[token])
            before = float(p[p > mine * stretch * stretch].sum())  # certainly in front of it in descending order
            upto = float(p[p >= mine / (stretch * stretch)].sum())  # in front of it at most, itself included
            kept_low, kept_high = settings.top_p, min(1.0, settings.top_p + float(p.max()) * stretch)
            if _mass_bounds(before, stretch)[0] >= settings.top_p:
                bad.append((index, token, f"cannot be kept: mass {before:.4f} lies in front of it, top_p {settings.top_p}"))
                continue
        lowest, highest = _mass_bounds(before, stretch)[0], _mass_bounds(upto, stretch)[1]
        if not (lowest <= u * kept_high and u * kept_low < highest):
            bad.append((index, token, f"draw {u:.4f} (kept mass {kept_low:.3f}-{kept_high:.3f}) outside [{lowest:.4f}, {highest:.4f})"))
    return bad


def random_tokens(count: int, vocab: int, seed: int) -> list[int]:
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=generator).tolist()
