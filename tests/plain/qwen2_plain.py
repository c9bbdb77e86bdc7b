"""Plain, slow Qwen2 decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference's `src/llmserve/model.py`; each
function cites the lines it restates.  It shares no code with the engine
package: it reads a model folder with the safetensors library directly and
does all math with elementary torch operations on the CPU.

Everything runs in the dtype of `weights` (the tests use float64 as oracle and
float32 where the reference's own rounding steps matter).
"""

from __future__ import annotations

import json
import math
from dataclasses import dataclass
from pathlib import Path

import torch


@dataclass(frozen=True)
class PlainConfig:
    """The config.json keys the reference reads (`config.py:10-22,46-54`), plus
    the explicit `head_dim`, rotary pairing and window that the engine adds."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    rope_theta: float
    rms_norm_eps: float
    attention_bias: bool
    tie_word_embeddings: bool
    rope_pairing: str = "adjacent"  # the reference's (`model.py:39-42`)
    # window[i] is None (all earlier keys) or the number of keys layer i sees.
    windows: tuple = ()

    @classmethod
    def from_folder(cls, folder: str | Path) -> "PlainConfig":
        values = json.loads((Path(folder) / "config.json").read_text())
        layers = values["num_hidden_layers"]
        heads = values["num_attention_heads"]
        windows = [None] * layers
        if values.get("use_sliding_window", False):
            for index in range(values.get("max_window_layers", layers), layers):
                windows[index] = values["sliding_window"]
        return cls(
            vocab_size=values["vocab_size"],
            hidden_size=values["hidden_size"],
            intermediate_size=values["intermediate_size"],
            num_layers=layers,
            num_heads=heads,
            num_kv_heads=values["num_key_value_heads"],
            head_dim=values.get("head_dim", values["hidden_size"] // heads),
            rope_theta=float(values["rope_theta"]),
            rms_norm_eps=float(values["rms_norm_eps"]),
            attention_bias=values.get("attention_bias", True),
            tie_word_embeddings=values.get("tie_word_embeddings", True),
            rope_pairing=values.get("rope_pairing", "adjacent"),
            windows=tuple(windows),
        )


def read_weights(folder: str | Path, dtype: torch.dtype = torch.float64) -> dict[str, torch.Tensor]:
    """All tensors of `model.safetensors`, names without the `model.` prefix
    (`checkpoint.py:52`), converted exactly (bf16 -> wider is lossless)."""
    from safetensors.torch import load_file

    tensors = load_file(str(Path(folder) / "model.safetensors"))
    return {name.removeprefix("model."): value.to(dtype) for name, value in tensors.items()}


# --------------------------------------------------------------------------- parts


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """`model.py:20-23`: mean of squares, rsqrt(var + eps), times the weight
    last; no mean subtraction, no `1 + w`."""
    variance = x.pow(2).mean(-1, keepdim=True)
    return x * torch.rsqrt(variance + eps) * weight


def rope_angles(head_dim: int, theta: float, positions: torch.Tensor) -> torch.Tensor:
    """`model.py:29-31`: inv[j] = 1 / theta^(2j/D) and ang[p, j] = p * inv[j],
    built in float32 exactly as the reference's tables are."""
    inverse = 1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))
    return torch.outer(positions.float(), inverse)  # [S, D/2] float32


def rope_adjacent(x: torch.Tensor, angles: torch.Tensor) -> torch.Tensor:
    """`model.py:39-43`: pairs are (2j, 2j+1); x is [S, heads, D]."""
    cos = angles.cos().to(x.dtype)[:, None, :]
    sin = angles.sin().to(x.dtype)[:, None, :]
    even, odd = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = even * cos - odd * sin
    out[..., 1::2] = odd * cos + even * sin
    return out


def rope_half(x: torch.Tensor, angles: torch.Tensor) -> torch.Tensor:
    """The same rotation with pairs (j, j + D/2): what `rope_adjacent` does to a
    head whose rows were permuted [0, 2, 4, ..., 1, 3, 5, ...] (the layout of
    published Qwen2 checkpoints; the reference has no such code)."""
    half = x.shape[-1] // 2
    cos = angles.cos().to(x.dtype)[:, None, :]
    sin = angles.sin().to(x.dtype)[:, None, :]
    first, second = x[..., :half], x[..., half:]
    return torch.cat([first * cos - second * sin, second * cos + first * sin], dim=-1)


def causal_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: float,
    window: int | None = None,
) -> torch.Tensor:
    """`model.py:84-95` (plain path) and `:140-175` (what the paged walk sums):
    query head h uses kv head h // G; scores = q.k * scale; a query at position
    i sees keys j <= i, and with a window only those with j > i - window
    (the window is the engine's addition: the reference has none).
    q: [S, Hq, D], k, v: [S, Hkv, D] -> [S, Hq, D].  Explicit loops on purpose."""
    length, heads, _ = q.shape
    group = heads // k.shape[1]
    out = torch.zeros_like(q)
    for head in range(heads):
        kv_head = head // group
        for i in range(length):
            first = 0 if window is None else max(0, i - window + 1)
            scores = (k[first : i + 1, kv_head] @ q[i, head]) * scale
            weights = torch.softmax(scores, dim=0)
            out[i, head] = weights @ v[first : i + 1, kv_head]
    return out


def swiglu(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """`model.py:187-188`: down(silu(gate(x)) * up(x)), silu(z) = z * sigmoid(z),
    no biases; weights are [out, in]."""
    g = x @ gate.T
    return ((g * torch.sigmoid(g)) * (x @ up.T)) @ down.T


def attention_layer(
    x: torch.Tensor,
    weights: dict[str, torch.Tensor],
    prefix: str,
    config: PlainConfig,
    positions: torch.Tensor,
    window: int | None,
) -> torch.Tensor:
    """`model.py:71-95`: q/k/v projections with bias, rotary on q and k (not v),
    attention, o projection without bias."""
    length = x.shape[0]

    def project(name: str, heads: int) -> torch.Tensor:
        y = x @ weights[f"{prefix}{name}.weight"].T
        if config.attention_bias:
            y = y + weights[f"{prefix}{name}.bias"]
        return y.view(length, heads, config.head_dim)

    q = project("q_proj", config.num_heads)
    k = project("k_proj", config.num_kv_heads)
    v = project("v_proj", config.num_kv_heads)
    angles = rope_angles(config.head_dim, config.rope_theta, positions)
    rotate = rope_adjacent if config.rope_pairing == "adjacent" else rope_half
    q, k = rotate(q, angles), rotate(k, angles)
    out = causal_attention(q, k, v, 1.0 / math.sqrt(config.head_dim), window)
    return out.reshape(length, -1) @ weights[f"{prefix}o_proj.weight"].T


def decoder_layer(
    h: torch.Tensor,
    weights: dict[str, torch.Tensor],
    index: int,
    config: PlainConfig,
    positions: torch.Tensor,
) -> torch.Tensor:
    """`model.py:199-201`: h += Attn(Norm_in(h)); h += MLP(Norm_post(h))."""
    prefix = f"layers.{index}."
    window = config.windows[index] if config.windows else None
    normed = rms_norm(h, weights[prefix + "input_layernorm.weight"], config.rms_norm_eps)
    h = h + attention_layer(normed, weights, prefix + "self_attn.", config, positions, window)
    normed = rms_norm(h, weights[prefix + "post_attention_layernorm.weight"], config.rms_norm_eps)
    return h + swiglu(
        normed,
        weights[prefix + "mlp.gate_proj.weight"],
        weights[prefix + "mlp.up_proj.weight"],
        weights[prefix + "mlp.down_proj.weight"],
    )


def forward(
    weights: dict[str, torch.Tensor],
    config: PlainConfig,
    token_ids: list[int],
    first_position: int = 0,
) -> torch.Tensor:
    """`model.py:260-268`: embed, all layers, final norm, lm_head (the embedding
    table itself when tied, `:249-250`).  Returns logits [S, V].  Positions are
    absolute indices starting at `first_position` (0 in the reference, `:263`)."""
    positions = torch.arange(first_position, first_position + len(token_ids))
    h = weights["embed_tokens.weight"][torch.tensor(token_ids, dtype=torch.long)]
    for index in range(config.num_layers):
        h = decoder_layer(h, weights, index, config, positions)
    head = weights["embed_tokens.weight"] if config.tie_word_embeddings else weights["lm_head.weight"]
    return rms_norm(h, weights["norm.weight"], config.rms_norm_eps) @ head.T


# --------------------------------------------------------------------------- sampling


def uniform_for(seed: int, step: int) -> float:
    """The engine's counter-based draw: a float in [0, 1) that depends only on
    the request's seed and on how many tokens it has sampled before (so it is the
    same whatever the batch holds or whether the request was preempted).  The
    reference draws from a per-request torch.Generator instead
    (`engine.py:41,218`), whose stream cannot be reproduced on another device.
    splitmix64 of seed * 2^32 + step, top 24 bits."""
    mask = (1 << 64) - 1
    z = ((seed & 0xFFFFFFFF) << 32 | (step & 0xFFFFFFFF)) & mask
    z = (z + 0x9E3779B97F4A7C15) & mask
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
    z = z ^ (z >> 31)
    return (z >> 40) / float(1 << 24)


def sample(logits: torch.Tensor, temperature: float, top_p: float, u: float) -> int:
    """`engine.py:29-41`: temperature <= 0 -> argmax; else p = softmax(logits /
    temperature) in float32; top_p < 1 keeps, in descending order of p, the
    entries whose preceding mass is < top_p (`:34-37`).  Where the reference
    calls torch.multinomial the engine inverts the CDF at u: the first entry, in
    index order (top_p == 1) or in descending order (top_p < 1, ties by index),
    whose running sum exceeds u * (kept mass)."""
    if temperature <= 0:
        return int(torch.argmax(logits))
    p = torch.softmax(logits.float() / temperature, dim=-1).double()
    if top_p < 1.0:
        order = sorted(range(p.numel()), key=lambda i: (-float(p[i]), i))
        kept, before = [], 0.0
        for index in order:
            if before >= top_p:
                break
            kept.append(index)
            before += float(p[index])
    else:
        order = list(range(p.numel()))
        kept = order
    target = u * sum(float(p[i]) for i in kept)
    running = 0.0
    for index in kept:
        running += float(p[index])
        if running > target:
            return index
    return kept[-1]


def generate(
    weights: dict[str, torch.Tensor],
    config: PlainConfig,
    prompt: list[int],
    max_new_tokens: int,
    temperature: float = 0.0,
    top_p: float = 1.0,
    seed: int = 7,
    stop_token_ids: tuple = (),
) -> list[int]:
    """`engine.py:83-105` (NaiveDecoder): the whole prefix again for every token;
    a stop token is kept in the output."""
    output: list[int] = []
    for step in range(max_new_tokens):
        logits = forward(weights, config, prompt + output)[-1]
        token = sample(logits, temperature, top_p, uniform_for(seed, step))
        output.append(token)
        if token in stop_token_ids:
            break
    return output
