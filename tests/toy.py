"""A toy architecture defined entirely in the tests, to show that parts and whole
architectures are added by registering them, without a change to the framework's files:

- a mixer with state of its own (a decaying sum per request, a fixed-size state slot),
- beside attention layers, chosen layer by layer,
- a feed-forward with routing (a few small experts, the best two per token) in one layer,
- a position encoding with a tensor of its own (a learned table added to queries and keys) in another,
- a position encoding that acts on the scores, not on queries and keys (a bias that grows with distance, and a
  soft cap), in a third attention layer,
- a run order that names one layer twice, and a run that reads another run's cache;
- and a second architecture all of whose parts are the same kernel launches whatever the data, among them a
  mixer with state of its own that runs on the device alone: its steps are captured into graphs and replayed;
  it also has a part between the embedding and the first layer (a learned table of absolute positions, and a
  scale) and one after the head (a bias and a soft cap on the logits);
- and a third whose cache needs are its own: a mixer that keeps one narrow key row and one wider value row per
  token in pages (a kind of need defined here, with its own page layout), a block with attention and the
  decaying mixer side by side (pages *and* a state slot for one run), and a feed-forward whose gate has
  another activation.

It is never a model of anyone's: it exists to exercise the interfaces."""

from __future__ import annotations

import json
import math
from dataclasses import dataclass
from pathlib import Path
from typing import Any, ClassVar

import torch

from llmserve_amd.config.model import ArchitectureConfig, KeyReader
from llmserve_amd.parts import (
    BLOCKS, FEED_FORWARDS, LOGIT_PARTS, MIXERS, NORMS, POSITIONS, STREAM_PARTS, AttentionSpec, Block, FeedForward, FixedState,
    GatedMLPSpec, LayerDefinition, LayerRun, Mixer, ModelSpec, NamedPart, NoPositionSpec, PagedNeed, Part, PositionEncoding,
    PreNormBlockSpec, RMSNormSpec, RotarySpec, TensorSpec,
)
from llmserve_amd.parts.base import prefixed, under
from llmserve_amd.registry import register_architecture, unregister_architecture


@dataclass(frozen=True)
class DecaySpec:
    hidden_size: int
    state_size: int
    decay: float
    kind: str = "toy_decay"


class DecayMixer(Mixer):
    """state <- decay * state + x W_in;  out = state W_out, token after token in order.
    The state of a request lives in its slot of the cell, across steps."""

    replayable = False  # a loop on the host over each request's tokens

    @classmethod
    def tensors(cls, spec: DecaySpec) -> dict[str, TensorSpec]:
        return {
            "in_proj.weight": TensorSpec((spec.state_size, spec.hidden_size)),
            "out_proj.weight": TensorSpec((spec.hidden_size, spec.state_size)),
        }

    @classmethod
    def cache_need(cls, spec: DecaySpec) -> FixedState:
        return FixedState((spec.state_size,))

    def __init__(self, spec: DecaySpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.w_in = tensors["in_proj.weight"].float()
        self.w_out = tensors["out_proj.weight"].float()

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        pushed = x.float() @ self.w_in.T  # [T, state]
        out = torch.empty(x.shape[0], self.spec.hidden_size, dtype=torch.float32, device=x.device)
        row = 0
        for chunk in batch.chunks:
            state = cell.state[chunk.slot]
            for _ in range(chunk.count):
                state = self.spec.decay * state + pushed[row]
                out[row] = state @ self.w_out.T
                row += 1
            if cell.writable:
                cell.state[chunk.slot] = state
        return out


@dataclass(frozen=True)
class RoutedSpec:
    hidden_size: int
    expert_size: int
    experts: int
    chosen: int
    kind: str = "toy_routed"


class RoutedFeedForward(FeedForward):
    """Router logits in float32; the `chosen` best experts of a token, weighted by the softmax
    over their logits alone; every expert a small gated MLP run through the kernel library on the
    rows that chose it."""

    replayable = False  # which rows go to which expert is looked up on the host

    @classmethod
    def tensors(cls, spec: RoutedSpec) -> dict[str, TensorSpec]:
        found = {"router.weight": TensorSpec((spec.experts, spec.hidden_size))}
        for expert in range(spec.experts):
            found[f"experts.{expert}.gate_proj.weight"] = TensorSpec((spec.expert_size, spec.hidden_size))
            found[f"experts.{expert}.up_proj.weight"] = TensorSpec((spec.expert_size, spec.hidden_size))
            found[f"experts.{expert}.down_proj.weight"] = TensorSpec((spec.hidden_size, spec.expert_size))
        return found

    def __init__(self, spec: RoutedSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.router = tensors["router.weight"].float()
        self.gate_up = [
            kernels.prepare_gated_linear(tensors[f"experts.{e}.gate_proj.weight"], tensors[f"experts.{e}.up_proj.weight"])
            for e in range(spec.experts)
        ]
        self.down = [kernels.prepare_linear([tensors[f"experts.{e}.down_proj.weight"]], None) for e in range(spec.experts)]

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        logits = x.float() @ self.router.T
        best, which = torch.topk(logits, self.spec.chosen, dim=-1)
        weights = torch.softmax(best, dim=-1)
        out = torch.zeros(x.shape[0], self.spec.hidden_size, dtype=torch.float32, device=x.device)
        for expert in range(self.spec.experts):
            rows, place = torch.nonzero(which == expert, as_tuple=True)
            if rows.numel() == 0:
                continue
            hidden = self.kernels.gated_linear(x[rows].contiguous(), self.gate_up[expert])
            result = self.kernels.linear(hidden, self.down[expert], out_dtype=torch.float32)
            out.index_add_(0, rows, result * weights[rows, place].unsqueeze(-1))
        return out


@dataclass(frozen=True)
class LearnedPositionSpec:
    head_dim: int
    max_length: int
    kind: str = "toy_learned"


class LearnedPosition(PositionEncoding):
    """Adds row `position` of a learned table to every query and key head; then stores."""

    @classmethod
    def tensors(cls, spec: LearnedPositionSpec) -> dict[str, TensorSpec]:
        return {"table": TensorSpec((spec.max_length, spec.head_dim))}

    def __init__(self, spec: LearnedPositionSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.table = tensors["table"]

    def encode_and_store(self, qkv, layout, batch, cell) -> None:
        rotated = layout.num_heads + layout.num_kv_heads
        heads = qkv.view(qkv.shape[0], -1, layout.head_dim)
        heads[:, :rotated] += self.table[batch.positions.long()].to(qkv.dtype).unsqueeze(1)
        self.kernels.rotate_and_store(qkv, layout, batch, cell, None, "none")


@dataclass(frozen=True)
class DistanceBiasSpec:
    num_heads: int
    steepest: float  # head h's slope is steepest / 2^h
    soft_cap: float
    kind: str = "toy_distance_bias"


class DistanceBias(PositionEncoding):
    """Nothing is done to queries and keys: a score loses slope[head] * distance after being
    squashed to soft_cap * tanh(score / soft_cap)."""

    def __init__(self, spec: DistanceBiasSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.slopes = kernels.to_device(torch.tensor([spec.steepest / 2.0 ** head for head in range(spec.num_heads)], dtype=torch.float32))

    def encode_and_store(self, qkv, layout, batch, cell) -> None:
        self.kernels.rotate_and_store(qkv, layout, batch, cell, None, "none")

    def encode_store_attend(self, qkv, layout, batch, cell, scale, window, project=None):
        self.encode_and_store(qkv, layout, batch, cell)
        mixed = self.kernels.paged_attention(qkv, layout, batch, cell, scale, window, score_slopes=self.slopes,
                                             soft_cap=self.spec.soft_cap)
        return mixed if project is None else self.kernels.linear(mixed, project, out_dtype=torch.float32, partial=True)


@dataclass(frozen=True)
class RunningSumSpec:
    hidden_size: int
    state_size: int
    kind: str = "toy_running_sum"


class RunningSumMixer(Mixer):
    """state <- state + x W_in;  out = state W_out, token after token in order: the decaying mixer without its
    decay, so that a request's tokens can be summed by a prefix sum on the device.  Nothing is looked at on the
    host and every shape depends on the step's shape alone: a step through it may be captured and replayed."""

    @classmethod
    def tensors(cls, spec: RunningSumSpec) -> dict[str, TensorSpec]:
        return {
            "in_proj.weight": TensorSpec((spec.state_size, spec.hidden_size)),
            "out_proj.weight": TensorSpec((spec.hidden_size, spec.state_size)),
        }

    @classmethod
    def cache_need(cls, spec: RunningSumSpec) -> FixedState:
        return FixedState((spec.state_size,))

    def __init__(self, spec: RunningSumSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.w_in = tensors["in_proj.weight"].float()
        self.w_out = tensors["out_proj.weight"].float()

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        pushed = x.float() @ self.w_in.T  # [T, state]
        request = batch.token_sequence.long()
        slots = batch.state_slots.long()[request]  # each token's state slot (padding tokens: the spare one)
        running = torch.cumsum(pushed, dim=0)
        first = batch.query_start.long()[request]  # row of the token's request's first token
        before = torch.where((first > 0).unsqueeze(1), running[(first - 1).clamp(min=0)], torch.zeros_like(running))
        state = cell.state[slots] + (running - before)  # the state after each token
        if cell.writable:
            cell.state.index_add_(0, slots, pushed)
        return state @ self.w_out.T


@dataclass(frozen=True)
class PagedRows(PagedNeed):
    """A cache need of this file's own: per token one key row and one value row of another width, each page
    holding its tokens' rows one after the other.  The cache manager has never heard of it."""

    key_width: int
    value_width: int
    window: int | None = None

    def page_fields(self, page_size: int) -> dict[str, tuple[int, ...]]:
        return {"key_rows": (page_size, self.key_width), "value_rows": (page_size, self.value_width)}

    def token_rows(self, page: dict[str, torch.Tensor], page_size: int) -> dict[str, torch.Tensor]:
        return dict(page)  # the token's place in the page leads already


@dataclass(frozen=True)
class LatentSpec:
    hidden_size: int
    key_width: int
    value_width: int
    kind: str = "toy_latent"


class LatentMixer(Mixer):
    """One head of attention over narrow keys and wider values: q = x Wq, k = x Wk (key_width), v = x Wv
    (value_width); softmax(q . k / sqrt(key_width)) over the keys up to the token's own; out = (.) Wo.  What it
    caches per token is a `PagedRows` entry, written and read here through the step's slot mapping and block
    tables with plain tensor indexing."""

    replayable = False  # a loop on the host over the step's requests

    @classmethod
    def tensors(cls, spec: LatentSpec) -> dict[str, TensorSpec]:
        return {
            "q_proj.weight": TensorSpec((spec.key_width, spec.hidden_size)),
            "k_proj.weight": TensorSpec((spec.key_width, spec.hidden_size)),
            "v_proj.weight": TensorSpec((spec.value_width, spec.hidden_size)),
            "o_proj.weight": TensorSpec((spec.hidden_size, spec.value_width)),
        }

    @classmethod
    def cache_need(cls, spec: LatentSpec) -> PagedRows:
        return PagedRows(spec.key_width, spec.value_width)

    def __init__(self, spec: LatentSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.w = {name.split(".")[0]: value.float() for name, value in tensors.items()}

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        x = x.float()
        q, k, v = x @ self.w["q_proj"].T, x @ self.w["k_proj"].T, x @ self.w["v_proj"].T
        group = batch.groups[cell.group]
        key_pages, value_pages = cell.fields["key_rows"], cell.fields["value_rows"]
        page_size = group.page_size
        if cell.writable:
            slots = group.slot_mapping.long()
            key_pages[slots // page_size, slots % page_size] = k.to(key_pages.dtype)
            value_pages[slots // page_size, slots % page_size] = v.to(value_pages.dtype)
        out = torch.empty(x.shape[0], self.spec.hidden_size, dtype=torch.float32, device=x.device)
        row = 0
        for index, chunk in enumerate(batch.chunks):
            context = chunk.start + chunk.count
            table = group.block_tables[index, : -(-context // page_size)].long()
            keys = key_pages[table].reshape(-1, self.spec.key_width)[:context].float()
            values = value_pages[table].reshape(-1, self.spec.value_width)[:context].float()
            scores = q[row : row + chunk.count] @ keys.T / math.sqrt(self.spec.key_width)
            position = torch.arange(chunk.start, context, device=x.device).unsqueeze(1)
            scores = scores.masked_fill(torch.arange(context, device=x.device).unsqueeze(0) > position, float("-inf"))
            out[row : row + chunk.count] = (torch.softmax(scores, dim=-1) @ values) @ self.w["o_proj"].T
            row += chunk.count
        return out


@dataclass(frozen=True)
class SideBySideBlockSpec:
    """h += attention(norm(h)) + decay(norm(h)); h += feed_forward(norm(h))."""

    norm: Any
    attention: Any
    decay: Any
    feed_forward_norm: Any
    feed_forward: Any
    kind: str = "toy_side_by_side"


class SideBySideBlock(Block):
    """Two mixers read the same normed rows and their results are added: one keeps keys and values in pages, the
    other a state per request, so one run of the layer needs both, by name."""

    _MEMBERS = (("input_layernorm.", NORMS, "norm"), ("attention.", MIXERS, "attention"), ("decay.", MIXERS, "decay"),
                ("post_attention_layernorm.", NORMS, "feed_forward_norm"), ("mlp.", FEED_FORWARDS, "feed_forward"))

    @classmethod
    def tensors(cls, spec: SideBySideBlockSpec) -> dict[str, TensorSpec]:
        found: dict[str, TensorSpec] = {}
        for name, registry, field in cls._MEMBERS:
            found.update(prefixed(registry.tensors(getattr(spec, field)), name))
        return found

    @classmethod
    def cache_need(cls, spec: SideBySideBlockSpec):
        return {"attention": MIXERS.cache_need(spec.attention), "decay": MIXERS.cache_need(spec.decay)}

    def __init__(self, spec: SideBySideBlockSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        for name, registry, field in self._MEMBERS:
            setattr(self, field, registry.build(getattr(spec, field), under(tensors, name), kernels))
        self.replayable = False

    def forward(self, hidden, delta, batch, cell) -> torch.Tensor:
        normed = self.norm.forward(hidden, delta)
        attended = self.attention.forward(normed, batch, cell["attention"])
        attended = attended if attended.ndim == 2 else attended.sum(0)
        mixed = attended + self.decay.forward(normed, batch, cell["decay"])
        normed = self.feed_forward_norm.forward(hidden, mixed)
        return self.feed_forward.forward(normed, batch)


@dataclass(frozen=True)
class AbsolutePositionsSpec:
    hidden_size: int
    max_length: int
    scale: float
    kind: str = "toy_absolute_positions"


class AbsolutePositions(Part):
    """h <- h * scale + table[position], on the embedded rows, before the first layer."""

    @classmethod
    def tensors(cls, spec: AbsolutePositionsSpec) -> dict[str, TensorSpec]:
        return {"table": TensorSpec((spec.max_length, spec.hidden_size))}

    def __init__(self, spec: AbsolutePositionsSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.table = tensors["table"].float()

    def forward(self, hidden: torch.Tensor, batch) -> None:
        hidden.mul_(self.spec.scale).add_(self.table[batch.positions.long()])


@dataclass(frozen=True)
class CappedLogitsSpec:
    vocab_size: int
    cap: float
    kind: str = "toy_capped_logits"


class CappedLogits(Part):
    """logits <- cap * tanh((logits + bias) / cap), after the head."""

    @classmethod
    def tensors(cls, spec: CappedLogitsSpec) -> dict[str, TensorSpec]:
        return {"bias": TensorSpec((spec.vocab_size,), role="bias")}

    def __init__(self, spec: CappedLogitsSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.bias = tensors["bias"].float()

    def forward(self, logits: torch.Tensor, batch) -> torch.Tensor:
        return self.spec.cap * torch.tanh((logits + self.bias) / self.spec.cap)


@dataclass(frozen=True)
class ToyConfig(ArchitectureConfig):
    architecture: ClassVar[str] = "ToyStateForCausalLM"
    vocab_size: int = 0
    hidden_size: int = 0
    state_size: int = 0
    decay: float = 0.0
    num_heads: int = 0
    head_dim: int = 0
    ffn_size: int = 0
    eps: float = 0.0
    max_length: int = 0
    experts: int = 0
    experts_chosen: int = 0
    expert_size: int = 0

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "ToyConfig":
        reader = KeyReader(values, "toy config")
        return cls(
            vocab_size=reader.integer("vocab_size"), hidden_size=reader.integer("hidden_size"),
            state_size=reader.integer("state_size"), decay=reader.number("decay"),
            num_heads=reader.integer("num_heads"), head_dim=reader.integer("head_dim"),
            ffn_size=reader.integer("ffn_size"), eps=reader.number("eps"), max_length=reader.integer("max_length"),
            experts=reader.integer("experts"), experts_chosen=reader.integer("experts_chosen"),
            expert_size=reader.integer("expert_size"),
        )

    @property
    def max_position_embeddings(self) -> int:
        return self.max_length

    def to_config_json(self) -> dict[str, Any]:
        return {"architectures": [self.architecture], **self.to_dict()}


def toy_spec(config: ToyConfig) -> ModelSpec:
    norm = RMSNormSpec(config.hidden_size, config.eps)
    ffn = GatedMLPSpec(config.hidden_size, config.ffn_size)
    decay = DecaySpec(config.hidden_size, config.state_size, config.decay)
    attention = AttentionSpec(
        config.hidden_size, config.num_heads, config.num_heads, config.head_dim, 1.0 / math.sqrt(config.head_dim),
        RotarySpec(config.head_dim, 100.0, "half"), qkv_bias=False,
    )
    unrotated = AttentionSpec(
        config.hidden_size, config.num_heads, config.num_heads, config.head_dim, 1.0 / math.sqrt(config.head_dim),
        LearnedPositionSpec(config.head_dim, config.max_length), qkv_bias=False,
    )
    routed = RoutedSpec(config.hidden_size, config.expert_size, config.experts, config.experts_chosen)
    biased = AttentionSpec(
        config.hidden_size, config.num_heads, config.num_heads, config.head_dim, 1.0 / math.sqrt(config.head_dim),
        DistanceBiasSpec(config.num_heads, BIAS_STEEPEST, BIAS_SOFT_CAP), qkv_bias=False,
    )
    layers = (
        LayerDefinition("layers.0.", PreNormBlockSpec(norm, decay, norm, routed, mixer_name="mixer.")),
        LayerDefinition("layers.1.", PreNormBlockSpec(norm, attention, norm, ffn, mixer_name="mixer.")),
        LayerDefinition("layers.2.", PreNormBlockSpec(norm, unrotated, norm, ffn, mixer_name="mixer.")),
        LayerDefinition("layers.3.", PreNormBlockSpec(norm, biased, norm, ffn, mixer_name="mixer.")),
    )
    # layer 0 runs twice (two state cells), layer 1 runs twice, its second run reading the first's pages
    run_order = (LayerRun(0), LayerRun(1), LayerRun(2), LayerRun(0), LayerRun(1, reads=1), LayerRun(3))
    return ModelSpec(
        config.vocab_size, config.hidden_size, layers, run_order, norm, tie_embeddings=True,
        embedding_name="embed.weight", final_norm_name="final_norm.",
    )


BIAS_STEEPEST, BIAS_SOFT_CAP = 0.5, 2.0
EMBEDDING_SCALE, LOGIT_CAP = 1.5, 3.0


def sum_spec(config: ToyConfig) -> ModelSpec:
    """The second architecture: a running-sum mixer, then attention whose scores carry a distance bias; every
    part is the same launches whatever the data."""
    norm = RMSNormSpec(config.hidden_size, config.eps)
    ffn = GatedMLPSpec(config.hidden_size, config.ffn_size)
    summing = RunningSumSpec(config.hidden_size, config.state_size)
    biased = AttentionSpec(
        config.hidden_size, config.num_heads, config.num_heads, config.head_dim, 1.0 / math.sqrt(config.head_dim),
        DistanceBiasSpec(config.num_heads, BIAS_STEEPEST, BIAS_SOFT_CAP), qkv_bias=False,
    )
    layers = (
        LayerDefinition("layers.0.", PreNormBlockSpec(norm, summing, norm, ffn, mixer_name="mixer.")),
        LayerDefinition("layers.1.", PreNormBlockSpec(norm, biased, norm, ffn, mixer_name="mixer.")),
    )
    return ModelSpec(
        config.vocab_size, config.hidden_size, layers, (LayerRun(0), LayerRun(1), LayerRun(0)), norm, tie_embeddings=True,
        embedding_name="embed.weight", final_norm_name="final_norm.",
        input_parts=(NamedPart("positions.", AbsolutePositionsSpec(config.hidden_size, config.max_length, EMBEDDING_SCALE)),),
        output_parts=(NamedPart("logits.", CappedLogitsSpec(config.vocab_size, LOGIT_CAP)),),
    )


@dataclass(frozen=True)
class SumConfig(ToyConfig):
    architecture: ClassVar[str] = "ToySumForCausalLM"


LATENT_KEY_WIDTH, LATENT_VALUE_WIDTH, LATENT_ACTIVATION = 12, 28, "gelu_tanh"


def latent_spec(config: ToyConfig) -> ModelSpec:
    """The third architecture: the latent mixer with a feed-forward whose gate is a gelu, then a block with
    attention and the decaying mixer side by side, then the first layer again (a second cell in its group)."""
    norm = RMSNormSpec(config.hidden_size, config.eps)
    gelu_ffn = GatedMLPSpec(config.hidden_size, config.ffn_size, activation=LATENT_ACTIVATION)
    ffn = GatedMLPSpec(config.hidden_size, config.ffn_size)
    latent = LatentSpec(config.hidden_size, LATENT_KEY_WIDTH, LATENT_VALUE_WIDTH)
    decay = DecaySpec(config.hidden_size, config.state_size, config.decay)
    attention = AttentionSpec(
        config.hidden_size, config.num_heads, config.num_heads, config.head_dim, 1.0 / math.sqrt(config.head_dim),
        RotarySpec(config.head_dim, 100.0, "half"), qkv_bias=False,
    )
    layers = (
        LayerDefinition("layers.0.", PreNormBlockSpec(norm, latent, norm, gelu_ffn, mixer_name="mixer.")),
        LayerDefinition("layers.1.", SideBySideBlockSpec(norm, attention, decay, norm, ffn)),
    )
    return ModelSpec(
        config.vocab_size, config.hidden_size, layers, (LayerRun(0), LayerRun(1), LayerRun(0)), norm, tie_embeddings=True,
        embedding_name="embed.weight", final_norm_name="final_norm.",
    )


@dataclass(frozen=True)
class LatentConfig(ToyConfig):
    architecture: ClassVar[str] = "ToyLatentForCausalLM"


TOY = ToyConfig(vocab_size=97, hidden_size=48, state_size=20, decay=0.8, num_heads=3, head_dim=16, ffn_size=64,
                eps=1e-5, max_length=256, experts=5, experts_chosen=2, expert_size=24)


SUM = SumConfig(**TOY.to_dict())
LATENT = LatentConfig(**TOY.to_dict())


def register_toy() -> None:
    MIXERS.register("toy_decay")(DecayMixer)
    MIXERS.register("toy_running_sum")(RunningSumMixer)
    FEED_FORWARDS.register("toy_routed")(RoutedFeedForward)
    POSITIONS.register("toy_learned")(LearnedPosition)
    POSITIONS.register("toy_distance_bias")(DistanceBias)
    STREAM_PARTS.register("toy_absolute_positions")(AbsolutePositions)
    LOGIT_PARTS.register("toy_capped_logits")(CappedLogits)
    register_architecture("ToyStateForCausalLM", ToyConfig, toy_spec)
    register_architecture("ToySumForCausalLM", SumConfig, sum_spec)
    MIXERS.register("toy_latent")(LatentMixer)
    BLOCKS.register("toy_side_by_side")(SideBySideBlock)
    register_architecture("ToyLatentForCausalLM", LatentConfig, latent_spec)


def unregister_toy() -> None:
    MIXERS.unregister("toy_decay")
    MIXERS.unregister("toy_running_sum")
    FEED_FORWARDS.unregister("toy_routed")
    POSITIONS.unregister("toy_learned")
    POSITIONS.unregister("toy_distance_bias")
    STREAM_PARTS.unregister("toy_absolute_positions")
    LOGIT_PARTS.unregister("toy_capped_logits")
    unregister_architecture("ToyStateForCausalLM")
    unregister_architecture("ToySumForCausalLM")
    MIXERS.unregister("toy_latent")
    BLOCKS.unregister("toy_side_by_side")
    unregister_architecture("ToyLatentForCausalLM")


def write_toy_folder(folder: Path, seed: int = 3, config: ToyConfig = TOY) -> Path:
    from llmserve_amd.weights import write_model_folder

    return write_model_folder(folder, config, seed, dtype=torch.float32, std=0.1, norm_std=0.1)


# ----------------------------------------------------------------------------- the toy's own plain forward


def plain_toy_forward(folder: Path, tokens: list[int], with_cached_rows: bool = False) -> torch.Tensor:
    """Whole sequence, no cache, float64; written apart from the parts above.  `with_cached_rows` (the third
    architecture): also the key and value rows that its first run would cache."""
    from safetensors.torch import load_file

    from tests.plain import qwen2_plain as plain

    config = json.loads((folder / "config.json").read_text())
    w = {name: value.double() for name, value in load_file(str(folder / "model.safetensors")).items()}
    eps, dim, heads = config["eps"], config["head_dim"], config["num_heads"]
    h = w["embed.weight"][tokens]
    length = len(tokens)

    def ffn(x, prefix):
        return plain.swiglu(x, w[prefix + "mlp.gate_proj.weight"], w[prefix + "mlp.up_proj.weight"], w[prefix + "mlp.down_proj.weight"])

    def routed(x, prefix):
        logits = x @ w[prefix + "mlp.router.weight"].T
        out = torch.zeros_like(x)
        for t in range(length):
            order = sorted(range(config["experts"]), key=lambda e: (-logits[t, e].item(), e))[: config["experts_chosen"]]
            weights = torch.softmax(logits[t, order], dim=0)
            for weight, e in zip(weights, order):
                name = f"{prefix}mlp.experts.{e}."
                out[t] += weight * plain.swiglu(x[t : t + 1], w[name + "gate_proj.weight"], w[name + "up_proj.weight"],
                                                w[name + "down_proj.weight"])[0]
        return out

    def decay_layer(h, prefix):
        x = plain.rms_norm(h, w[prefix + "input_layernorm.weight"], eps)
        state = torch.zeros(config["state_size"], dtype=torch.float64)
        out = []
        for t in range(length):
            state = config["decay"] * state + w[prefix + "mixer.in_proj.weight"] @ x[t]
            out.append(w[prefix + "mixer.out_proj.weight"] @ state)
        h = h + torch.stack(out)
        return h + routed(plain.rms_norm(h, w[prefix + "post_attention_layernorm.weight"], eps), prefix)

    def biased_attention(q, k, v, scale):
        """softmax over keys j <= i of cap * tanh(q_i . k_j * scale / cap) - slope_head * (i - j)"""
        scores = torch.einsum("ihd,jhd->hij", q, k) * scale
        scores = BIAS_SOFT_CAP * torch.tanh(scores / BIAS_SOFT_CAP)
        distance = (torch.arange(length).unsqueeze(1) - torch.arange(length).unsqueeze(0)).double()
        slopes = torch.tensor([BIAS_STEEPEST / 2.0 ** head for head in range(heads)], dtype=torch.float64)
        scores = scores - slopes.view(-1, 1, 1) * distance
        scores = scores.masked_fill(distance < 0, float("-inf"))
        return torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), v)

    def sum_layer(h, prefix):
        x = plain.rms_norm(h, w[prefix + "input_layernorm.weight"], eps)
        state = torch.cumsum(x @ w[prefix + "mixer.in_proj.weight"].T, dim=0)
        h = h + state @ w[prefix + "mixer.out_proj.weight"].T
        return h + ffn(plain.rms_norm(h, w[prefix + "post_attention_layernorm.weight"], eps), prefix)

    def attention_layer(h, prefix, rotate, shared=None):
        x = plain.rms_norm(h, w[prefix + "input_layernorm.weight"], eps)
        q = (x @ w[prefix + "mixer.q_proj.weight"].T).view(length, heads, dim)
        k = (x @ w[prefix + "mixer.k_proj.weight"].T).view(length, heads, dim)
        v = (x @ w[prefix + "mixer.v_proj.weight"].T).view(length, heads, dim)
        if rotate == "bias":
            mixed = biased_attention(q, k, v, 1.0 / math.sqrt(dim)).reshape(length, -1)
            h = h + mixed @ w[prefix + "mixer.o_proj.weight"].T
            return h + ffn(plain.rms_norm(h, w[prefix + "post_attention_layernorm.weight"], eps), prefix), (k, v)
        if rotate:
            angles = plain.rope_angles(dim, 100.0, torch.arange(length))
            q, k = plain.rope_half(q, angles), plain.rope_half(k, angles)
        else:  # the learned table's row of each position, added to every query and key head
            table = w[prefix + "mixer.position.table"][:length].unsqueeze(1)
            q, k = q + table, k + table
        if shared is not None:
            k, v = shared  # the run reads the keys and values another run stored
        mixed = plain.causal_attention(q, k, v, 1.0 / math.sqrt(dim)).reshape(length, -1)
        h = h + mixed @ w[prefix + "mixer.o_proj.weight"].T
        h = h + ffn(plain.rms_norm(h, w[prefix + "post_attention_layernorm.weight"], eps), prefix)
        return h, (k, v)

    def latent_layer(h, prefix):
        """One head over narrow keys and wider values, then a feed-forward whose gate is a gelu (tanh form).
        Returns the layer's output and the rows it would cache."""
        x = plain.rms_norm(h, w[prefix + "input_layernorm.weight"], eps)
        q, k, v = (x @ w[prefix + f"mixer.{name}_proj.weight"].T for name in "qkv")
        scores = (q @ k.T) / math.sqrt(LATENT_KEY_WIDTH)
        scores = scores.masked_fill(torch.arange(length).unsqueeze(0) > torch.arange(length).unsqueeze(1), float("-inf"))
        h = h + (torch.softmax(scores, dim=-1) @ v) @ w[prefix + "mixer.o_proj.weight"].T
        x = plain.rms_norm(h, w[prefix + "post_attention_layernorm.weight"], eps)
        gate = torch.nn.functional.gelu(x @ w[prefix + "mlp.gate_proj.weight"].T, approximate="tanh")
        return h + (gate * (x @ w[prefix + "mlp.up_proj.weight"].T)) @ w[prefix + "mlp.down_proj.weight"].T, (k, v)

    def side_by_side_layer(h, prefix):
        x = plain.rms_norm(h, w[prefix + "input_layernorm.weight"], eps)
        q = (x @ w[prefix + "attention.q_proj.weight"].T).view(length, heads, dim)
        k = (x @ w[prefix + "attention.k_proj.weight"].T).view(length, heads, dim)
        v = (x @ w[prefix + "attention.v_proj.weight"].T).view(length, heads, dim)
        angles = plain.rope_angles(dim, 100.0, torch.arange(length))
        q, k = plain.rope_half(q, angles), plain.rope_half(k, angles)
        mixed = plain.causal_attention(q, k, v, 1.0 / math.sqrt(dim)).reshape(length, -1) @ w[prefix + "attention.o_proj.weight"].T
        state = torch.zeros(config["state_size"], dtype=torch.float64)
        decayed = []
        for t in range(length):
            state = config["decay"] * state + w[prefix + "decay.in_proj.weight"] @ x[t]
            decayed.append(w[prefix + "decay.out_proj.weight"] @ state)
        h = h + mixed + torch.stack(decayed)
        x = plain.rms_norm(h, w[prefix + "post_attention_layernorm.weight"], eps)
        return h + plain.swiglu(x, w[prefix + "mlp.gate_proj.weight"], w[prefix + "mlp.up_proj.weight"], w[prefix + "mlp.down_proj.weight"])

    if config["architectures"] == ["ToyLatentForCausalLM"]:
        h, first_rows = latent_layer(h, "layers.0.")
        h = side_by_side_layer(h, "layers.1.")
        h, _ = latent_layer(h, "layers.0.")
        logits = plain.rms_norm(h, w["final_norm.weight"], eps) @ w["embed.weight"].T
        return (logits, first_rows) if with_cached_rows else logits
    if config["architectures"] == ["ToySumForCausalLM"]:
        h = h * EMBEDDING_SCALE + w["positions.table"][:length]
        h = sum_layer(h, "layers.0.")
        h, _ = attention_layer(h, "layers.1.", "bias")
        h = sum_layer(h, "layers.0.")
        logits = plain.rms_norm(h, w["final_norm.weight"], eps) @ w["embed.weight"].T
        return LOGIT_CAP * torch.tanh((logits + w["logits.bias"]) / LOGIT_CAP)
    h = decay_layer(h, "layers.0.")
    h, stored = attention_layer(h, "layers.1.", True)
    h, _ = attention_layer(h, "layers.2.", False)
    h = decay_layer(h, "layers.0.")
    h, _ = attention_layer(h, "layers.1.", True, shared=stored)
    h, _ = attention_layer(h, "layers.3.", "bias")
    return plain.rms_norm(h, w["final_norm.weight"], eps) @ w["embed.weight"].T
