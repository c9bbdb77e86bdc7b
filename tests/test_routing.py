"""Which kernel a product goes to, and in what shape, is decided on the host from its sizes alone
(`HipKernels._streaming`, `_ring_shape` and the other rules of `kernels/hip.py`); the kernels refuse what they
were not built for.  This walks the rules over the layer sizes of every configuration shipped here, over tiny
and odd sizes and over every number of rows up to 130, and checks each answer against what the entry points
in `csrc/gemm_bf16.hip` take (`pick_ring`, `launch_ring`; read from the source, restated here), so that a rule
cannot send a step to a refusal that only some batch size would meet.  No GPU needed: the tensors are `meta`."""

from __future__ import annotations

import json
import random
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

from llmserve_amd.kernels.hip import HipKernels, LinearWeights

ROOT = Path(__file__).resolve().parents[1]
LDS_KB = 160
STAGE_KB = 1  # sixteen rows of thirty-two bfloat16 k


def products_of_the_shipped_configurations():
    """(out_features, in_features, gated, may_split) of every product of every configuration under configs/."""
    found = set()
    for path in sorted((ROOT / "configs").glob("*.json")):
        sizes = json.loads(path.read_text())
        hidden, heads, kv_heads = sizes["hidden_size"], sizes["num_attention_heads"], sizes["num_key_value_heads"]
        head_dim = sizes.get("head_dim") or hidden // heads
        found.add(((heads + 2 * kv_heads) * head_dim, hidden, False, False))
        found.add((hidden, heads * head_dim, False, True))
        found.add((2 * sizes["intermediate_size"], hidden, True, False))
        found.add((hidden, sizes["intermediate_size"], False, True))
        found.add((sizes["vocab_size"], hidden, False, False))
    return sorted(found)


def ring_takes(tiles: int, rows: int) -> tuple[int, int, int] | None:
    """(tiles of x, k-steps a stage, stages) of the ring kernel that `pick_ring` launches, or None where it refuses."""
    if rows <= 64:
        x_tiles = 2 if rows <= 32 else 4
        if tiles in (2, 4, 6) or (tiles == 5 and rows > 32):
            return x_tiles, 4, 4
        if tiles in (8, 10, 12, 14):
            return x_tiles, 2, 4
        return None
    if rows <= 128:
        if tiles in (2, 4, 5):
            return 8, 4, 3
        if tiles in (8, 10):
            return 8, 2, 4
    return None


def check_ring(rows: int, out_features: int, in_features: int, may_split: bool) -> None:
    tiles, splits, rounds = HipKernels._ring_shape(rows, out_features, in_features, may_split)
    taken = ring_takes(tiles, rows)
    assert taken is not None, (rows, out_features, in_features, may_split, tiles)
    x_tiles, k_steps, depth = taken
    assert may_split or splits == 1
    assert in_features % splits == 0 and (in_features // splits) % (32 * k_steps) == 0, (rows, out_features, in_features, splits, tiles)
    assert depth * (tiles + x_tiles) * k_steps * STAGE_KB <= LDS_KB
    assert rounds >= 1 and splits <= 65535


def stand_in(**changes):
    settings = dict(ring_products=True, ring_rows_from=4, library_products=True, _for_replay=True, _ring_shape=HipKernels._ring_shape)
    settings.update(changes)
    return SimpleNamespace(**settings)


def route(kernels, rows: int, out_features: int, in_features: int, gated: bool, may_split: bool):
    x = torch.empty((rows, in_features), dtype=torch.bfloat16, device="meta")
    weights = LinearWeights(torch.empty((out_features, in_features), dtype=torch.bfloat16, device="meta"), None)
    return HipKernels._streaming(kernels, x, weights, gated=gated, may_split=may_split)


@pytest.mark.parametrize("for_replay", [True, False])
@pytest.mark.parametrize("library_products", [True, False])
def test_every_route_of_the_shipped_sizes_is_one_its_kernel_takes(for_replay, library_products):
    kernels = stand_in(_for_replay=for_replay, library_products=library_products)
    routes = set()
    for out_features, in_features, gated, may_split in products_of_the_shipped_configurations():
        for rows in list(range(1, 131)) + [192, 256, 2048]:
            way = route(kernels, rows, out_features, in_features, gated, may_split)
            routes.add(way)
            assert way in ("skinny", "ring", "medium", "tiled", None)
            if way == "ring":
                assert rows <= 128 and in_features % 128 == 0
                check_ring(rows, out_features, in_features, may_split and not gated)
            if way == "skinny":
                assert rows <= 64 and in_features % 32 == 0
            if way == "medium":
                assert 16 < rows <= 64 and in_features % 128 == 0
            if way == "tiled":
                assert rows > 64 and in_features % 32 == 0
            if way is None:  # the library, or (without it, and for sizes no matrix-core kernel takes) the generic kernel
                assert (library_products and rows > 16) or in_features % 32 != 0 or rows <= 0
    assert "ring" in routes and "skinny" in routes


def test_ring_shapes_at_random_sizes():
    draw = random.Random(5)
    for _ in range(20000):
        rows = draw.randint(1, 128)
        in_features = 128 * draw.randint(1, 260)
        out_features = draw.choice([draw.randint(1, 400), 16 * draw.randint(1, 4000), draw.randint(1, 160000)])
        check_ring(rows, out_features, in_features, draw.random() < 0.5)


def test_routes_at_random_sizes():
    draw = random.Random(6)
    kernels = [stand_in(_for_replay=a, library_products=b) for a in (True, False) for b in (True, False)]
    for _ in range(20000):
        rows = draw.choice([draw.randint(1, 130), draw.randint(1, 4096)])
        in_features = draw.choice([128 * draw.randint(1, 260), 32 * draw.randint(1, 900), draw.randint(1, 30000)])
        out_features = draw.choice([draw.randint(1, 400), 16 * draw.randint(1, 4000), draw.randint(1, 160000)])
        gated = draw.random() < 0.3
        if gated:
            out_features += out_features % 2
        may_split = not gated and draw.random() < 0.5
        way = route(draw.choice(kernels), rows, out_features, in_features, gated, may_split)
        if way == "ring":
            assert rows <= 128 and in_features % 128 == 0
            check_ring(rows, out_features, in_features, may_split)
        elif way in ("skinny", "medium"):
            assert rows <= 64 and in_features % 32 == 0
        elif way == "tiled":
            assert in_features % 32 == 0
        else:
            assert way is None


def test_attention_work_lists_cover_every_column_once_and_fit_the_padded_shape():
    """The attention kernels take their work from a list of (request, first token, first head of it, columns)
    items made on the host; a captured step's list has room for the most items its padded shape can hold.
    Steps drawn at random: the items cover every (token, head) column of the chosen chunks exactly once, no
    item is longer than the kernel's tile, and no step of a shape has more items than the shape's room."""
    from llmserve_amd.engine.batch import SequenceChunk

    draw = random.Random(9)
    for _ in range(3000):
        group = draw.choice([1, 2, 5, 6, 7, 8, 16, 17, 28])
        column_tiles = draw.choice([1, 2])
        packed = draw.choice([None, True, False])
        requests = draw.randint(1, 12)
        counts = [draw.choice([1, 1, 1, 2, 3, 16, 17, draw.randint(1, 700)]) for _ in range(requests)]
        chunks = [SequenceChunk(f"r{i}", i, draw.randint(0, 5000), count) for i, count in enumerate(counts)]
        longer_than, up_to = draw.choice([(0, None), (0, 16), (16, None), (1, None), (0, 1)])
        work, steps = HipKernels._work_items(chunks, group, column_tiles, longer_than, up_to, packed)
        is_packed = group <= 16 if packed is None else packed
        per_token = group if is_packed else 1
        per_item = column_tiles * (16 if is_packed else 1)
        chosen = [i for i, count in enumerate(counts) if count > longer_than and (up_to is None or count <= up_to)]
        starts = [sum(counts[:i]) for i in range(requests)]
        seen = set()
        for request, token, head, columns in work.tolist():
            assert request in chosen and 0 < columns <= per_item and 0 <= head < per_token
            for column in range(columns):
                at = (token - starts[request]) * per_token + head + column
                assert 0 <= at < counts[request] * per_token and (request, at) not in seen
                seen.add((request, at))
        assert len(seen) == sum(counts[i] * per_token for i in chosen)
        assert steps >= 0
        padded_tokens = sum(counts) + draw.randint(0, 64)
        assert len(work) <= HipKernels._work_capacity((padded_tokens, requests + draw.randint(0, 3)), group, column_tiles, packed)
