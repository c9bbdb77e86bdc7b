"""Each kernel alone against a plain float32 reference of the same operation, at sizes
other than the tiny models': widths and vocabularies that are no power of two, head sizes
in steps of 16, odd numbers of heads and groups, pages of several sizes, shuffled pages."""

from __future__ import annotations

import contextlib
import math
import types

import pytest
import torch
import torch.nn.functional as F

from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOLERANCE = {torch.float32: dict(atol=2e-5, rtol=2e-5), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}


@pytest.fixture(scope="module")
def kernels():
    from llmserve_amd.kernels import HipKernels

    return {dtype: HipKernels(dtype) for dtype in DTYPES}


@pytest.fixture(scope="module")
def own_kernels():
    """The library with every product on the hand-written kernels (none sent to the BLAS library)."""
    from llmserve_amd.kernels import HipKernels

    return HipKernels(torch.bfloat16, library_products=False)


def on_gpu(tensor, dtype=None):
    return tensor.to("cuda", dtype) if dtype else tensor.to("cuda")


def rounded(tensor, dtype):
    """What the kernel sees: the reference's inputs rounded to the run dtype."""
    return tensor.to(dtype).double()


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(kernels, dtype):
    table = torch.randn(301, 72)
    ids = torch.tensor([0, 300, 17, 17, 5], dtype=torch.int32)
    out = kernels[dtype].embedding(on_gpu(table, dtype), on_gpu(ids))
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.cpu().double(), rounded(table, dtype)[ids.long()], atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,eps", [(72, 1e-6), (1000, 1e-2), (4099, 1e-5)])
def test_add_rms_norm(kernels, dtype, width, eps):
    hidden, delta = torch.randn(7, width), 0.3 * torch.randn(7, width)
    weight = 1 + 0.2 * torch.randn(width)
    for weight_dtype in (dtype, torch.float32):
        device_hidden = on_gpu(hidden.clone())
        out = kernels[dtype].add_rms_norm(device_hidden, on_gpu(delta), on_gpu(weight, weight_dtype), eps)
        summed = hidden.double() + delta.double()
        torch.testing.assert_close(device_hidden.cpu().double(), summed, atol=1e-6, rtol=1e-6)
        expected = plain.rms_norm(summed, rounded(weight, weight_dtype), eps)
        assert out.dtype == dtype
        torch.testing.assert_close(out.cpu().double(), expected, **TOLERANCE[dtype])
    alone = kernels[dtype].add_rms_norm(on_gpu(hidden.clone()), None, on_gpu(weight, dtype), eps)
    torch.testing.assert_close(alone.cpu().double(), plain.rms_norm(hidden.double(), rounded(weight, dtype), eps), **TOLERANCE[dtype])
    small = 1e-4 * hidden  # eps decides here
    tiny = kernels[dtype].add_rms_norm(on_gpu(small.clone()), None, on_gpu(torch.ones(width), dtype), eps)
    torch.testing.assert_close(tiny.cpu().double(), plain.rms_norm(small.double(), torch.ones(width).double(), eps), **TOLERANCE[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,inner,outer", [(1, 72, 50), (5, 200, 333), (70, 129, 65), (130, 64, 1000),
                                              (1, 256, 48), (8, 1536, 272), (16, 96, 1000), (17, 1184, 50), (33, 512, 24),
                                              (64, 4480, 130), (64, 160, 2048),
                                              # up to 16 rows with two or four weight tiles a wave: a long K, all 16 rows, a vocabulary-sized N
                                              (8, 4096, 8192), (13, 512, 16400), (5, 1536, 66000)])
def test_linear_and_gated_linear(kernels, dtype, rows, inner, outer):
    k = kernels[dtype]
    # weights scaled so that every output is of order one, whatever `inner` is
    x, w, b = torch.randn(rows, inner), torch.randn(outer, inner) / math.sqrt(inner), torch.randn(outer)
    expected = rounded(x, dtype) @ rounded(w, dtype).T + rounded(b, dtype)
    parts = [w[: outer // 3], w[outer // 3 :]], [b[: outer // 3], b[outer // 3 :]]
    handle = k.prepare_linear([on_gpu(p, dtype) for p in parts[0]], [on_gpu(p, dtype) for p in parts[1]])
    for out_dtype in (None, torch.float32):
        out = k.linear(on_gpu(x, dtype), handle, out_dtype=out_dtype)
        assert out.dtype == (out_dtype or dtype)
        tolerance = TOLERANCE[dtype] if out_dtype is None else dict(atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(out.cpu().double(), expected, **tolerance)
    no_bias = k.linear(on_gpu(x, dtype), k.prepare_linear([on_gpu(w, dtype)], None), out_dtype=torch.float32)
    torch.testing.assert_close(no_bias.cpu().double(), expected - rounded(b, dtype), atol=1e-4, rtol=1e-4)
    # a weight kept in 32-bit under a bfloat16 run
    wide = k.linear(on_gpu(x, dtype), k.prepare_linear([on_gpu(w)], None), out_dtype=torch.float32)
    torch.testing.assert_close(wide.cpu().double(), rounded(x, dtype) @ w.double().T, atol=1e-4, rtol=1e-4)
    up = torch.randn(outer, inner) / math.sqrt(inner)
    gated = k.gated_linear(on_gpu(x, dtype), k.prepare_gated_linear(on_gpu(w, dtype), on_gpu(up, dtype)))
    want = F.silu(rounded(x, dtype) @ rounded(w, dtype).T) * (rounded(x, dtype) @ rounded(up, dtype).T)
    torch.testing.assert_close(gated.cpu().double(), want, **TOLERANCE[dtype])


@pytest.mark.parametrize("rows,inner,outer", [(17, 128, 64), (32, 256, 100), (33, 1536, 272), (64, 1280, 130), (64, 8960, 48),
                                              (40, 96, 77), (64, 160, 2048), (100, 256, 40), (65, 32, 128), (130, 1536, 272),
                                              (300, 96, 1000), (2048, 512, 384), (129, 129, 50), (2000, 64, 6500), (2048, 2048, 1500),
                                              (1100, 2048, 700), (2048, 416, 6400), (1000, 160, 12900), (2040, 96, 6401), (8, 18944, 3584)])
def test_products_without_the_library(own_kernels, rows, inner, outer):
    """17 to 64 rows: the kernel that shares x through LDS (K a multiple of 128), else the
    weight-streaming one with several tiles of x; more rows: the tiled one (K a multiple of 32; its
    256 x 256 tiles where there are 200 of them, with K steps that are and are not a multiple of its
    four stages, K cut into partial sums where a float32 result may stay in parts); else the generic one."""
    k, dtype = own_kernels, torch.bfloat16
    x, w, b = torch.randn(rows, inner), torch.randn(outer, inner) / math.sqrt(inner), torch.randn(outer)
    expected = rounded(x, dtype) @ rounded(w, dtype).T + rounded(b, dtype)
    handle = k.prepare_linear([on_gpu(w, dtype)], [on_gpu(b, dtype)])
    torch.testing.assert_close(k.linear(on_gpu(x, dtype), handle).cpu().double(), expected, **TOLERANCE[dtype])
    parts = k.linear(on_gpu(x, dtype), handle, out_dtype=torch.float32, partial=True)
    summed = parts if parts.ndim == 2 else parts.sum(0)
    torch.testing.assert_close(summed.cpu().double(), expected, atol=1e-4, rtol=1e-4)
    up = torch.randn(outer, inner) / math.sqrt(inner)
    gated = k.gated_linear(on_gpu(x, dtype), k.prepare_gated_linear(on_gpu(w, dtype), on_gpu(up, dtype)))
    want = F.silu(rounded(x, dtype) @ rounded(w, dtype).T) * (rounded(x, dtype) @ rounded(up, dtype).T)
    torch.testing.assert_close(gated.cpu().double(), want, **TOLERANCE[dtype])


def key_pieces(rows):
    """Key pages written as rows [pages, kv, offset, dim] -> as the cache keeps them, in pieces of eight
    elements, the same piece of all the keys of a page side by side: [pages, kv, dim / w, offset, w]
    (a head size that is no multiple of 8 is one piece)."""
    pages, kv, page, dim = rows.shape
    width = 8 if dim % 8 == 0 else dim
    return rows.view(pages, kv, page, dim // width, width).permute(0, 1, 3, 2, 4).contiguous()


def key_rows(pieces):
    """The inverse of `key_pieces`."""
    pages, kv, count, page, width = pieces.shape
    return pieces.permute(0, 1, 3, 2, 4).reshape(pages, kv, page, count * width)


def value_pieces(rows):
    """Value pages written transposed [pages, kv, dim, page] -> as the cache keeps them, in pieces of eight keys,
    the same piece of all dimensions side by side: [pages, kv, page / v, dim, v] (a page size that is no
    multiple of 8 is one piece)."""
    pages, kv, dim, page = rows.shape
    width = 8 if page % 8 == 0 else page
    return rows.view(pages, kv, dim, page // width, width).permute(0, 1, 3, 2, 4).contiguous()


def value_rows(pieces):
    """The inverse of `value_pieces`."""
    pages, kv, count, dim, width = pieces.shape
    return pieces.permute(0, 1, 3, 2, 4).reshape(pages, kv, dim, count * width)


def paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=0, spare_pages=3):
    """Requests with `lengths[i]` cached tokens of which the last `counts[i]` are this step's.
    Returns the step's batch, the cell with garbage in every unused slot, and per-request q, k, v."""
    from llmserve_amd.cache import CacheCell
    from llmserve_amd.engine.batch import GroupBatch, SequenceChunk, StepBatch
    from llmserve_amd.parts import HeadLayout, PagedKeyValue

    generator = torch.Generator().manual_seed(shuffle_seed)
    blocks = [math.ceil(n / page) for n in lengths]
    pages = sum(blocks) + spare_pages
    order = torch.randperm(pages, generator=generator).tolist()
    width = max(blocks)
    tables = torch.full((len(lengths), width), -1, dtype=torch.int32)
    keys = torch.full((pages, kv_heads, page, dim), float("nan"))
    values = torch.full((pages, kv_heads, dim, page), float("nan"))  # value pages are stored transposed
    per_request, slot_mapping, positions, token_sequence, chunks = [], [], [], [], []
    for index, (length, count) in enumerate(zip(lengths, counts)):
        mine = [order.pop() for _ in range(blocks[index])]
        tables[index, : len(mine)] = torch.tensor(mine, dtype=torch.int32)
        q = torch.randn(length, heads, dim, generator=generator)
        k = torch.randn(length, kv_heads, dim, generator=generator)
        v = torch.randn(length, kv_heads, dim, generator=generator)
        per_request.append((q, k, v))
        for position in range(length):
            keys[mine[position // page], :, position % page] = k[position]
            values[mine[position // page], :, :, position % page] = v[position]
        for position in range(length - count, length):
            slot_mapping.append(mine[position // page] * page + position % page)
            positions.append(position)
            token_sequence.append(index)
        chunks.append(SequenceChunk(f"r{index}", index, length - count, count))
    starts = [0]
    for count in counts:
        starts.append(starts[-1] + count)
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    group = GroupBatch(page, tables.cuda(), ints(slot_mapping), width)
    batch = StepBatch(
        num_tokens=sum(counts), chunks=chunks, token_ids=ints([0] * sum(counts)), positions=ints(positions),
        token_sequence=ints(token_sequence), query_start=ints(starts), context_lengths=ints(lengths),
        state_slots=ints(list(range(len(lengths)))), groups=[group], logit_rows=ints([]), num_logit_rows=0,
        max_query_length=max(counts), max_context_length=max(lengths),
    )
    cell = CacheCell(PagedKeyValue(kv_heads, dim), True, 0, key_pieces(keys).to("cuda", dtype), value_pieces(values).to("cuda", dtype))
    return batch, cell, per_request, HeadLayout(heads, kv_heads, dim)


def step_rows(per_request, counts, heads, kv_heads, dim):
    """The step's qkv rows [T, (heads + 2 kv) * dim] from the per-request tensors."""
    rows = []
    for (q, k, v), count in zip(per_request, counts):
        rows.append(torch.cat([q[-count:].flatten(1), k[-count:].flatten(1), v[-count:].flatten(1)], dim=1))
    return torch.cat(rows)


ATTENTION_SHAPES = [  # heads, kv_heads, dim, page
    (12, 2, 32, 16),  # the reference's own test shape (tests/test_triton_paged_attention.py:24)
    (6, 1, 48, 8),
    (5, 5, 80, 24),  # a page that is no power of two
    (8, 2, 128, 16),
    (3, 1, 112, 64),
    (4, 2, 256, 16),  # the widest head the matrix-core kernel takes: one column tile a wave
    (4, 4, 16, 1),
    (40, 8, 128, 16),  # the 32B sizes: five query heads a kv head
    (10, 2, 128, 16),
    (28, 4, 128, 16),  # the 7B sizes: seven
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,page", ATTENTION_SHAPES)
def test_paged_attention_at_page_edges(kernels, dtype, heads, kv_heads, dim, page):
    """Lengths around page edges (the reference's 1, 15, 16, 17, 31, 32, 33, scaled to the page),
    single decoded tokens beside portions, shuffled pages, garbage in unused slots."""
    lengths = [1, page - 1 or 1, page, page + 1, 2 * page - 1, 2 * page, 2 * page + 1, 5 * page + 3, 150]
    counts = [1, 1, page, 1, 3, 2 * page, 1, 2 * page + 2, 1]
    counts = [min(count, length) for count, length in zip(counts, lengths)]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=dim)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    scale = 0.37
    out = kernels[dtype].paged_attention(qkv, layout, batch, cell, scale, None).cpu().double()
    expected = []
    for (q, k, v), count in zip(per_request, counts):
        full = plain.causal_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale)
        expected.append(full[-count:].flatten(1))
    torch.testing.assert_close(out, torch.cat(expected), **TOLERANCE[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 5, 16, 17, 40])
def test_paged_attention_window_edge(kernels, dtype, window):
    """One key far back is made to stand out: it must count exactly while it is inside the window."""
    heads, kv_heads, dim, page = 4, 2, 32, 8
    lengths, counts = [70, 41], [30, 1]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=window)
    for q, k, v in per_request:  # the key at the window's far edge of the last query dominates its scores
        edge = q.shape[0] - window
        if edge >= 0:
            k[edge] = 4.0 * q[-1, ::2]
    batch, cell, _, _ = _rewrite_cell(batch, cell, per_request, page, dtype)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    out = kernels[dtype].paged_attention(qkv, layout, batch, cell, 0.25, window).cpu().double()
    expected = []
    for (q, k, v), count in zip(per_request, counts):
        full = plain.causal_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), 0.25, window)
        expected.append(full[-count:].flatten(1))
    torch.testing.assert_close(out, torch.cat(expected), **TOLERANCE[dtype])
    wider = kernels[dtype].paged_attention(qkv, layout, batch, cell, 0.25, window + 1).cpu().double()
    assert not torch.allclose(wider, out, atol=1e-2)


def _rewrite_cell(batch, cell, per_request, page, dtype):
    keys, values = key_rows(cell.keys.cpu().float()), value_rows(cell.values.cpu().float())
    tables = batch.groups[0].block_tables.cpu()
    for index, (q, k, v) in enumerate(per_request):
        for position in range(k.shape[0]):
            keys[tables[index, position // page], :, position % page] = k[position]
            values[tables[index, position // page], :, :, position % page] = v[position]
    cell.keys, cell.values = key_pieces(keys).to("cuda", dtype), value_pieces(values).to("cuda", dtype)
    return batch, cell, per_request, None


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_finds_a_far_key_among_hundreds(kernels, dtype):
    heads, kv_heads, dim, page = 6, 2, 64, 16
    lengths, counts = [700], [1]
    for far in (0, 15, 16, 337, 698):
        batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=far)
        q, k, v = per_request[0]
        k[far] = 3.0 * q[-1, ::3]  # for heads 0 and 3 this key dominates; v[far] must come out
        _rewrite_cell(batch, cell, per_request, page, dtype)
        qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
        out = kernels[dtype].paged_attention(qkv, layout, batch, cell, 1.0, None).cpu().double().view(heads, dim)
        full = plain.causal_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), 1.0)[-1]
        torch.testing.assert_close(out, full, **TOLERANCE[dtype])
        torch.testing.assert_close(out[0], rounded(v, dtype)[far, 0], atol=5e-2, rtol=0)


@pytest.mark.parametrize("splits", [1, 3])
@pytest.mark.parametrize("window", [None, 21, 64])
@pytest.mark.parametrize("heads,kv_heads,page", [(12, 2, 16), (28, 4, 8), (40, 2, 16), (5, 5, 24), (3, 1, 32), (40, 8, 16), (10, 2, 16), (12, 2, 64), (7, 1, 128)])
def test_prompt_portions_that_share_keys_through_lds(heads, kv_heads, page, window, splits):
    """At head size 128 prompt portions may go to the kernel whose four waves share each step's K and V
    through LDS (pages of a power of two from 16 keys on; the others stay with the kernel above): portions that
    fill its workgroups, that leave waves empty, that end inside a step of 32 keys and that begin long after the
    sequence's start, with and without a window, whole or in three runs of keys that a second kernel merges
    (some of them empty: a request of five keys has one step)."""
    from llmserve_amd.kernels import HipKernels

    dim, dtype = 128, torch.bfloat16
    shared = HipKernels(dtype, shared_portions="always")
    shared.portion_splits = splits
    apart = HipKernels(dtype, shared_portions="never")
    lengths = [130, 97, 33, 300, 64, 5]
    counts = [130, 40, 33, 70, 17, 3]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=heads)
    if window:
        # blocks that the window has passed are given back in the engine: here their table entries name a page
        # nobody wrote (all NaN), which a kernel that looked there would carry into its sums
        tables = batch.groups[0].block_tables.cpu()
        unwritten = int(torch.isnan(cell.keys.float()).flatten(1).all(dim=1).nonzero()[0])
        for index, (length, count) in enumerate(zip(lengths, counts)):
            tables[index, : max(0, length - count - window + 1) // page] = unwritten
        batch.groups[0].block_tables.copy_(tables)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    scale = 0.11
    out = shared.paged_attention(qkv, layout, batch, cell, scale, window).cpu().double()
    expected = []
    for (q, k, v), count in zip(per_request, counts):
        full = plain.causal_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale, window)
        expected.append(full[-count:].flatten(1))
    torch.testing.assert_close(out, torch.cat(expected), **TOLERANCE[dtype])
    other = apart.paged_attention(qkv, layout, batch, cell, scale, window).cpu().double()
    torch.testing.assert_close(out, other, **TOLERANCE[dtype])


@pytest.mark.parametrize("heads,kv_heads", [(12, 2), (40, 2), (7, 7)])
def test_decoded_tokens_beside_portions_that_share_keys_through_lds(heads, kv_heads):
    """A step of long portions beside single decoded tokens over long contexts: the portions go to the kernel
    that shares K and V through LDS, the decoded tokens to a launch of their own whose keys are cut into runs
    (partial results kept by work item, merged for those rows only); a far key dominates one decoded token."""
    from llmserve_amd.kernels import HipKernels

    dim, page, dtype = 128, 16, torch.bfloat16
    shared = HipKernels(dtype, shared_portions="always")
    lengths, counts = [3100, 4200, 600, 2500, 90], [1, 600, 300, 1, 1]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=5)
    q, k, v = per_request[0]
    k[40] = 3.0 * q[-1, :: heads // kv_heads]  # for the first query head of every kv head this key dominates
    _rewrite_cell(batch, cell, per_request, page, dtype)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    out = shared.paged_attention(qkv, layout, batch, cell, 1.0, None).cpu().double()
    expected = []
    for (q, k, v), count in zip(per_request, counts):
        full = plain.causal_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), 1.0, None)
        expected.append(full[-count:].flatten(1))
    torch.testing.assert_close(out, torch.cat(expected), **TOLERANCE[dtype])
    torch.testing.assert_close(out[0].view(heads, dim)[0], rounded(per_request[0][2], dtype)[40, 0], atol=5e-2, rtol=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("window", [None, 1500])
def test_paged_attention_portion_of_a_long_context(kernels, window, dtype):
    """A portion at the end of a context of more than 4,096 keys (hundreds of steps a wave, many
    pages; in float32 the keys are cut into splits that a second kernel merges), with a far key that
    dominates and, with a window, lies just inside it."""
    heads, kv_heads, dim, page = 6, 2, 64, 16
    lengths, counts = [4200, 37], [150, 37]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=3)
    q, k, v = per_request[0]
    far = 4199 - 1499 if window else 1
    k[far] = 3.0 * q[-1, ::3]  # for heads 0 and 3 of the last query this key dominates
    _rewrite_cell(batch, cell, per_request, page, dtype)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    out = kernels[dtype].paged_attention(qkv, layout, batch, cell, 1.0, window).cpu().double()
    expected = []
    for (q, k, v), count in zip(per_request, counts):
        full = plain.causal_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), 1.0, window)
        expected.append(full[-count:].flatten(1))
    torch.testing.assert_close(out, torch.cat(expected), **TOLERANCE[dtype])
    torch.testing.assert_close(out[149].view(heads, dim)[0], rounded(per_request[0][2], dtype)[far, 0], atol=5e-2, rtol=0)


@pytest.mark.parametrize("window", [None, 3000])
def test_float32_decode_attention_over_many_key_splits(kernels, window):
    """Two requests decode over 9,000 and 5,003 keys in float32: few items, so each is cut into several key
    splits (some of them empty for the shorter request, some wholly outside the window) that the merging
    kernel adds up; a far key per request dominates one head."""
    heads, kv_heads, dim, page, dtype = 10, 2, 128, 16, torch.float32
    lengths, counts = [9000, 5003], [1, 1]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=11)
    fars = [6500, 2100]
    for (q, k, v), far in zip(per_request, fars):
        k[far] = 2.0 * q[-1, ::5]  # heads 0 and 5 share kv heads 0 and 1
    _rewrite_cell(batch, cell, per_request, page, dtype)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    out = kernels[dtype].paged_attention(qkv, layout, batch, cell, 0.5, window).cpu().double()
    for row, ((q, k, v), far) in enumerate(zip(per_request, fars)):
        full = plain.causal_attention(q.double(), k.double(), v.double(), 0.5, window)[-1]
        torch.testing.assert_close(out[row].view(heads, dim), full, **TOLERANCE[dtype])
        torch.testing.assert_close(out[row].view(heads, dim)[0], v.double()[far, 0], atol=5e-2, rtol=0)


@pytest.mark.parametrize("rows,inner,outer", [(3, 100, 77), (8, 8960, 1536), (16, 1536, 48), (11, 2052, 130),
                                              (40, 8960, 200), (200, 4480, 130), (130, 100, 77), (2048, 264, 384),
                                              (129, 2048, 1030)])
def test_float32_products_in_parts_and_at_odd_sizes(kernels, rows, inner, outer):
    """The 32-bit path's products on the matrix cores: K that is a multiple of 4 but not of 16 or 64, rows and
    weight rows that fill no tile, and K cut into partial sums where the result may stay in parts (up to 16 rows:
    the weight-streaming kernel; more: the tiled one), with bias, and with SiLU(gate) * up over interleaved rows.
    The bound is that of a float32 sum of K terms in any order: a few times sqrt(K) * 2^-24 of its size."""
    k = kernels[torch.float32]
    x, w, b = torch.randn(rows, inner), torch.randn(outer, inner) / math.sqrt(inner), torch.randn(outer)
    expected = x.double() @ w.double().T + b.double()
    bound = dict(atol=8 * math.sqrt(inner) * 2.0 ** -24, rtol=1e-5)
    handle = k.prepare_linear([on_gpu(w)], [on_gpu(b)])
    torch.testing.assert_close(k.linear(on_gpu(x), handle).cpu().double(), expected, **bound)
    parts = k.linear(on_gpu(x), handle, out_dtype=torch.float32, partial=True)
    cut = k._float32_splits(rows, outer, inner)
    assert parts.shape == ((cut, rows, outer) if cut > 1 else (rows, outer)) and (cut > 1 or inner < 2048 or rows > 200 or outer > 1000)
    summed = parts if parts.ndim == 2 else parts.double().sum(0)
    torch.testing.assert_close(summed.cpu().double(), expected, **bound)
    up = torch.randn(outer, inner) / math.sqrt(inner)
    gated = k.gated_linear(on_gpu(x), k.prepare_gated_linear(on_gpu(w), on_gpu(up)))
    want = F.silu(x.double() @ w.double().T) * (x.double() @ up.double().T)
    torch.testing.assert_close(gated.cpu().double(), want, **bound)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pairing", ["adjacent", "half", "none"])
@pytest.mark.parametrize("heads,kv_heads,dim,page", [(6, 2, 32, 8), (5, 1, 48, 16), (2, 2, 128, 4)])
def test_rotate_and_store(kernels, dtype, pairing, heads, kv_heads, dim, page):
    lengths, counts = [9, 40, 1], [9, 3, 1]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype)
    before_keys, before_values = cell.keys.clone(), cell.values.clone()
    rows = step_rows(per_request, counts, heads, kv_heads, dim)
    qkv = on_gpu(rows, dtype)
    theta = 5000.0
    inverse = 1.0 / (theta ** (torch.arange(0, dim, 2).float() / dim))
    kernels[dtype].rotate_and_store(qkv, layout, batch, cell, None if pairing == "none" else on_gpu(inverse), pairing)
    positions = batch.positions.cpu().long()
    view = rounded(rows, dtype).view(-1, heads + 2 * kv_heads, dim)
    angles = plain.rope_angles(dim, theta, positions)
    rotate = {"adjacent": plain.rope_adjacent, "half": plain.rope_half, "none": lambda x, a: x}[pairing]
    expected = torch.cat([rotate(view[:, : heads + kv_heads], angles), view[:, heads + kv_heads :]], dim=1)
    torch.testing.assert_close(qkv.cpu().double().view_as(expected), expected, **TOLERANCE[dtype])
    slots = batch.groups[0].slot_mapping.cpu().long()
    stored_k = key_rows(cell.keys.cpu().double())[slots // page, :, slots % page]
    stored_v = value_rows(cell.values.cpu().double())[slots // page, :, :, slots % page]
    torch.testing.assert_close(stored_k, expected[:, heads : heads + kv_heads], **TOLERANCE[dtype])
    torch.testing.assert_close(stored_v, expected[:, heads + kv_heads :], atol=0, rtol=0)
    untouched = torch.ones(cell.keys.shape[0], page, dtype=torch.bool)
    untouched[slots // page, slots % page] = False
    same = lambda a, b: torch.equal(torch.nan_to_num(a.float().cpu(), nan=7.0), torch.nan_to_num(b.float().cpu(), nan=7.0))
    assert same(key_rows(cell.keys).transpose(1, 2)[untouched], key_rows(before_keys).transpose(1, 2)[untouched])
    assert same(value_rows(cell.values).permute(0, 3, 1, 2)[untouched], value_rows(before_values).permute(0, 3, 1, 2)[untouched])
    # a cell that is only read stores nothing
    readonly = types.SimpleNamespace(writable=False)
    again = on_gpu(rows, dtype)
    kernels[dtype].rotate_and_store(again, layout, batch, readonly, None if pairing == "none" else on_gpu(inverse), pairing)
    torch.testing.assert_close(again, qkv)


@pytest.mark.parametrize("width,parts", [(64, 1), (1536, 3), (4096, 8), (5120, 11), (12292, 2), (16384, 17), (4102, 9)])
def test_add_rms_norm_of_partial_sums(kernels, width, parts):
    """What a product cut over K leaves: [parts, rows, width] partial sums, added in order.  Widths
    with one, two and four pieces a thread, the widest the register-resident kernel takes, and one
    that is no multiple of four (the plain kernel)."""
    rows = 5
    hidden, delta = torch.randn(rows, width), 0.3 * torch.randn(parts, rows, width)
    weight = 1 + 0.2 * torch.randn(width)
    k = kernels[torch.bfloat16]
    device_hidden = on_gpu(hidden.clone())
    out = k.add_rms_norm(device_hidden, on_gpu(delta), on_gpu(weight, torch.bfloat16), 1e-6)
    summed = hidden.double() + delta.double().sum(0)
    torch.testing.assert_close(device_hidden.cpu().double(), summed, atol=2e-6, rtol=1e-6)
    expected = plain.rms_norm(summed, rounded(weight, torch.bfloat16), 1e-6)
    torch.testing.assert_close(out.cpu().double(), expected, **TOLERANCE[torch.bfloat16])
    # a row's result does not depend on how many rows there are
    one = on_gpu(hidden[2:3].clone())
    alone = k.add_rms_norm(one, on_gpu(delta[:, 2:3].contiguous()), on_gpu(weight, torch.bfloat16), 1e-6)
    assert torch.equal(alone[0], out[2]) and torch.equal(one[0], device_hidden[2])


@pytest.mark.parametrize("dtype", DTYPES)
def test_gather_rows(kernels, dtype):
    hidden, delta = torch.randn(9, 100), torch.randn(9, 100)
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32)
    out = kernels[dtype].gather_rows(on_gpu(hidden), on_gpu(delta), on_gpu(rows))
    torch.testing.assert_close(out.cpu(), (hidden + delta)[rows.long()])
    torch.testing.assert_close(kernels[dtype].gather_rows(on_gpu(hidden), None, on_gpu(rows)).cpu(), hidden[rows.long()])


@pytest.mark.parametrize("vocab", [5, 1000, 1025, 151936])
def test_argmax_and_sampling(kernels, vocab):
    k = kernels[torch.float32]
    torch.manual_seed(vocab)
    rows = 6
    logits = 3.0 * torch.randn(rows, vocab)
    logits[1, vocab // 2] = logits[1].max() + 1
    logits[2, [3, vocab - 1]] = 50.0  # a tie: the first wins
    assert k.argmax(on_gpu(logits)).cpu().tolist() == logits.argmax(-1).tolist()
    assert k.argmax(on_gpu(logits)).cpu().tolist()[2] == 3
    cases = [(0.0, 1.0), (0.8, 1.0), (0.7, 0.8), (1.5, 0.3), (0.2, 0.95), (1.0, 1.0)]
    for draw in range(12):
        uniforms = [plain.uniform_for(draw, row) for row in range(rows)]
        got = k.sample(
            on_gpu(logits), on_gpu(torch.tensor([c[0] for c in cases])), on_gpu(torch.tensor([c[1] for c in cases])),
            on_gpu(torch.tensor(uniforms)),
        ).cpu().tolist()
        want = [plain.sample(logits[row], cases[row][0], cases[row][1], uniforms[row]) for row in range(rows)]
        assert got == want, (draw, got, want)


def test_sampling_edges(kernels):
    k = kernels[torch.float32]
    logits = torch.tensor([[0.0, 0.0, 0.0, 0.0], [5.0, 1.0, 5.0, 5.0], [1.0, 2.0, 3.0, 4.0]])
    for u, want in ((0.0, [0, 0, 0]), (0.26, [1, 0, 0]), (0.9999, [3, 3, 3])):
        got = k.sample(on_gpu(logits), on_gpu(torch.full((3,), 1.0)), on_gpu(torch.ones(3)), on_gpu(torch.full((3,), u))).cpu().tolist()
        assert got[0] == want[0] and got[2] == plain.sample(logits[2], 1.0, 1.0, u)
    # top-p with ties: equal entries are kept in index order until the mass is reached
    for u in (0.0, 0.3, 0.4, 0.7, 0.99):
        got = k.sample(on_gpu(logits), on_gpu(torch.full((3,), 1.0)), on_gpu(torch.full((3,), 0.6)), on_gpu(torch.full((3,), u))).cpu().tolist()
        want = [plain.sample(logits[row], 1.0, 0.6, u) for row in range(3)]
        assert got == want, (u, got, want)


def test_sampling_refuses_a_workspace_that_is_too_small(kernels):
    from llmserve_amd.kernels.hip import _pointer

    k = kernels[torch.float32]
    library = k._sampling_library()
    rows, vocab = 5, 1000
    kib = library.llmserve_sample_workspace_kib(rows, vocab)
    assert kib > rows * vocab * 4 // 1024 and library.llmserve_sample_workspace_kib(0, vocab) < 0
    logits, values, out = torch.randn(rows, vocab).cuda(), torch.full((rows,), 0.5).cuda(), torch.zeros(rows, dtype=torch.int32).cuda()
    workspace = torch.empty(kib * 1024, dtype=torch.uint8, device="cuda")
    arguments = lambda space, size: (_pointer(logits), _pointer(values), _pointer(values), _pointer(values), space, size, _pointer(out), rows, vocab, 1, k._stream)
    assert library.llmserve_sample(*arguments(_pointer(workspace), kib - 1)) == 1001
    assert library.llmserve_sample(*arguments(None, kib)) == 1001
    assert library.llmserve_sample(*arguments(_pointer(workspace) + 16, kib)) == 1001  # not aligned to 256 bytes
    assert library.llmserve_sample(*arguments(_pointer(workspace), kib)) == 0
    torch.cuda.synchronize()
    assert all(0 <= token < vocab for token in out.cpu().tolist())


@pytest.mark.parametrize("rows,vocab", [(70, 1025), (300, 130), (3, 40000)])
def test_sampling_of_many_rows_and_hard_rows(kernels, rows, vocab):
    """The stages cut a row into fewer pieces when there are many rows; rows whose entries are all
    equal, tie in groups, underflow to zero or to subnormal numbers, or hold one entry far above the
    rest must come out as the plain rule says; and leaving the top-p stages out changes nothing for
    rows without top-p."""
    k = kernels[torch.float32]
    torch.manual_seed(rows + vocab)
    logits = 2.0 * torch.randn(rows, vocab)
    # all equal, as many as a power of two (the plain rule rounds p = 1 / n to float32 before it adds, the kernel
    # divides nothing: with every entry tied they agree only where 1 / n is exact); the rest can never come
    equal = 1 << (vocab.bit_length() - 1)
    logits[0] = 1.5
    logits[0, equal:] = -float("inf")
    if vocab <= 2048:
        # four values, many ties.  Not at the large size: float32 softmax, which the plain rule starts from, is
        # off from a sum of 1 by a few parts in a million there, and among ten thousand tied entries that
        # moves the end of the kept set by an entry; the kernel normalises nothing and has no such error
        logits[1] = torch.randint(0, 4, (vocab,)).float()
    logits[2, 1:] -= 200.0  # everything but one entry underflows
    logits[2, 0] = 3.0
    if rows > 3:
        logits[3] = torch.linspace(-180.0, 0.0, vocab)  # the low end is subnormal or zero after exp
        logits[4, vocab // 3] += 30.0
    temperatures = [(0.0, 0.6, 1.0, 1.7)[row % 4] for row in range(rows)]
    temperatures[0], temperatures[1], temperatures[2] = 1.0, 0.9, 1.0
    top_ps = [(1.0, 0.9, 0.5, 0.05, 0.999)[row % 5] for row in range(rows)]
    top_ps[0], top_ps[1] = 0.5, 0.7
    for draw in range(3):
        uniforms = [plain.uniform_for(draw + 20, row) for row in range(rows)]
        if draw == 2:
            uniforms[0], uniforms[1] = 0.0, 0.999999
        got = k.sample(on_gpu(logits), on_gpu(torch.tensor(temperatures)), on_gpu(torch.tensor(top_ps)), on_gpu(torch.tensor(uniforms))).cpu().tolist()
        want = [plain.sample(logits[row], temperatures[row], top_ps[row], uniforms[row]) for row in range(rows)]
        assert got == want, (draw, [(row, a, b) for row, (a, b) in enumerate(zip(got, want)) if a != b])
        ones = [1.0] * rows
        got = k.sample(on_gpu(logits), on_gpu(torch.tensor(temperatures)), on_gpu(torch.tensor(ones)), on_gpu(torch.tensor(uniforms)), False).cpu().tolist()
        want = k.sample(on_gpu(logits), on_gpu(torch.tensor(temperatures)), on_gpu(torch.tensor(ones)), on_gpu(torch.tensor(uniforms))).cpu().tolist()
        assert got == want
        assert got == [plain.sample(logits[row], temperatures[row], 1.0, uniforms[row]) for row in range(rows)]


@pytest.mark.parametrize("pairing", ["adjacent", "half", "none"])
@pytest.mark.parametrize("heads,kv_heads,dim,page", [(12, 2, 128, 16), (6, 1, 64, 8), (5, 5, 32, 4), (4, 2, 48, 16), (40, 2, 64, 16), (2, 1, 256, 16), (40, 8, 128, 16), (10, 2, 128, 16), (28, 4, 128, 16)])
def test_fused_decode_attention(kernels, pairing, heads, kv_heads, dim, page):
    """A step of single tokens: rotation, the store of the new key and value, attention and the
    merge of key splits in one kernel (or, where the sizes do not allow it, in the separate ones):
    the result and the pages must be what the separate steps give."""
    dtype = torch.bfloat16
    lengths = [1, 2, page, page + 1, 33, 64, 65, 700, 301]
    counts = [1] * len(lengths)
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=dim + page)
    theta = 800.0
    inverse = 1.0 / (theta ** (torch.arange(0, dim, 2).float() / dim))
    rotate = {"adjacent": plain.rope_adjacent, "half": plain.rope_half, "none": lambda x, a: x}[pairing]
    # the pages hold the earlier tokens' keys already rotated; the new token's slot holds garbage
    expected = []
    for index, (q, k, v) in enumerate(per_request):
        angles = plain.rope_angles(dim, theta, torch.arange(q.shape[0]))
        k_rot = rotate(rounded(k, dtype), angles).to(dtype).double()
        q_rot = rotate(rounded(q, dtype), angles).to(dtype).double()
        per_request[index] = (q, k_rot.float(), v)
        full = plain.causal_attention(q_rot, k_rot, rounded(v, dtype), 0.2)
        expected.append(full[-1:].flatten(1))
    _rewrite_cell(batch, cell, per_request, page, dtype)
    slots = batch.groups[0].slot_mapping.cpu().long()
    cell.keys[slots // page, :, :, slots % page] = float("nan")
    cell.put_value_rows(slots // page, slots % page, torch.full((len(slots), cell.values.shape[1], cell.values.shape[3]), float("nan"), device=cell.values.device))
    rows = []  # the step's rows carry unrotated q and k
    for (q, k, v), original in zip(per_request, [p[1] for p in paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=dim + page)[2]]):
        rows.append(torch.cat([q[-1:].flatten(1), original[-1:].flatten(1), v[-1:].flatten(1)], dim=1))
    qkv = on_gpu(torch.cat(rows), dtype)
    out = kernels[dtype].rotate_store_attend(qkv, layout, batch, cell, None if pairing == "none" else on_gpu(inverse), pairing, 0.2, None)
    torch.testing.assert_close(out.cpu().double(), torch.cat(expected), **TOLERANCE[dtype])
    stored_k = key_rows(cell.keys.cpu().double())[slots // page, :, slots % page]
    stored_v = value_rows(cell.values.cpu().double())[slots // page, :, :, slots % page]
    want_k = torch.stack([p[1][-1].double() for p in per_request])
    want_v = torch.stack([rounded(p[2][-1], dtype) for p in per_request])
    torch.testing.assert_close(stored_k, want_k, **TOLERANCE[dtype])
    torch.testing.assert_close(stored_v, want_v, atol=0, rtol=0)


@pytest.mark.parametrize("requests", [3, 12])
def test_fused_decode_attention_over_long_contexts(kernels, requests):
    """Single tokens against thousands of keys: the one-kernel decode step cuts the keys over several
    workgroups and merges them.  Every request has one far key made to dominate two of its heads (the
    value stored there must come out), at a place that differs from request to request, first and
    last keys and the edges of the cuts among them; the other heads are compared with plain attention."""
    dtype, heads, kv_heads, dim, page = torch.bfloat16, 12, 2, 128, 16
    lengths = [4100, 2049, 3333] + [1500 + 37 * i for i in range(requests - 3)]
    counts = [1] * len(lengths)
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=requests)
    places = [0, 2048, 3332] + [(211 * i) % 1500 for i in range(requests - 3)]
    for (q, k, v), far in zip(per_request, places):
        k[far] = 3.0 * q[-1, ::6]  # kv head g takes the query of its first head: heads 0 and 6 find this key
    _rewrite_cell(batch, cell, per_request, page, dtype)
    slots = batch.groups[0].slot_mapping.cpu().long()
    cell.keys[slots // page, :, :, slots % page] = float("nan")  # the step itself stores the newest key and value
    cell.put_value_rows(slots // page, slots % page, torch.full((len(slots), cell.values.shape[1], cell.values.shape[3]), float("nan"), device=cell.values.device))
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    out = kernels[dtype].rotate_store_attend(qkv, layout, batch, cell, None, "none", 1.0, None).cpu().double()
    for index, ((q, k, v), far) in enumerate(zip(per_request, places)):
        full = plain.causal_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), 1.0)[-1]
        got = out[index].view(heads, dim)
        torch.testing.assert_close(got, full, **TOLERANCE[dtype])
        for head in (0, 6):
            torch.testing.assert_close(got[head], rounded(v, dtype)[far, head // 6], atol=0.05, rtol=0.05)


def test_fused_decode_attention_over_tens_of_thousands_of_keys(kernels):
    """Beyond 4,096 keys a decode step cuts the keys into five to sixty-four parts and a kernel of its own
    merges them (up to there, at up to 16 rows, the output projection does).  Two requests of 30,000 and 9,000 keys, a
    far key planted to dominate heads 0 and 6 of each (deep inside the long one, near the start of the
    other): the value stored there must come out, and every head must agree with plain attention of the
    last token over all keys."""
    dtype, heads, kv_heads, dim, page = torch.bfloat16, 12, 2, 128, 16
    lengths, counts, places = [30000, 9000] + [30000 - 100 * i for i in range(6)], [1] * 8, [23456, 100] + [29000 - 4000 * i for i in range(6)]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=30)
    for (q, k, v), far in zip(per_request, places):
        k[far] = 3.0 * q[-1, ::6]
    _rewrite_cell(batch, cell, per_request, page, dtype)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    out = kernels[dtype].rotate_store_attend(qkv, layout, batch, cell, None, "none", 1.0, None).cpu().double()
    for index, ((q, k, v), far) in enumerate(zip(per_request, places)):
        last = rounded(q, dtype)[-1]  # [heads, dim]
        all_keys = rounded(k, dtype).repeat_interleave(heads // kv_heads, dim=1)  # [T, heads, dim]
        all_values = rounded(v, dtype).repeat_interleave(heads // kv_heads, dim=1)
        weights = torch.softmax(torch.einsum("hd,thd->ht", last, all_keys), dim=-1)
        want = torch.einsum("ht,thd->hd", weights, all_values)
        got = out[index].view(heads, dim)
        torch.testing.assert_close(got, want, **TOLERANCE[dtype])
        for head in (0, 6):
            torch.testing.assert_close(got[head], rounded(v, dtype)[far, head // 6], atol=0.05, rtol=0.05)
    # Keys of zero: every key weighs the same and the result is the mean of all values, which the
    # kernel's arithmetic gives almost exactly (weights of 1, sums in float32), so that thirty-two keys
    # left out anywhere would show (a value is of order one, the mean of 30,000 of order 0.006).
    for q, k, v in per_request:
        k.zero_()
    _rewrite_cell(batch, cell, per_request, page, dtype)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    out = kernels[dtype].rotate_store_attend(qkv, layout, batch, cell, None, "none", 1.0, None).cpu().double()
    for index, (q, k, v) in enumerate(per_request):
        want = rounded(v, dtype).mean(0).repeat_interleave(heads // kv_heads, dim=0)  # [heads, dim]
        torch.testing.assert_close(out[index].view(heads, dim), want, atol=6e-5, rtol=5e-3)


@pytest.mark.parametrize("heads,kv_heads,outer,requests", [(12, 2, 1536, 8), (40, 8, 272, 16), (28, 4, 1000, 3), (2, 1, 100, 1)])
def test_decode_attention_whose_key_splits_the_output_projection_merges(kernels, heads, kv_heads, outer, requests):
    """A step of up to 16 single tokens at head size 128 followed by the output projection: the attention
    leaves its key splits unmerged and the product merges them while it loads its x.  Contexts from one
    key (all splits but one see no key) to thousands, a far key planted to dominate a head; against
    plain attention followed by the plain product, and against the library's own unfused pair."""
    from llmserve_amd.kernels import HipKernels

    dtype, dim, page = torch.bfloat16, 128, 16
    lengths = ([1, 2, 700, 33, 2049, 301, 64, 17, 4100, 530, 65, 1500, 5, 999, 129, 48])[:requests]
    counts = [1] * requests
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=heads)
    for q, k, v in per_request:
        if k.shape[0] > 40:
            k[k.shape[0] // 3] = 3.0 * q[-1, :: heads // kv_heads]  # the first head of every kv head finds this key
    _rewrite_cell(batch, cell, per_request, page, dtype)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    weight, bias = torch.randn(outer, heads * dim) / math.sqrt(heads * dim), torch.randn(outer)
    k = kernels[dtype]
    project = k.prepare_linear([on_gpu(weight, dtype)], [on_gpu(bias, dtype)])
    got = k.rotate_store_attend(qkv.clone(), layout, batch, cell, None, "none", 0.3, None, project=project)
    got = (got if got.ndim == 2 else got.sum(0)).cpu().double()
    attended = torch.cat([
        plain.causal_attention(rounded(q, dtype), rounded(key, dtype), rounded(v, dtype), 0.3)[-1:].flatten(1)
        for q, key, v in per_request
    ])
    expected = attended @ rounded(weight, dtype).T + rounded(bias, dtype)
    # the attention's output is rounded to bfloat16 on its way into the product (once, or twice where splits
    # are merged): 2^-8 of values of order 1, through a product whose weights have unit row norm
    torch.testing.assert_close(got, expected, atol=2e-2, rtol=2e-2)
    apart = HipKernels(dtype)
    apart.merge_in_product = False
    other = apart.rotate_store_attend(qkv.clone(), layout, batch, cell, None, "none", 0.3, None, project=project)
    other = (other if other.ndim == 2 else other.sum(0)).cpu().double()
    torch.testing.assert_close(got, other, atol=1e-2, rtol=1e-2)
    assert float((got - expected).abs().mean()) < 1.5 * float((other - expected).abs().mean()) + 1e-4


@pytest.mark.parametrize("rows,inner,outer", [(130, 16384, 72), (600, 8960, 200), (70, 16448, 40)])
def test_library_products_cut_over_a_long_k(kernels, rows, inner, outer):
    """A product with a long K beside few weight rows goes to the library as a strided batch over slices of K
    and comes back as partial sums for the reader to add; the sum is the product."""
    from llmserve_amd.kernels import HipKernels

    dtype = torch.bfloat16
    k = kernels[dtype]
    assert HipKernels._library_splits(rows, outer, inner) > 1
    x, w = torch.randn(rows, inner), torch.randn(outer, inner) / math.sqrt(inner)
    handle = k.prepare_linear([on_gpu(w, dtype)], None)
    parts = k.linear(on_gpu(x, dtype), handle, out_dtype=torch.float32, partial=True)
    assert parts.ndim == 3 and parts.shape[1:] == (rows, outer)
    expected = rounded(x, dtype) @ rounded(w, dtype).T
    torch.testing.assert_close(parts.sum(0).cpu().double(), expected, atol=1e-3, rtol=1e-3)
    whole = k.linear(on_gpu(x, dtype), handle, out_dtype=torch.float32)
    assert whole.ndim == 2
    torch.testing.assert_close(whole.cpu().double(), expected, atol=1e-3, rtol=1e-3)
    # the norm that follows adds the parts in order
    hidden = torch.randn(rows, outer)
    device_hidden = hidden.cuda()
    normed = k.add_rms_norm(device_hidden, parts, on_gpu(torch.ones(outer), dtype), 1e-6)
    torch.testing.assert_close(device_hidden.cpu().double(), hidden.double() + expected, atol=2e-3, rtol=1e-3)
    torch.testing.assert_close(normed.cpu().double(), plain.rms_norm(hidden.double() + expected, torch.ones(outer).double(), 1e-6), **TOLERANCE[dtype])


@pytest.mark.parametrize("rows", [1, 7, 16, 17, 40, 64])
@pytest.mark.parametrize("outer,inner,gated,splits,bias", [
    (40, 128, False, 1, None), (1000, 384, False, 1, "bfloat16"), (4610, 3584, False, 1, "float32"),  # two tiles a wave
    (154, 2560, False, 5, None), (318, 256, True, 1, None), (6000, 1536, True, 1, None),
])
def test_products_streamed_through_lds(kernels, rows, outer, inner, gated, splits, bias):
    """The product for up to 64 rows that brings weights and x through LDS, quad by quad, alone: odd
    numbers of weight rows (the last tile is cut), one and two tiles a wave, one, two and four tiles of
    x (the last one cut), a bias of either type, K cut into partial sums, SiLU(gate) * up over
    interleaved rows; against the plain product."""
    from llmserve_amd.kernels.hip import _check, _pointer

    k = kernels[torch.bfloat16]
    x, w = torch.randn(rows, inner), torch.randn(outer, inner) / math.sqrt(inner)
    b = None if bias is None else torch.randn(outer)
    device_x, device_w = on_gpu(x, torch.bfloat16), on_gpu(w, torch.bfloat16)
    device_b = None if b is None else on_gpu(b, getattr(torch, bias))
    float_out = splits > 1 or bias == "float32"
    out = torch.full((splits, rows, outer // 2 if gated else outer), float("nan"), device="cuda",
                     dtype=torch.float32 if float_out else torch.bfloat16)
    status = k._gemm_bf16.llmserve_gemm_stream(
        _pointer(device_x), _pointer(device_w), _pointer(device_b), int(bias == "float32"), _pointer(out), int(float_out),
        int(gated), rows, outer, inner, splits, k._stream,
    )
    _check(status, "gemm_stream")
    expected = rounded(x, torch.bfloat16) @ rounded(w, torch.bfloat16).T
    if b is not None:
        expected = expected + rounded(b, getattr(torch, bias))
    if gated:
        expected = torch.nn.functional.silu(expected[:, 0::2]) * expected[:, 1::2]  # weight rows alternate gate, up
    got = out.sum(0).cpu().double()
    tolerance = dict(atol=2e-3, rtol=2e-3) if float_out else TOLERANCE[torch.bfloat16]
    torch.testing.assert_close(got, expected, **tolerance)
    # and it refuses what it cannot take: more than 64 rows, a K that is no multiple of 128
    assert k._gemm_bf16.llmserve_gemm_stream(_pointer(device_x), _pointer(device_w), None, 0, _pointer(out), int(float_out),
                                             0, 65, outer, inner, 1, k._stream) != 0
    assert k._gemm_bf16.llmserve_gemm_stream(_pointer(device_x), _pointer(device_w), None, 0, _pointer(out), int(float_out),
                                             0, rows, outer, inner - 32, 1, k._stream) != 0


@pytest.mark.parametrize("rows", [24, 33, 64])
@pytest.mark.parametrize("tiles,steps", [(1, 1), (1, 2), (2, 1), (2, 2), (4, 1)])
def test_streamed_products_of_many_rows_in_every_shape(kernels, rows, tiles, steps):
    """The same kernel at 17 to 64 rows with every shape it is built in (weight tiles a workgroup, steps
    a group), plain with a bias and gated, and through the entry point that the engine's small products
    of such steps take."""
    from llmserve_amd.kernels.hip import _check, _pointer

    k = kernels[torch.bfloat16]
    outer, inner = 1210, 640
    x, w, b = torch.randn(rows, inner), torch.randn(outer, inner) / math.sqrt(inner), torch.randn(outer)
    device_x, device_w, device_b = on_gpu(x, torch.bfloat16), on_gpu(w, torch.bfloat16), on_gpu(b, torch.bfloat16)
    expected = rounded(x, torch.bfloat16) @ rounded(w, torch.bfloat16).T
    for gated in (False, True):
        want = expected + rounded(b, torch.bfloat16)
        if gated:
            want = torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2]
        out = torch.full((rows, outer // 2 if gated else outer), float("nan"), device="cuda", dtype=torch.bfloat16)
        status = k._gemm_bf16.llmserve_gemm_stream_shaped(
            _pointer(device_x), _pointer(device_w), _pointer(device_b), 0, _pointer(out), 0, int(gated), rows, outer,
            inner, 1, tiles, steps, k._stream,
        )
        _check(status, "gemm_stream_shaped")
        torch.testing.assert_close(out.cpu().double(), want, **TOLERANCE[torch.bfloat16])
    out = torch.full((rows, outer), float("nan"), device="cuda", dtype=torch.bfloat16)
    status = k._gemm_bf16.llmserve_gemm_skinny(
        _pointer(device_x), _pointer(device_w), _pointer(device_b), 0, _pointer(out), 0, 0, rows, outer, inner, 1, k._stream,
    )
    _check(status, "gemm_skinny")
    torch.testing.assert_close(out.cpu().double(), expected + rounded(b, torch.bfloat16), **TOLERANCE[torch.bfloat16])
    # and with K cut into partial sums (what the output projection of such a step asks for)
    for splits in (2, 5):
        parts = torch.full((splits, rows, outer), float("nan"), device="cuda", dtype=torch.float32)
        status = k._gemm_bf16.llmserve_gemm_skinny(
            _pointer(device_x), _pointer(device_w), None, 0, _pointer(parts), 1, 0, rows, outer, inner, splits, k._stream,
        )
        _check(status, "gemm_skinny in parts")
        torch.testing.assert_close(parts.sum(0).cpu().double(), expected, atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pairing", ["adjacent", "half"])
@pytest.mark.parametrize("heads,kv_heads,dim,page,lengths,counts", [
    (12, 2, 128, 16, [700, 301, 40, 2100], [150, 1, 40, 33]),   # portions beside a decoded token, packed columns
    (28, 4, 128, 16, [512] * 9, [512] * 9),                     # many whole prompts: the kernel that shares K and V through LDS
    (6, 1, 64, 8, [90, 17], [90, 2]),
    (40, 2, 64, 16, [130, 64], [30, 64]),                       # more than 16 query heads a kv head
    (4, 2, 48, 16, [70, 5], [70, 5]),
])
def test_rotation_store_and_attention_of_prompt_portions(kernels, dtype, pairing, heads, kv_heads, dim, page, lengths, counts):
    """`rotate_store_attend` on steps that are not single tokens (rotation and store, then attention).
    The step's rows carry unrotated q and k, the pages hold the earlier tokens' rotated keys and garbage
    where the step's will go; results and pages against the plain implementation."""
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=dim + heads)
    originals = [(q.clone(), k.clone(), v.clone()) for q, k, v in per_request]
    theta = 3000.0
    inverse = 1.0 / (theta ** (torch.arange(0, dim, 2).float() / dim))
    rotate = {"adjacent": plain.rope_adjacent, "half": plain.rope_half}[pairing]
    expected, rotated_keys = [], []
    for index, (q, k, v) in enumerate(per_request):
        angles = plain.rope_angles(dim, theta, torch.arange(q.shape[0]))
        k_rot = rotate(rounded(k, dtype), angles).to(dtype).double()
        q_rot = rotate(rounded(q, dtype), angles).to(dtype).double()
        per_request[index] = (q, k_rot.float(), v)
        rotated_keys.append(k_rot)
        full = plain.causal_attention(q_rot, k_rot, rounded(v, dtype), 0.2)
        expected.append(full[-counts[index]:].flatten(1))
    _rewrite_cell(batch, cell, per_request, page, dtype)
    slots = batch.groups[0].slot_mapping.cpu().long()
    cell.keys[slots // page, :, :, slots % page] = float("nan")  # the step stores these itself
    cell.put_value_rows(slots // page, slots % page, torch.full((len(slots), cell.values.shape[1], cell.values.shape[3]), float("nan"), device=cell.values.device))
    qkv = on_gpu(step_rows(originals, counts, heads, kv_heads, dim), dtype)
    out = kernels[dtype].rotate_store_attend(qkv, layout, batch, cell, on_gpu(inverse), pairing, 0.2, None)
    torch.testing.assert_close(out.cpu().double(), torch.cat(expected), **TOLERANCE[dtype])
    stored_k = key_rows(cell.keys.cpu().double())[slots // page, :, slots % page]
    stored_v = value_rows(cell.values.cpu().double())[slots // page, :, :, slots % page]
    want_k = torch.cat([k_rot[-count:] for k_rot, count in zip(rotated_keys, counts)])
    want_v = torch.cat([rounded(v, dtype)[-count:] for (q, k, v), count in zip(originals, counts)])
    torch.testing.assert_close(stored_k, want_k, **TOLERANCE[dtype])
    torch.testing.assert_close(stored_v, want_v, atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("activation", ["silu", "gelu", "gelu_tanh", "relu"])
@pytest.mark.parametrize("rows,inner,outer", [(5, 96, 200), (70, 64, 333), (300, 128, 1000)])
def test_gated_products_with_every_gate_activation(kernels, dtype, activation, rows, inner, outer):
    """The gate's activation is a parameter of the gated product: SiLU is applied in the products' own epilogues,
    the others by the activation kernel behind a plain product; one that has no kernel is refused by name."""
    k = kernels[dtype]
    acts = {"silu": F.silu, "gelu": F.gelu, "gelu_tanh": lambda z: F.gelu(z, approximate="tanh"), "relu": torch.relu}
    x, gate, up = torch.randn(rows, inner), torch.randn(outer, inner) / math.sqrt(inner), torch.randn(outer, inner) / math.sqrt(inner)
    weights = k.prepare_gated_linear(on_gpu(gate, dtype), on_gpu(up, dtype), activation)
    out = k.gated_linear(on_gpu(x, dtype), weights)
    want = acts[activation](rounded(x, dtype) @ rounded(gate, dtype).T) * (rounded(x, dtype) @ rounded(up, dtype).T)
    torch.testing.assert_close(out.cpu().double(), want, **TOLERANCE[dtype])
    from llmserve_amd.kernels.hip import KernelError

    with pytest.raises(KernelError, match="swish7"):
        k.prepare_gated_linear(on_gpu(gate, dtype), on_gpu(up, dtype), "swish7")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,page,cap", [(6, 2, 32, 8, 1.5), (4, 1, 128, 16, None), (5, 5, 48, 4, 0.7)])
def test_paged_attention_with_a_distance_bias_and_a_soft_cap(kernels, dtype, heads, kv_heads, dim, page, cap):
    """Scores squashed to cap * tanh(score / cap), then lowered by slope[head] * distance: portions beside decoded
    tokens, on the matrix-core kernels of both precisions (pages of 4 in bfloat16: the generic one), against the
    formula."""
    lengths, counts = [45, 17, 70], [20, 1, 70]
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, page, dtype, shuffle_seed=heads)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    slopes = torch.tensor([0.3 / 2.0 ** head for head in range(heads)], dtype=torch.float32)
    scale = 1.0 / math.sqrt(dim)
    out = kernels[dtype].paged_attention(qkv, layout, batch, cell, scale, None, score_slopes=on_gpu(slopes), soft_cap=cap).cpu().double()
    expected = []
    for (q, k, v), count in zip(per_request, counts):
        q, k, v = rounded(q, dtype), rounded(k, dtype), rounded(v, dtype)
        length = q.shape[0]
        k, v = k.repeat_interleave(heads // kv_heads, dim=1), v.repeat_interleave(heads // kv_heads, dim=1)
        scores = torch.einsum("ihd,jhd->hij", q, k) * scale
        if cap:
            scores = cap * torch.tanh(scores / cap)
        distance = (torch.arange(length).unsqueeze(1) - torch.arange(length).unsqueeze(0)).double()
        scores = (scores - slopes.double().view(-1, 1, 1) * distance).masked_fill(distance < 0, float("-inf"))
        full = torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), v)
        expected.append(full[-count:].flatten(1))
    torch.testing.assert_close(out, torch.cat(expected), **TOLERANCE[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lengths,counts,window", [([2100, 700, 5], [1, 1, 1], None), ([300, 2100, 900], [300, 64, 1], 512)])
@pytest.mark.parametrize("heads,kv_heads,dim,cap", [(12, 2, 128, 4.0), (7, 7, 64, None)])
def test_changed_scores_over_long_contexts(kernels, dtype, lengths, counts, window, heads, kv_heads, dim, cap):
    """The same change of the scores where the keys are split over workgroups and merged (single tokens over long
    contexts), in long portions, and under a window; slopes small enough that far keys still count, one head's zero."""
    batch, cell, per_request, layout = paged_case(lengths, counts, heads, kv_heads, dim, 16, dtype, shuffle_seed=3)
    qkv = on_gpu(step_rows(per_request, counts, heads, kv_heads, dim), dtype)
    slopes = torch.tensor([0.0 if head == 1 else 0.004 * (1 + head % 3) for head in range(heads)], dtype=torch.float32)
    scale = 1.0 / math.sqrt(dim)
    out = kernels[dtype].paged_attention(qkv, layout, batch, cell, scale, window, score_slopes=on_gpu(slopes), soft_cap=cap).cpu().double()
    expected = []
    for (q, k, v), count in zip(per_request, counts):
        q, k, v = rounded(q, dtype)[-count:], rounded(k, dtype), rounded(v, dtype)
        length = k.shape[0]
        k, v = k.repeat_interleave(heads // kv_heads, dim=1), v.repeat_interleave(heads // kv_heads, dim=1)
        scores = torch.einsum("ihd,jhd->hij", q, k) * scale
        if cap:
            scores = cap * torch.tanh(scores / cap)
        distance = (torch.arange(length - count, length).unsqueeze(1) - torch.arange(length).unsqueeze(0)).double()
        unseen = (distance < 0) | (distance >= window if window else torch.zeros_like(distance, dtype=torch.bool))
        scores = (scores - slopes.double().view(-1, 1, 1) * distance).masked_fill(unseen, float("-inf"))
        expected.append(torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), v).flatten(1))
    torch.testing.assert_close(out, torch.cat(expected), **TOLERANCE[dtype])


def device_paged_case(requests, heads, kv_heads, dim, page, dtype, seed):
    """As `paged_case`, made on the device without a loop over positions, for contexts of thousands of keys:
    `requests` = [(cached tokens, of which this step's)].  Returns the batch, the cell (NaN in every slot that no
    token owns) and per request its step's queries and all its keys and values, as the kernel sees them."""
    from llmserve_amd.cache import CacheCell
    from llmserve_amd.engine.batch import GroupBatch, SequenceChunk, StepBatch
    from llmserve_amd.parts import HeadLayout, PagedKeyValue

    generator = torch.Generator(device="cuda").manual_seed(seed)
    blocks = [math.ceil(length / page) for length, _ in requests]
    pages = sum(blocks) + 3
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(seed)).cuda()
    width = max(blocks)
    tables = torch.full((len(requests), width), -1, dtype=torch.int32, device="cuda")
    keys = torch.full((pages, kv_heads, page, dim), float("nan"), dtype=dtype, device="cuda")
    values = torch.full((pages, kv_heads, dim, page), float("nan"), dtype=dtype, device="cuda")
    per_request, rows, slot_mapping, positions, token_sequence, chunks, taken = [], [], [], [], [], [], 0
    for index, (length, count) in enumerate(requests):
        mine = order[taken : taken + blocks[index]]
        taken += blocks[index]
        tables[index, : blocks[index]] = mine.int()
        q = torch.randn(count, heads, dim, generator=generator, device="cuda").to(dtype)
        k = torch.randn(length, kv_heads, dim, generator=generator, device="cuda").to(dtype)
        v = torch.randn(length, kv_heads, dim, generator=generator, device="cuda").to(dtype)
        where = torch.arange(length, device="cuda")
        keys[mine[where // page], :, where % page] = k
        values[mine[where // page], :, :, where % page] = v
        per_request.append((q, k, v))
        rows.append(torch.cat([q.flatten(1), k[-count:].flatten(1), v[-count:].flatten(1)], dim=1))
        mine_cpu = mine.cpu().tolist()
        for position in range(length - count, length):
            slot_mapping.append(mine_cpu[position // page] * page + position % page)
            positions.append(position)
            token_sequence.append(index)
        chunks.append(SequenceChunk(f"r{index}", index, length - count, count))
    counts = [count for _, count in requests]
    starts = [0]
    for count in counts:
        starts.append(starts[-1] + count)
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    batch = StepBatch(
        num_tokens=sum(counts), chunks=chunks, token_ids=ints([0] * sum(counts)), positions=ints(positions),
        token_sequence=ints(token_sequence), query_start=ints(starts), context_lengths=ints([length for length, _ in requests]),
        state_slots=ints(list(range(len(requests)))), groups=[GroupBatch(page, tables, ints(slot_mapping), width)],
        logit_rows=ints([]), num_logit_rows=0, max_query_length=max(counts), max_context_length=max(length for length, _ in requests),
    )
    cell = CacheCell(PagedKeyValue(kv_heads, dim), True, 0, key_pieces(keys), value_pieces(values))
    return batch, cell, per_request, torch.cat(rows), HeadLayout(heads, kv_heads, dim)


def device_attention(q, k, v, scale, window):
    """softmax(q k^T * scale) v of a request's last rows over all its keys, causal (and windowed), float32 on the
    device with torch's own operations, one kv head at a time."""
    count, heads, dim = q.shape
    length, kv_heads = k.shape[0], k.shape[1]
    group = heads // kv_heads
    position = torch.arange(length - count, length, device=q.device).view(1, -1, 1)
    key = torch.arange(length, device=q.device).view(1, 1, -1)
    unseen = key > position
    if window:
        unseen = unseen | (key <= position - window)
    out = torch.empty(count, heads, dim, dtype=torch.float32, device=q.device)
    for kv_head in range(kv_heads):
        mine = q[:, kv_head * group : (kv_head + 1) * group].float()
        scores = torch.einsum("igd,jd->gij", mine, k[:, kv_head].float()) * scale
        weights = torch.softmax(scores.masked_fill(unseen, float("-inf")), dim=-1)
        out[:, kv_head * group : (kv_head + 1) * group] = torch.einsum("gij,jd->igd", weights, v[:, kv_head].float())
    return out.flatten(1)


@pytest.mark.parametrize("dtype,draws", [(torch.bfloat16, 100), (torch.float32, 30)])
def test_attention_at_random_step_shapes(dtype, draws):
    """What a step holds decides which attention kernel it goes to and how its keys are cut (the kernel that shares
    keys through LDS whole or in runs, the tiles kernel with one or two column tiles, key splits merged by row or
    by work item): steps drawn at random around those rules (long portions far into their prompts, few or many
    decoded tokens over short and long contexts, several head counts and pages, windows), each against torch's own
    operations, and the bfloat16 draws together must have taken every way; the float32 kernel under the same draws."""
    import random

    from llmserve_amd.kernels import HipKernels

    kernels = HipKernels(dtype)
    library = kernels._attention_library(128)
    ways = {"shared whole": 0, "shared in runs": 0, "tiles": 0, "tiles split": 0, "by item": 0}
    shared_entry, tiles_entry = library.llmserve_attention_portions, library.llmserve_attention_tiles

    def counted_shared(*arguments):
        ways["shared in runs" if arguments[18] > 1 else "shared whole"] += 1  # (splits)
        return shared_entry(*arguments)

    def counted_tiles(*arguments):
        splits, fuse = arguments[19], arguments[20]
        ways["by item" if fuse & 4 and splits > 1 else "tiles split" if splits > 1 else "tiles"] += 1
        return tiles_entry(*arguments)

    library.llmserve_attention_portions, library.llmserve_attention_tiles = counted_shared, counted_tiles
    try:
        for seed in range(draws):
            draw = random.Random(seed)
            heads, kv_heads = draw.choice([(12, 2), (28, 4), (40, 8), (16, 2), (64, 8), (7, 7)])
            page = draw.choice([16, 16, 32, 8, 64])
            window = draw.choice([None, None, 700, 4096])
            requests = []
            for _ in range(draw.choice([0, 1, 1, 2, 3])):
                count = draw.choice([64, 300, 512, 1024, 2048])
                requests.append((count + draw.choice([0, 0, 700, 3000, 9000, 17000]), count))
            for _ in range(draw.choice([0, 1, 5, 20, 40]) if requests else draw.choice([1, 5, 20, 40])):
                requests.append((draw.randint(1, draw.choice([300, 3000, 12000])), 1))
            draw.shuffle(requests)
            batch, cell, per_request, qkv, layout = device_paged_case(requests, heads, kv_heads, 128, page, dtype, seed)
            scale = 1.0 / math.sqrt(128)
            out = kernels.paged_attention(qkv, layout, batch, cell, scale, window).float()
            expected = torch.cat([device_attention(q, k, v, scale, window) for q, k, v in per_request])
            torch.testing.assert_close(out, expected, **TOLERANCE[dtype], msg=lambda m: f"seed {seed}, {heads}/{kv_heads} heads, pages of {page}, window {window}, {requests}: {m}")
            del batch, cell, per_request, qkv, out, expected
    finally:
        library.llmserve_attention_portions, library.llmserve_attention_tiles = shared_entry, tiles_entry
    assert dtype == torch.float32 or all(ways.values()), ways


@pytest.mark.parametrize("own", [False, True])
def test_products_at_random_shapes(own):
    """Rows, K and N decide which product kernel runs (weight-streaming with one, two or four tiles a wave, through
    registers or LDS, K cut into partial sums, the kernels for 17 to 64 rows, the library or the tiled kernels beyond,
    inside and outside a step that a graph will replay): shapes drawn at random around those rules, plain, with a
    bias, as float32 partial sums and gated, against torch's float32 product of the same rounded operands."""
    import random

    from llmserve_amd.kernels import HipKernels

    dtype = torch.bfloat16
    k = HipKernels(dtype, library_products=not own)
    generator = torch.Generator(device="cuda").manual_seed(5)
    for seed in range(200):
        draw = random.Random(1000 + seed)
        rows = draw.choice([1, 2, 3, 5, 8, 13, 16, 17, 24, 32, 33, 48, 64, 65, 100, 128, 130, 300])
        inner = 32 * draw.choice([1, 3, 4, 8, 12, 16, 28, 40, 48, 64, 70, 112, 148, 160, 216, 280])
        outer = draw.choice([16, 48, 100, 256, 272, 1000, 1536, 2048, 4099, 5120, 17920])
        if rows > 64 and inner * outer > 1 << 24:
            outer = 1000
        x = torch.randn(rows, inner, generator=generator, device="cuda").to(dtype)
        w = (torch.randn(outer, inner, generator=generator, device="cuda") / math.sqrt(inner)).to(dtype)
        up = (torch.randn(outer, inner, generator=generator, device="cuda") / math.sqrt(inner)).to(dtype)
        b = torch.randn(outer, generator=generator, device="cuda").to(dtype)
        said = f"draw {seed}: {rows} rows, K {inner}, N {outer}"
        want = x.float() @ w.float().T
        plain_weights, biased = k.prepare_linear([w], None), k.prepare_linear([w], [b])
        gated_weights = k.prepare_gated_linear(w, up)
        want_gated = F.silu(want) * (x.float() @ up.float().T)
        for replayed in (False, True):
            with k.replay_scope() if replayed else contextlib.nullcontext():
                torch.testing.assert_close(k.linear(x, plain_weights).float(), want, **TOLERANCE[dtype], msg=lambda m: f"{said}, plain, replay {replayed}: {m}")
                torch.testing.assert_close(k.linear(x, biased).float(), want + b.float(), **TOLERANCE[dtype], msg=lambda m: f"{said}, bias, replay {replayed}: {m}")
                parts = k.linear(x, plain_weights, out_dtype=torch.float32, partial=True)
                summed = parts if parts.ndim == 2 else parts.sum(0)
                torch.testing.assert_close(summed, want, atol=2e-4, rtol=2e-4, msg=lambda m: f"{said}, partial sums, replay {replayed}: {m}")
                torch.testing.assert_close(k.gated_linear(x, gated_weights).float(), want_gated, **TOLERANCE[dtype], msg=lambda m: f"{said}, gated, replay {replayed}: {m}")


@pytest.mark.parametrize("tiles", [2, 4, 5, 6, 8, 10, 12, 14])
@pytest.mark.parametrize("rows,inner,outer,parts", [(17, 128, 48, 1), (33, 1536, 1000, 3), (64, 8960, 272, 10), (50, 384, 4099, 1), (32, 512, 130, 2),
                                                    (8, 1024, 300, 2), (65, 256, 100, 1), (100, 1536, 1000, 4), (128, 3584, 272, 7)])
def test_product_through_the_ring(kernels, tiles, rows, inner, outer, parts):
    """The product for up to 128 rows whose weights and x go through a ring of stages in LDS, in every shape of
    workgroup it has (2 to 14 tiles of 16 weight rows; 5 for more than 32 rows only, 6, 12 and 14 for up to 64): rows
    and weight rows that end inside a tile, a K of one stage and of fewer stages than the ring has, with a bias, as float32
    partial sums and gated."""
    from llmserve_amd.kernels.hip import KernelError, _check, _is_float, _pointer

    k, dtype = kernels[torch.bfloat16], torch.bfloat16
    library = k._gemm_bf16
    x, w, b = torch.randn(rows, inner), torch.randn(outer, inner) / math.sqrt(inner), torch.randn(outer)
    up = torch.randn(outer, inner) / math.sqrt(inner)
    want = rounded(x, dtype) @ rounded(w, dtype).T

    def run(weight, bias, out, gated, splits):
        return library.llmserve_gemm_ring(
            _pointer(on_gpu(x, dtype)), _pointer(weight), _pointer(bias), _is_float(bias) if bias is not None else 0, _pointer(out),
            _is_float(out), 1 if gated else 0, rows, weight.shape[0], inner, splits, tiles, k._stream)

    weight, bias = on_gpu(w, dtype), on_gpu(b, dtype)
    out = torch.empty(rows, outer, dtype=dtype, device="cuda")
    if (tiles == 5 and rows <= 32) or (tiles in (6, 12, 14) and rows > 64):
        with pytest.raises(KernelError):
            _check(run(weight, bias, out, False, 1), "ring")
        return
    _check(run(weight, bias, out, False, 1), "ring")
    torch.testing.assert_close(out.cpu().double(), want + rounded(b, dtype), **TOLERANCE[dtype])
    float_bias = on_gpu(b, torch.float32)
    partial = torch.empty(parts, rows, outer, dtype=torch.float32, device="cuda")
    _check(run(weight, float_bias, partial, False, parts), "ring")
    torch.testing.assert_close(partial.sum(0).cpu().double(), want + b.double(), atol=1e-4, rtol=1e-4)
    both = torch.stack([on_gpu(w, dtype), on_gpu(up, dtype)], dim=1).reshape(2 * outer, inner).contiguous()
    gated = torch.empty(rows, outer, dtype=dtype, device="cuda")
    _check(run(both, None, gated, True, 1), "ring")
    torch.testing.assert_close(gated.cpu().double(), F.silu(want) * (rounded(x, dtype) @ rounded(up, dtype).T), **TOLERANCE[dtype])
