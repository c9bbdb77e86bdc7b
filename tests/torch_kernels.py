"""A stand-in for the HIP kernel library, in elementary torch on the CPU.

It exists only so that the tests which need no GPU can run the engine's parts,
cache manager, step function, scheduler and entry points here; the product
never selects it.  It rounds to the run dtype at the same places as the HIP
kernels (activations between operations), and computes everything in float32.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch


@dataclass
class _Linear:
    weight: torch.Tensor  # [N, K] float32
    bias: torch.Tensor | None


class TorchKernels:
    def __init__(self, dtype: torch.dtype = torch.float32) -> None:
        self.device = torch.device("cpu")
        self.dtype = dtype
        self.calls: list[str] = []

    def to_device(self, tensor):
        return tensor

    def queued_to_device(self, tensor):
        return tensor

    def embedding(self, table, token_ids):
        return table[token_ids.long()].float()

    def add_rms_norm(self, hidden, delta, weight, eps):
        if delta is not None:
            hidden += delta if delta.ndim == 2 else delta.sum(0)
        variance = hidden.pow(2).mean(-1, keepdim=True)
        return (hidden * torch.rsqrt(variance + eps) * weight.float()).to(self.dtype)

    def prepare_linear(self, weights, biases):
        weight = torch.cat([w.float() for w in weights], dim=0)
        bias = torch.cat([b.float() for b in biases], dim=0) if biases else None
        return _Linear(weight, bias)

    def prepare_gated_linear(self, gate, up, activation="silu"):
        acts = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "relu": torch.relu,
                "gelu_tanh": lambda z: torch.nn.functional.gelu(z, approximate="tanh")}
        if activation not in acts:
            raise ValueError(f"gated_linear: no activation {activation!r}")
        return (_Linear(gate.float(), None), _Linear(up.float(), None), acts[activation])

    def linear(self, x, weights, out_dtype=None, partial=False):
        y = x.float() @ weights.weight.T
        if weights.bias is not None:
            y = y + weights.bias
        return y.to(out_dtype or self.dtype)

    def gated_linear(self, x, weights):
        gate = x.float() @ weights[0].weight.T
        up = x.float() @ weights[1].weight.T
        return (weights[2](gate) * up).to(self.dtype)

    def rotate_and_store(self, qkv, layout, batch, cell, inverse_frequencies, pairing):
        tokens = qkv.shape[0]
        heads, kv_heads, dim = layout.num_heads, layout.num_kv_heads, layout.head_dim
        view = qkv.view(tokens, heads + 2 * kv_heads, dim)
        if pairing != "none":
            angles = batch.positions.float()[:, None] * inverse_frequencies[None, :]
            cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
            part = view[:, : heads + kv_heads].float()
            if pairing == "adjacent":
                a, b = part[..., 0::2], part[..., 1::2]
                out = torch.empty_like(part)
                out[..., 0::2] = a * cos - b * sin
                out[..., 1::2] = b * cos + a * sin
            else:
                a, b = part[..., : dim // 2], part[..., dim // 2 :]
                out = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
            view[:, : heads + kv_heads] = out.to(qkv.dtype)
        if cell is not None and cell.writable:
            group = batch.groups[cell.group]
            slots = group.slot_mapping.long()
            pages, offsets = slots // group.page_size, slots % group.page_size
            cell.put_key_rows(pages, offsets, view[:, heads : heads + kv_heads])  # pages are [kv, dim / w, offset, w]
            cell.put_value_rows(pages, offsets, view[:, heads + kv_heads :])  # pages are [kv, offset / v, dim, v]

    def paged_attention(self, qkv, layout, batch, cell, scale, window, *, score_slopes=None, soft_cap=None):
        tokens = qkv.shape[0]
        heads, kv_heads, dim = layout.num_heads, layout.num_kv_heads, layout.head_dim
        queries = qkv.view(tokens, heads + 2 * kv_heads, dim)[:, :heads].float()
        group = batch.groups[cell.group]
        out = torch.zeros(tokens, heads, dim)
        row = 0
        for b, chunk in enumerate(batch.chunks):
            table = group.block_tables[b].long()
            for position in range(chunk.start, chunk.start + chunk.count):
                first = 0 if window is None else max(0, position - window + 1)
                where = torch.arange(first, position + 1)
                pages = table[where // group.page_size]
                assert (pages >= 0).all(), "attention reads a page that was given back"
                keys = cell.key_rows(pages, where % group.page_size).float()  # [n, kv, D]
                values = cell.value_rows(pages, where % group.page_size).float()
                keys = keys.repeat_interleave(heads // kv_heads, dim=1)
                values = values.repeat_interleave(heads // kv_heads, dim=1)
                scores = torch.einsum("hd,nhd->hn", queries[row], keys) * scale
                if soft_cap is not None:
                    scores = soft_cap * torch.tanh(scores / soft_cap)
                if score_slopes is not None:
                    scores = scores - score_slopes.float().view(-1, 1) * (position - where).float()
                out[row] = torch.einsum("hn,nhd->hd", torch.softmax(scores, dim=-1), values)
                row += 1
        return out.reshape(tokens, heads * dim).to(self.dtype)

    def rotate_store_attend(self, qkv, layout, batch, cell, inverse_frequencies, pairing, scale, window, project=None):
        self.rotate_and_store(qkv, layout, batch, cell, inverse_frequencies, pairing)
        mixed = self.paged_attention(qkv, layout, batch, cell, scale, window)
        return mixed if project is None else self.linear(mixed, project, out_dtype=torch.float32, partial=True)

    def gather_rows(self, hidden, delta, rows):
        picked = hidden[rows.long()]
        if delta is not None and delta.ndim == 3:
            delta = delta.sum(0)
        return picked + delta[rows.long()] if delta is not None else picked.clone()

    def argmax(self, logits):
        return torch.argmax(logits, dim=-1).to(torch.int32)

    def sample(self, logits, temperatures, top_ps, uniforms, with_top_p=True):
        chosen = []
        for row in range(logits.shape[0]):
            temperature, top_p, u = float(temperatures[row]), float(top_ps[row]), float(uniforms[row])
            if temperature <= 0:
                chosen.append(int(torch.argmax(logits[row])))
                continue
            p = torch.softmax(logits[row].float() / temperature, dim=-1).double()
            if top_p < 1.0:
                values, order = torch.sort(p, descending=True, stable=True)
                before = values.cumsum(0) - values
                keep = before < top_p
                values, order = values[keep], order[keep]
            else:
                values, order = p, torch.arange(p.numel())
            running = values.cumsum(0)
            hit = torch.nonzero(running > u * running[-1])
            chosen.append(int(order[hit[0, 0]] if hit.numel() else order[-1]))
        return torch.tensor(chosen, dtype=torch.int32)
