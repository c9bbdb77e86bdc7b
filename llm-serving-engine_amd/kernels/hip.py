"""The HIP kernel library: every operation of the model on gfx950.

There is no other implementation in the product: without a GPU, or without a
compiler to build a missing library, construction fails with an error.
Kernels are called through their C entry points with raw device pointers on
torch's current stream, so a step can be captured into a HIP graph.
"""

from __future__ import annotations

import contextlib
import ctypes
from dataclasses import dataclass
from typing import Any

import torch

from .build import _say, load_module

_PAIRINGS = {"none": 0, "adjacent": 1, "half": 2}
# gate activations of a gated product (csrc/elementwise.hip: gate_activation); the products' fused epilogues know silu alone
_ACTIVATIONS = {"silu": 0, "gelu": 1, "gelu_tanh": 2, "relu": 3}


class KernelError(RuntimeError):
    pass


def _is_float(tensor: torch.Tensor) -> int:
    if tensor.dtype == torch.float32:
        return 1
    if tensor.dtype == torch.bfloat16:
        return 0
    raise KernelError(f"kernels take float32 or bfloat16 tensors, not {tensor.dtype}")


def _pointer(tensor: torch.Tensor | None) -> int | None:
    """The tensor's device address (None: a null pointer) for an argument declared as a pointer."""
    if tensor is None:
        return None
    if not tensor.is_contiguous():
        raise KernelError("kernels take contiguous tensors")
    return tensor.data_ptr()


# Argument types of every entry point: p pointer, i int, f float.  Declared once, so that a call
# costs no guessing: a decode step is replayed from a graph, but every other step pays per launch.
_SIGNATURES = {
    "llmserve_embedding": "pippiip",
    "llmserve_add_rms_norm": "ppipipiiifp",
    "llmserve_rotary_table": "pppiip",
    "llmserve_rotate_and_store": "pipiiiiipppip",
    "llmserve_silu_mul": "pipiiip",
    "llmserve_gate_mul": "pipiiiip",
    "llmserve_gather_rows": "ppiippiip",
    "llmserve_gemm_generic": "pipipipiiiip",
    "llmserve_gemm_f32": "ppppiiiiip",
    "llmserve_gemm_skinny": "pppipiiiiiip",
    "llmserve_gemm_stream": "pppipiiiiiip",
    "llmserve_gemm_stream_shaped": "pppipiiiiiiiip",
    "llmserve_gemm_medium": "pppipiiiiiip",
    "llmserve_gemm_ring": "pppipiiiiiiip",
    "llmserve_gemm_merged": "ppippipiiiip",
    "llmserve_gemm_tiled": "pppipiiiiiip",
    "llmserve_attention_generic": "pipipppippiiiiifipfp",
    "llmserve_attention_f32": "pippppppippiiiiiifiipfp",
    "llmserve_attention_tiles": "pippppppippiiiiiifiiipippfp",
    "llmserve_attention_portions": "pippppppippiiiiiifiip",
    "llmserve_attention_can_fuse": "i",
    "llmserve_argmax": "ppppiip",
    "llmserve_argmax_static": "ppiip",
    "llmserve_sample_workspace_kib": "ii",
    "llmserve_sample": "pppppipiiip",
}
_TYPES = {"p": ctypes.c_void_p, "i": ctypes.c_int, "f": ctypes.c_float}


def _declared(library: ctypes.CDLL) -> ctypes.CDLL:
    for name, signature in _SIGNATURES.items():
        if hasattr(library, name):
            entry = getattr(library, name)
            entry.argtypes = [_TYPES[code] for code in signature]
            entry.restype = ctypes.c_int
    return library


def _check(status: int, what: str) -> None:
    if status == 1001:
        raise KernelError(f"{what}: the kernel refuses these sizes or arguments")
    if status != 0:
        raise KernelError(f"{what}: HIP error {status}")


@dataclass
class LinearWeights:
    """A product's right-hand side: weight [N, K] and bias [N] or None, as loaded."""

    weight: torch.Tensor
    bias: torch.Tensor | None

    @property
    def out_features(self) -> int:
        return self.weight.shape[0]

    @property
    def in_features(self) -> int:
        return self.weight.shape[1]


@dataclass
class GatedLinearWeights:
    """Gate and up weights as one [2 I, K] right-hand side with rows interleaved:
    gate_0, up_0, gate_1, up_1, ...  A kernel's output tile then holds a gate and
    its up side by side, and act(gate) * up is applied before anything is stored."""

    both: LinearWeights
    width: int
    activation: str = "silu"


class HipKernels:
    def __init__(
        self, dtype: torch.dtype = torch.bfloat16, device: str | torch.device = "cuda:0", *, library_products: bool = True,
        shared_portions: str = "auto",
    ) -> None:
        """`library_products=False` keeps every product on the hand-written kernels (the command line's and
        bench.py's --own-products): the weight-streaming ones up to 64 rows, the LDS-tiled ones above, with
        their fused epilogues.  Inside a whole step the library is ahead for many rows (at 2,048 rows of the
        1.5B sizes gate/up with its fused SiLU * up takes 150 us against the library's 120 + 18 for SiLU * up),
        so it is the default there.
        `shared_portions`:
        whether prompt portions at head size 128 go to the attention kernel whose waves share K and V
        through LDS: "auto" (when the step's walks, taken together, are long beside the longest), "always", "never"."""
        if dtype not in (torch.bfloat16, torch.float32):
            raise KernelError(f"run dtype must be bfloat16 or float32, not {dtype}")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the engine runs on an MI355X only and has no CPU path")
        self.dtype = dtype
        self.device = torch.device(device)
        self.library_products = library_products
        self.shared_portions = shared_portions
        self.portion_splits: int | None = None  # runs of keys a workgroup of that kernel's items is cut into; None: by rule
        self.merge_in_product = True  # decode attention leaves its key splits to the product that reads them
        self.merge_weight_bytes = 8 << 20  # ... where that product's weight is at most this large (measured at 4.7 and 25.7 MB)
        name = torch.cuda.get_device_properties(self.device).gcnArchName
        if not name.startswith("gfx950"):
            raise KernelError(f"the kernels are built for gfx950 (MI355X); this GPU is {name}")
        self._elementwise = _declared(load_module("elementwise"))
        self._gemm_generic = _declared(load_module("gemm_generic"))
        self._gemm_f32 = _declared(load_module("gemm_f32")) if dtype == torch.float32 else None
        self._attention_generic = _declared(load_module("attention_generic"))
        self._gemm_bf16 = _declared(load_module("gemm_bf16")) if dtype == torch.bfloat16 else None
        self._pinned_stream: int | None = None
        self.ring_products = True  # 17 to 64 rows of a large weight go to the kernel that streams it through a ring in LDS
        self.ring_rows_from = 4     # (and from this many rows on where K may be cut or the weight is very large)
        self._for_replay = False  # inside `replay_scope`: the step being launched is one that a graph will replay
        self._told: set[str] = set()
        if self._gemm_bf16 is not None and library_products:
            # The BLAS library sets itself up at its first product, which it cannot do while a stream is
            # being captured; a step of 17 to 64 rows meets the library only inside a capture.
            with torch.cuda.device(self.device):
                one = torch.ones((32, 32), dtype=torch.bfloat16, device=self.device)
                torch.nn.functional.linear(one, one, one[0])
                torch.mm(one, one.t(), out_dtype=torch.float32)
                torch.cuda.synchronize(self.device)
        self._attention_bf16: dict[int, ctypes.CDLL] = {}  # by head size, compiled when a model needs it
        self._attention_f32: dict[int, ctypes.CDLL] = {}
        self._sampling = None

    # ------------------------------------------------------------------ helpers

    @property
    def _stream(self) -> int:
        if self._pinned_stream is not None:
            return self._pinned_stream
        return torch.cuda.current_stream(self.device).cuda_stream

    @contextlib.contextmanager
    def stream_scope(self):
        """Within the scope every kernel goes to the stream that is current at its start (asked
        once instead of per launch); the caller must not switch streams inside."""
        previous = self._pinned_stream
        self._pinned_stream = torch.cuda.current_stream(self.device).cuda_stream
        try:
            yield
        finally:
            self._pinned_stream = previous

    @contextlib.contextmanager
    def replay_scope(self):
        """Within the scope the step is launched for a graph: its warm-up run and the run that is captured.
        Such a step costs the host nothing per launch when it is replayed, so products may go where the
        device is fastest rather than where a launch is cheapest; both runs take the same routes, so the
        library meets each of the capture's shapes before the capture begins."""
        previous, self._for_replay = self._for_replay, True
        try:
            yield
        finally:
            self._for_replay = previous

    def _tell_once(self, key: str, message: str) -> None:
        if key not in self._told:
            self._told.add(key)
            _say(message)

    def to_device(self, tensor: torch.Tensor) -> torch.Tensor:
        return tensor.to(self.device).contiguous()

    def queued_to_device(self, tensor: torch.Tensor) -> torch.Tensor:
        """A small host tensor's values on the device, by a copy that is only queued: it goes through
        pinned memory, so the host does not wait for the work queued before it (with a pageable
        source it would, and a step queued ahead would be waited for)."""
        pinned = torch.empty(tensor.shape, dtype=tensor.dtype, pin_memory=True)
        pinned.copy_(tensor)
        return pinned.to(self.device, non_blocking=True)

    def _empty(self, shape, dtype) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype, device=self.device)

    # ------------------------------------------------------------------ elementwise

    def embedding(self, table: torch.Tensor, token_ids: torch.Tensor) -> torch.Tensor:
        tokens, hidden = token_ids.shape[0], table.shape[1]
        out = self._empty((tokens, hidden), torch.float32)
        status = self._elementwise.llmserve_embedding(
            _pointer(table), _is_float(table), _pointer(token_ids), _pointer(out), tokens, hidden, self._stream
        )
        _check(status, "embedding")
        return out

    def add_rms_norm(self, hidden, delta, weight, eps: float) -> torch.Tensor:
        rows, width = hidden.shape
        if hidden.dtype != torch.float32 or (delta is not None and delta.dtype != torch.float32):
            raise KernelError("add_rms_norm: the residual stream and what is added to it are float32")
        out = self._empty((rows, width), self.dtype)
        parts = 1 if delta is None or delta.ndim == 2 else delta.shape[0]  # [parts, rows, width]: partial sums
        status = self._elementwise.llmserve_add_rms_norm(
            _pointer(hidden), _pointer(delta), parts, _pointer(weight), _is_float(weight), _pointer(out),
            _is_float(out), rows, width, eps, self._stream,
        )
        _check(status, "add_rms_norm")
        return out

    def rotary_table(self, batch, inverse_frequencies: torch.Tensor) -> torch.Tensor:
        """(cos, sin) [T, D/2, 2] float32 of position * frequency for the step's tokens.  Every
        layer with the same frequencies shares it: it is computed once per step and kept on the batch."""
        key = ("rotary_table", inverse_frequencies.data_ptr())
        table = batch.computed.get(key)
        if table is None:
            tokens, half = batch.positions.shape[0], inverse_frequencies.shape[0]
            table = self._empty((tokens, half, 2), torch.float32)
            status = self._elementwise.llmserve_rotary_table(
                _pointer(batch.positions), _pointer(inverse_frequencies), _pointer(table), tokens, half, self._stream
            )
            _check(status, "rotary_table")
            batch.computed[key] = table
        return table

    def rotate_and_store(self, qkv, layout, batch, cell, inverse_frequencies, pairing: str) -> None:
        tokens = qkv.shape[0]
        if qkv.shape[1] != layout.width:
            raise KernelError("rotate_and_store: qkv does not have the layout's width")
        store = cell is not None and cell.writable
        group = batch.groups[cell.group] if store else None
        if store and (cell.keys.dtype != qkv.dtype or cell.values.shape[1:] != cell.need.page_fields(group.page_size)["values"]):
            raise KernelError("rotate_and_store: the cell's pages do not fit the layout")
        table = self.rotary_table(batch, inverse_frequencies) if pairing != "none" else None
        status = self._elementwise.llmserve_rotate_and_store(
            _pointer(qkv), _is_float(qkv), _pointer(table), _PAIRINGS[pairing], tokens, layout.num_heads,
            layout.num_kv_heads, layout.head_dim, _pointer(cell.keys if store else None),
            _pointer(cell.values if store else None), _pointer(group.slot_mapping if store else None),
            group.page_size if store else 1, self._stream,
        )
        _check(status, "rotate_and_store")

    def gather_rows(self, hidden, delta, rows) -> torch.Tensor:
        count, width = rows.shape[0], hidden.shape[1]
        out = self._empty((count, width), torch.float32)
        parts = 1 if delta is None or delta.ndim == 2 else delta.shape[0]
        status = self._elementwise.llmserve_gather_rows(
            _pointer(hidden), _pointer(delta), parts, hidden.shape[0], _pointer(rows), _pointer(out), count, width,
            self._stream,
        )
        _check(status, "gather_rows")
        return out

    # ------------------------------------------------------------------ products

    def prepare_linear(self, weights: list[torch.Tensor], biases: list[torch.Tensor] | None) -> LinearWeights:
        kinds = {w.dtype for w in weights}
        if len(kinds) > 1:
            weights = [w.float() for w in weights]
        weight = torch.cat(list(weights), dim=0).contiguous() if len(weights) > 1 else weights[0].contiguous()
        bias = None
        if biases:
            if len({b.dtype for b in biases}) > 1:
                biases = [b.float() for b in biases]
            bias = torch.cat(list(biases), dim=0).contiguous() if len(biases) > 1 else biases[0].contiguous()
        return LinearWeights(weight, bias)

    def prepare_gated_linear(self, gate: torch.Tensor, up: torch.Tensor, activation: str = "silu") -> GatedLinearWeights:
        """`activation` is the gate's: silu is applied in the epilogue of the product itself; the others
        (gelu, gelu_tanh, relu) by a kernel of their own behind a plain product."""
        if activation not in _ACTIVATIONS:
            raise KernelError(f"gated_linear: no kernel applies the activation {activation!r} (known: {', '.join(_ACTIVATIONS)})")
        if gate.shape != up.shape:
            raise KernelError("gated_linear: gate and up differ in shape")
        if gate.dtype != up.dtype:
            gate, up = gate.float(), up.float()
        both = torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], gate.shape[1]).contiguous()
        return GatedLinearWeights(LinearWeights(both, None), gate.shape[0], activation)

    def _streaming(self, x: torch.Tensor, weights: LinearWeights, gated: bool = False, may_split: bool = False) -> str | None:
        """Which MFMA kernel takes this product: "skinny" (up to 16 rows of x, weights streamed),
        "ring" (17 to 64 rows of a middling weight, both operands through a ring of stages in LDS),
        "medium" (up to 64, x shared through LDS), "tiled" (any number, both operands through LDS),
        or None (the BLAS library, or the generic kernel)."""
        if x.dtype != torch.bfloat16 or weights.weight.dtype != torch.bfloat16:
            return None
        rows, inner = x.shape[0], weights.in_features
        size = weights.out_features * inner
        if self.ring_products and rows <= 16 and inner % 128 == 0 and size > (1 << 22):
            # A few rows of a large weight do as well or better on the kernel written for 17 to 64 rows where its
            # workgroups make one round: from 4 rows on where the weight is very large or is large and its K may be
            # cut over workgroups, from 12 rows on the middling ones.  Us at 4 / 8 / 16 rows in a captured chain over
            # different weights: 7B sizes down 27.5 / 28.0 / 29.6 -> 26.2 / 26.3 / 26.5, gate/up 46.9 / 49.9 / 58.9 -> 47.6 /
            # 47.7 / 47.9; 32B sizes gate/up 108.3 / 110.9 / 120.2 -> 100.8 / 101.1 / 101.3; the 1.5B sizes' down projection
            # and gate/up at 16 rows 10.3 and 15.8 -> 8.2 and 14.0 (at 8 rows 8.8 -> 8.1 alone, but the step it is in 1.434 ->
            # 1.441 ms); a single row, 7B qkv at 8 rows (11.8 -> 12.8) and what would take several rounds (the 1.5B sizes'
            # head 89.6 / 94.2 -> 93.3 / 94.9, the 32B sizes' down projection 52.5 -> 54.2) stay.
            heavy = size > (1 << 26) or (may_split and size > (1 << 24))
            if rows >= (self.ring_rows_from if heavy else max(12, self.ring_rows_from)) and (heavy or may_split or size > (1 << 24)):
                if self._ring_shape(rows, weights.out_features, inner, may_split)[2] == 1:
                    return "ring"
        if 0 < rows <= 16 and inner % 32 == 0:
            return "skinny"
        if self.ring_products and 16 < rows <= 64 and inner % 128 == 0 and size > (1 << 22) and (
            size <= 150_000_000 or weights.out_features <= 256 * 14 * 16
        ):
            # (a smaller weight: the kernels below; a larger one only while fourteen tiles a workgroup make one round of
            # workgroups: the 32B sizes' gate/up 100-110 us at the library, 98-106 here, 113-177 in several rounds; the 1.5B
            # sizes' head, 9,496 tiles, 108-120 against 101-165)
            return "ring"
        if self.ring_products and 64 < rows <= 128 and inner % 128 == 0 and (
            (may_split and (1 << 20) < size <= 150_000_000) or (gated and (1 << 22) < size <= 150_000_000)
        ):
            # 65 to 128 rows, where the step from the kernel above to the library was a cliff (a decode step of the 1.5B
            # sizes 2.01 ms at 64 rows and 2.76 at 65): the same kernel with eight tiles of x for the products whose K
            # may be cut and the smaller gated ones.  Us at 65 / 128 rows in a captured chain over different weights,
            # the library against it: 1.5B sizes gate/up with its activation 25.8 / 26.5 -> 21.9 / 22.3, down 21.8 / 23.2 ->
            # 13.4 / 14.7, o 7.5 -> 5.8 / 6.3; 7B sizes down 40.1 / 52.4 -> 44.3 / 45.1, o 18.6 / 22.6 -> 13.2 / 14.3; the
            # gate/up with ten weight tiles a workgroup, 237 workgroups, 67.1 / 72.1 -> 59.1 / 61.3 (80-82 with five, which
            # make 474); the library keeps qkv (7.5 against 10.2; 19-23 against 21-23).
            return "ring"
        if self.library_products and (rows > 64 or self._for_replay or weights.out_features * inner > 150_000_000):
            # On the device the library is ahead of "medium" as it stands, so a captured step (which
            # costs the host nothing per launch) takes the library; a step launched kernel by kernel
            # is bound by the host, where a torch call costs four times one of ours (but a weight beyond what the
            # ring takes goes to the library either way: the 1.5B sizes' head at 64 rows 112 us against 174).
            # Except a small weight: there the library's fixed cost shows (qkv and o of the 1.5B sizes in a
            # captured chain: 7.1-7.7 us each, against 4.8 and 4.0 at 17 rows, 5.0 and 4.5 at 32, 6.7 and 6.2 at
            # 64 for the kernel that brings two or four tiles of x through LDS beside a weight tile; where K is
            # no multiple of 128 an older kernel takes up to 32 rows).
            if not gated and inner % 32 == 0 and weights.out_features * inner <= (1 << 22) and (rows <= 32 or (rows <= 64 and inner % 128 == 0)):
                return "skinny"
            return None
        if 16 < rows <= 64 and inner % 128 == 0:
            return "medium"
        if 16 < rows <= 64 and inner % 32 == 0:
            return "skinny"
        if rows > 64 and inner % 32 == 0:
            return "tiled"
        return None

    def _library(self, x: torch.Tensor, weights: LinearWeights) -> bool:
        """Whether the product goes to the BLAS library (hipBLASLt through torch), as the
        reference's products go to its BLAS through nn.Linear: bfloat16 with more rows than
        the weight-streaming kernels take."""
        return (
            self.library_products
            and x.dtype == torch.bfloat16
            and weights.weight.dtype == torch.bfloat16
            and self._streaming(x, weights) is None
            and x.shape[0] > 16
        )

    @staticmethod
    def _partial_splits(out_features: int, in_features: int) -> int:
        """Into how many parts of K a weight-streaming product is cut when its float32 result
        may stay in parts: a weight with few rows has too few 16-row tiles to fill the chip, so
        K is cut (at most 8 ways) until about a thousand workgroups run.  A part is at least 512 long,
        and 1,536 where K allows it: shorter walks cost more in waves that start and end than
        they gain (the 1.5B sizes' down projection at 8 rows: five parts 7.8 us, seven 8.4, two 8.1)."""
        groups = in_features // 128
        if in_features % 128 or groups < 8:
            return 1
        tiles = -(-out_features // 16)
        shortest = 12 if groups >= 24 else 4
        best = 1
        for splits in range(2, 9):
            if groups % splits == 0 and groups // splits >= shortest and tiles * splits <= 1024:
                best = splits
        return best

    @staticmethod
    def _ring_shape(rows: int, out_features: int, in_features: int, may_split: bool) -> tuple[int, int, int]:
        """How the product that streams its weights through a ring in LDS is shaped: (weight tiles a workgroup,
        parts of K, rounds of workgroups).  A workgroup fills most of a CU's LDS, so the workgroups run in
        rounds of 256 (512 where two fit), and what decides is whether one round takes them all: five tiles a
        workgroup of the 1.5B sizes' gate/up (224 workgroups) take 16.4 us at 64 rows, four (280) 25.2; ten tiles of
        the 7B sizes' (237) 52.8, five (474) 56.3.  A stage costs a workgroup what bringing its tiles of x costs
        plus so much a weight tile, a part of K what its partial sums cost to write and to add up, further rounds
        a quarter more.  The weights of that estimate are fitted to measurements in a captured chain over
        different weights (us at 17 / 64 rows, the library or the older kernels against this one: 1.5B sizes
        gate/up 18.1 / 20.7 -> 14.4 / 16.4, down 9.5 / 13.0 -> 8.5 / 11.2; 7B sizes gate/up 55.9 / 64.5 -> 48.1 / 53.3,
        down 34.4 / 44.0 -> 26.7 / 35.9, qkv 14.9 / 19.1 -> 13.6 / 16.5, o 13.0 / 14.2 -> 8.4 / 11.7; 32B sizes gate/up
        103.4 / 114.8 -> 101.5 / 108.8, down 91.1 / 58.8 -> 52.1 / 59.1, o 20.2 / 22.3 -> 14.6 / 16.8, qkv 19.8 / 25.6 ->
        18.8 / 27.7)."""
        tiles = -(-out_features // 16)
        x_tiles = 2 if rows <= 32 else 4 if rows <= 64 else 8
        stages = in_features // 128
        best = None
        for nt in (14, 12, 10, 8, 6, 5, 4, 2):
            if (nt == 5 and x_tiles < 4) or (nt == 6 and x_tiles > 4) or (nt >= 8 and may_split) or (nt >= 12 and x_tiles > 4):
                continue  # (many tiles a workgroup are for the products whose K stays whole: cutting K makes workgroups enough)
            # of LDS a tile: four stages of 4 KB, three beside eight tiles of x; eight and ten weight tiles in stages of 2 KB
            stage_kb = 8 if nt >= 8 else 16 if x_tiles < 8 else 12
            groups = -(-tiles // nt)
            for splits in range(1, 17 if may_split else 2):
                if stages % splits or (stages // splits < 4 and splits > 1):
                    continue
                # (a CU's LDS holds one such workgroup or two; two share what one would have alone)
                held, workgroups = min(2, 160 // ((nt + x_tiles) * stage_kb)), groups * splits
                rounds = -(-workgroups // (256 * held))
                cost = rounds * (stages // splits) * (0.25 * x_tiles + 0.45 * nt) + 0.5 * splits
                if held == 2 and workgroups > 256:
                    cost *= 1.8
                if rounds > 1:
                    cost *= 1.25  # (the last round is seldom full, and every round starts and ends)
                if best is None or cost < best[0]:
                    best = (cost, nt, splits, rounds)
        return best[1], best[2], best[3]

    @staticmethod
    def _medium_splits(out_features: int, in_features: int) -> int:
        """Into how many parts of K the product for 17 to 64 rows is cut when its float32 result may stay
        in parts: its workgroups own 64 weight rows and fill a CU each, so as many parts as give at most one
        workgroup a CU (the 1.5B sizes' down projection: 10 parts, 240 workgroups, 12.9 us at 64 rows against
        15.1 with 7 and 19.1 with 14)."""
        groups = in_features // 128
        if in_features % 128 or groups < 8:
            return 1
        tiles = -(-out_features // 64)
        best = 1
        for splits in range(2, 17):
            if groups % splits == 0 and groups // splits >= 4 and tiles * splits <= 256:
                best = splits
        return best

    @staticmethod
    def _library_splits(rows: int, out_features: int, in_features: int) -> int:
        """Into how many slices of K a library product is cut when its float32 result may stay partial sums:
        only where K is long beside N (a down projection), and as many (a power of two up to eight) as bring
        the 128 x 128 tiles of the result to about a thousand.  Measured on torch.mm against torch.bmm over
        slices: K 8,960 x N 1,536: 2,048 rows 72 -> 53 us in four, 512 rows 42 -> 26, below that nothing
        gained; K 18,944 x N 3,584: 2,048 rows 342 -> 217 in two, 1,024 rows 189 -> 114 in four, 512 rows
        129 -> 68 and 136 rows 103 -> 43 in eight; K 27,648 x N 5,120: 2,048 rows 453 whole or cut, 512 rows
        235 -> 130 in four, 136 rows 190 -> 78 in eight."""
        if in_features < 2 * out_features or in_features < 8192 or (in_features < 16384 and rows < 512):
            return 1
        tiles = -(-rows // 128) * -(-out_features // 128)
        wanted = 8
        while wanted > 1 and (wanted * tiles > 1000 or in_features % (wanted * 32)):
            wanted //= 2
        return wanted

    @staticmethod
    def _tiled_splits(rows: int, out_features: int, in_features: int) -> int:
        """Into how many parts of K the tiled product is cut when its float32 result may stay in
        parts: as many (at most 8, K / parts a multiple of 256) as it takes for the 256 x 256 tiles
        to number about 256, one for every CU."""
        tiles = -(-rows // 256) * -(-out_features // 256)
        best = 1
        for splits in range(2, 9):
            if in_features % (splits * 256) == 0 and tiles * (splits - 1) < 256:
                best = splits
        return best

    def linear(
        self, x: torch.Tensor, weights: LinearWeights, out_dtype: torch.dtype | None = None, *, partial: bool = False
    ) -> torch.Tensor:
        """`partial` allows a float32 result to come back as [parts, T, N] partial sums that
        the reader adds up in order (`add_rms_norm` and `gather_rows` do)."""
        rows, inner = x.shape
        if inner != weights.in_features:
            raise KernelError(f"linear: x has {inner} columns, the weight {weights.in_features}")
        bias = weights.bias
        streaming = self._streaming(x, weights, may_split=partial and out_dtype == torch.float32)
        if (
            streaming is None
            and not self.ring_products
            and partial
            and out_dtype == torch.float32
            and x.dtype == torch.bfloat16
            and weights.weight.dtype == torch.bfloat16
            and 16 < rows <= 64
            and inner % 128 == 0
            and self._partial_splits(weights.out_features, inner) >= 4
        ):
            # a long K over few weight rows (the down projection): cut over K into partial sums, the
            # hand-written kernel is ahead of the library (16 against 25 us at 64 rows of the 1.5B sizes)
            streaming = "medium"
        if streaming is None and self._library(x, weights):
            if (out_dtype or self.dtype) == torch.float32:  # float32 straight from the accumulators
                cuts = self._library_splits(rows, weights.out_features, inner) if partial and bias is None else 1
                if cuts > 1:
                    # The library does not cut a long K over workgroups by itself (the down projection of the 7B
                    # sizes at 2,048 rows: 342 us in one piece, 217 in two; at 136 rows 103 and 43 in eight).  As a
                    # strided batch of `cuts` products over slices of K it does, and the batch is the partial sums.
                    slices = x.view(rows, cuts, inner // cuts).transpose(0, 1)
                    weight_slices = weights.weight.view(weights.out_features, cuts, inner // cuts).permute(1, 2, 0)
                    return torch.bmm(slices, weight_slices, out_dtype=torch.float32)
                out = torch.mm(x, weights.weight.t(), out_dtype=torch.float32)
                return out if bias is None else out.add_(bias.float())
            if bias is not None and bias.dtype != x.dtype:
                return (torch.mm(x, weights.weight.t(), out_dtype=torch.float32) + bias).to(torch.bfloat16)
            return torch.nn.functional.linear(x, weights.weight, bias)
        bias_is_float = _is_float(bias) if bias is not None else 0
        if streaming is not None:
            splits = 1
            if streaming == "ring":
                tiles, splits, _ = self._ring_shape(rows, weights.out_features, inner, partial and out_dtype == torch.float32)
                out = self._empty((rows, weights.out_features) if splits == 1 else (splits, rows, weights.out_features), out_dtype or self.dtype)
                status = self._gemm_bf16.llmserve_gemm_ring(
                    _pointer(x), _pointer(weights.weight), _pointer(bias), bias_is_float, _pointer(out), _is_float(out), 0,
                    rows, weights.out_features, inner, splits, tiles, self._stream,
                )
                _check(status, "linear")
                return out
            if partial and out_dtype == torch.float32:
                if streaming == "tiled":
                    splits = self._tiled_splits(rows, weights.out_features, inner)
                elif streaming == "medium":
                    splits = self._medium_splits(weights.out_features, inner)
                elif rows > 16 and weights.out_features * inner <= (1 << 22) and inner % 256 == 0:
                    splits = 2  # what the kernel for a small weight at 17 to 64 rows does best with
                else:
                    splits = self._partial_splits(weights.out_features, inner)
            shape = (rows, weights.out_features) if splits == 1 else (splits, rows, weights.out_features)
            out = self._empty(shape, out_dtype or self.dtype)
            if streaming == "tiled":
                status = self._gemm_bf16.llmserve_gemm_tiled(
                    _pointer(x), _pointer(weights.weight), _pointer(bias), bias_is_float, _pointer(out),
                    _is_float(out), 0, rows, weights.out_features, inner, splits, self._stream,
                )
            else:
                entry = self._gemm_bf16.llmserve_gemm_skinny if streaming == "skinny" else self._gemm_bf16.llmserve_gemm_medium
                status = entry(
                    _pointer(x), _pointer(weights.weight), _pointer(bias), bias_is_float, _pointer(out),
                    _is_float(out), 0, rows, weights.out_features, inner, splits, self._stream,
                )
            _check(status, "linear")
            return out
        if self._all_float32(x, weights) and (out_dtype or self.dtype) == torch.float32:
            splits = self._float32_splits(rows, weights.out_features, inner) if partial and out_dtype == torch.float32 else 1
            shape = (rows, weights.out_features) if splits == 1 else (splits, rows, weights.out_features)
            out = self._empty(shape, torch.float32)
            status = self._gemm_f32.llmserve_gemm_f32(
                _pointer(x), _pointer(weights.weight), _pointer(bias), _pointer(out), 0, rows, weights.out_features,
                inner, splits, self._stream,
            )
            _check(status, "linear")
            return out
        out = self._empty((rows, weights.out_features), out_dtype or self.dtype)
        status = self._gemm_generic.llmserve_gemm_generic(
            _pointer(x), _is_float(x), _pointer(weights.weight), _is_float(weights.weight), _pointer(bias),
            bias_is_float, _pointer(out), _is_float(out), rows, weights.out_features, inner, self._stream,
        )
        _check(status, "linear")
        return out

    def _all_float32(self, x: torch.Tensor, weights: LinearWeights) -> bool:
        """Whether the product is the true 32-bit path's: every operand float32 and a K that its 16-byte
        loads can take (the generic kernel takes the rest: mixed types, any K)."""
        return (
            self._gemm_f32 is not None
            and x.dtype == torch.float32
            and weights.weight.dtype == torch.float32
            and (weights.bias is None or weights.bias.dtype == torch.float32)
            and weights.in_features % 4 == 0
        )

    @staticmethod
    def _float32_splits(rows: int, out_features: int, in_features: int) -> int:
        """Into how many parts of K a float32 product is cut when its result may stay in parts: up to 64
        rows (the weight-streaming kernel, workgroups of 16 weight rows) until about a thousand workgroups
        run, a part at least 512 long; more rows (128 x 128 tiles) until there is one tile for every CU."""
        if rows <= 64:
            tiles, least, goal = -(-out_features // 16), 512, 1024
        else:
            tiles, least, goal = -(-rows // 128) * -(-out_features // 128), 256, 256
        best = 1
        for splits in range(2, 9):
            if in_features // splits >= least and tiles * splits <= goal:
                best = splits
        return best

    def gated_linear(self, x: torch.Tensor, weights: GatedLinearWeights) -> torch.Tensor:
        """silu (or another activation) of the even rows' products times the odd rows'."""
        out = self._empty((x.shape[0], weights.width), self.dtype)
        if weights.activation != "silu":  # no fused epilogue: the product plain, the activation behind it
            both = self.linear(x, weights.both, out_dtype=torch.bfloat16 if self._library(x, weights.both) else torch.float32)
            status = self._elementwise.llmserve_gate_mul(
                _pointer(both), _is_float(both), _pointer(out), _is_float(out), x.shape[0], weights.width,
                _ACTIVATIONS[weights.activation], self._stream,
            )
            _check(status, "gate_mul")
            return out
        if self._all_float32(x, weights.both) and self.dtype == torch.float32:
            status = self._gemm_f32.llmserve_gemm_f32(
                _pointer(x), _pointer(weights.both.weight), None, _pointer(out), 1, x.shape[0], 2 * weights.width,
                x.shape[1], 1, self._stream,
            )
            _check(status, "gated_linear")
            return out
        streaming = self._streaming(x, weights.both, gated=True)
        if streaming == "ring":
            tiles, _, _ = self._ring_shape(x.shape[0], 2 * weights.width, x.shape[1], False)
            status = self._gemm_bf16.llmserve_gemm_ring(
                _pointer(x), _pointer(weights.both.weight), None, 0, _pointer(out), _is_float(out), 1, x.shape[0],
                2 * weights.width, x.shape[1], 1, tiles, self._stream,
            )
            _check(status, "gated_linear")
            return out
        if streaming is not None:
            if streaming == "tiled":
                status = self._gemm_bf16.llmserve_gemm_tiled(
                    _pointer(x), _pointer(weights.both.weight), None, 0, _pointer(out), _is_float(out), 1,
                    x.shape[0], 2 * weights.width, x.shape[1], 1, self._stream,
                )
                _check(status, "gated_linear")
                return out
            entry = self._gemm_bf16.llmserve_gemm_skinny if streaming == "skinny" else self._gemm_bf16.llmserve_gemm_medium
            status = entry(
                _pointer(x), _pointer(weights.both.weight), _pointer(None), 0, _pointer(out), _is_float(out), 1,
                x.shape[0], 2 * weights.width, x.shape[1], 1, self._stream,
            )
            _check(status, "gated_linear")
            return out
        both = self.linear(x, weights.both, out_dtype=torch.bfloat16 if self._library(x, weights.both) else torch.float32)
        status = self._elementwise.llmserve_silu_mul(
            _pointer(both), _is_float(both), _pointer(out), _is_float(out), x.shape[0], weights.width, self._stream
        )
        _check(status, "silu_mul")
        return out

    # ------------------------------------------------------------------ attention

    def _attention_library(self, head_dim: int):
        if head_dim not in self._attention_bf16:
            self._attention_bf16[head_dim] = _declared(load_module("attention_bf16", {"HEAD_DIM": head_dim}))
        return self._attention_bf16[head_dim]

    @staticmethod
    def _work_items(chunks, group: int, column_tiles: int, longer_than: int, up_to: int | None, packed: bool | None = None):
        """Work items (request, first row, first head, columns), int32 [items, 4], for the requests of
        the step whose token count lies in (longer_than, up_to], and about how many 32-key steps the
        items walk all together.  With up to 16 query heads a kv head (`group`), or `packed` set, an item is
        a run of `column_tiles` * 16 (token, head) pairs of a request, token by token and head by head,
        wherever in a token it begins; else `column_tiles` tokens (and "columns" counts tokens)."""
        import numpy as np

        counts = np.array([chunk.count for chunk in chunks], dtype=np.int64)
        starts = np.concatenate([[0], np.cumsum(counts)[:-1]])
        chosen = counts > longer_than
        if up_to is not None:
            chosen &= counts <= up_to
        which = np.nonzero(chosen)[0]
        packed = group <= 16 if packed is None else packed
        per_token = group if packed else 1
        per_item = column_tiles * (16 if packed else 1)
        totals = counts[which] * per_token
        items = -(-totals // per_item)
        request = np.repeat(which, items)
        inside = np.arange(int(items.sum())) - np.repeat(np.cumsum(items) - items, items)
        first = inside * per_item
        columns = np.minimum(per_item, np.repeat(totals, items) - first)
        work = np.stack([request, starts[request] + first // per_token, first % per_token, columns], axis=1).astype(np.int32)
        begins = np.array([chunk.start for chunk in chunks], dtype=np.int64)[which]
        steps = int((items * ((begins + counts[which] / 2) / 32 + 1)).sum())
        # The kernels start the list's last item first, and an item walks the keys up to its last token: in the
        # order of those positions the longest walks start first, whichever request they belong to (portions of
        # several requests at different depths of their prompts).
        last_position = np.repeat(begins, items) + (first + columns - 1) // per_token
        work = work[np.argsort(last_position, kind="stable")]
        return work, steps

    @staticmethod
    def _work_capacity(padded_to: tuple[int, int], group: int, column_tiles: int, packed: bool | None = None) -> int:
        """The most items a work list can have in a step of `padded_to` = (tokens, requests)."""
        tokens, requests = padded_to
        packed = group <= 16 if packed is None else packed
        per_token = group if packed else 1
        per_item = column_tiles * (16 if packed else 1)
        return -(-tokens * per_token // per_item) + requests

    def _attention_work(self, batch, group: int, column_tiles: int, longer_than: int, up_to: int | None, packed: bool | None = None):
        """The work list of `_work_items` on the device, built once per step and kept on the batch:
        (tensor or None, items, steps).  A batch that is `padded_to` (tokens, requests) for a captured
        step gets a list of the most items such a step can have, the unused ones of no columns: the
        captured launch covers whatever step is replayed, once `refresh_step` has filled in its items."""
        key = ("attention_work", group, column_tiles, longer_than, up_to, packed)
        if key not in batch.scratch:
            work, steps = self._work_items(batch.chunks, group, column_tiles, longer_than, up_to, packed)
            padded_to = getattr(batch, "padded_to", None)
            if padded_to is not None:
                import numpy as np

                capacity = self._work_capacity(padded_to, group, column_tiles, packed)
                if len(work) > capacity:
                    raise KernelError("a step holds more attention work than its padded shape allows")
                work = np.concatenate([work, np.zeros((capacity - len(work), 4), np.int32)])
            batch.scratch[key] = (self.to_device(torch.from_numpy(work)) if len(work) else None, len(work), steps)
        return batch.scratch[key]

    def refresh_step(self, batch, turn: int = 0) -> None:
        """For a batch whose kernels were captured: `batch.chunks` now describes another step of the
        same padded shape; everything this library derived from the chunks on the host (the attention
        work lists) is made anew, in place, at the addresses the captured kernels read.  The lists go
        through pinned staging buffers, two of each, used in turn (`turn` 0 or 1): the caller does not
        come back to a turn before the copies it queued in it have left their buffers."""
        import numpy as np

        for key in [key for key in batch.scratch if key[0] == "attention_work"]:
            tensor, capacity, _ = batch.scratch[key]
            if tensor is None:
                continue
            work, _ = self._work_items(batch.chunks, *key[1:])
            if len(work) > capacity:
                raise KernelError("a step holds more attention work than the captured step has room for")
            staging = batch.scratch.get(("staging", key))
            if staging is None:
                staging = [torch.zeros((capacity, 4), dtype=torch.int32, pin_memory=True) for _ in range(2)]
                batch.scratch[("staging", key)] = staging
            host = staging[turn].numpy()
            host[: len(work)] = work
            host[len(work):] = 0
            tensor.copy_(staging[turn], non_blocking=True)

    def paged_attention(
        self, qkv, layout, batch, cell, scale: float, window: int | None, *,
        score_slopes: torch.Tensor | None = None, soft_cap: float | None = None,
    ) -> torch.Tensor:
        """`score_slopes` (float32 [heads]) and `soft_cap` change the scores before the softmax: cap * tanh(score /
        cap), then minus slope * distance.  The matrix-core kernels of both precisions take them (in bfloat16
        not the forms that fuse the rotation or share keys through LDS)."""
        tokens = qkv.shape[0]
        group = batch.groups[cell.group]
        if cell.keys.dtype != qkv.dtype:
            raise KernelError("paged_attention: queries and pages differ in type")
        if score_slopes is not None and (score_slopes.dtype != torch.float32 or score_slopes.shape != (layout.num_heads,)):
            raise KernelError("paged_attention: score_slopes is one float32 per query head")
        if soft_cap is not None and not soft_cap > 0:
            raise KernelError("paged_attention: soft_cap must be positive")
        out = self._empty((tokens, layout.num_heads * layout.head_dim), qkv.dtype)
        dim = layout.head_dim
        plain_scores = score_slopes is None and soft_cap is None
        if qkv.dtype == torch.bfloat16 and group.page_size % 8 == 0 and dim % 16 == 0 and 16 <= dim <= 256:
            changed = None if plain_scores else (score_slopes, float(soft_cap or 0.0))
            self._attention_tiles(qkv, out, layout, batch, cell, group, scale, int(window or 0), changed=changed)
            return out
        if qkv.dtype == torch.float32 and group.page_size % 4 == 0 and dim % 16 == 0 and 16 <= dim <= 256:
            self._attention_float32(qkv, out, layout, batch, cell, group, scale, int(window or 0), score_slopes, soft_cap)
            return out
        if qkv.dtype == torch.bfloat16:
            why = f"head size {dim} and pages of {group.page_size}"
            self._tell_once(f"generic attention: {why}", f"bfloat16 attention runs on the generic kernel, not on the matrix cores: {why}")
        status = self._attention_generic.llmserve_attention_generic(
            _pointer(qkv), layout.width, _pointer(out), _is_float(qkv), _pointer(cell.keys), _pointer(cell.values),
            _pointer(group.block_tables), group.width, _pointer(batch.token_sequence), _pointer(batch.positions),
            tokens, layout.num_heads, layout.num_kv_heads, dim, group.page_size,
            scale, int(window or 0), _pointer(score_slopes), float(soft_cap or 0.0), self._stream,
        )
        _check(status, "paged_attention")
        return out

    def _attention_float32(self, qkv, out, layout, batch, cell, group, scale: float, window: int, score_slopes=None, soft_cap=None) -> None:
        """The 32-bit path's attention on the matrix cores: an item is 16 (decoding) or 32 columns of one
        request, (token, head) pairs running through the tokens head by head whatever the number of heads; few
        items over long contexts are cut into key splits that a second kernel merges."""
        dim = layout.head_dim
        if dim not in self._attention_f32:
            self._attention_f32[dim] = _declared(load_module("attention_f32", {"HEAD_DIM": dim}))
        heads, kv_heads = layout.num_heads, layout.num_kv_heads
        group_size = heads // kv_heads
        column_tiles = 2 if batch.max_query_length * group_size > 16 else 1
        work, items, _ = self._attention_work(batch, group_size, column_tiles, 0, None, True)
        if items == 0:
            return
        tokens = qkv.shape[0]
        # A wave walks its share of the keys 16 at a time, a trip to memory and sixty-four products a step, so a
        # walk is as long as its steps are many: where the chip has room for more workgroups the keys are split
        # until a wave has two steps or so (a decode step of 8 requests over 530 keys: 61 us unsplit; the merge
        # kernel costs about 5).
        steps = -(-batch.max_context_length // 16)
        splits = max(1, min(32, 1024 // (items * kv_heads), steps // 8))
        partial_acc = partial_ml = None
        if splits > 1:
            partial_acc = self._empty((splits, tokens * heads, dim), torch.float32)
            partial_ml = self._empty((splits, tokens * heads, 2), torch.float32)
        status = self._attention_f32[dim].llmserve_attention_f32(
            _pointer(qkv), layout.width, _pointer(out), _pointer(partial_acc), _pointer(partial_ml), _pointer(cell.keys),
            _pointer(cell.values), _pointer(group.block_tables), group.width, _pointer(batch.positions), _pointer(work),
            items, column_tiles, tokens, heads, kv_heads, group.page_size, scale, window, splits, _pointer(score_slopes),
            float(soft_cap or 0.0), self._stream,
        )
        _check(status, "paged_attention")

    def _attention_tiles(self, qkv, out, layout, batch, cell, group, scale: float, window: int, fuse=None, unmerged=False, changed=None):
        """The MFMA kernel: requests that bring a few tokens (decoding) one column tile per
        wave, split over the keys when there are few of them; longer portions two tiles
        per wave.  `fuse` = (rotary table, pairing) lets a step of single tokens rotate and
        store inside the same kernel.  With `unmerged` (a step of single tokens whose reader merges
        key splits itself) the keys are split more finely and the splits are returned as they are
        (their results in bfloat16, laid out for `gemm_merged`; their maxima and sums in float32; how
        many), instead of `out`.  `changed` = (slopes or None, soft cap or 0.0): scores changed before the softmax,
        which neither `fuse` nor the kernel that shares keys through LDS takes."""
        if changed is not None and fuse is not None:
            raise KernelError("paged_attention: the fused decode form takes plain scores only")
        slopes, soft_cap = changed if changed is not None else (None, 0.0)
        library = self._attention_library(layout.head_dim)
        heads, kv_heads = layout.num_heads, layout.num_kv_heads
        per_tile = max(1, 16 // (heads // kv_heads))
        head_tiles = -(-(heads // kv_heads) // 16)
        tokens = qkv.shape[0]
        group_size = heads // kv_heads
        launches = [(1, *self._attention_work(batch, group_size, 1, 0, per_tile)[:2])]
        shared = False
        padded = getattr(batch, "padded_to", None) is not None  # a captured step: the same launches whatever it holds
        whole_pages = group.page_size >= 16 and group.page_size & (group.page_size - 1) == 0  # (what that kernel takes)
        if batch.max_query_length > per_tile and layout.head_dim == 128 and fuse is None and changed is None and self.shared_portions != "never" and not padded and whole_pages:
            # Prompt portions at this head size may go to the kernel whose waves share each step's K and V
            # through LDS (a quarter of the cache traffic; what bounds the kernel above over long walks is the
            # path from the caches into the registers).  Its workgroups take 128 columns and walk all their keys,
            # so there are few of them: 192 for a 2,048-token portion of the 1.5B sizes, where the chip holds 512
            # and the kernel above would start 768.  So it is taken where it has 400 workgroups by itself (or
            # half as many very short walks), and where walks of 256 steps or more can be cut into runs of at
            # least 64 steps that a second kernel merges, 768 workgroups or so.  Measured (us, this kernel against
            # the one above, the same box and process): at 12 / 2 heads one prompt of 8,192 tokens 289 / 333,
            # eight of 2,048 202 / 236, sixteen of 512 47 / 71, a 2,048-token portion behind 8,192 keys 142 / 152
            # (four runs), behind 16,384 245-254 / 305-315, behind 32,704 455-485 / 593-706, 512 tokens behind
            # 32,704 168 / 272; at 28 / 4 heads (448 workgroups a 2,048-token portion) behind 4,096 to 8,192 keys
            # 133-262 / 142-287, behind 32,704 1,035 / 1,223, one prompt of 8,192 582 / 729; left to the kernel
            # above at 12 / 2 heads: one prompt of 2,048 to 6,144 tokens (43 / 66, 95 / 116, 188 / 209 the other
            # way round) and a portion behind up to 6,144 keys (112 / 116).
            work, items, steps = self._attention_work(batch, group_size, 8, per_tile, None)
            groups = items * kv_heads * head_tiles
            longest = -(-batch.max_context_length // 32)
            splits = 1
            if groups >= 400 or (groups >= 192 and longest <= 32):
                shared = True
                # Enough workgroups, but one request's portion may lie far deeper in its prompt than the others':
                # where the longest walk is well beyond a slot's share of all walks the kernel would wait for those
                # few workgroups, and all walks are cut (the short ones into runs of a few steps).
                share = max(1, steps * kv_heads * head_tiles // 512)
                if longest >= 256 and 2 * longest > 3 * share:
                    splits = max(1, min(8, longest // 64, -(-longest // share)))
            elif longest >= 256:
                splits = max(1, min(8, longest // 64, -(-768 // groups)))
                shared = groups * splits >= 384
            if self.portion_splits:
                splits = int(self.portion_splits)
            shared = shared or self.shared_portions == "always"
        if shared:
            partial_acc = partial_ml = None
            if splits > 1:
                partial_acc = self._empty((tokens * heads * splits * layout.head_dim,), torch.float32)
                partial_ml = self._empty((tokens * heads * splits * 2,), torch.float32)
            status = library.llmserve_attention_portions(
                _pointer(qkv), layout.width, _pointer(out), _pointer(partial_acc), _pointer(partial_ml), _pointer(cell.keys),
                _pointer(cell.values), _pointer(group.block_tables), group.width, _pointer(batch.positions), _pointer(work),
                items, 2, tokens, heads, kv_heads, group.page_size, scale, window, splits, self._stream,
            )
            _check(status, "paged_attention")
        elif batch.max_query_length > per_tile:
            # two column tiles a wave (heads wider than 128 leave no registers for more than one); four, at
            # one wave a SIMD, were ahead beyond 4,096 keys only while the key pages were whole rows
            wide = 1 if layout.head_dim > 128 else 2
            # One launch takes the requests of few tokens along (a decoded token fills part of a tile): in a
            # step of portions beside decoded tokens two launches one after the other cost 11 us each at the
            # 1.5B sizes, and the walk of a decoded token's keys is the same in either kernel.
            launches = [(wide, *self._attention_work(batch, group_size, wide, 0, None)[:2])]
        for column_tiles, work, items in launches:
            if items == 0:
                continue
            splits, partial_acc, partial_ml = 1, None, None
            by_item = False
            if shared:
                # The few short requests (decoded tokens) of a step whose portions went to the other kernel: alone
                # in this launch, so a long context is walked by one workgroup a kv head (30,000 keys: 237 us) unless
                # it is cut; their partial results are kept by item, not by the step's rows, which are mostly the
                # portions'.
                longest_few = max((chunk.start + chunk.count for chunk in batch.chunks if chunk.count <= per_tile), default=0)
                steps = -(-longest_few // 32)
                # (about 384 workgroups of four waves in all, as many waves as the 192 of a step of single tokens:
                # 63 decoded tokens over 2,048 keys beside a 2,048-token portion at 40 / 8 heads 510 -> 478 us)
                splits = max(1, min(-(-steps // 32), max(1, 384 // (items * kv_heads * head_tiles)), 64))
                if splits > 1:
                    by_item = True
                    partial_acc = self._empty((items * per_tile * heads * splits * layout.head_dim,), torch.float32)
                    partial_ml = self._empty((items * per_tile * heads * splits * 2,), torch.float32)
            elif batch.max_query_length <= per_tile:  # few tiles, maybe long: split the keys
                # a wave walks its share of the keys step after step (32 keys each), and a walk of
                # a few steps costs less than the second kernel that merges splits: split only when
                # a wave would walk more than 8 steps and the chip has room for more workgroups.  Room: about
                # 192 workgroups of eight waves in all, swept over 1 to 64 requests and 1,500 to 30,000 keys at
                # 12 / 2 heads (us a layer, the splits this gives against the 2,048 workgroups allowed before: 64
                # requests over 4,096 keys 40.6 / 47.4, over 2,500 27.2 / 33.4, over 1,500 18.8 / 21.8; 32 over
                # 8,192 44.0 / 47.0; 16 over 16,384 43.9 / 48.1; up to 8 requests as before).
                blocks = items * kv_heads * head_tiles
                steps = -(-batch.max_context_length // 32)
                splits = max(1, min(-(-steps // 32), max(1, 192 // blocks), 64))
                if unmerged:
                    # Nothing merges in a kernel of its own here, so a split costs only what its reader pays to
                    # read it (about 0.8 us a split in the product): a workgroup's eight waves get one step each.
                    # Attention and product together at 8 rows of the 1.5B sizes, captured, against 15.3 us
                    # unsplit at 530 keys and 22.1 at 1,000: two splits 14.5 and 18.6, four 14.7 and 16.5, eight
                    # 17.0 and 17.8.
                    # The product takes up to eight splits.  Where the tables reach beyond 4,096 keys the
                    # kernel that merges (one trip for all splits' maxima and sums) is a small share of the
                    # walk and that way is taken (8 rows of the 1.5B sizes, a whole step, product against
                    # kernel: 2,048 keys in tables of 4,096 1.54 and 1.58 ms; 4,096 keys in tables of 8,192
                    # 1.65 and 1.62; 6,000 keys 1.73 and 1.71; 8,192 keys 1.83 and 1.76; 30,000 keys 2.76 and
                    # 2.71; 16 rows over 4,096 keys 1.93 and 1.88, one row 1.49 and 1.46).
                    if splits <= 4:
                        wanted = min(-(-steps // 8), max(1, 1024 // blocks), 8)
                        splits = next(allowed for allowed in (1, 2, 3, 4, 6, 8) if allowed >= wanted)
                    else:
                        unmerged = False
                if not unmerged and 24 <= blocks <= 48:
                    # Some tens of workgroups over a short context: since the kernel that merges asks for all splits at
                    # once, runs of a few steps pay where the chip has room (us a layer at 32 workgroups, unsplit
                    # against six runs: 640 keys 11.4 / 9.9, 1,024 keys 15.7 / 11.5; a whole step at the 7B sizes
                    # 3.33 -> 3.28 ms). At 64 workgroups three runs tie (12.5 / 12.3, the 32B step alike); at 16 they
                    # lose (8.7 / 8.9).
                    splits = max(splits, min(-(-steps // 4), 192 // blocks))
                if not unmerged and blocks <= 8 and steps >= 128:
                    # very few requests over a long context: runs of 16 steps, two a wave (one request over 8,192
                    # keys 12.6 -> 11.5 us a layer, four 15.1 -> 13.4)
                    splits = max(splits, min(-(-steps // 16), 192 // blocks, 64))
                if splits > 1:
                    held = 16 if unmerged else tokens  # the product that merges wants 16 rows side by side
                    partial_acc = self._empty((held * heads * splits * layout.head_dim,), qkv.dtype if unmerged else torch.float32)
                    partial_ml = self._empty((held * heads * splits * 2,), torch.float32)
            table, pairing = fuse if fuse is not None else (None, "none")
            status = library.llmserve_attention_tiles(
                _pointer(qkv), layout.width, _pointer(out), _pointer(partial_acc), _pointer(partial_ml),
                _pointer(cell.keys), _pointer(cell.values), _pointer(group.block_tables), group.width, _pointer(batch.positions), _pointer(work), items, column_tiles, tokens, heads, kv_heads,
                group.page_size, scale, window, splits, (1 if fuse is not None else 0) + (2 if unmerged else 0) + (4 if by_item else 0),
                _pointer(table), _PAIRINGS[pairing], _pointer(group.slot_mapping), _pointer(slopes), soft_cap, self._stream,
            )
            _check(status, "paged_attention")
            if unmerged and splits > 1:
                return partial_acc, partial_ml, splits
        return None

    def rotate_store_attend(
        self, qkv, layout, batch, cell, inverse_frequencies, pairing: str, scale: float, window: int | None,
        project: LinearWeights | None = None,
    ) -> torch.Tensor:
        """`rotate_and_store` followed by `paged_attention`; one kernel when every request of
        the step brings a single token and the MFMA kernel takes the sizes.  With `project`, the result
        is `linear(that, project, float32, partial=True)`: for up to 16 single tokens at head size 128
        the attention leaves its key splits unmerged and the product merges them as it loads its x."""
        out, projected = self._rotate_store_attend(qkv, layout, batch, cell, inverse_frequencies, pairing, scale, window, project)
        if project is None or projected:
            return out
        return self.linear(out, project, out_dtype=torch.float32, partial=True)

    def _rotate_store_attend(self, qkv, layout, batch, cell, inverse_frequencies, pairing, scale, window, project):
        """(the attention's output, False) or, where the key splits were left to the product, (the product's, True)."""
        group = batch.groups[cell.group]
        dim = layout.head_dim
        if (
            batch.max_query_length == 1
            and cell.writable
            and qkv.dtype == torch.bfloat16
            and cell.keys.dtype == torch.bfloat16
            and group.page_size % 8 == 0
            and dim % 16 == 0
            and 16 <= dim <= 256
            and self._attention_library(dim).llmserve_attention_can_fuse(_PAIRINGS[pairing])
        ):
            out = self._empty((qkv.shape[0], layout.num_heads * dim), qkv.dtype)
            table = self.rotary_table(batch, inverse_frequencies) if pairing != "none" else None
            rows = qkv.shape[0]
            merging = (
                project is not None
                and self.merge_in_product
                and dim == 128
                and rows <= 16
                and project.weight.dtype == torch.bfloat16
                and project.in_features == layout.num_heads * dim
                # Every workgroup of the product reads all splits of its K range, rows * splits / 16 times the bytes
                # of its weights more than a plain product, and the kernel that merges as it loads is built for a
                # small weight (one tile a wave).  Ahead at the 1.5B sizes (4.7 MB of weights: attention and projection
                # 14.5 us against 15.3), behind at the 7B sizes (25.7 MB) at every number of rows, also where the
                # splits are few bytes (a step of 1 / 2 / 4 / 8 rows 3.27 / 3.31 / 3.36 / 3.82 ms against 3.21 / 3.24 /
                # 3.29 / 3.67 with the merging kernel): what decides is the weight, so the gate is its size.
                and project.weight.numel() * project.weight.element_size() <= self.merge_weight_bytes
            )
            left = self._attention_tiles(qkv, out, layout, batch, cell, group, scale, int(window or 0), fuse=(table, pairing), unmerged=merging)
            if left is None:
                return out, False
            split_x, split_ml, splits = left
            k_splits = self._partial_splits(project.out_features, project.in_features)
            shape = (rows, project.out_features) if k_splits == 1 else (k_splits, rows, project.out_features)
            result = self._empty(shape, torch.float32)
            bias = project.bias
            status = self._gemm_bf16.llmserve_gemm_merged(
                _pointer(split_x), _pointer(split_ml), splits, _pointer(project.weight), _pointer(bias),
                _is_float(bias) if bias is not None else 0, _pointer(result), rows, project.out_features,
                project.in_features, k_splits, self._stream,
            )
            _check(status, "linear over unmerged key splits")
            return result, True
        self.rotate_and_store(qkv, layout, batch, cell, inverse_frequencies, pairing)
        return self.paged_attention(qkv, layout, batch, cell, scale, window), False

    # ------------------------------------------------------------------ sampling

    def _sampling_library(self):
        if self._sampling is None:
            self._sampling = _declared(load_module("sampling"))
        return self._sampling

    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        rows, vocab = logits.shape
        out = self._empty((rows,), torch.int32)
        piece_values = self._empty((rows * 64,), torch.float32)
        piece_indices = self._empty((rows * 64,), torch.int32)
        status = self._sampling_library().llmserve_argmax(
            _pointer(logits), _pointer(piece_values), _pointer(piece_indices), _pointer(out), rows, vocab, self._stream
        )
        _check(status, "argmax")
        return out

    def sample(self, logits, temperatures, top_ps, uniforms, with_top_p: bool = True) -> torch.Tensor:
        rows, vocab = logits.shape
        out = self._empty((rows,), torch.int32)
        library = self._sampling_library()
        kib = library.llmserve_sample_workspace_kib(rows, vocab)
        if kib <= 0:
            raise KernelError(f"sample: no workspace for {rows} rows of {vocab}")
        workspace = self._empty((kib * 1024,), torch.uint8)
        status = library.llmserve_sample(
            _pointer(logits), _pointer(temperatures), _pointer(top_ps), _pointer(uniforms), _pointer(workspace), kib,
            _pointer(out), rows, vocab, 1 if with_top_p else 0, self._stream,
        )
        _check(status, "sample")
        return out
