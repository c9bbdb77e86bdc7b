"""Helpers of the GPU tests: replaying traces through bin/trace_run."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent


def replay(folder: Path, dtype: str, steps: list[dict], out: Path, max_tokens: int, block_size: int,
           vocab: int, extra: tuple[str, ...] = ()) -> dict[int, torch.Tensor]:
    """Runs bin/trace_run on `steps` and returns {step: logits [wanted, vocab]}."""
    command = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype, "--out",
               str(out), "--max-tokens", str(max_tokens), "--block-size", str(block_size), *extra]
    text = "".join(json.dumps(step) + "\n" for step in steps)
    done = subprocess.run(command, input=text, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, f"trace_run failed:\n{done.stderr[-3000:]}"
    lines = [line for line in done.stdout.splitlines() if line.startswith("done ")]
    assert lines == [f"done {step['step']}" for step in steps], done.stdout[-2000:]
    results = {}
    for step in steps:
        wanted = sum(len(entry.get("want", ())) for entry in step["entries"])
        path = out / f"{step['step']}.f32"
        if wanted:
            data = np.fromfile(path, dtype="<f4")
            assert data.size == wanted * vocab, f"step {step['step']}: {data.size} values for {wanted} rows"
            results[step["step"]] = torch.from_numpy(data.reshape(wanted, vocab).copy())
        else:
            assert not path.exists()
    return results


class TraceBuilder:
    """Builds steps and remembers which (request, position) each wanted row is."""

    def __init__(self) -> None:
        self.steps: list[dict] = []
        self.rows: dict[int, list[tuple[str, int]]] = {}
        self.fed: dict[str, int] = {}

    def step(self, entries: list[tuple[str, list[int]]], end: list[str] = (), want: str = "all") -> None:
        number = len(self.steps)
        items, rows = [], []
        for name, tokens in entries:
            start = self.fed.get(name, 0)
            places = list(range(len(tokens))) if want == "all" else [len(tokens) - 1] if want == "last" else []
            items.append({"id": name, "tokens": list(tokens), "want": places})
            rows += [(name, start + place) for place in places]
            self.fed[name] = start + len(tokens)
        self.steps.append({"step": number, "entries": items, "end": list(end)})
        self.rows[number] = rows
        for name in end:
            del self.fed[name]

    def collect(self, results: dict[int, torch.Tensor]) -> dict[tuple[str, int], torch.Tensor]:
        found = {}
        for number, rows in self.rows.items():
            for index, key in enumerate(rows):
                found[key] = results[number][index]
        return found
