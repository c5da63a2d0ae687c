"""Trace replay: given token ids go through the model step by step and the
logits at the wanted places are written out.  Nothing is sampled and nothing
is scheduled; the model, step function, cache and kernels are the ones that
generation uses.

A trace is a sequence of JSON objects, one a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: for each request its next tokens and the places among them whose
logits are wanted.  A request is admitted when it first appears.  ``end``:
requests that are finished after this step; what they hold is given back.
"""
from __future__ import annotations

import json
import os
import sys
from typing import Dict, IO, Iterable, Optional

import numpy as np
import torch

from .runner import ModelRunner, StepEntry


class Replayer:
    def __init__(self, runner: ModelRunner, out_dir: Optional[str] = None):
        self.runner = runner
        self.out_dir = out_dir
        if out_dir is not None:
            os.makedirs(out_dir, exist_ok=True)

    def run_step(self, record: dict) -> Optional[np.ndarray]:
        """Run one trace step; returns float32 [wanted, vocab] or None."""
        entries = []
        for e in record.get("entries", []):
            key = e["id"]
            if key not in self.runner.cache:
                self.runner.admit(key)
            entries.append(StepEntry(key, [int(t) for t in e["tokens"]],
                                     [int(w) for w in e.get("want", [])]))
        out = None
        if entries:
            logits = self.runner.step(entries)
            if logits is not None:
                out = logits.detach().to("cpu", torch.float32).numpy()
                if self.out_dir is not None:
                    out.astype("<f4").tofile(os.path.join(self.out_dir, f"{record['step']}.f32"))
        for key in record.get("end", []):
            if key in self.runner.cache:
                self.runner.release(key)
        return out

    def run_stream(self, lines: Iterable[str], ack: Optional[IO[str]] = None) -> None:
        for line in lines:
            line = line.strip()
            if not line:
                continue
            record = json.loads(line)
            self.run_step(record)
            if ack is not None:
                ack.write(f"done {record['step']}\n")
                ack.flush()
