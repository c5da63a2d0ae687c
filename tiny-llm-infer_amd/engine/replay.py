"""Trace replay: given token ids go through the model step by step and the
logits at the wanted places are written out.  Nothing is sampled and nothing
is scheduled; the model, step function, cache and kernels are the ones that
generation uses.

A trace is a sequence of JSON objects, one a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: for each request its next tokens and the places among them whose
logits are wanted.  A request is admitted when it first appears.  ``end``:
requests that are finished after this step; what they hold is given back.

Output, in the folder given: ``<step>.f32`` for every step in which something
was wanted (little-endian float32 [wanted, vocab], in the order of the entries
and of ``want``), and ``index.jsonl``, one JSON object a step:

    {"step": 0, "file": "0.f32", "rows": [{"id": "a", "position": 0}, {"id": "a", "position": 2}],
     "block_tables": {"a": [[0]]}}

``rows`` names the request and the position in it of every row of the file;
``block_tables`` holds, for every request of the step and every group of cache
layers, the pages the step ran with: taken after the step's pages were reserved
and before a window gave any back (-1: given back by an earlier step).
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
        self.index = None
        if out_dir is not None:
            os.makedirs(out_dir, exist_ok=True)
            self.index = open(os.path.join(out_dir, "index.jsonl"), "w", encoding="utf-8")
            runner.keep_tables = True

    def close(self) -> None:
        if self.index is not None:
            self.index.close()
            self.index = None

    def run_step(self, record: dict) -> Optional[np.ndarray]:
        """Run one trace step; returns float32 [wanted, vocab] or None."""
        entries, rows = [], []
        for e in record.get("entries", []):
            key = e["id"]
            if key not in self.runner.cache:
                self.runner.admit(key)
            entries.append(StepEntry(key, [int(t) for t in e["tokens"]],
                                     [int(w) for w in e.get("want", [])]))
            at = self.runner.cache.get(key).num_tokens
            rows.extend({"id": key, "position": at + int(w)} for w in e.get("want", []))
        out = None
        if entries:
            logits = self.runner.step(entries)
            if logits is not None:
                out = logits.detach().to("cpu", torch.float32).numpy()      # a copy: the runner's buffer is written again
                if self.out_dir is not None:
                    out.astype("<f4").tofile(os.path.join(self.out_dir, f"{record['step']}.f32"))
        if self.index is not None:
            tables = {str(e.key): self.runner.tables_run[e.key] for e in entries}
            self.index.write(json.dumps({"step": record.get("step"), "file": f"{record['step']}.f32" if rows else None,
                                         "rows": rows, "block_tables": tables}) + "\n")
            self.index.flush()
        for key in record.get("end", []):
            if key in self.runner.cache:
                self.runner.release(key)
        return out

    def run_stream(self, lines: Iterable[str], ack: Optional[IO[str]] = None) -> None:
        try:
            for line in lines:
                line = line.strip()
                if not line:
                    continue
                record = json.loads(line)
                self.run_step(record)
                if ack is not None:
                    ack.write(f"done {record['step']}\n")
                    ack.flush()
        finally:
            self.close()
