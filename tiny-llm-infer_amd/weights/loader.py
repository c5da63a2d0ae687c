"""Loading a model's tensors by name, and writing a random-weights model folder.

What a model needs is a list of ``TensorDecl`` (name, shape, kind of
initialisation) collected from its parts.  ``load_tensors`` checks the whole
list against the checkpoint before reading anything and raises ONE
``WeightError`` that lists every missing tensor, every tensor of the wrong
shape and every tensor the model does not use.  (The reference stops at the
first problem: "Missing Qwen3 tensor", "Unexpected shape for Qwen3 tensor",
model/src/qwen3_layers.cpp:76-108.)

Storage rule: a floating tensor stored in 16 bits is kept in bfloat16 for a
bfloat16 run (float16 is converted) and widened exactly for a float32 run; a
tensor stored in 32 bits stays float32 in both; integer tables become int32.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Dict, Iterable, Iterator, List, Sequence, Tuple

import torch

from .safetensors_io import Checkpoint, write_safetensors


@dataclass(frozen=True)
class TensorDecl:
    name: str
    shape: Tuple[int, ...]
    init: str = "normal"      # "normal": N(0, 0.02); "ones_normal": 1 + N(0, 0.02); "int": zeros


class WeightError(ValueError):
    def __init__(self, missing: Sequence[str], wrong_shape: Sequence[Tuple[str, tuple, tuple]],
                 unexpected: Sequence[str], bad_dtype: Sequence[Tuple[str, str]] = ()):
        self.missing = list(missing)
        self.wrong_shape = list(wrong_shape)
        self.unexpected = list(unexpected)
        self.bad_dtype = list(bad_dtype)
        lines = ["the checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        if self.bad_dtype:
            lines.append(f"  unsupported dtypes ({len(self.bad_dtype)}): " + ", ".join(
                f"{n} is {d}" for n, d in self.bad_dtype))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        super().__init__("\n".join(lines))


def unique_decls(decls: Iterable[TensorDecl]) -> List[TensorDecl]:
    """Drop repeated declarations of one tensor (a tied head names the
    embedding's tensor again); the shapes must agree."""
    seen: Dict[str, TensorDecl] = {}
    for d in decls:
        if d.name in seen:
            if seen[d.name].shape != tuple(d.shape):
                raise ValueError(f"tensor '{d.name}' is declared with shapes "
                                 f"{seen[d.name].shape} and {tuple(d.shape)}")
            continue
        seen[d.name] = TensorDecl(d.name, tuple(d.shape), d.init)
    return list(seen.values())


def check_against(decls: Sequence[TensorDecl], checkpoint: Checkpoint) -> None:
    missing, wrong, bad = [], [], []
    wanted = set()
    for d in decls:
        wanted.add(d.name)
        if d.name not in checkpoint:
            missing.append(d.name)
            continue
        got = tuple(checkpoint.shape(d.name))
        if got != tuple(d.shape):
            wrong.append((d.name, got, tuple(d.shape)))
        dt = checkpoint.dtype(d.name)
        if d.init == "int":
            if dt.is_floating_point or dt == torch.bool:
                bad.append((d.name, str(dt)))
        elif dt not in (torch.bfloat16, torch.float16, torch.float32):
            bad.append((d.name, str(dt)))
    unexpected = sorted(n for n in checkpoint.names() if n not in wanted)
    if missing or wrong or unexpected or bad:
        raise WeightError(missing, wrong, unexpected, bad)


def stored_to_run_dtype(t: torch.Tensor, run_dtype: torch.dtype) -> torch.Tensor:
    if not t.dtype.is_floating_point:
        return t.to(torch.int32)
    if t.dtype == torch.float32:
        return t
    if run_dtype == torch.float32:
        return t.to(torch.float32)          # exact widening of bf16 / fp16
    return t.to(torch.bfloat16)


def load_tensors(model_path: str, decls: Sequence[TensorDecl], run_dtype: torch.dtype,
                 device) -> Iterator[Tuple[str, torch.Tensor]]:
    """Yield (name, tensor on ``device``) for every declared tensor, after the
    whole list has been checked against the files."""
    decls = unique_decls(decls)
    ck = Checkpoint(model_path)
    try:
        check_against(decls, ck)
        for d in decls:
            t = stored_to_run_dtype(ck.read(d.name), run_dtype)
            yield d.name, t.to(device, copy=True)
    finally:
        ck.close()


# --------------------------------------------------------------------------
# random weights
# --------------------------------------------------------------------------

def random_tensor(decl: TensorDecl, seed: int, index: int, dtype: torch.dtype,
                  device="cpu", std: float = 0.02) -> torch.Tensor:
    """The ``index``-th tensor of a random model: N(0, std^2) ("normal") or N(1, std^2)
    ("ones_normal") in float32, every element a function of (seed, index, its place) alone and
    the same bits wherever it is drawn (``random_init.draw_normal``), then rounded to ``dtype``."""
    if decl.init == "int":
        return torch.zeros(decl.shape, dtype=torch.int32, device=device)
    if decl.init not in ("normal", "ones_normal"):
        raise ValueError(f"unknown initialisation '{decl.init}' for {decl.name}")
    from .random_init import draw_normal
    t = draw_normal(tuple(decl.shape), seed, index, std, 1.0 if decl.init == "ones_normal" else 0.0, device)
    return t.to(dtype)


def random_tensors(decls: Sequence[TensorDecl], seed: int, dtype: torch.dtype,
                   device="cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    for i, d in enumerate(unique_decls(decls)):
        yield d.name, random_tensor(d, seed, i, dtype, device)


def write_model_folder(folder: str, config_json: dict, decls: Sequence[TensorDecl], seed: int,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Random-weights mode: write ``config.json`` and ``model.safetensors``."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config_json, fh, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      random_tensors(decls, seed, dtype))
    return folder
