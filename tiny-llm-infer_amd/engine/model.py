"""A model put together from a ``ModelSpec``: embedding, blocks, final norm,
head, and the order in which the blocks run."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import CacheNeed, StateNeed
from ..config.base import ConfigError, ModelSpec, PartSpec
from ..parts.base import BuildEnv, build_part
from ..weights.loader import TensorDecl, load_tensors, random_tensors, unique_decls


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = build_part("embedding", spec.embedding)
        self.blocks = []
        for b in spec.blocks:
            mixer = build_part("mixer", b.mixer)
            ffn = build_part("ffn", b.ffn) if b.ffn is not None else None
            norms = {role: build_part("norm", s) for role, s in b.norms.items()}
            self.blocks.append(build_part("block", PartSpec(b.arrangement), mixer, ffn, norms))
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.schedule = list(spec.schedule)
        self._check_schedule()

    def _check_schedule(self) -> None:
        written = set()
        needs: Dict[int, CacheNeed] = {}
        for i, call in enumerate(self.schedule):
            if not 0 <= call.block < len(self.blocks):
                raise ConfigError(f"run order entry {i} names block {call.block}, "
                                  f"the model has {len(self.blocks)}")
            need = self.blocks[call.block].mixer.cache_need()
            if need is None:
                continue
            if call.cache < 0:
                raise ConfigError(f"run order entry {i}: its mixer needs a cache layer")
            if call.cache in needs and needs[call.cache] != need:
                raise ConfigError(f"run order entry {i}: cache layer {call.cache} is used with "
                                  f"different sizes")
            needs[call.cache] = need
            if call.writes_cache:
                if call.cache in written:
                    raise ConfigError(f"run order entry {i}: cache layer {call.cache} is written twice")
                written.add(call.cache)
            elif call.cache not in written:
                raise ConfigError(f"run order entry {i} reads cache layer {call.cache} "
                                  f"before any entry writes it")
        self._needs = needs

    def cache_needs(self) -> List[Optional[CacheNeed]]:
        return [self._needs.get(i) for i in range(self.spec.num_cache_layers())]

    def state_needs(self) -> List[Optional[StateNeed]]:
        """Per run-order entry: the fixed-size state its mixer keeps per request."""
        return [self.blocks[c.block].mixer.state_need() for c in self.schedule]

    def tensors(self) -> List[TensorDecl]:
        out = self.embedding.tensors()
        for b in self.blocks:
            out += b.tensors()
        out += self.final_norm.tensors() + self.head.tensors()
        return unique_decls(out)

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        self.env = env
        self.embedding.load(weights, env)
        for b in self.blocks:
            b.load(weights, env)
        self.final_norm.load(weights, env)
        self.head.load(weights, env, share_with=self.embedding)

    def weight_bytes(self) -> int:
        """Bytes of device memory the loaded weights take: every tensor that a part holds (in
        whatever forms it holds a matrix), each storage counted once."""
        from ..parts.base import Part
        seen, total, stack = set(), 0, [self.embedding, self.final_norm, self.head, *self.blocks]
        visited = set()
        while stack:
            obj = stack.pop()
            if id(obj) in visited:
                continue
            visited.add(id(obj))
            if isinstance(obj, torch.Tensor):
                key = obj.untyped_storage().data_ptr()
                if key not in seen:
                    seen.add(key)
                    total += obj.untyped_storage().nbytes()
            elif isinstance(obj, (list, tuple)):
                stack.extend(obj)
            elif isinstance(obj, dict):
                stack.extend(obj.values())
            elif isinstance(obj, Part) or type(obj).__module__.endswith("parts.linear"):
                stack.extend(v for k, v in vars(obj).items() if k not in ("env", "ops", "spec"))
        return total

    # ---- convenience ------------------------------------------------------
    def load_from(self, model_path: str, env: BuildEnv) -> None:
        self._load_stream(load_tensors(model_path, self.tensors(), env.dtype, env.device), env)

    def load_random(self, seed: int, env: BuildEnv, stored: torch.dtype = torch.bfloat16) -> None:
        """Random weights drawn on the device, as if read from a file that
        stores them in ``stored``."""
        from ..weights.loader import stored_to_run_dtype
        gen = ((n, stored_to_run_dtype(t, env.dtype))
               for n, t in random_tensors(self.tensors(), seed, stored, env.device))
        self._load_stream(gen, env)

    def _load_stream(self, stream, env: BuildEnv) -> None:
        """Parts take their tensors block by block so that the unfused copies
        of a large model never all live on the device at once."""
        pending: Dict[str, torch.Tensor] = {}
        parts = [self.embedding] + self.blocks + [self.final_norm, self.head]
        wanted = [set(d.name for d in p.tensors()) for p in parts]
        done = [False] * len(parts)
        self.env = env

        def try_load():
            for i, p in enumerate(parts):
                if done[i] or not wanted[i] <= pending.keys():
                    continue
                if p is self.head:
                    if not done[0]:
                        continue
                    p.load(pending, env, share_with=self.embedding)
                else:
                    p.load(pending, env)
                done[i] = True
                still = set().union(*[wanted[j] for j in range(len(parts)) if not done[j]]) \
                    if not all(done) else set()
                for name in list(pending):
                    if name not in still:
                        del pending[name]

        for name, t in stream:
            pending[name] = t
            try_load()
        try_load()
        if not all(done):
            raise RuntimeError("some parts did not receive all their tensors")
