"""A stand-in for the HIP kernel library, in plain torch on the CPU, used only
by tests that check the engine's own logic (batch packing, block tables, cache
manager, run order, scheduler) without a GPU.  The product never loads this:
its kernel library is tiny_llm_infer_amd.kernels.ops.HipOps and nothing else.
"""
from __future__ import annotations

import torch


class CpuOps:
    name = "cpu-test-double"

    def check_attention_sizes(self, heads, kv_heads, head_dim):
        pass

    def check_page_size(self, page_size):
        pass

    def feed_tokens(self, token_ids, token_from, src, rows):
        take = token_from[:rows] >= 0
        token_ids[:rows][take] = src[token_from[:rows][take].long()]

    def embed(self, table, token_ids, num_rows):
        return table[token_ids.long()].to(torch.float32)

    def add_rmsnorm(self, resid, delta, weight, eps, out_dtype, rows=None, num_rows=None, lazy=False):
        if rows is None:
            if delta is not None:
                resid += delta.to(torch.float32)
            x = resid
        else:
            x = resid[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()].to(torch.float32)
        scale = torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)
        return (weight * x * scale).to(out_dtype)

    def resolve(self, y):
        return y

    def linear(self, x, w, out_dtype=None, deferred=False, sums_only=False):
        w = getattr(w, "w", w)
        y = x.to(torch.float32) @ w.to(torch.float32).t()
        return y.to(out_dtype or x.dtype)

    def linear_swiglu(self, x, m):
        return self.swiglu(self.linear(x, m))

    def swiglu(self, gu):
        inter = gu.shape[1] // 2
        g, u = gu[:, :inter].to(torch.float32), gu[:, inter:].to(torch.float32)
        return (g / (1 + torch.exp(-g)) * u).to(gu.dtype)

    def qkv_to_cache(self, qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary):
        T = step.num_rows
        qd, kd = heads * head_dim, kv_heads * head_dim
        x = qkv.to(torch.float32)
        q = x[:, :qd].reshape(T, heads, head_dim)
        k = x[:, qd:qd + kd].reshape(T, kv_heads, head_dim)
        v = x[:, qd + kd:].reshape(T, kv_heads, head_dim)

        def norm(t, wn):
            if wn is None:
                return t
            w, eps = wn
            return w * t * torch.rsqrt((t * t).mean(dim=-1, keepdim=True) + eps)

        q, k = norm(q, q_norm), norm(k, k_norm)
        pos = step.positions.long()
        if rotary is not None:
            cos, sin, rd = rotary
            half = rd // 2
            c, s = cos[pos][:, None, :], sin[pos][:, None, :]

            def rot(t):
                a, b, rest = t[..., :half], t[..., half:rd], t[..., rd:]
                return torch.cat([a * c - b * s, a * s + b * c, rest], dim=-1)
            q, k = rot(q), rot(k)
        if cache is not None and cache.writes:
            page = cache.group.page_size
            tables = cache.group.tables
            seq = step.seq_of_row.long()
            pages = tables[seq, pos // page].long()
            assert (pages >= 0).all(), "a row writes to a page that is not held"
            slots = pos % page
            cache.record("k")[pages, :, slots] = k.to(cache.record("k").dtype)
            cache.record("v")[pages, :, :, slots] = v.to(cache.record("v").dtype)        # values are kept transposed
        return q.reshape(T, qd).to(qkv.dtype)

    def qkv_attention(self, qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary, scale, window):
        q = self.qkv_to_cache(qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary)
        return self.paged_attention(q, step, cache, heads, kv_heads, head_dim, scale, window)

    def paged_attention(self, q, step, cache, heads, kv_heads, head_dim, scale, window):
        T = step.num_rows
        page = cache.group.page_size
        tables = cache.group.tables
        qf = q.to(torch.float32).reshape(T, heads, head_dim)
        out = torch.zeros(T, heads, head_dim, dtype=torch.float32)
        mul = heads // kv_heads
        pos_l = step.positions.tolist()
        seq_l = step.seq_of_row.tolist()
        for r in range(T):
            p = pos_l[r]
            lo = 0 if window is None else max(0, p - window + 1)
            idx = torch.arange(lo, p + 1)
            pages = tables[seq_l[r], idx // page].long()
            assert (pages >= 0).all(), "a row reads a page that is not held"
            kk = cache.record("k")[pages, :, idx % page].to(torch.float32)     # [n, kv, d]
            vv = cache.record("v")[pages, :, :, idx % page].to(torch.float32)
            for h in range(heads):
                s = (kk[:, h // mul] @ qf[r, h]) * scale
                w = torch.softmax(s, dim=0)
                out[r, h] = w @ vv[:, h // mul]
        return out.reshape(T, heads * head_dim).to(q.dtype)

    # ---- sampling: the same hash and rule as csrc/sampling.hip, in Python ----
    @staticmethod
    def _mix32(h):
        h &= 0xFFFFFFFF
        h ^= h >> 16
        h = (h * 0x85EBCA6B) & 0xFFFFFFFF
        h ^= h >> 13
        h = (h * 0xC2B2AE35) & 0xFFFFFFFF
        h ^= h >> 16
        return h

    @classmethod
    def uniform(cls, seed, token):
        seed &= (1 << 64) - 1
        lo, hi = seed & 0xFFFFFFFF, seed >> 32
        h = cls._mix32(token ^ 0x9E3779B9)
        h = cls._mix32(h ^ lo)
        h = cls._mix32((h + hi * 0x85EBCA6B + 0x27D4EB2F) & 0xFFFFFFFF)
        return ((h >> 9) + 0.5) / 8388608.0

    def sample(self, logits, temperatures=None, seeds=None, top_p=None):
        import math
        out = []
        for r in range(logits.shape[0]):
            row = logits[r].double()
            temp = 0.0 if temperatures is None else float(temperatures[r])
            if temp <= 1e-6:
                out.append(int(torch.argmax(row)))
                continue
            keep = torch.ones_like(row, dtype=torch.bool)
            if top_p is not None and float(top_p[r]) < 1.0:
                w = torch.exp((row - row.max()) / temp)
                order = torch.argsort(w, descending=True)
                csum = torch.cumsum(w[order], 0)
                n = int((csum < float(top_p[r]) * w.sum()).sum()) + 1
                keep[:] = False
                keep[order[:n]] = True
            seed = int(seeds[r])
            g = torch.tensor([-math.log(-math.log(self.uniform(seed, t))) for t in range(row.numel())],
                             dtype=torch.float64)
            score = torch.where(keep, row + temp * g, torch.full_like(row, -float("inf")))
            out.append(int(torch.argmax(score)))
        return torch.tensor(out, dtype=torch.int32)
