"""The attention kernels and the engine at the context lengths that are measured and
published: rows that decode over 8,200 to 40,000 keys (every way the keys are split over
workgroups: the cap of 64 splits, the limit of table entries a split keeps in LDS, a
window), portions of prompts behind up to 32,256 keys and one portion of 8,192 tokens in
every form of the prefill kernel, the variants that take the raw projections, and one
request of 9,000 tokens through the whole engine against the plain implementation.

Random keys weigh about the same, so a block of keys that is skipped or counted twice
among tens of thousands would stay below bfloat16 rounding.  The sweeps therefore plant one
key that takes all the weight, at one position after the other, and ask for its value."""
import math

import numpy as np
import pytest
import torch

from test_kernels_gpu import make_step, ref_attention

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF = torch.bfloat16


@pytest.fixture(scope="module")
def ops():
    from tiny_llm_infer_amd.kernels.ops import HipOps
    return HipOps(DEV)


def fill(step, tables, seq_lens, kv_heads, hd, seed, k_std=1.0, v_std=1.0):
    """Keys and values of whole sequences, drawn on the device and scattered into their pages
    in one indexed assignment a sequence; returns them ([tokens, kv heads, head_dim] each)."""
    gen = torch.Generator(device=DEV).manual_seed(seed)
    page = step.cache.group.page_size
    ks, vs = [], []
    for i, n in enumerate(seq_lens):
        kk = (torch.randn((n, kv_heads, hd), generator=gen, device=DEV) * k_std).to(BF)
        vv = (torch.randn((n, kv_heads, hd), generator=gen, device=DEV) * v_std).to(BF)
        t = torch.arange(n, device=DEV)
        pages = torch.as_tensor(tables[i], device=DEV).long()[t // page]
        step.cache.k[pages, :, t % page] = kk
        step.cache.v[pages, :, :, t % page] = vv
        ks.append(kk)
        vs.append(vv)
    return ks, vs


def ref_attention_dev(q, ks, vs, pos, seq, heads, kv_heads, scale, window, chunk=256):
    """``ref_attention`` of the kernel tests in float64 on the device, rows of a sequence
    taken ``chunk`` at a time against all the keys they can see."""
    T, hd = q.shape[0], q.shape[1] // heads
    group = heads // kv_heads
    q = q.to(DEV).double().reshape(T, kv_heads, group, hd)
    out = torch.empty((T, kv_heads, group, hd), dtype=torch.float64, device=DEV)
    pos_t = torch.as_tensor(np.asarray(pos), device=DEV)
    seq_a = np.asarray(seq)
    for s in np.unique(seq_a):
        rows = np.nonzero(seq_a == s)[0]
        K, V = ks[s].to(DEV).double(), vs[s].to(DEV).double()
        for c0 in range(0, len(rows), chunk):
            r = torch.as_tensor(rows[c0:c0 + chunk], device=DEV)
            p = pos_t[r]
            hi = int(p.max()) + 1
            lo = 0 if not window else max(0, int(p.min()) - window + 1)
            n = torch.arange(lo, hi, device=DEV)
            seen = n[None, :] <= p[:, None]
            if window:
                seen &= n[None, :] > (p[:, None] - window)
            s_ = torch.einsum("ckgd,nkd->ckgn", q[r], K[lo:hi]) * scale
            s_.masked_fill_(~seen[:, None, None, :], float("-inf"))
            out[r] = torch.einsum("ckgn,nkd->ckgd", torch.softmax(s_, -1), V[lo:hi])
    return out.reshape(T, heads * hd)


def rnd_dev(shape, seed, std=1.0):
    gen = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(shape, generator=gen, device=DEV) * std).to(BF)


def close(got, want, what, tol=1.2e-2, scale=None):
    want = want.to(DEV).double()
    s = float(want.abs().max()) if scale is None else scale
    err = float((got.double() - want).abs().max())
    assert err <= tol * s, f"{what}: error {err:.3e} against scale {s:.3e}"


def test_the_device_reference_is_the_loop_reference():
    """The float64 reference used at these lengths against the row by row one of the
    kernel tests, at a size where that one is quick: two sequences, grouped heads, a window."""
    heads, kv_heads, hd = 6, 2, 32
    seq_lens, counts = [70, 33], [40, 1]
    g = torch.Generator().manual_seed(1)
    ks = [torch.randn((n, kv_heads, hd), generator=g) for n in seq_lens]
    vs = [torch.randn((n, kv_heads, hd), generator=g) for n in seq_lens]
    pos = list(range(30, 70)) + [32]
    seq = [0] * 40 + [1]
    q = torch.randn((41, heads * hd), generator=g)
    for window in (None, 19):
        a = ref_attention(q, ks, vs, pos, seq, heads, kv_heads, 0.3, window)
        b = ref_attention_dev(q, ks, vs, pos, seq, heads, kv_heads, 0.3, window, chunk=16)
        assert float((a - b.cpu()).abs().max()) < 1e-12


def rotary_table(hd, positions, theta=1e6):
    half = hd // 2
    ang = torch.arange(positions, dtype=torch.float64)[:, None] * (theta ** (-2.0 * torch.arange(half, dtype=torch.float64) / hd))[None, :]
    return torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)


def raw_reference(qkv, pos, heads, kv_heads, hd, qw, kw, eps_q, eps_k, cos, sin):
    """q, k, v of the raw projections in float64 on the device: per-head norm, rotation of halves."""
    T = qkv.shape[0]
    qd, kd = heads * hd, kv_heads * hd
    x = qkv.to(DEV).double()
    qq = x[:, :qd].reshape(T, heads, hd)
    kk = x[:, qd:qd + kd].reshape(T, kv_heads, hd)
    vv = x[:, qd + kd:].reshape(T, kv_heads, hd)
    qq = qw.double() * qq / torch.sqrt((qq * qq).mean(-1, keepdim=True) + eps_q)
    kk = kw.double() * kk / torch.sqrt((kk * kk).mean(-1, keepdim=True) + eps_k)
    p = torch.as_tensor(np.asarray(pos), device=DEV).long()
    c, s = cos.double()[p][:, None, :], sin.double()[p][:, None, :]
    half = hd // 2

    def rot(t):
        a, b = t[..., :half], t[..., half:]
        return torch.cat([a * c - b * s, a * s + b * c], -1)
    return rot(qq), rot(kk), vv


# ------------------------------------------------------------------- decode --
DECODE_CASES = {
    # heads, kv_heads, head_dim, page, seq_lens, window
    "one-row-32000": (32, 8, 128, 16, [32000], None),
    "eight-rows": (32, 8, 128, 16, [8200, 16400, 32000, 5, 700, 8191, 8193, 12000], None),
    # 40,000 keys of one row over two kv heads: as many splits as the cap of 64 allows
    "cap-of-64-splits": (16, 2, 128, 8, [40000], None),
    # 256 (row, kv head) pairs fill the chip without a split: the keys are split all the same,
    # because a split keeps its table entries in LDS (pages of 8: 32,000 keys are 4,000 entries)
    "table-entries-a-split": (32, 32, 64, 8, [32000, 100, 9000, 16400, 33, 64, 8200, 1], None),
    "window-4096": (8, 2, 128, 16, [32000, 16400], 4096),
    "window-1000-page-8": (8, 8, 64, 8, [16400], 1000),
}


def _decode_case(case, seed=3):
    heads, kv_heads, hd, page, seq_lens, window = case
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 7
    step, tables, pos, seq = make_step(seq_lens, [1] * len(seq_lens), page, num_pages, seed, kv_heads, hd, BF, window)
    return step, tables, pos, seq


@pytest.mark.parametrize("name", list(DECODE_CASES))
def test_decode_rows_with_long_contexts(ops, name):
    """Random queries, keys and values against float64: the queries given (the kernel that
    reads finished queries), and from the raw projections (the kernel of a decode step, which
    norms and rotates q and k itself and writes the row's own key and value)."""
    case = DECODE_CASES[name]
    heads, kv_heads, hd, page, seq_lens, window = case
    step, tables, pos, seq = _decode_case(case)
    g = step.cache.group
    splits, per_split, _ = ops._decode_splits(len(seq_lens), step.reach, g, heads, kv_heads, hd, window)
    print(f"{name}: reach {step.reach}, {splits} splits of {per_split} keys, table width {g.table_width}")
    if name == "cap-of-64-splits":
        assert splits == 64 and step.reach // ops.DECODE_SPLIT_KEYS >= 64
    if name == "table-entries-a-split":
        assert splits > 1 and len(seq_lens) * kv_heads >= ops.DECODE_WORKGROUPS
    assert per_split // page <= 2046
    ks, vs = fill(step, tables, seq_lens, kv_heads, hd, 100)
    scale = 1.0 / math.sqrt(hd)
    q = rnd_dev((len(pos), heads * hd), 50)
    out = ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, scale, window)
    close(out, ref_attention_dev(q, ks, vs, pos, seq, heads, kv_heads, scale, window), f"{name}: decode attention")
    # from the raw projections
    T = len(pos)
    qkv = rnd_dev((T, (heads + 2 * kv_heads) * hd), 21)
    qw, kw = (1 + rnd_dev((hd,), 22, 0.2).float()), (1 + rnd_dev((hd,), 23, 0.2).float())
    cos, sin = rotary_table(hd, max(seq_lens))
    qq, kk, vv = raw_reference(qkv, pos, heads, kv_heads, hd, qw, kw, 1e-5, 3e-6, cos, sin)
    out = ops.qkv_attention(qkv, step, step.cache, heads, kv_heads, hd, (qw, 1e-5), (kw, 3e-6), (cos, sin, hd),
                            scale, window)
    for r in range(T):                      # the rows' own keys and values replace what the cache held there
        ks[seq[r]][pos[r]] = kk[r].to(BF)
        vs[seq[r]][pos[r]] = vv[r].to(BF)
    want = ref_attention_dev(qq.reshape(T, heads * hd).to(BF), ks, vs, pos, seq, heads, kv_heads, scale, window)
    close(out, want, f"{name}: decode attention from raw projections")
    for r in range(T):
        p = int(tables[seq[r], pos[r] // page])
        close(step.cache.k[p, :, pos[r] % page], kk[r], f"{name}: the row's key in the cache")
        assert torch.equal(step.cache.v[p, :, :, pos[r] % page], vv[r].to(BF))


def test_decode_rows_of_unequal_lengths_are_split_by_their_skew(ops):
    """One long sequence among many short ones: told of the skew (the runner sets it from the lengths),
    the launch rule splits the keys although the rows alone fill the chip, and not otherwise; both
    launches against float64, and the planted key of the long row found in every split."""
    heads, kv_heads, hd, page = 32, 8, 128, 16
    seq_lens = [4000] + [300] * 31
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 5
    step, tables, pos, seq = make_step(seq_lens, [1] * len(seq_lens), page, num_pages, 5, kv_heads, hd, BF, None)
    g = step.cache.group
    assert ops._decode_splits(len(seq_lens), step.reach, g, heads, kv_heads, hd, None)[0] == 1
    splits, per_split, _ = ops._decode_splits(len(seq_lens), step.reach, g, heads, kv_heads, hd, None, skew=8)
    assert splits > 1
    assert ops._decode_splits(len(seq_lens), step.reach, g, heads, kv_heads, hd, 1024, skew=8)[0] == 1     # a window evens the rows out
    ks, vs = fill(step, tables, seq_lens, kv_heads, hd, 100)
    scale = 1.0 / math.sqrt(hd)
    q = rnd_dev((len(pos), heads * hd), 50)
    want = ref_attention_dev(q, ks, vs, pos, seq, heads, kv_heads, scale, None)
    close(ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, scale, None), want, "unsplit")
    step.skew = 8
    close(ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, scale, None), want, "split by the skew")
    # a key that takes all the weight, in each split of the long row in turn
    table0 = torch.as_tensor(tables[0], device=DEV).long()
    q[0, :] = 2.0
    for spot in [per_split * i + d for i in range(splits) for d in (0, per_split // 2) if per_split * i + d < seq_lens[0]]:
        k, v = step.cache.k, step.cache.v
        p, slot = int(table0[spot // page]), spot % page
        old_k, old_v = k[p, :, slot].clone(), v[p, :, :, slot].clone()
        k[p, :, slot] = 4.0
        v[p, :, :, slot] = 3.0
        out = ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, scale, None)
        assert (out[0].float() - 3.0).abs().max() < 0.05, f"key {spot}"
        k[p, :, slot], v[p, :, :, slot] = old_k, old_v


@pytest.mark.parametrize("name,stride", [("one-row-32000", 37), ("cap-of-64-splits", 41),
                                         ("table-entries-a-split", 53), ("window-4096", 7)])
def test_decode_finds_a_planted_key_wherever_it_lies(ops, name, stride):
    """One key of the first sequence takes all the weight; it is planted at every ``stride``-th
    position in turn (every slot of a page, every block of 32 keys, both sides of every edge
    between splits, the first key and the row's own) and the output has to be its value.  With
    a window, keys before it are planted too and must change nothing."""
    case = DECODE_CASES[name]
    heads, kv_heads, hd, page, seq_lens, window = case
    step, tables, pos, seq = _decode_case(case, seed=11)
    ks, vs = fill(step, tables, seq_lens, kv_heads, hd, 7, k_std=0.1)
    n = seq_lens[0]
    splits, per_split, _ = ops._decode_splits(len(seq_lens), step.reach, step.cache.group, heads, kv_heads, hd, window)
    q = rnd_dev((len(pos), heads * hd), 8, 0.1)
    q[0, :] = 2.0
    first_seen = 0 if not window else n - window
    spots = set(range(first_seen, n, stride)) | {first_seen, n - 1, n - 2}
    for e in range(per_split, n, per_split):           # both sides of the edges between splits
        spots |= {e - 1, e, e + 1} if not window else set()
    spots = sorted(s for s in spots if first_seen <= s < n)
    table0 = torch.as_tensor(tables[0], device=DEV).long()
    far_key = torch.full((kv_heads, hd), 4.0, dtype=BF, device=DEV)
    group = heads // kv_heads
    errs = []
    for far in spots:
        p, slot = table0[far // page], far % page
        kept = step.cache.k[p, :, slot].clone()
        step.cache.k[p, :, slot] = far_key
        out = ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, 1.0, window)
        step.cache.k[p, :, slot] = kept
        want = vs[0][far].float().repeat_interleave(group, 0).reshape(-1)
        errs.append((out[0].float() - want).abs().max())
    errs = torch.stack(errs).cpu()
    worst = int(errs.argmax())
    assert float(errs.max()) <= 1e-3, f"{name}: the key planted at {spots[worst]} of {n} was not found (error {float(errs.max()):.3e}; {splits} splits of {per_split})"
    print(f"{name}: {len(spots)} places, {splits} splits of {per_split} keys")
    if window:
        plain = ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, 1.0, window).clone()
        for far in (0, first_seen - 4097, first_seen - 33, first_seen - 2, first_seen - 1):
            p, slot = table0[far // page], far % page
            kept = step.cache.k[p, :, slot].clone()
            step.cache.k[p, :, slot] = far_key
            out = ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, 1.0, window)
            step.cache.k[p, :, slot] = kept
            assert torch.equal(out, plain), f"{name}: a key at {far}, before the window ({first_seen}), was seen"


# ------------------------------------------------------------------ prefill --
PREFILL_CASES = {
    # heads, kv_heads, head_dim, page, seq_lens, new rows, window
    "whole-8192": (8, 2, 128, 16, [8192], [8192], None),
    "512-behind-7680": (8, 2, 128, 16, [8192], [512], None),
    "512-behind-15872": (8, 2, 128, 16, [16384], [512], None),
    "512-behind-32256": (8, 2, 128, 16, [32768], [512], None),
    # pages of 8: the register that holds 64 table entries is filled again 64 times
    "512-behind-32256-page-8-window": (8, 4, 64, 8, [32768], [512], 5000),
    "two-portions": (16, 4, 128, 32, [16684, 9000], [300, 2], None),
}
# the prefill kernel's forms: as the launch rule picks; the rule told that the rows have keys before
# them; two sets of waves a workgroup; one set; two column tiles a wave; one
FORMS = {"rule": 0, "keys-before": 13, "two-sets": 10, "one-set": 11, "two-tiles": 3, "one-tile": 2}


@pytest.mark.parametrize("form", list(FORMS))
@pytest.mark.parametrize("name", list(PREFILL_CASES))
def test_portions_behind_long_contexts(ops, name, form):
    heads, kv_heads, hd, page, seq_lens, counts, window = PREFILL_CASES[name]
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 7
    step, tables, pos, seq = make_step(seq_lens, counts, page, num_pages, 5, kv_heads, hd, BF, window)
    ks, vs = fill(step, tables, seq_lens, kv_heads, hd, 100)
    scale = 1.0 / math.sqrt(hd)
    q = rnd_dev((len(pos), heads * hd), 50)
    ops.prefill_direct = FORMS[form]
    try:
        out = ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, scale, window)
    finally:
        ops.prefill_direct = 0
    close(out, ref_attention_dev(q, ks, vs, pos, seq, heads, kv_heads, scale, window), f"{name}/{form}")


@pytest.mark.parametrize("form", ["rule", "two-sets", "one-set"])
@pytest.mark.parametrize("name", ["whole-8192", "512-behind-32256", "512-behind-32256-page-8-window", "two-portions"])
def test_portions_from_raw_projections_behind_long_contexts(ops, name, form):
    """The prefill path of a step: keys and values of the portion normed, rotated and written
    into the pages, queries normed and rotated inside the attention kernel."""
    heads, kv_heads, hd, page, seq_lens, counts, window = PREFILL_CASES[name]
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 7
    step, tables, pos, seq = make_step(seq_lens, counts, page, num_pages, 5, kv_heads, hd, BF, window)
    ks, vs = fill(step, tables, seq_lens, kv_heads, hd, 100)
    T = len(pos)
    scale = 1.0 / math.sqrt(hd)
    qkv = rnd_dev((T, (heads + 2 * kv_heads) * hd), 21)
    qw, kw = (1 + rnd_dev((hd,), 22, 0.2).float()), (1 + rnd_dev((hd,), 23, 0.2).float())
    cos, sin = rotary_table(hd, max(seq_lens))
    qq, kk, vv = raw_reference(qkv, pos, heads, kv_heads, hd, qw, kw, 1e-5, 3e-6, cos, sin)
    ops.prefill_direct = FORMS[form]
    try:
        out = ops.qkv_attention(qkv, step, step.cache, heads, kv_heads, hd, (qw, 1e-5), (kw, 3e-6), (cos, sin, hd),
                                scale, window)
    finally:
        ops.prefill_direct = 0
    seq_a, pos_t = np.asarray(seq), torch.as_tensor(np.asarray(pos), device=DEV).long()
    for s in range(len(seq_lens)):
        rows = torch.as_tensor(np.nonzero(seq_a == s)[0], device=DEV)
        ks[s][pos_t[rows]] = kk[rows].to(BF)
        vs[s][pos_t[rows]] = vv[rows].to(BF)
    want = ref_attention_dev(qq.reshape(T, heads * hd).to(BF), ks, vs, pos, seq, heads, kv_heads, scale, window)
    close(out, want, f"{name}/{form}: attention from raw projections")


@pytest.mark.parametrize("form", ["rule", "two-sets", "one-set", "two-tiles"])
@pytest.mark.parametrize("name", ["512-behind-32256", "512-behind-32256-page-8-window", "whole-8192"])
def test_portions_find_a_planted_key(ops, name, form):
    """One key takes all the weight of every row that sees it: at the first position, at the
    edges of a block of 64 keys, where the register of 64 table entries is filled again, at the
    last key before the portion, inside it, and (with a window) at the window's edges."""
    heads, kv_heads, hd, page, seq_lens, counts, window = PREFILL_CASES[name]
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 7
    step, tables, pos, seq = make_step(seq_lens, counts, page, num_pages, 9, kv_heads, hd, BF, window)
    ks, vs = fill(step, tables, seq_lens, kv_heads, hd, 7, k_std=0.1)
    n, first_row = seq_lens[0], seq_lens[0] - counts[0]
    q = torch.full((len(pos), heads * hd), 2.0, dtype=BF, device=DEV)
    entries = 64 * page                                     # keys that one filling of the table register covers
    spots = {0, 31, 32, 63, 64, entries - 1, entries, entries + 1, 7 * entries - 1, 7 * entries, n // 2 + 5,
             first_row - 1, first_row, first_row + 100, n - 2, n - 1}
    if window:
        spots |= {first_row - window, first_row - window + 1, first_row - window + 300, n - window - 1, n - window}
    table0 = torch.as_tensor(tables[0], device=DEV).long()
    far_key = torch.full((kv_heads, hd), 4.0, dtype=BF, device=DEV)
    ops.prefill_direct = FORMS[form]
    try:
        for far in sorted(s for s in spots if 0 <= s < n):
            p, slot = table0[far // page], far % page
            kept = step.cache.k[p, :, slot].clone()
            step.cache.k[p, :, slot] = far_key
            ks[0][far] = far_key
            out = ops.paged_attention(q, step, step.cache, heads, kv_heads, hd, 1.0, window)
            want = ref_attention_dev(q, ks, vs, pos, seq, heads, kv_heads, 1.0, window)
            step.cache.k[p, :, slot] = kept
            ks[0][far] = kept
            close(out, want, f"{name}/{form}: key planted at {far}", scale=float(vs[0].float().abs().max()))
            sees = [r for r in range(len(pos)) if pos[r] >= far and (not window or pos[r] - window < far)]
            if sees:                                          # those rows' output is the planted key's value
                rows = torch.as_tensor(sees, device=DEV)
                value = vs[0][far].float().repeat_interleave(heads // kv_heads, 0).reshape(-1)
                assert float((out[rows].float() - value).abs().max()) <= 2e-2 * float(value.abs().max()), far
    finally:
        ops.prefill_direct = 0


def test_decoding_rows_with_long_contexts_beside_a_portion(ops):
    """A step as the scheduler makes it: two sequences that decode over 32,000 and 8,200 keys
    in front of a portion of 512 tokens behind 2,048.  The rows that decode go to the decode
    kernel (their keys split over workgroups), the portion to the prefill kernel."""
    heads, kv_heads, hd, page = 32, 8, 128, 16
    seq_lens, counts = [32000, 8200, 2560], [1, 1, 512]
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 7
    step, tables, pos, seq = make_step(seq_lens, counts, page, num_pages, 5, kv_heads, hd, BF, None)
    ks, vs = fill(step, tables, seq_lens, kv_heads, hd, 100)
    T = len(pos)
    scale = 1.0 / math.sqrt(hd)
    qkv = rnd_dev((T, (heads + 2 * kv_heads) * hd), 21)
    qw, kw = (1 + rnd_dev((hd,), 22, 0.2).float()), (1 + rnd_dev((hd,), 23, 0.2).float())
    cos, sin = rotary_table(hd, max(seq_lens))
    qq, kk, vv = raw_reference(qkv, pos, heads, kv_heads, hd, qw, kw, 1e-5, 3e-6, cos, sin)
    out = ops.qkv_attention(qkv, step, step.cache, heads, kv_heads, hd, (qw, 1e-5), (kw, 3e-6), (cos, sin, hd),
                            scale, None)
    seq_a, pos_t = np.asarray(seq), torch.as_tensor(np.asarray(pos), device=DEV).long()
    for s in range(len(seq_lens)):
        rows = torch.as_tensor(np.nonzero(seq_a == s)[0], device=DEV)
        ks[s][pos_t[rows]] = kk[rows].to(BF)
        vs[s][pos_t[rows]] = vv[rows].to(BF)
    want = ref_attention_dev(qq.reshape(T, heads * hd).to(BF), ks, vs, pos, seq, heads, kv_heads, scale, None)
    close(out, want, "rows that decode beside a portion")


# ------------------------------------------------------------------- engine --
LONG = 9000


@pytest.fixture(scope="module")
def long_request(tmp_path_factory):
    """Tiny configuration D with its position limit raised, one request of 9,000 tokens and
    the plain implementation's logits for it (computed once for both run dtypes)."""
    from helpers import TINY, config_json, plain_logits, random_prompt
    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.loading import write_random_model
    conf = dict(config_json("D"), max_position_embeddings=16384)
    folder = write_random_model(str(tmp_path_factory.mktemp("long") / "D"), "Qwen3ForCausalLM",
                                Qwen3Config.from_dict(conf), seed=41)
    reqs = {"r0": random_prompt(TINY["D"]["vocab_size"], LONG, 4)}
    return folder, reqs, plain_logits(folder, reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_of_9000_tokens_through_the_engine(long_request, dtype):
    """One windowed layer, one that keeps all keys, pages of 8: most of the request in one
    step and the last 32 tokens one by one, and in portions of 2 to 2,048 tokens, against the
    plain implementation.  Block tables of 1,125 entries, a window group that gives its
    pages back all the way."""
    from helpers import collect, max_error, trace_prefill_then_decode
    from tiny_llm_infer_amd.engine.loading import load_model
    from tiny_llm_infer_amd.engine.replay import Replayer
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    folder, reqs, want = long_request
    n = LONG
    sizes = [2, 1000, 17, 2048, 333, 5, 64, 1500, 2, 31]
    portions, at, k = [], 0, 0
    while at < n:
        m = min(sizes[k % len(sizes)], n - at)
        portions.append({"step": len(portions), "entries": [{"id": "r0", "tokens": reqs["r0"][at:at + m],
                                                              "want": list(range(m))}],
                         "end": ["r0"] if at + m == n else []})
        at, k = at + m, k + 1
    model, _ = load_model(folder, dtype, "cuda:0")
    tol = {"float32": 2e-5, "bfloat16": 2.5e-2}[dtype]
    for cut, steps in (("decode", trace_prefill_then_decode(reqs)), ("portions", portions)):
        runner = ModelRunner(model, model.env, page_size=8, num_pages=(n + 7) // 8 + 2, max_requests=2,
                             max_batch_tokens=n)
        rp = Replayer(runner)
        got = collect(steps, {st["step"]: rp.run_step(st) for st in steps})
        err, row, scale = max_error(got["r0"], want["r0"])
        print(f"9000 tokens, {dtype}, {cut}: worst error {err / scale:.2e} of the largest logit, at token {row}")
        assert err <= tol * scale, f"{dtype}/{cut}: error {err:.3e} at token {row} (logit scale {scale:.3e})"
        runner.cache.check()
        assert runner.cache.free_pages() == runner.cache.pages_per_group()


def test_a_long_request_decodes_beside_short_ones(long_request):
    """The 9,000-token request's last 24 tokens one by one in steps that five short requests share
    (bfloat16, recorded steps): the lengths are so unequal that the decode attention's keys are split
    by the skew, and every request's logits still are the plain implementation's."""
    from helpers import TINY, collect, max_error, plain_logits, random_prompt
    from tiny_llm_infer_amd.engine.loading import load_model
    from tiny_llm_infer_amd.engine.replay import Replayer
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    folder, reqs, want = long_request
    n, tail = LONG, 24
    short = {f"s{i}": random_prompt(TINY["D"]["vocab_size"], 40 + 31 * i + tail, 50 + i) for i in range(5)}
    want = dict(want, **plain_logits(folder, short))
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": reqs["r0"][:n - tail], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": rid, "tokens": toks[:-tail], "want": []} for rid, toks in short.items()], "end": []}]
    for j in range(tail):
        entries = [{"id": "r0", "tokens": [reqs["r0"][n - tail + j]], "want": [0]}]
        entries += [{"id": rid, "tokens": [toks[len(toks) - tail + j]], "want": [0]} for rid, toks in short.items()]
        steps.append({"step": len(steps), "entries": entries, "end": list(short) + ["r0"] if j == tail - 1 else []})
    model, _ = load_model(folder, "bfloat16", "cuda:0")
    runner = ModelRunner(model, model.env, page_size=8, num_pages=(n + 7) // 8 + 5 * 40 + 8, max_requests=6,
                         max_batch_tokens=n)
    seen = []
    rule = type(model.env.ops)._decode_splits

    def spy(self, T, reach, g, heads, kv_heads, head_dim, window, skew=1):
        out = rule(self, T, reach, g, heads, kv_heads, head_dim, window, skew)
        seen.append((skew, window, out[0]))
        return out
    type(model.env.ops)._decode_splits = spy
    try:
        rp = Replayer(runner)
        got = collect(steps, {st["step"]: rp.run_step(st) for st in steps})
    finally:
        type(model.env.ops)._decode_splits = rule
    assert any(skew > 1 and not window and splits > 1 for skew, window, splits in seen), seen[:8]
    assert runner.graph_replays >= tail - 2
    for rid, toks in dict(short, r0=reqs["r0"]).items():
        err, row, scale = max_error(got[rid], want[rid][len(toks) - tail:])
        assert err <= 2.5e-2 * scale, f"{rid}: error {err:.3e} at decoded token {row} (logit scale {scale:.3e})"
    runner.cache.check()
    assert runner.cache.free_pages() == runner.cache.pages_per_group()
