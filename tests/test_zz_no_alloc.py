"""The sampling entry point that allocates nothing (``tli_sample_no_alloc``, its scratch
in a device array of the library) against ``tli_sample`` (scratch brought by the caller),
called through ctypes: two calls in a row, the second with a smaller input, so that what
the first call left in the array must not show."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from tiny_llm_infer_amd.kernels import build
    path = build.find_library() or build.build_library()
    lib = ctypes.CDLL(path)
    P, I = ctypes.c_void_p, ctypes.c_int
    lib.tli_last_error.restype = ctypes.c_char_p
    lib.tli_sample.argtypes = [P, I, I, P, P, P, P, P, P]
    lib.tli_sample_no_alloc.argtypes = [P, I, I, P, P, P, P, P]
    lib.tli_sample_scratch_bytes.argtypes = [I]
    for fn in (lib.tli_sample, lib.tli_sample_no_alloc, lib.tli_sample_scratch_bytes,
               lib.tli_sample_no_alloc_max_rows, lib.tli_sample_no_alloc_prepare):
        fn.restype = I
    return lib


def _both(lib, logits, temperatures, seeds):
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    t = None if temperatures is None else temperatures.data_ptr()
    s = None if seeds is None else seeds.data_ptr()
    want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    scratch = torch.empty(lib.tli_sample_scratch_bytes(rows), dtype=torch.uint8, device="cuda")
    assert lib.tli_sample(logits.data_ptr(), rows, vocab, t, s, None, want.data_ptr(),
                          scratch.data_ptr(), stream) == 0, lib.tli_last_error()
    assert lib.tli_sample_no_alloc(logits.data_ptr(), rows, vocab, t, s, None, got.data_ptr(),
                                   stream) == 0, lib.tli_last_error()
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_sampling_without_allocation_matches_sampling_with_a_callers_scratch():
    lib = _library()
    gen = torch.Generator(device="cuda").manual_seed(5)
    # first call: 64 rows of a large vocabulary that is no power of two; second call: fewer
    # rows and a smaller vocabulary, with other winners
    for rows, vocab in ((64, 151936), (5, 9001)):
        logits = torch.randn((rows, vocab), generator=gen, device="cuda", dtype=torch.float32)
        got, want = _both(lib, logits, None, None)
        assert torch.equal(got, want)
        assert torch.equal(got.long(), logits.argmax(dim=1).cpu())
        temps = torch.full((rows,), 0.8, device="cuda", dtype=torch.float32)
        temps[0] = 0.0                                   # one greedy row among drawn ones
        seeds = torch.arange(100, 100 + rows, device="cuda", dtype=torch.int64)
        got, want = _both(lib, logits, temps, seeds)
        assert torch.equal(got, want)
        assert int(got[0]) == int(logits[0].argmax())
        assert not torch.equal(got.long(), logits.argmax(dim=1).cpu())   # the draws are draws
    # the drawn rows of the last (small) call against the rule itself, written out in numpy: token =
    # argmax(logit + T * Gumbel(u)), u the hash of (seed, token) that tli_sample_uniform gives
    import numpy as np

    def uniforms(seed, n):
        def mix(h):
            h = h.copy()
            h ^= h >> np.uint32(16); h *= np.uint32(0x85EBCA6B); h ^= h >> np.uint32(13)
            h *= np.uint32(0xC2B2AE35); h ^= h >> np.uint32(16)
            return h
        lo, hi = np.uint32(seed & 0xFFFFFFFF), np.uint32(seed >> 32)
        with np.errstate(over="ignore"):
            h = mix(np.arange(n, dtype=np.uint32) ^ np.uint32(0x9E3779B9))
            h = mix(h ^ lo)
            h = mix(h + hi * np.uint32(0x85EBCA6B) + np.uint32(0x27D4EB2F))
        return ((h >> np.uint32(9)).astype(np.float64) + 0.5) / 8388608.0

    lib.tli_sample_uniform.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32]
    lib.tli_sample_uniform.restype = ctypes.c_float
    assert all(uniforms(104, 50)[t] == lib.tli_sample_uniform(104, 0, t) for t in range(50))
    host = logits.double().cpu().numpy()
    for r in range(1, rows):
        score = host[r] + float(temps[r]) * -np.log(-np.log(uniforms(int(seeds[r]), vocab)))
        order = np.argsort(-score)
        assert int(got[r]) == int(order[0]) or score[order[0]] - score[int(got[r])] < 1e-5     # float32 noise on a near-tie
    # beyond the array's size: refused, nothing launched, the output untouched
    limit = lib.tli_sample_no_alloc_max_rows()
    out = torch.full((4,), 7, dtype=torch.int32, device="cuda")
    small = torch.zeros((4, 16), device="cuda")
    assert lib.tli_sample_no_alloc(small.data_ptr(), limit + 1, 16, None, None, None, out.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream) != 0
    assert b"rows" in lib.tli_last_error()
    torch.cuda.synchronize()
    assert out.tolist() == [7, 7, 7, 7]


def test_sampling_without_allocation_recorded_into_a_graph():
    """What the entry point is for: after the address of the array has been looked up outside
    any capture, the call is recorded into a HIP graph, which is replayed several times on new
    logits, with eager work and synchronisation between the replays; every replay gives what
    tli_sample gives for the same logits."""
    lib = _library()
    assert lib.tli_sample_no_alloc_prepare() == 0, lib.tli_last_error()
    rows, vocab = 9, 40007
    gen = torch.Generator(device="cuda").manual_seed(11)
    logits = torch.randn((rows, vocab), generator=gen, device="cuda", dtype=torch.float32)
    temps = torch.full((rows,), 0.9, device="cuda", dtype=torch.float32)
    temps[3] = 0.0
    seeds = torch.arange(7, 7 + rows, device="cuda", dtype=torch.int64)
    out = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        code = lib.tli_sample_no_alloc(logits.data_ptr(), rows, vocab, temps.data_ptr(), seeds.data_ptr(), None,
                                       out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert code == 0, lib.tli_last_error()
    for replay in range(4):
        logits.copy_(torch.randn((rows, vocab), generator=gen, device="cuda"))          # eager work between replays
        seeds += 1000
        graph.replay()
        torch.cuda.synchronize()
        want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        scratch = torch.empty(lib.tli_sample_scratch_bytes(rows), dtype=torch.uint8, device="cuda")
        assert lib.tli_sample(logits.data_ptr(), rows, vocab, temps.data_ptr(), seeds.data_ptr(), None,
                              want.data_ptr(), scratch.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {replay}"
        assert int(out[3]) == int(logits[3].argmax())
