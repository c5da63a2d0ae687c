"""The matrix products of a decode step and of a prompt at the true layer shapes of the
larger models of the family (Qwen3-14B: hidden 5120, 40 query heads, intermediate 17408;
Qwen3-32B: hidden 5120, 64 query heads of 128 so that q is wider than the hidden size,
intermediate 25600), for 1 to 300 rows: every tuned kernel (the weight-streaming ones for
up to 16 rows with and without the norms taken in, the one for 17..128 rows with its split
of k and, for products without a gate, up to 256 rows as two row blocks, the one for more rows,
and the library) beside the plain float32 kernel on the same
bfloat16 values.  How the tuned kernels deal tiles and cut k depends on N and K, so shapes
that the smaller model never shows are compared here."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF = torch.bfloat16
SHAPES = {"14B": dict(H=5120, Q=5120, KV=1024, I=17408), "32B": dict(H=5120, Q=8192, KV=1024, I=25600)}
ROWS = [1, 8, 16, 64, 128, 200, 256, 300]


@pytest.fixture(scope="module")
def ops():
    from tiny_llm_infer_amd.kernels.ops import HipOps
    return HipOps(DEV)


def rnd(shape, seed, std=1.0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(shape, generator=g, device=DEV) * std).to(BF)


def near(got, want, what):
    """bfloat16 results against float32 ones: within 1.2e-2 of the largest value, as in
    the tests of the kernels at other sizes."""
    got, want = got.float(), want.float()
    scale = float(want.abs().max())
    err = float((got - want).abs().max())
    assert err <= 1.2e-2 * scale, f"{what}: error {err} against scale {scale}"


@pytest.mark.parametrize("which", list(SHAPES))
def test_products_of_a_layer_at_the_shapes_of_larger_models(ops, which):
    from tiny_llm_infer_amd.kernels.ops import DeferredSum, NormedRows, PendingProduct
    from tiny_llm_infer_amd.parts.base import BuildEnv
    from tiny_llm_infer_amd.parts.linear import GatedMatrix, Matrix
    s = SHAPES[which]
    H, Q, KV, I = s["H"], s["Q"], s["KV"], s["I"]
    env = BuildEnv(dtype=BF, device=torch.device(DEV), ops=ops, max_model_len=64)
    w_qkv, w_o = rnd((Q + 2 * KV, H), 1, 0.02), rnd((H, Q), 2, 0.02)
    w_gate, w_up, w_down = rnd((I, H), 3, 0.02), rnd((I, H), 4, 0.02), rnd((H, I), 5, 0.02)
    Wqkv, Wo, Wdown, Wgu = Matrix(w_qkv, env), Matrix(w_o, env), Matrix(w_down, env), GatedMatrix(w_gate, w_up, env)
    assert Wgu.gated is not None and Wqkv.tiled is not None
    norm_w = (1 + rnd((H,), 6, 0.1).float())
    eps = 1e-6

    def plain(x, w):
        return ops.linear_plain(x.float(), w.float())            # float32 FMA on the same bfloat16 values

    for M in ROWS:
        x, att, act = rnd((M, H), 10 + M), rnd((M, Q), 20 + M), rnd((M, I), 30 + M, 0.3)
        resid0 = rnd((M, H), 40 + M).float()
        want_qkv, want_o, want_down = plain(x, w_qkv), plain(att, w_o), plain(act, w_down)
        g, u = plain(x, w_gate), plain(x, w_up)
        want_act = torch.nn.functional.silu(g) * u
        modes = ("own", "library") if M > ops.MID_ROWS_TO else ("own",)
        for mode in modes:
            ops.many_rows = mode
            try:
                tag = f"{which}, {M} rows, {mode}"
                # q/k/v: what the attention takes (partial sums where k was split)
                near(ops.resolve(ops.linear(x, Wqkv, sums_only=True)), want_qkv, f"q/k/v product ({tag})")
                near(ops.linear_swiglu(x, Wgu), want_act, f"gated product ({tag})")
                # o and down: what the next norm takes as its delta
                for Wm, inp, want, what in ((Wo, att, want_o, "output projection"), (Wdown, act, want_down, "down projection")):
                    d = ops.linear(inp, Wm, deferred=True)
                    if M <= 16:
                        assert isinstance(d, PendingProduct)
                    near(ops.resolve(d), want, f"{what} ({tag})")
                    # and through the norm: the residual takes the sum, the rows are normed
                    r = resid0.clone()
                    n = ops.add_rmsnorm(r, ops.linear(inp, Wm, deferred=True), norm_w, eps, BF, lazy=True)
                    h = resid0 + want
                    assert float((r - h).abs().max()) <= 1.2e-2 * float(want.abs().max()), f"residual after the {what} ({tag})"
                    normed = norm_w * h * torch.rsqrt((h * h).mean(-1, keepdim=True) + eps)
                    if isinstance(n, NormedRows):               # up to 16 rows: the factor is still owed
                        assert M <= 16
                        near(ops.linear(n, Wqkv), plain(normed.to(BF), w_qkv), f"q/k/v of rows normed in the {what} ({tag})")
                        g2, u2 = plain(normed.to(BF), w_gate), plain(normed.to(BF), w_up)
                        near(ops.linear_swiglu(n, Wgu), torch.nn.functional.silu(g2) * u2,
                             f"gated product of rows normed in the {what} ({tag})")
                    else:
                        near(n, normed, f"norm after the {what} ({tag})")
            finally:
                ops.many_rows = "own"
