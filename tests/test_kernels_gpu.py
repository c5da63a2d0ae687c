"""Each HIP kernel alone against a plain float64 reference of the same
operation, at sizes other than the engine's tiny configurations: odd widths,
head sizes in steps of 16, one and many kv heads, windows, permuted pages."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from tiny_llm_infer_amd.kernels.ops import HipOps
    return HipOps(DEV)


def tol(dtype, scale=1.0):
    return (3e-6 if dtype == torch.float32 else 1.2e-2) * scale


def rnd(shape, dtype, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def close(got, want, dtype, what, scale=None):
    got = got.detach().to("cpu", torch.float64)
    want = want.to(torch.float64)
    s = float(want.abs().max()) if scale is None else scale
    err = float((got - want).abs().max())
    assert err <= tol(dtype, max(s, 1e-6)), f"{what}: error {err} against scale {s}"


# ---------------------------------------------------------------- simple ops --
@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(ops, dtype):
    table = rnd((301, 80), dtype, 1)
    ids = torch.tensor([0, 300, 17, 17, 255], dtype=torch.int32)
    out = ops.embed(table.to(DEV), ids.to(DEV), 5)
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), table[ids.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [80, 100, 4096, 5120])
def test_add_rmsnorm(ops, dtype, n):
    rows = 7
    resid = rnd((rows, n), torch.float32, 2, 3.0)
    delta = rnd((rows, n), dtype, 3)
    w = 1 + rnd((n,), torch.float32, 4, 0.1)
    eps = 1e-5

    def ref(x):
        x = x.double()
        return w.double() * x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)

    # without delta the residual is untouched
    r = resid.to(DEV)
    out = ops.add_rmsnorm(r, None, w.to(DEV), eps, dtype)
    assert torch.equal(r.cpu(), resid)
    close(out, ref(resid), dtype, "norm")
    # with delta the residual takes the float32 sum
    out = ops.add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, dtype)
    total = resid + delta.float()
    assert torch.equal(r.cpu(), total)
    close(out, ref(total), dtype, "add+norm")
    # with a row list only those rows are computed and the residual is left alone
    r = resid.to(DEV)
    pick = torch.tensor([5, 0, 5], dtype=torch.int32)
    out = ops.add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, dtype, rows=pick.to(DEV))
    assert torch.equal(r.cpu(), resid)
    close(out, ref(total[pick.long()]), dtype, "gathered add+norm")


def test_rmsnorm_weight_is_a_plain_multiplier(ops):
    x = rnd((3, 96), torch.float32, 5)
    zero = ops.add_rmsnorm(x.to(DEV), None, torch.zeros(96, device=DEV), 1e-6, torch.float32)
    assert float(zero.abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [112, 12288])
def test_swiglu(ops, dtype, inter):
    gu = rnd((5, 2 * inter), dtype, 6, 2.0)
    out = ops.swiglu(gu.to(DEV))
    g, u = gu[:, :inter].double(), gu[:, inter:].double()
    close(out, torch.nn.functional.silu(g) * u, dtype, "swiglu")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mnk", [(1, 301, 80), (37, 130, 100), (130, 70, 257), (64, 64, 64), (3, 1000, 4096)])
def test_linear(ops, dtype, mnk):
    M, N, K = mnk
    x, w = rnd((M, K), dtype, 7), rnd((N, K), dtype, 8, 0.05)
    want = x.double() @ w.double().t()
    close(ops.linear(x.to(DEV), w.to(DEV)), want, dtype, "linear")
    y32 = ops.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32)
    assert y32.dtype == torch.float32
    close(y32, want, torch.float32 if dtype == torch.float32 else dtype, "linear, float32 out",
          scale=float(want.abs().max()) * (1.0 if dtype == torch.float32 else 0.05))


@pytest.mark.parametrize("mnk", [(300, 5120, 17408), (300, 5120, 25600), (64, 51200, 5120)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_plain_product_at_the_widths_it_is_the_reference_for(ops, dtype, mnk):
    """The plain kernel is what the tuned products are compared with at the widths of the
    larger models; here it is itself compared with float64 at those widths (the sum over
    17,408 and 25,600 terms, 51,200 outputs)."""
    M, N, K = mnk
    g = torch.Generator(device=DEV).manual_seed(K)
    x = torch.randn((M, K), generator=g, device=DEV).to(dtype)
    w = (torch.randn((N, K), generator=g, device=DEV) * 0.02).to(dtype)
    want = x.double() @ w.double().t()
    got = ops.linear_plain(x, w, out_dtype=torch.float32)
    # A float32 sum of K terms in a fixed order is off by about sqrt(K) roundings of 2^-24 of the
    # sum's own size (the largest of 1.5 million outputs by five times the typical one); one term
    # left out or taken twice would be off by 1/sqrt(K) of it, a hundred times more.
    err = float((got.double() - want).abs().max())
    allowed = 1e-7 * math.sqrt(K) * float(want.abs().max())
    assert err <= allowed, f"error {err} against {float(want.abs().max())}, allowed {allowed}"


SKINNY = [(1, 4096, 4096), (8, 6144, 4096), (8, 4096, 12288), (16, 301, 80), (17, 1000, 264),
          (33, 24576, 512), (64, 130, 4096), (5, 151936, 128), (48, 70, 8),
          (65, 1000, 264), (100, 4096, 4096), (128, 130, 1032), (96, 6144, 512), (40, 96, 64), (70, 40, 200)]


@pytest.mark.parametrize("mnk", SKINNY)
@pytest.mark.parametrize("out", [torch.bfloat16, torch.float32])
def test_skinny_linear_against_plain_kernel_and_reference(ops, mnk, out):
    """The weight-streaming MFMA kernels for up to 128 rows, beside the plain tiled kernel."""
    M, N, K = mnk
    x, w = rnd((M, K), torch.bfloat16, 7), rnd((N, K), torch.bfloat16, 8, 0.05)
    # x lies in front of NaNs: a kernel that reads past a row's end and uses it shows
    behind = torch.full((M * K + 8192,), float("nan"), dtype=torch.bfloat16, device=DEV)
    xd, wd = behind[:M * K].view(M, K), w.to(DEV)
    xd.copy_(x)
    got = ops.linear(xd, wd, out_dtype=out)
    plain = ops.linear_plain(xd, wd, out_dtype=out)
    want = x.double() @ w.double().t()
    scale = float(want.abs().max())
    # float32 out: only the order of the float32 additions differs
    bound = 2e-5 * scale * (K ** 0.5) / 8 + 1e-6 if out == torch.float32 else 1.2e-2 * scale

    class Both:                      # the matrix with its decode layout, as the parts hold it
        w = wd
        tiled = ops.tile_matrix(wd)
    streamed = ops.linear(xd, Both, out_dtype=out)
    if M < ops.MID_ROWS_FROM:
        assert torch.equal(streamed, got)      # same additions in the same order, other addresses
    else:                                      # 17..128 rows: the kernel that shares x through LDS
        assert float((streamed.double().cpu() - want).abs().max()) <= bound
        # (ranges of k, launch shape: depth of the rings, column tiles a wave, waves; also numbers of
        # waves that do not divide the copies of a slice of x)
        shapes = (((1, 224), (2, 228), (4, 314), (3, 418), (5, 424), (7, 218), (2, 223), (1, 225), (3, 226), (1, 227))
                  if M <= 64 else ((1, 224), (3, 214), (5, 0), (1, 223), (2, 225), (1, 227)))
        for splits, cfg in shapes:
            ops.mid_splits, ops.mid_cfg = splits, cfg
            try:
                again = ops.linear(xd, Both, out_dtype=out)
            finally:
                ops.mid_splits = ops.mid_cfg = 0
            assert float((again.double().cpu() - want).abs().max()) <= bound, (splits, cfg)
    want = x.double() @ w.double().t()
    scale = float(want.abs().max())
    # float32 out: only the order of the float32 additions differs
    bound = 2e-5 * scale * (K ** 0.5) / 8 + 1e-6 if out == torch.float32 else 1.2e-2 * scale
    assert float((got.double().cpu() - want).abs().max()) <= bound
    assert float((plain.double().cpu() - want).abs().max()) <= bound


@pytest.mark.parametrize("mki", [(1, 64, 32), (8, 4096, 12288), (33, 96, 160), (64, 264, 1008), (100, 264, 1008),
                                 (128, 4096, 1024)])
def test_gated_product_writes_the_activation(ops, mki):
    """gate and up interleaved in the decode layout: one pass, silu(g)*u in the epilogue."""
    from tiny_llm_infer_amd.engine.loading import make_env
    from tiny_llm_infer_amd.parts.linear import GatedMatrix
    M, K, I = mki
    env = make_env(torch.bfloat16, DEV)
    gate, up = rnd((I, K), torch.bfloat16, 3, 0.05), rnd((I, K), torch.bfloat16, 4, 0.05)
    x = rnd((M, K), torch.bfloat16, 5)
    m = GatedMatrix(gate.to(DEV), up.to(DEV), env)
    assert m.gated is not None
    got = ops.linear_swiglu(x.to(DEV), m)
    g, u = x.double() @ gate.double().t(), x.double() @ up.double().t()
    close(got, torch.nn.functional.silu(g) * u, torch.bfloat16, "gated product")
    two_pass = ops.swiglu(ops.linear(x.to(DEV), m.w))
    close(two_pass, torch.nn.functional.silu(g) * u, torch.bfloat16, "stacked product, then activation")


@pytest.mark.parametrize("mnk", [(129, 264, 1008), (200, 4096, 4096), (256, 6144, 520), (177, 1000, 136), (255, 48, 8), (144, 5120, 384)])
def test_two_row_blocks_side_by_side_in_the_x_sharing_kernel(ops, mnk):
    """129..256 rows of a product without a gate: two blocks of 128 rows of gemm_mid in one launch (the
    second block's workgroups run beside the first's and find the W fragments in their die's L2), at
    sizes that are no multiples of its tiles, with the planned and with forced launch shapes and ranges
    of k, the partial sums left for the consumer, and rows that do not depend on the rows beside them."""
    from tiny_llm_infer_amd.kernels.ops import DeferredSum
    M, N, K = mnk
    x, w = rnd((M, K), torch.bfloat16, 1), rnd((N, K), torch.bfloat16, 2, 0.05)
    behind = torch.full((M * K + 8192,), float("nan"), dtype=torch.bfloat16, device=DEV)     # x lies in front of NaNs
    xd = behind[:M * K].view(M, K)
    xd.copy_(x)
    tiled = ops.tile_matrix(w.to(DEV))
    want = x.double() @ w.double().t()

    def product(rows=M, deferred=False):
        y = torch.full((rows, N), 7.0, dtype=torch.bfloat16, device=DEV)
        return ops._linear_mid(xd[:rows], tiled, y, rows, N, K, 0, deferred)
    first = product()
    close(first, want, torch.bfloat16, "two row blocks")
    assert ops.lib.tli_gemm_mid_splits_rows(M, N, K, 0) >= 1
    for splits, cfg in ((1, 0), (2, 0), (5, 0), (1, 224), (3, 223), (2, 214), (4, 228)):
        ops.mid_splits, ops.mid_cfg = splits, cfg
        try:
            close(product(), want, torch.bfloat16, f"{splits} ranges of k, shape {cfg}")
            left = product(deferred=True)
            if splits > 1:
                assert isinstance(left, DeferredSum) and tuple(left.parts.shape) == (splits, M, N)
                close(left.parts.sum(0), want, torch.float32, "partial sums")
            close(ops.resolve(left), want, torch.bfloat16, "partial sums resolved")
        finally:
            ops.mid_splits = ops.mid_cfg = 0
    # fewer rows, still two blocks: the same bits for the rows that are there
    if M > 140:
        assert torch.equal(product(rows=M - 9), first[:M - 9])
    # through linear(), which takes this kernel for a matrix held in the decode layout
    class Both:
        tiled_ = tiled
    Both.w, Both.tiled = w.to(DEV), tiled
    assert torch.equal(ops.linear(xd, Both), first)


@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("mnk", [(129, 264, 1008), (300, 4096, 4096), (2048, 6144, 512), (513, 1000, 136), (700, 48, 8), (4500, 520, 256),
                                 (1024, 5120, 384)])
def test_product_of_many_rows_from_the_decode_layout(ops, mnk, cfg):
    """gemm_rows (the alternative to the library for more than 128 rows) against float64, at
    sizes that are no multiples of its tiles, with both launch shapes; rows do not depend
    on what else is in the batch."""
    M, N, K = mnk
    x, w = rnd((M, K), torch.bfloat16, 1).to(DEV), rnd((N, K), torch.bfloat16, 2).to(DEV)
    tiled = ops.tile_matrix(w)
    y = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.rows_cfg, ops.rows_splits = cfg, 1
    try:
        ops._linear_rows(x, tiled, y, M, N, K, 0)
        want = x.double().cpu() @ w.double().cpu().t()
        close(y, want, torch.bfloat16, "product of many rows")
        part = torch.empty((M // 3, N), dtype=torch.bfloat16, device=DEV)
        ops._linear_rows(x[M // 5:M // 5 + M // 3].contiguous(), tiled, part, M // 3, N, K, 0)
        assert torch.equal(part, y[M // 5:M // 5 + M // 3])
        # k cut into ranges (more than there are slices of 128, too): the sum of the partial products,
        # and the partial sums left for the consumer
        for splits in (0, 3, 16):
            ops.rows_splits = splits
            y2 = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
            close(ops._linear_rows(x, tiled, y2, M, N, K, 0), want, torch.bfloat16, f"{splits} ranges of k")
            left = ops._linear_rows(x, tiled, y2, M, N, K, 0, deferred=True)
            if splits > 1:
                assert tuple(left.parts.shape) == (splits, M, N)
                close(left.parts.sum(0), want, torch.float32, "partial sums")
            close(ops.resolve(left), want, torch.bfloat16, "partial sums resolved")
    finally:
        ops.rows_cfg = ops.rows_splits = 0


@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("mki", [(130, 264, 1008), (2048, 512, 1536), (300, 4096, 96), (260, 256, 400)])
def test_gated_product_of_many_rows(ops, mki, cfg):
    """gemm_rows over the interleaved gate/up layout writes silu(x gate^T) * (x up^T), with every launch
    shape: with three column tiles a wave, a gate tile and its up tile lie in two waves, which exchange
    their sums; every shape but the last adds a row's products in the same order and gives the same bits."""
    from tiny_llm_infer_amd.parts.base import BuildEnv
    from tiny_llm_infer_amd.parts.linear import GatedMatrix
    M, K, inter = mki
    x = rnd((M, K), torch.bfloat16, 3, 0.5).to(DEV)
    gate, up = rnd((inter, K), torch.bfloat16, 4, 0.1).to(DEV), rnd((inter, K), torch.bfloat16, 5, 0.1).to(DEV)
    m = GatedMatrix(gate, up, BuildEnv(dtype=torch.bfloat16, device=torch.device(DEV), ops=ops, max_model_len=64))
    g, u = x.double().cpu() @ gate.double().cpu().t(), x.double().cpu() @ up.double().cpu().t()
    ops.many_rows, ops.rows_cfg = "own", cfg
    try:
        for splits in (1, 0, 4):
            ops.rows_splits = splits
            close(ops.linear_swiglu(x, m), g / (1 + torch.exp(-g)) * u, torch.bfloat16, f"gated product, {splits} ranges of k")
        ops.rows_splits = 1
        y = ops.linear_swiglu(x, m)
        ops.rows_cfg = 2
        if cfg != 6:                          # (two sets of waves that take the slices of k in turn add in another order)
            assert torch.equal(y, ops.linear_swiglu(x, m))
    finally:
        ops.many_rows, ops.rows_cfg, ops.rows_splits = "own", 0, 0
    g, u = x.double().cpu() @ gate.double().cpu().t(), x.double().cpu() @ up.double().cpu().t()
    close(y, g / (1 + torch.exp(-g)) * u, torch.bfloat16, "gated product of many rows")
    # the library reads the stacked row-major form, which this matrix does not hold: it is put
    # together from the interleaved decode layout
    assert m._w is None and torch.equal(m.w, torch.cat([gate, up]))
    ops.many_rows = "library"
    try:
        close(ops.linear_swiglu(x, m), g / (1 + torch.exp(-g)) * u, torch.bfloat16, "the library and the activation")
    finally:
        ops.many_rows = "own"


def test_a_matrix_is_held_once_unless_the_library_reads_it(ops):
    from tiny_llm_infer_amd.parts.base import BuildEnv
    from tiny_llm_infer_amd.parts.linear import GatedMatrix, Matrix
    env = BuildEnv(dtype=torch.bfloat16, device=torch.device(DEV), ops=ops, max_model_len=64)
    w = rnd((1000, 264), torch.bfloat16, 2, 0.05).to(DEV)            # sizes that the decode layout pads
    m = Matrix(w, env)
    assert m._w is None and m.tiled is not None and m.shape == (1000, 264)
    assert m.nbytes() == m.tiled.numel() * 2 and torch.equal(m.w, w)
    gate, up = rnd((48, 136), torch.bfloat16, 3).to(DEV), rnd((48, 136), torch.bfloat16, 4).to(DEV)
    g = GatedMatrix(gate, up, env)
    assert g._w is None and g.tiled is None and g.gated is not None and torch.equal(g.w, torch.cat([gate, up]))
    odd = GatedMatrix(gate[:40], up[:40], env)                         # 40 rows do not pair up in blocks of 16
    assert odd.gated is None and odd.tiled is not None and torch.equal(odd.w, torch.cat([gate[:40], up[:40]]))
    ops.many_rows = "library"
    try:
        both = Matrix(w, env)
        assert both._w is not None and both.tiled is not None and both.nbytes() > 2 * w.numel() * 2 - 1
    finally:
        ops.many_rows = "own"
    exact = Matrix(w.float(), BuildEnv(dtype=torch.float32, device=torch.device(DEV), ops=ops, max_model_len=64))
    assert exact.tiled is None and exact._w is not None


def test_products_of_many_rows_take_the_faster_kernel(ops):
    """With ``many_rows`` = "measure" a product of more than 128 rows is timed in gemm_rows and in
    the library when its shape first comes up, and goes to the faster one from then on (the same
    one for every number of rows in the same 128): the result is right whichever that is, nothing
    is timed during a graph capture, and a shape met there first goes to the library."""
    from tiny_llm_infer_amd.parts.base import BuildEnv
    from tiny_llm_infer_amd.parts.linear import GatedMatrix, Matrix
    env = BuildEnv(dtype=torch.bfloat16, device=torch.device(DEV), ops=ops, max_model_len=64)
    ops.many_rows = "measure"
    ops.measured.clear()
    M, N, K = 1000, 1024, 512
    x, w = rnd((M, K), torch.bfloat16, 1).to(DEV), rnd((N, K), torch.bfloat16, 2, 0.05).to(DEV)
    m = Matrix(w, env)
    want = x.double().cpu() @ w.double().cpu().t()
    close(ops.linear(x, m), want, torch.bfloat16, "product while its shape is measured")
    assert list(ops.measured) == [(8, N, K, 0)]
    first = ops.linear(x, m)
    close(first, want, torch.bfloat16, "product after")
    assert torch.equal(first, ops.linear(x, m)) and torch.equal(first[:900], ops.linear(x[:900].contiguous(), m))
    gm = GatedMatrix(rnd((256, K), torch.bfloat16, 3, 0.1).to(DEV), rnd((256, K), torch.bfloat16, 4, 0.1).to(DEV), env)
    g, u = x.double().cpu() @ gm.w[:256].double().cpu().t(), x.double().cpu() @ gm.w[256:].double().cpu().t()
    close(ops.linear_swiglu(x, gm), g / (1 + torch.exp(-g)) * u, torch.bfloat16, "gated product while measured")
    assert (8, 512, K, 1) in ops.measured
    # a shape that first comes up under capture is not measured
    x2 = rnd((300, K), torch.bfloat16, 5).to(DEV)
    ops.linear(x2[:10].contiguous(), m)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = ops.linear(x2, m)
    graph.replay()
    torch.cuda.synchronize()
    assert (3, N, K, 0) not in ops.measured
    close(y, x2.double().cpu() @ w.double().cpu().t(), torch.bfloat16, "product recorded before its shape was measured")
    ops.measured.clear()
    ops.many_rows = "own"


def test_library_linear_for_many_rows(ops):
    x, w = rnd((300, 264), torch.bfloat16, 1), rnd((130, 264), torch.bfloat16, 2, 0.05)
    close(ops.linear(x.to(DEV), w.to(DEV)), x.double() @ w.double().t(), torch.bfloat16, "library product")
    y32 = ops.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32)       # float32 out, 64 rows at a time
    assert y32.dtype == torch.float32
    close(y32, x.double() @ w.double().t(), torch.float32, "float32 logits for many rows", scale=5.0)


def test_float32_logits_for_hundreds_of_rows(ops):
    """A decode step of hundreds of requests (or a replay that wants every position) asks a matrix in
    the decode layout for float32 logits of more than 128 rows: 128 rows at a time through the
    x-sharing kernel; a row's logits are those it gets alone, and the same bits among more rows."""
    from tiny_llm_infer_amd.parts.base import BuildEnv
    from tiny_llm_infer_amd.parts.linear import Matrix
    env = BuildEnv(dtype=torch.bfloat16, device=torch.device(DEV), ops=ops, max_model_len=64)
    K, N = 264, 1003                                    # a vocabulary that is no multiple of anything
    w = rnd((N, K), torch.bfloat16, 2, 0.05)
    m = Matrix(w.to(DEV), env)
    for M in (129, 256, 300, 391):                      # a last portion of 1, 128, 44 and 7 rows
        x = rnd((M, K), torch.bfloat16, M)
        y = ops.linear(x.to(DEV), m, out_dtype=torch.float32)
        assert y.dtype == torch.float32 and tuple(y.shape) == (M, N)
        want = x.double() @ w.double().t()
        close(y, want, torch.float32, f"float32 logits for {M} rows", scale=float(want.abs().max()) * (K ** 0.5) / 8)
        for r in (0, 127, 128, M - 1):
            alone = ops.linear(x[r:r + 1].contiguous().to(DEV), m, out_dtype=torch.float32)
            close(y[r:r + 1], alone.double().cpu(), torch.float32, f"row {r} of {M} and alone", scale=float(want.abs().max()))
        # among more rows (a recorded step is filled up with rows of no request): the same bits
        more = torch.cat([x, rnd((23, K), torch.bfloat16, 77)])
        assert torch.equal(ops.linear(more.to(DEV), m, out_dtype=torch.float32)[:M], y)


def test_linear_rows_do_not_depend_on_the_batch(ops):
    """float32: a row's product is bit-identical whatever else is in the batch."""
    x, w = rnd((70, 100), torch.float32, 9), rnd((130, 100), torch.float32, 10)
    full = ops.linear(x.to(DEV), w.to(DEV))
    one = ops.linear(x[41:42].contiguous().to(DEV), w.to(DEV))
    assert torch.equal(full[41:42], one)


# ------------------------------------------------------ cache and attention --
def kv_layer_cache(group, layer=0, writes=True):
    """The cache of one layer call with the attention part's two records at hand as .k and .v."""
    from tiny_llm_infer_amd.parts.base import LayerCache

    class KeysAndValues(LayerCache):
        k = property(lambda self: self.record("k"))       # [pages, kv heads, page_size, head_dim]
        v = property(lambda self: self.record("v"))       # [pages, kv heads, head_dim, page_size]
    return KeysAndValues(group, layer, writes)


def make_step(seq_lens, new_counts, page, num_pages, seed, kv_heads, head_dim, dtype, window=None):
    """Sequences of ``seq_lens`` tokens of which the last ``new_counts`` are
    this step's rows; pages handed out in a random order."""
    from tiny_llm_infer_amd.parts.base import GroupView, LayerCache, StepView
    rng = np.random.default_rng(seed)
    perm = rng.permutation(num_pages)
    width = 4
    need = max((n + page - 1) // page for n in seq_lens)
    while width < need:
        width *= 2
    tables = -np.ones((len(seq_lens), width), dtype=np.int32)
    at = 0
    for i, n in enumerate(seq_lens):
        nb = (n + page - 1) // page
        tables[i, :nb] = perm[at:at + nb]
        at += nb
    assert at <= num_pages
    pos, seq, row_start = [], [], [0]
    for i, (n, c) in enumerate(zip(seq_lens, new_counts)):
        pos += list(range(n - c, n))
        seq += [i] * c
        row_start.append(len(pos))
    k = torch.zeros((1, num_pages, kv_heads, page, head_dim), dtype=dtype, device=DEV)
    v = torch.zeros((1, num_pages, kv_heads, head_dim, page), dtype=dtype, device=DEV)
    # garbage in every slot: pages not held and slots not yet written must never be read
    k.normal_(0, 50.0)
    v.normal_(0, 50.0)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)
    g = GroupView(tensors={"k": k, "v": v}, tables=i32(tables), table_width=width, page_size=page, window=window)
    step = StepView(num_rows=len(pos), num_seqs=len(seq_lens), token_ids=i32(pos), positions=i32(pos),
                    seq_of_row=i32(seq), row_start=i32(row_start),
                    seq_start=i32([n - c for n, c in zip(seq_lens, new_counts)]), seq_len=i32(seq_lens),
                    slots=i32(list(range(len(seq_lens)))), sample_rows=i32([0]),
                    h_row_start=row_start, h_seq_start=[n - c for n, c in zip(seq_lens, new_counts)],
                    h_seq_len=list(seq_lens), h_slots=list(range(len(seq_lens))),
                    max_rows_per_seq=max(new_counts), max_seq_len=max(seq_lens),
                    reach=max(128, 1 << (max(seq_lens) - 1).bit_length()), groups=[g])
    step.cache = kv_layer_cache(g)
    return step, tables, pos, seq


def fill_cache(step, tables, seq_lens, kv_heads, head_dim, dtype, seed, std=1.0):
    """Write keys and values of whole sequences into the pages; returns them."""
    page = step.cache.group.page_size
    ks, vs = [], []
    for i, n in enumerate(seq_lens):
        kk, vv = rnd((n, kv_heads, head_dim), dtype, seed + 2 * i, std), rnd((n, kv_heads, head_dim), dtype, seed + 2 * i + 1, std)
        for t in range(n):
            p = int(tables[i, t // page])
            step.cache.k[p, :, t % page] = kk[t].to(DEV)
            step.cache.v[p, :, :, t % page] = vv[t].to(DEV)
        ks.append(kk)
        vs.append(vv)
    return ks, vs


def ref_attention(q, ks, vs, pos, seq, heads, kv_heads, scale, window):
    T, hd = q.shape[0], q.shape[1] // heads
    q = q.double().reshape(T, heads, hd)
    out = torch.zeros(T, heads, hd, dtype=torch.float64)
    for r in range(T):
        p = pos[r]
        lo = 0 if not window else max(0, p - window + 1)
        kk, vv = ks[seq[r]][lo:p + 1].double(), vs[seq[r]][lo:p + 1].double()
        for h in range(heads):
            g = h // (heads // kv_heads)
            s = (kk[:, g] @ q[r, h]) * scale
            out[r, h] = torch.softmax(s, 0) @ vv[:, g]
    return out.reshape(T, heads * hd)


ATT_CASES = [
    # heads, kv_heads, head_dim, page, seq_lens, new_counts, window
    (4, 2, 16, 8, [5, 17, 33], [5, 1, 33], None),
    (5, 1, 48, 32, [300, 64, 1], [3, 64, 1], None),
    (8, 2, 128, 16, [700, 259], [1, 1], None),
    (8, 8, 64, 16, [130, 257], [130, 2], 19),
    (6, 3, 256, 16, [90], [7], 64),
    (32, 8, 128, 16, [513], [2], None),
    # one row per sequence (decode), long enough for the keys to be split over workgroups
    (32, 8, 128, 16, [1500, 40, 129, 1, 640], [1, 1, 1, 1, 1], None),
    (8, 8, 64, 16, [130, 257], [1, 1], 19),
    # few rows with many keys, split over few workgroups
    (32, 8, 128, 16, [3000], [1], None),
    (8, 2, 128, 16, [700, 2100, 513], [1, 1, 1], None),
    (16, 4, 64, 8, [5000, 1200], [1, 1], 700),
    (5, 1, 48, 32, [300, 64], [1, 1], 100),
    (32, 1, 32, 8, [70, 3], [1, 1], None),        # 32 heads on one kv head: two head tiles
    (32, 1, 32, 4, [70], [9], None),
    (6, 2, 80, 16, [200, 31], [200, 31], None),   # 3 heads a group: columns do not fill the tile
    (16, 2, 112, 64, [333], [100], 150),
    # heads of 128 and 64 with many rows: the blocks go straight from the cache into LDS
    (8, 2, 128, 8, [200, 75], [200, 40], None),
    (4, 4, 128, 16, [300], [150], 70),
    (6, 1, 64, 32, [260, 9], [131, 9], None),
    # long portions: many steps of 32 keys through the four LDS buffers, the block table's entries
    # taken from a register that is filled again on the way; windows whose edges lie inside a
    # portion (steps that need the comparison with the row's range before and after steps that do not);
    # pages of more keys than a step
    (8, 2, 128, 16, [2500], [2200], None),
    (32, 8, 128, 16, [1100, 300], [1000, 37], 200),
    (8, 4, 64, 8, [900, 40], [640, 40], 96),
    (8, 2, 128, 64, [700], [650], None),
    (4, 2, 128, 128, [700, 130], [333, 2], 100),
    (4, 1, 64, 256, [600], [600], None),
    # many sequences in a step: beyond 16 the workgroups of the prefill kernels look their sequence up
    # together (one sequence a thread, sums by shuffles and through LDS), in rounds when there are more
    # sequences than threads
    (8, 2, 128, 16, [13 + 7 * (i % 9) for i in range(40)], [2 + i % 5 for i in range(40)], None),
    (4, 2, 64, 8, [5 + i % 11 for i in range(600)], [2 + i % 3 for i in range(600)], 6),
    # rows with many keys before them (the caller tells the launch rule): with between 256 and 512
    # workgroups of two tiles a wave the rule then keeps one set of waves and two tiles, below that
    # it takes two sets
    (16, 8, 128, 16, [2700], [2100], None),
    (16, 8, 128, 16, [1200, 90], [700, 90], None),
]


PREFILL_MODES = {"bfloat16-direct": 1, "bfloat16-lds1": 2, "bfloat16-lds2": 3,
                 # the orders in which workgroups take row blocks (none, pairs in sequence, pairs that
                 # complement each other, long blocks first), which the launcher picks by the step's size
                 "bfloat16-order0": 4, "bfloat16-order1": 5, "bfloat16-order2": 6, "bfloat16-order3": 7,
                 "bfloat16-lds1-order3": 8,
                 # heads of 64 and 128: two sets of waves a workgroup that share out a block's keys; one set
                 "bfloat16-two-sets": 10, "bfloat16-one-set": 11}


@pytest.mark.parametrize("dtype", DTYPES + ["bfloat16-plain"] + list(PREFILL_MODES))
@pytest.mark.parametrize("case", ATT_CASES)
def test_paged_attention(ops, dtype, case):
    """float32: the plain kernel.  bfloat16: the MFMA kernels (decode when every
    sequence brings one row, prefill otherwise) in each of the prefill kernel's
    forms, and the plain kernel beside them."""
    if case in ATT_CASES[-2:] and dtype in PREFILL_MODES:
        pytest.skip("a case for the launch rule itself; the forced forms have their long cases above")
    ops.force_plain = dtype == "bfloat16-plain"
    ops.prefill_direct = PREFILL_MODES.get(dtype, 0)
    dtype = torch.bfloat16 if isinstance(dtype, str) else dtype
    try:
        _paged_attention_case(ops, dtype, case)
    finally:
        ops.force_plain, ops.prefill_direct = False, 0


def _paged_attention_case(ops, dtype, case):
    heads, kv_heads, hd, page, seq_lens, new_counts, window = case
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 5
    step, tables, pos, seq = make_step(seq_lens, new_counts, page, num_pages, 3, kv_heads, hd, dtype, window)
    ks, vs = fill_cache(step, tables, seq_lens, kv_heads, hd, dtype, 100)
    q = rnd((len(pos), heads * hd), dtype, 50)
    scale = 1.0 / math.sqrt(hd)
    out = ops.paged_attention(q.to(DEV), step, step.cache, heads, kv_heads, hd, scale, window)
    close(out, ref_attention(q, ks, vs, pos, seq, heads, kv_heads, scale, window), dtype, "attention")


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_one_far_key(ops, dtype):
    """One key among hundreds is made to stand out: the output must be its
    value, which a kernel that skips or misplaces a tile or a page would miss."""
    heads, kv_heads, hd, page = 4, 1, 64, 16
    n = 777
    for far in (0, 15, 16, 255, 256, 300, 776):
        step, tables, pos, seq = make_step([n], [1], page, 60, far, kv_heads, hd, dtype)
        ks, vs = fill_cache(step, tables, [n], kv_heads, hd, dtype, 7, std=0.1)
        q = rnd((1, heads * hd), dtype, 8, 0.1)
        direction = torch.ones(hd) * 2.0
        q[0, :] = direction.repeat(heads).to(dtype)
        kfar = (direction * 2.0).to(dtype)
        p = int(tables[0, far // page])
        step.cache.k[p, 0, far % page] = kfar.to(DEV)
        out = ops.paged_attention(q.to(DEV), step, step.cache, heads, kv_heads, hd, 1.0, None)
        want = vs[0][far, 0].double().repeat(heads)
        close(out[0], want, dtype, f"far key {far}", scale=1.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_window_edge(ops, dtype):
    """The key just outside the window is made to stand out and must be ignored;
    the key just inside must be found."""
    heads, kv_heads, hd, page, window, n = 2, 2, 32, 16, 40, 100
    for far, seen in ((n - window, True), (n - window - 1, False)):
        step, tables, pos, seq = make_step([n], [1], page, 12, 1, kv_heads, hd, dtype, window)
        ks, vs = fill_cache(step, tables, [n], kv_heads, hd, dtype, 9, std=0.1)
        q = torch.full((1, heads * hd), 2.0).to(dtype)
        p = int(tables[0, far // page])
        step.cache.k[p, :, far % page] = torch.full((kv_heads, hd), 4.0, dtype=dtype, device=DEV)
        ks[0][far] = 4.0
        out = ops.paged_attention(q.to(DEV), step, step.cache, heads, kv_heads, hd, 1.0, window)
        want = ref_attention(q, ks, vs, pos, seq, heads, kv_heads, 1.0, window)
        close(out, want, dtype, f"window edge {far}", scale=1.0)
        hit = float((out[0, :hd].cpu().double() - vs[0][far, 0].double()).abs().max()) < 0.05
        assert hit == seen


QKV_CASES = [
    # heads, kv_heads, head_dim, rotary_dim, norms, page
    (4, 2, 16, 16, True, 8),
    (5, 1, 48, 48, True, 32),
    (8, 2, 128, 128, True, 16),
    (3, 3, 64, 32, False, 16),      # partial rotation, no norms
    (2, 1, 80, 0, True, 16),        # no rotation at all
    (4, 4, 64, 64, True, 8),        # head sizes 64 and 256: the kernel without LDS, 1 and 4 elements a lane
    (3, 1, 256, 256, True, 16),
    (2, 2, 128, 0, False, 16),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", QKV_CASES)
def test_qkv_to_cache(ops, dtype, case):
    heads, kv_heads, hd, rd, norms, page = case
    seq_lens, new_counts = [37, 9, 70], [5, 9, 1]
    step, tables, pos, seq = make_step(seq_lens, new_counts, page, 20, 4, kv_heads, hd, dtype)
    before_k = step.cache.k.clone()
    T = len(pos)
    qd, kd = heads * hd, kv_heads * hd
    qkv = rnd((T, qd + 2 * kd), dtype, 11)
    qw, kw = 1 + rnd((hd,), torch.float32, 12, 0.2), 1 + rnd((hd,), torch.float32, 13, 0.2)
    eps_q, eps_k = 1e-5, 3e-6
    rotary = None
    if rd:
        half = rd // 2
        ang = torch.arange(128, dtype=torch.float64)[:, None] * (10000.0 ** (-2.0 * torch.arange(half, dtype=torch.float64) / rd))[None, :]
        cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
        rotary = (cos.to(DEV), sin.to(DEV), rd)
    q = ops.qkv_to_cache(qkv.to(DEV), step, step.cache, heads, kv_heads, hd,
                         (qw.to(DEV), eps_q) if norms else None, (kw.to(DEV), eps_k) if norms else None, rotary)
    x = qkv.double()
    qq = x[:, :qd].reshape(T, heads, hd)
    kk = x[:, qd:qd + kd].reshape(T, kv_heads, hd)
    vv = x[:, qd + kd:].reshape(T, kv_heads, hd)
    if norms:
        qq = qw.double() * qq / torch.sqrt((qq * qq).mean(-1, keepdim=True) + eps_q)
        kk = kw.double() * kk / torch.sqrt((kk * kk).mean(-1, keepdim=True) + eps_k)
    if rd:
        c, s = cos.double()[pos][:, None, :], sin.double()[pos][:, None, :]

        def rot(t):
            a, b, rest = t[..., :half], t[..., half:rd], t[..., rd:]
            return torch.cat([a * c - b * s, a * s + b * c, rest], -1)
        qq, kk = rot(qq), rot(kk)
    close(q, qq.reshape(T, qd), dtype, "q")
    written = torch.zeros(step.cache.k.shape[:1] + (page,), dtype=torch.bool)
    for r in range(T):
        p, slot = int(tables[seq[r], pos[r] // page]), pos[r] % page
        close(step.cache.k[p, :, slot], kk[r], dtype, "k in cache")
        assert torch.equal(step.cache.v[p, :, :, slot].cpu(), qkv[r, qd + kd:].reshape(kv_heads, hd))
        written[p, slot] = True
    # nothing else in the cache was touched
    untouched = ~written[:, None, :, None].expand_as(before_k.cpu())
    assert torch.equal(step.cache.k.cpu()[untouched], before_k.cpu()[untouched])


RAW_CASES = [
    # heads, kv_heads, head_dim, norms, rotation, page, seq_lens, new rows, window, writes
    (32, 8, 128, True, True, 16, [1500, 40, 129, 1, 640], [1] * 5, None, True),     # decode, keys split over workgroups
    (8, 8, 64, True, True, 8, [130, 257, 16, 17], [1] * 4, 19, True),
    (32, 8, 128, True, True, 16, [2000, 600], [1, 1], None, True),                  # few rows, many keys
    (5, 1, 256, False, True, 16, [90, 33], [1, 1], None, True),
    (6, 2, 192, True, False, 4, [70, 5], [1, 1], 64, True),
    (16, 1, 64, True, True, 16, [48, 1], [1, 1], None, False),                      # reads another layer's cache
    # portions of prompts beside single rows
    (32, 8, 128, True, True, 16, [300, 64, 1, 77], [130, 64, 1, 1], None, True),
    (8, 8, 64, True, True, 8, [130, 257], [130, 2], 19, True),
    (6, 3, 256, True, True, 16, [90, 17], [7, 17], 64, True),
    (4, 2, 128, False, False, 32, [45], [45], None, True),
    (16, 1, 64, True, True, 16, [48, 9], [5, 9], None, False),
    # sequences that decode in front of portions of prompts, as the scheduler puts them: where a few of
    # them have many more keys than the portions, or they are many beside short portions, they go to the
    # decode kernel and the rest of the step to the prefill kernel
    (32, 8, 128, True, True, 16, [3100, 40, 300, 64], [1, 1, 130, 64], None, True),
    (8, 8, 64, True, True, 8, [130, 257, 16, 17, 9, 700] * 11 + [200, 31], [1] * 66 + [150, 31], 19, True),
    (8, 2, 128, True, True, 16, [90, 3100, 513], [1, 1, 257], 300, True),
    (8, 2, 128, True, True, 16, [90, 300, 513], [1, 1, 257], None, True),          # (these stay in the one kernel)
    (8, 8, 64, True, True, 8, [130, 257, 16, 17, 9, 700] * 6 + [200, 31], [1] * 36 + [150, 31], 19, True),   # (and these)
]
MIXED_TO_DECODE = {-5: 2, -4: 66, -3: 2, -2: 0, -1: 0}     # how many leading sequences of those cases the decode kernel takes


def test_which_rows_of_a_mixed_step_go_to_the_decode_kernel(ops):
    """The rule itself, on the mixed cases above (so that both ways stay covered by them) and at its edges."""
    for at, want in MIXED_TO_DECODE.items():
        heads, kv_heads, hd, _, _, page, seq_lens, new_counts, window, _ = RAW_CASES[at]
        step, *_ = make_step(seq_lens, new_counts, page, sum((n + page - 1) // page for n in seq_lens) + 3, 7, kv_heads, hd,
                             torch.bfloat16, window)
        assert ops._rows_for_the_decode_kernel(step, heads, kv_heads) == want, RAW_CASES[at][6:8]
    few, many = ops.DECODE_BESIDE_FEW, ops.DECODE_BESIDE_MANY

    def takes(seq_lens, new_counts):
        step, *_ = make_step(seq_lens, new_counts, 16, sum((n + 15) // 16 for n in seq_lens) + 3, 7, 2, 64, torch.bfloat16, None)
        return ops._rows_for_the_decode_kernel(step, 8, 2)
    assert takes([few[1]] * few[0] + [200], [1] * few[0] + [200]) == few[0]
    assert takes([few[1]] * (few[0] + 1) + [200], [1] * (few[0] + 1) + [200]) == 0          # one row too many
    assert takes([few[1] - 1] * 2 + [200], [1, 1, 200]) == 0                                # a key too few
    assert takes([few[1]] * 2 + [few[1] // 2 + 1], [1, 1, 40]) == 0                         # not twice the portion's sequence
    assert takes([20] * many[0] + [many[1]], [1] * many[0] + [many[1]]) == many[0]
    assert takes([20] * many[0] + [many[1] + 1], [1] * many[0] + [many[1] + 1]) == 0        # a new token too many
    assert takes([20] * (many[0] - 1) + [100], [1] * (many[0] - 1) + [100]) == 0
    assert takes([500] * 70, [1] * 70) == 0                                                 # no portion: a decode step
    assert takes([500, 300], [2, 300]) == 0                                                 # no row that decodes in front


def _solo_cases():
    rng = np.random.default_rng(11)
    many = [int(n) for n in rng.integers(1, 500, 70)]
    many[3], many[17], many[40] = 1, 512, 33
    return [
        # heads, kv_heads, head_dim, norms, rotation, page, seq_lens, new rows, window, writes
        (32, 8, 128, True, True, 16, many, [1] * 70, None, True),
        (8, 8, 64, True, True, 8, [int(n) for n in rng.integers(1, 400, 41)], [1] * 41, 100, True),
        (4, 1, 256, True, False, 32, [1500, 31, 32, 33, 700, 1, 64, 65, 999], [1] * 9, 700, True),
        (16, 1, 64, False, True, 16, [48, 1, 300, 17, 16], [1] * 5, None, False),      # reads another layer's cache
        (5, 5, 128, False, False, 64, [3000, 129, 64], [1] * 3, 900, True),             # a window that begins inside a page
    ] + [c for c in RAW_CASES if max(c[7]) == 1 and c[2] in (64, 128, 256)]


@pytest.mark.parametrize("case", _solo_cases())
def test_decode_attention_with_a_wave_to_a_row(ops, case):
    """The decode kernel for steps of many rows with short contexts (a wave does a row's kv head on
    its own: norm and rotation, the row's key and value into the cache, all the row's keys, the
    output) wherever its limits allow it, against float64 and against the two-kernel path, with the
    cache it leaves; and given partial sums of the projections, bit for bit what their rounded sum
    gives."""
    from tiny_llm_infer_amd.kernels.ops import DeferredSum
    heads, kv_heads, hd, norms, rotation, page, seq_lens, new_counts, window, writes = case
    reach = max(128, 1 << (max(seq_lens) - 1).bit_length())

    class G:
        page_size = page
    _, keys, _ = ops._decode_splits(len(seq_lens), reach, G, heads, kv_heads, hd, window)
    ops.decode_solo = "always"
    try:
        takes = ops._decode_splits(len(seq_lens), reach, G, heads, kv_heads, hd, window)[0] == 1 and \
            ops._a_wave_a_row(len(seq_lens), keys, G, heads, kv_heads, hd)
        if not takes:
            pytest.skip("the keys are split over workgroups, or lie in more pages than a wave keeps entries of")
        _raw_projections_case(ops, case)
        # partial sums of the projections
        dtype = torch.bfloat16
        num_pages = sum((n + page - 1) // page for n in seq_lens) + 3
        step, tables, pos, seq = make_step(seq_lens, new_counts, page, num_pages, 7, kv_heads, hd, dtype, window)
        fill_cache(step, tables, seq_lens, kv_heads, hd, dtype, 300)
        step.cache.writes = writes
        T, width = len(pos), (heads + 2 * kv_heads) * hd
        planes = torch.stack([rnd((T, width), torch.float32, 60 + p) for p in range(3)]).to(DEV)
        total = planes[0].clone()
        for p in range(1, 3):
            total += planes[p]
        qn = ((1 + rnd((hd,), torch.float32, 22, 0.2)).to(DEV), 1e-5) if norms else None
        kn = ((1 + rnd((hd,), torch.float32, 23, 0.2)).to(DEV), 3e-6) if norms else None
        rotary = None
        if rotation:
            ang = torch.arange(4096, dtype=torch.float64)[:, None] * (10000.0 ** (-2.0 * torch.arange(hd // 2, dtype=torch.float64) / hd))[None, :]
            rotary = (torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV), hd)
        k0, v0 = step.cache.k.clone(), step.cache.v.clone()
        want = ops.qkv_attention(total.to(dtype), step, step.cache, heads, kv_heads, hd, qn, kn, rotary, hd ** -0.5, window)
        k1, v1 = step.cache.k.clone(), step.cache.v.clone()
        step.cache.k.copy_(k0)
        step.cache.v.copy_(v0)
        got = ops.qkv_attention(DeferredSum(planes, dtype), step, step.cache, heads, kv_heads, hd, qn, kn, rotary,
                                hd ** -0.5, window)
        assert torch.equal(got, want) and torch.equal(step.cache.k, k1) and torch.equal(step.cache.v, v1)
    finally:
        ops.decode_solo = "auto"


def test_the_prefill_kernel_is_told_of_keys_before_its_own_rows_only(ops):
    """The launch rule of the prefill kernel is told whether its rows have many keys before them.
    When the sequences that decode have gone to the decode kernel, the lengths that count are
    those of the portions that are left, not the longest sequence of the step."""
    class Step:
        num_seqs, h_seq_len, max_seq_len = 3, [6000, 90, 300], 6000
    assert ops._prefill_mode(Step, 302) == 13                  # all three in the prefill kernel: one has 5,999 keys before its row
    assert ops._prefill_mode(Step, 300, first=2) == 0          # the portion alone starts at position 0
    Step.h_seq_len = [6000, 90, 2300]
    assert ops._prefill_mode(Step, 300, first=2) == 13         # 300 rows behind 2,000 keys
    ops.prefill_direct = 3
    try:
        assert ops._prefill_mode(Step, 300, first=2) == 3      # a form forced by a test stays
    finally:
        ops.prefill_direct = 0


@pytest.mark.parametrize("mode", [0, 3])
@pytest.mark.parametrize("case", RAW_CASES)
def test_attention_from_raw_projections(ops, case, mode):
    """The attention kernels that norm and rotate q (and for a decode step k, writing the
    row's key and value) themselves: against float64 mathematics, and the cache they
    leave against the two-kernel path's.  mode: the prefill kernel's form (0: as the
    launcher picks, 3: two tiles a wave)."""
    heads, kv_heads, hd, norms, rotation, page, seq_lens, new_counts, window, writes = case
    if mode and (max(new_counts) == 1 or hd > 128):
        pytest.skip("the forms of the prefill kernel for heads up to 128")
    ops.prefill_direct = mode
    try:
        _raw_projections_case(ops, case)
    finally:
        ops.prefill_direct = 0


@pytest.mark.parametrize("case", [c for c in RAW_CASES if max(c[7]) == 1 and c[2] % 64 == 0])
@pytest.mark.parametrize("parts", [1, 2, 5])
def test_decode_attention_adds_partial_sums_of_the_projections(ops, case, parts):
    """The decode kernel given the projections as float32 partial sums of a split k range
    leaves the same output and the same cache, bit for bit, as given their sum rounded to
    bfloat16 (what the product's own reduction writes)."""
    from tiny_llm_infer_amd.kernels.ops import DeferredSum
    heads, kv_heads, hd, norms, rotation, page, seq_lens, new_counts, window, writes = case
    dtype = torch.bfloat16
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 3
    step, tables, pos, seq = make_step(seq_lens, new_counts, page, num_pages, 7, kv_heads, hd, dtype, window)
    fill_cache(step, tables, seq_lens, kv_heads, hd, dtype, 300)
    step.cache.writes = writes
    T = len(pos)
    width = (heads + 2 * kv_heads) * hd
    planes = torch.stack([rnd((T, width), torch.float32, 60 + p) for p in range(parts)]).to(DEV)
    planes[0, 0, (heads + kv_heads) * hd + 3] = float("inf")   # a value that has diverged is made finite on its way in
    total = planes[0].clone()
    for p in range(1, parts):
        total += planes[p]                                # the order of the reduction kernel
    qkv = total.to(dtype)
    qn = ((1 + rnd((hd,), torch.float32, 22, 0.2)).to(DEV), 1e-5) if norms else None
    kn = ((1 + rnd((hd,), torch.float32, 23, 0.2)).to(DEV), 3e-6) if norms else None
    rotary = None
    if rotation:
        half = hd // 2
        ang = torch.arange(4096, dtype=torch.float64)[:, None] * (10000.0 ** (-2.0 * torch.arange(half, dtype=torch.float64) / hd))[None, :]
        rotary = (torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV), hd)
    scale = 1.0 / math.sqrt(hd)
    k0, v0 = step.cache.k.clone(), step.cache.v.clone()
    want = ops.qkv_attention(qkv, step, step.cache, heads, kv_heads, hd, qn, kn, rotary, scale, window)
    k1, v1 = step.cache.k.clone(), step.cache.v.clone()
    step.cache.k.copy_(k0)
    step.cache.v.copy_(v0)
    got = ops.qkv_attention(DeferredSum(planes, dtype), step, step.cache, heads, kv_heads, hd, qn, kn, rotary,
                            scale, window)
    assert torch.equal(got, want)
    assert torch.equal(step.cache.k, k1) and torch.equal(step.cache.v, v1)
    assert bool(torch.isfinite(step.cache.v.float()).all())


def _raw_projections_case(ops, case):
    heads, kv_heads, hd, norms, rotation, page, seq_lens, new_counts, window, writes = case
    dtype = torch.bfloat16
    B = len(seq_lens)
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 3
    step, tables, pos, seq = make_step(seq_lens, new_counts, page, num_pages, 7, kv_heads, hd, dtype, window)
    ks, vs = fill_cache(step, tables, seq_lens, kv_heads, hd, dtype, 300)
    step.cache.writes = writes
    T = len(pos)
    qd, kd = heads * hd, kv_heads * hd
    qkv = rnd((T, qd + 2 * kd), dtype, 21)
    qw, kw = 1 + rnd((hd,), torch.float32, 22, 0.2), 1 + rnd((hd,), torch.float32, 23, 0.2)
    eps_q, eps_k = 1e-5, 3e-6
    qn = (qw.to(DEV), eps_q) if norms else None
    kn = (kw.to(DEV), eps_k) if norms else None
    rotary = None
    half = hd // 2
    if rotation:
        ang = torch.arange(4096, dtype=torch.float64)[:, None] * (10000.0 ** (-2.0 * torch.arange(half, dtype=torch.float64) / hd))[None, :]
        cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
        rotary = (cos.to(DEV), sin.to(DEV), hd)
    scale = 1.0 / math.sqrt(hd)
    k0, v0 = step.cache.k.clone(), step.cache.v.clone()
    out = ops.qkv_attention(qkv.to(DEV), step, step.cache, heads, kv_heads, hd, qn, kn, rotary, scale, window)
    k1, v1 = step.cache.k.clone(), step.cache.v.clone()
    # the same through qkv_to_cache and paged_attention
    step.cache.k.copy_(k0)
    step.cache.v.copy_(v0)
    ops.unfused_decode = True
    try:
        out2 = ops.qkv_attention(qkv.to(DEV), step, step.cache, heads, kv_heads, hd, qn, kn, rotary, scale, window)
    finally:
        ops.unfused_decode = False
    assert torch.equal(v1, step.cache.v)
    close(k1, step.cache.k.double().cpu(), dtype, "keys in the cache", scale=float(k1.abs().max()) / 50)
    if not writes:
        assert torch.equal(k1, k0) and torch.equal(v1, v0)
    # float64
    x = qkv.double()
    qq = x[:, :qd].reshape(T, heads, hd)
    kk = x[:, qd:qd + kd].reshape(T, kv_heads, hd)
    vv = x[:, qd + kd:].reshape(T, kv_heads, hd)
    if norms:
        qq = qw.double() * qq / torch.sqrt((qq * qq).mean(-1, keepdim=True) + eps_q)
        kk = kw.double() * kk / torch.sqrt((kk * kk).mean(-1, keepdim=True) + eps_k)
    if rotation:
        c, sn = cos.double()[pos][:, None, :], sin.double()[pos][:, None, :]

        def rot(t):
            a, b = t[..., :half], t[..., half:]
            return torch.cat([a * c - b * sn, a * sn + b * c], -1)
        qq, kk = rot(qq), rot(kk)
    if writes:                      # the rows' own keys and values replace what the cache held there
        for r in range(T):
            ks[seq[r]][pos[r]] = kk[r].to(dtype)
            vs[seq[r]][pos[r]] = vv[r].to(dtype)
    want = ref_attention(qq.reshape(T, qd).to(dtype), ks, vs, pos, seq, heads, kv_heads, scale, window)
    close(out, want, dtype, "attention from raw projections")
    close(out2, want, dtype, "attention through two kernels")


@pytest.mark.parametrize("hd,page,rotation,norms", [(128, 16, True, True), (64, 8, True, True), (256, 32, False, True),
                                                    (128, 64, True, False), (64, 16, False, False)])
def test_keys_and_values_of_portions_in_one_pass(ops, hd, page, rotation, norms):
    """Prompt portions write their keys (normed, rotated) and values into the pages with one
    kernel: the cache it leaves is bit for bit what the two kernels (keys; values) leave, for
    portions that start and end inside a page, single rows among them, and nothing else in the
    cache is touched."""
    heads, kv_heads = 4, 2
    seq_lens, new_counts = [137, 40, 9, 70, 300], [130, 40, 1, 3, 77]
    dtype = torch.bfloat16
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 3
    step, tables, pos, seq = make_step(seq_lens, new_counts, page, num_pages, 13, kv_heads, hd, dtype)
    T = len(pos)
    qkv = rnd((T, (heads + 2 * kv_heads) * hd), dtype, 31).to(DEV)
    qkv[5, (heads + kv_heads) * hd + 7] = float("inf")                  # made finite on its way in
    kn = ((1 + rnd((hd,), torch.float32, 23, 0.2)).to(DEV), 3e-6) if norms else None
    rotary = None
    if rotation:
        ang = torch.arange(512, dtype=torch.float64)[:, None] * (10000.0 ** (-2.0 * torch.arange(hd // 2, dtype=torch.float64) / hd))[None, :]
        rotary = (torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV), hd)
    k0, v0 = step.cache.k.clone(), step.cache.v.clone()
    assert ops.qkv_to_cache(qkv, step, step.cache, heads, kv_heads, hd, None, kn, rotary, queries=False) is None
    k1, v1 = step.cache.k.clone(), step.cache.v.clone()
    step.cache.k.copy_(k0)
    step.cache.v.copy_(v0)
    ops.separate_cache_writes = True
    try:
        ops.qkv_to_cache(qkv, step, step.cache, heads, kv_heads, hd, None, kn, rotary, queries=False)
    finally:
        ops.separate_cache_writes = False
    assert torch.equal(k1, step.cache.k) and torch.equal(v1, step.cache.v)
    written = torch.zeros((num_pages, page), dtype=torch.bool)
    for r in range(T):
        written[int(tables[seq[r], pos[r] // page]), pos[r] % page] = True
    untouched = ~written[:, None, :, None].expand_as(k0.cpu())
    assert torch.equal(k1.cpu()[untouched], k0.cpu()[untouched]) and not torch.equal(k1, k0)
    untouched_v = ~written[:, None, None, :].expand_as(v0.cpu())
    assert torch.equal(v1.cpu()[untouched_v], v0.cpu()[untouched_v])
    p5 = int(tables[seq[5], pos[5] // page])
    assert float(v1[p5, 0, 7, pos[5] % page]) == 0.0


@pytest.mark.parametrize("separate", [False, True])
def test_cache_writes_of_a_step_with_hundreds_of_sequences(ops, separate):
    """300 sequences in one step (more than a workgroup has threads), single rows and short
    portions mixed, some with no rows before them: every key and value lands in its slot."""
    heads, kv_heads, hd, page = 2, 2, 64, 16
    rng = np.random.default_rng(3)
    new_counts = [int(c) for c in rng.choice([1, 1, 1, 2, 5, 17, 33], 300)]
    seq_lens = [c + int(rng.integers(0, 40)) for c in new_counts]
    dtype = torch.bfloat16
    num_pages = sum((n + page - 1) // page for n in seq_lens) + 3
    step, tables, pos, seq = make_step(seq_lens, new_counts, page, num_pages, 17, kv_heads, hd, dtype)
    T = len(pos)
    qkv = rnd((T, (heads + 2 * kv_heads) * hd), dtype, 33).to(DEV)
    k0 = step.cache.k.clone()
    ops.separate_cache_writes = separate
    try:
        ops.qkv_to_cache(qkv, step, step.cache, heads, kv_heads, hd, None, None, None, queries=False)
    finally:
        ops.separate_cache_writes = False
    kd = (heads) * hd
    rows = torch.arange(T)
    pages = torch.as_tensor(tables)[torch.as_tensor(seq), torch.as_tensor(pos) // page].long()
    slots = torch.as_tensor(pos) % page
    want_k = qkv[:, kd:kd + kv_heads * hd].reshape(T, kv_heads, hd).cpu()
    want_v = qkv[:, kd + kv_heads * hd:].reshape(T, kv_heads, hd).cpu()
    assert torch.equal(step.cache.k.cpu()[pages, :, slots], want_k)
    assert torch.equal(step.cache.v.cpu()[pages, :, :, slots], want_v)
    written = torch.zeros((num_pages, page), dtype=torch.bool)
    written[pages, slots] = True
    untouched = ~written[:, None, :, None].expand_as(k0.cpu())
    assert torch.equal(step.cache.k.cpu()[untouched], k0.cpu()[untouched])


@pytest.mark.parametrize("hd,counts", [(128, [1, 1]), (128, [20, 1]), (48, [5, 1])])
def test_values_enter_the_cache_finite(ops, hd, counts):
    """Infinities and NaNs among the values become 0 on their way into the cache (every
    kernel that writes values), and the attention output of the other rows stays finite."""
    heads, kv_heads, page = 4, 2, 16
    seq_lens = [40, 23]
    dtype = torch.bfloat16
    step, tables, pos, seq = make_step(seq_lens, counts, page, 8, 5, kv_heads, hd, dtype)
    fill_cache(step, tables, seq_lens, kv_heads, hd, dtype, 70)
    T = len(pos)
    qd, kd = heads * hd, kv_heads * hd
    qkv = rnd((T, qd + 2 * kd), dtype, 71)
    qkv[0, qd + kd + 3] = float("inf")
    qkv[T - 1, qd + kd + hd + 5] = float("nan")
    out = ops.qkv_attention(qkv.to(DEV), step, step.cache, heads, kv_heads, hd, None, None, None, hd ** -0.5, None)
    assert bool(torch.isfinite(step.cache.v).all())
    p0, p1 = int(tables[seq[0], pos[0] // page]), int(tables[seq[T - 1], pos[T - 1] // page])
    assert float(step.cache.v[p0, 0, 3, pos[0] % page]) == 0.0
    assert float(step.cache.v[p1, 1, 5, pos[T - 1] % page]) == 0.0
    assert bool(torch.isfinite(out).all())


def test_rotation_pairs_halves_not_neighbours(ops):
    """A head with only element i set: after the rotation at a position whose
    angle for pair i is 90 degrees, the value has moved to element i + d/2."""
    heads, kv_heads, hd, page = 1, 1, 16, 8
    step, tables, pos, seq = make_step([2], [1], page, 2, 0, kv_heads, hd, torch.float32)
    half = hd // 2
    cos = torch.zeros(4, half)
    sin = torch.ones(4, half)           # every pair turned by 90 degrees
    qkv = torch.zeros(1, 3 * hd)
    qkv[0, 3] = 1.0
    q = ops.qkv_to_cache(qkv.to(DEV), step, step.cache, heads, kv_heads, hd, None, None,
                         (cos.to(DEV), sin.to(DEV), hd))
    want = torch.zeros(hd)
    want[3 + half] = 1.0
    assert torch.allclose(q[0].cpu(), want, atol=1e-7)


def test_partial_sums_as_residual_delta(ops):
    """A product of 17..128 rows whose k range is split may leave its partial sums to
    the norm that follows: the residual and the normed rows are bit for bit what the
    product's own reduction followed by the norm gives, also for a subset of rows."""
    from tiny_llm_infer_amd.kernels.ops import DeferredSum
    M, N, K = 37, 200, 1024
    x, w = rnd((M, K), torch.bfloat16, 1).to(DEV), rnd((N, K), torch.bfloat16, 2, 0.05).to(DEV)

    class Both:
        pass
    Both.w, Both.tiled = w, ops.tile_matrix(w)
    weight = (1 + rnd((N,), torch.float32, 3, 0.1)).to(DEV)
    resid = rnd((M, N), torch.float32, 4).to(DEV)
    ops.mid_splits = 4
    try:
        y = ops.linear(x, Both)
        d = ops.linear(x, Both, deferred=True)
    finally:
        ops.mid_splits = 0
    assert isinstance(d, DeferredSum) and tuple(d.parts.shape) == (4, M, N)
    assert torch.equal(ops.resolve(d), y)
    r1, r2 = resid.clone(), resid.clone()
    o1 = ops.add_rmsnorm(r1, y, weight, 1e-5, torch.bfloat16)
    o2 = ops.add_rmsnorm(r2, d, weight, 1e-5, torch.bfloat16)
    assert torch.equal(r1, r2) and torch.equal(o1, o2)
    rows = torch.tensor([36, 0, 5], dtype=torch.int32, device=DEV)
    r3 = resid.clone()
    o3 = ops.add_rmsnorm(r3, d, weight, 1e-5, torch.bfloat16, rows=rows)
    assert torch.equal(r3, resid)                                  # a subset of rows leaves the residual alone
    assert torch.equal(o3, ops.add_rmsnorm(resid.clone(), y, weight, 1e-5, torch.bfloat16, rows=rows))
    assert torch.equal(o3, o1[rows.long()])


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("hidden", [200, 4096])
def test_products_that_take_the_norm_in(ops, M, hidden):
    """A decode step's output projection adds into the residual and leaves the next norm's
    rows with their factor owed; the products that follow apply it.  Against float64
    mathematics and against the same done with a norm kernel between the products."""
    from tiny_llm_infer_amd.kernels.ops import NormedRows, PendingProduct
    from tiny_llm_infer_amd.parts.base import BuildEnv
    from tiny_llm_infer_amd.parts.linear import GatedMatrix, Matrix
    env = BuildEnv(dtype=torch.bfloat16, device=torch.device(DEV), ops=ops, max_model_len=64)
    K, N2, inter, eps = 320, 96, 64, 1e-5
    bf = torch.bfloat16
    x = rnd((M, K), bf, 1)
    wo, wn = rnd((hidden, K), bf, 2, 0.05), rnd((N2, hidden), bf, 3, 0.05)
    wg, wu = rnd((inter, hidden), bf, 4, 0.05), rnd((inter, hidden), bf, 5, 0.05)
    nw = 1 + rnd((hidden,), torch.float32, 6, 0.2)
    resid0 = rnd((M, hidden), torch.float32, 7)
    Wo, Wn, Wg = Matrix(wo.to(DEV), env), Matrix(wn.to(DEV), env), GatedMatrix(wg.to(DEV), wu.to(DEV), env)
    # float64
    h = resid0.double() + x.double() @ wo.double().t()
    n = nw.double() * h / torch.sqrt((h * h).mean(-1, keepdim=True) + eps)
    want_z = n @ wn.double().t()
    g, u = n @ wg.double().t(), n @ wu.double().t()
    want_act = g / (1 + torch.exp(-g)) * u
    # a norm kernel between the products
    ops.separate_norms = True
    try:
        ra = resid0.clone().to(DEV)
        y = ops.linear(x.to(DEV), Wo, deferred=True)
        assert isinstance(y, torch.Tensor)
        na = ops.add_rmsnorm(ra, y, nw.to(DEV), eps, bf, lazy=True)
        za, acta = ops.linear(na, Wn), ops.linear_swiglu(na, Wg)
    finally:
        ops.separate_norms = False
    # the norm taken into the products
    rb = resid0.clone().to(DEV)
    p = ops.linear(x.to(DEV), Wo, deferred=True)
    assert isinstance(p, PendingProduct)
    nb = ops.add_rmsnorm(rb, p, nw.to(DEV), eps, bf, lazy=True)
    assert isinstance(nb, NormedRows) and tuple(nb.ssq.shape) == ((hidden + 15) // 16, M)
    zb, actb = ops.linear(nb, Wn), ops.linear_swiglu(nb, Wg)
    close(rb, h, torch.float32, "residual", scale=float(h.abs().max()) * 4)     # bfloat16 inputs, float32 sums
    close(ra, h, bf, "residual through a bfloat16 delta")
    assert float((nb.ssq.sum(0).double().cpu() - (h * h).sum(-1)).abs().max()) <= 1e-4 * float((h * h).sum(-1).max())
    for got, want, what in ((zb, want_z, "product of normed rows"), (actb, want_act, "gated product of normed rows"),
                            (za, want_z, "the same with a norm kernel"), (acta, want_act, "gated, with a norm kernel")):
        close(got, want, bf, what)
    # without lazy the product is run as it is
    rc = resid0.clone().to(DEV)
    nc = ops.add_rmsnorm(rc, ops.linear(x.to(DEV), Wo, deferred=True), nw.to(DEV), eps, bf)
    assert torch.equal(nc, na) and torch.equal(rc, ra)


def test_launch_rules_know_the_chip(ops):
    assert ops.lib.tli_device_compute_units() == torch.cuda.get_device_properties(0).multi_processor_count
    assert ops.DECODE_WORKGROUPS == ops.lib.tli_device_compute_units()


# ------------------------------------------------------------------ sampling --
def test_greedy_takes_the_lowest_index_on_ties(ops):
    logits = torch.zeros(3, 5000)
    logits[0, 4000] = logits[0, 77] = logits[0, 4999] = 3.0
    logits[1, 0] = 1.0
    logits[2, 4999] = 1.0
    out = ops.sample(logits.to(DEV))
    assert out.cpu().tolist() == [77, 0, 4999]


def test_temperature_sampling_is_gumbel_max_over_a_hash(ops):
    from tiny_llm_infer_amd.kernels.ops import sample_uniform
    rows, vocab = 4, 301
    logits = rnd((rows, vocab), torch.float32, 21, 2.0)
    temps = torch.tensor([0.7, 0.0, 1.5, 0.7])
    seeds = torch.tensor([12345, 1, 2 ** 40 + 17, 12346], dtype=torch.int64)
    out = ops.sample(logits.to(DEV), temps.to(DEV), seeds.to(DEV)).cpu().tolist()
    for r in range(rows):
        if temps[r] <= 1e-6:
            want = int(torch.argmax(logits[r]))
        else:
            u = np.array([sample_uniform(int(seeds[r]), t) for t in range(vocab)], dtype=np.float64)
            assert 0 < u.min() and u.max() < 1
            score = logits[r].double().numpy() + float(temps[r]) * -np.log(-np.log(u))
            want = int(np.argmax(score))
        assert out[r] == want
    # the same seed gives the same token whatever else is in the batch
    alone = ops.sample(logits[3:4].contiguous().to(DEV), temps[3:4].to(DEV), seeds[3:4].to(DEV)).cpu().tolist()
    assert alone[0] == out[3]


def test_sampling_a_large_vocabulary_in_pieces(ops):
    """Large vocabularies are scanned in pieces; the winner and the tie rule are the same."""
    from tiny_llm_infer_amd.kernels.ops import sample_uniform
    rows, vocab = 3, 151936
    logits = rnd((rows, vocab), torch.float32, 5, 2.0)
    logits[0, 150000] = logits[0, 9] = logits[0, 77777] = 50.0           # a tie across pieces
    assert ops.sample(logits.to(DEV)).cpu().tolist() == [9, int(logits[1].argmax()), int(logits[2].argmax())]
    temps = torch.tensor([0.9, 0.0, 1.3])
    seeds = torch.tensor([5, 6, 2 ** 50 + 3], dtype=torch.int64)
    got = ops.sample(logits.to(DEV), temps.to(DEV), seeds.to(DEV)).cpu().tolist()
    def uniforms(seed, n):
        """The kernel's hash of (seed, token), vectorised: three rounds of the murmur3 finaliser."""
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

    assert abs(uniforms(12345, 10)[7] - sample_uniform(12345, 7)) < 1e-9
    # every uniform lies strictly inside (0, 1), the hash's largest and smallest values included, so no
    # token's Gumbel value is infinite: (k + 0.5) / 2^23 is a float32 as it stands for every k < 2^23
    u = uniforms(99, 1 << 20)
    assert all(sample_uniform(99, int(t)) == u[t] for t in (int(u.argmax()), int(u.argmin()), 0, 1, 12345))
    assert 0.0 < u.min() and u.max() < 1.0 and np.all(u.astype(np.float32).astype(np.float64) == u)
    ends = (np.array([0, 1, (1 << 23) - 2, (1 << 23) - 1], dtype=np.float32) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)
    assert ends.dtype == np.float32 and ends[0] > 0 and ends[-1] < 1 and np.all(np.diff(ends.astype(np.float64)) > 0)
    assert np.isfinite(-np.log(-np.log(ends.astype(np.float64)))).all()
    for r in (0, 2):
        u = uniforms(int(seeds[r]), vocab)
        score = logits[r].double().numpy() + float(temps[r]) * -np.log(-np.log(u))
        order = np.argsort(-score)
        assert got[r] == int(order[0]) or score[order[0]] - score[got[r]] < 1e-5     # float32 noise on a near-tie
    assert got[1] == int(logits[1].argmax())


def test_temperature_sampling_follows_softmax(ops):
    vocab, n = 6, 4000
    base = torch.tensor([2.0, 1.0, 0.0, -1.0, 0.5, 1.5])
    T = 0.8
    logits = base.repeat(n, 1)
    seeds = torch.arange(1, n + 1, dtype=torch.int64) * 7919
    out = ops.sample(logits.to(DEV), torch.full((n,), T).to(DEV), seeds.to(DEV)).cpu()
    freq = torch.bincount(out.long(), minlength=vocab).double() / n
    want = torch.softmax(base.double() / T, 0)
    assert float((freq - want).abs().max()) < 0.03
