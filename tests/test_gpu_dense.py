"""GPU parity of the MFMA dense layer (torch.ops.xpu_ops.dense -> xg_dense)
against the eager oracle: bf16 / fp16, weight as [K, N] and as [N, K],
bias / residual / activation variants, ragged edges.  Anchor: the layer evaluated
in fp32 on the same 16-bit inputs; rtol 1.6e-2 with the floor of one output ulp
at max|y| * 2^-7 (tests/tolerance.py).  Comparisons with the unfused 16-bit
eager graph, which rounds after every op, are a second, looser check and say so."""
import pytest
import torch
import torch.nn.functional as F

from oracle import eager, inputs
from tests.tolerance import assert_close_16bit, dense_floor

pytestmark = pytest.mark.gpu


def _ops():
    import xpu_graph_amd.ops  # noqa: F401

    return torch.ops.xpu_ops


def ref32(x, W, weight_trans, bias, residual, act):
    y = x.float() @ (W.float().t() if weight_trans else W.float())
    if bias is not None:
        y = y + bias.float()
    if residual is not None:
        y = y + residual.float()
    return {"none": lambda t: t, "relu": F.relu, "gelu": F.gelu, "silu": F.silu, "sigmoid": torch.sigmoid}[act](y)


def close(got, want, k):
    """Against the fp32 anchor `want` (k, the accumulation length, only labels the record)."""
    assert_close_16bit(got, want, dense_floor(want, got.dtype), f"dense K={k} {tuple(got.shape)} {got.dtype}")


def close_to_eager_16bit(got, want16):
    """Second, looser check against the UNFUSED 16-bit eager graph, which rounds the matmul, the bias add and the
    activation separately (up to three half-ulps of values of the size of the pre-activation): rtol 1.6e-2 plus two
    ulps of the output type at the largest value."""
    spacing = 2.0 ** (-7 if got.dtype == torch.bfloat16 else -10)
    torch.testing.assert_close(got.float(), want16.float(), rtol=1.6e-2, atol=2 * spacing * want16.float().abs().max().item())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("weight_trans", [False, True])
@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 768, 256), (300, 264, 200), (1, 8, 8), (1000, 1032, 72), (64, 4096, 4096)])
def test_dense_shapes(device, dtype, weight_trans, M, N, K):
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(dtype).to(device)
    W = (torch.randn(N, K, generator=g) / K**0.5).to(dtype).to(device)
    if not weight_trans:
        W = W.t().contiguous()
    b = torch.randn(N, generator=g).to(dtype).to(device)
    got = _ops().dense(x, W, weight_trans, b, None, "silu")
    assert got.shape == (M, N) and got.dtype == dtype
    close(got, ref32(x, W, weight_trans, b, None, "silu"), K)
    got = _ops().dense(x, W, weight_trans, None, None, "none")
    close(got, ref32(x, W, weight_trans, None, None, "none"), K)


@pytest.mark.parametrize("weight_trans", [False, True])
@pytest.mark.parametrize(
    "M,N,K", [(1, 8, 64), (70, 72, 128), (300, 264, 192), (33, 4096, 4096), (256, 11008, 4096), (1024, 4096, 512), (2048, 4096, 1024), (1300, 4104, 256)]
)
def test_dense_small_and_underfilled_grids(device, weight_trans, M, N, K):
    """Whole K slabs and at most a quarter of a machine of 256 x 256 tiles: the split-K 64 x 64 kernel; grids
    between that and one full round: 128 x 256 tiles throughout (the last two shapes).  Ragged M and N, one slab
    and many, bias + residual + activation, and exact integer products."""
    g = torch.Generator().manual_seed(M * 7 + N + K)
    x = torch.randn(M, K, generator=g).bfloat16().to(device)
    W = (torch.randn(N, K, generator=g) / K**0.5).bfloat16().to(device)
    if not weight_trans:
        W = W.t().contiguous()
    b = torch.randn(N, generator=g).bfloat16().to(device)
    res = torch.randn(M, N, generator=g).bfloat16().to(device)
    close(_ops().dense(x, W, weight_trans, None, None, "none"), ref32(x, W, weight_trans, None, None, "none"), K)
    close(_ops().dense(x, W, weight_trans, b, res, "gelu"), ref32(x, W, weight_trans, b, res, "gelu"), K)
    # exact products: small integers, so every partial sum is exact in fp32 and the result must be bit-exact
    xi = torch.randint(-2, 3, (M, K), generator=g).bfloat16().to(device)
    Wi = torch.randint(-2, 3, (N, K), generator=g).bfloat16().to(device)
    Wi = Wi if weight_trans else Wi.t().contiguous()
    want = (xi.float() @ (Wi.float().t() if weight_trans else Wi.float())).bfloat16()
    assert torch.equal(_ops().dense(xi, Wi, weight_trans, None, None, "none"), want)


@pytest.mark.parametrize("act", ["none", "relu", "gelu", "silu", "sigmoid"])
def test_dense_bias_residual_activation(device, act):
    M, N, K = 320, 520, 136
    g = torch.Generator().manual_seed(7)
    x = torch.randn(M, K, generator=g).bfloat16().to(device)
    W = (0.1 * torch.randn(K, N, generator=g)).bfloat16().to(device)
    b32 = torch.randn(N, generator=g).to(device)
    res = torch.randn(M, N, generator=g).bfloat16().to(device)
    got = _ops().dense(x, W, False, b32, res, act)  # fp32 bias + residual
    close(got, ref32(x, W, False, b32, res, act), K)
    got = _ops().dense(x, W, False, None, res, act)
    close(got, ref32(x, W, False, None, res, act), K)


def test_dense_identity_and_strided_views(device):
    x = torch.randn(256, 128, device=device).bfloat16()
    eye = torch.eye(128, device=device).bfloat16()
    assert torch.equal(_ops().dense(x, eye, False, None, None, "none"), x)  # W = I is exact
    assert torch.equal(_ops().dense(x, eye, True, None, None, "none"), x)
    big = torch.randn(256, 512, device=device).bfloat16()
    xv = big[:, 128:256]  # row stride 512
    Wv = torch.randn(128, 512, device=device).bfloat16()[:, 64:192]
    close(_ops().dense(xv, Wv, False, None, None, "none"), ref32(xv, Wv, False, None, None, "none"), 128)
    xt = torch.randn(128, 256, device=device).bfloat16().t()  # column stride != 1: copied by the op
    close(_ops().dense(xt, eye, False, None, None, "relu"), F.relu(xt.float()), 128)


def test_dense_c4_full_size(device):
    x, W, b = inputs.c4_dense(device=device)
    got = _ops().dense(x, W, False, b, None, "silu")
    want = eager.dense_silu_eager(x, W, b)  # the unfused bf16 graph on the same device
    close_to_eager_16bit(got, want)
    for r0 in range(0, x.shape[0], 1024):  # EVERY row against the fp32 anchor, 1024 rows of reference at a time
        close(got[r0 : r0 + 1024], ref32(x[r0 : r0 + 1024], W, False, b, None, "silu"), 4096)
    Wt = W.t().contiguous()
    got_t = _ops().dense(x, Wt, True, b, None, "silu")
    assert torch.equal(got_t, got)  # both weight layouts run the same arithmetic in the same order


def test_dense_c4_full_size_permutation_properties(device):
    """Size-independent properties at the full C4 shape: an output element is one dot product accumulated in a fixed
    order over K, so permuting weight columns (with the bias) or activation rows must permute the result BIT FOR BIT
    -- whichever tile, tile height or launch half an element lands in -- and the gated layer with equal gate and up
    weights must equal silu(z) * z of the plain layer's rounded z."""
    x, W, b = inputs.c4_dense(device=device)
    ops = _ops()
    base = ops.dense(x, W, False, b, None, "silu")
    g = torch.Generator().manual_seed(11)
    pc = torch.randperm(W.shape[1], generator=g).to(device)
    assert torch.equal(ops.dense(x, W[:, pc].contiguous(), False, b[pc].contiguous(), None, "silu"), base[:, pc])
    pr = torch.randperm(x.shape[0], generator=g).to(device)
    assert torch.equal(ops.dense(x[pr].contiguous(), W, False, b, None, "silu"), base[pr])
    # the [N, K] layout and a row-strided activation view go through other load paths, same arithmetic
    Wt = W.t().contiguous()
    wide = torch.empty(x.shape[0], x.shape[1] + 64, dtype=x.dtype, device=device)
    wide[:, : x.shape[1]] = x
    assert torch.equal(ops.dense(wide[:, : x.shape[1]], Wt, True, b, None, "silu"), base)
    z = ops.dense(x, Wt, True, None, None, "none")
    glu = ops.dense_glu(x, Wt, Wt)
    assert torch.equal(glu, ops.silu_mul2(z, z))


@pytest.mark.parametrize("weight_trans", [True, False])
@pytest.mark.parametrize("M,N,K", [(1024, 4096, 4096), (1024, 4096, 11008), (1000, 4000, 4096), (512, 8192, 8192)])
def test_dense_128_tile_kernel_matches_the_large_tiles(device, M, N, K, weight_trans):
    """Shapes whose 128 x 128 grid fills a round of compute units take the 128 x 128 kernel (either weight layout): every
    output element sees the MFMAs of the large-tile kernels in the same order, so the rows come out BIT FOR BIT as the
    same rows of a four times taller problem (which runs on large tiles), and close to the fp32 anchor."""
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(4 * M, K, generator=g).bfloat16().to(device)
    W = (torch.randn(N, K, generator=g) / K**0.5).bfloat16().to(device)
    if not weight_trans:
        W = W.t().contiguous()
    b = torch.randn(N, generator=g).bfloat16().to(device)
    res = torch.randn(4 * M, N, generator=g).bfloat16().to(device)
    ops = _ops()
    tall = ops.dense(x, W, weight_trans, b, res, "silu")
    for r0 in (0, M, 3 * M):
        got = ops.dense(x[r0 : r0 + M], W, weight_trans, b, res[r0 : r0 + M], "silu")
        assert torch.equal(got, tall[r0 : r0 + M])
    close(tall[:M], ref32(x[:M], W, weight_trans, b, res[:M], "silu"), K)


@pytest.mark.parametrize("weight_trans", [True, False])
@pytest.mark.parametrize("M,N,K", [(1536, 11008, 4096), (3072, 6144, 1024), (1300, 11008, 512), (4352, 4096, 2048)])
def test_dense_grid_of_a_round_and_a_little_runs_in_two_launches_with_the_same_bits(device, M, N, K, weight_trans):
    """A tile grid of whole rounds of compute units plus a few tiles is split: full tiles on the columns (or rows) that
    fill the rounds, a second launch for the strip that is left.  Every kernel involved adds in the same order, so the
    rows must equal the same rows of a taller problem BIT FOR BIT, bias, residual and activation included."""
    g = torch.Generator().manual_seed(M * 3 + N)
    x = torch.randn(2 * M + 512, K, generator=g).bfloat16().to(device)
    W = (torch.randn(N, K, generator=g) / K**0.5).bfloat16().to(device)
    if not weight_trans:
        W = W.t().contiguous()
    b = torch.randn(N, generator=g).bfloat16().to(device)
    res = torch.randn(2 * M + 512, N, generator=g).bfloat16().to(device)
    ops = _ops()
    tall = ops.dense(x, W, weight_trans, b, res, "gelu")
    got = ops.dense(x[:M], W, weight_trans, b, res[:M], "gelu")
    assert torch.equal(got, tall[:M])
    close(got[::7], ref32(x[:M:7], W, weight_trans, b, res[:M:7], "gelu"), K)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (3, 11008, 4096), (16, 4096, 11008), (13, 1032, 640), (32, 4096, 512), (17, 520, 1152)])
def test_dense_decode_sizes_stream_the_weights(device, dtype, M, N, K):
    """A few activation rows against [N, K] weights take the row-streaming kernel (16 output columns per workgroup, K
    split over its four waves): against the fp32 anchor with bias, residual and every activation, ragged M and N, and a
    batch of such layers must equal the layers one by one bit for bit."""
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(dtype).to(device)
    W = (torch.randn(N, K, generator=g) / K**0.5).to(dtype).to(device)
    b = torch.randn(N, generator=g).to(dtype).to(device)
    res = torch.randn(M, N, generator=g).to(dtype).to(device)
    ops = _ops()
    for act in ("none", "silu", "gelu"):
        close(ops.dense(x, W, True, b, res, act), ref32(x, W, True, b, res, act), K)
    close(ops.dense(x, W, True, None, None, "relu"), ref32(x, W, True, None, None, "relu"), K)
    xb = torch.randn(3, M, K, generator=g).to(dtype).to(device)
    wb = (torch.randn(3, N, K, generator=g) / K**0.5).to(dtype).to(device)
    got = ops.dense_batched(xb, wb, True, None, None, "none")
    for i in range(3):
        assert torch.equal(got[i], ops.dense(xb[i], wb[i], True, None, None, "none"))


def test_dense_rejects_what_the_kernel_cannot_take(device):
    from xpu_graph_amd._lib import XgError

    x = torch.randn(8, 12, device=device).bfloat16()
    W = torch.randn(12, 8, device=device).bfloat16()
    with pytest.raises(XgError):
        _ops().dense(x, W, False, None, None, "none")  # K % 8 != 0
    with pytest.raises(ValueError):
        _ops().dense(x, torch.randn(16, 8, device=device).bfloat16(), False, None, None, "none")
    with pytest.raises(ValueError):
        _ops().dense(x, W, False, None, None, "tanh")
    assert _ops().dense(torch.empty(0, 16, device=device).bfloat16(), torch.randn(16, 8, device=device).bfloat16(), False, None, None, "none").shape == (0, 8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("weight_trans", [False, True])
@pytest.mark.parametrize("B,M,K,N", [(5, 32, 256, 256), (3, 300, 128, 520), (16, 64, 64, 72), (2, 1024, 512, 4096)])
def test_dense_batched_is_one_launch_equal_to_the_per_entry_path(device, dtype, weight_trans, B, M, K, N):
    """xg_dense_batched (batch on the second grid axis) against B separate xg_dense calls, bit for bit, and against the
    fp32 anchor; shared and per-entry bias, residual, activation.  The first shape is the reference's
    (tests/mlu/test_custom_batchdenselayer.py: batch 5, 32 x 256 outputs viewed as [5, 32, 256])."""
    g = torch.Generator().manual_seed(B * 1000 + M + N)
    x = torch.randn(B, M, K, generator=g).to(dtype).to(device)
    w = (torch.randn(B, N, K, generator=g) / K**0.5).to(dtype).to(device)
    if not weight_trans:
        w = w.transpose(1, 2).contiguous()
    bias1 = torch.randn(N, generator=g).to(dtype).to(device)
    biasb = torch.randn(B, N, generator=g).to(dtype).to(device)
    res = torch.randn(B, M, N, generator=g).to(dtype).to(device)
    ops = _ops()
    for bias, residual, act in [(None, None, "none"), (bias1, None, "silu"), (biasb, res, "gelu"), (biasb.float(), None, "relu")]:
        got = ops.dense_batched(x, w, weight_trans, bias, residual, act)
        assert got.shape == (B, M, N) and got.dtype == dtype
        for i in range(B):
            bi = None if bias is None else (bias if bias.dim() == 1 else bias[i])
            ri = None if residual is None else residual[i]
            one = ops.dense(x[i], w[i], weight_trans, bi, ri, act)
            assert torch.equal(got[i], one), (i, act)
            close(got[i], ref32(x[i], w[i], weight_trans, bi, ri, act), K)


def test_dense_batched_beyond_one_launch(device, monkeypatch):
    """More batch entries than one launch holds (the batch is the second grid axis: 65535) go out in slices with every
    operand moved on by its batch stride: a real batch of 65540 tiny layers, and a small batch with the limit lowered so
    that per-entry bias, residual and strided views cross several slice boundaries."""
    import xpu_graph_amd.ops as xops

    ops = _ops()
    g = torch.Generator().manual_seed(65540)
    B = 65540
    x = torch.randn(B, 8, 8, generator=g).bfloat16().to(device)
    w = torch.randn(B, 8, 8, generator=g).bfloat16().to(device)
    got = ops.dense_batched(x, w, False, None, None, "none")
    want = torch.bmm(x.float(), w.float())
    close(got, want, 8)
    for i in (0, 65534, 65535, 65539):
        assert torch.equal(got[i], ops.dense(x[i], w[i], False, None, None, "none")), i

    B = 8
    big = torch.randn(B, 40, 320, generator=g).bfloat16().to(device)
    xs = big[:, :32, 64:320]
    ws = (torch.randn(B, 72, 256, generator=g) / 16).bfloat16().to(device)
    biasb = torch.randn(B, 72, generator=g).bfloat16().to(device)
    res = torch.randn(B, 32, 72, generator=g).bfloat16().to(device)
    whole = ops.dense_batched(xs, ws, True, biasb, res, "silu")
    monkeypatch.setattr(xops, "MAX_BATCH_PER_LAUNCH", 3)
    sliced = ops.dense_batched(xs, ws, True, biasb, res, "silu")
    assert torch.equal(whole, sliced)
    sliced = ops.dense_batched(xs, ws, True, biasb.float(), None, "none")
    monkeypatch.setattr(xops, "MAX_BATCH_PER_LAUNCH", 65535)
    assert torch.equal(ops.dense_batched(xs, ws, True, biasb.float(), None, "none"), sliced)


def test_dense_batched_strided_entries(device):
    """Batch entries that are views: a batch stride larger than an entry, rows wider than K; a misaligned view is copied."""
    ops = _ops()
    big = torch.randn(4, 40, 320, device=device).bfloat16()
    x = big[:, :32, 64:320]  # [4, 32, 256], row stride 320, batch stride 40 * 320
    w = (torch.randn(4, 256, 72, device=device) / 16).bfloat16()
    got = ops.dense_batched(x, w, False, None, None, "none")
    for i in range(4):
        assert torch.equal(got[i], ops.dense(x[i].contiguous(), w[i], False, None, None, "none"))
    odd = big[:, :32, 3:259]  # base 6 bytes off a 16-byte boundary: the wrapper copies
    got = ops.dense_batched(odd, w, False, None, None, "none")
    for i in range(4):
        assert torch.equal(got[i], ops.dense(odd[i].contiguous(), w[i], False, None, None, "none"))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "K,M,N",
    [(64, 256, 256), (256, 512, 768), (200, 264, 304), (1, 8, 8), (1000, 1032, 72), (4096, 320, 4096), (8192, 1024, 512), (77, 4096, 11008)],
)
def test_dense_with_transposed_left_operand(device, dtype, K, M, N):
    """xg_dense_at: a_t [K, M]^T @ b [K, N], the weight gradient of a dense layer, against the fp32 product of the same
    16-bit operands; K with and without whole 64-element slabs (direct loads / staged through registers), ragged M
    and N tiles, with and without a residual."""
    g = torch.Generator().manual_seed(K + M + N)
    a_t = (torch.randn(K, M, generator=g) / K**0.25).to(dtype).to(device)
    b = (torch.randn(K, N, generator=g) / K**0.25).to(dtype).to(device)
    res = torch.randn(M, N, generator=g).to(dtype).to(device)
    got = _ops().dense_at(a_t, b, None)
    assert got.shape == (M, N) and got.dtype == dtype
    want = a_t.float().t() @ b.float()
    close(got, want, K)
    got = _ops().dense_at(a_t, b, res)
    close(got, want + res.float(), K)


def test_dense_at_reads_strided_views_in_place(device):
    ops = _ops()
    big_a = torch.randn(300, 200, device=device).bfloat16()
    big_b = torch.randn(300, 400, device=device).bfloat16()
    a_t, b = big_a[:, 8:136], big_b[:, 16:336]  # row strides 200 and 400 elements, 16-byte aligned bases
    got = ops.dense_at(a_t, b, None)
    close(got, a_t.float().t() @ b.float(), 300)
    a_t = big_a[:, 3:131]  # base 6 bytes off: the wrapper copies
    close(ops.dense_at(a_t, b, None), a_t.float().t() @ b.float(), 300)
    with pytest.raises(ValueError, match="M % 8"):
        ops.dense_at(big_a[:, :12], b, None)


def ref64(x, W, weight_trans, bias, residual, act):
    z = x.double() @ (W.double().t() if weight_trans else W.double())
    if bias is not None:
        z = z + bias.double()
    if residual is not None:
        z = z + residual.double()
    return {"none": lambda t: t, "relu": torch.relu, "silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu,
            "sigmoid": torch.sigmoid}[act](z)


def close_fp32(got, want64, k):
    """fp32 layer against the float64 product: products are exact in fp32 MFMA arithmetic and the K-term sum is
    rounded to fp32 as it grows, a random walk of half-ulp steps at the size of the partial sums -- rtol 1e-5 plus
    sqrt(K) * 2^-24 of the largest output."""
    assert got.dtype == torch.float32
    atol = want64.abs().max().item() * (k**0.5) * 2.0**-24
    torch.testing.assert_close(got.double(), want64, rtol=1e-5, atol=atol)


@pytest.mark.parametrize("weight_trans", [False, True])
@pytest.mark.parametrize(
    "M,N,K", [(256, 256, 32), (512, 768, 256), (300, 264, 200), (1, 8, 4), (1000, 1032, 76), (4096, 16, 768), (64, 4096, 4096), (2048, 2048, 2048)]
)
def test_dense_fp32_shapes(device, weight_trans, M, N, K):
    """The fp32 layer (32x32x2 fp32 MFMA): whole and partial 32-element slabs, ragged tiles, the reference's own
    dense-layer test shape ([4096, 768] x [768, 16], tests/mlu/test_custom_denselayer.py:112-119), both weight
    layouts, bias / residual / activation in the epilogue."""
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(device)
    W = (torch.randn(N, K, generator=g) / K**0.5).to(device)
    if not weight_trans:
        W = W.t().contiguous()
    b = torch.randn(N, generator=g).to(device)
    res = torch.randn(M, N, generator=g).to(device)
    got = _ops().dense(x, W, weight_trans, None, None, "none")
    assert got.shape == (M, N)
    close_fp32(got, ref64(x, W, weight_trans, None, None, "none"), K)
    got = _ops().dense(x, W, weight_trans, b, res, "gelu")
    close_fp32(got, ref64(x, W, weight_trans, b, res, "gelu"), K)


def test_dense_fp32_exact_on_small_integers(device):
    """Integer-valued operands whose products and sums stay below 2^24 come out exact: a dropped k-step, a swapped
    fragment or a wrong swizzle cannot hide behind a tolerance."""
    g = torch.Generator().manual_seed(5)
    for weight_trans in (False, True):
        x = torch.randint(-8, 9, (520, 328), generator=g).float().to(device)
        W = torch.randint(-8, 9, (328, 264), generator=g).float().to(device)
        want = x.double() @ W.double()
        Wk = W.t().contiguous() if weight_trans else W
        got = _ops().dense(x, Wk, weight_trans, None, None, "none")
        assert torch.equal(got.double(), want)


def test_dense_takes_column_sliced_views(device):
    """A linear layer fed by a column slice of a wider tensor: row strides or bases that are not multiples of 16 bytes
    (what eager accepts anywhere) are copied by the wrapper instead of being refused by the kernel."""
    ops = _ops()
    big = torch.randn(128, 100, device=device).bfloat16()
    w = (torch.randn(64, 72, device=device) / 8).bfloat16()
    for x in (big[:, :64], big[:, 4:68], big[:, 3:67]):  # pitch 200 bytes; bases 0, 8 and 6 bytes in
        got = ops.dense(x, w, False, None, None, "none")
        close(got, ref32(x, w, False, None, None, "none"), 64)
    wbig = (torch.randn(72, 100, device=device) / 8).bfloat16()
    got = ops.dense(big[:, 4:68], wbig[:, 4:68], True, None, big[:, 20:92], "silu")  # strided weight and residual too
    close(got, ref32(big[:, 4:68], wbig[:, 4:68], True, None, big[:, 20:92], "silu"), 64)
    glu = ops.dense_glu(big[:, 4:68], wbig[:, 4:68], wbig[:, 30:94])
    close_glu(glu, big[:, 4:68], wbig[:, 4:68], wbig[:, 30:94])


def close_glu(got, x, wg, wu):
    """The gated layer rounds each projection to the storage type before the gate (as the two separate layers it
    replaces do), so its anchor is silu(round(x Wg^T)) * round(x Wu^T) with the products in fp32."""
    gate = (x.float() @ wg.float().t()).to(got.dtype).float()
    up = (x.float() @ wu.float().t()).to(got.dtype).float()
    want = torch.nn.functional.silu(gate) * up
    assert_close_16bit(got, want, dense_floor(want, got.dtype), f"dense_glu {tuple(got.shape)} {got.dtype}")


@pytest.mark.parametrize("form", ["plain", "bias_act", "residual", "w_trans"])
def test_batch_dense_compiled(device, form):
    """bmm-based layers through torch.compile on the mi355x target: all batch entries in one xg_dense_batched launch."""
    from xpu_graph_amd import mi355x_compiler

    B, M, K, N = 5, 300, 256, 520
    g = torch.Generator().manual_seed(3)
    x = torch.randn(B, M, K, generator=g).bfloat16().to(device)
    w = (0.1 * torch.randn(B, K, N, generator=g)).bfloat16().to(device)
    wt = w.transpose(1, 2).contiguous()
    bias = torch.randn(B, 1, N, generator=g).bfloat16().to(device)
    res = torch.randn(B, M, N, generator=g).bfloat16().to(device)
    fns = {
        "plain": (lambda x, w: torch.bmm(x, w), (x, w)),
        "bias_act": (lambda x, w, b: F.silu(torch.bmm(x, w) + b), (x, w, bias)),
        "residual": (lambda x, w, r: torch.bmm(x, w) + r, (x, w, res)),
        "w_trans": (lambda x, w: F.gelu(torch.bmm(x, w.transpose(1, 2))), (x, wt)),
    }
    fn, args = fns[form]
    backend = mi355x_compiler()
    with torch.no_grad():
        got = torch.compile(fn, backend=backend, dynamic=False)(*args)
    assert [n.target for n in backend.compiled_graphs[-1].graph.nodes if n.op == "call_module"] == ["custom_batch_dense_layer_replacement"]
    want = fn(*[a.float() for a in args])
    close(got, want, K)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "M,N,K",
    [
        (256, 128, 64),      # one tile, one slab
        (8192, 1280, 256),   # 8 full tile columns + a 2-column tail computed as half-height tiles in the same launch
        (1000, 200, 128),    # ragged rows and a last tile with 72 of 128 columns
        (130, 8, 4096),      # a sliver of columns, deep K
        (4096, 11008, 512),  # the Llama gate / up width
        (1, 11008, 4096),    # a decode step: both weights streamed row by row
        (4, 4096, 1024),
        (32, 4096, 512),     # two 16-row tiles of activations
        (13, 1032, 640),     # ragged rows and columns
        (16, 11008, 4096),   # where the plain layer takes the 64 x 64 kernel, so does the gated one
        (64, 11008, 512),
        (128, 11008, 512),   # the last row count at which the gated layer follows the plain layer's small-size choices
    ],
)
def test_dense_glu_bit_identical_to_the_unfused_ops(device, dtype, M, N, K):
    """silu(x Wg^T) * (x Wu^T) in one launch == two dense launches + the gate kernel, bit for bit, and within the
    16-bit tolerance of the fp32 evaluation."""
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(dtype).to(device)
    wg = (torch.randn(N, K, generator=g) / K**0.5).to(dtype).to(device)
    wu = (torch.randn(N, K, generator=g) / K**0.5).to(dtype).to(device)
    ops = _ops()
    got = ops.dense_glu(x, wg, wu)
    gate, up = ops.dense(x, wg, True, None, None, "none"), ops.dense(x, wu, True, None, None, "none")
    two = ops.silu_mul2(gate, up)
    assert torch.equal(got, two)
    close_glu(got, x, wg, wu)
    if M <= 64:  # the variant that also hands back the two projections, at the decode sizes
        y, g_out, u_out = ops.dense_glu_save(x, wg, wu)
        assert torch.equal(y, got) and torch.equal(g_out, gate) and torch.equal(u_out, up)


@pytest.mark.parametrize("M,N,K", [(1024, 4096, 256), (900, 2056, 128)])
def test_dense_glu_half_height_grid(device, M, N, K):
    """A gated layer whose full-size grid would leave most of a round empty runs as 128-row tiles throughout."""
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).bfloat16().to(device)
    wg = (torch.randn(N, K, generator=g) / K**0.5).bfloat16().to(device)
    wu = (torch.randn(N, K, generator=g) / K**0.5).bfloat16().to(device)
    got = torch.ops.xpu_ops.dense_glu(x, wg, wu)
    close_glu(got, x, wg, wu)
    xi = torch.randint(-2, 3, (M, K), generator=g).bfloat16().to(device)
    wi = torch.randint(-2, 3, (N, K), generator=g).bfloat16().to(device)
    gate = (xi.float() @ wi.float().t()).bfloat16().float()
    want = (torch.nn.functional.silu(gate) * gate).bfloat16()
    torch.testing.assert_close(torch.ops.xpu_ops.dense_glu(xi, wi, wi).float(), want.float(), rtol=8e-3, atol=1e-2)


def test_dense_glu_strided_operands_and_rejects(device):
    ops = _ops()
    big = torch.randn(64, 512, device=device).bfloat16()
    x = big[:, 128:384]  # row stride 512, K = 256
    wbig = (torch.randn(2, 40, 256, device=device) / 16).bfloat16()
    got = ops.dense_glu(x, wbig[0], wbig[1])
    close_glu(got, x, wbig[0], wbig[1])
    with pytest.raises(ValueError):
        ops.dense_glu(x[:, :96], wbig[0][:, :96], wbig[1][:, :96])  # K not a multiple of 64
    with pytest.raises(ValueError):
        ops.dense_glu(x, wbig[0], wbig[1][:32])  # weights of different shape
    with pytest.raises(ValueError):
        ops.dense_glu(x.float(), wbig[0].float(), wbig[1].float())
