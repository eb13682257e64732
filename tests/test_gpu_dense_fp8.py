"""GPU parity of the fp8 (OCP e4m3) dense layer (torch.ops.xpu_ops.dense_fp8 ->
xg_dense_fp8): activations quantised per tensor, weights per output channel,
fp32 accumulation, scales / bias / activation in the epilogue.  The reference
has no fp8 path; the oracle is the dequantised fp32 product (exact for the
same quantised operands), tolerance rtol 1.6e-2 with the fp8 floor of
tests/tolerance.py (2^-10 of the largest output: the e4m3 MFMA's shortened sum)."""
import json
import os

import pytest
import torch

from oracle import eager, inputs
from tests.tolerance import assert_close_16bit, fp8_dense_floor

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _ops():
    import xpu_graph_amd.ops  # noqa: F401

    return torch.ops.xpu_ops


def close(got, want):
    """Against the dequantised fp32 product `want` of the same e4m3 operands."""
    if got.dtype == torch.float32:  # fp32 output: no output rounding, only the MFMA's own accumulation error
        torch.testing.assert_close(got, want, rtol=1e-3, atol=want.abs().max().item() * 2.0**-10)
        return
    assert_close_16bit(got, want, fp8_dense_floor(want, got.dtype), f"dense_fp8 {tuple(got.shape)} {got.dtype}")


def quantised(M, N, K, device, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    W = torch.randn(K, N, generator=g) / K**0.5
    b = 0.1 * torch.randn(N, generator=g)
    x_q, s_x = eager.quantize_fp8_per_tensor(x)
    W_q, s_w = eager.quantize_fp8_per_out_channel(W)
    return x_q.to(device), W_q.to(device), s_x.to(device), s_w.to(device), b.to(device)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (512, 768, 256), (300, 264, 208), (1, 8, 16), (1000, 1032, 80), (64, 2048, 4096)])
def test_dense_fp8_shapes(device, out_dtype, M, N, K):
    x_q, W_q, s_x, s_w, b = quantised(M, N, K, device, seed=M + N + K)
    w_nk = W_q.t().contiguous()  # the kernel takes the weight as [N, K]
    got = _ops().dense_fp8(x_q, w_nk, True, s_x, s_w, b, "silu", out_dtype)
    assert got.shape == (M, N) and got.dtype == out_dtype
    want = eager.dense_fp8_silu_eager(x_q, W_q, s_x, s_w, b)
    close(got, want)
    got = _ops().dense_fp8(x_q, w_nk, True, s_x, s_w, None, "none", out_dtype)
    want = (x_q.float() @ W_q.float()) * s_x * s_w
    close(got, want)


def test_dense_fp8_accumulation_precision(device):
    """The e4m3 MFMA adds its 64 products per instruction with a shortened aligned mantissa: measured error
    is about 2^-13 of the largest product, far inside the fp8 tolerance but not fp32-exact.  Pin that bound."""
    x_q, W_q, _, _, _ = quantised(512, 512, 4096, device, seed=2)
    one = torch.ones(1, device=device)
    got = _ops().dense_fp8(x_q, W_q.t().contiguous(), True, one, one.expand(512).contiguous(), None, "none", torch.float32)
    exact = x_q.double() @ W_q.double()
    weight = x_q.double().abs() @ W_q.double().abs()
    assert ((got.double() - exact).abs() / weight).max().item() < 1e-4


def test_dense_fp8_decodes_every_code(device):
    """Every finite e4m3 code times 1.0 comes back as the value the format defines (known-answer table)."""
    with open(os.path.join(GOLDEN, "fp8_e4m3fn_kat.json")) as f:
        kat = json.load(f)
    codes = torch.arange(256, dtype=torch.uint8)
    finite = (codes & 0x7F) != 0x7F
    a = torch.zeros(256, 16, dtype=torch.uint8)
    a[:, 3] = torch.where(finite, codes, torch.zeros_like(codes))
    w = torch.zeros(8, 16, dtype=torch.uint8)
    w[5, 3] = 0x38  # 1.0
    one = torch.ones(1, device=device)
    got = _ops().dense_fp8(a.view(torch.float8_e4m3fn).to(device), w.view(torch.float8_e4m3fn).to(device), True, one, one.expand(8), None, "none", torch.float32)
    want = a[:, 3].view(torch.float8_e4m3fn).float()
    assert torch.equal(got[:, 5].cpu(), want)
    assert torch.count_nonzero(got[:, :5]) == 0 and torch.count_nonzero(got[:, 6:]) == 0
    for code, val in zip(kat["codes"], kat["decoded"]):  # the committed known answers, through the MFMA decode
        assert got[code, 5].item() == val


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize(
    "M,N,K",
    [(1, 4096, 4096), (16, 4096, 4096), (17, 4096, 4096), (32, 4096, 11008), (5, 11008, 4096), (3, 520, 1024), (32, 1000, 1280), (9, 512, 2304)],
)
def test_dense_fp8_decode_sizes(device, out_dtype, M, N, K):
    """At most 32 rows against a whole weight matrix: the row-streaming e4m3 kernel (a workgroup per 16 weight rows, K
    split over its four wavefronts).  Ragged N (not a multiple of 16), K quarters that leave a tail after the unrolled
    groups (1280, 2304), both row-tile counts."""
    x_q, W_q, s_x, s_w, b = quantised(M, N, K, device, seed=M + N + K)
    w_nk = W_q.t().contiguous()
    for bias, act in ((b, "silu"), (None, "none"), (b.to(out_dtype), "gelu")):
        got = _ops().dense_fp8(x_q, w_nk, True, s_x, s_w, bias, act, out_dtype)
        assert got.shape == (M, N) and got.dtype == out_dtype
        z = (x_q.float() @ W_q.float()) * s_x * s_w
        if bias is not None:
            z = z + bias.float()
        want = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "none": lambda t: t}[act](z)
        close(got, want)
    # a row of the batch equals the same row computed alone: the kernels of 1..16 and of 17..32 rows add in one order
    alone = _ops().dense_fp8(x_q[M - 1 :], w_nk, True, s_x, s_w, b, "silu", out_dtype)
    batch = _ops().dense_fp8(x_q, w_nk, True, s_x, s_w, b, "silu", out_dtype)
    assert torch.equal(alone[0], batch[M - 1])


def test_dense_fp8_decode_kernel_pairs_every_k(device):
    """One non-zero activation at position k and one-hot weight rows: the output is the product exactly when the
    kernel pairs activation byte k with weight byte k, for every k of a wavefront's quarter and every quarter."""
    K, N = 1024, 512
    one = torch.ones(1, device=device)
    for k in list(range(0, 80)) + [255, 256, 511, 777, 1023]:
        x = torch.zeros(2, K, dtype=torch.uint8)
        x[1, k] = 0x40  # 2.0
        w = torch.zeros(N, K, dtype=torch.uint8)
        w[:, k] = 0x38  # 1.0
        w[7, k] = 0x34  # 0.75
        w[7, (k + 8) % K] = 0x48  # 4.0 at a position the activation does not have
        got = _ops().dense_fp8(x.view(torch.float8_e4m3fn).to(device), w.view(torch.float8_e4m3fn).to(device), True, one, one.expand(N).contiguous(), None, "none", torch.float32)
        want = torch.full((N,), 2.0)
        want[7] = 1.5
        assert torch.equal(got[1].cpu(), want), k
        assert torch.count_nonzero(got[0]) == 0


def test_dense_fp8_c4_full_size(device):
    x, W, b = inputs.c4_dense(device=device)
    x_q, s_x = eager.quantize_fp8_per_tensor(x)
    W_q, s_w = eager.quantize_fp8_per_out_channel(W)
    got = _ops().dense_fp8(x_q, W_q.t().contiguous(), True, s_x, s_w, b, "silu", torch.bfloat16)
    for r0 in range(0, 8192, 1024):  # every row against the dequantised fp32 product, 1024 rows of reference at a time
        rows = slice(r0, r0 + 1024)
        close(got[rows], eager.dense_fp8_silu_eager(x_q[rows], W_q, s_x, s_w, b))
    # against the unquantised layer: per-tensor / per-channel e4m3 keeps about two significant digits
    rows = torch.arange(0, 8192, 61, device=device)
    full = eager.dense_silu_eager(x[rows], W, b).float()
    err = (got[rows].float() - full).abs().mean() / full.abs().mean()
    assert err < 0.08


def test_dense_fp8_rejects_kn_weight(device):
    x_q, W_q, s_x, s_w, b = quantised(64, 64, 64, device, seed=1)
    with pytest.raises(Exception):
        _ops().dense_fp8(x_q, W_q, False, s_x, s_w, b, "none", torch.bfloat16)


def test_fp8_dense_plugin_pattern_end_to_end(device):
    """The user's eager fp8 layer, compiled for the mi355x target with the plugin pattern registered, runs on the
    fp8 MFMA kernel and agrees with the same eager function (reference plugin API: plugin_pattern.py:114-284)."""
    from xpu_graph_amd import enable_plugin_patterns, mi355x_compiler, plugins

    M, N, K = 512, 1024, 2048
    x_q, W_q, s_x, s_w, b = quantised(M, N, K, device, seed=4)
    w_nk = W_q.t().contiguous()
    b16 = b.bfloat16()
    with enable_plugin_patterns():
        plugins.register_fp8_dense(plugins.fp8_linear_silu_eager, act="silu")
        be = mi355x_compiler()
        got = torch.compile(plugins.fp8_linear_silu_eager, backend=be, dynamic=False)(x_q, w_nk, s_x, s_w, b16)
    assert any("dense_fp8" in str(n.target) for n in be.compiled_graphs[-1].graph.nodes)
    want = plugins.fp8_linear_silu_eager(x_q, w_nk, s_x, s_w, b16)
    torch.testing.assert_close(got.float(), want.float(), rtol=1.6e-2, atol=4e-3)
