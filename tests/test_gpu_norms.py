"""GPU parity of the norm kernels (through torch.ops.xpu_ops -> C ABI) against
the eager oracle.  Tolerances: fp32 rtol 1e-5 (atol 1e-5); bf16/fp16 rtol
1.6e-2 (atol 1e-5 against the single-rounding definition; the residual sum is
bit-exact)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import eager, inputs

pytestmark = pytest.mark.gpu

F32 = dict(rtol=1e-5, atol=1e-5)
LOW = dict(rtol=1.6e-2, atol=1e-5)


def _ops():
    import xpu_graph_amd.ops  # noqa: F401  (registers torch.ops.xpu_ops)

    return torch.ops.xpu_ops


def _tol(dtype):
    return F32 if dtype == torch.float32 else LOW


@pytest.mark.parametrize("rows,cols", [(2048, 4096), (1, 4096), (7, 128), (33, 8), (5, 12288), (3, 32768), (4, 100), (2, 4097), (9, 3)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_rms_norm(device, rows, cols, dtype):
    x, w = inputs.c1_rmsnorm(rows, cols, device)
    x, w = x.to(dtype), w.to(dtype)
    got = _ops().rms_norm(x, w, 1e-6)
    torch.testing.assert_close(got, eager.default_rms_norm(x, w, 1e-6), **_tol(dtype))
    torch.testing.assert_close(got, F.rms_norm(x.float(), (cols,), w.float(), 1e-6).to(dtype), **_tol(dtype))
    if dtype == torch.float32:
        torch.testing.assert_close(got, eager.rmsnorm_eager(x, w, 1e-6), **F32)
    # no weight; fp32 weight with low-precision input
    got = _ops().rms_norm(x, None, 1e-5)
    torch.testing.assert_close(got, eager.default_rms_norm(x, None, 1e-5), **_tol(dtype))
    got = _ops().rms_norm(x, w.float(), 1e-6)
    torch.testing.assert_close(got, eager.default_rms_norm(x, w.float(), 1e-6), **_tol(dtype))


def test_rms_norm_c1_full_bitwise_repeatable(device):
    x, w = inputs.c1_rmsnorm(device=device)
    a = _ops().rms_norm(x, w, 1e-6)
    b = _ops().rms_norm(x, w, 1e-6)
    assert torch.equal(a, b)
    torch.testing.assert_close(a, eager.rmsnorm_eager(x, w, 1e-6), **F32)
    # invariant: rows of the un-weighted norm have mean square 1 (up to eps)
    u = _ops().rms_norm(x, None, 1e-6)
    torch.testing.assert_close(u.pow(2).mean(-1), torch.ones(x.shape[0], device=device), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("rows,cols", [(64, 4096), (3, 768), (5, 1000), (2, 16384), (1, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_layer_norm(device, rows, cols, dtype):
    x, _, g, b = inputs.c2_add_layernorm(rows, cols, device, dtype=dtype)
    got = _ops().layer_norm(x, g, b, 1e-5)
    torch.testing.assert_close(got, eager.default_layer_norm(x, g, b, 1e-5), **_tol(dtype))
    torch.testing.assert_close(got, F.layer_norm(x.float(), (cols,), g.float(), b.float(), 1e-5).to(dtype), **_tol(dtype))
    got = _ops().layer_norm(x, None, None, 1e-5)
    torch.testing.assert_close(got, eager.default_layer_norm(x, None, None, 1e-5), **_tol(dtype))
    got = _ops().layer_norm(x, g.float(), b.float(), 1e-5)
    torch.testing.assert_close(got, eager.default_layer_norm(x, g.float(), b.float(), 1e-5), **_tol(dtype))


@pytest.mark.parametrize("rows,cols", [(8192, 4096), (17, 4096), (3, 520), (2, 77)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_add_layer_norm(device, rows, cols, dtype):
    x, r, g, b = inputs.c2_add_layernorm(rows, cols, device, dtype=dtype)
    y, h = _ops().add_layer_norm(x, r, g, b, 1e-5)
    y_ref, h_ref = eager.add_layernorm_eager(x, r, g, b, 1e-5)
    assert torch.equal(h, h_ref)  # the updated residual is a rounded sum: bit-exact
    torch.testing.assert_close(y, y_ref, **_tol(dtype))
    torch.testing.assert_close(y, eager.default_layer_norm(h_ref, g, b, 1e-5), **_tol(dtype))
    y1 = _ops().add_layer_norm_only(x, r, g, b, 1e-5)
    assert torch.equal(y1, y)
    if dtype != torch.float32:
        # decomposed spelling rounds three times in low precision: same rtol, atol of one bf16 ulp at |y|~4
        y_dec, _ = eager.add_layernorm_decomposed_eager(x, r, g, b, 1e-5)
        torch.testing.assert_close(y, y_dec, rtol=1.6e-2, atol=3.2e-2)


@pytest.mark.parametrize("rows,cols", [(8192, 4096), (5, 4096), (3, 136), (2, 50)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_add_rms_norm(device, rows, cols, dtype):
    x, r, g, _ = inputs.c2_add_layernorm(rows, cols, device, dtype=dtype)
    y, h = _ops().add_rms_norm(x, r, g, 1e-6)
    y_ref, h_ref = eager.add_rmsnorm_eager(x, r, g, 1e-6)
    assert torch.equal(h, h_ref)
    torch.testing.assert_close(y, y_ref, **_tol(dtype))
    assert torch.equal(_ops().add_rms_norm_only(x, r, g, 1e-6), y)


def test_norm_strided_rows(device):
    big = torch.randn(64, 8192, device=device)
    x = big[:, :4096]  # row stride 8192, unit column stride: taken without a copy
    w = torch.randn(4096, device=device)
    torch.testing.assert_close(_ops().rms_norm(x, w, 1e-6), eager.default_rms_norm(x, w, 1e-6), **F32)
    x3 = torch.randn(4, 16, 512, device=device, dtype=torch.bfloat16)
    torch.testing.assert_close(_ops().rms_norm(x3, None, 1e-6), eager.default_rms_norm(x3, None, 1e-6), **LOW)
    xt = torch.randn(512, 64, device=device).t()  # column stride != 1: copied
    torch.testing.assert_close(_ops().rms_norm(xt, None, 1e-6), eager.default_rms_norm(xt, None, 1e-6), **F32)


def test_norm_empty_and_errors(device):
    x = torch.empty(0, 128, device=device)
    assert _ops().rms_norm(x, None, 1e-6).shape == (0, 128)
    with pytest.raises(NotImplementedError):
        _ops().rms_norm(torch.randn(4, 8), None, 1e-6)  # CPU tensors: there is no fallback
    with pytest.raises(TypeError):
        _ops().rms_norm(torch.randn(4, 8, device=device, dtype=torch.float64), None, 1e-6)


def test_add_layer_norm_c2_full_size_properties(device):
    """Size-independent properties at the full C2 shape: unit-affine rows come out with mean 0 and variance 1; a shift
    of the input by a per-row constant does not change the result (up to the rounding of the shifted input); the
    second output is the rounded sum, bit for bit; repeated launches agree bit for bit."""
    x, r, g, b = inputs.c2_add_layernorm(device=device)
    ops = _ops()
    one, zero = torch.ones_like(g), torch.zeros_like(b)
    y, h = ops.add_layer_norm(x, r, one, zero, 1e-5)
    assert torch.equal(h, x + r)
    yf = y.float()
    torch.testing.assert_close(yf.mean(-1), torch.zeros(x.shape[0], device=device), rtol=0, atol=2e-3)
    torch.testing.assert_close(yf.var(-1, unbiased=False), torch.ones(x.shape[0], device=device), rtol=1e-2, atol=1e-2)
    y2, h2 = ops.add_layer_norm(x, r, one, zero, 1e-5)
    assert torch.equal(y, y2) and torch.equal(h, h2)
    # fp32 inputs for the shift property (a bf16 shift would round the data itself)
    xf = x.float()
    shift = torch.randn(x.shape[0], 1, device=device) * 4
    a = ops.layer_norm(xf, g.float(), b.float(), 1e-5)
    c = ops.layer_norm(xf + shift, g.float(), b.float(), 1e-5)
    torch.testing.assert_close(a, c, rtol=1e-4, atol=1e-4)
