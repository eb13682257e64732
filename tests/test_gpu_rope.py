"""GPU parity of the rotary-embedding kernel (torch.ops.xpu_ops.rope -> xg_rope)
against the eager rotate-half form used by the Llama block oracle
(oracle/eager.py: llama_block_eager), evaluated in fp32 on the same bf16 / fp16
inputs; tolerance rtol 1.6e-2.  The reference has no rotary pattern."""
import pytest
import torch

from oracle import eager

pytestmark = pytest.mark.gpu


def _ops():
    import xpu_graph_amd.ops  # noqa: F401

    return torch.ops.xpu_ops


def ref32(x, cos, sin):
    xf = x.float()
    return xf * cos.float() + eager._rotate_half(xf) * sin.float()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,S,D", [(1, 1, 1, 16), (2, 3, 17, 64), (2, 8, 300, 128), (1, 4, 64, 256)])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
def test_rope_shapes_and_layouts(device, dtype, B, H, S, D, layout):
    g = torch.Generator().manual_seed(B + H + S + D)
    if layout == "bhsd":
        x = torch.randn(B, H, S, D, generator=g).to(dtype).to(device)
    else:
        x = torch.randn(B, S, H, D, generator=g).to(dtype).to(device).transpose(1, 2)
    cos, sin = eager.rope_tables(S, D, device=device, dtype=dtype)
    got = _ops().rope(x, cos, sin)
    assert got.shape == x.shape and got.dtype == dtype and got.stride() == x.stride()
    torch.testing.assert_close(got.float(), ref32(x, cos, sin), rtol=1.6e-2, atol=1e-2)
    got = _ops().rope(x, cos.float()[None, None], sin.float()[None, None])  # fp32 tables with leading unit dims
    torch.testing.assert_close(got.float(), ref32(x, cos.float(), sin.float()), rtol=1.6e-2, atol=1e-2)


@pytest.mark.parametrize("S", [1, 5])
@pytest.mark.parametrize("table_shape", ["row", "one_by_d", "leading_ones"])
def test_rope_with_one_table_row_for_every_position(device, S, table_shape):
    """A decode step rotates its one new position with that position's row of the tables: cos / sin [D] (or [1, D],
    [1, 1, 1, D]) are shared by every position of x, as broadcasting in the eager form says."""
    g = torch.Generator().manual_seed(S)
    x = torch.randn(3, 4, S, 128, generator=g).bfloat16().to(device)
    cos, sin = (t[37] for t in eager.rope_tables(64, 128, device=device, dtype=torch.bfloat16))
    if table_shape == "one_by_d":
        cos, sin = cos[None], sin[None]
    elif table_shape == "leading_ones":
        cos, sin = cos[None, None, None], sin[None, None, None]
    got = _ops().rope(x, cos, sin)
    assert got.shape == x.shape and got.dtype == x.dtype
    torch.testing.assert_close(got.float(), ref32(x, cos, sin), rtol=1.6e-2, atol=1e-2)


def test_rope_invariants(device):
    """cos = 1, sin = 0 is the identity; cos = 0, sin = 1 is rotate-half exactly; position 0 of the real tables
    leaves x unchanged; the rotation preserves the norm of every (c, c + D/2) pair."""
    x = torch.randn(2, 4, 33, 128, device=device).bfloat16()
    one, zero = torch.ones(33, 128, device=device).bfloat16(), torch.zeros(33, 128, device=device).bfloat16()
    assert torch.equal(_ops().rope(x, one, zero), x)
    assert torch.equal(_ops().rope(x, zero, one), eager._rotate_half(x))
    cos, sin = eager.rope_tables(33, 128, device=device, dtype=torch.float32)
    out = _ops().rope(x, cos, sin)
    assert torch.equal(out[:, :, 0], x[:, :, 0])
    n_in = x.float()[..., :64] ** 2 + x.float()[..., 64:] ** 2
    n_out = out.float()[..., :64] ** 2 + out.float()[..., 64:] ** 2
    torch.testing.assert_close(n_out, n_in, rtol=3e-2, atol=1e-2)


def test_rope_c5_full_size(device):
    B, H, S, D = 4, 32, 2048, 128
    x = torch.randn(B, S, H, D, device=device).bfloat16().transpose(1, 2)
    cos, sin = eager.rope_tables(S, D, device=device, dtype=torch.bfloat16)
    got = _ops().rope(x, cos, sin)
    torch.testing.assert_close(got.float(), ref32(x, cos, sin), rtol=1.6e-2, atol=1e-2)
    # the eager bf16 form rounds four times; it must agree at the same tolerance
    want = x * cos + eager._rotate_half(x) * sin
    torch.testing.assert_close(got.float(), want.float(), rtol=1.6e-2, atol=3e-2)


def test_rope_rejects_what_the_kernel_cannot_take(device):
    x = torch.randn(1, 2, 8, 64, device=device).bfloat16()
    t = torch.randn(8, 64, device=device).bfloat16()
    with pytest.raises(Exception):
        _ops().rope(x.float(), t.float(), t.float())  # fp32 activations
    with pytest.raises(Exception):
        _ops().rope(x, t[:4], t[:4])  # table length
    with pytest.raises(Exception):
        _ops().rope(x[..., :24], t[:, :24], t[:, :24])  # head dim not a multiple of 16
