"""The one place that states how close a 16-bit kernel result must be to its anchor.

Anchor: the same op evaluated in fp32 on the SAME low-precision inputs (no intermediate rounding).  Against it a
kernel that accumulates in fp32 and rounds once is off by half a unit in the last place of the output type plus its
accumulation-order noise, so the assertion is

    |got - want| <= 1.6e-2 * |want| + floor

with rtol 1.6e-2 as the benchmark definition states it for bf16 / fp8-dequantised outputs, and an absolute `floor`
that only matters for outputs that are nearly zero by cancellation.  The floor is stated per kernel family in terms
of the tensor's own range (never a constant typed into a test):

* dense (one rounding of an fp32 sum of exact products): one ulp of the output type at max|want| * 2^-7.
* attention (the probabilities are rounded to the storage type before they multiply V, as in every single-pass
  attention kernel): 2^-9 * max|want| for bf16 (half an ulp of a probability, times the largest value), 2^-12 for
  fp16.
* fp8 dense (the e4m3 MFMA adds its 64 products with a shortened, aligned mantissa: measured 2^-13 of the largest
  product per instruction): 2^-10 * max|want|.

Every call records the largest error in units of the output type's ulp at |want| (over the elements within 2^-6 of
the largest magnitude); the session prints the worst per kernel family at the end, so a drift shows long before an
assertion trips.
"""
import torch

RTOL_16BIT = 1.6e-2
RECORDS = []  # (label, max ulp error, max abs error, floor)


def _spacing(want32, dtype):
    """Distance between neighbouring `dtype` values at the magnitude of each element of want32."""
    bits = {torch.bfloat16: 8, torch.float16: 11}[dtype]  # significand bits incl. the implicit one
    emin = {torch.bfloat16: -126, torch.float16: -14}[dtype]
    _, e = torch.frexp(want32.abs().clamp_min(2.0**emin))  # |w| = m * 2^e, m in [0.5, 1)
    return torch.ldexp(torch.ones_like(want32), e - bits)


def ulp_error(got, want32):
    """max |got - want| in ulps of got's dtype at |want|, over the elements within 2^-6 of the largest magnitude
    (below that the absolute floor decides, and an ulp of a nearly cancelled sum says nothing about the kernel)."""
    g = got.float()
    big = want32.abs().max()
    if big == 0:  # an exactly cancelled result: only the absolute floor applies
        return 0.0
    ok = torch.isfinite(want32) & (want32.abs() >= big * 2.0**-6)
    if not ok.any():
        return 0.0
    return ((g - want32).abs() / _spacing(want32, got.dtype))[ok].max().item()


def dense_floor(want32, dtype):
    m = want32.abs().max().clamp_min(1e-30)
    return _spacing(m * 2.0**-7, dtype).item()


def attention_floor(want32, dtype):
    return want32.abs().max().item() * (2.0**-9 if dtype == torch.bfloat16 else 2.0**-12)


def fp8_dense_floor(want32, dtype):
    return max(want32.abs().max().item() * 2.0**-10, dense_floor(want32, dtype))


def assert_close_16bit(got, want32, floor, label):
    """got: bf16 / fp16 kernel output; want32: the fp32 anchor; floor: one of the *_floor values above."""
    assert got.dtype in (torch.bfloat16, torch.float16), got.dtype
    want32 = want32.float()
    err = (got.float() - want32).abs()
    ulps = ulp_error(got, want32)
    RECORDS.append((label, ulps, err.max().item() if err.numel() else 0.0, floor))
    torch.testing.assert_close(got.float(), want32, rtol=RTOL_16BIT, atol=floor, msg=lambda m: f"{label}: {m} (max {ulps:.2f} ulp)")


def attention_grad_floor(want32, dtype):
    """Gradients of attention: the probabilities and the score gradients are rounded to the storage type before
    they multiply dO / Q / K (as in every tiled attention backward), and a gradient element sums one such product
    per key (or query), so its error is a random walk of half-ulp steps: 2^-7 of the largest gradient for bf16,
    2^-10 for fp16."""
    return want32.abs().max().item() * (2.0**-7 if dtype == torch.bfloat16 else 2.0**-10)
