"""xg_sdpa_backward_static (the attention backward that allocates nothing: its workspace is an array in the
library's device image) against xg_sdpa_backward, through the C ABI, bit for bit; two calls in a row, the second
on a smaller problem, so that what the first left in the shared workspace cannot leak into the second."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

S3 = ctypes.c_int64 * 3


def _call_both(lib, B, H, Hkv, Sq, Skv, D, causal, seed, device):
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    q = torch.randn(B, H, Sq, D, generator=g).to(bf).to(device)
    k = torch.randn(B, Hkv, Skv, D, generator=g).to(bf).to(device)
    v = torch.randn(B, Hkv, Skv, D, generator=g).to(bf).to(device)
    d_out = torch.randn(B, H, Sq, D, generator=g).to(bf).to(device)
    out = torch.empty_like(q)
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device=device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    st = lambda t: S3(*t.stride()[:3])  # noqa: E731
    scale = D**-0.5
    assert lib.xg_sdpa_lse(P(q), P(k), P(v), P(out), P(lse), B, H, Hkv, Sq, Skv, D, st(q), st(k), st(v), st(out), scale, causal, 2, stream) == 0
    results = []
    for static in (False, True):
        dq, dk, dv = torch.full_like(q, float("nan")), torch.full_like(k, float("nan")), torch.full_like(v, float("nan"))
        tail = (B, H, Hkv, Sq, Skv, D, st(q), st(k), st(v), st(out), st(d_out), st(dq), st(dk), st(dv), scale, causal, 2, stream)
        if static:
            rc = lib.xg_sdpa_backward_static(P(q), P(k), P(v), P(out), P(d_out), P(lse), P(dq), P(dk), P(dv), *tail)
        else:
            delta = torch.empty(B, H, Sq, dtype=torch.float32, device=device)
            rc = lib.xg_sdpa_backward(P(q), P(k), P(v), P(out), P(d_out), P(lse), P(dq), P(dk), P(dv), P(delta), *tail)
        assert rc == 0, rc
        torch.cuda.synchronize()
        results.append((dq, dk, dv))
    for a, b in zip(*results):
        assert not torch.isnan(a.float()).any()
        assert torch.equal(a, b)


def test_static_workspace_backward_matches_the_workspace_argument_form(device):
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    _call_both(lib, 2, 8, 4, 700, 650, 128, 1, 1, device)  # 11 200 query rows
    _call_both(lib, 1, 3, 3, 130, 257, 64, 0, 2, device)   # then 390: rows 390.. of the workspace keep the first call's values
    rows = (1 << 21) + 1
    p = ctypes.c_void_p(256)  # never dereferenced: the size check comes first
    assert lib.xg_sdpa_backward_static(p, p, p, p, p, p, p, p, p, 1, 1, 1, rows, 64, 64, *[S3()] * 8, 1.0, 0, 2, None) == -5
