"""TEST INFRASTRUCTURE ONLY -- seeded synthetic inputs of the five benchmark
configurations.  Values are generated on the CPU (so they do not depend on the
device RNG) and moved to the requested device afterwards.
"""
import json
import os

import torch

_GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "tests", "golden")


def _gen(seed):
    return torch.Generator(device="cpu").manual_seed(seed)


def c1_rmsnorm(rows=2048, cols=4096, device="cpu", seed=0):
    g = _gen(seed)
    x = torch.randn(rows, cols, generator=g)
    w = 1.0 + 0.1 * torch.randn(cols, generator=g)
    return x.to(device), w.to(device)


def c2_add_layernorm(rows=8192, cols=4096, device="cpu", seed=0, dtype=torch.bfloat16):
    g = _gen(seed)
    x = torch.randn(rows, cols, generator=g).to(dtype)
    res = torch.randn(rows, cols, generator=g).to(dtype)
    gamma = (1.0 + 0.1 * torch.randn(cols, generator=g)).to(dtype)
    beta = (0.1 * torch.randn(cols, generator=g)).to(dtype)
    return x.to(device), res.to(device), gamma.to(device), beta.to(device)


def make_slice_offsets(n_slices=64, width=32, src_cols=8192, seed=0):
    """n_slices non-overlapping `width`-wide column blocks at arbitrary (not
    width-aligned) starts, in shuffled order."""
    g = _gen(seed)
    slack = src_cols - n_slices * width
    draws = torch.sort(torch.randint(0, slack + 1, (n_slices,), generator=g)).values
    starts = draws + width * torch.arange(n_slices)
    order = torch.randperm(n_slices, generator=g)
    return [int(s) for s in starts[order]]


def c3_slice_offsets():
    """The committed 64-offset table of config 3 (tests/golden/c3_slice_offsets.json)."""
    with open(os.path.join(_GOLDEN, "c3_slice_offsets.json")) as f:
        return json.load(f)["starts"]


def c3_slice_cat(rows=4096, src_cols=8192, device="cpu", seed=0, starts=None, width=32):
    g = _gen(seed)
    src = torch.randn(rows, src_cols, generator=g)
    starts = c3_slice_offsets() if starts is None else starts
    slices = [(s, s + width) for s in starts]
    return src.to(device), slices


def c3_addn(n=32, rows=4096, cols=256, device="cpu", seed=0, dtype=torch.float32):
    g = _gen(seed)
    return [torch.randn(rows, cols, generator=g).to(dtype).to(device) for _ in range(n)]


def c4_dense(M=8192, K=4096, N=11008, device="cpu", seed=0, dtype=torch.bfloat16):
    g = _gen(seed)
    x = torch.randn(M, K, generator=g).to(dtype)
    W = (0.02 * torch.randn(K, N, generator=g)).to(dtype)
    b = (0.02 * torch.randn(N, generator=g)).to(dtype)
    return x.to(device), W.to(device), b.to(device)


def c5_llama_block(B=4, S=2048, hidden=4096, inter=11008, device="cpu", seed=0, dtype=torch.bfloat16):
    g = _gen(seed)

    def w(o, i):
        return (0.02 * torch.randn(o, i, generator=g)).to(dtype).to(device)

    p = {
        "wq": w(hidden, hidden),
        "wk": w(hidden, hidden),
        "wv": w(hidden, hidden),
        "wo": w(hidden, hidden),
        "wg": w(inter, hidden),
        "wu": w(inter, hidden),
        "wd": w(hidden, inter),
        "ln1": torch.ones(hidden, dtype=dtype, device=device),
        "ln2": torch.ones(hidden, dtype=dtype, device=device),
    }
    x = torch.randn(B, S, hidden, generator=g).to(dtype).to(device)
    return x, p
