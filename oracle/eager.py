"""TEST INFRASTRUCTURE ONLY -- the numeric oracle of the mi355x hot path.

The reference defines every fused replacement as "equal to the unfused Aten
subgraph it matched" and its own tests compare against the eager function.
These are those eager functions, restated for this build.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package; nothing under xpu_graph_amd/ does.

Every function cites the reference lines whose behaviour it restates.  Each is
pinned in tests/test_oracle.py by checks that do not repeat its formula:
float64 numpy closed forms, torch library routines (F.rms_norm, F.layer_norm,
F.scaled_dot_product_attention), invariants and brute force on tiny inputs.
Parity status: every function below is pinned; none is "parity unpinned".
"""
import math

import torch
import torch.nn.functional as F


# --- C1: RMSNorm ---------------------------------------------------------------
def rmsnorm_eager(x, w, eps=1e-6):
    """BASELINE config 1; the form FusedRMSNorm matches
    (src/xpu_graph/passes/patterns/common/fuse_rmsnorm.py:29-114; test fixture
    tests/common/test_fuse_rmsnorm.py:20-49)."""
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def default_rms_norm(x, weight, eps):
    """Semantic definition of the fused op: DefaultRMSNorm.forward
    (src/xpu_graph/passes/patterns/utils/default_replacements.py:19-25): fp32
    math, one rounding to the input dtype."""
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * weight.float()
    return y.to(x.dtype)


# --- C2: residual add + LayerNorm ------------------------------------------------
def default_layer_norm(x, weight, bias, eps):
    """DefaultLayerNorm.forward (default_replacements.py:28-36)."""
    xf = x.float()
    mean = xf.mean(-1, keepdim=True)
    var = ((xf - mean) ** 2).mean(-1, keepdim=True)
    y = (xf - mean) * torch.rsqrt(var + eps)
    if weight is not None:
        y = y * weight.float()
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype)


def add_layernorm_eager(x, res, gamma, beta, eps=1e-5):
    """BASELINE config 2: returns (normalised, updated residual).  The residual
    sum is rounded to the storage dtype before statistics are taken, exactly as
    the unfused graph does (add.Tensor in bf16, then the norm); shape of the
    reference test: tests/mlu/test_fuse_addlayernorm.py:17-54; replacement
    semantics: passes/patterns/targets/mlu/fuse_add_norm.py:21-83."""
    h = x + res
    y = F.layer_norm(h, (h.shape[-1],), gamma, beta, eps)
    return y, h


def add_layernorm_decomposed_eager(x, res, gamma, beta, eps=1e-5):
    """The decomposed (HF style) spelling that FusedLayerNorm recognises
    (passes/patterns/common/fuse_layernorm.py:32-150;
    tests/common/test_fuse_layernorm.py:20-55)."""
    h = x + res
    hf = h.float()
    mean = hf.mean(-1, keepdim=True)
    var = hf.var(-1, unbiased=False, keepdim=True)
    n = ((hf - mean) * torch.rsqrt(var + eps)).to(h.dtype)
    return n * gamma + beta, h


def add_rmsnorm_eager(x, res, w, eps=1e-6):
    """Residual add + RMSNorm as the NPU test writes it
    (tests/npu/test_add_rmsnorm.py:16-25): the sum is rounded to the storage
    dtype first, the norm runs on fp32 copies of the ROUNDED sum."""
    h = x + res
    hf = h.float()
    y = hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + eps)
    return (y * w.float()).to(h.dtype), h


# --- C3: slice/cat and combo-sum ---------------------------------------------------
def slice_cat_eager(src, slices):
    """torch.cat of column slices (the graph FusedCatSlice matches,
    passes/patterns/structure/fuse_slice_cat.py:30-116); out[r, j] = src[r, idx[j]]
    as in passes/patterns/targets/mlu/triton_kernel/fused_slice_cat.py:10-73."""
    return torch.cat([src[:, s:e] for s, e in slices], dim=1)


def addn_eager(tensors):
    """Left-leaning add chain, the graph FusedAddN matches
    (passes/patterns/common/fuse_addn.py:27-76; tests/common/test_fuse_addn.py:9-71)."""
    acc = tensors[0]
    for t in tensors[1:]:
        acc = acc + t
    return acc


def combo_sum_eager(inputs, dim):
    """N independent 3-D -> 2-D sums (ComboSumModule,
    passes/patterns/targets/mlu/structure_replacements/__init__.py:147-165)."""
    return [t.sum(dim=dim) for t in inputs]


def fused_slice_eager(src, starts, width):
    """The slices FusedSlice gathers (passes/patterns/structure/fuse_slice.py:75-121), stacked as FuseSliceModule
    returns them (targets/mlu/structure_replacements/__init__.py:21-47): [n, *src.shape[:-1], width]."""
    return torch.stack([src[..., s : s + width] for s in starts], dim=0)


def slice_sum_cat_eager(x, slice_param):
    """cat of row-slice sums of one 3-D tensor, the graph FusedCatSum matches
    (passes/patterns/targets/mlu/fuse_sum_cat.py:118-252; tests/mlu/test_slice_sum_cat.py:13-20)."""
    return torch.cat([torch.sum(x[:, a:b, :], dim=[1]) for a, b in slice_param], dim=1)


# --- C4: dense layer ----------------------------------------------------------------
def dense_silu_eager(x, W, b):
    """BASELINE config 4: F.silu(x @ W + b); the graph FusedAddMM + CustomDenseLayer
    match (passes/patterns/common/fuse_addmm.py:12-90,
    passes/patterns/structure/custom_denselayer.py:31-99)."""
    return F.silu(torch.addmm(b, x, W))


def dense_eager(x, W, weight_trans, bias, act):
    """DenseLayerModule.forward semantics
    (passes/patterns/targets/mlu/structure_replacements/dense_layer_modules.py:4-56):
    1-D bias is a bias, 2-D bias is a residual added before the activation."""
    y = x @ (W.t() if weight_trans else W)
    if bias is not None:
        y = y + bias
    if act == "relu":
        y = F.relu(y)
    elif act == "gelu":
        y = F.gelu(y)
    elif act == "silu":
        y = F.silu(y)
    elif act == "sigmoid":
        y = torch.sigmoid(y)
    return y


FP8_MAX = 448.0  # largest finite OCP e4m3fn value


def quantize_fp8_per_tensor(x):
    s = x.abs().max().float() / FP8_MAX
    return (x.float() / s).to(torch.float8_e4m3fn), s.reshape(1)


def quantize_fp8_per_out_channel(W):
    """W is [K, N]; one absmax scale per output channel (column)."""
    s = W.abs().amax(dim=0).float() / FP8_MAX
    return (W.float() / s).to(torch.float8_e4m3fn), s


def dense_fp8_silu_eager(x_q, W_q, s_x, s_w, b):
    """fp8 variant of config 4 (no counterpart in the reference): dequantise,
    fp32 matmul, scales and bias in fp32, SiLU."""
    acc = x_q.float() @ W_q.float()
    return F.silu(acc * s_x.float() * s_w.float() + b.float())


# --- C5: attention / SwiGLU / Llama block --------------------------------------------
def causal_sdpa_eager(q, k, v, scale=None):
    """softmax(q k^T * scale + causal mask) v with fp32 softmax: the HF "eager"
    attention form FusedSDPA rewrites
    (passes/patterns/common/fuse_scaled_dot_product_attention.py:63-242)."""
    D = q.shape[-1]
    scale = (1.0 / math.sqrt(D)) if scale is None else scale
    Sq, Sk = q.shape[-2], k.shape[-2]
    s = torch.matmul(q, k.transpose(-1, -2)) * scale
    mask = torch.full((Sq, Sk), float("-inf"), device=q.device, dtype=torch.float32).triu(1)
    p = torch.softmax(s.float() + mask, dim=-1).to(q.dtype)
    return torch.matmul(p, v)


def sdpa_eager(q, k, v, mask=None, scale=None):
    """softmax(q k^T * scale + mask) v with fp32 softmax and no causal mask: the same attention form
    (passes/patterns/common/fuse_scaled_dot_product_attention.py:63-242) as a decode step meets it -- few query rows,
    an optional additive mask, key/value heads shared by groups of query heads (repeated here)."""
    D = q.shape[-1]
    scale = (1.0 / math.sqrt(D)) if scale is None else scale
    rep = q.shape[1] // k.shape[1]
    if rep > 1:
        k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    s = torch.matmul(q, k.transpose(-1, -2)).float() * scale
    if mask is not None:
        s = s + mask.float()
    return torch.matmul(torch.softmax(s, dim=-1).to(q.dtype), v)


def silu_mul_eager(x):
    """SwiGLU gate as tests/npu/test_silu_mul.py:8-16 writes it."""
    d = x.shape[-1] // 2
    return F.silu(x[..., :d]) * x[..., d:]


def rope_tables(S, D, base=10000.0, device="cpu", dtype=torch.float32):
    inv = 1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float32, device=device) / D))
    t = torch.arange(S, dtype=torch.float32, device=device)
    fr = torch.outer(t, inv)
    emb = torch.cat([fr, fr], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def _rotate_half(x):
    d = x.shape[-1] // 2
    return torch.cat([-x[..., d:], x[..., :d]], dim=-1)


def llama_block_eager(x, p, n_heads=32, eps=1e-6, rope_base=10000.0):
    """BASELINE config 5: a Llama decoder block written in plain eager torch (HF
    style): pre-attention RMSNorm, q/k/v projections, RoPE, causal attention with
    fp32 softmax, output projection, residual, pre-MLP RMSNorm, SwiGLU MLP.
    `p` maps names to weights laid out as nn.Linear stores them ([out, in])."""
    B, S, Hd = x.shape
    D = Hd // n_heads

    def rms(t, w):
        tf = t.float()
        return (w * (tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps)).to(t.dtype))

    h = rms(x, p["ln1"])
    q = F.linear(h, p["wq"]).view(B, S, n_heads, D).transpose(1, 2)
    k = F.linear(h, p["wk"]).view(B, S, n_heads, D).transpose(1, 2)
    v = F.linear(h, p["wv"]).view(B, S, n_heads, D).transpose(1, 2)
    cos, sin = rope_tables(S, D, rope_base, x.device, x.dtype)
    q = q * cos + _rotate_half(q) * sin
    k = k * cos + _rotate_half(k) * sin
    att = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(D)
    mask = torch.full((S, S), float("-inf"), device=x.device, dtype=x.dtype).triu(1)
    att = att + mask
    att = torch.softmax(att, dim=-1, dtype=torch.float32).to(q.dtype)
    o = torch.matmul(att, v).transpose(1, 2).reshape(B, S, Hd)
    x = x + F.linear(o, p["wo"])
    h = rms(x, p["ln2"])
    mlp = F.linear(F.silu(F.linear(h, p["wg"])) * F.linear(h, p["wu"]), p["wd"])
    return x + mlp


def llama_block_decode_eager(x, p, k_cache, v_cache, cos_row, sin_row, n_heads=32, eps=1e-6):
    """llama_block_eager for ONE new token per sequence against cached keys and values (incremental decoding of the same
    block).  x [B, 1, hidden]; k_cache / v_cache [B, H, S, D] hold the rotated keys and the values of every position the
    token attends to, its own included (the caller stores the k_new, v_new of an earlier call there: they do not depend on
    the caches); cos_row / sin_row [D] are the rotary table's row of the token's position.  No mask: every cached position
    is visible.  Returns (out [B, 1, hidden], k_new [B, H, 1, D], v_new [B, H, 1, D])."""
    B, _, Hd = x.shape
    D = Hd // n_heads

    def rms(t, w):
        tf = t.float()
        return (w * (tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps)).to(t.dtype))

    h = rms(x, p["ln1"])
    q = F.linear(h, p["wq"]).view(B, 1, n_heads, D).transpose(1, 2)
    k_new = F.linear(h, p["wk"]).view(B, 1, n_heads, D).transpose(1, 2)
    v_new = F.linear(h, p["wv"]).view(B, 1, n_heads, D).transpose(1, 2)
    q = q * cos_row + _rotate_half(q) * sin_row
    k_new = k_new * cos_row + _rotate_half(k_new) * sin_row
    att = torch.matmul(q, k_cache.transpose(2, 3)) / math.sqrt(D)
    att = torch.softmax(att, dim=-1, dtype=torch.float32).to(q.dtype)
    o = torch.matmul(att, v_cache).transpose(1, 2).reshape(B, 1, Hd)
    x = x + F.linear(o, p["wo"])
    h = rms(x, p["ln2"])
    mlp = F.linear(F.silu(F.linear(h, p["wg"])) * F.linear(h, p["wu"]), p["wd"])
    return x + mlp, k_new, v_new
