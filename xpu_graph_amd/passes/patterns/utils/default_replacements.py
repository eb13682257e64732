"""Device-independent replacement modules the common patterns emit.  They define
the semantics every target module must reproduce: fp32 math, one rounding to
the input dtype (reference utils/default_replacements.py:19-55)."""
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F


class DefaultRMSNorm(nn.Module):
    def forward(self, x, weight, eps):
        w = None if weight is None else weight.float()
        return F.rms_norm(x.float(), x.shape[-1:], weight=w, eps=eps).to(x.dtype)


class DefaultLayerNorm(nn.Module):
    def forward(self, x, weight, bias, eps):
        w = None if weight is None else weight.float()
        b = None if bias is None else bias.float()
        return F.layer_norm(x.float(), x.shape[-1:], weight=w, bias=b, eps=eps).to(x.dtype)


@torch.library.custom_op("xpu_graph::sdpa_wrapped_scale", mutates_args=())
def sdpa_wrapped_scale(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attn_mask: Optional[torch.Tensor], scale: torch.Tensor) -> torch.Tensor:
    """SDPA whose scale arrives as a one-element tensor; reading it costs a device sync."""
    return F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, scale=scale.item())


@sdpa_wrapped_scale.register_fake
def _(q, k, v, attn_mask, scale):
    return F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, scale=1.0)


class SDPAWrappedScale(nn.Module):
    def forward(self, q, k, v, attn_mask, scale):
        return torch.ops.xpu_graph.sdpa_wrapped_scale(q, k, v, attn_mask, scale)
