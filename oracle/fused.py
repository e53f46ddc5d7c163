"""Oracle: per-head q/k RMSNorm + rotary embedding (+ what lands in the KV cache), and the two
element-wise steps between a decoder layer's GEMMs (residual add + RMSNorm, SiLU-and-multiply).
Test infrastructure only.

Reference followed, including where it rounds to the storage type:
  engines/nano_dvlm/nanovllm/layers/layernorm.py:16-26   x.float() * rsqrt(mean(x^2) + eps) -> bf16, then * weight (bf16)
  engines/nano_dvlm/nanovllm/layers/rotary_embedding.py:6-14  fp32 rotation of (x[:d/2], x[d/2:]), one rounding
  engines/nano_dvlm/nanovllm/models/sdar.py:73-83        split of the fused projection, norm, rope
  engines/nano_dvlm/nanovllm/layers/layernorm.py:28-41   (x.float() + residual.float()) -> new residual (rounded),
                                                         mean of squares of the UNROUNDED sum, then as :16-26
  engines/nano_dvlm/nanovllm/layers/activation.py:7-16   SiluAndMul = liger-kernel 0.6.4 SwiGLU forward (third party,
                                                         not under the reference tree): silu(a) in fp32, cast to the
                                                         storage type, times b in the storage type
"""
from __future__ import annotations

import torch


def rms_norm_ref(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return xf.to(x.dtype) * w.to(x.dtype)


def rope_ref(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    x1, x2 = torch.chunk(x.float(), 2, dim=-1)
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).to(x.dtype)


def qk_norm_rope(qkv: torch.Tensor, q_w, k_w, eps, cos_table, sin_table, positions, hq, hkv, d):
    """qkv [N, (hq+2hkv)*d] -> (q [N,hq,d], k [N,hkv,d], v [N,hkv,d]) on the CPU."""
    qkv = qkv.cpu()
    N = qkv.shape[0]
    q, k, v = qkv.split([hq * d, hkv * d, hkv * d], dim=-1)
    cos = cos_table.cpu()[positions.cpu()].unsqueeze(1)
    sin = sin_table.cpu()[positions.cpu()].unsqueeze(1)
    q = rope_ref(rms_norm_ref(q.reshape(N, hq, d), q_w.cpu(), eps), cos, sin)
    k = rope_ref(rms_norm_ref(k.reshape(N, hkv, d), k_w.cpu(), eps), cos, sin)
    return q, k, v.reshape(N, hkv, d)


def add_rms_norm(x: torch.Tensor, residual: torch.Tensor | None, w: torch.Tensor, eps: float):
    """layernorm.py:43-51: (normed, new_residual); with residual None, (normed, None)."""
    x = x.cpu()
    if residual is None:
        return rms_norm_ref(x, w.cpu(), eps), None
    s = x.float() + residual.cpu().float()
    new_residual = s.to(x.dtype)
    y = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps)
    return y.to(x.dtype) * w.cpu().to(x.dtype), new_residual


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """activation.py:13-16: x [..., 2I] -> silu(x[..., :I]) * x[..., I:]."""
    a, b = x.cpu().chunk(2, -1)
    af = a.float()
    return (af * torch.sigmoid(af)).to(x.dtype) * b
