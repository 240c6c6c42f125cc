"""Norm-after-sum with an fp32 residual stream and one gain for all coordinates, and the xIELU activation.

GPU: ``csrc/hip/post_norm.hip``. CPU: PyTorch formulations of the same arithmetic (fp32).
"""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib as L


def scaled_add_norm(x: torch.Tensor, y: Optional[torch.Tensor], gain: torch.Tensor, alpha: float, eps: float,
                    dtype: torch.dtype, inplace: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """z = alpha * x + y;  x' = z / sqrt(mean(z^2) + eps) * gain  (gain: a tensor holding ONE number).

    x: fp32 residual stream [T, W] (replaced in place unless `inplace` is False); y: sublayer output [T, W] in
    `dtype` or None. Returns (x' in fp32, x' in `dtype`): the stream and the operand of the next projection (the same
    tensor when `dtype` is fp32)."""
    assert x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
    T, W = x.shape
    out32 = x if inplace else torch.empty_like(x)
    if L.use_hip(x):
        assert y is None or (y.dtype == dtype and y.is_contiguous() and y.shape == x.shape)
        assert gain.dtype == dtype and gain.numel() == 1
        outc = out32 if dtype == torch.float32 else torch.empty(T, W, dtype=dtype, device=x.device)
        L.check(L.lib().areal_scaled_add_norm(
            L.ptr(x), L.ptr(y), L.ptr(gain), L.ptr(out32), L.ptr(outc) if outc is not out32 else None, L.c_int(T),
            L.c_int(W), L.c_float(alpha), L.c_float(eps), L.c_int(L.dtype_flag(gain)), L.stream_ptr()),
            "scaled_add_norm")
        return out32, outc
    z = alpha * x if y is None else alpha * x + y.float()
    z = z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps) * gain.float().reshape(())
    if inplace:
        x.copy_(z)
        z = x
    return z, (z if dtype == torch.float32 else z.to(dtype))


def xielu(z: torch.Tensor, act: torch.Tensor) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2  with (p, q) = act."""
    if L.use_hip(z):
        assert z.is_contiguous() and act.dtype == z.dtype and act.numel() == 2
        out = torch.empty_like(z)
        L.check(L.lib().areal_xielu(L.ptr(z), L.ptr(act), L.ptr(out), L.c_int64(z.numel()),
                                    L.c_int(L.dtype_flag(z)), L.stream_ptr()), "xielu")
        return out
    zf = z.float()
    ap, an = F.softplus(act.float()[0]), 0.5 + F.softplus(act.float()[1])
    return torch.where(zf > 0, ap * zf * zf + 0.5 * zf, an * (torch.expm1(zf.clamp(max=0)) - zf) + 0.5 * zf).to(z.dtype)
