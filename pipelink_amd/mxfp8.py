"""Host-side MXFP8 block quantiser (torch, CPU or GPU tensors).

Same rule as the device quantiser in ``csrc/plk_mok.cpp``: per 32 elements of the last
axis, scale byte = clamp(exponent_field(amax) - 8, 0, 254) and elements are
e4m3(RNE(clamp(v * 2**(127 - byte), -448, 448))).  Used to prepare weights and inputs the
way the reference's harness calls ``ops.mxfp8_quantize``
(campaigns/mok/host/mok_port_host.py:122)."""
from __future__ import annotations

import torch

MX_BLOCK = 32


def scale_pitch(k: int) -> int:
    return ((k // MX_BLOCK) + 15) // 16 * 16


def quantize(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """x [..., K] float -> (codes uint8 [..., K], scales uint8 [..., scale_pitch(K)])."""
    k = x.shape[-1]
    if k % MX_BLOCK:
        raise ValueError("last dimension must be a multiple of 32")
    nb = k // MX_BLOCK
    xf = x.float().reshape(x.shape[:-1] + (nb, MX_BLOCK))
    amax = xf.abs().amax(dim=-1)
    efield = (amax.view(torch.int32) >> 23) & 0xFF
    b = (efield - 8).clamp_(0, 254)
    inv = ((254 - b) << 23).view(torch.float32)
    scaled = (xf * inv.unsqueeze(-1)).clamp_(-448.0, 448.0)
    codes = scaled.to(torch.float8_e4m3fn).view(torch.uint8).reshape(x.shape)
    sc = torch.zeros(x.shape[:-1] + (scale_pitch(k),), dtype=torch.uint8, device=x.device)
    sc[..., :nb] = b.to(torch.uint8)
    return codes, sc


def dequantize(codes: torch.Tensor, sc: torch.Tensor) -> torch.Tensor:
    k = codes.shape[-1]
    nb = k // MX_BLOCK
    vals = codes.view(torch.float8_e4m3fn).float().reshape(codes.shape[:-1] + (nb, MX_BLOCK))
    scale = torch.ldexp(torch.ones((), dtype=torch.float32, device=codes.device), sc[..., :nb].to(torch.int32) - 127)
    return (vals * scale.unsqueeze(-1)).reshape(codes.shape)
