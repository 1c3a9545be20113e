"""CPU oracle of the three-package GEMM example: C = GELU(A . B + bias).  TEST INFRASTRUCTURE ONLY.

The case the reference's plumbing example is evaluated on: A and B 512 x 512 bf16 drawn from
N(0,1) * 0.05, bias 512 from N(0,1) * 0.1, seed 0, math in fp32 on the CPU.  The package split
follows examples/hopper-gemm-split (loader / MMA / epilogue, src/channels.cuh:33-71), whose
epilogue is bias + ReLU; GELU (erf form, torch's default) is this build's variant.

Pins: ``gemm_bias_gelu`` (numpy, float64 erf from the math library) against
``gemm_bias_gelu_torch`` (library matmul + ``torch.nn.functional.gelu``); GELU closed forms
(GELU(0) = 0, GELU(x) - GELU(-x) = x, GELU(x) -> x for large x, -> 0 for very negative x);
``erf_as`` -- the rational approximation the device epilogue uses -- against ``math.erf`` to
its published 1.5e-7 bound.
"""
from __future__ import annotations

import math

import numpy as np
import torch

_erf = np.vectorize(math.erf, otypes=[np.float64])


def inputs(m: int = 512, n: int = 512, k: int = 512, seed: int = 0):
    """(A [m,k] bf16, B [k,n] bf16, bias [n] fp32) as torch tensors; draw order A, B, bias."""
    g = torch.Generator().manual_seed(seed)
    a = (torch.randn(m, k, generator=g) * 0.05).to(torch.bfloat16)
    b = (torch.randn(k, n, generator=g) * 0.05).to(torch.bfloat16)
    bias = torch.randn(n, generator=g) * 0.1
    return a, b, bias


def gelu(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=np.float64)
    return 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))


def erf_as(x: np.ndarray) -> np.ndarray:
    """Abramowitz & Stegun 7.1.26 in fp32, as the device epilogue evaluates it."""
    x = np.asarray(x, dtype=np.float32)
    ax = np.abs(x)
    t = (np.float32(1.0) / (np.float32(1.0) + np.float32(0.3275911) * ax)).astype(np.float32)
    poly = t * (np.float32(0.254829592) + t * (np.float32(-0.284496736) + t * (np.float32(1.421413741)
                + t * (np.float32(-1.453152027) + t * np.float32(1.061405429)))))
    y = np.float32(1.0) - poly * np.exp(-(ax * ax), dtype=np.float32)
    return np.where(x < 0, -y, y).astype(np.float32)


def gemm_bias_gelu(a: np.ndarray, b: np.ndarray, bias: np.ndarray) -> np.ndarray:
    """fp32 result before the bf16 rounding of the store; a [m,k], b [k,n], bias [n] (float arrays)."""
    acc = a.astype(np.float32) @ b.astype(np.float32) + bias.astype(np.float32)[None, :]
    return gelu(acc).astype(np.float32)


def gemm_bias_gelu_torch(a: torch.Tensor, b: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """The same with library routines: fp32 matmul and torch's erf GELU; returns bf16."""
    return torch.nn.functional.gelu(a.float() @ b.float() + bias.float()).to(torch.bfloat16)


def bf16_ulp_distance(x: np.ndarray, y: np.ndarray, floor: float = 2.0 ** -126) -> np.ndarray:
    """|x - y| in units of the bf16 spacing at max(|x|, |y|, floor) (inputs are bf16 values held in
    fp32).  `floor` keeps results that cancel to almost nothing -- where the fp32 summation order
    alone moves the value by many of its own tiny steps -- from being measured in those steps."""
    mag = np.maximum(np.abs(x), np.abs(y)).astype(np.float32)
    expo = np.floor(np.log2(np.maximum(mag, np.float32(floor))))
    return np.abs(x.astype(np.float64) - y.astype(np.float64)) / np.exp2(expo - 7)


# ---- one epilogue, many producers: C = (A . B) * scale[col] + bias[col] -----------------------------------
# (examples/one-epilogue-many-producers/consumer/epilogue.cu:62-69 in the reference computes
# acc * scale + bias with a per-row scale and a ReLU; the case evaluated here is the per-column scale
# without an activation.)  Pins: against the library matmul on a small case; linearity in scale and bias.

def scale_bias_inputs(m: int, n: int, k: int, seed: int = 0):
    """(A [m,k] bf16, B [k,n] bf16, scale [n], bias [n]); A and B from N(0,1) * 0.02; draw order A, B, scale, bias."""
    g = torch.Generator().manual_seed(seed)
    a = (torch.randn(m, k, generator=g) * 0.02).to(torch.bfloat16)
    b = (torch.randn(k, n, generator=g) * 0.02).to(torch.bfloat16)
    scale = 1.0 + torch.randn(n, generator=g) * 0.1
    bias = torch.randn(n, generator=g) * 0.1
    return a, b, scale, bias


def gemm_scale_bias_torch(a: torch.Tensor, b: torch.Tensor, scale: torch.Tensor, bias: torch.Tensor,
                          rows: torch.Tensor | None = None) -> torch.Tensor:
    """fp32 matmul, then * scale + bias per column, rounded to bf16; `rows` restricts it to a sample of rows."""
    a = a if rows is None else a[rows]
    return ((a.float() @ b.float()) * scale.float() + bias.float()).to(torch.bfloat16)
