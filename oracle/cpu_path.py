"""The reference CPU path used as the timed CPU baseline: torch dequantise +
matmul on the host cores.  TEST / BENCH INFRASTRUCTURE ONLY (see oracle/__init__.py).

Same arithmetic as oracle.ops.dequant_matmul (fp32 dequantise-then-matmul,
one rounding to fp16), written with torch so that the matmul runs on torch's
multi-threaded CPU BLAS, as the benchmark definition asks ("torch dequant +
matmul")."""
import torch


def dequant_matmul(x, q, scale):
    """x [M, K] fp16, q [K, N] int8 (unprocessed), scale [N] fp16 -> [M, N] fp16.
    Dequantisation is part of the timed work."""
    wd = q.to(torch.float32) * scale.to(torch.float32)
    return (x.to(torch.float32) @ wd).to(torch.float16)


def dequant_matmul_layer(layer):
    return [dequant_matmul(x, q, s) for (x, q, s) in layer]
