"""Small numeric helpers of the public API (same names and results as the reference's
deep_ep/utils/math.py)."""
from typing import Tuple

import torch

FP8_E4M3_MAX = 448.0
SF_GROUP = 128


def ceil_div(x: int, y: int) -> int:
    return -(-x // y)


def align(x: int, y: int) -> int:
    return ceil_div(x, y) * y


def safe_div(a, b) -> float:
    if b == 0:
        if a == 0:
            return 0
        raise ZeroDivisionError
    return a / b


def calc_diff(x: torch.Tensor, y: torch.Tensor) -> float:
    """1 - cosine-like similarity of (x+1, y+1) in fp64."""
    xd, yd = x.double() + 1, y.double() + 1
    return (1 - 2 * (xd * yd).sum() / (xd * xd + yd * yd).sum()).item()


def count_bytes(*tensors) -> int:
    n = 0
    for t in tensors:
        if t is None:
            continue
        n += count_bytes(*t) if isinstance(t, (tuple, list)) else t.numel() * t.element_size()
    return n


def per_token_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Caller-side quantiser (reference: deep_ep/utils/math.py:30-38): per token and per group of
    128 channels, scale = max(|x|, 1e-4) / 448 in fp32 and payload = e4m3fn(x * (448 / amax)).

    A contiguous bfloat16 tensor on the GPU (hidden a multiple of 8) is quantised by the library's own
    kernel: its bytes are those `EPBuffer.dispatch(..., fused_fp8_quant=True)` writes into the slots and
    those the formula below gives on CPU tensors.  Anything else goes through the torch formula on the
    tensor's own device; on the GPU torch evaluates `448 / amax` and `amax / 448` with a different rounding
    than on the CPU, so bytes of such inputs can differ in the last bit from the CPU's and the library's."""
    assert x.dim() == 2
    rows, cols = x.shape
    if x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous() and cols % 8 == 0 and 0 < cols <= 16384:
        from .. import _C
        return _C.per_token_cast_to_fp8(x)
    padded = align(cols, SF_GROUP)
    groups = torch.nn.functional.pad(x, (0, padded - cols)).view(rows, padded // SF_GROUP, SF_GROUP)
    amax = groups.abs().float().amax(dim=2).clamp(1e-4)
    payload = (groups * (FP8_E4M3_MAX / amax.unsqueeze(2))).to(torch.float8_e4m3fn)
    return payload.view(rows, padded)[:, :cols].contiguous(), amax / FP8_E4M3_MAX


def per_token_cast_back(x_fp8: torch.Tensor, x_scales: torch.Tensor) -> torch.Tensor:
    """Inverse of `per_token_cast_to_fp8` up to rounding; int32 scales are read as UE8M0 exponents."""
    if x_fp8.numel() == 0:
        return x_fp8.to(torch.bfloat16)
    assert x_fp8.dim() == 2
    rows, cols = x_fp8.shape
    padded = align(cols, SF_GROUP)
    if x_scales.dtype == torch.int:
        x_scales = (x_scales.view(torch.uint8).to(torch.int) << 23).view(torch.float)
    wide = torch.nn.functional.pad(x_fp8, (0, padded - cols)).to(torch.float32).view(rows, -1, SF_GROUP)
    out = wide * x_scales.view(rows, -1, 1)
    return out.view(rows, padded).to(torch.bfloat16)[:, :cols].contiguous()
