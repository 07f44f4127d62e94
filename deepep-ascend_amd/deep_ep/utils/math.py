"""Numeric helpers with the names of the reference's deep_ep/utils/math.py.  The FP8 cast runs the
HIP kernel (bit-exact with the reference's eager torch recipe, math.py:30-39)."""
import ctypes
from typing import Tuple

import torch

from .. import _abi


def ceil_div(x: int, y: int) -> int:
    return (x + y - 1) // y


def align(x: int, y: int) -> int:
    return ceil_div(x, y) * y


def calc_diff(x: torch.Tensor, y: torch.Tensor) -> float:
    """1 - cosine-like similarity of (x+1, y+1) in fp64 (math.py:5-9)."""
    x, y = x.double() + 1, y.double() + 1
    denominator = (x * x + y * y).sum()
    return (1 - 2 * (x * y).sum() / denominator).item()


def per_token_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """BF16 [m, n] on device -> (e4m3fn [m, n], fp32 scales [m, ceil(n/128)]); per 128 channels
    amax clamped at 1e-4, payload x * (448 / amax), scale amax / 448."""
    assert x.dim() == 2 and x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous()
    m, n = x.shape
    out = torch.empty((m, n), dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty((m, ceil_div(n, 128)), dtype=torch.float32, device=x.device)
    args = _abi.CastArgs()
    args.x, args.out, args.scales = _abi.ptr(x), _abi.ptr(out), _abi.ptr(scales)
    args.num_tokens, args.hidden = m, n
    _abi.check(_abi.lib.deep_ep_hip_launch_cast_fp8(ctypes.byref(args), torch.cuda.current_stream().cuda_stream),
               "per_token_cast_to_fp8")
    return out, scales


def per_token_cast_back(x_fp8: torch.Tensor, x_scales: torch.Tensor) -> torch.Tensor:
    """(e4m3fn [m, n], scales [m, ceil(n/128)] fp32 or packed UE8M0 int32) -> BF16 [m, n] (math.py:42-56)."""
    if x_fp8.numel() == 0:
        return x_fp8.to(torch.bfloat16)
    m, n = x_fp8.shape
    aligned_n = align(n, 128)
    padded = torch.nn.functional.pad(x_fp8.to(torch.float32), (0, aligned_n - n))
    if x_scales.dtype == torch.int:
        x_scales = (x_scales.view(dtype=torch.uint8).to(torch.int) << 23).view(dtype=torch.float)
    out = padded.view(m, -1, 128) * x_scales.reshape(m, -1, 1)
    return out.view(m, aligned_n).to(torch.bfloat16)[:, :n].contiguous()


def hash_tensor(t: torch.Tensor) -> int:
    return t.view(torch.int).sum().item()


def count_bytes(*tensors) -> int:
    total = 0
    for t in tensors:
        if isinstance(t, (tuple, list)):
            total += count_bytes(*t)
        elif t is not None:
            total += t.numel() * t.element_size()
    return total
