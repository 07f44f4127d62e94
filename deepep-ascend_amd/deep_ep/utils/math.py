"""Numeric helpers with the names of the reference's deep_ep/utils/math.py.  The FP8 cast runs the
HIP kernel (bit-exact with the reference's eager torch recipe, math.py:30-39)."""
import ctypes
from typing import Tuple

import torch

from .. import _abi


def ceil_div(x: int, y: int) -> int:
    return -(-x // y)


def align(x: int, y: int) -> int:
    return -(-x // y) * y


def calc_diff(x: torch.Tensor, y: torch.Tensor) -> float:
    """The reference's distance between two tensors (math.py:5-9): 1 - 2<a, b> / (<a, a> + <b, b>) with a = x + 1,
    b = y + 1 in fp64."""
    a = x.to(torch.float64) + 1.0
    b = y.to(torch.float64) + 1.0
    return float(1.0 - 2.0 * torch.sum(a * b) / (torch.sum(a * a) + torch.sum(b * b)))


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
    """(e4m3fn [m, n], scales [m, ceil(n/128)] fp32, or UE8M0 exponent bytes packed four to an int32) -> BF16 [m, n]:
    every group of 128 channels times its scale (math.py:42-56)."""
    m, n = x_fp8.shape
    if m * n == 0:
        return x_fp8.to(torch.bfloat16)
    if x_scales.dtype == torch.int32:                      # exponent byte -> fp32 power of two
        exponents = x_scales.contiguous().view(torch.uint8).to(torch.int32)
        x_scales = (exponents << 23).view(torch.float32)
    groups = ceil_div(n, 128)
    values = torch.zeros((m, groups * 128), dtype=torch.float32, device=x_fp8.device)
    values[:, :n] = x_fp8.to(torch.float32)
    values = values.view(m, groups, 128) * x_scales.reshape(m, groups, 1).to(torch.float32)
    return values.view(m, groups * 128)[:, :n].to(torch.bfloat16).contiguous()


def hash_tensor(t: torch.Tensor) -> int:
    """Order-independent checksum of the raw 32-bit words."""
    return int(t.contiguous().view(torch.int32).sum())


def count_bytes(*tensors) -> int:
    """Bytes held by tensors, tuples / lists of tensors and Nones, recursively."""
    return sum(count_bytes(*t) if isinstance(t, (tuple, list)) else t.numel() * t.element_size()
               for t in tensors if t is not None)
