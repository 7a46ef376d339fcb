"""bf16 helpers shared by the oracle (torch CPU; round-to-nearest-even like the hardware)."""
import numpy as np
import torch

BF16_MIN = torch.finfo(torch.bfloat16).min


def rb(x: torch.Tensor) -> torch.Tensor:
    """fp32 value of the bf16 rounding of x."""
    return x.to(torch.bfloat16).to(torch.float32)


def bf16_bits(x: torch.Tensor) -> np.ndarray:
    """uint16 bit patterns of a bf16 tensor."""
    return x.contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_ulp(x: torch.Tensor) -> torch.Tensor:
    """spacing of bf16 numbers at |x| (fp32 tensor in, fp32 out)."""
    a = x.abs().to(torch.float32).clamp_min(2.0 ** -126)
    e = torch.floor(torch.log2(a))
    return torch.exp2(e - 7)


def ulp16(x: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """spacing of the numbers of a 16-bit float type at |x|: bfloat16 (8 significant bits) or float16
    (11 significant bits, subnormal below 2^-14)."""
    if dtype == torch.bfloat16:
        return bf16_ulp(x)
    a = x.abs().to(torch.float32).clamp_min(2.0 ** -14)
    e = torch.floor(torch.log2(a))
    return torch.exp2(e - 10)
