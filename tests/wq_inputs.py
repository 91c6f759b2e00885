"""Seeded input builders shared by the CPU and GPU tests (always generated on the CPU, then uploaded:
torch's CPU and device generators give different streams for one seed)."""

import torch


def gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def weights(M: int, N: int, seed: int = 0, std: float = 0.02, outlier_p: float = 1e-3, outlier_x: float = 20.0):
    """bf16 N(0, std) with a fraction outlier_p of entries scaled by outlier_x."""
    g = gen(seed)
    w = torch.randn(M, N, generator=g) * std
    if outlier_p > 0:
        mask = torch.rand(M, N, generator=g) < outlier_p
        w[mask] *= outlier_x
    return w.to(torch.bfloat16)


def zero_blocks(w: torch.Tensor, frac: float, seed: int, bm: int = 128, bn: int = 128):
    """Zeroes a fraction of the (bm x bn) blocks of w (in place) and returns it."""
    g = gen(seed)
    M, N = w.shape
    tm, tn = -(-M // bm), -(-N // bn)
    kill = torch.rand(tm, tn, generator=g) < frac
    for i, j in kill.nonzero().tolist():
        w[i * bm:(i + 1) * bm, j * bn:(j + 1) * bn] = 0
    return w


def subnormal_block(M: int = 128, N: int = 128, seed: int = 0):
    """Every element a bf16 subnormal (bits 0x0001..0x007F, either sign)."""
    g = gen(seed)
    bits = torch.randint(1, 0x80, (M, N), generator=g, dtype=torch.int32)
    sign = torch.randint(0, 2, (M, N), generator=g, dtype=torch.int32) << 15
    return (bits | sign).to(torch.int16).view(torch.bfloat16)


def near_max_block(M: int = 128, N: int = 128, seed: int = 0, amax: float = 0.171875):
    """Values clustered at +-amax*(1 +- 2^-8 k): they land on and around the 448 end of the e4m3 range."""
    g = gen(seed)
    k = torch.randint(-3, 1, (M, N), generator=g).float()
    sign = torch.randint(0, 2, (M, N), generator=g).float() * 2 - 1
    w = (sign * amax * (1 + k * 2.0 ** -8)).to(torch.bfloat16)
    w[0, 0] = amax
    return w


def all_bf16_values():
    """All 65536 bf16 bit patterns as a [256, 256] tensor (includes NaNs and infinities)."""
    return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).view(256, 256)


def finite_bf16_values():
    b = torch.arange(65536, dtype=torch.int32)
    b = b[(b & 0x7FFF) < 0x7F80]
    return b.to(torch.int16).view(torch.bfloat16)


def fp8_codes(M: int, N: int, seed: int = 0):
    """uint8 codes uniform over the 254 finite e4m3fn codes."""
    g = gen(seed)
    c = torch.randint(0, 254, (M, N), generator=g, dtype=torch.int32)
    c = c + (c >= 0x7F).int()          # skip 0x7F
    c = torch.where(c >= 0xFF, torch.full_like(c, 0xFE), c)
    assert int(((c == 0x7F) | (c == 0xFF)).sum()) == 0
    return c.to(torch.uint8)


def log_uniform_scales(tm: int, tn: int, seed: int = 0, lo: float = 1e-4, hi: float = 1e-1):
    g = gen(seed)
    u = torch.rand(tm, tn, generator=g, dtype=torch.float64)
    import math
    return torch.exp(u * (math.log(hi) - math.log(lo)) + math.log(lo)).to(torch.float32)


def same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Bit equality of two tensors of one dtype and shape."""
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    view = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[a.element_size()]
    return bool(torch.equal(a.contiguous().view(view), b.contiguous().view(view)))
