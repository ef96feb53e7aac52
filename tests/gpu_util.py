"""Helpers shared by the GPU parity tests: seeded inputs that the GPU path and the
CPU checker see bit-for-bit, and conversions between torch tensors and the
checker's uint16 bit patterns."""
import numpy as np
import torch

F16, BF16 = 0, 1
TORCH_DTYPE = {F16: torch.float16, BF16: torch.bfloat16}


def bits_of(t):
    """16-bit float tensor (any device) -> numpy uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(bits, dtype, device="cuda"):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(TORCH_DTYPE[dtype]).to(device)


def seeded(shape, dtype, seed, scale=1.0, dist="normal"):
    """CPU-generated fp32 -> 16-bit; returns (gpu tensor, bits)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g) if dist == "normal" else torch.rand(*shape, generator=g) * 2 - 1
    x16 = (x * scale).to(TORCH_DTYPE[dtype])
    return x16.cuda(), bits_of(x16)


def ulp_diff_ok(got_bits, ref_bits, dtype, max_ulp=1, frac=1.0):
    """Fraction of elements within max_ulp units in the last place (same-sign
    finite values compare by integer distance of their bit patterns)."""
    a = got_bits.astype(np.int32)
    b = ref_bits.astype(np.int32)
    a = np.where(a & 0x8000, 0x8000 - a, a)   # sign-magnitude -> monotone integers
    b = np.where(b & 0x8000, 0x8000 - b, b)
    d = np.abs(a - b)
    return (d <= max_ulp).mean() >= frac and d.max() <= max(max_ulp, 1) * (1 if frac == 1.0 else 4)


def max_rel_err(got, ref):
    """max |got-ref| / max(|ref|, floor): the north-star tolerance metric (<= 1e-2)."""
    got, ref = got.double(), ref.double()
    floor = ref.abs().mean().clamp_min(1e-6)   # elements near zero are measured against the typical magnitude
    return ((got - ref).abs() / ref.abs().clamp_min(floor)).max().item()
