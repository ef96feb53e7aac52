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


def _f32(bits, dtype):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    if dtype == F16:
        return bits.view(np.float16).astype(np.float32)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def ulp_diff_ok(got_bits, ref_bits, dtype, max_ulp=1, frac=1.0):
    """Both sides accumulate in fp32 and round once, so they may differ by the
    16-bit rounding of slightly different fp32 sums: |got - ref| <= max_ulp units in
    the last place of ref, plus an absolute term (1e-3 of the mean magnitude) for
    results that cancel to near zero.  `frac` of the elements must satisfy the
    bound with max_ulp; all of them with 4 * max_ulp."""
    got, ref = _f32(got_bits, dtype).astype(np.float64), _f32(ref_bits, dtype).astype(np.float64)
    eps = 2.0 ** (-10 if dtype == F16 else -7)
    atol = 1e-3 * np.abs(ref).mean()
    d = np.abs(got - ref)
    bound = max_ulp * eps * np.abs(ref) + atol
    return bool((d <= bound).mean() >= frac and (d <= 4 * bound).all())


def max_rel_err(got, ref):
    """max |got-ref| / max(|ref|, floor): the north-star tolerance metric (<= 1e-2)."""
    got, ref = got.double(), ref.double()
    floor = ref.abs().mean().clamp_min(1e-6)   # elements near zero are measured against the typical magnitude
    return ((got - ref).abs() / ref.abs().clamp_min(floor)).max().item()


def rmsnorm_f64(x16, w16, eps):
    """RMSNorm of the 16-bit inputs in float64 with no intermediate rounding: the
    reference the 1e-2 relative tolerance is measured against (a correctly
    double-rounded 16-bit result is within 2 * 2^-8 of it even in bf16)."""
    x = x16.detach().cpu().double()
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w16.detach().cpu().double()
