"""Seeded synthetic operands, generated on the device.

The reference fills its test and benchmark buffers with ``rand()`` under a fixed seed
(common.cuh:86-158).  Here element *i* of stream (seed, stream_id) is a pure function of
(seed, stream_id, i) - a splitmix64 finaliser over a counter, Box-Muller for normals - so a
buffer of any size can be produced in pieces, on any device, and always holds the same values.
The arithmetic is integer except for the Box-Muller step, whose ``log`` / ``cos`` may differ from
another maths library's in the last bit of the double; after rounding to fp32 that shows in about
one element per million.
"""
import torch

_MASK64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_M1, _M2 = 0xBF58476D1CE4E5B9, 0x94D049BB133111EB


def _s64(v):
    """Python integer (mod 2^64) -> the int64 with the same bits."""
    v &= _MASK64
    return v - (1 << 64) if v >= (1 << 63) else v


def _mix_int(z):
    z &= _MASK64
    z = ((z ^ (z >> 30)) * _M1) & _MASK64
    z = ((z ^ (z >> 27)) * _M2) & _MASK64
    return z ^ (z >> 31)


def _lsr(z, s):
    """Logical right shift of int64 tensors holding uint64 bit patterns."""
    return (z >> s) & ((1 << (64 - s)) - 1)


def _mix(z):
    z = (z ^ _lsr(z, 30)) * _s64(_M1)
    z = (z ^ _lsr(z, 27)) * _s64(_M2)
    return z ^ _lsr(z, 31)


def rng_u64(seed, stream_id, index):
    """uint64 bit patterns (as int64) of elements `index` (an int64 tensor) of stream (seed, stream_id)."""
    key = _mix_int(seed + _GOLDEN) ^ _mix_int(stream_id * 0xD1B54A32D192ED03 + 0x2545F4914F6CDD1D)
    return _mix((index + 1) * _s64(_GOLDEN) + _s64(key))


def normal_f32(shape, seed, stream_id, device="cuda", chunk=1 << 24):
    """N(0,1) as fp32, element i = Box-Muller of counters 2i and 2i + 1 (53-bit uniforms, the first in (0, 1])."""
    n = 1
    for d in shape:
        n *= d
    out = torch.empty(n, dtype=torch.float32, device=device)
    for lo in range(0, n, chunk):
        i = torch.arange(lo, min(lo + chunk, n), dtype=torch.int64, device=device)
        u1 = (_lsr(rng_u64(seed, stream_id, 2 * i), 11) + 1).double() * 2.0 ** -53
        u2 = _lsr(rng_u64(seed, stream_id, 2 * i + 1), 11).double() * 2.0 ** -53
        out[lo:lo + i.numel()] = (torch.sqrt(-2.0 * torch.log(u1)) * torch.cos(6.283185307179586476925286766559 * u2)).float()
    return out.reshape(shape)


def quantize_tensor(x):
    """Per-tensor scale absmax / 448 (1 for an all-zero tensor) and the OCP E4M3 codes of x / scale, round to
    nearest even.  Returns (uint8 codes, fp32 scalar tensor)."""
    amax = x.abs().max()
    scale = torch.where(amax == 0, torch.ones_like(amax), amax / 448.0)
    return (x / scale).to(torch.float8_e4m3fn).view(torch.uint8), scale


def gemm_operands(m, n, k, seed=0, device="cuda"):
    """The seeded GEMM recipe of the benchmark configurations: A = N(0,1) from stream 1, B = N(0,1) from stream 2,
    each quantised per tensor.  Returns (a8 [m, k], b8 [n, k], scale = sA * sB as a one-element fp32 tensor)."""
    a8, sa = quantize_tensor(normal_f32((m, k), seed, 1, device))
    b8, sb = quantize_tensor(normal_f32((n, k), seed, 2, device))
    return a8, b8, (sa * sb).reshape(1).float().contiguous()
