"""Oracle for fp8-e4m3 K/V quantisation (test infrastructure only).

The reference has no fp8 path: it asserts ``kv_scale == 1.0``
(additional_designs/attention/backends/aptserve_flash_attn.py:311-312) and
only stores ``_kv_scale = 1.0`` (additional_designs/attention/aptserve_layer.py:49-55).
The format is therefore defined here, from the OCP 8-bit floating point
specification's E4M3 ("fn": finite, one NaN code per sign, no infinities):

    bits  s eeee mmm, bias 7
    e == 0        -> (-1)^s * 2^-6 * (m / 8)              subnormal
    0 < e         -> (-1)^s * 2^(e-7) * (1 + m / 8)       normal
    e == 15, m==7 -> NaN;  largest finite = 0x7E = 448

Quantisation: ``q = e4m3(clamp(float32(x) / scale, -448, +448))`` with
round-to-nearest, ties to even mantissa.  Dequantisation: ``float32(q) * scale``.
Written with explicit integer arithmetic so that it is independent of
PyTorch's cast, which the tests use as a second witness.
"""

from __future__ import annotations

import numpy as np
import torch

E4M3_MAX = 448.0


def decode_table() -> np.ndarray:
    """float32 value of each of the 256 codes (NaN for 0x7F and 0xFF)."""
    codes = np.arange(256, dtype=np.int64)
    s = np.where(codes & 0x80, -1.0, 1.0)
    e = (codes >> 3) & 0xF
    m = codes & 0x7
    val = np.where(e == 0, np.ldexp(m / 8.0, -6), np.ldexp(1.0 + m / 8.0, e - 7))
    val = s * val
    val[(e == 15) & (m == 7)] = np.nan
    return val.astype(np.float32)


def encode_e4m3(x: np.ndarray) -> np.ndarray:
    """float32 array (already scaled and clamped to +-448) -> uint8 codes, RNE."""
    x = np.asarray(x, dtype=np.float32)
    sign = np.signbit(x).astype(np.uint8) << 7
    a = np.abs(x).astype(np.float64)
    nan = np.isnan(a)
    a = np.where(nan, 0.0, a)
    # exponent of the binade holding a; below 2^-6 everything shares the
    # subnormal quantum 2^-9
    _, ex = np.frexp(a)            # a = f * 2^ex, f in [0.5, 1)
    e = np.maximum(ex - 1, -6)     # a in [2^e, 2^(e+1)) for normals
    quantum = np.ldexp(1.0, e - 3)
    steps = np.rint(a / quantum)   # numpy rint = ties to even; exact in float64
    # steps in [0, 16]; 16 means the value rounded up into the next binade
    carry = steps >= 16
    e = np.where(carry, e + 1, e)
    steps = np.where(carry, 8, steps)
    is_sub = steps < 8             # only possible when e == -6
    mant = np.where(is_sub, steps, steps - 8).astype(np.int64)
    expo = np.where(is_sub, 0, e + 7).astype(np.int64)
    code = ((expo << 3) | mant).astype(np.uint8)
    assert not np.any((expo > 15) | ((expo == 15) & (mant == 7))), "input not clamped to +-448"
    code = code | sign
    code = np.where(nan, np.uint8(0x7F) | sign, code).astype(np.uint8)
    return code


def quantize_e4m3(x: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """``uint8`` tensor of e4m3 codes of ``clamp(float32(x)/scale, +-448)``."""
    xf = x.detach().to(torch.float32).numpy()
    scaled = (xf / np.float32(scale)).astype(np.float32)
    clamped = np.clip(scaled, -E4M3_MAX, E4M3_MAX)  # NaN passes through np.clip
    return torch.from_numpy(encode_e4m3(clamped).reshape(xf.shape))


def dequantize_e4m3(codes: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 tensor ``table[codes] * scale``."""
    tab = decode_table()
    out = tab[codes.detach().numpy().astype(np.int64)] * np.float32(scale)
    return torch.from_numpy(out.astype(np.float32))
