"""fp8 e4m3fn (OCP) weight quantisation -- CPU oracle (test infrastructure, not the product).

Follows the reference's recipe:

* ``quantize_weight_rows``  tybok/policies/pi05/models/triton_expert_mlp_fp8.py:32-48
* ``FP8Linear.from_linear`` tybok/policies/fastwam/models/fp8_linear.py:298-310
* prose + invariants        docs/fastWAM_weight_quantization.md:14-30,141-158

``scale[n] = max(amax_k |W[n,k]| / 448, 1e-12)`` (fp32), ``W8 = RNE(W.float() / scale)`` stored as
``torch.float8_e4m3fn``.  The code table and the software encoder below are written from the OCP
e4m3fn definition (1 sign, 4 exponent bits bias 7, 3 mantissa bits, no inf, NaN = 0x7F/0xFF,
max finite 448) so that they check torch's cast instead of restating it.
"""

from __future__ import annotations

import numpy as np
import torch

FP8_MAX = 448.0


def e4m3fn_table() -> np.ndarray:
    """Value of each of the 256 e4m3fn codes as float32 (NaN for 0x7F / 0xFF)."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if exp == 0xF and man == 0x7:
            out[code] = np.nan
        elif exp == 0:
            out[code] = sign * (man / 8.0) * 2.0**-6
        else:
            out[code] = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 7)
    return out


def decode_e4m3fn(codes: torch.Tensor) -> torch.Tensor:
    """uint8 codes -> float32 values through the table (no torch fp8 dtype involved)."""
    table = torch.from_numpy(e4m3fn_table())
    return table[codes.to(torch.int64)]


def encode_e4m3fn_rne(x: torch.Tensor) -> torch.Tensor:
    """float32 -> e4m3fn codes (uint8), round-to-nearest-even, written independently of torch's cast.

    Values whose magnitude rounds above 448 become NaN (0x7F), as torch's non-saturating cast
    does; the quantiser never produces them because ``|W/scale| <= 448``.
    """
    xf = x.detach().to(torch.float64).flatten()
    sign = (torch.signbit(xf)).to(torch.int64) << 7
    a = xf.abs()
    codes = torch.zeros_like(a, dtype=torch.int64)
    # quantum per binade: subnormals and the first normal binade share 2^-9
    e = torch.floor(torch.log2(torch.clamp(a, min=2.0**-30)))
    e = torch.clamp(e, min=-6.0, max=8.0)
    quantum = 2.0 ** (e - 3.0)
    q = a / quantum
    r = torch.floor(q)
    frac = q - r
    up = (frac > 0.5) | ((frac == 0.5) & (torch.remainder(r, 2.0) == 1.0))
    r = r + up.to(r.dtype)
    val = r * quantum  # exactly representable in e4m3 unless it overflowed
    # re-derive exponent/mantissa from the rounded value
    nz = val > 0
    e2 = torch.floor(torch.log2(torch.clamp(val, min=2.0**-30)))
    sub = val < 2.0**-6
    man_sub = torch.round(val / 2.0**-9).to(torch.int64)
    exp_n = (e2 + 7).to(torch.int64)
    man_n = torch.round((val / 2.0**e2 - 1.0) * 8.0).to(torch.int64)
    codes = torch.where(sub, man_sub, (exp_n << 3) | man_n)
    codes = torch.where(nz, codes, torch.zeros_like(codes))
    overflow = (val > FP8_MAX) | torch.isnan(xf)
    codes = torch.where(overflow, torch.full_like(codes, 0x7F), codes)
    return (codes | sign).to(torch.uint8).reshape(x.shape)


def quantize_weight_rows(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``[N, K]`` float weight -> (``float8_e4m3fn [N, K]``, fp32 scale ``[N]``).

    tybok/policies/pi05/models/triton_expert_mlp_fp8.py:41-44 (same as fp8_linear.py:299-301).
    """
    wf = w.detach().float()
    amax = wf.abs().amax(dim=1, keepdim=True)
    s = (amax / FP8_MAX).clamp_min(1e-12)
    w8 = (wf / s).to(torch.float8_e4m3fn).contiguous()
    return w8, s.squeeze(1).contiguous()


def dequantize_rows(w8: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """fp32 ``W8 * scale[:, None]`` (what the fp8 GEMM's epilogue is equivalent to)."""
    return w8.float() * scale.float()[:, None]
