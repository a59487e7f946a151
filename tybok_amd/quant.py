"""Per-output-channel e4m3fn weight quantisation (host/offline side of the fp8 path).

Same recipe as the reference's ``quantize_weight_rows``
(tybok/policies/pi05/models/triton_expert_mlp_fp8.py:32-48) and ``FP8Linear.from_linear``
(tybok/policies/fastwam/models/fp8_linear.py:298-310):
``scale[n] = max(amax_k |W[n, k]| / 448, 1e-12)`` in fp32, ``W8 = RNE(W / scale)`` as
``float8_e4m3fn`` (torch's cast is round-to-nearest-even and ``|W/scale| <= 448`` never saturates).
"""

from __future__ import annotations

import torch

FP8_MAX = 448.0


def quantize_weight_rows(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``[N, K]`` weight (any float dtype, any device) -> (e4m3fn ``[N, K]``, fp32 scale ``[N]``)."""
    if w.dim() != 2:
        raise ValueError("expected a 2-D [out, in] weight")
    wf = w.detach().to(torch.float32)
    # tensor / tensor: a true fp32 division on every device (dividing by a Python scalar is turned into
    # a multiplication by 1/448 on the GPU, one ulp off for some rows -- the codes of a checkpoint
    # quantised offline on the CPU and at load time on the GPU would then differ)
    amax = wf.abs().amax(dim=1, keepdim=True)
    scale = torch.div(amax, torch.full_like(amax, FP8_MAX)).clamp_min(1e-12)
    w8 = (wf / scale).to(torch.float8_e4m3fn).contiguous()
    return w8, scale.squeeze(1).contiguous()


def dequantize_weight_rows(w8: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """fp32 ``W8 * scale[:, None]``."""
    return w8.to(torch.float32) * scale.to(torch.float32)[:, None]
