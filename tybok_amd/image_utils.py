"""Image resizing conventions of the policies (same results as the reference's
``tybok/image_utils.py:22-70``): aspect-preserving bilinear resize, then padding on the left/top
(SmolVLA) or centred with the odd pixel at the bottom/right (pi0.5)."""

from __future__ import annotations

import torch
import torch.nn.functional as F  # noqa: N812


def _resized(img: torch.Tensor, height: int, width: int) -> torch.Tensor:
    if img.ndim != 4:
        raise ValueError(f"(b,c,h,w) expected, but got {tuple(img.shape)}")
    cur_h, cur_w = img.shape[2:]
    ratio = max(cur_w / width, cur_h / height)
    return F.interpolate(img, size=(int(cur_h / ratio), int(cur_w / ratio)), mode="bilinear", align_corners=False)


def resize_with_pad(img: torch.Tensor, height: int, width: int, *, pad_value: float = 0.0) -> torch.Tensor:
    if tuple(img.shape[2:]) == (height, width):
        return img
    r = _resized(img, height, width)
    return F.pad(r, (max(0, width - r.shape[3]), 0, max(0, height - r.shape[2]), 0), value=pad_value)


def resize_with_pad_center(img: torch.Tensor, height: int, width: int, *, pad_value: float = 0.0) -> torch.Tensor:
    if tuple(img.shape[2:]) == (height, width):
        return img
    r = _resized(img, height, width).clamp(0.0, 1.0)
    ph0, rem_h = divmod(height - r.shape[2], 2)
    pw0, rem_w = divmod(width - r.shape[3], 2)
    return F.pad(r, (pw0, pw0 + rem_w, ph0, ph0 + rem_h), value=pad_value)
