"""Offline fp8 checkpoints: ``<module>.weight`` as e4m3fn ``[out, in]`` plus ``<module>.scale_weight`` fp32 ``[out]``.

The on-disk convention is the reference's (docs/fastWAM_weight_quantization.md:14-30, loader rule
at :9): every selected ``nn.Linear`` weight is stored as its fp8 codes under the module's own
``.weight`` key with a sibling ``.scale_weight``; everything else keeps its dtype, so the file is
self-contained, and a ``*.safetensors`` file that contains a ``*.scale_weight`` key is an fp8 file
-- when one is present it is the only weight file read.  The recipe is ``tybok_amd.quant``'s
(``scale = max(row amax / 448, 1e-12)``, ``W8 = RNE(W / scale)``), so requantising the dequantised
weights with the stored scales reproduces the stored codes byte for byte.

Selection (same rule, :65-71): 2-D weights with both sides >= 256 among the modules the fp8 tiers
run on fp8 -- the gate / up / down projections of the VLM and action-expert MLPs.

    python -m tybok_amd.fp8_checkpoint /ckpt/smolvla            # writes /ckpt/smolvla/model.fp8.safetensors
"""

from __future__ import annotations

import glob
import os
import sys

import torch

from .quant import dequantize_weight_rows, quantize_weight_rows

FP8_FILE = "model.fp8.safetensors"
SCALE_SUFFIX = ".scale_weight"
MIN_SIDE = 256
_MLP_PROJECTIONS = (".mlp.gate_proj.weight", ".mlp.up_proj.weight", ".mlp.down_proj.weight")


def is_fp8_selected(name: str, tensor: torch.Tensor) -> bool:
    """True for the weights this backend stores as fp8: decoder-MLP projections, both sides >= 256."""
    return name.endswith(_MLP_PROJECTIONS) and tensor.dim() == 2 and min(tensor.shape) >= MIN_SIDE and tensor.is_floating_point()


def quantize_state_dict(sd: dict[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    """Replace every selected weight by its e4m3fn codes and add ``<module>.scale_weight``."""
    out: dict[str, torch.Tensor] = {}
    for name, t in sd.items():
        if t.dtype != torch.float8_e4m3fn and is_fp8_selected(name, t):
            w8, scale = quantize_weight_rows(t)
            out[name] = w8
            out[name[: -len(".weight")] + SCALE_SUFFIX] = scale
        else:
            out[name] = t
    return out


def dequantize_entry(sd: dict[str, torch.Tensor], weight_name: str, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """The bf16 weight a non-fp8 tier multiplies with: ``W8 * scale`` rounded once."""
    scale = sd[weight_name[: -len(".weight")] + SCALE_SUFFIX]
    return dequantize_weight_rows(sd[weight_name], scale).to(dtype)


def fp8_files(checkpoint_dir: str) -> list[str]:
    """The ``*.safetensors`` files of the directory that carry ``*.scale_weight`` keys."""
    from safetensors import safe_open

    found = []
    for file in sorted(glob.glob(os.path.join(checkpoint_dir, "*.safetensors"))):
        with safe_open(file, "pt", "cpu") as f:
            if any(k.endswith(SCALE_SUFFIX) for k in f.keys()):
                found.append(file)
    return found


def write_fp8_checkpoint(checkpoint_dir: str, out_name: str = FP8_FILE) -> str:
    """Quantise the checkpoint's weight files into one self-contained fp8 file next to them."""
    from safetensors import safe_open
    from safetensors.torch import save_file

    sd: dict[str, torch.Tensor] = {}
    for file in sorted(glob.glob(os.path.join(checkpoint_dir, "*.safetensors"))):
        base = os.path.basename(file)
        if "processor" in base or base == out_name:
            continue
        with safe_open(file, "pt", "cpu") as f:
            for name in f.keys():
                sd[name] = f.get_tensor(name)
    if not sd:
        raise FileNotFoundError(f"no weight *.safetensors under {checkpoint_dir}")
    q = {k: v.contiguous() for k, v in quantize_state_dict(sd).items()}
    n_fp8 = sum(1 for k in q if k.endswith(SCALE_SUFFIX))
    if n_fp8 == 0:
        raise ValueError("no weight matched the fp8 selection rule (decoder MLP projections with both sides >= 256)")
    path = os.path.join(checkpoint_dir, out_name)
    save_file(q, path, metadata={"format": "pt", "fp8_matrices": str(n_fp8), "recipe": "e4m3fn rows, scale=max(amax/448,1e-12)"})
    return path


def main(argv: list[str] | None = None) -> int:
    args = list(sys.argv[1:] if argv is None else argv)
    if len(args) != 1:
        print(__doc__)
        return 2
    path = write_fp8_checkpoint(args[0])
    print(path)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
