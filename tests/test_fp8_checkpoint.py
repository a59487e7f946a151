"""The offline fp8 checkpoint format (``<module>.weight`` e4m3fn + ``<module>.scale_weight`` fp32) and its loader.

Format and invariants: docs/fastWAM_weight_quantization.md:14-30 (recipe, key names, byte-exact
requantisation, error bound 16/448 of the row amax) and :9 (a file with ``*.scale_weight`` keys is the
only one read).
"""

import os

import pytest
import torch

from tybok_amd import fp8_checkpoint as F8
from tybok_amd.policies.common import load_state_dict
from tybok_amd.quant import quantize_weight_rows


def _toy_state_dict():
    g = torch.Generator().manual_seed(0)
    return {
        "model.layers.0.mlp.gate_proj.weight": (torch.randn(512, 256, generator=g) * 0.02).to(torch.bfloat16),
        "model.layers.0.mlp.up_proj.weight": (torch.randn(512, 256, generator=g) * 0.02).to(torch.bfloat16),
        "model.layers.0.mlp.down_proj.weight": (torch.randn(256, 512, generator=g) * 0.02).to(torch.bfloat16),
        "model.layers.0.self_attn.q_proj.weight": torch.randn(256, 256, generator=g).to(torch.bfloat16),  # not an MLP projection
        "model.small.mlp.gate_proj.weight": torch.randn(128, 256, generator=g).to(torch.bfloat16),  # one side < 256
        "model.layers.0.input_layernorm.weight": torch.ones(256, dtype=torch.bfloat16),
    }


def test_selection_recipe_and_invariants():
    sd = _toy_state_dict()
    q = F8.quantize_state_dict(sd)
    fp8_names = sorted(k for k, v in q.items() if v.dtype == torch.float8_e4m3fn)
    assert fp8_names == sorted(k for k in sd if ".layers.0.mlp." in k)
    for name in fp8_names:
        w, w8, s = sd[name].float(), q[name], q[name[: -len(".weight")] + ".scale_weight"]
        assert s.dtype == torch.float32 and s.shape == (w.shape[0],) and w8.shape == w.shape
        assert torch.equal(s, (w.abs().amax(dim=1) / 448.0).clamp_min(1e-12))
        deq = w8.float() * s[:, None]
        # pure e4m3 rounding: at most half an ulp of the top binade, 16/448 of the row amax
        assert float(((deq - w).abs() / w.abs().amax(dim=1, keepdim=True)).max()) <= 16.0 / 448.0 + 1e-7
        # requantising the dequantised weight with the stored scale reproduces the codes byte for byte
        again = (deq / s[:, None]).to(torch.float8_e4m3fn)
        assert torch.equal(again.view(torch.uint8), w8.view(torch.uint8))
        assert torch.equal(F8.dequantize_entry(q, name), deq.to(torch.bfloat16))
    # everything else is untouched, and quantising twice changes nothing
    for name in sd:
        if name not in fp8_names:
            assert q[name] is sd[name]
    q2 = F8.quantize_state_dict(q)
    assert all(torch.equal(q2[k].view(torch.uint8) if q[k].dtype == torch.float8_e4m3fn else q2[k], q[k].view(torch.uint8) if q[k].dtype == torch.float8_e4m3fn else q[k]) for k in q)


def test_writer_and_loader_read_only_the_fp8_file(tmp_path):
    from safetensors.torch import save_file

    sd = _toy_state_dict()
    save_file(sd, os.path.join(tmp_path, "model.safetensors"))
    assert F8.fp8_files(str(tmp_path)) == []
    wanted = {k[len("model.") :]: tuple(v.shape) for k, v in sd.items()}
    plain = load_state_dict(str(tmp_path), wanted)
    assert all(plain[k].dtype == torch.bfloat16 for k in wanted)
    path = F8.write_fp8_checkpoint(str(tmp_path))
    assert os.path.basename(path) == F8.FP8_FILE and F8.fp8_files(str(tmp_path)) == [path]
    # poison the bf16 file: with an fp8 file present it must not be read any more
    save_file({k: torch.zeros_like(v) for k, v in sd.items()}, os.path.join(tmp_path, "model.safetensors"))
    loaded = load_state_dict(str(tmp_path), wanted)
    for k in wanted:
        if "layers.0.mlp." in k:
            w8, s = quantize_weight_rows(sd["model." + k])
            assert loaded[k].dtype == torch.float8_e4m3fn and torch.equal(loaded[k].view(torch.uint8), w8.view(torch.uint8))
            assert torch.equal(loaded[k[: -len(".weight")] + ".scale_weight"], s)
        else:
            assert torch.equal(loaded[k], sd["model." + k])
    # writing again is idempotent (the writer skips its own output)
    assert F8.write_fp8_checkpoint(str(tmp_path)) == path
    with pytest.raises(FileNotFoundError):
        load_state_dict(str(tmp_path), {**wanted, "layers.9.mlp.gate_proj.weight": (1, 1)})


def test_cli_usage(tmp_path, capsys):
    assert F8.main([]) == 2
    with pytest.raises(FileNotFoundError):
        F8.main([str(tmp_path)])


@pytest.mark.gpu
def test_engine_from_fp8_checkpoint_equals_load_time_quantisation(tmp_path):
    # the engine built from an fp8 file uses the stored codes and scales as they are: same recipe as
    # the load-time quantisation of the bf16 weights, hence the same action chunk bit for bit
    import numpy as np

    from tybok_amd.policies.synthetic import write_smolvla_checkpoint, write_weight_files
    from tybok_amd.registry import create_engine

    ckpt = write_weight_files(write_smolvla_checkpoint(str(tmp_path / "ckpt"), cameras=2, seed=8, num_vlm_layers=2, vision_layers=1, num_steps=2))
    flags = dict(tl_fused_expert=True, tl_fp8_expert_mlp=True, tl_fp8_llm_mlp=True, tl_llm_fused_attn=True)
    noise = torch.zeros(1, 50, 6)
    from_bf16 = create_engine(ckpt, device="cuda", warmup=False, **flags)
    frame = from_bf16._profile_frame(cameras=2, seed=1)
    a = from_bf16.predict_action_chunk(frame, noise=noise)
    F8.write_fp8_checkpoint(ckpt)
    os.remove(os.path.join(ckpt, "model.safetensors"))  # the fp8 file is self-contained
    from_fp8 = create_engine(ckpt, device="cuda", warmup=False, **flags)
    assert np.array_equal(a, from_fp8.predict_action_chunk(frame, noise=noise))
    # without the fp8 tiers the stored codes are dequantised once to bf16: close to, not equal to, the bf16 weights
    plain = create_engine(ckpt, device="cuda", warmup=False).predict_action_chunk(frame, noise=noise)
    assert np.isfinite(plain).all() and float(np.abs(plain - a).max()) < 5e-2
