"""Pins oracle/pi05.py (model wiring) to golden vectors written from the reference's own torch
modules (tests/golden/make_golden.py).  CPU only."""

import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import cases  # noqa: E402
from oracle import pi05 as O  # noqa: E402
from oracle.smolvla import Weights  # noqa: E402


def shape_of(cfg) -> O.PI05Shape:
    return O.PI05Shape(depth=cfg.paligemma_dims["depth"], vis_layers=cfg.vision_layers, num_steps=cfg.num_steps)


def _maxdiff(a, b) -> float:
    return float(np.abs(np.asarray(a, dtype=np.float64) - np.asarray(b, dtype=np.float64)).max())


@pytest.mark.parametrize("name", ["small", "full"])
def test_oracle_matches_reference_golden(name):
    gold = np.load(os.path.join(HERE, "golden", f"pi05_{name}.npz"))
    cfg, sd, inp = cases.pi05_build(cases.PI05_CASES[name])
    shape = shape_of(cfg)
    w = Weights(sd)
    trace: dict = {}
    with torch.no_grad():
        images = [img * 2.0 - 1.0 for img in inp["images"]]
        chunk = O.sample_actions(w, shape, images, inp["img_masks"], inp["lang_tokens"], inp["lang_masks"], inp["noise"], trace=trace)
        x0 = torch.zeros(1, shape.chunk, shape.max_action_dim)
        v_half = O.denoise_step(w, shape, trace["pad_masks"], trace["kv"], x0, 0.5)
    embs = trace["prefix_embs"]
    if "prefix_embs_head" in gold:  # the full-depth fixture stores the chunk and the probe velocity only
        assert _maxdiff(embs[0, :4].float().numpy(), gold["prefix_embs_head"]) <= 1e-6
        assert _maxdiff(embs[0, -8:, :64].float().numpy(), gold["prefix_embs_tail"]) == 0.0
        assert _maxdiff(trace["kv"][0][0][0, 0, ::32].float().numpy(), gold["k_first"]) <= 1e-6
        assert _maxdiff(trace["kv"][-1][1][0, 0, ::32].float().numpy(), gold["v_last"]) <= 1e-6
    assert _maxdiff(v_half[0].numpy(), gold["v_t_half"]) <= 1e-5
    assert _maxdiff(chunk[0].numpy(), gold["chunk"]) <= 1e-5
    assert float(np.abs(gold["chunk"]).max()) > 0.1


@pytest.mark.parametrize("tag,dt", [("fp32", None), ("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_oracle_vision_mlp_tiers_match_the_reference_eager_tower(tag, dt):
    # the reference's own tower after set_mlp_dtype (tybok/policies/pi05/models/vision.py:79-87,223-235), written by
    # tests/golden/make_golden.py pi05_vit: samples of both cameras' image embeddings
    gold = np.load(os.path.join(HERE, "golden", "pi05_small_vit_tiers.npz"))
    cfg, sd, inp = cases.pi05_build(cases.PI05_CASES["small"])
    shape = O.PI05Shape(depth=cfg.paligemma_dims["depth"], vis_layers=cfg.vision_layers, num_steps=cfg.num_steps, vit_mlp_dtype=dt)
    w = Weights(sd)
    with torch.no_grad():
        for cam, img in enumerate(inp["images"]):
            emb = O.embed_image(w, shape, img * 2.0 - 1.0)
            want = gold[f"emb_{tag}_cam{cam}"]
            # same torch CPU kernels on the same operands: equal up to the summation order of a reshaped GEMM
            assert _maxdiff(emb[0, ::8, ::16].numpy(), want) <= 2e-5 * max(1.0, float(np.abs(want).max()))
    # the tiers are real: the low-precision fixtures differ from the fp32 one
    assert _maxdiff(gold["emb_bf16_cam0"], gold["emb_fp32_cam0"]) > 1e-4
    assert _maxdiff(gold["emb_fp16_cam0"], gold["emb_fp32_cam0"]) > 1e-6


def test_oracle_fused_vision_fp16_half_matches_the_reference_kernels():
    # The fp16 kernels of the reference's fused tower (triton_vision.py: `_vision_qkv_kernel`, `_vision_attn_kernel`)
    # run through Triton's CPU interpreter by tests/golden/make_golden.py pi05_vit_fused on seeded hidden states:
    # q, k, v as the projection stores them (fp32) and the attention output (bf16).  The restatement differs from
    # the kernels in summation order and in how many key blocks share a running maximum (the probabilities are
    # rounded to fp16 relative to it): rounding-level differences.  The last assertions show what the fixture pins:
    # a q|k|v projection in bf16 instead of fp16 -- what this backend's tier used to compute -- sits an order of
    # magnitude farther away.
    gold = np.load(os.path.join(HERE, "golden", "pi05_small_vit_fused.npz"))
    cfg, sd, _ = cases.pi05_build(cases.PI05_CASES["small"])
    shape = O.PI05Shape(depth=cfg.paligemma_dims["depth"], vis_layers=cfg.vision_layers, num_steps=cfg.num_steps, vit_fused=True)
    w = Weights(sd)
    hidden = cases.pi05_vit_fused_hidden(cfg)
    with torch.no_grad():
        for i in range(cfg.vision_layers):
            x = hidden[f"layer{i}"]
            (q, k, v), a = O.vit_fused_qkv_attention(w, shape, i, x)
            for name, t in (("q", q), ("k", k), ("v", v)):
                want = gold[f"{name}_layer{i}"]
                err = _maxdiff(t[0, ::4, ::8, ::4].numpy(), want)
                print(f"fused tower layer {i} {name}: oracle vs the reference kernel {err:.3g}, |{name}|max {float(np.abs(want).max()):.3g}")
                assert err <= 1e-4 * float(np.abs(want).max())  # fp16 products are exact in fp32: summation order, and a normalised value that rounds to the other fp16 neighbour under the kernel's two-pass variance
            want = gold[f"attn_layer{i}"]
            err = _maxdiff(a[0, :, ::4].float().numpy(), want)
            scale = float(np.abs(want).max())
            print(f"fused tower layer {i} attention: oracle vs the reference kernel {err:.3g}, |out|max {scale:.3g}")
            assert err <= 2.0 ** (np.floor(np.log2(scale)) - 7)  # one bf16 step at the magnitude of the largest output
            # the same half with bf16 in place of fp16 (q|k|v operands, q, k, v and the probabilities)
            p = f"{O.VIS}encoder.layers.{i}."
            h = torch.nn.functional.layer_norm(x, (shape.vis_hidden,), w[p + "layer_norm1.weight"], w[p + "layer_norm1.bias"], O.EPS)
            qb = O._lin16(h, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"], torch.bfloat16)
            hd = shape.vis_hidden // shape.vis_heads
            qb = qb.view(1, -1, shape.vis_heads, hd).transpose(1, 2)
            assert _maxdiff(qb[0, ::4, ::8, ::4].numpy(), gold[f"q_layer{i}"]) >= 10 * _maxdiff(q[0, ::4, ::8, ::4].numpy(), gold[f"q_layer{i}"])
