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
