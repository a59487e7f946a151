"""pi0.5 request-shape flags on the host: ``pad_free`` (live cameras only, language block on a grid of 16 tokens)
and ``skip_empty_images`` (eager path: a masked-out slot skips the vision tower), restated from
tybok/policies/pi05/config.py:113-123, models/flow_matching.py:415-437,725-760 and engine.py:510-541.
CPU only: the model's plain torch path, checked against the oracle on the packed request."""

import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
sys.path.insert(0, os.path.dirname(HERE))

import cases  # noqa: E402
from oracle import pi05 as O  # noqa: E402
from oracle.smolvla import Weights  # noqa: E402


def _model(cfg, sd):
    from tybok_amd.policies.pi05.model import PI05Model

    return PI05Model(cfg, sd, "cpu")


def test_language_bucket_grid_and_live_cameras():
    cfg, sd, inp = cases.pi05_build(cases.PI05_CASES["small"])
    m = _model(cfg, sd)
    tokens, masks = inp["lang_tokens"], inp["lang_masks"]
    # flag off: nothing moves, the length is the tokenizer's
    assert m.packed_lang_len(3) == cfg.tokenizer_max_length
    t0, k0 = m.pack_language(tokens, masks)
    assert t0 is tokens and k0 is masks
    m.pad_free = True
    # the grid: next multiple of 16, capped at the tokenizer's length; 0 live tokens -> 0
    assert [m.packed_lang_len(n) for n in (0, 1, 16, 17, 140, 193, 200, 500)] == [0, 16, 16, 32, 144, 200, 200, 200]
    live = int(masks.sum())
    t, k = m.pack_language(tokens, masks)
    want = (live + 15) // 16 * 16
    assert t.shape == (1, want) and k.shape == (1, want) and int(k.sum()) == live
    assert torch.equal(t[:, :live], tokens[:, :live]) and not bool(k[:, live:].any())
    # a block that already has the bucket's length is returned as it is
    t2, k2 = m.pack_language(t, k)
    assert t2 is t and k2 is k
    # camera slots of a request: the real cameras the frame holds, in the checkpoint's order
    cfg.image_features = ["observation.images.base_0_rgb", "observation.images.left_wrist_0_rgb", "observation.images.empty_camera_0"]
    batch = {"observation.images.left_wrist_0_rgb": 1, "observation.images.empty_camera_0": 2, "observation.state": 3}
    assert cfg.live_camera_keys(batch) == ["observation.images.left_wrist_0_rgb"]
    batch["observation.images.base_0_rgb"] = 4
    assert cfg.live_camera_keys(batch) == ["observation.images.base_0_rgb", "observation.images.left_wrist_0_rgb"]


def test_pad_free_request_matches_the_oracle_on_the_packed_block():
    cfg, sd, inp = cases.pi05_build(cases.PI05_CASES["small"])
    m = _model(cfg, sd)
    m.pad_free = True
    images = [i * 2.0 - 1.0 for i in inp["images"]]
    tokens, masks = inp["lang_tokens"].clone(), inp["lang_masks"].clone()
    masks[:, 37:] = False  # 37 live tokens -> a block of 48
    with torch.inference_mode():
        trace: dict = {}
        got = m.sample_actions(images, inp["img_masks"], tokens, masks, inp["noise"], trace=trace)
    n_img = cfg.image_tokens * len(images)
    assert trace["prefix_embs"].shape[1] == n_img + 48
    shape = O.PI05Shape(depth=cfg.paligemma_dims["depth"], vis_layers=cfg.vision_layers, num_steps=cfg.num_steps)
    w = Weights(sd, O.fp8_linear_names(shape, False, False))
    with torch.no_grad():
        want = O.sample_actions(w, shape, images, inp["img_masks"], tokens[:, :48], masks[:, :48], inp["noise"])
    err = float((got - want).abs().max())
    print(f"pad_free, 37 live tokens in a block of 48: max|err| vs oracle on the packed block {err:.3g}")
    assert err <= 1e-2 * max(1.0, float(want.abs().max()))


def test_skipping_an_empty_camera_changes_no_bit():
    cfg, sd, inp = cases.pi05_build(cases.PI05_CASES["small"])
    m = _model(cfg, sd)
    images = [i * 2.0 - 1.0 for i in inp["images"]]
    images[1] = torch.full_like(images[1], -1.0)  # the placeholder of a missing camera
    img_masks = [inp["img_masks"][0], torch.zeros_like(inp["img_masks"][1])]
    with torch.inference_mode():
        plain = m.sample_actions(images, img_masks, inp["lang_tokens"], inp["lang_masks"], inp["noise"])
        m.skip_empty_images = True
        trace: dict = {}
        skipped = m.sample_actions(images, img_masks, inp["lang_tokens"], inp["lang_masks"], inp["noise"], trace=trace)
    n = cfg.image_tokens
    assert float(trace["prefix_embs"][:, n : 2 * n].abs().max()) == 0.0  # the slot went in as zeros
    assert torch.equal(plain, skipped)
