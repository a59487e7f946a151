"""Write golden vectors for the model-level wiring from the reference's own torch modules.

Run ONCE in the build container (the reference is not available elsewhere):

    python tests/golden/make_golden.py [smolvla|pi05|pi05_vit|pi05_vit_fused|all] [case]

For each case the reference's eager model classes (``/root/reference/tybok/policies/<model>/models``)
are constructed on the CPU from plain config dataclasses (no checkpoint, no tokenizer), loaded with
the seeded random state dict of ``tybok_amd.policies.<model>.weights.random_state_dict`` and run on
seeded inputs.  Only outputs are stored (``tests/golden/<case>.npz``): the final action chunk, the
step-0 velocity, and a few slices of prefix embedding / prefix KV.  Inputs and weights are
regenerated from the same seeds by ``tests/golden/cases.py``.
"""

from __future__ import annotations

import os
import sys
import time

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import cases  # noqa: E402

REFERENCE_ROOT = "/root/reference"


def _import_reference():
    if REFERENCE_ROOT not in sys.path:
        sys.path.insert(0, REFERENCE_ROOT)


def _load(module: torch.nn.Module, sd: dict) -> None:
    missing = []
    own = dict(module.named_parameters())
    for name, p in own.items():
        if name not in sd:
            missing.append(name)
            continue
        assert tuple(p.shape) == tuple(sd[name].shape), (name, tuple(p.shape), tuple(sd[name].shape))
        assert p.dtype == sd[name].dtype, (name, p.dtype, sd[name].dtype)
        p.data.copy_(sd[name])
    extra = sorted(set(sd) - set(own))
    assert not missing, f"reference parameters without a value: {missing[:5]} (+{len(missing)})"
    assert not extra, f"state dict entries the reference does not have: {extra[:5]} (+{len(extra)})"


def smolvla_case(name: str) -> dict:
    _import_reference()
    from tybok.policies.smolvla import config as rcfg
    from tybok.policies.smolvla.models.flow_matching import VLAFlowMatching, make_att_2d_masks

    case = cases.SMOLVLA_CASES[name]
    cfg, sd, inputs = cases.smolvla_build(case)
    vis = cfg.vlm_config.vision_config
    ref_cfg = rcfg.SmolVLAConfig(
        num_vlm_layers=cfg.num_vlm_layers,
        num_steps=cfg.num_steps,
        sampler=cfg.sampler,
        vlm_config=rcfg.VLMConfig(
            text_config=rcfg.TextConfig(), vision_config=rcfg.VisionConfig(num_hidden_layers=vis.num_hidden_layers)
        ),
    )
    default = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)  # the engine builds the model under a bf16 default
    try:
        model = VLAFlowMatching(ref_cfg, tokenizer=None)
    finally:
        torch.set_default_dtype(default)
    model.eval()
    _load(model, sd)
    images = [img * 2.0 - 1.0 for img in inputs["images"]]  # prepare_images at the model resolution
    out: dict[str, np.ndarray] = {}
    with torch.inference_mode():
        embs, pads, att = model.embed_prefix(images, inputs["img_masks"], inputs["lang_tokens"], inputs["lang_masks"], state=inputs["state"])
        out["prefix_embs_head"] = embs[0, :4].float().numpy()
        out["prefix_embs_tail"] = embs[0, -50:, :64].float().numpy()
        out["pad_masks"] = pads.numpy()
        mask2d = make_att_2d_masks(pads, att)
        pos = torch.cumsum(pads, dim=1) - 1
        _, kv = model.vlm_with_expert.forward(
            attention_mask=mask2d, position_ids=pos, past_key_values=None, inputs_embeds=[embs, None], use_cache=True, fill_kv_cache=True
        )
        last = cfg.num_vlm_layers - 1
        out["k_first"] = kv[0]["key_states"][0, ::16].float().numpy()
        out["v_last"] = kv[last]["value_states"][0, ::16].float().numpy()
        x0 = torch.zeros(1, cfg.chunk_size, cfg.max_action_dim)
        v_half = model.denoise_step(prefix_pad_masks=pads, past_key_values=kv, x_t=x0, timestep=torch.tensor([0.5], dtype=torch.float32))
        out["v_t_half"] = v_half[0].float().numpy()
        chunk = model.sample_actions(images, inputs["img_masks"], inputs["lang_tokens"], inputs["lang_masks"], inputs["state"], noise=inputs["noise"])
        out["chunk"] = chunk[0].float().numpy()
    if cfg.sampler != "euler":  # everything before the loop is the Euler case's: keep the chunk only
        out = {"chunk": out["chunk"]}
    return out


def pi05_case(name: str) -> dict:
    _import_reference()
    from tybok.policies.pi05 import config as rcfg
    from tybok.policies.pi05.models.flow_matching import PI05FlowMatching, make_att_2d_masks, prepare_attention_masks_4d

    case = cases.PI05_CASES[name]
    cfg, sd, inputs = cases.pi05_build(case)
    rcfg.GEMMA_VARIANTS["golden_vlm"] = dict(cfg.paligemma_dims)
    rcfg.GEMMA_VARIANTS["golden_expert"] = dict(cfg.expert_dims)
    ref_cfg = rcfg.PI05Config(
        paligemma_variant="golden_vlm", action_expert_variant="golden_expert", num_steps=cfg.num_steps,
        tokenizer_max_length=cfg.tokenizer_max_length,
    )  # fmt: skip
    ref_cfg._image_features = list(cfg.image_features)
    default = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        model = PI05FlowMatching(ref_cfg)
    finally:
        torch.set_default_dtype(default)
    vt = model.paligemma_with_expert.paligemma.model.vision_tower.vision_model
    vt.encoder.layers = vt.encoder.layers[: cfg.vision_layers]
    model.eval()
    _load(model, sd)
    images = [img * 2.0 - 1.0 for img in inputs["images"]]
    out: dict[str, np.ndarray] = {}
    with torch.inference_mode():
        embs, pads, att = model.embed_prefix(images, inputs["img_masks"], inputs["lang_tokens"], inputs["lang_masks"])
        out["prefix_embs_head"] = embs[0, :4].float().numpy()
        out["prefix_embs_tail"] = embs[0, -8:, :64].float().numpy()
        mask4d = prepare_attention_masks_4d(make_att_2d_masks(pads, att))
        pos = torch.cumsum(pads, dim=1) - 1
        _, kv = model.paligemma_with_expert.forward(
            attention_mask=mask4d, position_ids=pos, past_key_values=None, inputs_embeds=[embs, None], use_cache=True
        )
        out["k_first"] = kv[0][0][0, 0, ::32].float().numpy()
        out["v_last"] = kv[-1][1][0, 0, ::32].float().numpy()
        x0 = torch.zeros(1, cfg.chunk_size, cfg.max_action_dim)
        v_half = model.denoise_step(prefix_pad_masks=pads, past_key_values=kv, x_t=x0, timestep=torch.tensor([0.5], dtype=torch.float32))
        out["v_t_half"] = v_half[0].float().numpy()
        chunk = model.sample_actions(images, inputs["img_masks"], inputs["lang_tokens"], inputs["lang_masks"], noise=inputs["noise"])
        out["chunk"] = chunk[0].float().numpy()
    if name == "full":  # full depth: the chunk and the probe velocity only (small fixture)
        out = {k: out[k] for k in ("chunk", "v_t_half")}
    return out


def pi05_vit_tiers() -> dict:
    """The reference's eager SigLIP tower with ``set_mlp_dtype`` (tybok/policies/pi05/models/vision.py:79-87,
    223-235; the engine's ``--vit-mlp-dtype``, engine.py:211-230) on the small case: samples of both cameras' image
    embeddings (tower + projector) for the fp32 tower and for the bf16 and fp16 MLP tiers."""
    _import_reference()
    from tybok.policies.pi05 import config as rcfg
    from tybok.policies.pi05.models.flow_matching import PI05FlowMatching

    case = cases.PI05_CASES["small"]
    cfg, sd, inputs = cases.pi05_build(case)
    rcfg.GEMMA_VARIANTS["golden_vlm"] = dict(cfg.paligemma_dims)
    rcfg.GEMMA_VARIANTS["golden_expert"] = dict(cfg.expert_dims)
    ref_cfg = rcfg.PI05Config(
        paligemma_variant="golden_vlm", action_expert_variant="golden_expert", num_steps=cfg.num_steps,
        tokenizer_max_length=cfg.tokenizer_max_length,
    )  # fmt: skip
    ref_cfg._image_features = list(cfg.image_features)
    images = [img * 2.0 - 1.0 for img in inputs["images"]]
    out: dict[str, np.ndarray] = {}
    for tag, dt in (("fp32", None), ("bf16", torch.bfloat16), ("fp16", torch.float16)):
        default = torch.get_default_dtype()
        torch.set_default_dtype(torch.bfloat16)
        try:
            model = PI05FlowMatching(ref_cfg)
        finally:
            torch.set_default_dtype(default)
        vt = model.paligemma_with_expert.paligemma.model.vision_tower.vision_model
        vt.encoder.layers = vt.encoder.layers[: cfg.vision_layers]
        model.eval()
        _load(model, sd)
        if dt is not None:
            vt.set_mlp_dtype(dt)
        with torch.inference_mode():
            for cam, img in enumerate(images):
                emb = model.paligemma_with_expert.embed_image(img)
                out[f"emb_{tag}_cam{cam}"] = emb[0, ::8, ::16].float().numpy()  # 32 patches x 128 channels
    return out


def pi05_vit_fused() -> dict:
    """The fp16 half of the reference's FUSED SigLIP tier (``--tl-fused-vit``): LayerNorm + packed fp16 q|k|v
    projection (`_vision_qkv_kernel`) and the flash attention over fp16 q, k, v with fp16 probabilities
    (`_vision_attn_kernel`), tybok/policies/pi05/models/vision.py:133-156 and triton_vision.py:38-110, 248-326 --
    run through Triton's CPU interpreter (``TRITON_INTERPRET=1``; set by ``main`` before anything imports triton):
    both layers of the small case's tower applied to seeded fp32 hidden states.  The bf16 kernels of that tier
    (out_proj, MLP, projector) get no fixture: this interpreter multiplies bf16 operands as their raw 16-bit
    integers (its out_proj returns 1e12 for inputs of order one), and the MLP kernel calls CUDA's libdevice tanh,
    which it does not have."""
    assert os.environ.get("TRITON_INTERPRET") == "1"
    _import_reference()
    from tybok.policies.pi05 import config as rcfg
    from tybok.policies.pi05.models.flow_matching import PI05FlowMatching
    from tybok.policies.pi05.models.triton_vision import triton_vision_attention

    case = cases.PI05_CASES["small"]
    cfg, sd, _ = cases.pi05_build(case)
    rcfg.GEMMA_VARIANTS["golden_vlm"] = dict(cfg.paligemma_dims)
    rcfg.GEMMA_VARIANTS["golden_expert"] = dict(cfg.expert_dims)
    ref_cfg = rcfg.PI05Config(
        paligemma_variant="golden_vlm", action_expert_variant="golden_expert", num_steps=cfg.num_steps,
        tokenizer_max_length=cfg.tokenizer_max_length,
    )  # fmt: skip
    ref_cfg._image_features = list(cfg.image_features)
    default = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        model = PI05FlowMatching(ref_cfg)
    finally:
        torch.set_default_dtype(default)
    vt = model.paligemma_with_expert.paligemma.model.vision_tower.vision_model
    vt.encoder.layers = vt.encoder.layers[: cfg.vision_layers]
    model.eval()
    _load(model, sd)
    vt.set_fused_attn()
    hidden = cases.pi05_vit_fused_hidden(cfg)
    out: dict[str, np.ndarray] = {}
    with torch.inference_mode():
        for i, layer in enumerate(vt.encoder.layers):
            q, k, v, b, length, c, attn = layer._fused_qkv(hidden[f"layer{i}"])  # fp32 [B, H, L, HD]
            a = triton_vision_attention(q, k, v, attn.scale)  # bf16 [B, H, L, HD]
            assert q.dtype == torch.float32 and a.dtype == torch.bfloat16
            for name, t in (("q", q), ("k", k), ("v", v)):
                out[f"{name}_layer{i}"] = t[0, ::4, ::8, ::4].numpy()  # 4 heads x 32 patches x 18 channels
            out[f"attn_layer{i}"] = a[0, :, ::4].float().numpy()  # every head, 64 patches, 72 channels
    return out


def main() -> None:
    which = sys.argv[1] if len(sys.argv) > 1 else "all"
    if which == "pi05_vit_fused":
        # the reference's fused tower kernels, through Triton's interpreter: its own run (the variable must be set
        # before triton is imported, and it changes nothing for the other fixtures, which launch no Triton kernel)
        os.environ["TRITON_INTERPRET"] = "1"
        t0 = time.time()
        path = os.path.join(HERE, "pi05_small_vit_fused.npz")
        np.savez_compressed(path, **pi05_vit_fused())
        print(f"pi05 fused vit (fp16 q|k|v + attention): wrote {path} ({os.path.getsize(path) / 1024:.0f} KiB) in {time.time() - t0:.1f}s", flush=True)
        return
    torch.manual_seed(0)
    jobs = []
    if which in ("smolvla", "all"):
        jobs += [("smolvla", n) for n in cases.SMOLVLA_CASES]
    if which in ("pi05", "all"):
        jobs += [("pi05", n) for n in cases.PI05_CASES]
    if which in ("pi05_vit", "all"):
        t0 = time.time()
        path = os.path.join(HERE, "pi05_small_vit_tiers.npz")
        np.savez_compressed(path, **pi05_vit_tiers())
        print(f"pi05 vit tiers: wrote {path} ({os.path.getsize(path) / 1024:.0f} KiB) in {time.time() - t0:.1f}s", flush=True)
    only = sys.argv[2] if len(sys.argv) > 2 else None  # optional: one case name
    for model, name in jobs:
        if only and name != only:
            continue
        t0 = time.time()
        out = smolvla_case(name) if model == "smolvla" else pi05_case(name)
        path = os.path.join(HERE, f"{model}_{name}.npz")
        np.savez_compressed(path, **out)
        print(f"{model}:{name}: wrote {path} ({os.path.getsize(path) / 1024:.0f} KiB) in {time.time() - t0:.1f}s", flush=True)


if __name__ == "__main__":
    main()
