"""pi0.5 policy engine, registered as ``model_type="pi05"``.

Constructor keywords, ``describe()`` keys and the ``predict_action_chunk`` / ``select_action``
semantics are the reference's (tybok/policies/pi05/engine.py:104-132, 472-481, 668-741).  Tier
flags wired to the HIP kernels:

* ``tl_fused_expert``     expert denoising attention on ``tk_expert_attn`` (bf16 logits)
* ``tl_fp8_expert_mlp``   expert GeGLU FFN on e4m3fn weights with the gated residual fused
* ``tl_fp8_llm_mlp``      VLM prefill GeGLU FFN on e4m3fn weights
* ``tl_llm_flash_attn``   VLM prefill layers on the fused launches (norm + q|k|v + RoPE, attention
                          under the pad mask, o_proj + residual), K/V cache written by the projection

* ``vit_mlp_dtype``       SigLIP fc1 / gelu / fc2 in fp16 or bf16, everything else fp32 (drift tier)
* ``tl_fused_vit``        every linear of the SigLIP tower in bf16, scores / softmax / norms /
                          residuals fp32 (drift tier; owns the MLP precision)

* ``pad_free``            the prefix holds only the cameras a request sends (no ``empty_camera_*`` placeholder
                          slots) and the language block is cut to the next multiple of 16 live tokens; shapes
                          are recorded per ``(cameras, language length)``, new ones on first sight
                          (tybok/policies/pi05/engine.py:510-541,612-630; flow_matching.py:725-760)
* ``skip_empty_images``   eager path only: a masked-out camera slot behind a real one skips the vision tower and
                          contributes zero rows (flow_matching.py:415-437); inert under ``graph``, as in the reference

``compile_model`` and Real-Time Chunking are not implemented here and are rejected when requested.
"""

from __future__ import annotations

import logging
import os
from typing import Any

import numpy as np
import torch

from ...base import ChunkRuntime, PolicyEngine
from ...graph import StaticCall, camera_counts
from ...image_utils import resize_with_pad_center
from ...registry import register, reject_unsupported_flags
from ..common import (
    ACTION,
    OBS_LANGUAGE_ATTENTION_MASK,
    OBS_LANGUAGE_TOKENS,
    OBS_STATE,
    ErrorReport,
    FileTokenizer,
    SyntheticTokenizer,
    load_normalizer,
    load_reference_dump,
    load_state_dict,
    load_unnormalizer,
)
from .config import PI05Config
from .model import PI05Model
from .weights import parameter_inventory, random_state_dict

log = logging.getLogger("tybok.pi05")

# the checkpoint stores the VLM embedding table under the tied lm_head
# (tybok/policies/pi05/models/policy.py:35-42)
_KEY_REMAP = {
    "model.paligemma_with_expert.paligemma.lm_head.weight": "model.paligemma_with_expert.paligemma.model.language_model.embed_tokens.weight",
    "paligemma_with_expert.paligemma.lm_head.weight": "paligemma_with_expert.paligemma.model.language_model.embed_tokens.weight",
}


def build_prompt(task: str, normalized_state: torch.Tensor) -> str:
    """``"Task: <task>, State: <256-bin ints>;\\nAction: "`` (tybok/policies/pi05/preprocess.py:112-123)."""
    state = normalized_state.detach().cpu().numpy()
    bins = np.linspace(-1, 1, 256 + 1)[:-1]
    digits = np.digitize(state, bins=bins) - 1
    text = task.strip().replace("_", " ").replace("\n", " ")
    return f"Task: {text}, State: {' '.join(map(str, digits.tolist()))};\nAction: "


@register("pi05")
class PI05Engine(ChunkRuntime, PolicyEngine):
    _UNSUPPORTED_FLAGS = {
        "tl_llm_fused_attn": False,
        "tl_vit_oproj": False,
        "pack_qkv": False,
        "text_fused": False,
        "text_fused_split": False,
        "action_fused": False,
        "action_fused_split": False,
        "video_fused": False,
        "video_fused_split": False,
        "action_pre_fused": False,
        "video_pre_fused": False,
        "require_fused": False,
        "text_encoder_dir": None,
        "vae_dir": None,
    }

    def __init__(
        self,
        checkpoint_dir: str,
        device: str = "auto",
        compile_model: bool = False,
        warmup: bool = True,
        graph: bool = False,
        graph_cameras: tuple[int, ...] | None = None,
        num_steps: int | None = None,
        seed: int | None = None,
        sampler: str = "euler",
        cache_expert_prefix_kv: bool = True,
        profile: bool = False,
        overlap: bool = True,
        tl_fused_vit: bool = False,
        tl_llm_flash_attn: bool = False,
        tl_fused_expert: bool = False,
        tl_fp8_llm_mlp: bool = False,
        tl_fp8_expert_mlp: bool = False,
        vit_mlp_dtype: str | None = None,
        skip_empty_images: bool = False,
        pad_free: bool = False,
        camera_alias: dict[str, str] | None = None,
        tokenizer_dir: str | None = None,
        rtc_config: dict | None = None,
        **kwargs: Any,
    ):
        super().__init__(checkpoint_dir, device=device)
        reject_unsupported_flags(type(self), "pi05", kwargs)
        if sampler != "euler":
            raise ValueError(f"sampler {sampler!r} not supported for pi05 (only 'euler')")
        if compile_model:
            raise NotImplementedError("--compile is not supported by this backend (the HIP tiers replace it)")
        if rtc_config and rtc_config.get("enabled"):
            raise NotImplementedError("Real-Time Chunking is not implemented by this backend")
        hip_flags = [
            n
            for n, on in (
                ("--tl-fused-expert", tl_fused_expert), ("--tl-fp8-llm-mlp", tl_fp8_llm_mlp),
                ("--tl-fp8-expert-mlp", tl_fp8_expert_mlp), ("--tl-llm-flash-attn", tl_llm_flash_attn),
            )
            if on
        ]  # fmt: skip
        if hip_flags and not str(self.device).startswith("cuda"):
            # same gate as the reference's _require_fp8_mma (engine.py:51-71), for this hardware
            raise RuntimeError(f"{' / '.join(hip_flags)} run gfx950 HIP kernels, but the engine is running on {self.device!r}")
        self.compile_model = False
        self.config = PI05Config.from_pretrained(checkpoint_dir, tokenizer_dir=tokenizer_dir)
        if num_steps is not None:
            self.config.num_steps = int(num_steps)

        tok_dir = self.config.tokenizer_dir
        if tok_dir and os.path.isfile(os.path.join(tok_dir, "tokenizer.json")):
            self.tokenizer = FileTokenizer(tok_dir, self.config.tokenizer_max_length, "<pad>")
        elif self.config.random_init is not None:
            self.tokenizer = SyntheticTokenizer(self.config.vocab_size, self.config.tokenizer_max_length)
        else:
            raise FileNotFoundError("no tokenizer.json: pass --tokenizer-dir")

        if self.config.random_init is not None and self.config.random_init.get("weights") != "files":
            sd = random_state_dict(self.config, seed=int(self.config.random_init.get("seed", 0)))
        else:
            sd = load_state_dict(checkpoint_dir, {n: s for n, s, _, _ in parameter_inventory(self.config)}, remap=_KEY_REMAP)
        # vision drift tiers (tybok/policies/pi05/engine.py:196-230): --vit-mlp-dtype converts fc1 / fc2 only;
        # --tl-fused-vit runs every linear of the tower in bf16 (scores and softmax stay fp32) and owns
        # the MLP precision, so --vit-mlp-dtype is inert under it
        if vit_mlp_dtype not in (None, "fp16", "bf16"):
            raise ValueError(f"--vit-mlp-dtype must be 'fp16' or 'bf16', got {vit_mlp_dtype!r}")
        self.tl_fused_vit = bool(tl_fused_vit)
        self.vit_mlp_dtype = None
        if self.tl_fused_vit:
            self.vit_mlp_dtype = torch.bfloat16
        elif vit_mlp_dtype is not None:
            self.vit_mlp_dtype = torch.float16 if vit_mlp_dtype == "fp16" else torch.bfloat16
        self.tl_fused_expert = bool(tl_fused_expert)
        self.tl_fp8_llm_mlp = bool(tl_fp8_llm_mlp)
        # tl_fp8_llm_mlp="w8a8": the reference tier's arithmetic -- activations quantised per token with the scale and
        # the quotient rounded to bf16 (triton_prefill_mlp.py:26-59), fp8 x fp8 products; True keeps the activations
        # in bf16 (weight-only).  The weight scales stay fp32 (the reference prefill computes them in bf16)
        self.fp8_llm_act = isinstance(tl_fp8_llm_mlp, str) and tl_fp8_llm_mlp.lower() == "w8a8"
        self.tl_fp8_expert_mlp = bool(tl_fp8_expert_mlp)
        self.model = PI05Model(
            self.config, sd, self.device,
            fused_expert=self.tl_fused_expert, fp8_expert_mlp=self.tl_fp8_expert_mlp, fp8_llm_mlp=self.tl_fp8_llm_mlp, fp8_llm_act=self.fp8_llm_act,
            fused_prefill=bool(tl_llm_flash_attn), vit_mlp_dtype=self.vit_mlp_dtype, vit_lowp_attn=self.tl_fused_vit,
        )  # fmt: skip
        del sd

        norm_map = self.config.normalization_mapping
        self.normalizer = load_normalizer(checkpoint_dir, norm_map)
        self.unnormalizer = load_unnormalizer(checkpoint_dir, norm_map)
        self.camera_alias: dict[str, str] = {}
        for src, dst in (camera_alias or {}).items():
            s = src if src.startswith("observation.images.") else f"observation.images.{src}"
            d = dst if dst.startswith("observation.images.") else f"observation.images.{dst}"
            if d not in self.config.image_features:
                raise ValueError(f"camera_alias target {dst!r} is not an expected image feature")
            self.camera_alias[s] = d

        self._init_sampling(seed)
        self._mask_cache: dict[tuple[int, bool, str], torch.Tensor] = {}
        self.rtc_processor = None
        self._init_graphs(graph, "pi05 graph", log)
        self.overlap = False  # prefill x step-0 two-stream overlap is not implemented; accepted, inert
        if overlap and graph:
            log.info("overlap requested: the prefill x step-0 overlap is not built for pi0.5 here; requests run sequentially (engine.overlap is False)")
        self.pad_free = bool(pad_free)
        self.model.pad_free = self.pad_free
        self.skip_empty_images = bool(skip_empty_images)
        self.model.skip_empty_images = self.skip_empty_images
        if self.skip_empty_images:
            if self.graph_enabled:
                log.info("skip_empty_images is inert on the graph path (a recorded shape runs every slot); pad_free drops the empty slots from the prefix instead")
            else:
                log.info("empty camera slots skip the vision tower")
        self._start(warmup=warmup, graph_keys=self._graph_keys(graph_cameras), profile=profile, logger=log)

    def _graph_keys(self, graph_cameras) -> list[tuple[int, int]]:
        """``(camera count, language length)`` shapes recorded at start-up (tybok/policies/pi05/engine.py:527-541):
        every image slot plus the full language block; with ``pad_free`` one shape per requested camera count at the
        full language length -- shorter language buckets are recorded on first sight."""
        full_lang = self.config.tokenizer_max_length
        if not self.pad_free:
            return [(len(self.config.image_features), full_lang)]
        max_cams = len(self.config.real_camera_keys)
        return [(c, full_lang) for c in camera_counts(graph_cameras, default=min(2, max_cams), max_images=max_cams)]

    # ------------------------------------------------------------------ API
    def supports_rtc(self) -> bool:
        return False

    def describe(self) -> dict[str, Any]:
        return {
            "model_type": "pi05",
            "cameras": [k[len("observation.images.") :] for k in self.config.real_camera_keys],
            "resize": [self.config.image_resolution[1], self.config.image_resolution[0]],
            "pad_mode": "center",
            "action_dim": int(self.config.action_feature_shape[0]),
            "chunk_size": int(self.config.chunk_size),
            "rtc": False,
        }

    @torch.inference_mode()
    def predict_action_chunk(self, frame: dict[str, Any], noise: torch.Tensor | None = None, *, return_normalized: bool = False, **rtc: Any) -> Any:
        if any(v is not None for v in rtc.values()):
            raise NotImplementedError("Real-Time Chunking guidance arguments are not supported by this backend")
        actions = self._robot_actions(frame, noise)
        chunk = self._to_robot_units(actions)
        return (chunk, actions.cpu().numpy()[0]) if return_normalized else chunk

    @torch.inference_mode()
    def select_action(self, frame: dict[str, Any], noise: torch.Tensor | None = None) -> np.ndarray:
        return self._next_queued_action(frame, noise)

    @torch.inference_mode()
    def validate(self, reference_dir: str) -> dict[str, float]:
        """Per-component max / mean-abs errors against a reference dump, keyed like the reference's
        report (tybok/policies/pi05/engine.py:740-857): ``batch.*``, ``prefix.{embs,pad_masks,att_masks}``,
        ``prefix_kv.layer<i>.{keys,values}``, ``denoise.v_t`` (zero ``x_t``, t = 0.5), ``chunk`` (zero
        noise, through the graph when enabled) and ``chunk_post``.  ``frame.pt`` and ``chunk.pt`` are
        required, the other dump files are compared when present."""
        dump = load_reference_dump(reference_dir)
        report = ErrorReport()
        cfg, m = self.config, self.model
        batch = self._batch_from_frame(dump["frame"])
        report.compare_batch(batch, dump["batch"], (OBS_STATE, OBS_LANGUAGE_TOKENS, OBS_LANGUAGE_ATTENTION_MASK))
        images, img_masks = self.prepare_images(batch)
        embs, pads = m.embed_prefix(images, img_masks, batch[OBS_LANGUAGE_TOKENS], batch[OBS_LANGUAGE_ATTENTION_MASK])
        if dump["prefix"] is not None:
            report.compare("prefix.embs", embs, dump["prefix"]["embs"])
            report.compare("prefix.pad_masks", pads, dump["prefix"]["pad_masks"])
            if "att_masks" in dump["prefix"]:  # every prefix token attends to every valid one: all zeros
                report.compare("prefix.att_masks", torch.zeros_like(pads), dump["prefix"]["att_masks"])
        if dump["prefix_kv"] is not None or dump["denoise"] is not None:
            kv = m.prefill_fused(embs, pads)[0] if m.fused_prefill and embs.shape[0] == 1 else m.prefill(embs, pads)
            report.compare_prefix_kv(kv, dump["prefix_kv"])
            if dump["denoise"] is not None:
                x_t = torch.zeros(1, cfg.chunk_size, cfg.max_action_dim, device=self.device)
                report.compare("denoise.v_t", m.velocity_at(pads, kv, x_t, 0.5), dump["denoise"]["v_t"])
        chunk = self._infer(batch, torch.zeros(1, cfg.chunk_size, cfg.max_action_dim, device=self.device))[:, :, : cfg.action_feature_shape[0]]
        if "chunk" in dump["chunk"]:
            report.compare("chunk", chunk, dump["chunk"]["chunk"].reshape(chunk.shape))
        post = self.unnormalizer.unnormalize(chunk, ACTION, "ACTION")
        report.compare("chunk_post", post, dump["chunk"]["chunk_post"].reshape(post.shape))
        return report

    # ------------------------------------------------------------------ request plumbing
    def _batch_from_frame(self, frame: dict[str, Any]) -> dict[str, torch.Tensor]:
        """Batch dimension, state normalisation, state-in-prompt tokenisation (preprocess.py:159-189)."""
        frame = dict(frame)
        for src, dst in self.camera_alias.items():
            if src in frame and dst not in frame:
                frame[dst] = frame.pop(src)
        batch: dict[str, torch.Tensor] = {}
        for key, value in frame.items():
            if key.startswith("observation.") and isinstance(value, torch.Tensor):
                batch[key] = value.unsqueeze(0) if value.ndim in (1, 3) else value
        if OBS_STATE in batch:
            batch[OBS_STATE] = self.normalizer.normalize(batch[OBS_STATE], OBS_STATE, "STATE")
        if OBS_LANGUAGE_TOKENS not in batch:
            state = batch.get(OBS_STATE)
            if state is None:
                raise ValueError("state is required for PI05")
            task = frame.get("task", "")
            if not isinstance(task, str):
                raise ValueError(f"task must be a string, got {type(task).__name__}")
            prompt = build_prompt(task, state[0] if state.ndim == 2 else state)
            batch[OBS_LANGUAGE_TOKENS], batch[OBS_LANGUAGE_ATTENTION_MASK] = self.tokenizer.encode_task(prompt)
        return {k: v.to(self.device) for k, v in batch.items()}

    def prepare_images(self, batch: dict[str, torch.Tensor]):
        """Centre-padded resize to 224x224, [0,1] -> [-1,1]; missing slots become -1 images with a zero mask
        (policy.py:170-234).  With ``pad_free`` the slots are the cameras the frame holds, nothing else."""
        h, w = self.config.image_resolution
        slots = self.config.live_camera_keys(batch) if self.pad_free else self.config.image_features
        present = [k for k in slots if k in batch]
        if not present:
            raise ValueError(f"All image features are missing from the batch (expected {self.config.image_features})")
        images01, masks = self.prepare_images01(batch)
        return [img * 2.0 - 1.0 for img in images01], masks

    def prepare_images01(self, batch: dict[str, torch.Tensor]):
        """:meth:`prepare_images` before the change of range: images in [0, 1] (an empty slot all zeros, which
        ``x * 2 - 1`` turns into the -1 filler) and the cached all-true / all-false masks."""
        h, w = self.config.image_resolution
        slots = self.config.live_camera_keys(batch) if self.pad_free else self.config.image_features
        present = [k for k in slots if k in batch]
        if not present:
            raise ValueError(f"All image features are missing from the batch (expected {self.config.image_features})")
        images, masks = [], []
        for key in present:
            img = resize_with_pad_center(batch[key].float(), h, w)
            images.append(img)
            masks.append(self._mask(img.shape[0], True, img.device))
        for _ in [k for k in slots if k not in batch]:
            images.append(torch.zeros_like(images[-1]))
            masks.append(self._mask(images[-1].shape[0], False, images[-1].device))
        return images, masks

    def _mask(self, batch_size: int, value: bool, device) -> torch.Tensor:
        """A cached all-true / all-false image mask (never written to) on the images' device."""
        key = (batch_size, value, str(device))
        if key not in self._mask_cache:
            self._mask_cache[key] = torch.full((batch_size,), value, dtype=torch.bool, device=device)
        return self._mask_cache[key]

    def _core(self, images01, img_masks, tokens, masks, noise) -> torch.Tensor:
        """The unit a graph records: the change of range of the images and the whole model."""
        return self.model.sample_actions(images01, img_masks, tokens, masks, noise, image_range01=True)

    def _infer(self, batch: dict[str, torch.Tensor], noise: torch.Tensor | None) -> torch.Tensor:
        images, img_masks = self.prepare_images01(batch)
        tokens, masks = batch[OBS_LANGUAGE_TOKENS], batch[OBS_LANGUAGE_ATTENTION_MASK]
        if self.pad_free:
            # the language block on the bucket grid, for the eager path and the recorded shapes alike
            tokens, masks = self.model.pack_language(tokens, masks)
        if self.graph_enabled and self._graph_runner:
            entry = self._graph_runner.entry((len(images), int(tokens.shape[1])))
            return self._run_graph(entry, images, img_masks, tokens, masks, noise)
        noise = self._sample_noise() if noise is None else self._pad_noise(noise)
        return self._core(images, img_masks, tokens, masks, noise)

    # ------------------------------------------------------------------ hipGraph path
    def _capture_graph(self, key, request=None) -> StaticCall:
        """Record the whole inference core once for ``key = (n_cams, lang_len)`` (the reference records the
        same unit: tybok/policies/pi05/engine.py:542-606).  Static tensors are named after the keyword
        arguments of ``PI05Model.sample_actions``."""
        cfg, dev = self.config, self.device
        n_cams, lang_len = int(key[0]), int(key[1])
        height, width = cfg.image_resolution
        f32 = dict(dtype=torch.float32, device=dev)
        call = StaticCall(
            torch.zeros(1, cfg.chunk_size, cfg.max_action_dim, **f32),
            images01=[torch.zeros(1, 3, height, width, **f32) for _ in range(n_cams)],
            img_masks=[torch.ones(1, dtype=torch.bool, device=dev) for _ in range(n_cams)],
            tokens=torch.zeros(1, lang_len, dtype=torch.int64, device=dev),
            masks=torch.ones(1, lang_len, dtype=torch.bool, device=dev),
            noise=torch.zeros(1, cfg.chunk_size, cfg.max_action_dim, **f32),
        )
        log.info(f"capturing one graph for {n_cams} camera(s), lang={lang_len}, steps={cfg.num_steps}")
        return call.record(self._sess, self._core)

    def _run_graph(self, call: StaticCall, images, img_masks, tokens, masks, noise) -> torch.Tensor:
        """The request's tensors go into the static ones on the input stream (images still in [0, 1]: the change
        of range is part of the recorded unit; the noise at the caller's width), then the replay.  Returns the
        graph's static output: every caller is done with it, or has copied it, before the next request replays."""
        with self._graph_runner.copy_inputs():
            call.store(images01=images, tokens=tokens, masks=masks)
            call.store_owned(img_masks=img_masks)  # always the engine's cached all-true / all-false masks
            if noise is None:
                self._sample_noise(out=call.inputs["noise"])  # drawn outside the graph, from the engine's generator
                call.forget_leading("noise")
            else:
                call.store_leading(noise=noise)
        self._graph_runner.wait_inputs()
        return call.replay(copy=False)
