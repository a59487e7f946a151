"""SmolVLA policy engine, registered as ``model_type="smolvla"``.

Constructor keywords, ``describe()`` keys and the ``predict_action_chunk`` / ``select_action``
semantics are the reference's (tybok/policies/smolvla/engine.py:78-96, 332-400), so the worker and
gateway need no change.  The tier flags select the HIP kernels:

* ``tl_fused_expert``     expert layers on the fused launches: norm + q|k|v + RoPE
                          (``tk_bf16w_linear``), ``tk_expert_attn``, o_proj + residual
* ``tl_fp8_expert_mlp``   expert gated FFN on e4m3fn weights (``tk_fp8w_gated_ffn``)
* ``tl_fp8_llm_mlp``      VLM prefill gated FFN on e4m3fn weights
* ``tl_llm_fused_attn``   VLM prefill layers on the same fused launches (2-D prefix mask)
* ``tl_vit_oproj``        vision tower with packed q|k|v and ``tk_batched_attn``

The reference's SmolVLA backend rejects the two fp8 flags (engine.py:47-55); here they are
implemented, because the fp8 action-inference path is what this backend is for.
``compile_model`` has no implementation here and is rejected when requested.
"""

from __future__ import annotations

import logging
import os
from typing import Any

import numpy as np
import torch
import torch.nn.functional as F  # noqa: N812

from ...base import ChunkRuntime, PolicyEngine
from ...graph import StaticCall, camera_counts
from ...image_utils import resize_with_pad
from ...registry import register
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
from .config import SmolVLAConfig
from .model import SmolVLAModel
from .weights import parameter_inventory, random_state_dict

log = logging.getLogger("tybok.smolvla")


@register("smolvla")
class SmolVLAEngine(ChunkRuntime, PolicyEngine):
    # flags owned by other backends or not implemented here: inert default -> accepted, else rejected
    _UNSUPPORTED_FLAGS = {
        "tl_fused_vit": False,
        "tl_llm_flash_attn": False,
        "vit_mlp_dtype": None,
        "skip_empty_images": False,
        "pad_free": False,
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
        overlap: bool = False,
        camera_alias: dict[str, str] | None = None,
        tl_llm_fused_attn: bool = False,
        tl_vit_oproj: bool = False,
        tl_fused_expert: bool = False,
        tl_fp8_llm_mlp: bool = False,
        tl_fp8_expert_mlp: bool = False,
    ):
        super().__init__(checkpoint_dir, device=device)
        if sampler not in ("euler", "heun"):
            raise ValueError(f"unknown sampler {sampler!r} (expected 'euler' or 'heun')")
        if compile_model:
            raise NotImplementedError("--compile is not supported by this backend (the HIP tiers replace it)")
        self.compile_model = False
        self.config = SmolVLAConfig.from_pretrained(checkpoint_dir)
        if self.config.vlm_config is None:
            raise ValueError(
                f"Could not locate the VLM backbone config for {self.config.vlm_model_name!r}; "
                "check `vlm_model_name` in the checkpoint config.json"
            )
        if num_steps is not None:
            self.config.num_steps = int(num_steps)
        self.config.sampler = sampler  # Heun keeps the sequential path: no prefill x step-0 overlap (reference engine :229-237)
        self.config.cache_expert_prefix_kv = bool(cache_expert_prefix_kv)
        hip_flags = [
            n
            for n, on in (
                ("--tl-fused-expert", tl_fused_expert), ("--tl-fp8-llm-mlp", tl_fp8_llm_mlp),
                ("--tl-fp8-expert-mlp", tl_fp8_expert_mlp), ("--tl-llm-fused-attn", tl_llm_fused_attn),
                ("--tl-vit-oproj", tl_vit_oproj),
            )
            if on
        ]  # fmt: skip
        if hip_flags and not str(self.device).startswith("cuda"):
            raise RuntimeError(f"{' / '.join(hip_flags)} run gfx950 HIP kernels, but the engine is running on {self.device!r}")

        vocab = self.config.vlm_config.text_config.vocab_size
        tok_dir = self.config.vlm_dir or checkpoint_dir
        if os.path.isfile(os.path.join(tok_dir, "tokenizer.json")):
            self.tokenizer = FileTokenizer(tok_dir, self.config.tokenizer_max_length, "<|im_end|>")
        elif self.config.random_init is not None:
            self.tokenizer = SyntheticTokenizer(vocab, self.config.tokenizer_max_length)
        else:
            raise FileNotFoundError(f"no tokenizer.json under {tok_dir}")

        if self.config.random_init is not None and self.config.random_init.get("weights") != "files":
            sd = random_state_dict(self.config, seed=int(self.config.random_init.get("seed", 0)))
        else:
            sd = load_state_dict(checkpoint_dir, {n: s for n, s, _, _ in parameter_inventory(self.config)})
        self.tl_fused_expert = bool(tl_fused_expert)
        self.tl_fp8_llm_mlp = bool(tl_fp8_llm_mlp)
        self.tl_fp8_expert_mlp = bool(tl_fp8_expert_mlp)
        # --tl-llm-fused-attn: the VLM prefill layers on the fused HIP launches (norm + q/k/v + RoPE +
        # KV write, attention under the 2-D prefix mask, o_proj + residual)
        self.tl_llm_fused_attn = bool(tl_llm_fused_attn)
        # --tl-vit-oproj: vision tower with q/k/v packed into one GEMM and the self-attention on the
        # HIP kernel (the reference's tier packs q/k/v and fuses out_proj over the SDPA layout)
        self.tl_vit_oproj = bool(tl_vit_oproj)
        self.model = SmolVLAModel(
            self.config, sd, self.device,
            fused_expert=self.tl_fused_expert, fp8_expert_mlp=self.tl_fp8_expert_mlp, fp8_llm_mlp=self.tl_fp8_llm_mlp,
            fused_prefill=self.tl_llm_fused_attn, fused_vit=self.tl_vit_oproj,
            # graph mode only, like the reference (smolvla/engine.py:229-237); needs both fused tiers
            overlap=bool(overlap) and bool(graph) and sampler == "euler" and str(self.device).startswith("cuda"),
        )  # fmt: skip
        del sd

        norm_map = self.config.normalization_mapping
        self.normalizer = load_normalizer(checkpoint_dir, norm_map)
        self.unnormalizer = load_unnormalizer(checkpoint_dir, norm_map)
        self.camera_alias = self._resolve_alias(camera_alias)

        self._init_sampling(seed)
        self._token_cache: dict[str, tuple[torch.Tensor, torch.Tensor]] = {}
        self._mask_cache: dict[tuple[int, bool], torch.Tensor] = {}
        self._init_graphs(graph, "smolvla graph", log)
        self.overlap = self.model.overlap  # step 0 of the Euler loop hidden inside the prefill (two streams)
        self._graph_fallback_warned = False
        cameras = len(self.config.image_features)
        keys = [(n,) for n in camera_counts(graph_cameras, default=cameras, max_images=cameras)]
        self._start(warmup=warmup, graph_keys=keys, profile=profile, logger=log)

    # ------------------------------------------------------------------ API
    def describe(self) -> dict[str, Any]:
        return {
            "model_type": "smolvla",
            "cameras": [k[len("observation.images.") :] for k in self.config.image_features],
            "resize": list(self.config.resize_imgs_with_padding),
            "action_dim": int(self.config.action_feature_shape[0]),
            "chunk_size": int(self.config.chunk_size),
        }

    @torch.inference_mode()
    def predict_action_chunk(self, frame: dict[str, Any], noise: torch.Tensor | None = None) -> np.ndarray:
        return self._to_robot_units(self._robot_actions(frame, noise))

    @torch.inference_mode()
    def select_action(self, frame: dict[str, Any], noise: torch.Tensor | None = None) -> np.ndarray:
        return self._next_queued_action(frame, noise)

    @torch.inference_mode()
    def validate(self, reference_dir: str) -> dict[str, float]:
        """Per-component max / mean-abs errors against a reference dump, keyed like the reference's
        report (tybok/policies/smolvla/engine.py:655-752): ``batch.*``, ``prefix.{embs,pad_masks,
        att_masks}``, ``prefix_kv.layer<i>.{keys,values}``, ``denoise.v_t`` (zero ``x_t``, t = 0.5),
        ``chunk`` (zero noise, through the graph when enabled) and ``chunk_post``.  ``frame.pt`` and
        ``chunk.pt`` are required, the other dump files are compared when present."""
        dump = load_reference_dump(reference_dir)
        report = ErrorReport()
        cfg, m = self.config, self.model
        batch = self._batch_from_frame(dump["frame"])
        report.compare_batch(batch, dump["batch"], (OBS_STATE, OBS_LANGUAGE_TOKENS, OBS_LANGUAGE_ATTENTION_MASK))
        images, img_masks = self.prepare_images(batch)
        embs, pads, att = m.embed_prefix(images, img_masks, batch[OBS_LANGUAGE_TOKENS], batch[OBS_LANGUAGE_ATTENTION_MASK], self.prepare_state(batch))
        if dump["prefix"] is not None:
            for name, got in (("embs", embs), ("pad_masks", pads), ("att_masks", att)):
                report.compare(f"prefix.{name}", got, dump["prefix"][name])
        if dump["prefix_kv"] is not None or dump["denoise"] is not None:
            fused = m.fused_prefill and embs.shape[0] == 1
            keys, values = m.prefill_fused(embs, pads, att)[:2] if fused else m.prefill(embs, pads, att)
            report.compare_prefix_kv(list(zip(keys, values))[: cfg.num_vlm_layers], dump["prefix_kv"])
            if dump["denoise"] is not None:
                from .model import sinusoidal_time_embedding

                x_t = torch.zeros(1, cfg.chunk_size, cfg.max_action_dim, device=self.device)
                te = sinusoidal_time_embedding(torch.tensor([0.5]), cfg.expert_hidden_size, cfg.min_period, cfg.max_period)
                v_t = m.denoise_step(pads, keys, values, m.expert_prefix_kv(keys, values), x_t, te.float().to(self.device))
                report.compare("denoise.v_t", v_t, dump["denoise"]["v_t"])
        chunk = self._infer(batch, torch.zeros(1, cfg.chunk_size, cfg.max_action_dim, device=self.device))[:, :, : cfg.action_feature_shape[0]]
        if "chunk" in dump["chunk"]:
            report.compare("chunk", chunk, dump["chunk"]["chunk"].reshape(chunk.shape))
        post = self.unnormalizer.unnormalize(chunk, ACTION, "ACTION")
        report.compare("chunk_post", post, dump["chunk"]["chunk_post"].reshape(post.shape))
        return report

    # ------------------------------------------------------------------ request plumbing
    def _resolve_alias(self, camera_alias: dict[str, str] | None) -> dict[str, str]:
        full: dict[str, str] = {}
        for src, dst in (camera_alias or {}).items():
            s = src if src.startswith("observation.images.") else f"observation.images.{src}"
            d = dst if dst.startswith("observation.images.") else f"observation.images.{dst}"
            if d not in self.config.image_features:
                raise ValueError(f"camera_alias target {dst!r} is not an expected image feature")
            if s in self.config.image_features:
                raise ValueError(f"camera_alias source {src!r} is already an expected image feature")
            full[s] = d
        return full

    def _batch_from_frame(self, frame: dict[str, Any]) -> dict[str, torch.Tensor]:
        """Batch dimension, task tokens, device move, state normalisation (preprocess.py:138-171)."""
        frame = dict(frame)
        for src, dst in self.camera_alias.items():
            if src in frame and dst not in frame:
                frame[dst] = frame.pop(src)
        batch: dict[str, torch.Tensor] = {}
        for key, value in frame.items():
            if key.startswith("observation.") and isinstance(value, torch.Tensor):
                batch[key] = value.unsqueeze(0) if value.ndim in (1, 3) else value
        if OBS_LANGUAGE_TOKENS not in batch:
            task = frame.get("task", "")
            if isinstance(task, str) and not task.endswith("\n"):
                task = f"{task}\n"
            batch[OBS_LANGUAGE_TOKENS], batch[OBS_LANGUAGE_ATTENTION_MASK] = self._task_tokens(task)
        batch = {k: v.to(self.device) for k, v in batch.items()}
        if OBS_STATE in batch:
            batch[OBS_STATE] = self.normalizer.normalize(batch[OBS_STATE], OBS_STATE, "STATE")
        return batch

    def _task_tokens(self, task: str) -> tuple[torch.Tensor, torch.Tensor]:
        """Token ids and mask of a task string, on the device; the last few tasks are kept (a robot
        repeats its task every request), so the tokenizer and two host-to-device copies run once per task."""
        hit = self._token_cache.get(task)
        if hit is None:
            ids, mask = self.tokenizer.encode_task(task)
            hit = (ids.to(self.device), mask.to(self.device))
            if len(self._token_cache) >= 8:
                self._token_cache.pop(next(iter(self._token_cache)))
            self._token_cache[task] = hit
        return hit

    def _mask(self, batch_size: int, value: bool) -> torch.Tensor:
        """A cached all-true / all-false image mask (never written to)."""
        key = (batch_size, value)
        if key not in self._mask_cache:
            self._mask_cache[key] = torch.full((batch_size,), value, dtype=torch.bool, device=self.device)
        return self._mask_cache[key]

    def prepare_images01(self, batch: dict[str, torch.Tensor]):
        """Camera images resized (left/top pad) to the model resolution, still in [0, 1], and their
        masks; configured cameras the frame lacks become black-after-scaling images with a false mask,
        up to ``empty_cameras`` of them (policy.py:117-163)."""
        w, h = self.config.resize_imgs_with_padding
        present = [k for k in self.config.image_features if k in batch]
        if not present:
            raise ValueError(f"All image features are missing from the batch (expected {self.config.image_features})")
        images = [resize_with_pad(batch[key], h, w, pad_value=0) for key in present]
        masks = [self._mask(img.shape[0], True) for img in images]
        missing = len(self.config.image_features) - len(present)
        for _ in range(min(missing, self.config.empty_cameras)):
            images.append(torch.zeros_like(images[-1]))  # 0 * 2 - 1 = -1: the reference's filler value
            masks.append(self._mask(images[-1].shape[0], False))
        return images, masks

    @staticmethod
    def _to_model_range(images01):
        return [img * 2.0 - 1.0 for img in images01]

    def prepare_images(self, batch: dict[str, torch.Tensor]):
        """:meth:`prepare_images01` scaled to the tower's [-1, 1] input range."""
        images01, masks = self.prepare_images01(batch)
        return self._to_model_range(images01), masks

    def _core(self, images01, img_masks, lang_tokens, lang_masks, state, noise) -> torch.Tensor:
        """The unit a graph records: input scaling and the whole model."""
        return self.model.sample_actions(images01, img_masks, lang_tokens, lang_masks, state, noise, image_range01=True)

    def prepare_state(self, batch: dict[str, torch.Tensor]) -> torch.Tensor:
        state = batch[OBS_STATE]
        if state.shape[-1] < self.config.max_state_dim:
            state = F.pad(state, (0, self.config.max_state_dim - state.shape[-1]))
        return state

    def _infer(self, batch: dict[str, torch.Tensor], noise: torch.Tensor | None) -> torch.Tensor:
        images, img_masks = self.prepare_images01(batch)
        tokens, lang_masks = batch[OBS_LANGUAGE_TOKENS], batch[OBS_LANGUAGE_ATTENTION_MASK]
        if self.graph_enabled and self._graph_runner:
            entry = None
            try:
                entry = self._graph_runner.entry((len(images),))
            except Exception as e:  # noqa: BLE001 - unseen shape that cannot be captured: eager for this request
                if not self._graph_fallback_warned:
                    log.warning(f"graph replay skipped ({e}); falling back to eager for this request")
                    self._graph_fallback_warned = True
            if entry is not None:  # state and noise at the frame's widths: the static tensors hold the zero padding
                return self._run_graph(entry, images, img_masks, tokens, lang_masks, batch[OBS_STATE], noise)
        noise = self._sample_noise() if noise is None else self._pad_noise(noise)
        return self._core(images, img_masks, tokens, lang_masks, self.prepare_state(batch), noise)

    # ------------------------------------------------------------------ hipGraph path
    def _prefix_len_for(self, n_cams: int) -> int:
        return n_cams * self.config.vlm_config.image_seq_len + self.config.tokenizer_max_length + 1

    def _capture_graph(self, key, request=None) -> StaticCall:
        """Record the whole inference core once for ``key = (n_cams,)`` (the reference records the same
        unit: tybok/policies/smolvla/engine.py:408-472).  Static tensors are named after the keyword
        arguments of ``SmolVLAModel.sample_actions``."""
        cfg, dev, n_cams = self.config, self.device, int(key[0])
        width, height = cfg.resize_imgs_with_padding
        f32 = dict(dtype=torch.float32, device=dev)
        call = StaticCall(
            torch.zeros(1, cfg.chunk_size, cfg.max_action_dim, **f32),
            images01=[torch.zeros(1, 3, height, width, **f32) for _ in range(n_cams)],
            img_masks=[torch.ones(1, dtype=torch.bool, device=dev) for _ in range(n_cams)],
            lang_tokens=torch.zeros(1, cfg.tokenizer_max_length, dtype=torch.long, device=dev),
            lang_masks=torch.ones(1, cfg.tokenizer_max_length, dtype=torch.bool, device=dev),
            state=torch.zeros(1, cfg.max_state_dim, **f32),
            noise=torch.zeros(1, cfg.chunk_size, cfg.max_action_dim, **f32),
        )
        log.info(f"capturing one graph for {n_cams} camera(s) (prefix_len={self._prefix_len_for(n_cams)}, steps={cfg.num_steps})")
        return call.record(self._sess, self._core)

    def _run_graph(self, call: StaticCall, images01, img_masks, tokens, lang_masks, state, noise) -> torch.Tensor:
        """The request's tensors go into the static ones on the input stream (one copy per camera, one for
        the state and one for the noise, each at the frame's width: the static tensors keep the zero padding;
        token ids and masks only when they are not the cached objects stored last time), then the replay.  Returns the graph's static output: every caller is done with it, or has
        copied it, before the next request replays."""
        with self._graph_runner.copy_inputs():
            call.store(images01=images01)
            call.store_leading(state=state)
            call.store_owned(img_masks=img_masks)  # always the engine's cached all-true / all-false masks
            # token ids and masks: skipped only when they are the engine's own cached pair for the task; a
            # frame that carries its own token tensors may change them in place between requests
            if any(tokens is t and lang_masks is m for t, m in self._token_cache.values()):
                call.store_owned(lang_tokens=tokens, lang_masks=lang_masks)
            else:
                call.store(lang_tokens=tokens, lang_masks=lang_masks)
                call.forget_owned("lang_tokens", "lang_masks")
            if noise is None:
                self._sample_noise(out=call.inputs["noise"])  # drawn outside the graph, from the engine's generator
                call.forget_leading("noise")
            else:
                call.store_leading(noise=noise)
        self._graph_runner.wait_inputs()
        return call.replay(copy=False)
