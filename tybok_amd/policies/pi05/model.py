"""pi0.5 flow-matching model on one MI355X.

Same computation as the reference's ``PI05FlowMatching`` + ``PaliGemmaWithExpertModel`` +
``GemmaDecoder`` (tybok/policies/pi05/models/flow_matching.py:261-838,
tybok/policies/pi05/models/paligemma_with_expert.py:129-276, tybok/policies/pi05/models/gemma.py,
tybok/policies/pi05/models/layers.py), with the reference's seams wired to the HIP kernels:

* ``fp8_expert_mlp`` / ``fp8_llm_mlp``  -- the GeGLU FFN of the expert / VLM layers runs as
  ``tk_fp8w_gated_ffn`` on e4m3fn weights; for the expert the AdaRMS gated residual
  ``x + y * gate`` is fused into the down projection's epilogue (the seam of
  ``_forward_fp8_mlp`` / ``make_fp8_mlp_forward``: layers.py:397-419, triton_prefill_mlp.py:145-166);
* ``fused_expert``  -- the denoising attention over ``[prefix KV; suffix]`` runs as
  ``tk_expert_attn`` with bf16 logits (the seam of ``_forward_fused_attn``: layers.py:330-371).

The per-step AdaRMS modulations ``dense(time_mlp(time_emb))`` depend only on the step index and
are computed once (the reference's static path does the same: flow_matching.py:321-358).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F  # noqa: N812

from ... import ops as tk
from ..smolvla.model import GatedMLP, sinusoidal_time_embedding
from .config import PI05Config
from .weights import EXP, PROJ, VIS, VLM

BF16 = torch.bfloat16
EPS = 1e-6
MASK_VALUE = -2.3819763e38  # additive mask of the openpi attention
_ROPE_POSITIONS = 2048


def gemma_norm(x: torch.Tensor, weight: torch.Tensor | None = None, modulation: torch.Tensor | None = None):
    """Gemma RMSNorm (``* (1 + w)``) or AdaRMS (``* (1 + scale) + shift``, returns the gate) -- layers.py:51-84."""
    dim = x.shape[-1]
    var = torch.mean(torch.square(x.float()), dim=-1, keepdim=True)
    normed = x * torch.rsqrt(var + EPS)
    if modulation is None:
        return (normed * (1.0 + weight.float())).to(x.dtype), None
    mod = modulation.unsqueeze(1) if (x.dim() == 3 and modulation.dim() == 2) else modulation
    if mod.shape[-1] == 2 * dim:
        scale, shift = mod.chunk(2, dim=-1)
        return (normed * (1 + scale.float()) + shift.float()).to(x.dtype), None
    scale, shift, gate = mod.chunk(3, dim=-1)
    return (normed * (1 + scale.float()) + shift.float()).to(x.dtype), gate.to(x.dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``x [B,H,L,D]`` rotated in its own dtype with ``cos/sin [B,L,D]`` (rope.py:44-75)."""
    half = x.shape[-1] // 2
    rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return x * cos.unsqueeze(1) + rot * sin.unsqueeze(1)


def attention_core(q, k, v, add_mask, scaling: float) -> torch.Tensor:
    """bf16 logits, fp32 softmax (layers.py:179-191): ``q [B,H,Lq,D]``, ``k/v [B,G,Lk,D]`` -> ``[B,Lq,H*D]``."""
    b, h, lq, d = q.shape
    g = k.shape[1]
    if h != g:
        k = k[:, :, None].expand(b, g, h // g, k.shape[2], d).reshape(b, h, k.shape[2], d)
        v = v[:, :, None].expand(b, g, h // g, v.shape[2], d).reshape(b, h, v.shape[2], d)
    logits = torch.matmul(q, k.transpose(2, 3)) * scaling + add_mask
    probs = F.softmax(logits, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.matmul(probs, v).transpose(1, 2).reshape(b, lq, h * d)


class PI05Model:
    def __init__(
        self,
        cfg: PI05Config,
        state_dict: dict[str, torch.Tensor],
        device: str | torch.device,
        *,
        fused_expert: bool = False,
        fp8_expert_mlp: bool = False,
        fp8_llm_mlp: bool = False,
        fp8_llm_act: bool = False,
        fused_prefill: bool = False,
        vit_mlp_dtype: torch.dtype | None = None,
        vit_lowp_attn: bool = False,
    ):
        self.cfg = cfg
        self.vit_mlp_dtype = vit_mlp_dtype
        self.vit_lowp_attn = bool(vit_lowp_attn)
        self.device = torch.device(device)
        self.fused_expert = bool(fused_expert)
        self.fp8_expert_mlp = bool(fp8_expert_mlp)
        self.fp8_llm_mlp = bool(fp8_llm_mlp)
        # W8A8: the VLM MLP's activations are quantised per token as well and the products run on the fp8 matrix
        # instruction -- what the reference's fp8 prefill tier computes (tybok/policies/pi05/models/triton_prefill_mlp.py:145-166)
        self.fp8_llm_act = bool(fp8_llm_act) and self.fp8_llm_mlp
        self.fused_prefill = bool(fused_prefill)
        # request-shape flags the engine sets (tybok/policies/pi05/models/flow_matching.py:279-285)
        self.pad_free = False
        self.skip_empty_images = False
        self.tokenizer_max_length = int(cfg.tokenizer_max_length)
        self.use_hip = self.fused_expert or self.fp8_expert_mlp or self.fp8_llm_mlp or self.fused_prefill or self.vit_lowp_attn
        if self.use_hip and self.device.type != "cuda":
            raise RuntimeError("the fused / fp8 tiers run HIP kernels and need a GPU device")
        self.vd, self.ed = cfg.paligemma_dims, cfg.expert_dims
        self.depth = self.vd["depth"]
        self.head_dim = self.vd["head_dim"]
        mlp_keys = tuple(f".mlp.{p}_proj.weight" for p in ("gate", "up", "down"))
        self.p = {k: v.to(self.device) for k, v in state_dict.items() if not k.endswith(mlp_keys)}
        self.vlm_mlp = [GatedMLP(state_dict, f"{VLM}layers.{i}.mlp.", self.device, self.fp8_llm_mlp, act="gelu_tanh", w8a8=self.fp8_llm_act) for i in range(self.depth)]
        self.exp_mlp = [GatedMLP(state_dict, f"{EXP}layers.{i}.mlp.", self.device, self.fp8_expert_mlp, act="gelu_tanh") for i in range(self.ed["depth"])]
        self.ws = tk.default_workspace(self.device) if self.use_hip else None
        self.vt_suf = None  # zero-padded V^T of the action tokens, allocated on first use

        inv = 1.0 / (10000.0 ** (torch.arange(0, self.head_dim, 2, dtype=torch.int64).float() / self.head_dim))
        inv = inv.to(BF16).float()  # the reference's inverse frequencies go through a bf16 buffer
        freqs = torch.arange(_ROPE_POSITIONS, dtype=torch.float32)[:, None] * inv[None, :]
        emb = torch.cat([freqs, freqs], dim=-1)
        self.rope_cos, self.rope_sin = emb.cos().to(self.device), emb.sin().to(self.device)
        half = self.head_dim // 2

        def pack_stack(stack: str, depth: int):
            qkv, o = [], []
            for i in range(depth):
                lp = f"{stack}layers.{i}.self_attn."
                w = torch.cat([self.p[lp + n + "_proj.weight"] for n in "qkv"], dim=0).to(BF16)
                qkv.append(tk.pack_bf16_weight(w, rope_half=half))
                o.append(tk.pack_bf16_weight(self.p[lp + "o_proj.weight"].to(BF16)))
            return qkv, o

        if self.fused_expert or self.fused_prefill:
            # the fused rotary epilogue reads fp32 tables holding the bf16 values the eager path uses
            self.rope_tables_hip = tk.RopeTables(
                self.rope_cos[:, :half].to(BF16).float().contiguous(), self.rope_sin[:, :half].to(BF16).float().contiguous()
            )
        if self.fused_expert:
            self.exp_qkv, self.exp_o = pack_stack(EXP, self.ed["depth"])
        if self.fused_prefill:
            self.vlm_qkv, self.vlm_o = pack_stack(VLM, self.depth)
            # Gemma RMSNorm x * rstd * (1 + w) is the adaptive norm with scale = w and shift = 0
            zeros = torch.zeros(self.vd["width"], dtype=torch.float32, device=self.device)
            self.vlm_norms = [
                tuple((self.p[f"{VLM}layers.{i}.{n}.weight"].float().contiguous(), zeros) for n in ("input_layernorm", "post_attention_layernorm"))
                for i in range(self.depth)
            ]
        self.embed_scale = torch.tensor(self.vd["width"] ** 0.5, dtype=BF16, device=self.device)
        self._embed_scale_value = float(torch.tensor(self.vd["width"] ** 0.5, dtype=BF16))  # the same bf16-rounded factor, on the host
        self.patch_w = self.p[VIS + "embeddings.patch_embedding.weight"].reshape(cfg.vision_hidden, -1)
        # low-precision copies of the vision tower's linears (the drift tiers convert weights and bias)
        self.vis_lowp: dict[str, tuple[torch.Tensor, torch.Tensor]] = {}
        # head size the attention kernel runs: the smallest supported one that holds the tower's heads
        self.vis_head_pad = next((d for d in (64, 96, 128, 256) if d >= cfg.vision_hidden // cfg.vision_heads), 0)
        if self.vit_lowp_attn and not self.vis_head_pad:
            raise ValueError("vision heads wider than 256 are not supported by the attention kernel")
        # q|k|v of the fused tier run on fp16 operands, as the reference's fused tower does (its q/k/v "need a >= 10-bit
        # mantissa", tybok/policies/pi05/models/triton_vision.py:23-25) -- where the fp16 kernels take the shape (the
        # tower attention kernel at a padded head size of 96 on the GPU); elsewhere bf16
        self.vit_qkv_dtype = torch.float16 if self.device.type == "cuda" and self.vis_head_pad == 96 else BF16
        for i in range(cfg.vision_layers):
            lp = f"{VIS}encoder.layers.{i}."
            if self.vit_mlp_dtype is not None:
                for n in ("mlp.fc1", "mlp.fc2"):
                    self.vis_lowp[lp + n] = (self.p[lp + n + ".weight"].to(self.vit_mlp_dtype), self.p[lp + n + ".bias"].to(self.vit_mlp_dtype))
            if self.vit_lowp_attn:
                # q|k|v as one bf16 GEMM whose output is already the attention kernel's layout: every
                # head padded with zero rows from 72 to 96 columns (zero q/k columns add nothing to the
                # scores, zero value columns give zero outputs that out_proj's zero columns ignore)
                heads, hd, hp = cfg.vision_heads, cfg.vision_hidden // cfg.vision_heads, self.vis_head_pad

                def pad_rows(t: torch.Tensor) -> torch.Tensor:  # [heads * hd, ...] -> [heads * hp, ...]
                    out = torch.zeros(heads, hp, *t.shape[1:], dtype=t.dtype, device=t.device)
                    out[:, :hd] = t.view(heads, hd, *t.shape[1:])
                    return out.view(heads * hp, *t.shape[1:])

                self.vis_lowp[lp + "self_attn.qkv"] = (
                    torch.cat([pad_rows(self.p[lp + f"self_attn.{n}_proj.weight"]) for n in "qkv"], dim=0).to(self.vit_qkv_dtype).contiguous(),
                    torch.cat([pad_rows(self.p[lp + f"self_attn.{n}_proj.bias"]) for n in "qkv"], dim=0).to(self.vit_qkv_dtype).contiguous(),
                )
                self.vis_lowp[lp + "self_attn.out_proj"] = (
                    pad_rows(self.p[lp + "self_attn.out_proj.weight"].t().contiguous()).t().to(BF16).contiguous(),
                    self.p[lp + "self_attn.out_proj.bias"].to(BF16),
                )
        # with both low-precision tiers in bf16 every linear of the tower runs on the many-row MFMA kernel: the
        # same weights in its tile order (shapes it does not take -- K % 16, N % 8 -- stay on the library GEMM)
        self.vis_dense: dict[str, tuple] = {}
        if self.vit_lowp_attn and self.vit_mlp_dtype == BF16 and self.device.type == "cuda" and self.vis_head_pad in (64, 96):
            if all(w.shape[1] % 16 == 0 and w.shape[0] % 8 == 0 for w, _ in self.vis_lowp.values()):
                self.vis_dense = {n: (tk.pack_bf16_weight(w), b.contiguous()) for n, (w, b) in self.vis_lowp.items()}
        elif self.vit_mlp_dtype is not None and not self.vit_lowp_attn and self.device.type == "cuda":
            # the MLP-only tiers: fc1 / fc2 on the many-row kernel in their 16-bit type (bf16 or fp16)
            if all(w.shape[1] % 16 == 0 and w.shape[0] % 8 == 0 for w, _ in self.vis_lowp.values()):
                self.vis_dense = {n: (tk.pack_bf16_weight(w), b.contiguous()) for n, (w, b) in self.vis_lowp.items()}
        self.set_num_steps(cfg.num_steps)

    def lin(self, name: str, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.p[name + ".weight"], self.p.get(name + ".bias"))

    def _modulations_at(self, t: float):
        """AdaRMS modulations of every expert norm at flow time ``t``: per layer ``(input, post_attention)``
        raw ``[1, 3W]`` rows, the final norm's row, and the same split into contiguous (scale fp32, shift
        fp32, gate bf16) vectors for the fused launches (flow_matching.py:505-556)."""
        tt = torch.tensor(float(t), dtype=torch.float32).expand(1)
        te = sinusoidal_time_embedding(tt, self.ed["width"], self.cfg.min_period, self.cfg.max_period).float().to(self.device)
        cond = F.silu(self.lin("time_mlp_out", F.silu(self.lin("time_mlp_in", te))))
        mods = [
            (self.lin(f"{EXP}layers.{i}.input_layernorm.dense", cond), self.lin(f"{EXP}layers.{i}.post_attention_layernorm.dense", cond))
            for i in range(self.ed["depth"])
        ]
        final = self.lin(EXP + "norm.dense", cond)
        w = self.ed["width"]

        def split(mod: torch.Tensor):
            m = mod.reshape(-1).float()
            return m[:w].contiguous(), m[w : 2 * w].contiguous(), m[2 * w :].to(BF16).contiguous()

        return mods, final, [(split(a), split(b)) for a, b in mods], split(final)[:2]

    def set_num_steps(self, n: int) -> None:
        """Per-step AdaRMS modulations of every expert norm (computed on the device, once)."""
        self.num_steps = int(n)
        dt = -1.0 / self.num_steps
        self.mods, self.final_mods, self.mods_split, self.final_split = [], [], [], []
        with torch.inference_mode():
            for step in range(self.num_steps):
                mods, final, mods_split, final_split = self._modulations_at(1.0 + step * dt)
                self.mods.append(mods)
                self.final_mods.append(final)
                self.mods_split.append(mods_split)
                self.final_split.append(final_split)

    def velocity_at(self, prefix_pad, kv, x_t, t: float) -> torch.Tensor:
        """One velocity evaluation at an arbitrary flow time (the per-step tables hold only the Euler
        grid): used by the engine's ``validate`` for the reference's t = 0.5 probe."""
        saved = self.mods, self.final_mods, self.mods_split, self.final_split
        mods, final, mods_split, final_split = self._modulations_at(t)
        self.mods, self.final_mods, self.mods_split, self.final_split = [mods], [final], [mods_split], [final_split]
        try:
            return self.denoise_step(prefix_pad, kv, x_t, 0)
        finally:
            self.mods, self.final_mods, self.mods_split, self.final_split = saved

    def rope_tables(self, pos: torch.Tensor, dtype) -> tuple[torch.Tensor, torch.Tensor]:
        return self.rope_cos[pos].to(dtype), self.rope_sin[pos].to(dtype)

    # ------------------------------------------------------------------ vision + prefix
    def _patch_rows_ok(self, images01) -> bool:
        """One launch can scale and unfold these [0, 1] images: one to four fp32 batch-1 images of one size on the GPU,
        an even patch size that divides them."""
        ps = self.cfg.vision_patch
        first = images01[0]
        return (
            1 <= len(images01) <= 4 and first.is_cuda and ps % 2 == 0 and first.dim() == 4 and first.shape[2] % ps == 0 and first.shape[3] % ps == 0
            and all(i.dtype == torch.float32 and i.shape == first.shape and i.shape[0] == 1 and i.shape[1] == 3 and i.is_contiguous() for i in images01)
        )  # fmt: skip

    def embed_image(self, image: torch.Tensor | None, images01=None) -> torch.Tensor:
        """``[1, 3, 224, 224]`` fp32 in [-1, 1] -> ``[1, 256, vlm_width]`` fp32 (SigLIP tower + projector, fp32).
        ``images01``: a list of batch-1 images still in [0, 1] instead (see :meth:`_patch_rows_ok`): ``x * 2 - 1`` and
        the unfolding of all of them are one launch."""
        cfg, p = self.cfg, self.p
        ps = cfg.vision_patch
        if images01 is not None:
            b = len(images01)
            x = tk.patchify_images(images01, ps, 2.0, -1.0, out_dtype=torch.float32)
        else:
            b = image.shape[0]
            n_h, n_w = image.shape[2] // ps, image.shape[3] // ps
            x = image.float().view(b, 3, n_h, ps, n_w, ps).permute(0, 2, 4, 1, 3, 5).reshape(b, n_h * n_w, 3 * ps * ps)
        x = F.linear(x, self.patch_w, p[VIS + "embeddings.patch_embedding.bias"])
        x = x + p[VIS + "embeddings.position_embedding.weight"][None]
        vh, heads = cfg.vision_hidden, cfg.vision_heads
        hd = vh // heads
        if self.vit_lowp_attn and self.vit_mlp_dtype == BF16 and x.is_cuda and self.vis_head_pad in (64, 96):
            return self._tower_bf16_linears(x.contiguous())
        for i in range(cfg.vision_layers):
            lp = f"{VIS}encoder.layers.{i}."
            if self.vit_lowp_attn:
                # LayerNorm + cast in one launch, bf16 projections (one packed q|k|v GEMM), then the HIP
                # attention, one problem per image: fp32 scores and softmax, probabilities rounded to bf16
                # for P.V (fp32 accumulate)
                hp = self.vis_head_pad
                h = tk.layer_norm(x, p[lp + "layer_norm1.weight"], p[lp + "layer_norm1.bias"], EPS, out_dtype=self.vit_qkv_dtype)
                qkv = F.linear(h, *self.vis_lowp[lp + "self_attn.qkv"]).view(b, -1, 3, heads, hp)
                vt = tk.transpose_v(qkv[:, :, 2]) if hp in (64, 96) else qkv[:, :, 2].permute(0, 2, 3, 1).contiguous()
                a = tk.batched_attn(qkv[:, :, 0], qkv[:, :, 1], vt, scale=hd**-0.5, ws=self.ws)
                x = x + F.linear(a, *self.vis_lowp[lp + "self_attn.out_proj"])  # fp32 + bf16: promoted inside the add
            else:
                h = F.layer_norm(x, (vh,), p[lp + "layer_norm1.weight"], p[lp + "layer_norm1.bias"], EPS)
                q = self.lin(lp + "self_attn.q_proj", h).view(b, -1, heads, hd).transpose(1, 2)
                k = self.lin(lp + "self_attn.k_proj", h).view(b, -1, heads, hd).transpose(1, 2)
                v = self.lin(lp + "self_attn.v_proj", h).view(b, -1, heads, hd).transpose(1, 2)
                att = torch.softmax(torch.matmul(q, k.transpose(2, 3)) * hd**-0.5, dim=-1)
                a = torch.matmul(att, v).transpose(1, 2).reshape(b, -1, vh)
                x = x + self.lin(lp + "self_attn.out_proj", a)
            if self.vit_mlp_dtype is not None:
                # MLP-only low precision: fc1, gelu and fc2 in that dtype, cast at the boundary (for bf16 on a
                # GPU the LayerNorm and the cast are one launch)
                if x.is_cuda:
                    h = tk.layer_norm(x, p[lp + "layer_norm2.weight"], p[lp + "layer_norm2.bias"], EPS, out_dtype=self.vit_mlp_dtype)
                else:
                    h = F.layer_norm(x, (vh,), p[lp + "layer_norm2.weight"], p[lp + "layer_norm2.bias"], EPS).to(self.vit_mlp_dtype)
                if self.vis_dense and not self.vit_lowp_attn:
                    # fc1 with the tanh-GELU on its 16-bit output (gelu(fc1(h)) on 16-bit tensors), then fc2: two
                    # launches of the many-row kernel in the tier's type
                    w1, b1 = self.vis_dense[lp + "mlp.fc1"]
                    w2, b2 = self.vis_dense[lp + "mlp.fc2"]
                    m = tk.bf16w_dense(h.view(-1, vh), w1, b1, "gelu_tanh", ws=self.ws)
                    x = x + tk.bf16w_dense(m, w2, b2, ws=self.ws).view(x.shape)  # fp32 + 16-bit: promoted inside the add
                else:
                    m = F.gelu(F.linear(h, *self.vis_lowp[lp + "mlp.fc1"]), approximate="tanh")
                    x = x + F.linear(m, *self.vis_lowp[lp + "mlp.fc2"])  # fp32 + low precision: promoted inside the add
            else:
                h = F.layer_norm(x, (vh,), p[lp + "layer_norm2.weight"], p[lp + "layer_norm2.bias"], EPS)
                x = x + self.lin(lp + "mlp.fc2", F.gelu(self.lin(lp + "mlp.fc1", h), approximate="tanh"))
        x = F.layer_norm(x, (vh,), p[VIS + "post_layernorm.weight"], p[VIS + "post_layernorm.bias"], EPS)
        return self.lin(PROJ, x)

    def _tower_bf16_linears(self, x: torch.Tensor) -> torch.Tensor:
        """The fused tower (``tl_fused_vit``), after the reference's (tybok/policies/pi05/models/vision.py:120-173,
        237-273; triton_vision.py): q|k|v and the attention on fp16 operands (fp32 scores and softmax, probabilities
        rounded to fp16 for P.V, bf16 attention output), out_proj / fc1 / fc2 on bf16 operands with the GELU on fc1's
        fp32 pre-activation; fp32 residual stream updated in place, each residual add in the launch of the LayerNorm
        that follows it.  Two things are rounded once more than there: the out_proj and fc2 results pass through bf16
        before they join the fp32 residual stream (the reference's kernels add the residual to the fp32 accumulator),
        and the post-LayerNorm + projector stay the fp32 pair of the unfused tower (its fused projector runs bf16
        operands)."""
        cfg, p = self.cfg, self.p
        b, vh, heads, hp = x.shape[0], cfg.vision_hidden, cfg.vision_heads, self.vis_head_pad
        hd = vh // heads
        ln = lambda i, n: (p[f"{VIS}encoder.layers.{i}.layer_norm{n}.weight"], p[f"{VIS}encoder.layers.{i}.layer_norm{n}.bias"])  # noqa: E731
        qdt = self.vit_qkv_dtype
        h = tk.layer_norm(x, *ln(0, 1), EPS, out_dtype=qdt)

        def dense(name: str, t: torch.Tensor, act: str | None = None) -> torch.Tensor:
            if self.vis_dense:
                w, bias = self.vis_dense[name]
                return tk.bf16w_dense(t.reshape(-1, t.shape[-1]), w, bias, act, ws=self.ws).view(*t.shape[:-1], w.n)
            if act:  # library GEMM with the activation in its epilogue
                return tk.linear_gelu_tanh(t, *self.vis_lowp[name])
            return F.linear(t, *self.vis_lowp[name])

        for i in range(cfg.vision_layers):
            lp = f"{VIS}encoder.layers.{i}."
            tokens = h.shape[1]
            if self.vis_dense and tokens % 32 == 0:
                # V^T for the attention launch written by the projection's epilogue (one launch less per layer)
                w, bias = self.vis_dense[lp + "self_attn.qkv"]
                vt = torch.empty(b, heads, hp, tokens, dtype=qdt, device=h.device)
                qkv = tk.bf16w_dense(h.reshape(-1, h.shape[-1]), w, bias, vt_out=vt, vt_col0=2 * heads * hp, ws=self.ws).view(b, -1, 3, heads, hp)
            else:
                qkv = dense(lp + "self_attn.qkv", h).view(b, -1, 3, heads, hp)
                vt = tk.transpose_v(qkv[:, :, 2])
            a = tk.batched_attn(qkv[:, :, 0], qkv[:, :, 1], vt, scale=hd**-0.5, ws=self.ws)
            x, h = tk.add_layer_norm(x, dense(lp + "self_attn.out_proj", a), *ln(i, 2), EPS)
            # fc1's GELU on the fp32 pre-activation, the activation rounded to bf16 for fc2: the reference's fused MLP
            # (`_vision_mlp_up_kernel`, tybok/policies/pi05/models/triton_vision.py:113-187)
            m = dense(lp + "mlp.fc2", dense(lp + "mlp.fc1", h, "gelu_tanh_fp32"))
            if i + 1 < cfg.vision_layers:
                x, h = tk.add_layer_norm(x, m, *ln(i + 1, 1), EPS, out_dtype=qdt)
            else:
                x = x + m
        x = F.layer_norm(x, (vh,), p[VIS + "post_layernorm.weight"], p[VIS + "post_layernorm.bias"], EPS)
        return self.lin(PROJ, x)

    LANG_BUCKET = 16

    def packed_lang_len(self, n_live: int) -> int:
        """Language length ``pad_free`` packs ``n_live`` live tokens into: the next multiple of ``LANG_BUCKET``,
        at most the tokenizer's length, so that the number of distinct request shapes stays bounded
        (tybok/policies/pi05/models/flow_matching.py:727-737)."""
        if not self.pad_free:
            return self.tokenizer_max_length
        bucketed = (int(n_live) + self.LANG_BUCKET - 1) // self.LANG_BUCKET * self.LANG_BUCKET
        return min(bucketed, self.tokenizer_max_length)

    def pack_language(self, tokens: torch.Tensor, masks: torch.Tensor):
        """The language block on the bucket grid: the live tokens, then zero ids with False masks up to the bucket
        (flow_matching.py:739-760).  Needs the live count on the host, so never under graph capture."""
        if not self.pad_free:
            return tokens, masks
        lang_len = self.packed_lang_len(int(masks.sum().item()))
        if tokens.shape[1] == lang_len and masks.shape[1] == lang_len:
            return tokens, masks
        tokens_packed = torch.zeros(tokens.shape[0], lang_len, dtype=tokens.dtype, device=tokens.device)
        masks_packed = torch.zeros(masks.shape[0], lang_len, dtype=masks.dtype, device=masks.device)
        keep = min(lang_len, int(tokens.shape[1]))
        tokens_packed[:, :keep] = tokens[:, :keep]
        masks_packed[:, :keep] = masks[:, :keep]
        return tokens_packed, masks_packed

    def embed_prefix(self, images, img_masks, tokens, masks):
        """-> ``(embs fp32 [1,P,W], pad_masks [1,P])``; every prefix token attends to every valid one."""
        embs, pads = [], []
        capturing = self.device.type == "cuda" and torch.cuda.is_current_stream_capturing()
        if self.skip_empty_images and not capturing and not all(bool(m.all()) for m in img_masks):
            # eager path only (the check reads the masks on the host): a masked-out slot behind a real camera skips
            # the vision tower and contributes zero rows -- it is pad-masked out of every attention, so nothing of
            # it reaches the chunk (flow_matching.py:415-437).  The cameras that remain go through the tower one at
            # a time here and in one batch otherwise; the HIP linears pick tiles by row count, so their embeddings
            # can differ in summation order (bf16 noise).  An empty slot in front of any real one is embedded
            shape = None
            for img, m in zip(images, img_masks):
                if shape is not None and not bool(m.all()):
                    e = torch.zeros(img.shape[0], *shape, dtype=torch.float32, device=img.device)
                else:
                    e = self.embed_image(img)
                    shape = (e.shape[1], e.shape[2])
                embs.append(e)
                pads.append(m[:, None].expand(e.shape[0], e.shape[1]))
            lang = F.embedding(tokens, self.p[VLM + "embed_tokens.weight"]) * self.embed_scale
            embs.append(lang)
            pads.append(masks)
            return torch.cat(embs, dim=1), torch.cat(pads, dim=1)
        if len(images) > 1 and all(img.shape == images[0].shape for img in images):
            # one pass of the vision tower over all cameras (rows are independent)
            per_image = self.embed_image(torch.cat(list(images), dim=0)).split(images[0].shape[0], dim=0)
        else:
            per_image = [self.embed_image(img) for img in images]
        for e, m in zip(per_image, img_masks):
            embs.append(e)
            pads.append(m[:, None].expand(e.shape[0], e.shape[1]))
        lang = F.embedding(tokens, self.p[VLM + "embed_tokens.weight"]) * self.embed_scale
        embs.append(lang)
        pads.append(masks)
        return torch.cat(embs, dim=1), torch.cat(pads, dim=1)

    def prefix_hidden(self, images01, img_masks, tokens, masks):
        """The prefill's bf16 hidden rows ``[P, W]`` and the pad flags ``[1, P]`` straight from [0, 1] images, for one
        request on the GPU: what ``embed_prefix(images * 2 - 1, ...)`` followed by ``.to(bfloat16)`` gives, with the
        change of range and the unfolding in one launch and the embedding lookup, its scale, the concatenation, the cast
        and the flags in another.  None when a piece does not have the form those launches take."""
        table = self.p[VLM + "embed_tokens.weight"]
        if not (
            self._patch_rows_ok(images01) and tokens.shape[0] == 1 and tokens.dtype == torch.int64 and masks.dtype == torch.bool
            and table.dtype == BF16 and len(img_masks) == len(images01) and all(m.dtype == torch.bool and m.numel() == 1 for m in img_masks)
        ):  # fmt: skip
            return None
        per_all = self.embed_image(None, images01=list(images01))
        if per_all.dtype != torch.float32:
            return None
        hidden, pads = tk.prefix_rows(
            per_all.contiguous(), 1.0, table, tokens[0].contiguous(), self._embed_scale_value, None, cam_flags=img_masks,
            tok_flags=masks[0].contiguous(), out_dtype=BF16,
        )  # fmt: skip
        return hidden[0], pads

    def _attn_proj(self, lp: str, h: torch.Tensor, cos, sin):
        b, length = h.shape[0], h.shape[1]
        q = self.lin(lp + "q_proj", h).view(b, length, -1, self.head_dim).transpose(1, 2)
        k = self.lin(lp + "k_proj", h).view(b, length, -1, self.head_dim).transpose(1, 2)
        v = self.lin(lp + "v_proj", h).view(b, length, -1, self.head_dim).transpose(1, 2)
        return apply_rope(q, cos, sin), apply_rope(k, cos, sin), v

    def prefill(self, embs: torch.Tensor, pad_masks: torch.Tensor):
        """VLM prefill -> per-layer post-RoPE ``(K, V)`` bf16 ``[1, G, P, D]``."""
        mask = pad_masks[:, None, :] & pad_masks[:, :, None]
        add = torch.where(mask[:, None], 0.0, MASK_VALUE)
        pos = torch.cumsum(pad_masks, dim=1) - 1
        hidden = embs.to(BF16)
        cos, sin = self.rope_tables(pos, hidden.dtype)
        kv = []
        scaling = self.head_dim**-0.5
        for i in range(self.depth):
            lp = f"{VLM}layers.{i}."
            h, _ = gemma_norm(hidden, weight=self.p[lp + "input_layernorm.weight"])
            q, k, v = self._attn_proj(lp + "self_attn.", h, cos, sin)
            kv.append((k, v))
            hidden = hidden + self.lin(lp + "self_attn.o_proj", attention_core(q, k, v, add, scaling))
            h, _ = gemma_norm(hidden, weight=self.p[lp + "post_attention_layernorm.weight"])
            hidden = self.vlm_mlp[i](h, hidden)
        return kv

    def prefill_fused(self, embs: torch.Tensor | None, pad_masks: torch.Tensor, hidden: torch.Tensor | None = None, suffix_len: int = 0):
        """VLM prefill on the fused launches (norm + q|k|v + RoPE, attention under the pad x pad mask,
        o_proj + residual, GeGLU FFN) -> ``(kv, caches)``: ``kv`` per-layer ``(K, V) [1, G, P, D]`` views
        of the projection outputs, ``caches`` the same keys with V^T in the attention kernel's layout.
        ``hidden``: the bf16 rows ``[P, W]`` when the caller already has them (``embs`` is then not read).
        ``suffix_len``: also return, as a third value, the rotary positions of that many action tokens behind the
        valid prefix (from the bookkeeping launch that writes the mask and the prefix positions)."""
        p_len = pad_masks.shape[1]
        p_pad = (p_len + 31) // 32 * 32
        heads, g, d = self.vd["num_heads"], self.vd["num_kv_heads"], self.head_dim
        nq, nkv = heads * d, g * d
        # pad x pad visibility bytes and clamp(cumsum(pad) - 1) positions: one launch
        mask2d, pos32, suf_pos = tk.prefix_meta(pad_masks[0].contiguous(), None, _ROPE_POSITIONS, suffix_len)
        qkv_all = torch.empty(self.depth, p_len, nq + 2 * nkv, dtype=BF16, device=self.device)
        vt_all = torch.zeros(self.depth, nkv, p_pad, dtype=BF16, device=self.device)
        if hidden is None:
            hidden = embs[0].to(BF16)
        kv, caches = [], []
        many_rows = p_len >= 256  # the projections on the many-row MFMA kernels
        for i in range(self.depth):
            norm_in, norm_post = self.vlm_norms[i]
            if many_rows:
                # the norm as a launch of its own, then the many-row GEMM with the rotary epilogue (q | k rotated, V^T
                # written beside V): the skinny kernel's launch below, at many rows
                qkv = tk.bf16w_dense_rope(
                    tk.rms_norm_rows(hidden, ada=norm_in, eps=EPS), self.vlm_qkv[i], self.rope_tables_hip, pos32, nq + nkv, rope_bf16=True,
                    vt_out=vt_all[i], vt_col0=nq + nkv, out=qkv_all[i], ws=self.ws,
                )  # fmt: skip
            else:
                qkv = tk.bf16w_linear(
                    hidden, self.vlm_qkv[i], ada=norm_in, eps=EPS, rope=self.rope_tables_hip, rope_pos=pos32, rope_cols=nq + nkv,
                    rope_bf16=True, vt_out=vt_all[i], vt_col0=nq + nkv, out=qkv_all[i], ws=self.ws,
                )  # fmt: skip
            k = qkv[:, nq : nq + nkv].view(p_len, g, d)
            cache = tk.PrefixKV(k, vt_all[i].view(g, d, p_pad))
            att = tk.expert_attn(qkv[:, :nq].view(p_len, heads, d), cache, None, None, tk.MASK_NONE, mask2d=mask2d, logits_bf16=True, ws=self.ws)
            if many_rows:
                out = tk.bf16w_dense(att, self.vlm_o[i], resid=hidden, ws=self.ws)  # bf16(bf16(att . Wo^T) + hidden), as below
            else:
                out = tk.bf16w_linear(att, self.vlm_o[i], resid=hidden, ws=self.ws)
            mlp = self.vlm_mlp[i]
            if mlp.w8a8:
                normed = tk.rms_norm_rows(out, ada=norm_post, eps=EPS)
                hidden = tk.w8a8_gated_ffn(normed, mlp.wgu, mlp.wd, "gelu_tanh", resid=out, ws=self.ws, mode="bf16")
            elif mlp.fp8:
                hidden = tk.fp8w_gated_ffn(out, mlp.wgu, mlp.wd, "gelu_tanh", resid=out, ada=norm_post, eps=EPS, ws=self.ws)
            else:
                h, _ = gemma_norm(out[None], weight=self.p[f"{VLM}layers.{i}.post_attention_layernorm.weight"])
                hidden = mlp(h, out[None])[0]
            kv.append((k.transpose(0, 1)[None], qkv[:, nq + nkv :].view(p_len, g, d).transpose(0, 1)[None]))
            caches.append(cache)
        return (kv, caches, suf_pos) if suffix_len else (kv, caches)

    # ------------------------------------------------------------------ denoising
    def attention_caches(self, kv) -> list:
        """Per-layer prefix K/V in the attention kernel's layout (V transposed), once per request."""
        return [tk.prepare_prefix_kv(k[0].transpose(0, 1), v[0].transpose(0, 1)) for k, v in kv]

    def _denoise_layers_fused(self, prefix_pad, caches, hidden, pos, step: int) -> torch.Tensor:
        """Expert stack on the fused launches (per layer: AdaRMS + q|k|v + RoPE, attention, o_proj with
        gated residual, AdaRMS + GeGLU FFN with gated residual); ``hidden [S, W]`` bf16."""
        heads, d = self.ed["num_heads"], self.head_dim
        g = self.vt_suf.shape[0]
        nq, nkv = heads * d, g * d
        s = hidden.shape[0]
        pos32 = pos if pos.dtype == torch.int32 else pos[0].clamp(0, _ROPE_POSITIONS - 1).to(torch.int32)
        pad = prefix_pad[0]
        for i in range(self.ed["depth"]):
            (sc_in, sh_in, gate_in), (sc_post, sh_post, gate_post) = self.mods_split[step][i]
            qkv = tk.bf16w_linear(
                hidden, self.exp_qkv[i], ada=(sc_in, sh_in), eps=EPS, rope=self.rope_tables_hip, rope_pos=pos32,
                rope_cols=nq + nkv, rope_bf16=True, vt_out=self.vt_suf.view(nkv, -1), vt_col0=nq + nkv, ws=self.ws,
            )  # fmt: skip
            suffix = tk.SuffixKV(qkv[:, nq : nq + nkv].view(s, g, d), self.vt_suf)
            att = tk.expert_attn(qkv[:, :nq].view(s, heads, d), caches[i], suffix, pad, tk.MASK_BIDIR, logits_bf16=True, ws=self.ws)
            hidden = tk.bf16w_linear(att, self.exp_o[i], resid=hidden, gate=gate_in, ws=self.ws)
            mlp = self.exp_mlp[i]
            # the adaptive norm as the gate/up launch's prologue: eight waves per block, every round of the short K in
            # flight, the row statistics taken from the staged pieces (no second pass over the rows)
            hidden = tk.fp8w_gated_ffn(hidden, mlp.wgu, mlp.wd, "gelu_tanh", resid=hidden, gate=gate_post, ada=(sc_post, sh_post), eps=EPS, ws=self.ws)
        return hidden

    def denoise_step(self, prefix_pad, kv, x_t, step: int, caches: list | None = None) -> torch.Tensor:
        """Velocity fp32 ``[1, chunk, max_action_dim]`` at denoising step ``step`` (flow_matching.py:505-556)."""
        hidden = self.lin("action_in_proj", x_t).to(BF16)
        b, s = hidden.shape[0], hidden.shape[1]
        if self.fused_expert:
            if caches is None:
                caches = self.attention_caches(kv)
            if self.vt_suf is None or self.vt_suf.shape[2] < (s + 31) // 32 * 32:
                g = kv[0][0].shape[1]
                self.vt_suf = torch.zeros(g, self.head_dim, (s + 31) // 32 * 32, dtype=BF16, device=self.device)
        p_len = prefix_pad.shape[1]
        pos = prefix_pad.sum(dim=-1)[:, None] + torch.arange(s, device=self.device)[None, :]
        if self.fused_expert and b == 1 and all(m.fp8 for m in self.exp_mlp):
            hidden = self._denoise_layers_fused(prefix_pad, caches, hidden[0], pos, step)
            v, _ = tk.expert_tail(hidden, self.p["action_out_proj.weight"], self.p["action_out_proj.bias"], ada=self.final_split[step], eps=EPS)
            return v[None]
        cos, sin = self.rope_tables(pos, hidden.dtype)
        scaling = self.head_dim**-0.5
        if not self.fused_expert:
            vis = torch.cat([prefix_pad[:, None, :].expand(b, s, p_len), torch.ones(b, s, s, dtype=torch.bool, device=self.device)], dim=2)
            add = torch.where(vis[:, None], 0.0, MASK_VALUE)
        for i in range(self.ed["depth"]):
            lp = f"{EXP}layers.{i}."
            mod_in, mod_post = self.mods[step][i]
            h, gate = gemma_norm(hidden, modulation=mod_in)
            q, k, v = self._attn_proj(lp + "self_attn.", h, cos, sin)
            if self.fused_expert:
                self.vt_suf[:, :, :s].copy_(v[0].transpose(1, 2))
                att = tk.expert_attn(
                    q[0].transpose(0, 1), caches[i], tk.SuffixKV(k[0].transpose(0, 1), self.vt_suf), prefix_pad[0],
                    tk.MASK_BIDIR, logits_bf16=True, ws=self.ws,
                )[None]  # fmt: skip
            else:
                att = attention_core(q, torch.cat([kv[i][0], k], dim=2), torch.cat([kv[i][1], v], dim=2), add, scaling)
            hidden = hidden + self.lin(lp + "self_attn.o_proj", att) * gate
            h, gate = gemma_norm(hidden, modulation=mod_post)
            mlp = self.exp_mlp[i]
            if mlp.fp8:
                y = tk.fp8w_gated_ffn(h.view(b * s, -1), mlp.wgu, mlp.wd, "gelu_tanh", resid=hidden.view(b * s, -1), gate=gate.reshape(-1), ws=self.ws)
                hidden = y.view(b, s, -1)
            else:
                a = F.gelu(F.linear(h, mlp.wg), approximate="tanh") * F.linear(h, mlp.wu)
                hidden = hidden + F.linear(a, mlp.wdn) * gate
        out, _ = gemma_norm(hidden, modulation=self.final_mods[step])
        return self.lin("action_out_proj", out.to(torch.float32))

    def sample_actions(self, images, img_masks, tokens, masks, noise, trace: dict | None = None, image_range01: bool = False) -> torch.Tensor:
        """Prefix embed, prefill, Euler loop -> ``[1, chunk, max_action_dim]`` fp32.  ``image_range01``: the images are
        still in [0, 1] (``x * 2 - 1`` is applied here, inside the unfolding launch where that is possible)."""
        capturing = self.device.type == "cuda" and torch.cuda.is_current_stream_capturing()
        if self.pad_free and not capturing:
            tokens, masks = self.pack_language(tokens, masks)  # (a recorded shape already has the bucket's length)
        fused_loop = self.fused_expert and noise.shape[0] == 1 and noise.dtype == torch.float32 and noise.is_contiguous() and all(m.fp8 for m in self.exp_mlp)
        suffix_len = noise.shape[1] if fused_loop else 0
        caches = suf_pos = direct = None
        if image_range01 and trace is None and self.fused_prefill and (capturing or not self.skip_empty_images):
            direct = self.prefix_hidden(images, img_masks, tokens, masks)
        if direct is not None:
            hidden, pads = direct
            kv, caches, *rest = self.prefill_fused(None, pads, hidden=hidden, suffix_len=suffix_len)
            suf_pos = rest[0] if rest else None
        else:
            if image_range01:
                images = [img * 2.0 - 1.0 for img in images]
            embs, pads = self.embed_prefix(images, img_masks, tokens, masks)
            if self.fused_prefill and embs.shape[0] == 1:
                kv, caches, *rest = self.prefill_fused(embs, pads, suffix_len=suffix_len)
                suf_pos = rest[0] if rest else None
            else:
                kv = self.prefill(embs, pads)
            if trace is not None:
                trace.update(prefix_embs=embs, pad_masks=pads, kv=kv)
        dt = -1.0 / self.num_steps
        x_t = noise
        if caches is None or not self.fused_expert:
            caches = self.attention_caches(kv) if self.fused_expert else None
        if fused_loop:
            # fused loop: positions once per request, Euler update inside the step's last launch
            s = x_t.shape[1]
            if self.vt_suf is None or self.vt_suf.shape[2] < (s + 31) // 32 * 32:
                self.vt_suf = torch.zeros(kv[0][0].shape[1], self.head_dim, (s + 31) // 32 * 32, dtype=BF16, device=self.device)
            # clamp(sum(pad) + arange(s)): from the prefill's bookkeeping launch, or a launch of its own
            pos32 = suf_pos if suf_pos is not None else tk.prefix_meta(pads[0].contiguous(), None, _ROPE_POSITIONS, s, want_mask=False)[2]
            # (`action_in_proj` stays the library's fp32 product + cast, two launches a step: carried in the tail launch
            # of the step before -- tk_expert_tail_embed -- it sums its 32 terms in another order, and that re-draw of
            # a few bf16 roundings moved one frame's maximum error from under to over the cap held for this path)
            for step in range(self.num_steps):
                hidden = self.lin("action_in_proj", x_t)[0].to(BF16)
                hidden = self._denoise_layers_fused(pads, caches, hidden, pos32, step)
                _, x_new = tk.expert_tail(
                    hidden, self.p["action_out_proj.weight"], self.p["action_out_proj.bias"], ada=self.final_split[step], eps=EPS,
                    x_t=x_t[0], dt=dt,
                )  # fmt: skip
                x_t = x_new[None]
            return x_t
        for step in range(self.num_steps):
            x_t = x_t + dt * self.denoise_step(pads, kv, x_t, step, caches)
        return x_t
