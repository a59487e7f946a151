"""SmolVLA flow-matching model on one MI355X.

Same computation as the reference's ``VLAFlowMatching`` + ``SmolVLMWithExpertModel``
(tybok/policies/smolvla/models/flow_matching.py:86-644,
tybok/policies/smolvla/models/vlm_with_expert.py:41-511), with the reference's seams wired to
the HIP kernels of this package:

* ``fp8_expert_mlp`` / ``fp8_llm_mlp``  -- the gated FFN of the expert / VLM layers runs as
  ``tk_fp8w_gated_ffn`` on e4m3fn weights (second residual fused), the seam where the reference
  calls ``triton_norm_gate_up`` + ``down_proj`` (vlm_with_expert.py:391-408);
* ``fused_expert``  -- a denoising expert layer is five launches: input RMSNorm + packed q|k|v
  projection + RoPE (``tk_bf16w_linear``), attention over the cached prefix KV
  (``tk_expert_attn``), o_proj + residual (``tk_bf16w_linear``), and -- with ``fp8_expert_mlp`` --
  post-attention RMSNorm + gate/up, down + residual (``tk_fp8w_norm_gated_ffn``); the seam of
  ``triton_self_attn`` / ``triton_cross_attn`` (vlm_with_expert.py:166-190, 275-297).

Everything else (VLM prefill, vision tower, action/time projections) is plain torch on the GPU.  The model
is capture-clean: every constant is built at construction time, nothing copies from the host or
synchronises inside :meth:`sample_actions`.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F  # noqa: N812

from ... import ops as tk
from ...fp8_checkpoint import SCALE_SUFFIX, dequantize_entry
from ...quant import quantize_weight_rows
from .config import SmolVLAConfig
from .weights import CONNECTOR, EXP, TXT, VIS

BF16 = torch.bfloat16
_ROPE_POSITIONS = 16384


def sinusoidal_time_embedding(time: torch.Tensor, dim: int, min_period: float, max_period: float) -> torch.Tensor:
    """``cat(sin, cos)(2*pi*t/period)`` in float64 (flow_matching.py:27-42)."""
    frac = torch.linspace(0.0, 1.0, dim // 2, dtype=torch.float64)
    period = min_period * (max_period / min_period) ** frac
    ang = (1.0 / period * 2 * math.pi)[None, :] * time.to(torch.float64)[:, None]
    return torch.cat([torch.sin(ang), torch.cos(ang)], dim=1)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Llama RMSNorm: fp32 statistics, cast back, then the weight (layers.py:22-27)."""
    x32 = x.to(torch.float32)
    var = x32.pow(2).mean(-1, keepdim=True)
    return weight * (x32 * torch.rsqrt(var + eps)).to(x.dtype)


def eager_attention(mask: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """fp32-score GQA attention (attention.py:136-187): ``q [B,Lq,H,D]``, ``k/v [B,Lk,G,D]``, bool ``mask [B,Lq,Lk]``."""
    b, lq, h, d = q.shape
    g = k.shape[2]
    rep = h // g
    kf = k[:, :, :, None, :].expand(b, k.shape[1], g, rep, d).reshape(b, k.shape[1], h, d)
    vf = v[:, :, :, None, :].expand(b, v.shape[1], g, rep, d).reshape(b, v.shape[1], h, d)
    scores = torch.matmul(q.float().transpose(1, 2), kf.float().permute(0, 2, 3, 1)) * d**-0.5
    scores = torch.where(mask[:, None], scores, torch.finfo(torch.float32).min)
    probs = F.softmax(scores, dim=-1).to(vf.dtype)
    out = torch.matmul(probs, vf.permute(0, 2, 1, 3))
    return out.permute(0, 2, 1, 3).reshape(b, lq, h * d)


class GatedMLP:
    """gate/up/down of one decoder layer: bf16 torch linears, or fp8 weights on the HIP kernel."""

    def __init__(self, sd: dict, prefix: str, device, fp8: bool, act: str = "silu", w8a8: bool = False):
        self.act = act
        self.fp8 = fp8
        self.w8a8 = bool(w8a8) and fp8  # activations quantised per token too (the W8A8 tier)
        names = [prefix + n + ".weight" for n in ("gate_proj", "up_proj", "down_proj")]

        def codes_and_scale(name: str):
            # an fp8 checkpoint stores the e4m3fn codes with their row scales: used as they are
            w = sd[name]
            if w.dtype == torch.float8_e4m3fn:
                return w.to(device), sd[name[: -len(".weight")] + SCALE_SUFFIX].to(device=device, dtype=torch.float32)
            return quantize_weight_rows(w.to(device))

        if fp8:
            (g8, sg), (u8, su), (d8, sdn) = (codes_and_scale(n) for n in names)
            self.wgu = tk.pack_fp8_gate_up(g8, sg, u8, su)
            self.wd = tk.pack_fp8_weight(d8, sdn)
        else:
            self.wg, self.wu, self.wdn = (
                (dequantize_entry(sd, n) if sd[n].dtype == torch.float8_e4m3fn else sd[n]).to(device) for n in names
            )

    def __call__(self, x: torch.Tensor, resid: torch.Tensor) -> torch.Tensor:
        """``down(act(gate(x)) * up(x)) + resid`` for ``x [B, L, hidden]`` bf16 (in-place add semantics)."""
        if self.fp8:
            b, length, hidden = x.shape
            ffn = tk.w8a8_gated_ffn if self.w8a8 else tk.fp8w_gated_ffn
            y = ffn(x.reshape(b * length, hidden), self.wgu, self.wd, self.act, resid=resid.reshape(b * length, hidden))
            return y.view(b, length, hidden)
        a = F.silu(F.linear(x, self.wg)) if self.act == "silu" else F.gelu(F.linear(x, self.wg), approximate="tanh")
        out = F.linear(a * F.linear(x, self.wu), self.wdn)
        out += resid
        return out


class SmolVLAModel:
    def __init__(
        self,
        cfg: SmolVLAConfig,
        state_dict: dict[str, torch.Tensor],
        device: str | torch.device,
        *,
        fused_expert: bool = False,
        fp8_expert_mlp: bool = False,
        fp8_llm_mlp: bool = False,
        fused_prefill: bool = False,
        fused_vit: bool = False,
        overlap: bool = False,
    ):
        assert cfg.vlm_config is not None
        self.cfg = cfg
        self.device = torch.device(device)
        self.fused_expert = bool(fused_expert)
        self.fp8_expert_mlp = bool(fp8_expert_mlp)
        self.fp8_llm_mlp = bool(fp8_llm_mlp)
        self.fused_prefill = bool(fused_prefill)
        self.fused_vit = bool(fused_vit)
        self.use_hip = self.fused_expert or self.fp8_expert_mlp or self.fp8_llm_mlp or self.fused_prefill or self.fused_vit
        if self.use_hip and self.device.type != "cuda":
            raise RuntimeError("the fused / fp8 tiers run HIP kernels and need a GPU device")
        t = cfg.vlm_config.text_config
        self.heads, self.kv_heads, self.head_dim = t.num_attention_heads, t.num_key_value_heads, t.head_dim
        self.eps = t.rms_norm_eps
        self.num_layers = cfg.num_vlm_layers
        mlp_keys = tuple(f".mlp.{p}_proj.weight" for p in ("gate", "up", "down"))
        # everything except the MLP weights (owned by GatedMLP, possibly as fp8) moves as is
        self.p = {k: v.to(self.device) for k, v in state_dict.items() if not k.endswith(mlp_keys)}
        self.vlm_mlp = [GatedMLP(state_dict, f"{TXT}layers.{i}.mlp.", self.device, self.fp8_llm_mlp) for i in range(self.num_layers)]
        self.exp_mlp = [GatedMLP(state_dict, f"{EXP}layers.{i}.mlp.", self.device, self.fp8_expert_mlp) for i in range(cfg.n_expert_layers)]
        self.ws = tk.default_workspace(self.device) if self.use_hip else None
        # prefill x step-0 overlap (flow_matching.py:455-531): step-0 expert layer i runs on a second
        # stream as soon as prefill layer i has produced its K/V.  Kernels that may run at the same
        # time must not share split-K partials / counters: the side stream has its own workspace.
        self.fuse_cross_q = True  # cross layers: q projection inside the attention launch (tk.cross_attn_fused)
        self.overlap = bool(overlap) and self.fused_prefill and self.fused_expert
        self.side_stream = torch.cuda.Stream(self.device) if self.overlap else None
        self.ws_side = tk.Workspace(self.device) if self.overlap else None
        if self.fused_prefill:
            self.vlm_qkv, self.vlm_o = self._pack_attention_weights(TXT, lambda i: False)
        if self.fused_vit:
            # vision q|k|v as one projection (one GEMM over all cameras' patches instead of three)
            # and every linear of the tower in the tile order of the many-row MFMA kernel
            self.vis_qkv = []
            self.vis_dense: dict[str, tuple] = {}

            def packed(w: torch.Tensor):
                # the many-row kernel takes K % 16 == 0 and N % 8 == 0; another shape stays a plain linear
                return tk.pack_bf16_weight(w) if w.shape[1] % 16 == 0 and w.shape[0] % 8 == 0 else w

            for i in range(cfg.vlm_config.vision_config.num_hidden_layers):
                lp = f"{VIS}encoder.layers.{i}."
                w = torch.cat([self.p[lp + "self_attn." + n + "_proj.weight"] for n in "qkv"], dim=0).contiguous()
                b = torch.cat([self.p[lp + "self_attn." + n + "_proj.bias"] for n in "qkv"], dim=0).contiguous()
                self.vis_qkv.append((packed(w), b))
                for n in ("self_attn.out_proj", "mlp.fc1", "mlp.fc2"):
                    self.vis_dense[lp + n] = (packed(self.p[lp + n + ".weight"]), self.p[lp + n + ".bias"].contiguous())
            pw = self.p[VIS + "embeddings.patch_embedding.weight"]
            self.vis_dense["patch"] = (packed(pw.reshape(pw.shape[0], -1).contiguous()), self.p[VIS + "embeddings.patch_embedding.bias"].contiguous())
            self.vis_dense["connector"] = (packed(self.p[CONNECTOR + ".weight"]), self.p.get(CONNECTOR + ".bias"))
        if self.fused_expert:
            self._pack_expert_projections()
            # V^T of the action tokens [G, D, chunk rounded up to 32]; the projection kernel writes
            # columns < chunk, the zero padding beyond is never touched
            self.vt_suf = torch.zeros(self.kv_heads, self.head_dim, (cfg.chunk_size + 31) // 32 * 32, dtype=BF16, device=self.device)

        # constants (built once: nothing below copies from the host at inference time)
        d_half = self.head_dim // 2
        exponents = (2.0 / (d_half * 2)) * torch.arange(d_half, dtype=torch.float32)
        radians = torch.arange(_ROPE_POSITIONS, dtype=torch.float32)[:, None] / (10_000.0**exponents)[None, :]
        self.rope_sin = torch.sin(radians).to(self.device)
        self.rope_cos = torch.cos(radians).to(self.device)
        self.rope_tables = tk.RopeTables(self.rope_cos, self.rope_sin) if self.fused_expert or self.fused_prefill else None
        self.set_num_steps(cfg.num_steps)
        v = cfg.vlm_config.vision_config
        side = v.image_size // v.patch_size
        self.vis_pos = torch.arange(side * side, device=self.device)
        self._pos0_32 = torch.arange(int(cfg.chunk_size), device=self.device).clamp(0, _ROPE_POSITIONS - 1).to(torch.int32)
        # constants of the prefix for one to four cameras: the state token's pad flag and the attention-block flags (only
        # the state token opens a block); built here because a tensor first written inside a graph capture must not be kept
        self._true11 = torch.ones(1, 1, dtype=torch.bool, device=self.device)
        self._att_const = {}
        for n_cams in range(1, 5):
            p_len = n_cams * (side // cfg.vlm_config.scale_factor) ** 2 + int(cfg.tokenizer_max_length) + 1
            att = torch.zeros(1, p_len, dtype=torch.bool, device=self.device)
            att[:, -1] = True
            self._att_const[p_len] = att
        # pixel shuffle (scale_factor x scale_factor neighbouring tokens side by side in one row) as a permutation of tokens
        sf, seq = cfg.vlm_config.scale_factor, side * side
        tok = torch.arange(seq, device=self.device).view(1, side, side // sf, sf).permute(0, 2, 1, 3)
        self.shuffle_perm = tok.reshape(1, side // sf, side // sf, sf * sf).permute(0, 2, 1, 3).reshape(seq).contiguous()
        # ... and as destination rows of the tower's closing LayerNorm, for up to four cameras: token i of camera c goes
        # where the shuffle puts it (the inverse permutation), so the norm launch writes the shuffled layout itself
        inv = torch.empty_like(self.shuffle_perm)
        inv[self.shuffle_perm] = torch.arange(seq, device=self.device)
        self.shuffle_rows = torch.cat([inv + c * seq for c in range(4)]).to(torch.int32).contiguous()
        # the tower's position embedding repeated for four cameras, as the residual operand of the patch launch
        pos_w = self.p[VIS + "embeddings.position_embedding.weight"]
        self.vis_pos_rows = pos_w[self.vis_pos].repeat(4, 1).contiguous() if self.fused_vit and pos_w.dtype == BF16 else None
        self.img_scale = torch.tensor(t.hidden_size**0.5, dtype=BF16, device=self.device)
        self._img_scale_value = float(torch.tensor(t.hidden_size**0.5, dtype=BF16))  # the same bf16-rounded factor, on the host
        self.patch_w = self.p[VIS + "embeddings.patch_embedding.weight"].reshape(v.hidden_size, -1)

    def set_num_steps(self, n: int) -> None:
        self.num_steps = int(n)
        dt = -1.0 / self.num_steps
        # Euler: one velocity evaluation per step at t = 1 + step * dt.  Heun: two, at t and t + dt
        # (entries 2 * step and 2 * step + 1: tybok/policies/smolvla/models/flow_matching.py:583-644).
        heun = getattr(self.cfg, "sampler", "euler") == "heun"
        times = [1.0 + step * dt + (dt if second else 0.0) for step in range(self.num_steps) for second in ((False, True) if heun else (False,))]
        embs = []
        for time in times:
            t = torch.tensor(time, dtype=torch.float32).expand(1)
            embs.append(sinusoidal_time_embedding(t, self.cfg.expert_hidden_size, self.cfg.min_period, self.cfg.max_period).float())
        self.time_embs = [e.to(self.device) for e in embs]
        if getattr(self, "fused_expert", False):
            # Suffix embedding with its constants folded (exact algebra, evaluated in float64):
            #   mlp_in(cat[in_proj(x), te]) = (Wa Win) x + (Wa b_in + Wt te + b_mlp)
            # so a step embeds the noisy actions with two small GEMMs and one SiLU.
            f64 = lambda name: self.p[name].to(torch.float64)  # noqa: E731
            w_in, b_in = f64("action_in_proj.weight"), f64("action_in_proj.bias")
            w_mlp, b_mlp = f64("action_time_mlp_in.weight"), f64("action_time_mlp_in.bias")
            e = w_in.shape[0]
            w_a, w_t = w_mlp[:, :e], w_mlp[:, e:]
            self.suffix_w = (w_a @ w_in).float().contiguous()
            self.suffix_b = [(w_a @ b_in + w_t @ te[0].to(torch.float64) + b_mlp).float().contiguous() for te in self.time_embs]

    def _pack_attention_weights(self, stack: str, q_only) -> tuple[list, list]:
        """bf16 attention weights of a decoder stack in tile order: q|k|v concatenated (or q alone
        where ``q_only(i)``) in rotary pair order, o_proj in natural order."""
        qkv, o = [], []
        for i in range(self.num_layers):
            lp = f"{stack}layers.{i}.self_attn."
            names = ("q_proj",) if q_only(i) else ("q_proj", "k_proj", "v_proj")
            w = torch.cat([self.p[lp + n + ".weight"] for n in names], dim=0).to(BF16)
            qkv.append(tk.pack_bf16_weight(w, rope_half=self.head_dim // 2))
            o.append(tk.pack_bf16_weight(self.p[lp + "o_proj.weight"].to(BF16)))
        return qkv, o

    def _pack_expert_projections(self) -> None:
        self.exp_qkv, self.exp_o = self._pack_attention_weights(EXP, self.cfg.is_cross_layer)

    # ------------------------------------------------------------------ helpers
    def lin(self, name: str, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.p[name + ".weight"], self.p.get(name + ".bias"))

    def rope(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Half-split RoPE of ``x [B, L, H, D]`` at integer ``positions [B, L]`` (rope.py:51-73)."""
        d_half = x.shape[-1] // 2
        pos = positions.clamp(0, _ROPE_POSITIONS - 1)
        sin = self.rope_sin[pos][..., None, :]
        cos = self.rope_cos[pos][..., None, :]
        x32 = x.to(torch.float32)
        a, b = x32[..., :d_half], x32[..., d_half:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1).to(x.dtype)

    # ------------------------------------------------------------------ vision + prefix
    def _patch_rows_ok(self, images01) -> bool:
        """Whether the images of a request (still in [0, 1]) can go through the one-launch patch unfolding."""
        ps = self.cfg.vlm_config.vision_config.patch_size
        return (
            self.fused_vit and 1 <= len(images01) <= 4 and ps % 8 == 0
            and all(i.is_cuda and i.dtype == torch.float32 and i.is_contiguous() and i.shape == images01[0].shape and i.shape[0] == 1 for i in images01)
            and images01[0].shape[2] % ps == 0 and images01[0].shape[3] % ps == 0
        )  # fmt: skip

    def embed_image(self, image: torch.Tensor | None, images01=None) -> torch.Tensor:
        """``[1, 3, H, W]`` in [-1, 1] -> ``[1, 64, hidden]`` bf16 (vision.py; plain torch).  With ``images01`` (a list
        of ``[1, 3, H, W]`` fp32 images still in [0, 1], see ``_patch_rows_ok``) the scaling to [-1, 1], the cast and
        the unfolding are one launch over all of them."""
        cfg = self.cfg.vlm_config
        v = cfg.vision_config
        p = self.p
        ps = v.patch_size
        if images01 is not None:
            b = len(images01)
            x = tk.patchify_images(images01, ps, 2.0, -1.0)
        else:
            b = image.shape[0]
            n_h, n_w = image.shape[2] // ps, image.shape[3] // ps
            # non-overlapping patch convolution as one GEMM over unfolded patches
            x = image.to(BF16).view(b, 3, n_h, ps, n_w, ps).permute(0, 2, 4, 1, 3, 5).reshape(b, n_h * n_w, 3 * ps * ps)
        pos_added, post, shuffled = False, None, False
        if self.fused_vit:
            w_patch, b_patch = self.vis_dense["patch"]
            rows = b * x.shape[1]
            if not isinstance(w_patch, torch.Tensor) and self.vis_pos_rows is not None and rows <= self.vis_pos_rows.shape[0] and x.shape[1] == self.vis_pos.shape[0]:
                # the position embedding enters as the launch's residual: bf16(pos + bf16(x . W^T + b)), what the add computes
                x = tk.bf16w_dense(x.reshape(rows, -1), w_patch, b_patch, resid=self.vis_pos_rows[:rows], ws=self.ws).view(b, -1, w_patch.n)
                pos_added = True
            else:
                x = self._dense("patch", x)
        else:
            x = F.linear(x, self.patch_w, p[VIS + "embeddings.patch_embedding.bias"])
        if not pos_added:
            x = x + p[VIS + "embeddings.position_embedding.weight"][self.vis_pos][None]
        heads = v.num_attention_heads
        hd = v.hidden_size // heads
        for i in range(v.num_hidden_layers):
            lp = f"{VIS}encoder.layers.{i}."
            if self.fused_vit:
                # each residual add runs in the launch of the LayerNorm that follows it (x is updated in place)
                if i == 0:
                    h = tk.layer_norm(x, p[lp + "layer_norm1.weight"], p[lp + "layer_norm1.bias"], v.layer_norm_eps)
                # packed q|k|v GEMM, then the HIP attention (one problem per camera): q.K^T rounded to
                # bf16 before the fp32 scale and softmax, exactly what the bf16 matmul below produces
                w_qkv, b_qkv = self.vis_qkv[i]
                tokens = h.shape[1]
                if not isinstance(w_qkv, torch.Tensor) and tokens % 32 == 0:
                    # V^T for the attention launch written by the projection's epilogue (one launch less per layer)
                    vt = torch.empty(b, heads, hd, tokens, dtype=h.dtype, device=h.device)
                    qkv = tk.bf16w_dense(h.reshape(-1, h.shape[-1]), w_qkv, b_qkv, vt_out=vt, vt_col0=2 * heads * hd, ws=self.ws).view(b, -1, 3, heads, hd)
                else:
                    qkv = self._dense_w(w_qkv, b_qkv, h).view(b, -1, 3, heads, hd)
                    vt = tk.transpose_v(qkv[:, :, 2])
                a = tk.batched_attn(qkv[:, :, 0], qkv[:, :, 1], vt, logits_bf16=True, ws=self.ws)
                x, h = tk.add_layer_norm(x, self._dense(lp + "self_attn.out_proj", a), p[lp + "layer_norm2.weight"], p[lp + "layer_norm2.bias"], v.layer_norm_eps)
                # fc1's GELU on the bf16-rounded linear output, as gelu(linear(h)) on bf16 tensors computes it
                m = self._dense(lp + "mlp.fc2", self._dense(lp + "mlp.fc1", h, "gelu_tanh"))
                if i + 1 < v.num_hidden_layers:
                    nx = f"{VIS}encoder.layers.{i + 1}."
                    x, h = tk.add_layer_norm(x, m, p[nx + "layer_norm1.weight"], p[nx + "layer_norm1.bias"], v.layer_norm_eps)
                else:  # the last residual add in the launch of the tower's closing LayerNorm (and the pixel shuffle's row moves)
                    shuffled = x.shape[1] == self.shuffle_perm.shape[0] and b * x.shape[1] <= self.shuffle_rows.shape[0]
                    post = tk.add_layer_norm(x, m, p[VIS + "post_layernorm.weight"], p[VIS + "post_layernorm.bias"], v.layer_norm_eps,
                                             y_rows=self.shuffle_rows if shuffled else None)[1]  # fmt: skip
                continue
            h = F.layer_norm(x, (v.hidden_size,), p[lp + "layer_norm1.weight"], p[lp + "layer_norm1.bias"], v.layer_norm_eps)
            q = self.lin(lp + "self_attn.q_proj", h).view(b, -1, heads, hd).transpose(1, 2)
            k = self.lin(lp + "self_attn.k_proj", h).view(b, -1, heads, hd).transpose(1, 2)
            val = self.lin(lp + "self_attn.v_proj", h).view(b, -1, heads, hd).transpose(1, 2)
            att = torch.softmax(torch.matmul(q, k.transpose(2, 3)).float() * hd**-0.5, dim=-1).to(val.dtype)
            a = torch.matmul(att, val).transpose(1, 2).reshape(b, -1, v.hidden_size)
            x = x + self.lin(lp + "self_attn.out_proj", a)
            h = F.layer_norm(x, (v.hidden_size,), p[lp + "layer_norm2.weight"], p[lp + "layer_norm2.bias"], v.layer_norm_eps)
            x = x + self.lin(lp + "mlp.fc2", F.gelu(self.lin(lp + "mlp.fc1", h), approximate="tanh"))
        if post is not None:
            x = post
        else:
            x = F.layer_norm(x, (v.hidden_size,), p[VIS + "post_layernorm.weight"], p[VIS + "post_layernorm.bias"], v.layer_norm_eps)
        s = cfg.scale_factor
        seq, dim = x.shape[1], x.shape[2]
        if self.fused_vit and seq == self.shuffle_perm.shape[0]:
            # the pixel shuffle moves whole token rows: done by the closing norm's launch, or one gather by the token
            # permutation built with the model
            if not shuffled:
                x = torch.index_select(x, 1, self.shuffle_perm)
            return self._dense("connector", x.reshape(b, seq // (s * s), dim * s * s))
        side = int(seq**0.5)
        x = x.view(b, side, side, dim).view(b, side, side // s, dim * s).permute(0, 2, 1, 3)
        x = x.reshape(b, side // s, side // s, dim * s * s).permute(0, 2, 1, 3).reshape(b, seq // (s * s), dim * s * s)
        return self._dense("connector", x.contiguous()) if self.fused_vit else self.lin(CONNECTOR, x)

    def _dense(self, name: str, x: torch.Tensor, act: str | None = None) -> torch.Tensor:
        """A linear of the vision tower on the many-row MFMA kernel; ``x [..., K]`` bf16 -> ``[..., N]`` bf16."""
        w, bias = self.vis_dense[name]
        return self._dense_w(w, bias, x, act)

    def _dense_w(self, w, bias, x: torch.Tensor, act: str | None = None) -> torch.Tensor:
        if isinstance(w, torch.Tensor):  # a shape the many-row kernel does not take: the same arithmetic in torch
            y = F.linear(x, w, bias)
            return F.gelu(y, approximate="tanh") if act else y
        return tk.bf16w_dense(x.reshape(-1, x.shape[-1]), w, bias, act, ws=self.ws).view(*x.shape[:-1], w.n)

    def embed_prefix(self, images, img_masks, lang_tokens, lang_masks, state, image_range01: bool = False):
        """-> ``(embs fp32 [1,P,hidden], pad_masks bool [1,P], att_masks bool [1,P])`` (flow_matching.py:160-257).
        ``image_range01``: the images are still in [0, 1] (``x * 2 - 1`` is applied here, in the patch launch where
        that is possible)."""
        embs, pads = [], []
        stacked = None  # the embeddings of all cameras as one [cameras, tokens, hidden] tensor, when they are batch-1 images
        if image_range01 and self._patch_rows_ok(images):
            raw = self.embed_image(None, images01=list(images))
            table = self.p[TXT + "embed_tokens.weight"]
            p_len = raw.shape[0] * raw.shape[1] + lang_tokens.shape[1] + 1
            if (
                state.shape[0] == 1 and lang_tokens.shape[0] == 1 and p_len in self._att_const and raw.dtype == BF16 and table.dtype == BF16
                and lang_tokens.dtype == torch.int64 and lang_masks.dtype == torch.bool and raw.shape[0] <= 4
                and len(img_masks) == raw.shape[0] and all(m.dtype == torch.bool and m.numel() == 1 for m in img_masks)
            ):  # fmt: skip
                st = self.lin("state_proj", state)
                if st.dtype == torch.float32:
                    # scaling, embedding lookup, casts, concatenation and the pad flags in one launch
                    out, pads = tk.prefix_rows(
                        raw.contiguous(), self._img_scale_value, table, lang_tokens[0].contiguous(), math.sqrt(table.shape[1]), st.contiguous(),
                        cam_flags=img_masks, tok_flags=lang_masks[0].contiguous(),
                    )  # fmt: skip
                    return out, pads, self._att_const[p_len]
            stacked = raw * self.img_scale
            per_image = stacked.split(1, dim=0)
            images = ()
        elif image_range01:
            images = [img * 2.0 - 1.0 for img in images]
        if not images:
            pass
        elif len(images) > 1 and all(img.shape == images[0].shape for img in images):
            # one pass of the vision tower over all cameras: rows are independent, and the tower's
            # GEMMs fill the device three times better than one 1024-patch image at a time
            per_all = self.embed_image(torch.cat(list(images), dim=0)) * self.img_scale
            per_image = per_all.split(images[0].shape[0], dim=0)
            stacked = per_all if images[0].shape[0] == 1 else None
        else:
            per_image = [self.embed_image(img) * self.img_scale for img in images]
        for e, m in zip(per_image, img_masks):
            embs.append(e)
            pads.append(m[:, None].expand(e.shape[0], e.shape[1]))
        lang = F.embedding(lang_tokens, self.p[TXT + "embed_tokens.weight"])
        lang = lang * math.sqrt(lang.shape[-1])
        embs.append(lang)
        pads.append(lang_masks)
        st = self.lin("state_proj", state)[:, None, :]
        p_len = sum(e.shape[1] for e in embs) + 1
        if stacked is not None and lang.shape[0] == 1 and st.shape[0] == 1 and p_len in self._att_const:
            # the three pieces written (and cast) straight into the prefix buffer, the attention-block flags taken from
            # the constants built with the model: 4 launches where concatenation, casts and fills took 10
            n_img = stacked.shape[0] * stacked.shape[1]
            dt = torch.promote_types(torch.promote_types(stacked.dtype, lang.dtype), st.dtype)
            out = torch.empty(1, p_len, st.shape[-1], dtype=dt, device=self.device)
            out[0, :n_img].copy_(stacked.reshape(n_img, -1))
            out[0, n_img : p_len - 1].copy_(lang[0])
            out[0, p_len - 1].copy_(st[0, 0])
            pads.append(self._true11)
            return out, torch.cat(pads, dim=1), self._att_const[p_len]
        embs.append(st)
        pads.append(torch.ones(st.shape[0], 1, dtype=torch.bool, device=self.device))
        embs = torch.cat(embs, dim=1)
        pads = torch.cat(pads, dim=1)
        att = torch.zeros(pads.shape, dtype=torch.bool, device=self.device)
        att[:, -1] = True  # image / language tokens do not attend to the state token
        return embs, pads, att

    @staticmethod
    def make_att_2d_masks(pad_masks: torch.Tensor, att_masks: torch.Tensor) -> torch.Tensor:
        c = torch.cumsum(att_masks, dim=1)
        return (c[:, None, :] <= c[:, :, None]) & (pad_masks[:, None, :] & pad_masks[:, :, None])

    def _layer_tail(self, prefix: str, mlp: GatedMLP, att_out: torch.Tensor, hidden: torch.Tensor) -> torch.Tensor:
        out = self.lin(prefix + "self_attn.o_proj", att_out.to(BF16))
        out += hidden  # first residual; downcasts an fp32 hidden exactly like the reference's in-place add
        h = rms_norm(out, self.p[prefix + "post_attention_layernorm.weight"], self.eps)
        return mlp(h, out)

    def prefill(self, embs, pad_masks, att_masks):
        """VLM prefill -> ``(K, V)`` bf16 ``[layers, 1, P, G, D]`` (post-RoPE prefix cache)."""
        mask = self.make_att_2d_masks(pad_masks, att_masks)
        pos = torch.cumsum(pad_masks, dim=1) - 1
        b, length = embs.shape[0], embs.shape[1]
        keys = torch.empty(self.num_layers, b, length, self.kv_heads, self.head_dim, dtype=BF16, device=self.device)
        values = torch.empty_like(keys)
        hidden = embs
        for i in range(self.num_layers):
            lp = f"{TXT}layers.{i}."
            h = rms_norm(hidden, self.p[lp + "input_layernorm.weight"], self.eps).to(BF16)
            q = self.rope(self.lin(lp + "self_attn.q_proj", h).view(b, length, -1, self.head_dim), pos)
            k = self.rope(self.lin(lp + "self_attn.k_proj", h).view(b, length, -1, self.head_dim), pos)
            v = self.lin(lp + "self_attn.v_proj", h).view(b, length, -1, self.head_dim)
            keys[i].copy_(k)
            values[i].copy_(v)
            att = eager_attention(mask, q, k, v)
            hidden = self._layer_tail(lp, self.vlm_mlp[i], att, hidden)
        return keys, values

    def _prefill_setup(self, embs, pad_masks, att_masks, suffix_len: int = 0) -> dict:
        """Per-request operands of the fused prefill: 2-D visibility bytes, positions (and those of ``suffix_len``
        action tokens, under ``suf_pos``), output buffers.  The bookkeeping is one launch: ``make_att_2d_masks``,
        ``cumsum(pad_masks) - 1`` and ``prefix_pad.sum() + arange(s)`` clamped into the rotary table."""
        p_len = embs.shape[1]
        p_pad = (p_len + 31) // 32 * 32
        nq, nkv = self.heads * self.head_dim, self.kv_heads * self.head_dim
        mask2d, pos32, suf_pos = tk.prefix_meta(pad_masks[0].contiguous(), att_masks[0].contiguous(), _ROPE_POSITIONS, suffix_len)
        qkv_all = torch.empty(self.num_layers, p_len, nq + 2 * nkv, dtype=BF16, device=self.device)
        vt_all = torch.zeros(self.num_layers, nkv, p_pad, dtype=BF16, device=self.device)
        return dict(p_len=p_len, p_pad=p_pad, mask2d=mask2d, pos32=pos32, suf_pos=suf_pos, qkv_all=qkv_all, vt_all=vt_all)

    def _prefill_layer_fused(self, i: int, hidden: torch.Tensor, c: dict) -> torch.Tensor:
        """One VLM layer on the fused launches: norm + q|k|v + RoPE, attention under the 2-D prefix
        mask, o_proj + residual, gated FFN.  Fills ``qkv_all[i]`` / ``vt_all[i]`` (the layer's K/V cache)."""
        h_q, h_kv, d = self.heads, self.kv_heads, self.head_dim
        nq, nkv = h_q * d, h_kv * d
        p_len, p_pad = c["p_len"], c["p_pad"]
        lp = f"{TXT}layers.{i}."
        qkv = tk.bf16w_linear(
            hidden, self.vlm_qkv[i], norm_w=self.p[lp + "input_layernorm.weight"], eps=self.eps, rope=self.rope_tables,
            rope_pos=c["pos32"], rope_cols=nq + nkv, vt_out=c["vt_all"][i], vt_col0=nq + nkv, out=c["qkv_all"][i], ws=self.ws,
        )  # fmt: skip
        cache = tk.PrefixKV(qkv[:, nq : nq + nkv].view(p_len, h_kv, d), c["vt_all"][i].view(h_kv, d, p_pad))
        att = tk.expert_attn(qkv[:, :nq].view(p_len, h_q, d), cache, None, None, tk.MASK_NONE, mask2d=c["mask2d"], ws=self.ws)
        out = tk.bf16w_linear(att, self.vlm_o[i], resid=hidden, ws=self.ws)
        mlp = self.vlm_mlp[i]
        post_w = self.p[lp + "post_attention_layernorm.weight"]
        if mlp.fp8:
            return tk.fp8w_gated_ffn(out, mlp.wgu, mlp.wd, mlp.act, resid=out, norm_w=post_w, eps=self.eps, ws=self.ws)
        return mlp(rms_norm(out, post_w, self.eps)[None], out[None])[0]

    def _prefill_views(self, c: dict):
        """``(K, V, V^T)`` of the fused prefill: K / V ``[layers, 1, P, G, D]`` views of the projection
        outputs, V^T ``[layers, G, D, P rounded up to 32]`` (the attention kernel's value layout)."""
        h_kv, d = self.kv_heads, self.head_dim
        nq, nkv = self.heads * d, h_kv * d
        keys = c["qkv_all"][:, None, :, nq : nq + nkv].unflatten(-1, (h_kv, d))
        values = c["qkv_all"][:, None, :, nq + nkv :].unflatten(-1, (h_kv, d))
        return keys, values, c["vt_all"].view(self.num_layers, h_kv, d, c["p_pad"])

    def prefill_fused(self, embs, pad_masks, att_masks, suffix_len: int = 0):
        """VLM prefill on the fused launches -> ``(K, V, V^T)`` (see ``_prefill_views``); with ``suffix_len`` also
        the int32 rotary positions of that many action tokens behind the valid prefix, as a fourth item."""
        c = self._prefill_setup(embs, pad_masks, att_masks, suffix_len)
        hidden = embs[0]
        for i in range(self.num_layers):
            hidden = self._prefill_layer_fused(i, hidden, c)
        return (*self._prefill_views(c), c["suf_pos"]) if suffix_len else self._prefill_views(c)

    def _suffix_pos0(self, s: int) -> torch.Tensor:
        """int32 ``[s]`` positions of the action tokens counted from 0 (the cross layers'): ``pos - pos.min()``."""
        if self._pos0_32.shape[0] == s:
            return self._pos0_32  # built with the model: a tensor first written inside a graph capture must not be kept
        return torch.arange(s, device=self.device).clamp(0, _ROPE_POSITIONS - 1).to(torch.int32)

    def _expert_prefix_kv_layer(self, i: int, keys_i, values_i):
        lp = f"{EXP}layers.{i}.self_attn."
        b, length = keys_i.shape[0], keys_i.shape[1]
        ek = self.lin(lp + "k_proj", keys_i.float().reshape(b, length, -1)).view(b, length, -1, self.head_dim)
        ev = self.lin(lp + "v_proj", values_i.float().reshape(b, length, -1)).view(b, length, -1, self.head_dim)
        return ek, ev

    def expert_prefix_kv(self, keys, values):
        """fp32 expert K/V projections of the prefix for the cross layers (flow_matching.py:553-578)."""
        return {i: self._expert_prefix_kv_layer(i, keys[i], values[i]) for i in range(self.num_layers) if self.cfg.is_cross_layer(i)}

    # ------------------------------------------------------------------ denoising
    def embed_suffix(self, x_t: torch.Tensor, time_emb: torch.Tensor) -> torch.Tensor:
        a = self.lin("action_in_proj", x_t)
        te = time_emb[:, None, :].expand_as(a)
        h = self.lin("action_time_mlp_in", torch.cat([a, te], dim=2))
        return self.lin("action_time_mlp_out", F.silu(h))

    def suffix_positions(self, prefix_pad: torch.Tensor, s: int) -> tuple[torch.Tensor, torch.Tensor]:
        """Positions of the action tokens: after the valid prefix (self layers) and from 0 (cross layers)."""
        pos = prefix_pad.sum(dim=-1)[:, None] + torch.arange(s, device=self.device)[None, :]
        pos0 = pos - pos.min(dim=1, keepdim=True).values
        return pos, pos0

    def _cross_cache(self, i: int, keys_i: torch.Tensor, values_i: torch.Tensor):
        """Cross layer ``i``: fp32 expert K/V projection of the prefix ``[P, G, D]`` views, written as the
        attention kernel's hi + lo planes by one launch."""
        lp = f"{EXP}layers.{i}.self_attn."
        return tk.project_prefix_kv(keys_i.flatten(1), values_i.flatten(1), self.p[lp + "k_proj.weight"], self.p[lp + "v_proj.weight"], self.head_dim)

    def attention_caches(self, keys, values, ekv, vt=None) -> list:
        """Per-layer prefix K/V in the attention kernel's layout, once per request: V transposed
        (self layers, bf16 cache; ``vt`` when the prefill already produced it) or K and V^T split
        into bf16 hi + lo planes (cross layers, fp32)."""
        caches = []
        crossed = {}
        if ekv is None:  # projection and operand layout of every cross layer in one launch (16 layers at most each)
            idx = [i for i in range(self.num_layers) if self.cfg.is_cross_layer(i)]
            for c0 in range(0, len(idx), 16):
                part = idx[c0 : c0 + 16]
                lps = [f"{EXP}layers.{i}.self_attn." for i in part]
                planes = tk.project_prefix_kv_layers(
                    [keys[i, 0].flatten(1) for i in part], [values[i, 0].flatten(1) for i in part],
                    [self.p[lp + "k_proj.weight"] for lp in lps], [self.p[lp + "v_proj.weight"] for lp in lps], self.head_dim,
                )  # fmt: skip
                crossed.update(zip(part, planes))
        for i in range(self.num_layers):
            if self.cfg.is_cross_layer(i):
                if ekv is None:
                    caches.append(crossed[i])
                    continue
                ek, ev = ekv[i]
                caches.append(tk.prepare_prefix_kv(ek[0], ev[0]))
            elif vt is not None:
                caches.append(tk.PrefixKV(keys[i, 0], vt[i]))
            else:
                caches.append(tk.prepare_prefix_kv(keys[i, 0], values[i, 0]))
        return caches

    def _cross_fusable(self, hidden: torch.Tensor, cache) -> bool:
        """The one-launch cross layer applies: bf16 hidden rows, head size 64, fp32 (hi + lo) prefix planes
        that one block covers."""
        return (
            self.fuse_cross_q and hidden.dtype == BF16 and self.head_dim == 64 and hidden.shape[1] <= tk.CROSS_FUSED_MAX_K
            and cache.k_lo is not None and cache.k.shape[0] <= tk.CROSS_FUSED_MAX_P
        )  # fmt: skip

    def _denoise_layer_fused(self, i: int, hidden: torch.Tensor, cache, pad, pos32, pos0_32, ws) -> torch.Tensor:
        """Expert layer ``i`` on the fused launches (``hidden [S, E]``: fp32 into layer 0, bf16 after)."""
        h_q, h_kv, d = self.heads, self.kv_heads, self.head_dim
        nq, nkv = h_q * d, h_kv * d
        s = hidden.shape[0]
        lp = f"{EXP}layers.{i}."
        cross = self.cfg.is_cross_layer(i)
        norm_w = self.p[lp + "input_layernorm.weight"]
        if cross and self._cross_fusable(hidden, cache):
            # norm + q projection + RoPE inside the attention launch
            att = tk.cross_attn_fused(hidden, self.exp_qkv[i], norm_w, self.eps, self.rope_tables, pos0_32, cache, pad)
        else:
            qkv = tk.bf16w_linear(
                hidden, self.exp_qkv[i], norm_w=norm_w, eps=self.eps, rope=self.rope_tables,
                rope_pos=pos0_32 if cross else pos32, rope_cols=nq if cross else nq + nkv,
                vt_out=None if cross else self.vt_suf.view(nkv, -1), vt_col0=nq + nkv, ws=ws,
            )  # fmt: skip
            q = qkv[:, :nq].view(s, h_q, d)
            if cross:
                att = tk.expert_attn(q, cache, None, pad, tk.MASK_NONE, ws=ws)
            else:
                suffix = tk.SuffixKV(qkv[:, nq : nq + nkv].view(s, h_kv, d), self.vt_suf)
                att = tk.expert_attn(q, cache, suffix, pad, tk.MASK_CAUSAL, ws=ws)
        out = tk.bf16w_linear(att, self.exp_o[i], resid=hidden, ws=ws)
        mlp = self.exp_mlp[i]
        post_w = self.p[lp + "post_attention_layernorm.weight"]
        if mlp.fp8:
            return tk.fp8w_gated_ffn(out, mlp.wgu, mlp.wd, mlp.act, resid=out, norm_w=post_w, eps=self.eps, ws=ws)
        return mlp(rms_norm(out, post_w, self.eps)[None], out[None])[0]

    def _denoise_step_fused(self, prefix_pad, caches, hidden, pos32, pos0_32):
        """Expert stack on the fused launches; ``hidden [S, E]`` fp32 in, bf16 out."""
        for i in range(self.num_layers):
            hidden = self._denoise_layer_fused(i, hidden, caches[i], prefix_pad[0], pos32, pos0_32, self.ws)
        return hidden

    def fused_euler_step(self, prefix_pad, caches, x_t, step: int, positions, dt: float, want_v: bool = False, h=None, next_step=None):
        """One velocity evaluation on the fused launches (time entry ``step``): folded suffix embedding, expert
        stack, then final norm + action projection + ``x_t + dt * v_t`` in one launch.  ``x_t [1, chunk, A]``
        fp32.  Returns the updated ``x``; with ``want_v`` the pair ``(v_t, x_t + dt * v_t)``.

        ``h``: the first (folded) linear + SiLU of this step's suffix embedding when the previous step's last
        launch already computed it.  ``next_step``: compute it for that time entry from the updated ``x`` in this
        step's last launch; the return value is then ``(x_new, h_next)``."""
        pos32, pos0_32 = positions
        if h is None:
            h = F.silu(F.linear(x_t[0], self.suffix_w, self.suffix_b[step]))
        hidden = F.linear(h, self.p["action_time_mlp_out.weight"], self.p["action_time_mlp_out.bias"])
        hidden = self._denoise_step_fused(prefix_pad, caches, hidden, pos32, pos0_32)
        h_next = None
        if next_step is not None:
            h_next = torch.empty(x_t.shape[1], self.suffix_w.shape[0], dtype=torch.float32, device=x_t.device)
        v, x_new = tk.expert_tail(
            hidden, self.p["action_out_proj.weight"], self.p["action_out_proj.bias"], norm_w=self.p[EXP + "norm.weight"],
            eps=self.eps, x_t=x_t[0], dt=dt, want_v=want_v,
            embed=None if h_next is None else (self.suffix_w, self.suffix_b[next_step], "silu", h_next),
        )  # fmt: skip
        if next_step is not None:
            return x_new[None], h_next
        return (v[None], x_new[None]) if want_v else x_new[None]

    def _fused_embed_ok(self, x_t) -> bool:
        """The step tail can carry the next step's embedding: the padded action width it is built for."""
        return self.suffix_w.is_contiguous() and self.suffix_w.shape[1] == 32 and x_t.shape[-1] == 32

    def denoise_step(self, prefix_pad, keys, values, ekv, x_t, time_emb, positions=None, caches=None):
        """Velocity ``v_t`` fp32 ``[1, chunk, max_action_dim]`` (flow_matching.py:316-350)."""
        hidden = self.embed_suffix(x_t, time_emb)
        b, s = hidden.shape[0], hidden.shape[1]
        p_len = prefix_pad.shape[1]
        pos, pos0 = positions if positions is not None else self.suffix_positions(prefix_pad, s)
        if self.fused_expert and b == 1:
            clamp = lambda t: t[0].clamp(0, _ROPE_POSITIONS - 1).to(torch.int32)  # noqa: E731
            pos32, pos0_32 = (pos, pos0) if pos.dtype == torch.int32 else (clamp(pos), clamp(pos0))
            if caches is None:
                caches = self.attention_caches(keys, values, ekv)
            hidden = self._denoise_step_fused(prefix_pad, caches, hidden[0], pos32, pos0_32)[None]
            out = rms_norm(hidden, self.p[EXP + "norm.weight"], self.eps)
            return self.lin("action_out_proj", out.to(torch.float32))
        causal = torch.ones(s, s, dtype=torch.bool, device=self.device).tril()[None]
        full_mask = torch.cat([prefix_pad[:, None, :].expand(b, s, p_len), causal], dim=2)
        for i in range(self.num_layers):
            lp = f"{EXP}layers.{i}."
            h = rms_norm(hidden, self.p[lp + "input_layernorm.weight"], self.eps).to(BF16)
            q = self.lin(lp + "self_attn.q_proj", h).view(b, s, -1, self.head_dim)
            if not self.cfg.is_cross_layer(i):
                k = self.rope(self.lin(lp + "self_attn.k_proj", h).view(b, s, -1, self.head_dim), pos)
                v = self.lin(lp + "self_attn.v_proj", h).view(b, s, -1, self.head_dim)
                q = self.rope(q, pos)
                att = eager_attention(full_mask, q, torch.cat([keys[i], k], dim=1), torch.cat([values[i], v], dim=1))
            else:
                q = self.rope(q, pos0)
                ek, ev = ekv[i]
                att = eager_attention(prefix_pad[:, None, :].expand(b, s, p_len), q, ek, ev)
            hidden = self._layer_tail(lp, self.exp_mlp[i], att, hidden)
        out = rms_norm(hidden, self.p[EXP + "norm.weight"], self.eps)
        return self.lin("action_out_proj", out.to(torch.float32))

    def _sample_actions_overlapped(self, embs, pads, att, noise) -> torch.Tensor:
        """Same result as the sequential core, bit for bit, with step 0 of the Euler loop hidden inside
        the prefill: the main stream runs prefill layer i and records an event; the side stream waits
        for it, builds layer i's attention cache (cross layers: the fp32 expert K/V projection) and
        runs step-0 expert layer i.  Both are chains of small latency-bound launches that leave most
        of the device idle, so they overlap almost completely.  The streams join before step 1."""
        main, side = torch.cuda.current_stream(), self.side_stream
        dt = -1.0 / self.num_steps
        c = self._prefill_setup(embs, pads, att, noise.shape[1])
        positions = (c["suf_pos"], self._suffix_pos0(noise.shape[1]))
        keys, values, vt = self._prefill_views(c)
        side.wait_stream(main)
        with torch.cuda.stream(side):
            h = F.silu(F.linear(noise[0], self.suffix_w, self.suffix_b[0]))
            hid_s = F.linear(h, self.p["action_time_mlp_out.weight"], self.p["action_time_mlp_out.bias"])
        hidden = embs[0]
        caches: list = [None] * self.num_layers
        for i in range(self.num_layers):
            hidden = self._prefill_layer_fused(i, hidden, c)
            done = torch.cuda.Event()
            done.record(main)
            with torch.cuda.stream(side):
                side.wait_event(done)
                if self.cfg.is_cross_layer(i):
                    caches[i] = self._cross_cache(i, keys[i, 0], values[i, 0])
                else:
                    caches[i] = tk.PrefixKV(keys[i, 0], vt[i])
                hid_s = self._denoise_layer_fused(i, hid_s, caches[i], pads[0], positions[0], positions[1], self.ws_side)
        carry = self._fused_embed_ok(noise) and self.num_steps > 1
        h = torch.empty(noise.shape[1], self.suffix_w.shape[0], dtype=torch.float32, device=noise.device) if carry else None
        with torch.cuda.stream(side):
            _, x_new = tk.expert_tail(
                hid_s, self.p["action_out_proj.weight"], self.p["action_out_proj.bias"], norm_w=self.p[EXP + "norm.weight"],
                eps=self.eps, x_t=noise[0], dt=dt, embed=(self.suffix_w, self.suffix_b[1], "silu", h) if carry else None,
            )  # fmt: skip
        main.wait_stream(side)
        x_t = x_new[None]
        for step in range(1, self.num_steps):
            if carry and step + 1 < self.num_steps:
                x_t, h = self.fused_euler_step(pads, caches, x_t, step, positions, dt, h=h, next_step=step + 1)
            else:
                x_t = self.fused_euler_step(pads, caches, x_t, step, positions, dt, h=h)
        return x_t

    def sample_actions_core(self, embs, pads, att, noise, trace: dict | None = None) -> torch.Tensor:
        if self.overlap and getattr(self.cfg, "sampler", "euler") == "euler" and trace is None and embs.shape[0] == 1 and noise.shape[0] == 1 and noise.dtype == torch.float32 and noise.is_contiguous():
            return self._sample_actions_overlapped(embs, pads, att, noise)
        vt = suf_pos = None
        fused = self.fused_expert and noise.shape[0] == 1
        if self.fused_prefill and embs.shape[0] == 1:
            keys, values, vt, suf_pos = self.prefill_fused(embs, pads, att, noise.shape[1])
        else:
            keys, values = self.prefill(embs, pads, att)
        # the fused tier projects the cross layers' K/V inside attention_caches (one launch per layer)
        ekv = None if fused and trace is None else self.expert_prefix_kv(keys, values)
        if trace is not None:
            trace.update(prefix_embs=embs, pad_masks=pads, keys=keys, values=values, ekv=ekv)
        dt = -1.0 / self.num_steps
        x_t = noise
        if fused and suf_pos is not None:
            positions = (suf_pos, self._suffix_pos0(noise.shape[1]))  # from the prefill's bookkeeping launch
        else:
            positions = self.suffix_positions(pads, noise.shape[1])
            if fused:
                positions = tuple(t[0].clamp(0, _ROPE_POSITIONS - 1).to(torch.int32) for t in positions)
        caches = self.attention_caches(keys, values, ekv, vt) if self.fused_expert and noise.shape[0] == 1 else None
        fused_loop = caches is not None and x_t.dtype == torch.float32 and x_t.is_contiguous()
        if getattr(self.cfg, "sampler", "euler") == "heun":
            # predictor at t, corrector at t + dt, then x <- x + (dt / 2) (v0 + v1)
            # (tybok/policies/smolvla/models/flow_matching.py:596-625)
            for step in range(self.num_steps):
                if fused_loop:
                    v0, x_pred = self.fused_euler_step(pads, caches, x_t, 2 * step, positions, dt, want_v=True)
                    v1, _ = self.fused_euler_step(pads, caches, x_pred, 2 * step + 1, positions, dt, want_v=True)
                else:
                    v0 = self.denoise_step(pads, keys, values, ekv, x_t, self.time_embs[2 * step], positions, caches)
                    v1 = self.denoise_step(pads, keys, values, ekv, x_t + dt * v0, self.time_embs[2 * step + 1], positions, caches)
                x_t = x_t + (dt * 0.5) * (v0 + v1)
            return x_t
        h = None
        carry = fused_loop and self._fused_embed_ok(x_t)
        for step in range(self.num_steps):
            if fused_loop:
                if carry and step + 1 < self.num_steps:
                    x_t, h = self.fused_euler_step(pads, caches, x_t, step, positions, dt, h=h, next_step=step + 1)
                else:
                    x_t = self.fused_euler_step(pads, caches, x_t, step, positions, dt, h=h)
                continue
            v_t = self.denoise_step(pads, keys, values, ekv, x_t, self.time_embs[step], positions, caches)
            x_t = x_t + dt * v_t
        return x_t

    def sample_actions(self, images, img_masks, lang_tokens, lang_masks, state, noise, trace: dict | None = None, image_range01: bool = False) -> torch.Tensor:
        """Prefix embed, prefill, expert prefix KV, Euler loop -> ``[1, chunk, max_action_dim]`` fp32."""
        embs, pads, att = self.embed_prefix(images, img_masks, lang_tokens, lang_masks, state, image_range01)
        return self.sample_actions_core(embs, pads, att, noise, trace)
