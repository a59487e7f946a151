/*
 * tybok_hip.h -- C ABI of libtybok_hip.so: MI355X (gfx950) kernels for tybok's fp8
 * action-inference path.
 *
 * Conventions (the ones the reference's own native layer uses for its fused kernels,
 * tybok/policies/fastwam/kernels/adit_fused_bindings.cpp:21-71):
 *   - every pointer is a DEVICE pointer unless said otherwise; the caller owns every buffer,
 *     workspace included; no entry point allocates, frees or synchronises;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all work is enqueued
 *     on it, so the calls are legal under stream capture (hipGraph);
 *   - every entry point returns 0 on success or a negative TK_E* code; tk_last_error() gives
 *     the message of the calling thread's last failure (the reference's host helpers throw
 *     std::runtime_error and never exit(): tybok/policies/fastwam/kernels/coop_grid.h:20-27);
 *   - reductions are fixed-order: the same inputs give the same bits on every run and under
 *     graph replay (the reference's rule: tybok/policies/fastwam/kernels/vdit_gemm_core.cu:7-9).
 *
 * Workspace: one caller-owned buffer per stream of at least tk_workspace_bytes() bytes, passed
 * once through tk_workspace_init() (which zeroes its arrival counters with a fill kernel).
 * Entry points leave the counters zero on exit.  Two calls that may overlap in time (different
 * streams) need different workspaces.
 */
#ifndef TYBOK_HIP_H
#define TYBOK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TK_OK 0
#define TK_EINVAL (-1)   /* bad shape / alignment / argument */
#define TK_EWORKSPACE (-2) /* workspace too small */
#define TK_ELAUNCH (-3)  /* HIP launch error */

/* activation of the gated FFN */
#define TK_ACT_SILU 0      /* SwiGLU: tybok/policies/smolvla/models/layers.py:75-76 */
#define TK_ACT_GELU_TANH 1 /* GeGLU:  tybok/policies/pi05/models/layers.py:94-95 */

/* suffix mask mode of the expert attention */
#define TK_MASK_NONE 0   /* no suffix keys (cross-attention over the prefix only) */
#define TK_MASK_BIDIR 1  /* every action token sees every action token (pi0.5) */
#define TK_MASK_CAUSAL 2 /* action token i sees action tokens j <= i (SmolVLA) */

/* element types */
#define TK_BF16 0
#define TK_F32 1

int tk_version(void);
const char* tk_last_error(void);

/* Number of compute units of the current device (0 on error); diagnostic only. */
int tk_device_cus(void);

/* ---- workspace ------------------------------------------------------------------------- */
/* Bytes that cover every entry point at the shapes of both policies (split-K partials,
 * attention partials, the FFN's [M, I] intermediate, arrival counters). */
size_t tk_workspace_bytes(void);
/* Zero the arrival counters at the head of `ws` (fill kernel, capture-safe). Call once. */
int tk_workspace_init(void* ws, size_t ws_bytes, void* stream);

/* ---- fp8 weight packing ------------------------------------------------------------------ */
/* The GEMM reads weights as 32x32-byte tiles in MFMA operand order: tile (nt, kt) holds rows
 * 32*nt.. and k bytes 32*kt.., stored as 64 consecutive 16-byte lane chunks, so one wave loads a
 * tile with one fully coalesced 1 KiB global_load_dwordx4.  Rows >= N and k >= K are zero.
 * Replaces the reference's cached transposed copy `quantize_weight_rows_transposed`
 * (tybok/policies/pi05/models/triton_expert_mlp_fp8.py:200-218): a layout-only, once-per-model
 * transform of the checkpoint's row-major `[N, K]` e4m3fn weight
 * (docs/fastWAM_weight_quantization.md:23-24).  Requires K % 16 == 0. */
size_t tk_fp8w_packed_bytes(int N, int K);
int tk_pack_fp8_weight(const void* w8_rowmajor, void* packed, int N, int K, void* stream);
/* Gate and up weights ([I, K] each) packed into one buffer with their 32-row tiles interleaved
 * (gate tile j, up tile j, gate tile j+1, ...), so one wave owns matching gate/up columns.
 * Size = tk_fp8w_packed_bytes(2*I, K); requires I % 32 == 0. */
int tk_pack_fp8_gate_up(const void* wg8_rowmajor, const void* wu8_rowmajor, void* packed, int I, int K,
                        void* stream);

/* ---- fp8-weight split-K GEMM ------------------------------------------------------------- */
/* y[M, N] = bf16( (x[M, K] . W8[N, K]^T) * scale[n] )   (+ optional residual, see below)
 * bf16 activations, e4m3fn weights (packed), fp32 per-output-channel scale, fp32 accumulate.
 * Replaces `_w8a8_gemm` / `_down_fp8_splitk_kernel` + `_down_fp8_splitk_reduce_kernel`
 * (tybok/policies/pi05/models/triton_prefill_mlp.py:62-130,
 *  tybok/policies/pi05/models/triton_expert_mlp_fp8.py:312-435) with weight-only semantics
 * (no activation quantisation).
 *   x: bf16, row stride ldx elements (ldx % 8 == 0, 16-byte aligned); y: bf16, row stride ldy.
 *   resid: NULL, or a [M, N] tensor (row stride ldr, type resid_dtype) added AFTER the bf16
 *          rounding of the product: y = bf16(float(bf16(acc*scale)) + float(resid)) -- the
 *          reference's in-place `out_emb += hidden_states`
 *          (tybok/policies/smolvla/models/vlm_with_expert.py:386-408).
 *   gate:  NULL, or bf16 [N]: the product is multiplied by gate[n] (one more bf16 rounding)
 *          before the residual is added: y = bf16(resid + bf16(bf16(acc*scale) * gate[n])) -- the
 *          AdaRMS gated residual `x + y * gate` of pi0.5 (tybok/policies/pi05/models/layers.py:27-31,
 *          tybok/policies/pi05/models/triton_expert_residual.py:26-60).
 *   split_k: 0 = pick automatically; otherwise the number of K splits (>= 1).
 */
int tk_fp8w_gemm(const void* x, int ldx, const void* w_packed, const void* scale, void* y, int ldy,
                 const void* resid, int ldr, int resid_dtype, const void* gate, int M, int N, int K, int split_k,
                 void* ws, size_t ws_bytes, void* stream);

/* tk_fp8w_gemm for callers that cannot allocate or carry a workspace (code under graph capture that
 * owns no buffers, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference, whose native layer always receives caller-owned scratch.  Arguments and results as
 * tk_fp8w_gemm (same kernels, same bits), without `ws`: the split-K partials and arrival counters live
 * in an array inside the library's device image -- tk_static_scratch_bytes() bytes (64 KiB of counters
 * + 8 MiB of partials) that each GPU the library runs on holds until the process ends.
 *   Limits: M <= 64 (the action chunk); an explicit split_k whose partials exceed the 8 MiB is
 *   rejected with TK_EWORKSPACE; split_k = 0 never chooses more than fits.
 *   The first call on a device looks the array's address up; on a capturing stream that first call is
 *   refused with TK_EINVAL -- tk_static_scratch_bytes() resolves the address for the current device, call
 *   it (or run one launch) before capturing.  "Same bits" holds because the automatic split never needs
 *   more than the 8 MiB here on a 256-CU device; a device with more CUs could pick another split under
 *   tk_fp8w_gemm's larger workspace.  No call allocates, frees or synchronises.  All calls on one GPU share the one array: calls that
 *   may overlap in time (two streams, two threads) race -- serialise them or use tk_fp8w_gemm with
 *   one workspace per stream.  The counters a split launch uses are cleared by a fill kernel
 *   right before it, so a call does not depend on what the previous one left behind. */
int tk_fp8w_gemm_static(const void* x, int ldx, const void* w_packed, const void* scale, void* y, int ldy,
                        const void* resid, int ldr, int resid_dtype, const void* gate, int M, int N, int K,
                        int split_k, void* stream);
size_t tk_static_scratch_bytes(void);

/* ---- fused gated FFN ----------------------------------------------------------------------- */
/* y[M, K] = down( act(gate(x)) * up(x) ) with fp8 weights, bf16 in/out:
 *   g = bf16(x.Wg^T * sg), u = bf16(x.Wu^T * su), h = bf16(bf16(act(g)) * u), y = bf16(h.Wd^T * sd)
 * Replaces `MLP.forward` / `GemmaMLP.forward` and the fused chains `triton_norm_gate_up` + down
 * and `triton_mlp_fp8_chain` (tybok/policies/smolvla/models/layers.py:61-76,
 * tybok/policies/pi05/models/layers.py:87-95, tybok/policies/smolvla/models/triton_mlp.py:30-144,
 * tybok/policies/pi05/models/triton_expert_mlp_fp8.py:438-469).
 *   wgu_packed: tk_pack_fp8_gate_up output; wd_packed: tk_pack_fp8_weight of [K, I].
 *   resid/ldr/resid_dtype/gate: as in tk_fp8w_gemm, applied to y.
 * The [M, I] intermediate lives in the workspace (never returned). */
int tk_fp8w_gated_ffn(const void* x, int ldx, const void* wgu_packed, const void* sg, const void* su,
                      const void* wd_packed, const void* sd, void* y, int ldy, const void* resid, int ldr,
                      int resid_dtype, const void* gate, int M, int K, int I, int act, void* ws,
                      size_t ws_bytes, void* stream);

/* y = tk_fp8w_gated_ffn(rms_norm(x, norm_w, norm_eps), ...): the post-attention RMSNorm runs inside
 * the gate/up launch while the activations are staged (bf16 x: bf16(w * bf16(x * rstd)), fp32
 * statistics), as the reference's `triton_norm_gate_up(x, norm_w, eps, gate_w, up_w)` folds it
 * (tybok/policies/smolvla/models/triton_mlp.py:105-144, call site vlm_with_expert.py:391-408).
 *   norm_w: bf16 [K], 16-byte aligned; or NULL with ada_scale / ada_shift (fp32 [K] each): the
 *           adaptive RMSNorm of pi0.5, bf16((x * rstd) * (1 + scale) + shift) in fp32, as
 *           `triton_norm_gate_up_fp8` folds it (tybok/policies/pi05/models/triton_expert_mlp_fp8.py:54-197;
 *           eager: tybok/policies/pi05/models/layers.py:51-84).  Other arguments as tk_fp8w_gated_ffn. */
int tk_fp8w_norm_gated_ffn(const void* x, int ldx, const void* norm_w, float norm_eps, const void* ada_scale,
                           const void* ada_shift, const void* wgu_packed,
                           const void* sg, const void* su, const void* wd_packed, const void* sd, void* y, int ldy,
                           const void* resid, int ldr, int resid_dtype, const void* gate, int M, int K, int I,
                           int act, void* ws, size_t ws_bytes, void* stream);

/* The action chunk's FFN (M <= 64, the expert shapes of both models) can run as ONE launch: its down blocks
 * request their weights, then wait inside the kernel until the gate/up blocks their k range depends on have
 * written their slices of the intermediate through and raised their flags -- the fusion `triton_norm_gate_up` +
 * down (tybok/policies/smolvla/models/triton_mlp.py:30-144) and `triton_mlp_fp8_chain`
 * (tybok/policies/pi05/models/triton_expert_mlp_fp8.py:438-469) stand for.  Same bits as the two-launch form,
 * which every other shape takes.  On MI355X the hand-off between blocks of different XCDs costs more than the
 * launch boundary it replaces (measured: 10.9 against 8.6 us per FFN), so the single-launch form is OFF unless
 * asked for.  The three calls below have no counterpart in the reference:
 *   tk_set_ffn_fusion(on): 1 runs the action chunk's FFN as one launch; returns the previous setting (default 0).
 *   tk_set_handoff_spin(polls): how often a waiting block polls before it gives up (default 200000, about 0.1 s);
 *     returns the previous value.  A block that gives up sets the workspace's sticky error word (int32 at byte
 *     offset tk_workspace_handoff_error_offset()) and goes on, so the launch always ends; its output is then
 *     undefined and the workspace must be re-initialised (tk_workspace_init) before the next call. */
int tk_set_ffn_fusion(int on);
int tk_set_handoff_spin(int polls);
size_t tk_workspace_handoff_error_offset(void);

/* ---- W8A8 tier: per-token activation quantisation + fp8 x fp8 GEMM (VLM prefill MLP) --------- */
/* Per-token (per-row) activation quantisation to e4m3fn:
 *   sa[m] = max_k |x[m, k]| / 448 (fp32),  a8[m, k] = RNE(x[m, k] / sa[m]) computed in fp32, one rounding;
 *   an all-zero row gives sa = 0 and zero codes.
 * Replaces `quantize_activation` / `_quant_act` (tybok/policies/pi05/models/triton_prefill_mlp.py:26-59,103-114),
 * `_quant_act_fp8_kernel` (tybok/policies/pi05/models/triton_expert_mlp_fp8.py:234-277) and `quantize_act`
 * (tybok/policies/fastwam/models/fp8_linear.py:223-243: `sa = amax/448; a8 = RNE(x/sa)`).
 *   mode 0: the recipe above.  mode 1: the arithmetic of the prefill path's torch expression on bf16 tensors --
 *           the scale rounded to bf16 and the quotient rounded to bf16 before the fp8 cast
 *           (triton_prefill_mlp.py:30-36); sa then holds the bf16 value as fp32.
 *   x: bf16 [M, K], pitch ldx (elements, a multiple of 8), 16-byte aligned; a8: [M, K] bytes, pitch lda (a multiple
 *   of 8), 8-byte aligned; sa: fp32 [M]; K a multiple of 8, at most 16384. */
int tk_quant_act_rows(const void* x, int ldx, void* a8, int lda, void* sa, int M, int K, int mode, void* stream);

/* y[M, N] = bf16( (a8[M, K] . W8[N, K]^T) * sa[m] * sw[n] )  (+ residual: bf16(y + resid))
 * e4m3fn activations and weights multiplied on the fp8 matrix instruction, fp32 accumulate.  Replaces `_w8a8_gemm`
 * / `w8a8_gemm` (tybok/policies/pi05/models/triton_prefill_mlp.py:62-130).  Built for many rows (block tile
 * 128 x 256: the VLM prefill); w_packed as for tk_fp8w_gemm; lda in bytes, a multiple of 16; N and ldy
 * multiples of 4; split_k 0 = automatic (K splits hand fp32 partials through the workspace, fixed order). */
int tk_w8a8_gemm(const void* a8, int lda, const void* sa, const void* w_packed, const void* w_scale, void* y, int ldy,
                 const void* resid, int ldr, int resid_dtype, int M, int N, int K, int split_k, void* ws, size_t ws_bytes,
                 void* stream);

/* The prefill MLP in W8A8, `make_fp8_mlp_forward` (tybok/policies/pi05/models/triton_prefill_mlp.py:145-166):
 *   (x8, sx) = quant(x);  g = w8a8(x8, Wg), u = w8a8(x8, Wu)  (bf16 each);  h = bf16(bf16(act(g)) * u);
 *   (h8, sh) = quant(h);  y = w8a8(h8, Wd)  (+ residual)
 * in four launches (quantise, gate/up with the gated epilogue, quantise, down); quantised copies and the [M, I]
 * intermediate live in the workspace.  Arguments as tk_fp8w_gated_ffn (no per-column gate).  quant_mode is the
 * mode of tk_quant_act_rows for both quantisations: 1 is what `quantize_activation` / `_quant_act` compute
 * (scale and quotient rounded to bf16 before the fp8 cast, triton_prefill_mlp.py:26-59,103-114), 0 keeps the
 * scale and the quotient in fp32 (one rounding). */
int tk_w8a8_gated_ffn(const void* x, int ldx, const void* wgu_packed, const void* sg, const void* su, const void* wd_packed,
                      const void* sd, void* y, int ldy, const void* resid, int ldr, int resid_dtype, int M, int K, int I,
                      int act, int quant_mode, void* ws, size_t ws_bytes, void* stream);

/* Byte offsets, inside the workspace, of what tk_w8a8_gated_ffn(M, K, I) leaves behind: the bf16 [M, I] intermediate
 * h, its e4m3fn codes h8 [M, I] and their fp32 row scales [M] -- so a caller (or a test) can check the second
 * quantisation and the down projection on exactly the operands the library used.  No counterpart in the
 * reference, whose forward keeps `act`, `act_q` and `act_scale` as tensors (triton_prefill_mlp.py:157-161). */
int tk_w8a8_ffn_layout(int M, int K, int I, size_t* h_off, size_t* h8_off, size_t* sh_off);

/* ---- bf16-weight expert projections (norm prologue, rotary epilogue, residual epilogue) ----- */
/* Bytes of a packed bf16 [N, K] weight (2 KiB per 32x32 tile). */
size_t tk_bf16w_packed_bytes(int N, int K);
/* Row-major bf16 [N, K] -> tile order.  rope_half = 0 keeps the natural n-tile order; rope_half =
 * head_dim/2 orders the tiles so that each pair of adjacent tiles holds columns (c, c + rope_half)
 * of one head (2*rope_half must divide N).  Offline, once per weight; the same role as the
 * reference's `_packed_qkv_interleaved` (tybok/policies/pi05/models/
 * triton_expert_fused_qkv_rope_attn.py:226-251). */
int tk_pack_bf16_weight(const void* w, void* packed, int N, int K, int rope_half, void* stream);
/* y[M, N] (bf16) = epilogue( prologue(x)[M, K] . W[N, K]^T ) with bf16 weights.
 *   prologue: norm_w == NULL -> x is bf16, used as is.  Otherwise Llama RMSNorm with fp32
 *             statistics: x bf16 (x_dtype TK_BF16) -> bf16(w * bf16(x * rstd)); x fp32 (TK_F32,
 *             the first expert layer) -> bf16(w * (x * rstd)).
 *   epilogue: rope_pos == NULL -> y = bf16(acc) (+ residual: bf16(y + resid), bf16 or fp32 resid)
 *             -- the o_proj + in-place residual add of a decoder layer
 *             (tybok/policies/smolvla/models/vlm_with_expert.py:380-389).
 *             rope_pos != NULL -> half-split rotary embedding on columns < rope_cols: the pair
 *             (c, c + rope_half) of each head at row m becomes, in fp32 from the bf16-rounded
 *             projection, (a*cos - b*sin, b*cos + a*sin) with cos/sin = table[pos[m]][c % rope_half],
 *             rounded to bf16; columns >= rope_cols (the v projection) pass through.  W must have
 *             been packed with the same rope_half.  One launch for the concatenated q|k|v weight:
 *             `triton_self_attn`'s norm + q/k/v + RoPE phase and `triton_qkv_rope_fused`
 *             (tybok/policies/smolvla/models/triton_attn.py:99-172,586-655,
 *              tybok/policies/pi05/models/triton_expert_fused_qkv_rope_attn.py:254-320;
 *              eager: tybok/policies/smolvla/models/rope.py:51-73).
 *   rope_pos: int32 [M] (clamped into [0, rope_positions)); rope_cos/rope_sin: fp32
 *             [rope_positions, rope_half].
 *   ada_scale / ada_shift: fp32 [K], instead of norm_w: adaptive RMSNorm prologue (pi0.5),
 *             bf16((x * rstd) * (1 + scale) + shift) with every step rounded in fp32
 *             (tybok/policies/pi05/models/layers.py:51-84).
 *   rope_bf16: 1 = rotate in bf16 arithmetic, every product and the sum rounded to bf16 and the
 *             tables holding bf16 values: pi0.5's `x * cos + rotate_half(x) * sin` on bf16 tensors
 *             (tybok/policies/pi05/models/rope.py:59-75).
 *   gate:     optional bf16 [N], plain epilogue only: y = bf16(bf16(acc) * gate[n]) before the
 *             residual -- pi0.5's gated residual `res + o_proj(att) * gate`
 *             (tybok/policies/pi05/models/triton_expert_residual.py:26-60).
 *   vt:       optional (rotary epilogue only): the columns n >= vt_col0 (the value projection;
 *             vt_col0 a head boundary >= rope_cols) are also written transposed,
 *             vt[(n - vt_col0) * vt_ld + m], the suffix V^T operand of tk_expert_attn; entries
 *             m >= M of a row are left as they are (keep them zero).
 * Built for the action-chunk tile shape (any M, tiled 64 rows at a time); the norm prologue is
 * built together with the rotary epilogue only. */
int tk_bf16w_linear(const void* x, int ldx, int x_dtype, const void* w_packed, const void* norm_w, float norm_eps,
                    const void* ada_scale, const void* ada_shift, const void* rope_pos, const void* rope_cos,
                    const void* rope_sin, int rope_positions, int rope_cols, int rope_half, int rope_bf16, void* vt,
                    int vt_col0, int vt_ld, void* y, int ldy, const void* resid, int ldr, int resid_dtype,
                    const void* gate, int M, int N, int K, int split_k, void* ws, size_t ws_bytes, void* stream);

/* y[M, N] (bf16) = bf16( resid + act( bf16( x[M, K] . W[N, K]^T + bias[N] ) ) ): the linears of the vision towers
 * (q|k|v, out_proj, fc1 + GELU, fc2) and any other bf16 linear over hundreds of rows, on the many-row MFMA kernel.
 * Replaces the reference's fused tower kernels' GEMM parts (`triton_vision_qkv`, `triton_vision_out_proj`,
 * `triton_vision_mlp`, tybok/policies/pi05/models/vision.py:116-173; SmolVLA: the bf16 `nn.Linear`s of
 * tybok/policies/smolvla/models/vision.py:197-257).
 *   x:     bf16 [M, K], pitch ldx (elements, a multiple of 8; K a multiple of 16; 16-byte aligned).
 *   w_packed: tk_pack_bf16_weight(..., rope_half = 0).
 *   bias:  bf16 [N] or NULL.
 *   act:   0 none; 1 tanh GELU of the bf16-rounded linear output (`gelu(linear(x))` on bf16 tensors,
 *          tybok/policies/pi05/models/vision.py:79-87); 2 tanh GELU of the fp32 pre-activation (the reference's fused
 *          MLP keeps fc1's output in fp32 through the GELU, vision.py:259-273).
 *   resid: optional bf16 or fp32 [M, N] (resid_dtype TK_BF16 / TK_F32), added to the bf16-rounded result.
 *   y:     bf16 [M, N], pitch ldy (a multiple of 8, 16-byte aligned); N a multiple of 4.
 *   tile:  0 = chosen from the shape; 42, 41, 32, 31, 22, 21, 12, 11 = (32-row tiles per block, 32-column tiles per
 *          wave of a 4-wave block).
 *   split_k: 0 = automatic; > 1 needs the workspace (fp32 partials, summed in split order: bit-deterministic). */
int tk_bf16w_dense(const void* x, int ldx, const void* w_packed, const void* bias, int act, void* y, int ldy,
                   const void* resid, int ldr, int resid_dtype, int M, int N, int K, int tile, int split_k, void* ws,
                   size_t ws_bytes, void* stream);

/* tk_bf16w_dense with every 16-bit operand in IEEE fp16 instead of bf16 (x, the packed weight -- tk_pack_bf16_weight
 * moves 16-bit words and serves both --, bias, y and a TK_BF16-typed residual, which is then read as fp16), on
 * `v_mfma_f32_32x32x16_f16`: the fp16 GEMMs of pi0.5's vision tower -- the `--vit-mlp-dtype fp16` tier
 * (tybok/policies/pi05/models/vision.py:79-87,223-235) and the fused tier's q|k|v projection
 * (`_vision_qkv_kernel`, tybok/policies/pi05/models/triton_vision.py:38-110: fp16 operands, fp32 accumulate). */
int tk_f16w_dense(const void* x, int ldx, const void* w_packed, const void* bias, int act, void* y, int ldy,
                   const void* resid, int ldr, int resid_dtype, int M, int N, int K, int tile, int split_k, void* ws,
                   size_t ws_bytes, void* stream);

/* The many-row linear with the rotary epilogue of tk_bf16w_linear: y[M, N] = bf16(x . W^T) with the columns
 * < rope_cols rotated in pairs (i, i + rope_half) of heads of 2 * rope_half columns by the table row of rope_pos[m]
 * (int32 [M], clamped into fp32 tables [rope_positions, rope_half]; rope_bf16 selects pi0.5's bf16 arithmetic) and,
 * when vt is given, the columns >= vt_col0 also written transposed, vt[(n - vt_col0) * vt_ld + m] (rows past M of
 * vt are left as they are: the caller zero-fills it once) -- the q|k|v projection of a many-row prefill in one
 * launch (`_fused_gemm_rope_kernel`, tybok/policies/pi05/models/triton_expert_fused_qkv_rope_attn.py:103-251).
 * w_packed: tk_pack_bf16_weight with the same rope_half (rotary pair order).  N, rope_cols and vt_col0 whole heads;
 * vt_ld a multiple of 8 >= M rounded up to 32; tile 0 (automatic) or one of the two-tile shapes 42, 32, 22, 12.
 * Same bits as tk_bf16w_dense on naturally packed weights followed by tk_rope_rows and tk_batched_transpose_v. */
int tk_bf16w_dense_rope(const void* x, int ldx, const void* w_packed, void* y, int ldy, const void* rope_pos,
                        const void* rope_cos, const void* rope_sin, int rope_positions, int rope_cols, int rope_half,
                        int rope_bf16, void* vt, int vt_col0, int vt_ld, int M, int N, int K, int tile, int split_k,
                        void* ws, size_t ws_bytes, void* stream);

/* The packed q|k|v projection of a vision tower with the value columns also written transposed, so that the
 * attention launch needs no transpose in front of it: y[M, N] = 16-bit(x . W^T + bias) as tk_bf16w_dense
 * (f16 = 1: tk_f16w_dense) and vt[(m / vt_rows) * vt_bs + (n - vt_col0) * vt_ld + m % vt_rows] = y[m, n] for the
 * columns n >= vt_col0 -- the rows are vt_rows-row problems (cameras; 0 = one problem), which is the layout
 * [B, G, D, P] that tk_batched_attn reads.  vt_col0 a multiple of 64, vt_rows of 32, vt_ld and vt_bs of 8.
 * Replaces tk_bf16w_dense + tk_batched_transpose_v (same bits); reference: the towers' `attn @ v` operand,
 * tybok/policies/smolvla/models/vision.py:197-257, tybok/policies/pi05/models/vision.py:115-170. */
int tk_bf16w_dense_vt(const void* x, int ldx, const void* w_packed, const void* bias, void* y, int ldy, void* vt,
                      int vt_col0, int vt_ld, int vt_rows, long long vt_bs, int f16, int M, int N, int K, int tile,
                      int split_k, void* ws, size_t ws_bytes, void* stream);

/* ---- action-expert attention over the cached prefix ------------------------------------------ */
/* Lays one layer's prefix K/V out for tk_expert_attn, once per request (the counterpart of the
 * reference filling its static per-layer prefix cache after the VLM prefill,
 * tybok/policies/smolvla/models/flow_matching.py:553-578):
 *   k, v:   [L, G, D] of kv_dtype with element strides (sl, sh), d contiguous.
 *   vt_hi:  bf16 [G, D, vt_ld] <- V transposed (keys contiguous), zero-filled from L to vt_ld;
 *           vt_ld >= L rounded up to 32, a multiple of 8.
 *   TK_BF16: k is used in place by the attention (k may be NULL here); k_hi/k_lo/vt_lo unused.
 *   TK_F32 (the SmolVLA cross layers, whose expert K/V projections are fp32): K -> k_hi + k_lo
 *           (bf16 [L, G, D] contiguous each, x = hi + lo to 16 mantissa bits), V^T -> vt_hi + vt_lo. */
int tk_attn_prepare_kv(const void* k, const void* v, int kv_dtype, int sl, int sh, int L, int G, int D, void* k_hi,
                       void* k_lo, void* vt_hi, void* vt_lo, int vt_ld, void* stream);

/* out[M, H*D] (bf16) = softmax(q.K^T * D^-0.5 + mask) . V over keys [prefix(P); suffix(S)].
 * Replaces `EagerAttention._forward_eager` / `GemmaAttention._forward_eager`'s core and the fused
 * `triton_self_attn` / `triton_cross_attn` / `_splitk_flash_kernel`
 * (tybok/policies/smolvla/models/attention.py:136-187, tybok/policies/pi05/models/layers.py:166-191,
 *  tybok/policies/smolvla/models/triton_attn.py:586-855,
 *  tybok/policies/pi05/models/triton_expert_fused_qkv_rope_attn.py:322-433).
 *   q:      bf16 [M, H, D], element strides (q_sm, q_sh), d contiguous.
 *   k_pre:  bf16 [P, G, D], element strides (pre_sl, pre_sh).
 *   vt_pre: bf16 V^T [G, D, >= P rounded up to 32] (zero padded), element strides (pre_vt_sh, pre_vt_sd),
 *           keys contiguous -- tk_attn_prepare_kv's output.
 *   k_pre_lo / vt_pre_lo: low planes of fp32 K/V (same strides), or NULL for bf16 K/V; only with
 *           S == 0 and D == 64 (the SmolVLA cross layers).
 *   k_suf:  bf16 [S, G, D], strides (suf_sl, suf_sh); vt_suf: bf16 V^T [G, D, >= S rounded up to
 *           32] (zero padded), strides (suf_vt_sh, suf_vt_sd) -- tk_bf16w_linear's `vt` output.
 *           Both NULL when S == 0.
 *   pad:    uint8 [P], 1 = prefix token visible (NULL = all visible).
 *   mask2d: optional uint8 [M, mask_ld] (mask_ld >= P rounded up to 32, a multiple of 8): byte
 *           (m, p) != 0 = prefix key p visible to query m; replaces `pad`.  This is the 2-D mask of
 *           the VLM prefill (`make_att_2d_masks`, tybok/policies/smolvla/models/flow_matching.py:44-83,
 *           `triton_prefill_layer`'s mask2d, tybok/policies/smolvla/models/triton_attn.py:465-583).
 *   mask_mode: TK_MASK_*; q head h reads kv head h / (H / G).
 *   logits_bf16: 0 = fp32 logits (SmolVLA); 1 = logits rounded to bf16 before the softmax and
 *           masked with the additive -2.3819763e38 (pi0.5).
 *   D in {64, 96, 128, 256}; masked logits use finfo(float32).min, so a fully masked row is uniform.
 *   out:    8-byte aligned, out_sm a multiple of 4.
 */
int tk_expert_attn(const void* q, int q_sm, int q_sh, const void* k_pre, const void* k_pre_lo, int pre_sl, int pre_sh,
                   const void* vt_pre, const void* vt_pre_lo, int pre_vt_sd, int pre_vt_sh, const void* k_suf,
                   int suf_sl, int suf_sh, const void* vt_suf, int suf_vt_sd, int suf_vt_sh, const void* pad,
                   const void* mask2d, int mask_ld, void* out, int out_sm, int M, int P, int S, int H, int G, int D,
                   int mask_mode, int logits_bf16, void* ws, size_t ws_bytes, void* stream);

/* Expert K/V projection of the cached VLM prefix for the cross-attention layers, straight into the
 * attention kernel's fp32 operand layout (bf16 hi + lo planes):
 *   ek = float(k) . wk^T, ev = float(v) . wv^T with fp32 weights and fp32 accumulation, then
 *   k_hi / k_lo [P, N] and vt_hi / vt_lo [N, vt_ld] (V transposed, keys contiguous, zero filled
 *   from P to P rounded up to 32) -- N = kv_heads * head_dim.
 * Replaces `_compute_expert_prefix_kv` + the cache fill: two `.float()` casts, two fp32 linears
 * and tk_attn_prepare_kv (tybok/policies/smolvla/models/flow_matching.py:553-578,
 * tybok/policies/smolvla/models/expert.py:35-39).
 *   k, v: bf16 [P, KV] rows with element stride sl (a multiple of 8), 16-byte aligned; wk, wv: fp32
 *   [N, KV]; N a multiple of 32, KV of 16; k_hi / k_lo 8-byte aligned; vt_ld >= P rounded up to 32. */
int tk_expert_kv_project(const void* k, const void* v, int sl, int P, int KV, const void* wk, const void* wv, int N,
                         void* k_hi, void* k_lo, void* vt_hi, void* vt_lo, int vt_ld, void* stream);

/* tk_expert_kv_project for several cross layers in one launch (the projections are independent; each of them alone
 * leaves 96 of 256 compute units idle and pays a launch of its own):
 *   k, v, wk, wv: host arrays of `layers` device pointers (1..16), shapes and strides as above, the same for every layer;
 *   k_hi / k_lo: [layers][P, N]; vt_hi / vt_lo: [layers][N, vt_ld].  Same bits as `layers` single calls. */
int tk_expert_kv_project_layers(int layers, const void* const* k, const void* const* v, int sl, int P, int KV,
                                const void* const* wk, const void* const* wv, int N, void* k_hi, void* k_lo, void* vt_hi,
                                void* vt_lo, int vt_ld, void* stream);

/* Cross-attention layer of the action expert with the query projection inside the attention launch:
 *   q = rope(bf16(RMSNorm(x) . Wq^T)) per head (bf16(w * bf16(x * rstd)) norm, fp32 half-split rotary
 *   embedding with table rows rope_pos[m]), then attention over the fp32 (hi + lo planes) expert
 *   prefix K/V under the prefix pad mask.  Replaces `triton_cross_attn` (norm + q projection + RoPE
 *   + attention in one kernel: tybok/policies/smolvla/models/triton_attn.py:791-855; call site
 *   vlm_with_expert.py:275-297) and equals tk_bf16w_linear (norm + q + RoPE) followed by tk_expert_attn.
 *   x: bf16 [M, K] (row pitch ldx), K a multiple of 8 and at most 768; norm_w bf16 [K];
 *   wq_packed: tk_pack_bf16_weight of the [H*D, K] q weight with rope_half = D/2;
 *   D = 64; P at most 256 (8 key tiles: one block covers the prefix); K/V layouts, pad, out as tk_expert_attn. */
int tk_expert_cross_attn_fused(const void* x, int ldx, const void* norm_w, float norm_eps, const void* wq_packed, int K,
                               const void* rope_pos, const void* rope_cos, const void* rope_sin, int rope_positions,
                               const void* k_hi, const void* k_lo, int pre_sl, int pre_sh, const void* vt_hi,
                               const void* vt_lo, int pre_vt_sd, int pre_vt_sh, const void* pad, void* out, int out_sm,
                               int M, int P, int H, int G, int D, void* stream);

/* B independent unmasked attentions in one launch (the vision tower's self-attention, one problem
 * per camera image): out[b][M, H*D] = softmax(q[b].K[b]^T * D^-0.5) . V[b].  Layouts as the prefix
 * operands of tk_expert_attn (K [P, G, D]; V^T [G, D, >= P rounded up to 32], zero padded), with
 * element strides q_sb / k_sb / vt_sb / out_sb between problems.  logits_bf16 = 1 rounds q.K^T to
 * bf16 before the fp32 scale and softmax, as a bf16 matmul followed by `.float() * scale` does
 * (tybok/policies/smolvla/models/vision.py:197-257).  logits_bf16 = 2: q, K and V^T hold IEEE fp16 values
 * and the probabilities are rounded to fp16 for P.V, both products on the fp16 matrix instruction with fp32
 * logits and accumulation, bf16 output -- `_vision_attn_kernel` of pi0.5's fused tower
 * (tybok/policies/pi05/models/triton_vision.py:248-326); built for D = 96 and >= 128 queries and keys.  scale > 0 replaces D^-0.5: a head whose true
 * size is not supported (SigLIP-So400m: 72) is padded with zero columns to the next D and passes
 * 72^-0.5 (tybok/policies/pi05/models/vision.py:52-66); scale = 0 keeps the default. */
int tk_batched_attn(const void* q, long long q_sb, int q_sm, int q_sh, const void* k, long long k_sb, int k_sl, int k_sh,
                    const void* vt, long long vt_sb, int vt_sd, int vt_sh, void* out, long long out_sb, int out_sm, int B,
                    int M, int P, int H, int G, int D, int logits_bf16, float scale, void* ws, size_t ws_bytes,
                    void* stream);

/* V^T for tk_batched_attn from the projection output, one launch for all problems:
 *   v:  bf16 [B, P, G, D], element strides (v_sb, v_sl, v_sh), d contiguous (a view into a packed
 *       q|k|v buffer is fine);  vt: bf16 [B, G, D, vt_keys], element strides (vt_sb, vt_sh, vt_sd),
 *       keys contiguous, vt_keys >= P rounded up to 32, zero filled from P on (up to the end of the
 *       last 64-key tile or vt_keys).  D in {64, 96}; all strides multiples of 8 elements.
 * Replaces the `v.transpose(1, 2)` operand of the towers' `attn @ v`
 * (tybok/policies/smolvla/models/vision.py:197-257, tybok/policies/pi05/models/vision.py:115-170). */
int tk_batched_transpose_v(const void* v, long long v_sb, int v_sl, int v_sh, void* vt, long long vt_sb, int vt_sh,
                           int vt_sd, int vt_keys, int B, int P, int G, int D, void* stream);

/* ---- vision tower glue ------------------------------------------------------------------------ */
/* RMSNorm of bf16 rows into a bf16 buffer, for projections that run as a plain library GEMM (many
 * rows): y[m, :] = bf16(norm_w * bf16(x * rstd))  (Llama RMSNorm, norm_w bf16 [K]) or
 * bf16((x * rstd) * (1 + ada_scale) + ada_shift)  (Gemma / adaptive RMSNorm, fp32 [K] vectors; a
 * plain Gemma norm passes its weight as ada_scale and zeros as ada_shift) -- the prologues of
 * tk_bf16w_linear / tk_fp8w_norm_gated_ffn as a launch of their own
 * (tybok/policies/smolvla/models/layers.py:23-58, tybok/policies/pi05/models/layers.py:51-84). */
int tk_rms_norm_rows(const void* x, int ldx, const void* norm_w, const void* ada_scale, const void* ada_shift, float eps,
                     void* y, int ldy, int M, int K, void* stream);

/* Rotary embedding in place on the columns < rope_cols of a bf16 projection output y [M, ldy] (heads
 * of 2 * rope_half columns, pairs (i, i + rope_half)); positions int32 [M] clamped into the fp32
 * tables [rope_positions, rope_half]; rope_bf16 selects pi0.5's bf16 arithmetic -- the rotary
 * epilogue of tk_bf16w_linear as a launch of its own
 * (tybok/policies/smolvla/models/rope.py:51-73, tybok/policies/pi05/models/layers.py:101-128). */
int tk_rope_rows(void* y, int ldy, const void* rope_pos, const void* rope_cos, const void* rope_sin, int rope_positions,
                 int rope_cols, int rope_half, int rope_bf16, int M, void* stream);

/* Per-request bookkeeping of the prefix in one launch: from the pad flags (and the attention-block flags) of the P
 * prefix tokens, the prefill's 2-D visibility, the rotary positions of the prefix and those of the S action tokens:
 *   mask2d[i][j] = (cumsum(att)[j] <= cumsum(att)[i]) & pad[i] & pad[j]   bytes, row pitch p_pad (columns >= P zero)
 *   pos32[j]     = clamp(cumsum(pad)[j] - 1, 0, rope_positions - 1)       int32
 *   suf_pos[s]   = clamp(sum(pad) + s, 0, rope_positions - 1)             int32
 * (`make_att_2d_masks` and `position_ids = cumsum(pad_masks) - 1`, tybok/policies/smolvla/models/flow_matching.py:
 * 40-58,527-546; `prefix_pad.sum(-1) + arange(S)`, :343-350; tybok/policies/pi05/models/flow_matching.py:
 * 440-470,609-640 with att all zero.)  pad, att: P bytes of 0 / 1 (att may be NULL); any output may be NULL;
 * P <= 2048; p_pad a multiple of 16 >= P; mask2d 16-byte aligned. */
int tk_prefix_meta(const void* pad, const void* att, int P, int p_pad, int rope_positions, int S, void* mask2d, void* pos32,
                   void* suf_pos, void* stream);

/* The unfolded input of a vision tower's patch embedding in one launch: n <= 4 fp32 images [3, H, W] ->
 * bf16 rows [(image, patch row, patch column)][(channel, i, j)] of x * scale + shift (product and sum rounded to
 * fp32 one after the other, then to bf16) -- `images * 2 - 1`, the cast and `unfold` in front of the patch GEMM
 * (tybok/policies/smolvla/policy.py:117-163, tybok/policies/smolvla/models/vision.py:120-160).  patch a multiple of 8
 * that divides H and W; images and out 16-byte aligned; images beyond n are ignored. */
int tk_patchify_images(const void* img0, const void* img1, const void* img2, const void* img3, int n, int H, int W, int patch,
                       float scale, float shift, void* out, void* stream);
/* The same with fp32 patch rows and any even patch size (pi0.5's SigLIP tower: 14 x 14 patches, fp32 patch embedding,
 * tybok/policies/pi05/models/vision.py:100-118 after `img * 2 - 1` of tybok/policies/pi05/policy.py:170-234). */
int tk_patchify_images_f32(const void* img0, const void* img1, const void* img2, const void* img3, int n, int H, int W, int patch,
                           float scale, float shift, void* out, void* stream);

/* The prefix rows of a request in one launch, in the type the prefill reads (fp32): the connector's rows of all cameras
 * times the image scale, the language tokens' embedding rows times theirs (both products rounded to bf16 first, as a bf16
 * tensor times a scalar is), then closing rows as they are (the projected state) -- what scaling, embedding lookup and
 * concatenation build in `embed_prefix` (tybok/policies/smolvla/models/flow_matching.py:160-257) -- and, optionally, the
 * pad flags of the same rows (a flag per camera, a flag per token, 1 for the closing rows).
 *   img: bf16 [n_img, H] (img_dtype TK_BF16), or fp32 (TK_F32: pi0.5's projector output,
 *   tybok/policies/pi05/models/flow_matching.py:415-437 -- those rows are taken as they are, img_scale unused);
 *   table: bf16 [vocab, H]; tokens: int64 [n_tok] (ids are clamped into the table); last: fp32 [n_last, H];
 *   out: [n_img + n_tok + n_last, H] fp32 (out_dtype TK_F32) or rounded to bf16 (TK_BF16: the prefill's hidden rows,
 *   `embs.to(bfloat16)`); H a multiple of 8; 16-byte aligned rows.
 *   pad_out: bytes [n_img + n_tok + n_last] or NULL; cam_flag0..3: one byte each (the first `cams` are read, n_img a
 *   multiple of cams); tok_flag: bytes [n_tok]. */
int tk_prefix_rows(const void* img, int img_dtype, int n_img, float img_scale, const void* table, const void* tokens, int n_tok,
                   int vocab, float tok_scale, const void* last, int n_last, void* out, int out_dtype, int H, const void* cam_flag0,
                   const void* cam_flag1, const void* cam_flag2, const void* cam_flag3, int cams, const void* tok_flag, void* pad_out,
                   void* stream);

/* LayerNorm of token rows with the cast to the GEMM input type folded in:
 *   y[m, :] = bf16((x[m, :] - mean) * rstd * w + b), statistics in fp32 (biased variance).
 * Replaces `layer_norm1/2(x)` (+ the `.to(bf16)` of the low-precision tiers) in the encoder layers
 * (tybok/policies/pi05/models/vision.py:115-170, tybok/policies/smolvla/models/vision.py:197-257).
 *   x: fp32 or bf16 [M, K] (x_dtype, element pitch ldx); w, b: [K] of the same type (wb_dtype);
 *   y: bf16 [M, K] (pitch ldy); K a multiple of 8, at most 2048; pitches multiples of 8; 16-byte aligned. */
int tk_layer_norm(const void* x, int ldx, int x_dtype, const void* w, const void* b, int wb_dtype, float eps, void* y, int ldy,
                  int M, int K, void* stream);

/* The residual add that closes a tower branch and the LayerNorm that opens the next one, in one
 * launch: xsum = x + r (r bf16 [M, K]: the branch's last linear; the sum in x's type -- fp32 rows:
 * x + float(r); bf16 rows: rounded once -- and xsum may be x itself), y = bf16(LayerNorm(xsum) * w + b).
 * Other arguments as tk_layer_norm (`hidden = residual + hidden; hidden = layer_norm(hidden)`,
 * tybok/policies/smolvla/models/vision.py:197-257, tybok/policies/pi05/models/vision.py:115-170). */
int tk_add_layer_norm(const void* x, int ldx, int x_dtype, const void* r, int ldr, void* xsum, int ldxs, const void* w,
                      const void* b, int wb_dtype, float eps, void* y, int ldy, int M, int K, void* stream);

/* tk_add_layer_norm with the normalised rows written in another order: row m of the result goes to row y_rows[m] of y
 * (int32 [M] on the device, a permutation of 0..M-1; values outside that range are clamped into it).  The tower's
 * closing LayerNorm followed by the pixel shuffle, which moves whole token rows
 * (tybok/policies/smolvla/models/vision.py:197-257 and the connector's `pixel_shuffle` in front of its projection).
 * y must not alias x or xsum. */
int tk_add_layer_norm_rows(const void* x, int ldx, int x_dtype, const void* r, int ldr, void* xsum, int ldxs, const void* w,
                           const void* b, int wb_dtype, float eps, void* y, int ldy, const void* y_rows, int M, int K,
                           void* stream);

/* tk_layer_norm for fp32 rows and fp32 parameters with the normalised row rounded to IEEE fp16 instead of bf16:
 * the LayerNorm + cast in front of the fp16 q|k|v projection of pi0.5's fused tower (`n.to(tl.float16)`,
 * tybok/policies/pi05/models/triton_vision.py:93-95) and of the `--vit-mlp-dtype fp16` MLP
 * (tybok/policies/pi05/models/vision.py:79-87). */
int tk_layer_norm_f16(const void* x, int ldx, const void* w, const void* b, float eps, void* y, int ldy, int M, int K,
                      void* stream);
/* tk_add_layer_norm for fp32 rows and parameters (bf16 residual branch) with the normalised row rounded to fp16. */
int tk_add_layer_norm_f16(const void* x, int ldx, const void* r, int ldr, void* xsum, int ldxs, const void* w, const void* b,
                          float eps, void* y, int ldy, int M, int K, void* stream);

/* ---- tail of a denoising step ---------------------------------------------------------------- */
/* Final norm of the expert hidden state + fp32 action projection + Euler update in one launch:
 *   h = norm(x) (bf16 row; norm_w: Llama RMSNorm bf16(w * bf16(x * rstd)); or ada_scale / ada_shift:
 *   adaptive RMSNorm bf16((x * rstd) * (1 + scale) + shift)),  v = float(h) . W^T + bias (fp32),
 *   x_out = x_t + dt * v.
 * Replaces the tail of `denoise_step` and the `x_t + dt * v_t` of the Euler loop
 * (tybok/policies/smolvla/models/flow_matching.py:343-350,612-620,
 *  tybok/policies/pi05/models/flow_matching.py:547-556,228-240).
 *   x: bf16 [M, K] (row pitch ldx); w: fp32 [N, K]; bias: fp32 [N] or NULL; N must divide 256.
 *   v_out: fp32 [M, N] or NULL; x_t / x_out: fp32 [M, N] or both NULL (x_out may alias x_t). */
int tk_expert_tail(const void* x, int ldx, const void* norm_w, const void* ada_scale, const void* ada_shift, float eps,
                   const void* w, const void* bias, void* v_out, const void* x_t, void* x_out, float dt, int M, int N,
                   int K, void* stream);

/* tk_expert_tail plus the next denoising step's suffix embedding from the updated x, in the same launch:
 *   emb_out[m, j] = act( sum_n x_out[m, n] * emb_w[j, n] + emb_b[j] ),  j < emb_n, fp32 arithmetic
 * -- the first linear of `embed_suffix` applied to the action chunk: SmolVLA's `action_in_proj` folded with the
 * action half of `action_time_mlp_in` (the time half, constant per step, folded into emb_b) and its SiLU
 * (tybok/policies/smolvla/models/flow_matching.py:259-311); pi0.5's `action_in_proj` with the cast to bf16
 * (tybok/policies/pi05/models/flow_matching.py:464-502).
 *   x_t / x_out required; N must be 32 (the padded action width).
 *   emb_w: fp32 [emb_n, N], 16-byte aligned; emb_b: fp32 [emb_n] or NULL; emb_act: 0 none, 1 SiLU;
 *   emb_out: [M, emb_n] with row pitch emb_ld (elements), emb_dtype TK_F32 or TK_BF16 (rounded once). */
int tk_expert_tail_embed(const void* x, int ldx, const void* norm_w, const void* ada_scale, const void* ada_shift, float eps,
                         const void* w, const void* bias, void* v_out, const void* x_t, void* x_out, float dt, int M, int N,
                         int K, const void* emb_w, const void* emb_b, int emb_n, int emb_act, void* emb_out, int emb_ld,
                         int emb_dtype, void* stream);

/* ---- diagnostics: helpers of the tests and the benchmark; no policy path calls them -------------- */
/* out_f32[256] = value of every e4m3fn code as decoded by the device's conversion instruction
 * (the weight path of the GEMM); used to assert the OCP (not FNUZ) flavour on the box. */
int tk_debug_decode_fp8(void* out_f32, void* stream);

/* Reads `bytes` of device memory at `src` with a plain streaming kernel (16 bytes per lane, `blocks`
 * blocks of 256 threads, bytes a multiple of blocks * 4096) and discards them: the yardstick for the
 * weight-streaming launches -- what one dependent launch of that size can pull from HBM on this device.
 * `sink` (int32, may be NULL) is never written for real data.  No counterpart in the reference. */
int tk_debug_stream_read(const void* src, size_t bytes, int blocks, void* sink, void* stream);

/* Measurement forms of the weight-streaming fp8 GEMM (the kernel tk_fp8w_gemm launches for 33..64 rows
 * over a large matrix): same grid, same schedule, the work behind a point dropped.  cut 1 = the weight
 * and activation loads and the barrier per round only; 2 = + activations staged into LDS; 3 = + operands
 * read back from LDS; 4 = + fp8 -> bf16 conversion and the matrix instructions (no exchange between
 * waves, no scales, no output).  Nothing is written to y.  Timed by `bench.py --gemm-only` beside the
 * whole kernel to show where its time above a plain read of the weights goes.  Only unsplit launches of
 * the 16-round kernel (K = 2048, M <= 64, N >= 64); TK_EINVAL otherwise.  No counterpart in the reference. */
int tk_debug_fp8w_gemm_cut(const void* x, int ldx, const void* w_packed, const void* scale, void* y, int ldy,
                           int M, int N, int K, int cut, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TYBOK_HIP_H */
