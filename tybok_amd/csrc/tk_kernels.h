// Internal launch interface between the C ABI (tk_api.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

struct GemmArgs {
  const void* x;  // bf16 (or fp32 when x_f32) [M, K]
  int ldx;
  int x_f32;
  int w16;  // weights are bf16 tiles (2 KiB) instead of e4m3 tiles (1 KiB)
  const uint8_t* w;  // packed 32x32-byte tiles, tile (nt, kt) at ((nt*KT)+kt)*1024
  const float* s0;   // scale (plain) or gate scale (gated)
  const float* s1;   // up scale (gated) or nullptr
  unsigned short* y;
  int ldy;
  const void* resid;
  int ldr;
  int resid_f32;
  const unsigned short* gate;  // bf16 [N] per-column gate applied before the residual, or nullptr
  int M, N, K;  // N: logical output columns (gated: the intermediate size I)
  int KT;       // k tiles of 32
  int ntiles;   // n tiles of 32 in the packed buffer (gated: 2 * I / 32)
  int ksplit;
  int kt_q, kt_r;  // KT = ksplit * kt_q + kt_r
  float* partial;
  int* counters;
  int cstride;  // int32 words between two arrival counters (16: a 64-byte line each -- counters that share a line queue up)
  int act;
  int vec;  // the plain epilogue may use 8/16-byte accesses (alignment and N % 4 checked by the host)
  // RMSNorm prologue (norm_w != nullptr): bf16 [K] weight, eps
  const unsigned short* norm_w;
  float norm_eps;
  // adaptive RMSNorm prologue (ada_scale != nullptr): fp32 [K] scale and shift, same eps
  const float* ada_scale;
  const float* ada_shift;
  // rotary epilogue (rope_pos != nullptr): int32 [M] positions, fp32 [positions, rope_half] tables,
  // columns < rope_cols are rotated in pairs (c, c + rope_half)
  const int* rope_pos;
  const float* rope_cos;
  const float* rope_sin;
  int rope_positions;  // rows of the tables (positions are clamped into them)
  int rope_cols;
  int rope_half;
  int rope_bf16;  // rotate in bf16 arithmetic (tables hold bf16 values)
  // rotary epilogue only: columns >= vt_col0 are also written transposed, vt[(n - vt_col0) * vt_ld + m]
  unsigned short* vt;
  int vt_col0;
  int vt_ld;
  // many-row 16-bit kernel only: the rows are vt_rows-row problems (0 = one problem) and problem b's transposed
  // columns start vt_bs elements after problem b-1's: vt[(m / vt_rows) * vt_bs + (n - vt_col0) * vt_ld + m % vt_rows]
  int vt_rows;
  long long vt_bs;
  // W8A8 launches only: x holds e4m3fn codes (ldx in bytes) and row_scale the per-token fp32 scales
  const float* row_scale;
  // many-row kernels: y (and the residual) allow 16-byte row-contiguous accesses (pitches multiples of 8
  // elements, 16-byte aligned pointers): the epilogue stores whole row segments through LDS
  int vec16;
  // bf16-weight many-row kernel only: bf16 [N] bias added to the accumulator, or nullptr; there act is
  // 0 none, 1 tanh-GELU of the bf16-rounded pre-activation, 2 tanh-GELU of the fp32 pre-activation
  const unsigned short* bias;
  // many-row fp8 kernels: 32-row tiles per block, chosen by the host (2 / 4: four-wave blocks; 6 / 8: eight-wave
  // blocks with both operands through LDS, weight-only kernel)
  int mtiles;
  // many-row 16-bit-weight kernel only: activations, weights, bias, output and a 16-bit residual are fp16, not bf16
  int f16;
  // single-launch gated FFN only: the hand-off words in the workspace (TK_FUSE_* below), the down blocks per row
  // block, and the bound on a down block's wait (polls)
  int* fuse;
  int fuse_consumers, fuse_spin;
  // many-row fp8 kernels, K splits of a plain launch: 1 = every block leaves its fp32 partial in `partial` and ends;
  // a second launch (all CUs, not one block per output tile) sums them in split order and runs the epilogue
  int split_reduce;
};
// int32 words of the single-launch FFN's hand-off: a flag per (row block, gate/up strip), the number of down blocks
// past their wait per row block, then the sticky error word
#define TK_FUSE_ROWBLOCKS 2
#define TK_FUSE_STRIPS 512
#define TK_FUSE_PAST (TK_FUSE_ROWBLOCKS * TK_FUSE_STRIPS)
#define TK_FUSE_ERROR (TK_FUSE_PAST + TK_FUSE_ROWBLOCKS)
#define TK_FUSE_WORDS 2048

struct QuantActArgs {
  const unsigned short* x;  // bf16 [M, K], element pitch ldx
  int ldx;
  unsigned char* a8;  // e4m3fn [M, K], byte pitch lda
  int lda;
  float* sa;  // fp32 [M]
  int M, K;
  int mode;  // 0: fp32 scale, one rounding; 1: bf16-rounded scale and quotient
};

struct AttnArgs {
  const unsigned short* q;
  int q_sm, q_sh;
  // prefix: K [P, G, D] (element strides pre_sl, pre_sh) and V^T [G, D, >= roundup(P, 32)]
  // (element strides pre_vt_sh, pre_vt_sd); the *_lo planes are nullptr unless K/V were fp32
  const unsigned short* k_pre;
  const unsigned short* k_pre_lo;
  const unsigned short* vt_pre;
  const unsigned short* vt_pre_lo;
  int pre_sl, pre_sh, pre_vt_sd, pre_vt_sh;
  const unsigned short* k_suf;
  const unsigned short* vt_suf;
  int suf_sl, suf_sh, suf_vt_sd, suf_vt_sh;
  const uint8_t* pad;
  const uint8_t* mask2d;  // [M, mask_ld] per-(query, prefix key) visibility; overrides pad when set
  int mask_ld;
  unsigned short* out;
  int out_sm;
  int M, P, S, H, G;
  // independent problems in one launch (prefix-only): element strides between them, 0 = single
  int batch;
  int xcd_remap;  // batched, unsplit launches: 1-D grid with (problem, head) pairs pinned to an XCD
  long long q_sb, k_sb, vt_sb, out_sb;
  int mask_mode, logits_bf16;
  int f16;  // tower kernel only: q, K, V^T and the probabilities are fp16 (the output stays bf16)
  int kv_splits;
  int tile_q, tile_r;  // key tiles = kv_splits * tile_q + tile_r
  int gqa_mul;         // kv head of query head h = (h * gqa_mul) >> 16
  float* partial;
  int* counters;
  float scale;
  // in-kernel query projection (cross layers; nullptr / 0 otherwise): hidden rows bf16 [M, qp_ldx],
  // RMSNorm weight bf16 [qp_K], packed bf16 q weight (rotary pair order, tiles of 2 KiB, qp_KT k
  // tiles per n tile), rotary tables fp32 [qp_positions, D/2] and int32 positions [M]
  const unsigned short* qp_x;
  int qp_ldx;
  const unsigned short* qp_norm_w;
  float qp_eps;
  const uint8_t* qp_w;
  int qp_K, qp_KT;
  const int* qp_rope_pos;
  const float* qp_cos;
  const float* qp_sin;
  int qp_positions;
};

struct KvPrepArgs {
  const void* k;  // [L, G, D] with element strides (sl, sh); fp32 when f32, else bf16 (k unused)
  const void* v;
  int f32;
  int sl, sh;
  int L, G, D;
  unsigned short* k_hi;  // [L, G, D] contiguous (fp32 sources only)
  unsigned short* k_lo;
  unsigned short* vt_hi;  // [G, D, ld]
  unsigned short* vt_lo;  // fp32 sources only
  int ld;
};

constexpr int kKvProjMaxLayers = 16;
struct KvProjArgs {
  int L;                                        // layers in this launch (<= kKvProjMaxLayers)
  const unsigned short* k[kKvProjMaxLayers];    // per layer: bf16 [P, KV] rows (element stride sl)
  const unsigned short* v[kKvProjMaxLayers];
  int sl;
  const float* wk[kKvProjMaxLayers];            // per layer: fp32 [N, KV]
  const float* wv[kKvProjMaxLayers];
  int P, KV, N;
  unsigned short* k_hi;  // [L][P, N]
  unsigned short* k_lo;
  unsigned short* vt_hi;  // [L][N, ld], ld >= P rounded up to 32
  unsigned short* vt_lo;
  int ld;
};

struct LayerNormArgs {
  const void* x;  // fp32 (x_f32) or bf16 [M, K] rows, element pitch ldx
  int ldx, x_f32;
  const void* w;  // fp32 (wb_f32) or bf16 [K]
  const void* b;
  int wb_f32;
  float eps;
  unsigned short* y;  // bf16 (fp16 when y_f16) [M, K], element pitch ldy
  int ldy;
  int y_f16;
  int M, K;
  // optional residual branch: rows are x + r (r bf16, pitch ldr), the sum goes to xsum in x's type
  // (pitch ldxs; may be x itself)
  const unsigned short* r;
  int ldr;
  void* xsum;
  int ldxs;
  // optional: row m of the result goes to row y_rows[m] of y (a permutation of 0..M-1; values outside are clamped)
  const int* y_rows;
};

struct TailArgs {
  const unsigned short* x;  // bf16 [M, K]
  int ldx;
  const unsigned short* norm_w;  // bf16 [K] (RMSNorm) or nullptr with ada_scale / ada_shift
  const float* ada_scale;
  const float* ada_shift;
  float eps;
  const float* w;     // fp32 [N, K]
  const float* bias;  // fp32 [N] or nullptr
  float* v_out;       // fp32 [M, N] or nullptr
  const float* x_t;   // fp32 [M, N] (with x_out)
  float* x_out;       // fp32 [M, N] or nullptr
  float dt;
  int M, N, K;
  // optional (with x_out, N == 32): emb_out[m, j] = act(sum_n x_out[m, n] * emb_w[j, n] + emb_b[j]), j < emb_J
  const float* emb_w;  // fp32 [emb_J, N]
  const float* emb_b;  // fp32 [emb_J] or nullptr
  void* emb_out;       // fp32 or bf16 [M, emb_J], row pitch emb_ld elements
  int emb_J, emb_ld, emb_act, emb_bf16;  // act: 0 none, 1 SiLU
};

struct NormRowsArgs {
  const unsigned short* x;  // bf16 [M, K]
  int ldx;
  const unsigned short* norm_w;  // bf16 [K] (RMSNorm) or nullptr with ada_scale / ada_shift
  const float* ada_scale;
  const float* ada_shift;
  float eps;
  unsigned short* out;  // bf16 [M, K]
  int ldo;
  int M, K;
};

struct RopeRowsArgs {
  unsigned short* y;  // bf16 [M, ldy], rotated in place in columns < rope_cols
  int ldy;
  const int* pos;  // int32 [M], clamped into the table
  const float* cos;  // fp32 [positions, half]
  const float* sin;
  int positions, rope_cols, half, bf16_math;
  int M;
};
int tk_launch_rope_rows(RopeRowsArgs a, hipStream_t st);

struct PrefixMetaArgs {
  const unsigned char* pad;  // [P] 0 / 1
  const unsigned char* att;  // [P] 0 / 1, or null (all zero)
  int P, p_pad, positions, S;
  unsigned char* mask2d;  // [P][p_pad] or null
  int* pos;               // [P] or null
  int* suf_pos;           // [S] or null
};
int tk_prefix_meta_max_tokens();
int tk_launch_prefix_meta(PrefixMetaArgs a, hipStream_t st);

struct PatchifyArgs {
  const float* img[4];  // fp32 [3][H][W] each
  int n, H, W, ps;
  float scale, shift;
  void* out;  // bf16 (ps a multiple of 8) or fp32 (out_f32; ps even) [n * (H/ps) * (W/ps)][3 * ps * ps]
  int out_f32;
};
int tk_launch_patchify(PatchifyArgs a, hipStream_t st);

struct PrefixRowsArgs {
  const void* img;  // bf16 [n_img, H]: rows 0 .. n_img-1 of the result are bf16(img * img_scale); fp32 (img_f32): the rows as they are
  int n_img, img_f32;
  float img_scale;
  const unsigned short* table;  // bf16 [vocab, H]: rows n_img .. n_img+n_tok-1 are bf16(table[tokens[t]] * tok_scale)
  const long long* tokens;
  int n_tok, vocab;
  float tok_scale;
  const float* last;  // fp32 [n_last, H]: the closing rows, as they are
  int n_last;
  void* out;  // fp32, or bf16 (out_bf16: every value rounded once more, a no-op for the scaled rows) [n_img + n_tok + n_last, H]
  int H, out_bf16;
  // optional pad flags of the same rows: a flag per camera (n_img = cams * per_cam rows), a flag per token, 1 for the closing rows
  const unsigned char* cam_flag[4];
  int cams, per_cam;
  const unsigned char* tok_flag;
  unsigned char* pad_out;
};
int tk_launch_prefix_rows(PrefixRowsArgs a, hipStream_t st);
int tk_launch_norm_rows(NormRowsArgs a, hipStream_t st);
int tk_launch_tail(TailArgs a, hipStream_t st);
int tk_tail_embed_width();  // the embedding's input width the tail kernel is built for
int tk_launch_kv_proj(KvProjArgs a, hipStream_t st);
int tk_layer_norm_max_k();
int tk_launch_layer_norm(LayerNormArgs a, hipStream_t st);
int tk_wide_cols();  // columns of the many-row GEMM's block tile (rows: 32 * GemmArgs::mtiles)
int tk_launch_gemm_wide(GemmArgs a, hipStream_t st);
int tk_launch_norm_rows(NormRowsArgs a, hipStream_t st);
int tk_launch_gemm(GemmArgs a, int MT, int NT, int mblocks, hipStream_t st);
// the action chunk's gated FFN in one launch (32-row blocks; g: the gate/up half without a K split, d: the down half
// with NT n tiles per strip); -1 when the pair of shapes is not one of the built combinations
int tk_launch_ffn_fused(GemmArgs g, GemmArgs d, int d_nt, int mblocks, hipStream_t st);
// at most 64 rows over a large fp8 matrix, plain epilogue, every block 8 or 16 rounds of four k tiles: the
// software-pipelined kernel of fp8w_gemm_stream.hip (same grid and partial layout as tk_launch_gemm with MT = NT = 2)
bool tk_gemm_stream_takes(const GemmArgs& a);
int tk_launch_gemm_stream(GemmArgs a, hipStream_t st);
int tk_launch_gemm_stream_cut(GemmArgs a, int cut, hipStream_t st);  // measurement forms, nothing stored
// W8A8 tier: per-token activation quantisation and the fp8 x fp8 many-row GEMM (block tile 32 * mtiles x tk_w8a8_cols())
int tk_w8a8_cols();
int tk_quant_act_max_k();
int tk_launch_w8a8_gemm(GemmArgs a, hipStream_t st);
int tk_launch_quant_act_rows(QuantActArgs a, hipStream_t st);
int tk_launch_pack(const void* w0, const void* w1, void* out, int N, int K, int interleave, hipStream_t st);
int tk_launch_pack_bf16(const void* w, void* out, int N, int K, int pair_off, hipStream_t st);
int tk_launch_fill_zero(int* p, int n, hipStream_t st);
int tk_launch_decode_fp8(float* out, hipStream_t st);
// tile = 10 * (m tiles per block) + (n tiles per wave): 42, 41, 32, 31, 22, 21, 12 or 11
int tk_launch_bf16w_wide(const GemmArgs& a, int tile, hipStream_t st);
// plain 16-byte-per-lane read of `bytes` (a multiple of blocks * 4096) by `blocks` blocks of 256 threads
int tk_launch_stream_read(const void* src, size_t bytes, int blocks, int* sink, hipStream_t st);
struct TransposeVArgs {
  const unsigned short* v;  // bf16 [B, P, G, D], element strides (v_sb, v_sl, v_sh), d contiguous
  long long v_sb;
  int v_sl, v_sh;
  unsigned short* vt;  // bf16 [B, G, D, ld], element strides (vt_sb, vt_sh, vt_sd), keys contiguous
  long long vt_sb;
  int vt_sh, vt_sd;
  int ld;  // keys a V^T row can hold (a multiple of 8)
  int B, P, G;
};
int tk_launch_transpose_v(TransposeVArgs a, int D, hipStream_t st);
// vision-tower self-attention (batched, unmasked, prefix-only, head size 64 / 96): 128 queries per block
int tk_launch_tower_attn(AttnArgs a, int D, int cus, hipStream_t st);  // cus: compute units of the device (block shape by grid fill)
int tk_attn_waves(int D, int split_planes, int ntiles);
int tk_launch_attn(AttnArgs a, int D, int waves, hipStream_t st);
// 256-wide heads: blocks of 8 waves that walk their share of the key tiles 8 at a time (a.kv_splits blocks per query tile)
int tk_launch_attn_d256(AttnArgs a, hipStream_t st);
int tk_attn_d256_max_splits();
int tk_attn_d256_tiles_per_block();
// 64-wide heads, whole key range (at most tk_attn_px_max_tiles() tiles) in one block: probabilities exchanged
// between the waves instead of partial outputs
int tk_launch_attn_px(AttnArgs a, int D, hipStream_t st);
int tk_attn_px_max_tiles();
int tk_launch_attn_cross_px(AttnArgs a, hipStream_t st);
int tk_launch_kv_prepare(KvPrepArgs p, hipStream_t st);
