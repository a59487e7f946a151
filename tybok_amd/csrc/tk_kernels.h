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
  float* partial;
  int* counters;
  int act;
  int vec;  // the plain epilogue may use 8/16-byte accesses (alignment and N % 4 checked by the host)
  // RMSNorm prologue (norm_w != nullptr): bf16 [K] weight, eps
  const unsigned short* norm_w;
  float norm_eps;
  // rotary epilogue (rope_pos != nullptr): int32 [M] positions, fp32 [positions, rope_half] tables,
  // columns < rope_cols are rotated in pairs (c, c + rope_half)
  const int* rope_pos;
  const float* rope_cos;
  const float* rope_sin;
  int rope_positions;  // rows of the tables (positions are clamped into them)
  int rope_cols;
  int rope_half;
};

struct AttnArgs {
  const unsigned short* q;
  int q_sm, q_sh;
  const void* k_pre;
  const void* v_pre;
  int pre_sl, pre_sh;
  const unsigned short* k_suf;
  const unsigned short* v_suf;
  int suf_sl, suf_sh;
  const uint8_t* pad;
  unsigned short* out;
  int out_sm;
  int M, P, S, H, G;
  int mask_mode, logits_bf16;
  int kv_splits;
  float* partial;
  int* counters;
  float scale;
};

int tk_launch_gemm(GemmArgs a, int MT, int NT, int mblocks, hipStream_t st);
int tk_launch_pack(const void* w0, const void* w1, void* out, int N, int K, int interleave, hipStream_t st);
int tk_launch_pack_bf16(const void* w, void* out, int N, int K, int pair_off, hipStream_t st);
int tk_launch_fill_zero(int* p, int n, hipStream_t st);
int tk_launch_decode_fp8(float* out, hipStream_t st);
int tk_launch_attn(AttnArgs a, int D, int kv_f32, hipStream_t st);
