// Action-expert attention over [cached prefix KV ; suffix KV] for one request on gfx950.
//
//   out[M, H*D] = softmax(q . K^T * D^-0.5 (+mask)) . V        (GQA: q head h -> kv head h/(H/G))
//
// Tiny and latency-bound (50 queries, a few hundred keys): the kernel is built so that a wave
// issues every global load it needs up front and then runs a short, branch-light instruction
// stream.  Grid = (head, 32-query tile, kv split); the four waves of a block take 32-key tiles
// round-robin (normally one tile per wave).
//   * Both MFMA operands stream from global memory in operand order, 16 bytes per lane, with no
//     LDS staging: K rows as the A operand of S^T[key, q] = K . Q^T, and V from a TRANSPOSED
//     cache V^T[kv head, d, key] as the A operand of O^T[d, q] += V^T . P^T.  The prefix V^T is
//     laid out once per request (tk_attn_prepare_kv), the suffix V^T by the projection kernel's
//     epilogue.  Keys beyond a segment's length read zero-padded V^T columns.
//   * In this orientation one lane owns one query column, so the softmax max/sum are in-lane plus
//     one cross-half exchange, and P^T is already the B operand of P.V.  K rows are assigned to
//     lanes through a fixed permutation so that accumulator registers 8s..8s+7 of a lane are
//     eight CONSECUTIVE keys -- exactly one 16-byte chunk of a V^T row.
//   * fp32 K/V (SmolVLA cross layers) come as bf16 hi + lo planes (x = hi + lo to 16 mantissa
//     bits), split once per request; P is split the same way in registers (3 MFMAs for P.V).
//   * Online softmax per wave, then a fixed-order merge over waves (LDS) and kv splits (global
//     partials handed over with device-coherent accesses, last-arriving block finishes) --
//     deterministic, no atomics on data.  Wave w owns rows d = 8w + 4*(lane/32) + 0..3 of every
//     output d tile in the merges and writes them as one 8-byte store per query.
#include <math.h>
#include "tk_common.h"
#include "tk_kernels.h"


namespace {

constexpr float kF32Min = -3.4028234663852886e38f;    // finfo(float32).min
constexpr float kOpenpiMask = -2.3819763e38f;         // additive mask of the pi0.5 path

// K row held by MFMA row r of a key tile: swaps bits 2 and 3 of r (see the header comment)
__device__ __forceinline__ int key_of_row(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

__device__ __forceinline__ bf16x8 pack_bf16x8(const float* v) {
  union { unsigned u[4]; bf16x8 b; } r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r.u[j] = pack_bf16x2(v[2 * j], v[2 * j + 1]);
  return r.b;
}

// NWV waves per block, one 32-key tile each per pass.  With few key tiles (the action expert:
// 8-10) a block of 8 or 12 waves covers the whole key range, so the waves merge through LDS only and
// the global partial hand-off between kv splits (two more round trips) is not needed.
template <int D, bool SPLIT, int NWV>
__global__ __launch_bounds__(NWV * 64) void expert_attn_kernel(AttnArgs a) {
  constexpr int kNW = NWV;
  constexpr int DT = D / 32;                 // d tiles of the output
  constexpr int DS = D / 16;                 // k steps of Q.K^T
  constexpr int PL = SPLIT ? 2 : 1;          // operand planes (hi, lo)
  constexpr int PF = (NWV > 4 || D > 128) ? 1 : 2;  // key tiles in flight per wave
  // D = 256: the query tile (the same for every wave of the block) lives in LDS instead of 64
  // registers per lane -- with it in registers the kernel spills to scratch
  constexpr bool QLDS = D >= 256;
  constexpr int QPITCH = D * 2 + 16;         // bytes; 16-byte operand reads of 32 rows stay conflict-free
  __shared__ __align__(16) f32x4 red[DT][kNW][4][64];  // every wave's partial output tiles, exchanged at once
  __shared__ float st_m[kNW][32], st_l[kNW][32];
  __shared__ __align__(16) unsigned char qs[QLDS ? 32 * QPITCH : 16];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: keeps tile indices scalar
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int mtiles = (a.M + 31) >> 5;
  int h = blockIdx.x;
  int bi = blockIdx.y / mtiles;              // problem of a batched launch
  int mtile = blockIdx.y % mtiles;
  const int split = blockIdx.z;
  if (a.xcd_remap) {
    // Large batched launches (vision tower): a 1-D grid whose workgroups the dispatcher deals
    // round-robin to the 8 XCDs.  All query tiles of one (problem, head) pair are given to the same
    // XCD, so that pair's K / V^T (re-read by every query tile) stays in that XCD's L2.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int pair = (slot / mtiles) * 8 + xcd;
    if (pair >= a.batch * a.H) return;
    mtile = slot % mtiles;
    bi = pair / a.H;
    h = pair % a.H;
  }
  a.q += bi * a.q_sb;
  a.k_pre += bi * a.k_sb;
  a.vt_pre += bi * a.vt_sb;
  a.out += bi * a.out_sb;
  const int g = (h * a.gqa_mul) >> 16;       // h / (H / G) without a runtime divide
  const int tp = (a.P + 31) >> 5;            // prefix tiles; suffix tiles follow
  const int t_lo = split * a.tile_q + (split < a.tile_r ? split : a.tile_r);
  const int t_hi = t_lo + a.tile_q + (split < a.tile_r ? 1 : 0);
  const int qi = mtile * 32 + l32;
  const bool q_ok = qi < a.M;

  struct Stage {
    i32x4 k[PL][DS];
    i32x4 v[PL][DT][2];
    int pad;
    unsigned long long m2[2];  // per-query visibility bytes of the tile's keys (mask2d)
  };
  // every load of a key tile, issued back to back (t is wave-uniform)
  auto load = [&](Stage& st, int t) {
    const bool pre = t < tp;
    const int tt = pre ? t : t - tp;
    const int len = pre ? a.P : a.S;
    int kr = tt * 32 + key_of_row(l32);
    if (kr > len - 1) kr = len - 1;  // masked below; keeps the address valid and the value finite
    const size_t koff = (size_t)kr * (pre ? a.pre_sl : a.suf_sl) + (size_t)g * (pre ? a.pre_sh : a.suf_sh) + 8 * half;
    const size_t vsd = pre ? a.pre_vt_sd : a.suf_vt_sd;
    const size_t voff = (size_t)g * (pre ? a.pre_vt_sh : a.suf_vt_sh) + (size_t)l32 * vsd + tt * 32 + 8 * half;
#pragma unroll
    for (int pl = 0; pl < PL; ++pl) {
      const u16* kb = pre ? (pl ? a.k_pre_lo : a.k_pre) : a.k_suf;
      const u16* vb = pre ? (pl ? a.vt_pre_lo : a.vt_pre) : a.vt_suf;
#pragma unroll
      for (int s = 0; s < DS; ++s) st.k[pl][s] = *(const i32x4*)(kb + koff + 16 * s);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int s = 0; s < 2; ++s) st.v[pl][dt][s] = *(const i32x4*)(vb + voff + (size_t)dt * 32 * vsd + 16 * s);
    }
    // visibility operands, always requested (from a harmless valid address when unused): a branch
    // around a load would make the compiler wait for every outstanding load before each tile
    const bool use_m2 = pre && a.mask2d != nullptr;
    const bool use_pad = pre && a.mask2d == nullptr && a.pad != nullptr;
    const int key = tt * 32 + l32;
    const uint8_t* mp = use_m2 ? a.mask2d + (size_t)(q_ok ? qi : a.M - 1) * a.mask_ld + tt * 32 + 8 * half : (const uint8_t*)a.q;
    st.m2[0] = *(const unsigned long long*)mp;  // eight consecutive keys: registers 8s..8s+7 of this lane
    st.m2[1] = *(const unsigned long long*)(mp + (use_m2 ? 16 : 8));
    const uint8_t* pp = (use_pad && key < a.P) ? a.pad + key : (const uint8_t*)a.q;
    const int padv = *pp;
    st.pad = use_pad ? (key < a.P ? padv : 0) : 1;
  };

  // tiles of this wave: t_lo + wave + kNW * i, i < nt_w; indices past the end are clamped to a valid
  // tile so that every prefetch is unconditional (never processed)
  const int nt_w = t_hi - t_lo > wave ? (t_hi - t_lo - wave + kNW - 1) / kNW : 0;
  auto tile_of = [&](int i) {
    const int t = t_lo + wave + kNW * i;
    return t < t_hi ? t : (t_hi > 0 ? t_hi - 1 : 0);
  };
  // ---- Q as B operand, resident in registers (or LDS); the first tiles' loads go out with it ----
  bf16x8 qf[QLDS ? 1 : DS];
  Stage stg[PF];
  {
  constexpr int QPT = QLDS ? 32 * (D / 8) / (kNW * 64) : 1;  // 16-byte pieces of the query tile per thread
  i32x4 qraw[QPT];
  if (QLDS) {
#pragma unroll
    for (int i = 0; i < QPT; ++i) {
      const int p = threadIdx.x + i * kNW * 64;
      int row = mtile * 32 + p / (D / 8);
      if (row > a.M - 1) row = a.M - 1;
      qraw[i] = *(const i32x4*)(a.q + (size_t)row * a.q_sm + (size_t)h * a.q_sh + (p % (D / 8)) * 8);
    }
  } else {
    const u16* qp = a.q + (size_t)(q_ok ? qi : a.M - 1) * a.q_sm + (size_t)h * a.q_sh + 8 * half;
#pragma unroll
    for (int s = 0; s < DS; ++s) qf[QLDS ? 0 : s] = as_bf16x8(*(const i32x4*)(qp + 16 * s));
  }
#pragma unroll
  for (int p = 0; p < PF; ++p) load(stg[p], tile_of(p));
  if (QLDS) {
#pragma unroll
    for (int i = 0; i < QPT; ++i) {
      const int p = threadIdx.x + i * kNW * 64;
      *(i32x4*)(qs + (p / (D / 8)) * QPITCH + (p % (D / 8)) * 16) = qraw[i];
    }
    __syncthreads();
  }
  }

  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  auto process = [&](const Stage& st, int t) {
    const bool pre = t < tp;
    const int tt = pre ? t : t - tp;
    const int len = pre ? a.P : a.S;
    // ---- S^T tile = K . Q^T ----
    f32x16 sT;
#pragma unroll
    for (int i = 0; i < 16; ++i) sT[i] = 0.f;
#pragma unroll
    for (int s = 0; s < DS; ++s)
#pragma unroll
      for (int pl = 0; pl < PL; ++pl) {
        const bf16x8 qv = QLDS ? as_bf16x8(*(const i32x4*)(qs + l32 * QPITCH + (16 * s + 8 * half) * 2)) : qf[QLDS ? 0 : s];
        sT = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(st.k[pl][s]), qv, sT, 0, 0, 0);
      }

    // ---- scale, mask, online softmax (one query column per lane) ----
    // Register i of this lane holds key kl(i) = 16*(i/8) + 8*half + i%8 of the tile.  Visibility and
    // range are first reduced to two 16-bit masks (bit i = register i) with wave-uniform branches, so
    // the per-element code below is straight-line selects.
    unsigned vbits, ibits;
    {
      const int k0 = tt * 32 + 8 * half;  // key of register 0; registers 8..15 are 16 keys further
      const int left = len - k0;          // keys from k0 on that exist
      const unsigned lo8 = left >= 8 ? 0xffu : (left > 0 ? (1u << left) - 1u : 0u);
      const unsigned hi8 = left >= 24 ? 0xffu : (left > 16 ? (1u << (left - 16)) - 1u : 0u);
      ibits = lo8 | (hi8 << 8);
      if (!pre) {
        if (a.mask_mode == 1) {
          vbits = 0xffffu;
        } else {  // causal among the suffix tokens: key <= query
          const int c = qi - k0 + 1;  // visible keys from k0 on
          const unsigned cl = c >= 8 ? 0xffu : (c > 0 ? (1u << c) - 1u : 0u);
          const unsigned ch = c >= 24 ? 0xffu : (c > 16 ? (1u << (c - 16)) - 1u : 0u);
          vbits = cl | (ch << 8);
        }
      } else if (a.mask2d) {
        // one byte (0 or 1) per key: gather bit 0 of the 8 bytes of each word
        const unsigned long long gather = 0x0102040810204080ull, ones = 0x0101010101010101ull;
        vbits = (unsigned)(((st.m2[0] & ones) * gather) >> 56) | ((unsigned)(((st.m2[1] & ones) * gather) >> 56) << 8);
      } else {
        const unsigned pmask = (unsigned)__ballot(st.pad != 0);  // lanes 0..31: keys of this tile
        vbits = ((pmask >> (8 * half)) & 0xffu) | (((pmask >> (16 + 8 * half)) & 0xffu) << 8);
      }
    }
    const bool lb = a.logits_bf16 != 0;
    float p[16];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float sv = sT[i];
      sv = lb ? round_bf16(sv) : sv;
      sv *= a.scale;
      const float masked = lb ? sv + kOpenpiMask : kF32Min;
      sv = (vbits >> i) & 1u ? sv : masked;
      sv = (ibits >> i) & 1u ? sv : -INFINITY;
      p[i] = sv;
      tmax = fmaxf(tmax, sv);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
    const float m_new = fmaxf(m_run, tmax);
    const float alpha = __expf(m_run - m_new);
    float lsum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      p[i] = __expf(p[i] - m_new);
      lsum += p[i];
    }
    lsum += __shfl_xor(lsum, 32);
    l_run = l_run * alpha + lsum;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;

    // P^T as B operand: step s uses registers 8s..8s+7 = keys 16s + 8*half + 0..7
    bf16x8 pb[2], pbl[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      pb[s] = pack_bf16x8(p + 8 * s);
      if (SPLIT) {
        float lo[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) lo[j] = p[8 * s + j] - round_bf16(p[8 * s + j]);
        pbl[s] = pack_bf16x8(lo);
      }
    }
    // ---- O^T += V^T . P^T ----
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(st.v[0][dt][s]), pb[s], o[dt], 0, 0, 0);
        if (SPLIT) {
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(st.v[PL - 1][dt][s]), pb[s], o[dt], 0, 0, 0);
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(st.v[0][dt][s]), pbl[s], o[dt], 0, 0, 0);
        }
      }
  };

  {
    if (D > 128) {
      // one tile in flight and one copy of the tile code: with the pipelined form below the
      // register allocator spills this head size to scratch
      for (int i = 0; i < nt_w; ++i) {
        process(stg[0], tile_of(i));
        if (i + 1 < nt_w) load(stg[0], tile_of(i + 1));
      }
    } else {
      // software pipeline over this wave's tiles: the steady-state loop has no branch (precise
      // wait counts), the tail (< 2*PF tiles) uses wave-uniform conditions
      int i = 0;
      for (; i + 2 * PF <= nt_w; i += PF) {
#pragma unroll
        for (int p = 0; p < PF; ++p) {
          process(stg[p], tile_of(i + p));
          load(stg[p], tile_of(i + p + PF));
        }
      }
#pragma unroll
      for (int q = 0; q < 2 * PF - 1; ++q) {
        if (i + q < nt_w) {
          process(stg[q % PF], tile_of(i + q));
          if (i + q + PF < nt_w) load(stg[q % PF], tile_of(i + q + PF));
        }
      }
    }
  }
  // ---- merge the four waves in fixed order (LDS) ----
  if (half == 0) {
    st_m[wave][l32] = m_run;
    st_l[wave][l32] = l_run;
  }
  // waves 0..3 own the four register groups (output rows 8w + 4*(lane/32) + 0..3 of every d tile);
  // further waves only contribute their tiles
  const bool owner = wave < 4;
  const int wg = wave & 3;
  f32x4 own[DT];
  float ew[kNW];
  float bm = -INFINITY, bl = 0.f;  // block-level (m, l) of this lane's query
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      f32x4 v = {o[dt][4 * gq], o[dt][4 * gq + 1], o[dt][4 * gq + 2], o[dt][4 * gq + 3]};
      red[dt][wave][gq][lane] = v;
    }
  __syncthreads();
  {
    float mw[kNW];
#pragma unroll
    for (int w = 0; w < kNW; ++w) {
      mw[w] = st_m[w][l32];
      bm = fmaxf(bm, mw[w]);
    }
#pragma unroll
    for (int w = 0; w < kNW; ++w) {
      ew[w] = (mw[w] == -INFINITY) ? 0.f : __expf(mw[w] - bm);
      bl += st_l[w][l32] * ew[w];
    }
  }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    if (owner) {
      sum = red[dt][0][wg][lane] * ew[0];
#pragma unroll
      for (int w = 1; w < kNW; ++w) sum += red[dt][w][wg][lane] * ew[w];
    }
    own[dt] = sum;
  }
  // this lane's output: query qi, columns d0 .. d0+3 of every d tile
  u16* op = a.out + (size_t)(q_ok ? qi : 0) * a.out_sm + (size_t)h * D + 8 * wg + 4 * half;
  if (a.kv_splits == 1) {
    if (q_ok && owner) {
      const float inv = 1.0f / bl;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *(i32x2*)(op + dt * 32) = pack_bf16x4(own[dt] * inv);
    }
    return;
  }

  // ---- kv-split merge by the last-arriving block ----
  // partials per (block, split): [2][32] stats, then [DT][4 groups][64 lanes][4 floats]
  const int blk_lin = blockIdx.y * a.H + h;
  constexpr size_t PSTRIDE = 64 + (size_t)DT * 1024;  // floats
  float* pmine = a.partial + ((size_t)blk_lin * a.kv_splits + split) * PSTRIDE;
  if (wave == 0 && half == 0) {
    st_agent(pmine + l32, bm);
    st_agent(pmine + 32 + l32, bl);
  }
  if (owner) {
    unsigned long long* dst = (unsigned long long*)(pmine + 64) + ((size_t)wave * 64 + lane) * 2;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      st_agent64(dst + (size_t)dt * 512, own[dt][0], own[dt][1]);
      st_agent64(dst + (size_t)dt * 512 + 1, own[dt][2], own[dt][3]);
    }
  }
  __shared__ int s_last;
  handoff_publish();  // partials acknowledged (written through) before the count
  __syncthreads();
  if (threadIdx.x == 0) {
    int old = __hip_atomic_fetch_add(a.counters + blk_lin, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == a.kv_splits - 1);
  }
  __syncthreads();
  if (!s_last || !owner) return;
  handoff_acquire();
  if (threadIdx.x == 0) __hip_atomic_store(a.counters + blk_lin, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  constexpr int MAXS = D > 128 ? 7 : 8;  // the host never asks for more kv splits
  const float* pblk = a.partial + (size_t)blk_lin * a.kv_splits * PSTRIDE;
  // every read of the hand-off goes out before the first one is consumed (the read-back costs round
  // trips, not bandwidth): the statistics first, then the partial tiles in batches of DTB d tiles
  float ms[MAXS], ls[MAXS], es[MAXS];
#pragma unroll
  for (int s = 0; s < MAXS; ++s) {
    const int sc = s < a.kv_splits ? s : a.kv_splits - 1;
    ms[s] = ld_agent(pblk + (size_t)sc * PSTRIDE + l32);
    ls[s] = ld_agent(pblk + (size_t)sc * PSTRIDE + 32 + l32);
  }
  constexpr int DTB = DT >= 4 ? 4 : DT;
  unsigned long long raw[DTB][MAXS][2];
  auto fetch = [&](int d0) {
#pragma unroll
    for (int dd = 0; dd < DTB; ++dd)
#pragma unroll
      for (int s = 0; s < MAXS; ++s) {
        const int sc = s < a.kv_splits ? s : a.kv_splits - 1;
        const unsigned long long* src = (const unsigned long long*)(pblk + (size_t)sc * PSTRIDE + 64) +
                                        (size_t)(d0 + dd) * 512 + ((size_t)wave * 64 + lane) * 2;
        raw[dd][s][0] = ld_agent64(src);
        raw[dd][s][1] = ld_agent64(src + 1);
      }
  };
  fetch(0);
  float mt = -INFINITY;
#pragma unroll
  for (int s = 0; s < MAXS; ++s)
    if (s < a.kv_splits) mt = fmaxf(mt, ms[s]);
  float lt = 0.f;
#pragma unroll
  for (int s = 0; s < MAXS; ++s) {
    es[s] = (s < a.kv_splits && ms[s] != -INFINITY) ? __expf(ms[s] - mt) : 0.f;
    if (s < a.kv_splits) lt += ls[s] * es[s];
  }
  const float inv = 1.0f / lt;
#pragma unroll
  for (int d0 = 0; d0 < DT; d0 += DTB) {
    f32x4 acc[DTB];
#pragma unroll
    for (int dd = 0; dd < DTB; ++dd) {
      acc[dd] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < MAXS; ++s) {
        if (s < a.kv_splits) {
          f32x4 v = {__uint_as_float((unsigned)raw[dd][s][0]), __uint_as_float((unsigned)(raw[dd][s][0] >> 32)),
                     __uint_as_float((unsigned)raw[dd][s][1]), __uint_as_float((unsigned)(raw[dd][s][1] >> 32))};
          acc[dd] += v * es[s];
        }
      }
    }
    if (d0 + DTB < DT) fetch(d0 + DTB);  // the next batch is on its way while this one is stored
#pragma unroll
    for (int dd = 0; dd < DTB; ++dd)
      if (q_ok) *(i32x2*)(op + (d0 + dd) * 32) = pack_bf16x4(acc[dd] * inv);
  }
}

// Lays a [L, G, D] K/V pair out for the attention kernel: V transposed to [G, D, ld] (keys
// contiguous, zero-filled from L to ld), and -- for fp32 sources -- K and V^T split into bf16
// hi + lo planes.  One thread per (key, kv head, 8 d columns).
__global__ void kv_prepare_kernel(KvPrepArgs p) {
  const int chunks = p.D / 8;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long total = (long long)p.ld * p.G * chunks;
  if (idx >= total) return;
  const int dc = (int)(idx % chunks);
  const int g = (int)((idx / chunks) % p.G);
  const int key = (int)(idx / ((long long)chunks * p.G));
  float kf[8], vf[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) kf[j] = vf[j] = 0.f;
  if (key < p.L) {
    const size_t off = (size_t)key * p.sl + (size_t)g * p.sh + dc * 8;
    if (p.f32) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        kf[j] = ((const float*)p.k)[off + j];
        vf[j] = ((const float*)p.v)[off + j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) vf[j] = bf16_bits_to_f32(((const u16*)p.v)[off + j]);
    }
  }
  const size_t vt0 = ((size_t)g * p.D + dc * 8) * p.ld + key;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const u16 hi = f32_to_bf16_bits(vf[j]);
    p.vt_hi[vt0 + (size_t)j * p.ld] = hi;
    if (p.f32) p.vt_lo[vt0 + (size_t)j * p.ld] = f32_to_bf16_bits(vf[j] - bf16_bits_to_f32(hi));
  }
  if (p.f32 && key < p.L) {
    const size_t ko = ((size_t)key * p.G + g) * p.D + dc * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const u16 hi = f32_to_bf16_bits(kf[j]);
      p.k_hi[ko + j] = hi;
      p.k_lo[ko + j] = f32_to_bf16_bits(kf[j] - bf16_bits_to_f32(hi));
    }
  }
}

template <int D, bool SPLIT, int NWV>
int launch_attn(const AttnArgs& a, hipStream_t st) {
  dim3 grid(a.H, ((a.M + 31) / 32) * (a.batch > 0 ? a.batch : 1), a.kv_splits);
  if (a.xcd_remap) grid = dim3(8 * ((a.batch * a.H + 7) / 8) * ((a.M + 31) / 32), 1, 1);
  hipLaunchKernelGGL((expert_attn_kernel<D, SPLIT, NWV>), grid, dim3(NWV * 64), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace

int tk_attn_waves(int D, int split_planes, int ntiles) {
  // a block of 8 or 12 waves when that covers every key tile (D = 64 only: register budget)
  if (D != 64) return 4;
  if (ntiles <= 8 && ntiles > 4) return 8;
  if (!split_planes && ntiles <= 12 && ntiles > 8) return 12;
  // long key ranges (vision tower: 32 tiles): two waves per SIMD hide more of the per-tile latency
  if (!split_planes && ntiles > 12) return 8;
  return 4;
}

int tk_launch_attn(AttnArgs a, int D, int waves, hipStream_t st) {
  const bool split = a.k_pre_lo != nullptr;
  if (split) {
    if (D != 64) return -1;
    return waves == 8 ? launch_attn<64, true, 8>(a, st) : launch_attn<64, true, 4>(a, st);
  }
  if (D == 64) {
    if (waves == 12) return launch_attn<64, false, 12>(a, st);
    if (waves == 8) return launch_attn<64, false, 8>(a, st);
    return launch_attn<64, false, 4>(a, st);
  }
  if (D == 96) return launch_attn<96, false, 4>(a, st);
  if (D == 128) return launch_attn<128, false, 4>(a, st);
  if (D == 256) return launch_attn<256, false, 4>(a, st);
  return -1;
}

int tk_launch_kv_prepare(KvPrepArgs p, hipStream_t st) {
  const long long total = (long long)p.ld * p.G * (p.D / 8);
  hipLaunchKernelGGL(kv_prepare_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, p);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
