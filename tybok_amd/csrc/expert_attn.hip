// Action-expert attention over [cached prefix KV ; suffix KV] for one request on gfx950.
//
//   out[M, H*D] = softmax(q . K^T * D^-0.5 (+mask)) . V        (GQA: q head h -> kv head h/(H/G))
//
// Tiny and latency-bound (50 queries, a few hundred keys), so the grid is (head, 32-query tile,
// kv split) and the four waves of a block take 32-key tiles round-robin:
//   * S^T[key, q] = K . Q^T on v_mfma_f32_32x32x16_bf16: K rows are read from global memory in
//     A-operand order (16 bytes per lane), Q is held in registers as the B operand.  In this
//     orientation one lane owns one query column, so the softmax max/sum are in-lane plus one
//     cross-half exchange (wavefront reduction), and P^T is already the B operand of P.V.
//   * V tiles go through wave-private LDS (coalesced 16-byte rows in, key-strided 2-byte reads
//     out) to form the A operand of O^T[d, q] += V^T . P^T.
//   * fp32 K/V (SmolVLA cross layers) are split into bf16 hi + lo planes; P too (3 MFMAs).
//   * Online softmax per wave, then a fixed-order merge over waves (LDS) and kv splits (global
//     partials, last-arriving block) -- deterministic, no atomics on data.
#include <math.h>
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

constexpr float kF32Min = -3.4028234663852886e38f;    // finfo(float32).min
constexpr float kOpenpiMask = -2.3819763e38f;         // additive mask of the pi0.5 path
constexpr int kNW = 4;

__device__ __forceinline__ bf16x8 pack_bf16x8(const float* v) {
  union { u16 h[8]; bf16x8 b; } u;
#pragma unroll
  for (int j = 0; j < 8; ++j) u.h[j] = f32_to_bf16_bits(v[j]);
  return u.b;
}

template <int D, bool KVF32>
__global__ __launch_bounds__(kNW * 64) void expert_attn_kernel(AttnArgs a) {
  constexpr int DT = D / 32;                 // d tiles of the output
  constexpr int DS = D / 16;                 // k steps of Q.K^T
  constexpr int DCH = D > 128 ? 128 : D;     // d columns staged per V pass
  constexpr int NPASS = D / DCH;
  constexpr int VP = DCH + 8;                // LDS row pitch (u16 elements)
  constexpr int PLANES = KVF32 ? 2 : 1;
  constexpr int STAGE_BYTES = kNW * PLANES * 32 * VP * 2;
  constexpr int MERGE_BYTES = kNW * 2 * 16 * 64 * 4 + kNW * 2 * 32 * 4;
  constexpr int SMEM = STAGE_BYTES > MERGE_BYTES ? STAGE_BYTES : MERGE_BYTES;
  __shared__ __align__(16) unsigned char smem[SMEM];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int h = blockIdx.x;
  const int mtile = blockIdx.y;
  const int split = blockIdx.z;
  const int g = h / (a.H / a.G);
  const int L = a.P + a.S;
  const int ntiles = (L + 31) / 32;
  const int t_lo = (split * ntiles) / a.kv_splits;
  const int t_hi = ((split + 1) * ntiles) / a.kv_splits;
  const int qi = mtile * 32 + l32;
  const bool q_ok = qi < a.M;

  // ---- Q as B operand, resident in registers ----
  bf16x8 qf[DS];
  {
    const u16* qp = a.q + (size_t)qi * a.q_sm + (size_t)h * a.q_sh + 8 * half;
#pragma unroll
    for (int st = 0; st < DS; ++st) {
      i32x4 v = {0, 0, 0, 0};
      if (q_ok) v = *(const i32x4*)(qp + 16 * st);
      qf[st] = as_bf16x8(v);
    }
  }

  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  u16* vstage = (u16*)smem + (size_t)wave * PLANES * 32 * VP;

  for (int t = t_lo + wave; t < t_hi; t += kNW) {
    // ---- S^T tile = K . Q^T ----
    f32x16 sT;
#pragma unroll
    for (int i = 0; i < 16; ++i) sT[i] = 0.f;
    {
      const int kr = t * 32 + l32;
      const bool k_ok = kr < L;
      const bool in_pre = kr < a.P;
      if (KVF32) {
        const float* kp = (const float*)a.k_pre + (size_t)kr * a.pre_sl + (size_t)g * a.pre_sh + 8 * half;
#pragma unroll
        for (int st = 0; st < DS; ++st) {
          float f[8], lo[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) f[j] = 0.f;
          if (k_ok) {
            const float4* p4 = (const float4*)(kp + 16 * st);
            float4 x0 = p4[0], x1 = p4[1];
            f[0] = x0.x; f[1] = x0.y; f[2] = x0.z; f[3] = x0.w;
            f[4] = x1.x; f[5] = x1.y; f[6] = x1.z; f[7] = x1.w;
          }
#pragma unroll
          for (int j = 0; j < 8; ++j) lo[j] = f[j] - round_bf16(f[j]);
          sT = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pack_bf16x8(f), qf[st], sT, 0, 0, 0);
          sT = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pack_bf16x8(lo), qf[st], sT, 0, 0, 0);
        }
      } else {
        const u16* kp = in_pre ? (const u16*)a.k_pre + (size_t)kr * a.pre_sl + (size_t)g * a.pre_sh
                               : a.k_suf + (size_t)(kr - a.P) * a.suf_sl + (size_t)g * a.suf_sh;
        kp += 8 * half;
#pragma unroll
        for (int st = 0; st < DS; ++st) {
          i32x4 v = {0, 0, 0, 0};
          if (k_ok) v = *(const i32x4*)(kp + 16 * st);
          sT = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(v), qf[st], sT, 0, 0, 0);
        }
      }
    }

    // ---- scale, mask, online softmax (one query column per lane) ----
    float p[16];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = t * 32 + mfma32_row(lane, i);
      float s = sT[i];
      if (a.logits_bf16) s = round_bf16(s);
      s *= a.scale;
      bool vis;
      if (key < a.P) {
        vis = a.pad ? (a.pad[key < L ? key : 0] != 0) : true;
      } else {
        vis = (a.mask_mode == 1) || ((key - a.P) <= qi);
      }
      if (!vis) s = a.logits_bf16 ? (s + kOpenpiMask) : kF32Min;
      if (key >= L) s = -INFINITY;
      p[i] = s;
      tmax = fmaxf(tmax, s);
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

    // P^T as B operand: step s uses registers 8s..8s+7 (keys 8*(2s+j/4) + 4*half + j%4)
    bf16x8 pb[2], pbl[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      pb[s] = pack_bf16x8(p + 8 * s);
      if (KVF32) {
        float lo[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) lo[j] = p[8 * s + j] - round_bf16(p[8 * s + j]);
        pbl[s] = pack_bf16x8(lo);
      }
    }

    // ---- O^T += V^T . P^T, V staged through wave-private LDS ----
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
      constexpr int CH_PER_ROW = DCH / 8;  // 16-byte chunks per staged row
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int c0 = 0; c0 < 32 * CH_PER_ROW; c0 += 64) {
        const int c = c0 + lane;
        const int kl = c / CH_PER_ROW;
        const int dc = c % CH_PER_ROW;
        const int kv = t * 32 + kl;
        const int dcol = pass * DCH + dc * 8;
        if (KVF32) {
          float f[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) f[j] = 0.f;
          if (kv < L) {
            const float4* p4 =
                (const float4*)((const float*)a.v_pre + (size_t)kv * a.pre_sl + (size_t)g * a.pre_sh + dcol);
            float4 x0 = p4[0], x1 = p4[1];
            f[0] = x0.x; f[1] = x0.y; f[2] = x0.z; f[3] = x0.w;
            f[4] = x1.x; f[5] = x1.y; f[6] = x1.z; f[7] = x1.w;
          }
          float lo[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) lo[j] = f[j] - round_bf16(f[j]);
          union { bf16x8 b; i32x4 i; } uh, ul;
          uh.b = pack_bf16x8(f);
          ul.b = pack_bf16x8(lo);
          *(i32x4*)(vstage + (size_t)kl * VP + dc * 8) = uh.i;
          *(i32x4*)(vstage + (size_t)(32 + kl) * VP + dc * 8) = ul.i;
        } else {
          i32x4 v = {0, 0, 0, 0};
          if (kv < L) {
            const u16* vp = kv < a.P ? (const u16*)a.v_pre + (size_t)kv * a.pre_sl + (size_t)g * a.pre_sh
                                     : a.v_suf + (size_t)(kv - a.P) * a.suf_sl + (size_t)g * a.suf_sh;
            v = *(const i32x4*)(vp + dcol);
          }
          *(i32x4*)(vstage + (size_t)kl * VP + dc * 8) = v;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int dl = 0; dl < DCH / 32; ++dl) {
        const int dt = pass * (DCH / 32) + dl;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          union { u16 hh[8]; bf16x8 b; } va, vl;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int kl = 8 * (2 * s + (j >> 2)) + 4 * half + (j & 3);
            va.hh[j] = vstage[(size_t)kl * VP + dl * 32 + l32];
            if (KVF32) vl.hh[j] = vstage[(size_t)(32 + kl) * VP + dl * 32 + l32];
          }
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va.b, pb[s], o[dt], 0, 0, 0);
          if (KVF32) {
            o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vl.b, pb[s], o[dt], 0, 0, 0);
            o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va.b, pbl[s], o[dt], 0, 0, 0);
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }

  // ---- merge the four waves in fixed order (LDS), two d tiles per round ----
  float* st_m = (float*)smem;                 // [kNW][32]
  float* st_l = st_m + kNW * 32;              // [kNW][32]
  float* obuf = st_l + kNW * 32;              // [kNW][2][16][64]
  __syncthreads();                            // staging region is dead from here on
  if (half == 0) {
    st_m[wave * 32 + l32] = m_run;
    st_l[wave * 32 + l32] = l_run;
  }
  const int blk_lin = mtile * a.H + h;
  float* part_stats = a.partial;  // [blk][split][2][32]
  float* part_o = a.partial + (size_t)gridDim.x * gridDim.y * a.kv_splits * 64;  // [blk][split][DT][16][64]
  float bm = 0.f, bl = 0.f;       // block-level (m, l) of this lane's query
#pragma unroll
  for (int r = 0; r < DT / 2; ++r) {
#pragma unroll
    for (int dd = 0; dd < 2; ++dd)
#pragma unroll
      for (int i = 0; i < 16; ++i) obuf[((wave * 2 + dd) * 16 + i) * 64 + lane] = o[2 * r + dd][i];
    __syncthreads();
    if (wave < 2) {
      const int dd = wave;
      const int dt = 2 * r + dd;
      float mw[kNW], ew[kNW];
      float mt = -INFINITY;
#pragma unroll
      for (int w = 0; w < kNW; ++w) {
        mw[w] = st_m[w * 32 + l32];
        mt = fmaxf(mt, mw[w]);
      }
      float lt = 0.f;
#pragma unroll
      for (int w = 0; w < kNW; ++w) {
        ew[w] = (mw[w] == -INFINITY) ? 0.f : __expf(mw[w] - mt);
        lt += st_l[w * 32 + l32] * ew[w];
      }
      bm = mt;
      bl = lt;
      float accv[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < kNW; ++w) s += obuf[((w * 2 + dd) * 16 + i) * 64 + lane] * ew[w];
        accv[i] = s;
      }
      if (a.kv_splits == 1) {
        if (q_ok) {
          const float inv = 1.0f / lt;
          u16* op = a.out + (size_t)qi * a.out_sm + (size_t)h * D + dt * 32;
#pragma unroll
          for (int i = 0; i < 16; ++i) op[mfma32_row(lane, i)] = f32_to_bf16_bits(accv[i] * inv);
        }
      } else {
        float* dst = part_o + ((((size_t)blk_lin * a.kv_splits + split) * DT + dt) * 16) * 64 + lane;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[i * 64] = accv[i];
      }
    }
    __syncthreads();
  }
  if (a.kv_splits == 1) return;

  // ---- kv-split merge by the last-arriving block ----
  if (wave == 0 && half == 0) {
    float* ps = part_stats + ((size_t)blk_lin * a.kv_splits + split) * 64;
    ps[l32] = bm;
    ps[32 + l32] = bl;
  }
  __shared__ int s_last;
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    int old = atomicAdd(a.counters + blk_lin, 1);
    s_last = (old == a.kv_splits - 1);
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  float mt = -INFINITY;
  for (int s = 0; s < a.kv_splits; ++s) mt = fmaxf(mt, part_stats[((size_t)blk_lin * a.kv_splits + s) * 64 + l32]);
  float lt = 0.f;
  for (int s = 0; s < a.kv_splits; ++s) {
    const float* ps = part_stats + ((size_t)blk_lin * a.kv_splits + s) * 64;
    const float e = (ps[l32] == -INFINITY) ? 0.f : __expf(ps[l32] - mt);
    lt += ps[32 + l32] * e;
  }
  const float inv = 1.0f / lt;
  for (int dt = wave; dt < DT; dt += kNW) {
    float accv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) accv[i] = 0.f;
    for (int s = 0; s < a.kv_splits; ++s) {
      const float ms = part_stats[((size_t)blk_lin * a.kv_splits + s) * 64 + l32];
      const float e = (ms == -INFINITY) ? 0.f : __expf(ms - mt);
      const float* src = part_o + ((((size_t)blk_lin * a.kv_splits + s) * DT + dt) * 16) * 64 + lane;
#pragma unroll
      for (int i = 0; i < 16; ++i) accv[i] += src[i * 64] * e;
    }
    if (q_ok) {
      u16* op = a.out + (size_t)qi * a.out_sm + (size_t)h * D + dt * 32;
#pragma unroll
      for (int i = 0; i < 16; ++i) op[mfma32_row(lane, i)] = f32_to_bf16_bits(accv[i] * inv);
    }
  }
  if (threadIdx.x == 0) a.counters[blk_lin] = 0;
}

template <int D, bool KVF32>
int launch_attn(const AttnArgs& a, hipStream_t st) {
  dim3 grid(a.H, (a.M + 31) / 32, a.kv_splits);
  hipLaunchKernelGGL((expert_attn_kernel<D, KVF32>), grid, dim3(kNW * 64), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace

int tk_launch_attn(AttnArgs a, int D, int kv_f32, hipStream_t st) {
  if (kv_f32) {
    if (D == 64) return launch_attn<64, true>(a, st);
    return -1;
  }
  if (D == 64) return launch_attn<64, false>(a, st);
  if (D == 128) return launch_attn<128, false>(a, st);
  if (D == 256) return launch_attn<256, false>(a, st);
  return -1;
}
