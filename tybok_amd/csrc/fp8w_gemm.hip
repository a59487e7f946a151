// fp8-weight GEMM for skinny M on gfx950:  y[M,N] = bf16((x[M,K] . W8[N,K]^T) * scale[n]).
//
// Memory-bound (weight streaming), so the layout is built around the weight read:
//   * W8 is pre-packed into 32(n) x 32(k)-byte tiles in MFMA B-operand lane order; a wave reads a
//     tile with ONE coalesced 1 KiB global_load_dwordx4 straight into operand registers.
//   * e4m3 -> bf16 is exact and done in registers (v_cvt_scalef32_pk_bf16_fp8, scale 1.0), the
//     product runs on v_mfma_f32_32x32x16_bf16 with fp32 accumulation.
//   * x (bf16, tiny, L2 resident) is read directly in A-operand order: 32 contiguous bytes/lane.
//   * A block owns NT n-tiles x MT m-tiles and a contiguous range of k-tiles; its NW waves take
//     k-tiles round-robin, so concurrently issued loads of a block are contiguous in memory.
//   * Reductions are fixed-order: waves through LDS (w = 0..NW-1), K splits through an fp32
//     partial buffer summed by the last-arriving block in split order (no float atomics).
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

template <int MT, int NT>
struct Frag {
  i32x4 w[NT];
  i32x4 xa[MT][2];
};

template <int MT, int NT, int NW, bool GATED, int PF>
__global__ __launch_bounds__(NW * 64) void fp8w_gemm_kernel(GemmArgs a) {
  constexpr int TILES = MT * NT;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int strip = blockIdx.x;
  const int split = blockIdx.y;
  const int mblock = blockIdx.z;
  const int half = lane >> 5;
  const int l32 = lane & 31;

  const int kt_lo = (int)(((long long)split * a.KT) / a.ksplit);
  const int kt_hi = (int)(((long long)(split + 1) * a.KT) / a.ksplit);

  // weight tile streams of this wave
  const uint8_t* wbase[NT];
  bool nt_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int ntg = strip * NT + nt;
    nt_ok[nt] = ntg < a.ntiles;
    wbase[nt] = a.w + ((size_t)ntg * a.KT) * 1024 + lane * 16;
  }
  // activation rows of this lane
  const u16* xrow[MT];
  bool m_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = (mblock * MT + mt) * 32 + l32;
    m_ok[mt] = m < a.M;
    xrow[mt] = a.x + (size_t)m * a.ldx + 16 * half;
  }

  f32x16 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;

  auto load = [&](Frag<MT, NT>& f, int kt) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      i32x4 v = {0, 0, 0, 0};
      if (nt_ok[nt]) v = *(const i32x4*)(wbase[nt] + (size_t)kt * 1024);
      f.w[nt] = v;
    }
    const bool k_ok = (kt * 32 + 16 * half) < a.K;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      i32x4 v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
      if (m_ok[mt] && k_ok) {
        const i32x4* p = (const i32x4*)(xrow[mt] + kt * 32);
        v0 = p[0];
        v1 = p[1];
      }
      f.xa[mt][0] = v0;
      f.xa[mt][1] = v1;
    }
  };
  auto compute = [&](const Frag<MT, NT>& f) {
    bf16x8 wb[NT][2];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      wb[nt][0] = fp8x8_to_bf16x8(f.w[nt][0], f.w[nt][1]);
      wb[nt][1] = fp8x8_to_bf16x8(f.w[nt][2], f.w[nt][3]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(f.xa[mt][j]), wb[nt][j], acc[mt][nt], 0, 0, 0);
  };

  // software pipeline: PF k-tiles of this wave in flight
  Frag<MT, NT> buf[PF];
  const int kt0 = kt_lo + wave;
#pragma unroll
  for (int p = 0; p < PF; ++p)
    if (kt0 + p * NW < kt_hi) load(buf[p], kt0 + p * NW);
  for (int kt = kt0; kt < kt_hi; kt += NW * PF) {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      const int k = kt + p * NW;
      if (k < kt_hi) {
        compute(buf[p]);
        const int kn = k + PF * NW;
        if (kn < kt_hi) load(buf[p], kn);
      }
    }
  }

  // ---- in-block reduction over waves (fixed order), tile by tile, double-buffered LDS ----
  __shared__ float red[2][NW][16][64];
  constexpr int OWN = GATED ? 2 * ((TILES / 2 + NW - 1) / NW) : (TILES + NW - 1) / NW;
  float own[OWN][16];
#pragma unroll
  for (int o = 0; o < OWN; ++o)
#pragma unroll
    for (int i = 0; i < 16; ++i) own[o][i] = 0.f;

#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    const int mt = t / NT, nt = t % NT;
    const int owner = GATED ? (t / 2) % NW : t % NW;
    const int slot = GATED ? ((t / 2) / NW) * 2 + (t & 1) : t / NW;
    if (NW > 1) {
#pragma unroll
      for (int i = 0; i < 16; ++i) red[t & 1][wave][i][lane] = acc[mt][nt][i];
      __syncthreads();
      if (wave == owner) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float s = 0.f;
#pragma unroll
          for (int w = 0; w < NW; ++w) s += red[t & 1][w][i][lane];
          own[slot][i] = s;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) own[slot][i] = acc[mt][nt][i];
    }
  }

  // ---- K-split reduction through global partials; the last-arriving block finishes ----
  const int blk_lin = mblock * gridDim.x + strip;
  if (a.ksplit > 1) {
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const int owner = GATED ? (t / 2) % NW : t % NW;
      const int slot = GATED ? ((t / 2) / NW) * 2 + (t & 1) : t / NW;
      if (wave == owner) {
        float* dst = a.partial + (((size_t)blk_lin * a.ksplit + split) * TILES + t) * 1024 + lane;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[i * 64] = own[slot][i];
      }
    }
    __shared__ int s_last;
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
      int old = atomicAdd(a.counters + blk_lin, 1);
      s_last = (old == a.ksplit - 1);
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const int owner = GATED ? (t / 2) % NW : t % NW;
      const int slot = GATED ? ((t / 2) / NW) * 2 + (t & 1) : t / NW;
      if (wave == owner) {
#pragma unroll
        for (int i = 0; i < 16; ++i) own[slot][i] = 0.f;
        for (int s = 0; s < a.ksplit; ++s) {
          const float* src = a.partial + (((size_t)blk_lin * a.ksplit + s) * TILES + t) * 1024 + lane;
#pragma unroll
          for (int i = 0; i < 16; ++i) own[slot][i] += __builtin_nontemporal_load(src + i * 64);
        }
      }
    }
    if (threadIdx.x == 0) a.counters[blk_lin] = 0;  // leave the counter ready for the next launch
  }

  // ---- epilogue ----
  if (!GATED) {
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const int mt = t / NT, nt = t % NT;
      if (wave != t % NW) continue;
      const int slot = t / NW;
      const int n = (strip * NT + nt) * 32 + l32;
      if (n >= a.N) continue;
      const float sc = a.s0[n];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = (mblock * MT + mt) * 32 + mfma32_row(lane, i);
        if (m < a.M) {
          u16 r = f32_to_bf16_bits(own[slot][i] * sc);
          if (a.resid) {
            float rv = a.resid_f32 ? ((const float*)a.resid)[(size_t)m * a.ldr + n]
                                   : bf16_bits_to_f32(((const u16*)a.resid)[(size_t)m * a.ldr + n]);
            r = f32_to_bf16_bits(bf16_bits_to_f32(r) + rv);
          }
          a.y[(size_t)m * a.ldy + n] = r;
        }
      }
    }
  } else {
    // tiles come in (gate, up) pairs over the same logical columns
#pragma unroll
    for (int u = 0; u < TILES / 2; ++u) {
      if (wave != u % NW) continue;
      const int t = 2 * u;
      const int mt = t / NT, nt = t % NT;
      const int sg = (u / NW) * 2, su = sg + 1;
      const int col = ((strip * NT + nt) / 2) * 32 + l32;  // logical column in [0, I)
      if (col >= a.N) continue;
      const float scg = a.s0[col], scu = a.s1[col];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = (mblock * MT + mt) * 32 + mfma32_row(lane, i);
        if (m < a.M) {
          float g = round_bf16(own[sg][i] * scg);
          float up = round_bf16(own[su][i] * scu);
          float act = a.act == 0 ? silu_f(g) : gelu_tanh_f(g);
          a.y[(size_t)m * a.ldy + col] = f32_to_bf16_bits(round_bf16(act) * up);
        }
      }
    }
  }
}

__global__ void pack_kernel(const uint8_t* __restrict__ w0, const uint8_t* __restrict__ w1, uint8_t* __restrict__ out,
                            int N, int K, int KT, long long nchunks, int interleave) {
  // one thread per 16-byte lane chunk of the packed buffer
  long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= nchunks) return;
  const int lane = (int)(c & 63);
  const long long tile = c >> 6;
  const int kt = (int)(tile % KT);
  const int ntg = (int)(tile / KT);
  const uint8_t* src = w0;
  int nt = ntg;
  if (interleave) {
    src = (ntg & 1) ? w1 : w0;
    nt = ntg >> 1;
  }
  const int n = nt * 32 + (lane & 31);
  const int k = kt * 32 + 16 * (lane >> 5);
  i32x4 v = {0, 0, 0, 0};
  if (n < N && k < K) v = *(const i32x4*)(src + (size_t)n * K + k);
  *(i32x4*)(out + c * 16) = v;
}

__global__ void fill_zero_kernel(int* p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

__global__ void decode_fp8_kernel(float* out) {
  // decodes code c (= threadIdx.x) through the same instruction the GEMM uses
  int c = threadIdx.x;
  bf16x2 lo, hi;
  fp8x4_to_bf16x4(c, lo, hi);
  union { bf16x2 v; unsigned u; } cv;
  cv.v = lo;
  out[c] = bf16_bits_to_f32((u16)(cv.u & 0xffff));
}

template <int MT, int NT, int NW, bool GATED, int PF>
int launch(const GemmArgs& a, dim3 grid, hipStream_t st) {
  hipLaunchKernelGGL((fp8w_gemm_kernel<MT, NT, NW, GATED, PF>), grid, dim3(NW * 64), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace

int tk_launch_gemm(GemmArgs a, int MT, int NT, int mblocks, hipStream_t st) {
  dim3 grid((a.ntiles + NT - 1) / NT, a.ksplit, mblocks);
  const bool gated = a.s1 != nullptr;
  if (gated) {
    if (NT != 2) return -1;
    return MT == 1 ? launch<1, 2, 4, true, 4>(a, grid, st) : launch<2, 2, 4, true, 4>(a, grid, st);
  }
  if (NT == 1) return MT == 1 ? launch<1, 1, 4, false, 4>(a, grid, st) : launch<2, 1, 4, false, 4>(a, grid, st);
  return MT == 1 ? launch<1, 2, 4, false, 4>(a, grid, st) : launch<2, 2, 4, false, 4>(a, grid, st);
}

int tk_launch_pack(const void* w0, const void* w1, void* out, int N, int K, int interleave, hipStream_t st) {
  const int KT = (K + 31) / 32;
  const int ntiles = ((N + 31) / 32) * (interleave ? 2 : 1);
  const long long nchunks = (long long)ntiles * KT * 64;
  const int threads = 256;
  const long long blocks = (nchunks + threads - 1) / threads;
  hipLaunchKernelGGL(pack_kernel, dim3((unsigned)blocks), dim3(threads), 0, st, (const uint8_t*)w0, (const uint8_t*)w1,
                     (uint8_t*)out, N, K, KT, nchunks, interleave);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

int tk_launch_fill_zero(int* p, int n, hipStream_t st) {
  hipLaunchKernelGGL(fill_zero_kernel, dim3((n + 255) / 256), dim3(256), 0, st, p, n);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

int tk_launch_decode_fp8(float* out, hipStream_t st) {
  hipLaunchKernelGGL(decode_fp8_kernel, dim3(1), dim3(256), 0, st, out);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
