// LayerNorm of the vision towers' token rows with the cast to the GEMM input type folded in:
//   y[m, :] = bf16((x[m, :] - mean) * rstd * w + b),   mean / biased variance / rstd in fp32
// for fp32 rows with fp32 parameters (SigLIP tower of pi0.5: F.layer_norm(x) followed by .to(bf16),
// tybok/policies/pi05/models/vision.py:115-170) or bf16 rows with bf16 parameters (SmolVLA's tower,
// which torch normalises in fp32 and rounds once: tybok/policies/smolvla/models/vision.py:197-257).
// One wave per row, the row stays in registers between the mean, variance and output passes; sums
// by wave shuffles in a fixed order.
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

constexpr int PMAX = 4;  // 8-element pieces per lane: rows up to 64 * 8 * PMAX = 2048 columns

// ADD: the rows are x + r first (r bf16: the output of the linear that closes a residual branch), the
// sum is written back in x's type (fp32: x + float(r); bf16: rounded once, as torch's bf16 add) and
// normalised -- the residual add and the next LayerNorm of a tower layer in one launch.
template <bool XF32, bool WF32, bool ADD>
__global__ __launch_bounds__(256) void layer_norm_kernel(LayerNormArgs a) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.M) return;
  const int pieces = a.K / 8;
  int yrow = a.y_rows ? a.y_rows[row] : row;  // (requested with everything else)
  yrow = yrow < 0 ? 0 : (yrow > a.M - 1 ? a.M - 1 : yrow);
  // the parameters of this lane's pieces are requested with the row (they depend on nothing computed here): asked
  // for after the two reductions they would cost the launch one more memory round trip
  i32x4 wq[PMAX][WF32 ? 2 : 1], bq[PMAX][WF32 ? 2 : 1];
#pragma unroll
  for (int i = 0; i < PMAX; ++i) {
    const int p = lane + 64 * i < pieces ? lane + 64 * i : pieces - 1;
    if (WF32) {
      const i32x4* wp = (const i32x4*)((const float*)a.w + 8 * p);
      const i32x4* bp = (const i32x4*)((const float*)a.b + 8 * p);
      wq[i][0] = wp[0];
      wq[i][WF32 ? 1 : 0] = wp[1];
      bq[i][0] = bp[0];
      bq[i][WF32 ? 1 : 0] = bp[1];
    } else {
      wq[i][0] = *(const i32x4*)((const u16*)a.w + 8 * p);
      bq[i][0] = *(const i32x4*)((const u16*)a.b + 8 * p);
    }
  }
  float v[PMAX][8];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < PMAX; ++i) {
    const int p = lane + 64 * i;
    if (p < pieces) {
      if (XF32) {
        const f32x4* src = (const f32x4*)((const float*)a.x + (size_t)row * a.ldx + 8 * p);
        const f32x4 lo = src[0], hi = src[1];
#pragma unroll
        for (int e = 0; e < 4; ++e) { v[i][e] = lo[e]; v[i][4 + e] = hi[e]; }
      } else {
        union { i32x4 q; unsigned u[4]; } xu;
        xu.q = *(const i32x4*)((const u16*)a.x + (size_t)row * a.ldx + 8 * p);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[i][2 * e] = __uint_as_float(xu.u[e] << 16);
          v[i][2 * e + 1] = __uint_as_float(xu.u[e] & 0xffff0000u);
        }
      }
      if (ADD) {
        union { i32x4 q; unsigned u[4]; } ru;
        ru.q = *(const i32x4*)(a.r + (size_t)row * a.ldr + 8 * p);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[i][2 * e] += __uint_as_float(ru.u[e] << 16);
          v[i][2 * e + 1] += __uint_as_float(ru.u[e] & 0xffff0000u);
        }
        if (XF32) {
          f32x4* dst = (f32x4*)((float*)a.xsum + (size_t)row * a.ldxs + 8 * p);
          const f32x4 lo = {v[i][0], v[i][1], v[i][2], v[i][3]}, hi = {v[i][4], v[i][5], v[i][6], v[i][7]};
          dst[0] = lo;
          dst[1] = hi;
        } else {
          union { i32x4 q; unsigned u[4]; } su;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            su.u[e] = pack_bf16x2(v[i][2 * e], v[i][2 * e + 1]);
            v[i][2 * e] = __uint_as_float(su.u[e] << 16);
            v[i][2 * e + 1] = __uint_as_float(su.u[e] & 0xffff0000u);
          }
          *(i32x4*)((u16*)a.xsum + (size_t)row * a.ldxs + 8 * p) = su.q;
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += v[i][e];
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
  const float mean = sum / (float)a.K;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < PMAX; ++i)
    if (lane + 64 * i < pieces) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = v[i][e] - mean;
        sq = fmaf(d, d, sq);
      }
    }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
  const float rstd = rsqrtf(sq / (float)a.K + a.eps);
#pragma unroll
  for (int i = 0; i < PMAX; ++i) {
    const int p = lane + 64 * i;
    if (p < pieces) {
      float w[8], b[8];
      if (WF32) {
        union { i32x4 q[2]; float f[8]; } wu, bu;
        wu.q[0] = wq[i][0];
        wu.q[1] = wq[i][WF32 ? 1 : 0];
        bu.q[0] = bq[i][0];
        bu.q[1] = bq[i][WF32 ? 1 : 0];
#pragma unroll
        for (int e = 0; e < 8; ++e) { w[e] = wu.f[e]; b[e] = bu.f[e]; }
      } else {
        union { i32x4 q; unsigned u[4]; } wu, bu;
        wu.q = wq[i][0];
        bu.q = bq[i][0];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          w[2 * e] = __uint_as_float(wu.u[e] << 16);
          w[2 * e + 1] = __uint_as_float(wu.u[e] & 0xffff0000u);
          b[2 * e] = __uint_as_float(bu.u[e] << 16);
          b[2 * e + 1] = __uint_as_float(bu.u[e] & 0xffff0000u);
        }
      }
      union { i32x4 q; unsigned u[4]; } o4;
#pragma unroll
      for (int e = 0; e < 4; ++e)
      {
        const float y0 = (v[i][2 * e] - mean) * rstd * w[2 * e] + b[2 * e], y1 = (v[i][2 * e + 1] - mean) * rstd * w[2 * e + 1] + b[2 * e + 1];
        o4.u[e] = a.y_f16 ? pack_f16x2(y0, y1) : pack_bf16x2(y0, y1);
      }
      *(i32x4*)(a.y + (size_t)yrow * a.ldy + 8 * p) = o4.q;
    }
  }
}

}  // namespace

int tk_layer_norm_max_k() { return 64 * 8 * PMAX; }

int tk_launch_layer_norm(LayerNormArgs a, hipStream_t st) {
  dim3 grid((a.M + 3) / 4);
  const bool add = a.r != nullptr;
  if (a.x_f32 && a.wb_f32) {
    if (add)
      hipLaunchKernelGGL((layer_norm_kernel<true, true, true>), grid, dim3(256), 0, st, a);
    else
      hipLaunchKernelGGL((layer_norm_kernel<true, true, false>), grid, dim3(256), 0, st, a);
  } else if (!a.x_f32 && !a.wb_f32) {
    if (add)
      hipLaunchKernelGGL((layer_norm_kernel<false, false, true>), grid, dim3(256), 0, st, a);
    else
      hipLaunchKernelGGL((layer_norm_kernel<false, false, false>), grid, dim3(256), 0, st, a);
  } else {
    return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
