// Tail of a denoising step on gfx950: final (adaptive) RMSNorm of the expert hidden state, the fp32
// action projection, and the Euler update, in one launch.
//
//   h[m, :]  = norm(x[m, :])                       bf16, the reference's rounding points
//   v[m, n]  = sum_k float(h[m, k]) * W[n, k] + b[n]            fp32
//   x_out[m, n] = x_t[m, n] + dt * v[m, n]                      fp32 (product and sum rounded separately)
//
// Tiny (50 rows x 32 outputs x 720..1024 inputs): one block per row, the normalised row lives in
// LDS, each thread owns one (output, k-slice) pair and the slices are summed in a fixed order.
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

constexpr int kThreads = 256;
constexpr int kHeld = 32;  // weight pieces per thread held in registers (K = 1024 with 32 outputs)

__global__ __launch_bounds__(kThreads) void expert_tail_kernel(TailArgs a) {
  extern __shared__ __align__(16) float hrow[];  // [K] normalised row, as fp32 values of bf16 numbers
  __shared__ float red[kThreads / 64];
  __shared__ float part[kThreads];
  const int m = blockIdx.x;
  const int tid = threadIdx.x;
  const u16* x = a.x + (size_t)m * a.ldx;

  // thread -> (output n, k slice): slices of an output are consecutive threads
  const int slices = kThreads / a.N;  // host guarantees N divides kThreads and N <= kThreads
  const int n = tid / slices, sl = tid % slices;
  const float* w = a.w + (size_t)n * a.K;
  const int pieces = a.K / 4;  // 16-byte pieces of a weight row (K is a multiple of 4: checked by the host)
  // The weights, the bias and x_t depend on nothing computed here: requested before the row statistics,
  // they arrive during the first round trip instead of starting three more after it.  The slices of an
  // output read consecutive pieces; the first kHeld pieces of a thread are held in registers.
  f32x4 wreg[kHeld];
#pragma unroll
  for (int i = 0; i < kHeld; ++i) {
    const int p = sl + i * slices;
    const f32x4 wv = *(const f32x4*)(w + 4 * (p < pieces ? p : 0));
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    wreg[i] = p < pieces ? wv : zero;
  }
  const size_t oidx = (size_t)m * a.N + n;
  const float bias_n = a.bias ? a.bias[n] : 0.f;
  const float xt_n = a.x_out ? a.x_t[oidx] : 0.f;

  float ss = 0.f;
  for (int k = tid; k < a.K; k += kThreads) {
    const float f = bf16_bits_to_f32(x[k]);
    ss = fmaf(f, f, ss);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < kThreads / 64; ++w) tot += red[w];
  const float rstd = rsqrtf(tot / (float)a.K + a.eps);

  for (int k = tid; k < a.K; k += kThreads) {
    const float f = bf16_bits_to_f32(x[k]);
    float h;
    if (a.ada_scale) {
      // adaptive: bf16((x * rstd) * (1 + scale) + shift), fp32 steps rounded separately
      h = round_bf16(add_rn(mul_rn(mul_rn(f, rstd), add_rn(1.0f, a.ada_scale[k])), a.ada_shift[k]));
    } else {
      // Llama RMSNorm on a bf16 row: bf16(w * bf16(x * rstd))
      h = round_bf16(bf16_bits_to_f32(a.norm_w[k]) * round_bf16(f * rstd));
    }
    hrow[k] = h;
  }
  __syncthreads();

  float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
  for (int i = 0; i < kHeld; ++i) {
    const int p = sl + i * slices;
    const f32x4 hv = *(const f32x4*)(hrow + 4 * (p < pieces ? p : 0));  // (a piece past the row meets zero weights)
    acc0 = fmaf(hv[0], wreg[i][0], acc0);
    acc1 = fmaf(hv[1], wreg[i][1], acc1);
    acc0 = fmaf(hv[2], wreg[i][2], acc0);
    acc1 = fmaf(hv[3], wreg[i][3], acc1);
  }
#pragma unroll 8
  for (int p = sl + kHeld * slices; p < pieces; p += slices) {  // rows wider than the held pieces cover
    const f32x4 wv = *(const f32x4*)(w + 4 * p);
    const f32x4 hv = *(const f32x4*)(hrow + 4 * p);
    acc0 = fmaf(hv[0], wv[0], acc0);
    acc1 = fmaf(hv[1], wv[1], acc1);
    acc0 = fmaf(hv[2], wv[2], acc0);
    acc1 = fmaf(hv[3], wv[3], acc1);
  }
  part[tid] = acc0 + acc1;
  __syncthreads();
  if (sl == 0) {
    float v = 0.f;
    for (int j = 0; j < slices; ++j) v += part[tid + j];
    if (a.bias) v += bias_n;
    if (a.v_out) a.v_out[oidx] = v;
    if (a.x_out) a.x_out[oidx] = add_rn(xt_n, mul_rn(a.dt, v));
  }
}

}  // namespace

int tk_launch_tail(TailArgs a, hipStream_t st) {
  hipLaunchKernelGGL(expert_tail_kernel, dim3(a.M), dim3(kThreads), (size_t)a.K * sizeof(float), st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
