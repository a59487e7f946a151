// Tail of a denoising step on gfx950: final (adaptive) RMSNorm of the expert hidden state, the fp32
// action projection, and the Euler update, in one launch.
//
//   h[m, :]  = norm(x[m, :])                       bf16, the reference's rounding points
//   v[m, n]  = sum_k float(h[m, k]) * W[n, k] + b[n]            fp32
//   x_out[m, n] = x_t[m, n] + dt * v[m, n]                      fp32 (product and sum rounded separately)
//   e[m, j]  = act(sum_n x_out[m, n] * E[j, n] + c[j])          optional: the next step's suffix embedding
//
// Tiny (50 rows x 32 outputs x 720..1024 inputs): one block per row, the normalised row lives in
// LDS, each thread owns one (output, k-slice) pair and the slices are summed in a fixed order.
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

constexpr int kThreads = 256;
constexpr int kHeld = 32;  // weight pieces per thread held in registers (K = 1024 with 32 outputs)
constexpr int kXHeld = 4;  // elements of the row per thread held in registers (K = 1024)
constexpr int kEmbN = 32;  // the embedding's input width (= N) its rows are held for
constexpr int kEmbHeld = 4;  // embedding outputs per thread whose weight rows are held (J = 1024)

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
  // Requests in the order of use (memory returns in order): the row, then the weights, the bias and x_t, then the
  // embedding's weights -- none depends on anything computed here, so all are out before the first wait.  The
  // slices of an output read consecutive pieces; the first kHeld pieces of a thread are held in registers.
  u16 xreg[kXHeld];
#pragma unroll
  for (int i = 0; i < kXHeld; ++i) {
    const int k = tid + i * kThreads;
    xreg[i] = x[k < a.K ? k : a.K - 1];
  }
  // the norm's operands of the same elements
  float nw0[kXHeld], nw1[kXHeld];  // RMSNorm: the weight; adaptive: scale, shift
#pragma unroll
  for (int i = 0; i < kXHeld; ++i) {
    const int k = tid + i * kThreads < a.K ? tid + i * kThreads : a.K - 1;
    if (a.ada_scale) {
      nw0[i] = a.ada_scale[k];
      nw1[i] = a.ada_shift[k];
    } else {
      nw0[i] = bf16_bits_to_f32(a.norm_w[k]);
      nw1[i] = 0.f;
    }
  }
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

  // the embedding's weight rows of this thread's outputs j = tid, tid + 256, ... (N = kEmbN wide)
  f32x4 ereg[kEmbHeld][kEmbN / 4];
  const bool emb = a.emb_out != nullptr;
  if (emb) {  // block-uniform
#pragma unroll
    for (int i = 0; i < kEmbHeld; ++i) {
      const int j = tid + i * kThreads;
      const float* er = a.emb_w + (size_t)(j < a.emb_J ? j : 0) * kEmbN;  // past the last output: a valid row, not used
#pragma unroll
      for (int q = 0; q < kEmbN / 4; ++q) ereg[i][q] = *(const f32x4*)(er + 4 * q);
    }
  }

  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kXHeld; ++i) {
    const float f = bf16_bits_to_f32(xreg[i]);
    if (tid + i * kThreads < a.K) ss = fmaf(f, f, ss);
  }
  for (int k = tid + kXHeld * kThreads; k < a.K; k += kThreads) {
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

  auto norm_to_lds = [&](int k, float f, float n0, float n1) {
    float h;
    if (a.ada_scale) {
      // adaptive: bf16((x * rstd) * (1 + scale) + shift), fp32 steps rounded separately
      h = round_bf16(add_rn(mul_rn(mul_rn(f, rstd), add_rn(1.0f, n0)), n1));
    } else {
      // Llama RMSNorm on a bf16 row: bf16(w * bf16(x * rstd))
      h = round_bf16(n0 * round_bf16(f * rstd));
    }
    hrow[k] = h;
  };
#pragma unroll
  for (int i = 0; i < kXHeld; ++i)
    if (tid + i * kThreads < a.K) norm_to_lds(tid + i * kThreads, bf16_bits_to_f32(xreg[i]), nw0[i], nw1[i]);
  for (int k = tid + kXHeld * kThreads; k < a.K; k += kThreads) {
    if (a.ada_scale) norm_to_lds(k, bf16_bits_to_f32(x[k]), a.ada_scale[k], a.ada_shift[k]);
    else norm_to_lds(k, bf16_bits_to_f32(x[k]), bf16_bits_to_f32(a.norm_w[k]), 0.f);
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
  __shared__ float xn[kThreads];  // the updated row (N values)
  if (sl == 0) {
    float v = 0.f;
    for (int j = 0; j < slices; ++j) v += part[tid + j];
    if (a.bias) v += bias_n;
    if (a.v_out) a.v_out[oidx] = v;
    if (a.x_out) {
      const float xo = add_rn(xt_n, mul_rn(a.dt, v));
      a.x_out[oidx] = xo;
      xn[n] = xo;
    }
  }
  if (!emb) return;  // block-uniform
  // ---- the next step's suffix embedding of this row: e[j] = act(sum_n x_out[n] * E[j, n] + c[j]), fp32 ----
  __syncthreads();
  for (int i = 0; tid + i * kThreads < a.emb_J; ++i) {
    const int j = tid + i * kThreads;
    float e0 = 0.f, e1 = 0.f;
    if (i < kEmbHeld) {
#pragma unroll
      for (int ii = 0; ii < kEmbHeld; ++ii) {
        if (ii == i) {
#pragma unroll
          for (int q = 0; q < kEmbN / 4; ++q) {
            e0 = fmaf(xn[4 * q], ereg[ii][q][0], e0);
            e1 = fmaf(xn[4 * q + 1], ereg[ii][q][1], e1);
            e0 = fmaf(xn[4 * q + 2], ereg[ii][q][2], e0);
            e1 = fmaf(xn[4 * q + 3], ereg[ii][q][3], e1);
          }
        }
      }
    } else {
      const float* er = a.emb_w + (size_t)j * kEmbN;
#pragma unroll
      for (int q = 0; q < kEmbN / 4; ++q) {
        const f32x4 ev = *(const f32x4*)(er + 4 * q);
        e0 = fmaf(xn[4 * q], ev[0], e0);
        e1 = fmaf(xn[4 * q + 1], ev[1], e1);
        e0 = fmaf(xn[4 * q + 2], ev[2], e0);
        e1 = fmaf(xn[4 * q + 3], ev[3], e1);
      }
    }
    float e = e0 + e1;
    if (a.emb_b) e += a.emb_b[j];
    if (a.emb_act == 1) e = e / (1.0f + expf(-e));  // SiLU in fp32
    if (a.emb_bf16) ((u16*)a.emb_out)[(size_t)m * a.emb_ld + j] = f32_to_bf16_bits(e);
    else ((float*)a.emb_out)[(size_t)m * a.emb_ld + j] = e;
  }
}

}  // namespace

int tk_tail_embed_width() { return kEmbN; }

int tk_launch_tail(TailArgs a, hipStream_t st) {
  hipLaunchKernelGGL(expert_tail_kernel, dim3(a.M), dim3(kThreads), (size_t)a.K * sizeof(float), st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
