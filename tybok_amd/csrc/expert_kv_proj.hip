// Expert K/V projection of the cached VLM prefix for the cross-attention layers, fused with the
// attention kernel's operand layout: one launch instead of two casts, two fp32 GEMMs and a split.
//
//   ek = float(K_pre) . Wk^T,  ev = float(V_pre) . Wv^T      (fp32 weights, fp32 accumulate:
//   tybok/policies/smolvla/models/expert.py:35-39, flow_matching.py:553-578)
//   -> K as bf16 hi + lo planes [P, G, D], V^T as bf16 hi + lo planes [G, D, ld] (keys contiguous,
//      zero filled from P to the next multiple of 32) -- what tk_attn_prepare_kv produces from ek, ev.
//
// A block computes a 32 (output columns) x 32 (prefix rows) tile of K or V on the fp32 matrix
// instruction v_mfma_f32_32x32x2_f32 (full fp32 products and sums), its four waves splitting the input columns.  The weight rows are the A
// operand and the prefix rows the B operand, both read straight from global memory: lane (r, h)
// loads 16 consecutive input columns' worth of its row in 16-byte pieces -- columns 16j + 8h .. + 7
// for step j -- and feeds them to 8 MFMAs; which k pairs meet in one instruction does not matter
// as long as both operands use the same assignment.  The accumulators hold C^T like the GEMM
// kernels: a lane owns one prefix row and, per register group, four consecutive output columns.
// Fixed instruction order -> same bits every run.
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

constexpr int JB = 5;  // k steps (of 16 input columns) a wave has in flight together (KV = 320: all of its five)

// A block of four waves owns one 32 x 32 tile: wave w walks every fourth batch of JB k steps (a 160-instruction
// fp32 MFMA chain on one wave took 5 us of the launch; four waves of 40 on one CU, 160 blocks instead of 48), the
// partial tiles meet in LDS and wave g finishes register group g (columns 8g .. 8g + 7): sum in wave order.
__global__ __launch_bounds__(256) void expert_kv_proj_kernel(KvProjArgs a) {
  __shared__ f32x4 red[4][4][64];  // [wave][register group][lane]
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const int nt = blockIdx.y;  // 32-column tile of the output
  const bool is_v = (blockIdx.z & 1) != 0;
  const int layer = blockIdx.z >> 1;  // (several layers' projections in one launch: independent problems)
  int p = blockIdx.x * 32 + l32;
  const int pc = p < a.P ? p : a.P - 1;  // rows past P: valid data, zeroed / skipped below
  const u16* xrow = (is_v ? a.v[layer] : a.k[layer]) + (size_t)pc * a.sl + 8 * half;
  const float* wrow = (is_v ? a.wv[layer] : a.wk[layer]) + (size_t)(nt * 32 + l32) * a.KV + 8 * half;

  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  const int steps = a.KV / 16;
  for (int j0 = wave * JB; j0 < steps; j0 += 4 * JB) {  // wave-uniform
    i32x4 xr[JB];
    f32x4 wr[JB][2];
#pragma unroll
    for (int jj = 0; jj < JB; ++jj) {
      const int j = j0 + jj < steps ? j0 + jj : steps - 1;  // clamped: unconditional loads
      xr[jj] = *(const i32x4*)(xrow + 16 * j);
      wr[jj][0] = *(const f32x4*)(wrow + 16 * j);
      wr[jj][1] = *(const f32x4*)(wrow + 16 * j + 4);
    }
#pragma unroll
    for (int jj = 0; jj < JB; ++jj) {
      if (j0 + jj < steps) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const unsigned pair = (unsigned)xr[jj][i >> 1];
          const float xv = __uint_as_float((i & 1) ? (pair & 0xffff0000u) : (pair << 16));
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[jj][i >> 2][i & 3], xv, acc, 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int g = 0; g < 4; ++g) red[wave][g][lane] = f32x4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
  __syncthreads();

  // lane: prefix row p, output columns nt*32 + 8g + 4*half + 0..3 of register group g = wave
  {
    const int g = wave;
    const int n = nt * 32 + 8 * g + 4 * half;
    f32x4 v = red[0][g][lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) v += red[w][g][lane];
    if (p >= a.P) v = f32x4{0.f, 0.f, 0.f, 0.f};
    const i32x2 hi = pack_bf16x4(v);
    const i32x2 lo = pack_bf16x4(v - unpack_bf16x4(hi));
    if (!is_v) {
      if (p < a.P) {
        const size_t o = ((size_t)layer * a.P + p) * a.N + n;
        *(i32x2*)(a.k_hi + o) = hi;
        *(i32x2*)(a.k_lo + o) = lo;
      }
    } else if (p < a.ld) {
      // V^T rows are output columns, keys contiguous: the 32 lanes of a half write 64 contiguous bytes
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const size_t o = ((size_t)layer * a.N + n + j) * a.ld + p;
        a.vt_hi[o] = (u16)(((unsigned)hi[j >> 1]) >> (16 * (j & 1)));
        a.vt_lo[o] = (u16)(((unsigned)lo[j >> 1]) >> (16 * (j & 1)));
      }
    }
  }
}

}  // namespace

int tk_launch_kv_proj(KvProjArgs a, hipStream_t st) {
  dim3 grid((a.P + 31) / 32, a.N / 32, 2 * a.L);
  hipLaunchKernelGGL(expert_kv_proj_kernel, grid, dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
