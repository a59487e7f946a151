// Rotary embedding applied in place to the q | k columns of a projection output on gfx950:
//   y[m, h*D + i], y[m, h*D + D/2 + i]  <-  rotate(pair, cos/sin[pos[m], i])     for heads in columns < rope_cols
// for projections that ran as a plain library GEMM (many rows: the VLM prefill).  Same arithmetic as
// the rotary epilogue of the fused projection kernel: fp32 products rounded separately (SmolVLA, fp32
// tables) or every product and the sum rounded to bf16 (pi0.5: x * cos + rotate_half(x) * sin on
// bf16 tensors; the tables then hold bf16 values).  One thread per 8-column chunk of a pair.
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

__global__ __launch_bounds__(256) void rope_rows_kernel(RopeRowsArgs a) {
  const int chunks_per_head = a.half / 8;
  const int chunks = (a.rope_cols / (2 * a.half)) * chunks_per_head;  // per row
  const int m = blockIdx.x;
  int pos = a.pos[m];
  pos = pos < 0 ? 0 : (pos > a.positions - 1 ? a.positions - 1 : pos);
  const float* cs_row = a.cos + (size_t)pos * a.half;
  const float* sn_row = a.sin + (size_t)pos * a.half;
  u16* row = a.y + (size_t)m * a.ldy;
  for (int c = threadIdx.x; c < chunks; c += 256) {
    const int head = c / chunks_per_head, i0 = (c % chunks_per_head) * 8;
    u16* pa = row + head * 2 * a.half + i0;
    u16* pb = pa + a.half;
    union { i32x4 q; i32x2 h[2]; } xa, xb, oa, ob;
    xa.q = *(const i32x4*)pa;
    xb.q = *(const i32x4*)pb;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const f32x4 va = unpack_bf16x4(xa.h[e]), vb = unpack_bf16x4(xb.h[e]);
      const f32x4 cs = *(const f32x4*)(cs_row + i0 + 4 * e), sn = *(const f32x4*)(sn_row + i0 + 4 * e);
      f32x4 ra, rb;
      if (a.bf16_math) {
        const f32x4 ac = unpack_bf16x4(pack_bf16x4(va * cs)), bs = unpack_bf16x4(pack_bf16x4(vb * sn));
        const f32x4 bc = unpack_bf16x4(pack_bf16x4(vb * cs)), as = unpack_bf16x4(pack_bf16x4(va * sn));
        ra = ac - bs;
        rb = bc + as;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          ra[j] = sub_rn(mul_rn(va[j], cs[j]), mul_rn(vb[j], sn[j]));
          rb[j] = add_rn(mul_rn(vb[j], cs[j]), mul_rn(va[j], sn[j]));
        }
      }
      oa.h[e] = pack_bf16x4(ra);
      ob.h[e] = pack_bf16x4(rb);
    }
    *(i32x4*)pa = oa.q;
    *(i32x4*)pb = ob.q;
  }
}

}  // namespace

int tk_launch_rope_rows(RopeRowsArgs a, hipStream_t st) {
  hipLaunchKernelGGL(rope_rows_kernel, dim3(a.M), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
