// Per-request bookkeeping of the prefix and the image patches on gfx950: two launches that replace the two dozen
// tiny elementwise / scan launches which the same work costs as separate tensor operations inside a replayed graph
// (each of them a dependent graph node with its launch gap).
//
//   prefix_meta_kernel   pad[P], att[P] (bytes, 0 / 1) ->
//                          mask2d[i][j] = (cumsum(att)[j] <= cumsum(att)[i]) & pad[i] & pad[j]   (bytes, row pitch p_pad,
//                                         columns P .. p_pad-1 zero): the prefill's 2-D visibility
//                          pos[j]       = clamp(cumsum(pad)[j] - 1, 0, positions - 1)            (rotary positions)
//                          suf_pos[s]   = clamp(sum(pad) + s, 0, positions - 1)                  (the action tokens')
//   prefix_rows_kernel   the fp32 prefix rows [image tokens; language tokens; closing rows] from the connector's bf16 rows
//                        (times a scale, rounded to bf16 as the tensor product rounds it), the bf16 embedding table
//                        gathered by token id (times its scale, likewise) and fp32 closing rows (the state token), and the
//                        pad flags of the same rows from per-camera and per-token flags.
//   patchify_kernel      up to four fp32 images [3][H][W] -> bf16 patch rows [(camera, py, px)][(c, i, j)] of
//                        x * scale + shift (product and sum rounded separately, as two tensor operations round them):
//                        the unfolded input of a non-overlapping patch convolution run as one GEMM.
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

constexpr int kMaxP = 2048;  // prefix tokens (8 per thread)

__global__ __launch_bounds__(256) void prefix_meta_kernel(PrefixMetaArgs a) {
  __shared__ unsigned short c_att[kMaxP], c_pad[kMaxP];
  __shared__ unsigned char s_pad[kMaxP];
  __shared__ int wave_tot[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // inclusive scans of both flag rows: 8 consecutive tokens per thread, wave scan of the thread sums, wave offsets
  // (all sixteen byte loads of a thread are unconditional -- clamped index -- so that they are in flight together:
  // behind a range check each of them waited for the one before, 16 round trips to memory in a row)
  unsigned char rp[8], ra[8];
  const unsigned char* att_or_pad = a.att ? a.att : a.pad;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    int j = tid * 8 + e;
    if (j > a.P - 1) j = a.P - 1;
    rp[e] = a.pad[j];
    ra[e] = att_or_pad[j];
  }
  int la[8], lp[8], sa = 0, sp = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int j = tid * 8 + e;
    const int pv = j < a.P ? (rp[e] != 0) : 0;
    const int av = (j < a.P && a.att) ? (ra[e] != 0) : 0;
    sa += av;
    sp += pv;
    la[e] = sa;
    lp[e] = sp;
    s_pad[j] = (unsigned char)pv;
  }
  int xa = sa, xp = sp;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int ta = __shfl_up(xa, o), tp = __shfl_up(xp, o);
    if (lane >= o) xa += ta, xp += tp;
  }
  if (lane == 63) wave_tot[0][wave] = xa, wave_tot[1][wave] = xp;
  __syncthreads();
  int oa = xa - sa, op = xp - sp;  // exclusive over the lanes before
  for (int w = 0; w < wave; ++w) oa += wave_tot[0][w], op += wave_tot[1][w];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int j = tid * 8 + e;
    c_att[j] = (unsigned short)(oa + la[e]);
    c_pad[j] = (unsigned short)(op + lp[e]);
  }
  __syncthreads();
  const int hi = a.positions - 1;
  if (blockIdx.x == 0) {
    if (a.pos)
      for (int j = tid; j < a.P; j += 256) {
        const int v = (int)c_pad[j] - 1;
        a.pos[j] = v < 0 ? 0 : (v > hi ? hi : v);
      }
    if (a.suf_pos) {
      const int total = a.P > 0 ? (int)c_pad[a.P - 1] : 0;
      for (int s = tid; s < a.S; s += 256) {
        const int v = total + s;
        a.suf_pos[s] = v > hi ? hi : v;
      }
    }
  }
  if (!a.mask2d) return;
  // rows blockIdx.x, + gridDim.x, ..: a thread owns 16 columns of every row (p_pad <= 2048: one pass) and keeps their
  // flags and block counts in registers, so a row costs two broadcast LDS reads and one 16-byte store
  const int j0 = tid * 16;
  if (j0 >= a.p_pad) return;
  unsigned short cj[16];
  unsigned char pj[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    pj[e] = s_pad[j0 + e];  // zero from P on
    cj[e] = c_att[j0 + e];
  }
  for (int i = blockIdx.x; i < a.P; i += gridDim.x) {
    const int ci = c_att[i], pi = s_pad[i];
    union { i32x4 v; unsigned char b[16]; } o;
#pragma unroll
    for (int e = 0; e < 16; ++e) o.b[e] = (unsigned char)(pi & pj[e] & ((int)cj[e] <= ci ? 1 : 0));
    *(i32x4*)(a.mask2d + (size_t)i * a.p_pad + j0) = o.v;
  }
}

// one thread per 8 consecutive pixels of an image row (W a multiple of 8, so is the patch size or the 8 pixels would
// straddle two patches: the host checks ps % 8 == 0)
__global__ __launch_bounds__(256) void patchify_kernel(PatchifyArgs a) {
  const int per_row = a.W / 8;
  const long long per_img = (long long)3 * a.H * per_row;
  const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= per_img * a.n) return;
  const int cam = (int)(gid / per_img);
  long long r = gid % per_img;
  const int xs = (int)(r % per_row) * 8;
  r /= per_row;
  const int y = (int)(r % a.H), c = (int)(r / a.H);
  const float* src = a.img[cam] + ((size_t)c * a.H + y) * a.W + xs;
  const f32x4 v0 = *(const f32x4*)src, v1 = *(const f32x4*)(src + 4);
  f32x4 w0, w1;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    w0[e] = add_rn(mul_rn(v0[e], a.scale), a.shift);
    w1[e] = add_rn(mul_rn(v1[e], a.scale), a.shift);
  }
  const i32x2 lo = pack_bf16x4(w0), hi = pack_bf16x4(w1);
  const int ps = a.ps, py = y / ps, iy = y % ps, px = xs / ps, ix = xs % ps;
  const int n_w = a.W / ps, n_h = a.H / ps;
  u16* dst = (u16*)a.out + (((size_t)cam * n_h + py) * n_w + px) * (size_t)(3 * ps * ps) + ((size_t)c * ps + iy) * ps + ix;
  *(i32x4*)dst = i32x4{lo[0], lo[1], hi[0], hi[1]};
}

// the same with fp32 patch rows and any even patch size: one thread per 2 consecutive pixels of an image row
__global__ __launch_bounds__(256) void patchify_f32_kernel(PatchifyArgs a) {
  const int per_row = a.W / 2;
  const long long per_img = (long long)3 * a.H * per_row;
  const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= per_img * a.n) return;
  const int cam = (int)(gid / per_img);
  long long r = gid % per_img;
  const int xs = (int)(r % per_row) * 2;
  r /= per_row;
  const int y = (int)(r % a.H), c = (int)(r / a.H);
  const f32x2 v = *(const f32x2*)(a.img[cam] + ((size_t)c * a.H + y) * a.W + xs);
  const f32x2 w = {add_rn(mul_rn(v[0], a.scale), a.shift), add_rn(mul_rn(v[1], a.scale), a.shift)};
  const int ps = a.ps, py = y / ps, iy = y % ps, px = xs / ps, ix = xs % ps;
  const int n_w = a.W / ps, n_h = a.H / ps;
  float* dst = (float*)a.out + (((size_t)cam * n_h + py) * n_w + px) * (size_t)(3 * ps * ps) + ((size_t)c * ps + iy) * ps + ix;
  *(f32x2*)dst = w;
}

// one thread per 8 consecutive columns of a prefix row: bf16 image rows and the token rows are scaled in bf16 (product in
// fp32, rounded once, which is what a bf16 tensor times a scalar gives); fp32 image rows and the closing rows are taken
// as they are; the result is written in fp32 or rounded to bf16
__global__ __launch_bounds__(256) void prefix_rows_kernel(PrefixRowsArgs a) {
  const int per_row = a.H / 8;
  const int rows = a.n_img + a.n_tok + a.n_last;
  const int gid = blockIdx.x * 256 + threadIdx.x;
  if (gid >= rows * per_row) return;
  const int row = gid / per_row, c0 = (gid % per_row) * 8;
  const size_t o = (size_t)row * a.H + c0;
  unsigned char flag = 1;
  f32x4 lo, hi;
  const bool closing = row >= a.n_img + a.n_tok;
  if (closing || (row < a.n_img && a.img_f32)) {
    const float* src = closing ? a.last + (size_t)(row - a.n_img - a.n_tok) * a.H + c0 : (const float*)a.img + (size_t)row * a.H + c0;
    lo = *(const f32x4*)src;
    hi = *(const f32x4*)(src + 4);
    if (!closing && a.pad_out) flag = a.cam_flag[row / a.per_cam][0];
  } else {
    const u16* src;
    float scale;
    if (row < a.n_img) {
      src = (const u16*)a.img + (size_t)row * a.H + c0;
      scale = a.img_scale;
      if (a.pad_out) flag = a.cam_flag[row / a.per_cam][0];
    } else {
      const int t = row - a.n_img;
      long long id = a.tokens[t];
      id = id < 0 ? 0 : (id > a.vocab - 1 ? a.vocab - 1 : id);
      src = a.table + (size_t)id * a.H + c0;
      scale = a.tok_scale;
      if (a.pad_out) flag = a.tok_flag[t];
    }
    union { i32x4 q; unsigned u[4]; } x;
    x.q = *(const i32x4*)src;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const unsigned pk = pack_bf16x2(mul_rn(__uint_as_float(x.u[e] << 16), scale), mul_rn(__uint_as_float(x.u[e] & 0xffff0000u), scale));
      const float v0 = __uint_as_float(pk << 16), v1 = __uint_as_float(pk & 0xffff0000u);
      if (e < 2) { lo[2 * e] = v0; lo[2 * e + 1] = v1; } else { hi[2 * (e - 2)] = v0; hi[2 * (e - 2) + 1] = v1; }
    }
  }
  if (a.out_bf16) {
    const i32x2 p0 = pack_bf16x4(lo), p1 = pack_bf16x4(hi);
    *(i32x4*)((u16*)a.out + o) = i32x4{p0[0], p0[1], p1[0], p1[1]};
  } else {
    *(f32x4*)((float*)a.out + o) = lo;
    *(f32x4*)((float*)a.out + o + 4) = hi;
  }
  if (a.pad_out && c0 == 0) a.pad_out[row] = flag ? 1 : 0;
}

}  // namespace

int tk_launch_prefix_rows(PrefixRowsArgs a, hipStream_t st) {
  const long long threads = (long long)(a.n_img + a.n_tok + a.n_last) * (a.H / 8);
  hipLaunchKernelGGL(prefix_rows_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

int tk_prefix_meta_max_tokens() { return kMaxP; }

int tk_launch_prefix_meta(PrefixMetaArgs a, hipStream_t st) {
  // every block repeats the two scans (P bytes each); a block then writes every gridDim-th row of the mask
  int blocks = a.mask2d ? (a.P + 7) / 8 : 1;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(prefix_meta_kernel, dim3(blocks), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

int tk_launch_patchify(PatchifyArgs a, hipStream_t st) {
  const long long threads = (long long)a.n * 3 * a.H * (a.W / (a.out_f32 ? 2 : 8));
  if (a.out_f32)
    hipLaunchKernelGGL(patchify_f32_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL(patchify_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
