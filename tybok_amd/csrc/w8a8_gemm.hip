// W8A8 tier of the VLM prefill MLP on gfx950: per-token activation quantisation and the fp8 x fp8 GEMM.
//
//   quant_act_rows_kernel   x[M,K] bf16 -> a8[M,K] e4m3fn, sa[M] fp32 with sa = amax_k|x| / 448 and
//                           a8 = RNE(x / sa) in fp32 (one rounding); an all-zero row gives sa = 0 and zero codes.
//   w8a8_wide_kernel<EPI>   y[M,N] = bf16((a8 . W8^T) * sa[m] * sw[n]) on v_mfma_f32_32x32x64_f8f6f4 (e4m3 x e4m3,
//                           fp32 accumulate, 64 k per instruction).  Same packed weight tiles and the same block
//                           shape as the weight-only many-row kernel: 4 waves own 128 rows x 256 packed columns,
//                           wave w the n tiles 2w, 2w+1 for all rows; weights go straight from global memory into
//                           operand registers (a lane's 16-byte chunks of two consecutive k tiles are one 32-byte
//                           operand), the quantised activations of a round (128 rows x 128 k) are staged once per
//                           block through LDS as bytes -- half the LDS traffic per k of the bf16 kernel at twice
//                           the product rate.  The order of k inside an instruction is the same permutation for both
//                           operands (bytes 0-15 of a lane: k tile 2s, bytes 16-31: k tile 2s+1), which a dot
//                           product does not see.
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

constexpr int NT = 2;   // n tiles per wave
constexpr int NW = 4;   // waves per block
constexpr int RK = 4;   // 32-wide k tiles per round (two 64-wide product steps)
constexpr int PF = 3;   // rounds in flight

// EPI: 0 plain (scales, optional residual), 1 gated (gate/up tile pairs -> act(g) * u).  MT: 32-row tiles per block
// (and per wave): 4 with one block per CU, 2 with two -- co-resident blocks cover each other's first loads
// and epilogue, which weigh as much as the k loop when K is a few thousand.
template <int EPI, int MT, int OCC>
__global__ __launch_bounds__(NW * 64, OCC) void w8a8_wide_kernel(GemmArgs a, int nblk_m, int ngroups) {
  constexpr int ROWS = MT * 32;
  constexpr int ROWB = RK * 32;            // bytes of one staged (fp8) activation row per round
  constexpr int PITCH = ROWB + 16;
  constexpr int XBUF = ROWS * PITCH;
  constexpr int PPR = ROWB / 16;           // 16-byte pieces per staged row
  constexpr int XPT = ROWS * PPR / (NW * 64);
  constexpr int TILES = MT * NT;
  constexpr int STEPS = RK / 2;            // 64-wide product steps per round
  constexpr int EPB = NW * 32 * ((EPI == 0 ? NT * 32 : 32) * 2 + 16);  // the epilogue's per-wave tiles
  __shared__ __align__(16) unsigned char lds[2 * XBUF > EPB ? 2 * XBUF : EPB];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5;
  const int l32 = lane & 31;

  // blocks that share weights (same n tiles and k range, different rows) get consecutive slots of one XCD
  const unsigned id = blockIdx.x;
  const unsigned slot = id >> 3;
  const int mblock = (int)(slot % (unsigned)nblk_m);
  const int group = (int)((slot / (unsigned)nblk_m) * 8 + (id & 7));
  if (group >= ngroups) return;
  const int split = group % a.ksplit;
  const int nblk = group / a.ksplit;

  const int kt_lo = split * a.kt_q + (split < a.kt_r ? split : a.kt_r);
  const int kt_hi = kt_lo + a.kt_q + (split < a.kt_r ? 1 : 0);
  const int nrounds = (kt_hi - kt_lo + RK - 1) / RK;
  const int k_end = kt_hi * 32 < a.K ? kt_hi * 32 : a.K;

  const int strip = nblk * NW + wave;
  const uint8_t* wbase[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int ntg = strip * NT + nt;
    if (ntg > a.ntiles - 1) ntg = a.ntiles - 1;  // overhanging tiles are computed on valid data, never stored
    wbase[nt] = a.w + ((size_t)ntg * a.KT) * 1024 + lane * 16;
  }

  const char* xsrc[XPT];
  int xcol[XPT], xdst[XPT];
#pragma unroll
  for (int i = 0; i < XPT; ++i) {
    const int p = tid + i * NW * 64;
    const int r = p / PPR, c = p % PPR;
    int m = mblock * ROWS + r;
    if (m > a.M - 1) m = a.M - 1;  // rows past M: valid data, never stored
    xsrc[i] = (const char*)a.x + (size_t)m * a.ldx;  // one byte per element
    xcol[i] = c * 16;
    xdst[i] = r * PITCH + c * 16;
  }

  f32x16 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;

  struct WFrag {
    i32x4 w[RK][NT];
  };
  struct XFrag {
    i32x4 v[XPT];
  };
  // One piece of each kind of work, so that a round can deal them out between its matrix instructions: a wave
  // cannot issue anything while it waits for the matrix pipe to take its next instruction, so whatever stands
  // between two groups of matrix instructions in program order runs with the pipe empty.
  auto wload1 = [&](WFrag& f, int r, int st, int q) {  // q in [0, 2*NT): k tile 2*st + q/NT of round r, n tile q%NT
    const int j = 2 * st + q / NT, nt = q % NT;
    int kt = kt_lo + r * RK + j;
    if (kt > a.KT - 1) kt = a.KT - 1;  // its activation columns are zeroed
    f.w[j][nt] = *(const i32x4*)(wbase[nt] + (size_t)kt * 1024);
  };
  auto xload1 = [&](XFrag& f, int r, int i) {
    int k = (kt_lo + r * RK) * 32 + xcol[i];
    if (k > a.K - 16) k = a.K - 16;
    f.v[i] = *(const i32x4*)(xsrc[i] + k);
  };
  auto xstore1 = [&](const XFrag& f, int r, int b, int i) {
    const i32x4 z = {0, 0, 0, 0};
    *(i32x4*)(lds + b * XBUF + xdst[i]) = ((kt_lo + r * RK) * 32 + xcol[i]) < k_end ? f.v[i] : z;
  };
  // operand fragments of the round's two 64-wide steps, as the 16-byte halves they are read in
  static_assert(STEPS == 2, "a round is two phases");
  i32x4 xa[STEPS][MT][2];
  auto xread1 = [&](int st, int b, int u) {  // u in [0, 2*MT): half u%2 of m tile u/2
    xa[st][u / 2][u % 2] = *(const i32x4*)(lds + b * XBUF + ((u / 2) * 32 + l32) * PITCH + st * 64 + 16 * half + 32 * (u % 2));
  };
  auto mma1 = [&](const WFrag& f, int st, int t) {  // t in [0, MT*NT): m tile t/NT, n tile t%NT
    const int mt = t / NT, nt = t % NT;
    const i32x4 wl = f.w[2 * st][nt], wh = f.w[2 * st + 1][nt], xl = xa[st][mt][0], xh = xa[st][mt][1];
    const i32x8 wb = {wl[0], wl[1], wl[2], wl[3], wh[0], wh[1], wh[2], wh[3]};
    const i32x8 xb = {xl[0], xl[1], xl[2], xl[3], xh[0], xh[1], xh[2], xh[3]};
    acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wb, xb, acc[mt][nt], 0, 0, 0, 0, 0, 0);
  };

  // PF rounds in flight, every load unconditional (clamped addresses; columns past the block's k range are
  // zeroed when staged).  Round r, phase A: multiplies step 0 while step 1's operands are fetched from LDS, round
  // r+1 is staged into the other LDS buffer and the weight registers that round r-1's step 1 has left are
  // refilled; then the round's only barrier (a wave can write buffer b for round r+2 only after every wave has
  // passed the barrier of round r+1, i.e. has its round-r operands in registers); phase B: fetches round r+1's
  // first operands, multiplies step 1 and refills step 0's weight registers.  A phase never reloads registers its
  // own matrix instructions read.  Each of a phase's MT*NT matrix instructions is followed by its share of the
  // other work, fenced so that the order stands.
  constexpr int SLOTS = MT * NT;
  static_assert(SLOTS == 2 * MT && SLOTS >= 2 * NT && 2 * XPT <= SLOTS, "one operand read per slot; the other pieces fit");
  WFrag wbuf[PF];
  XFrag xbuf[PF];
#pragma unroll
  for (int p = 0; p < PF; ++p) {
#pragma unroll
    for (int i = 0; i < XPT; ++i) xload1(xbuf[p], p, i);
#pragma unroll
    for (int q = 0; q < 2 * NT; ++q) {
      wload1(wbuf[p], p, 0, q);
      wload1(wbuf[p], p, 1, q);
    }
  }
#pragma unroll
  for (int i = 0; i < XPT; ++i) xstore1(xbuf[0], 0, 0, i);
#pragma unroll
  for (int i = 0; i < XPT; ++i) xload1(xbuf[0], PF, i);
  lds_barrier();
#pragma unroll
  for (int u = 0; u < 2 * MT; ++u) xread1(0, 0, u);
  auto round = [&](int p, int r) {
    const int b = r & 1;
    const int pn = (p + 1) % PF, pp = (p + PF - 1) % PF;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      mma1(wbuf[p], 0, i);
      xread1(1, b, i);
      if (i < XPT) xstore1(xbuf[pn], r + 1, b ^ 1, i);
      if (i >= SLOTS - XPT) xload1(xbuf[pn], r + 1 + PF, i - (SLOTS - XPT));
      if (i < 2 * NT) wload1(wbuf[pp], r - 1 + PF, 1, i);  // the registers round r-1 finished with in its phase B
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      mma1(wbuf[p], 1, i);
      xread1(0, b ^ 1, i);
      if (i < 2 * NT) wload1(wbuf[p], r + PF, 0, i);  // step 0's registers: free since phase A
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  {
    int it = 0;
    for (; it + PF <= nrounds; it += PF) {
#pragma unroll
      for (int p = 0; p < PF; ++p) round(p, it + p);
    }
    const int rem = nrounds - it;  // in [0, PF)
#pragma unroll
    for (int q = 0; q < PF - 1; ++q)
      if (q < rem) round(q, it + q);  // block-uniform
  }

  // ---- K-split hand-off: fp32 partials [(block, split)][wave][tile][group][lane][4], last arriver sums in split order
  const int blk_lin = nblk * nblk_m + mblock;
  if (a.ksplit > 1 && a.split_reduce) {
    // the partial leaves as it is (plain 16-byte stores: the kernel boundary publishes it); w8a8_split_reduce_kernel
    // finishes
    f32x4* mine = (f32x4*)a.partial + ((size_t)blk_lin * a.ksplit + split) * (NW * TILES * 4 * 64) + (size_t)wave * TILES * 4 * 64 + lane;
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x16& c = acc[t / NT][t % NT];
        mine[(t * 4 + g) * 64] = f32x4{c[4 * g], c[4 * g + 1], c[4 * g + 2], c[4 * g + 3]};
      }
    return;
  }
  if (a.ksplit > 1) {
    unsigned long long* pbase = (unsigned long long*)a.partial + ((size_t)wave * TILES * 4 * 64 + lane) * 2;
    unsigned long long* mine = pbase + ((size_t)blk_lin * a.ksplit + split) * (NW * TILES * 4 * 64 * 2);
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x16& c = acc[t / NT][t % NT];
        unsigned long long* dst = mine + (size_t)(t * 4 + g) * 128;
        st_agent64(dst, c[4 * g], c[4 * g + 1]);
        st_agent64(dst + 1, c[4 * g + 2], c[4 * g + 3]);
      }
    __shared__ int s_last;
    handoff_publish();  // the write-through stores are acknowledged: visible to every block
    __syncthreads();
    if (threadIdx.x == 0) {
      int old = __hip_atomic_fetch_add(a.counters + blk_lin, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = (old == a.ksplit - 1);
    }
    __syncthreads();
    if (!s_last) return;
    handoff_acquire();
    if (threadIdx.x == 0) __hip_atomic_store(a.counters + blk_lin, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;
    for (int s = 0; s < a.ksplit; ++s) {
      const unsigned long long* src = pbase + ((size_t)blk_lin * a.ksplit + s) * (NW * TILES * 4 * 64 * 2);
      unsigned long long raw[TILES][4][2];
#pragma unroll
      for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          raw[t][g][0] = ld_agent64(src + (size_t)(t * 4 + g) * 128);
          raw[t][g][1] = ld_agent64(src + (size_t)(t * 4 + g) * 128 + 1);
        }
#pragma unroll
      for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x16& c = acc[t / NT][t % NT];
          c[4 * g] += __uint_as_float((unsigned)raw[t][g][0]);
          c[4 * g + 1] += __uint_as_float((unsigned)(raw[t][g][0] >> 32));
          c[4 * g + 2] += __uint_as_float((unsigned)raw[t][g][1]);
          c[4 * g + 3] += __uint_as_float((unsigned)(raw[t][g][1] >> 32));
        }
    }
  }

  // ---- epilogue: lane l of a tile owns row m = l % 32 and, per register group g, columns 8g + 4*(l/32) .. +3;
  // out = (acc * sa[m]) * sw[n], one bf16 rounding (the reference's `acc * a_scale[:, None] * w_scale[None, :]`)
  float sa[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = (mblock * MT + mt) * 32 + l32;
    if (m > a.M - 1) m = a.M - 1;
    sa[mt] = a.row_scale[m];
  }
  if (a.vec16) {
    // Coalesced stores: a lane holds, per tile, row l % 32 and four 4-column pieces 16 bytes apart -- stored as
    // they are, one instruction would touch 32 rows with 16 bytes each.  Each wave therefore passes its 32 rows of
    // an m tile through a private LDS tile (a wave's LDS instructions execute in order, so it needs no barrier of its own) and stores
    // them as 16-byte chunks of consecutive columns, whole 64- or 128-byte segments of a row per 4 or 8 lanes.
    constexpr int COLS = EPI == 0 ? NT * 32 : 32;       // output columns of a wave per row
    constexpr int EP = COLS * 2 + 16;                   // LDS row pitch (bytes)
    constexpr int LPR = COLS / 8;                       // lanes (16-byte chunks) per row
    constexpr int RPI = 64 / LPR;                       // rows per store instruction
    static_assert(NW * 32 * EP == EPB, "the epilogue tiles fit the LDS array");
    lds_barrier();  // every wave has left the staged activations behind
    unsigned char* wl = lds + wave * 32 * EP;
    const int ncol0 = EPI == 0 ? strip * NT * 32 : strip * 32;  // first output column of this wave
    f32x4 sc0[EPI == 0 ? NT : 1][4], sc1[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (EPI == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          int n0 = (strip * NT + nt) * 32 + 8 * g + 4 * half;
          if (n0 > a.N - 4) n0 = a.N - 4;  // columns past N are never stored
          sc0[EPI == 0 ? nt : 0][g] = *(const f32x4*)(a.s0 + n0);
        }
      } else {
        int col = strip * 32 + 8 * g + 4 * half;
        if (col > a.N - 4) col = a.N - 4;
        sc0[0][g] = *(const f32x4*)(a.s0 + col);
        sc1[g] = *(const f32x4*)(a.s1 + col);
      }
    }
    const int lrow = lane / LPR, lchunk = lane % LPR;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (EPI == 0) {
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const f32x16& c = acc[mt][nt];
            f32x4 v = {c[4 * g], c[4 * g + 1], c[4 * g + 2], c[4 * g + 3]};
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = mul_rn(mul_rn(v[j], sa[mt]), sc0[EPI == 0 ? nt : 0][g][j]);
            *(i32x2*)(wl + l32 * EP + (nt * 32 + 8 * g + 4 * half) * 2) = pack_bf16x4(v);
          }
        } else {
          const f32x16& cg = acc[mt][0];
          const f32x16& cu = acc[mt][1];
          f32x4 vg = {cg[4 * g], cg[4 * g + 1], cg[4 * g + 2], cg[4 * g + 3]};
          f32x4 vu = {cu[4 * g], cu[4 * g + 1], cu[4 * g + 2], cu[4 * g + 3]};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            vg[j] = mul_rn(mul_rn(vg[j], sa[mt]), sc0[0][g][j]);
            vu[j] = mul_rn(mul_rn(vu[j], sa[mt]), sc1[g][j]);
          }
          const f32x4 gg = unpack_bf16x4(pack_bf16x4(vg));
          const f32x4 up = unpack_bf16x4(pack_bf16x4(vu));
          f32x4 act;
#pragma unroll
          for (int j = 0; j < 4; ++j) act[j] = a.act == 0 ? silu_f(gg[j]) : gelu_tanh_f(gg[j]);
          act = unpack_bf16x4(pack_bf16x4(act));
          *(i32x2*)(wl + l32 * EP + (8 * g + 4 * half) * 2) = pack_bf16x4(act * up);
        }
      }
#pragma unroll
      for (int j = 0; j < 32 / RPI; ++j) {
        const int row = j * RPI + lrow;
        const int m = (mblock * MT + mt) * 32 + row;
        const int n = ncol0 + lchunk * 8;
        i32x4 t = *(const i32x4*)(wl + row * EP + lchunk * 16);
        if (m >= a.M || n >= a.N) continue;
        if (EPI == 0 && a.resid) {
          // bf16(y + resid) on the bf16-rounded product, as the scattered path computes it
          f32x4 r0, r1 = {0.f, 0.f, 0.f, 0.f};
          if (a.resid_f32) {
            const f32x4* rp = (const f32x4*)((const float*)a.resid + (size_t)m * a.ldr + n);
            r0 = rp[0];
            if (n + 8 <= a.N) r1 = rp[1];
          } else if (n + 8 <= a.N) {
            const i32x4 rr = *(const i32x4*)((const u16*)a.resid + (size_t)m * a.ldr + n);
            r0 = unpack_bf16x4(i32x2{rr[0], rr[1]});
            r1 = unpack_bf16x4(i32x2{rr[2], rr[3]});
          } else {
            r0 = unpack_bf16x4(*(const i32x2*)((const u16*)a.resid + (size_t)m * a.ldr + n));
          }
          const i32x2 lo = pack_bf16x4(unpack_bf16x4(i32x2{t[0], t[1]}) + r0), hi = pack_bf16x4(unpack_bf16x4(i32x2{t[2], t[3]}) + r1);
          t = i32x4{lo[0], lo[1], hi[0], hi[1]};
        }
        u16* dst = a.y + (size_t)m * a.ldy + n;
        if (n + 8 <= a.N) *(i32x4*)dst = t;
        else *(i32x2*)dst = i32x2{t[0], t[1]};  // N % 8 == 4: the row's last four columns
      }
    }
    return;
  }
  if (EPI == 0) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n0 = (strip * NT + nt) * 32 + 8 * g + 4 * half;
        if (n0 >= a.N) continue;
        const f32x4 sc = *(const f32x4*)(a.s0 + n0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int m = (mblock * MT + mt) * 32 + l32;
          if (m >= a.M) continue;
          const f32x16& c = acc[mt][nt];
          f32x4 v = {c[4 * g], c[4 * g + 1], c[4 * g + 2], c[4 * g + 3]};
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = mul_rn(mul_rn(v[j], sa[mt]), sc[j]);
          i32x2 r = pack_bf16x4(v);
          if (a.resid) {
            const f32x4 rv = a.resid_f32 ? *(const f32x4*)((const float*)a.resid + (size_t)m * a.ldr + n0)
                                         : unpack_bf16x4(*(const i32x2*)((const u16*)a.resid + (size_t)m * a.ldr + n0));
            r = pack_bf16x4(unpack_bf16x4(r) + rv);
          }
          *(i32x2*)(a.y + (size_t)m * a.ldy + n0) = r;
        }
      }
  } else {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int col = strip * 32 + 8 * g + 4 * half;
      if (col >= a.N) continue;
      const f32x4 scg = *(const f32x4*)(a.s0 + col), scu = *(const f32x4*)(a.s1 + col);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = (mblock * MT + mt) * 32 + l32;
        if (m >= a.M) continue;
        const f32x16& cg = acc[mt][0];
        const f32x16& cu = acc[mt][1];
        f32x4 vg = {cg[4 * g], cg[4 * g + 1], cg[4 * g + 2], cg[4 * g + 3]};
        f32x4 vu = {cu[4 * g], cu[4 * g + 1], cu[4 * g + 2], cu[4 * g + 3]};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          vg[j] = mul_rn(mul_rn(vg[j], sa[mt]), scg[j]);
          vu[j] = mul_rn(mul_rn(vu[j], sa[mt]), scu[j]);
        }
        const f32x4 gg = unpack_bf16x4(pack_bf16x4(vg));
        const f32x4 up = unpack_bf16x4(pack_bf16x4(vu));
        f32x4 act;
#pragma unroll
        for (int j = 0; j < 4; ++j) act[j] = a.act == 0 ? silu_f(gg[j]) : gelu_tanh_f(gg[j]);
        act = unpack_bf16x4(pack_bf16x4(act));
        *(i32x2*)(a.y + (size_t)m * a.ldy + col) = pack_bf16x4(act * up);
      }
    }
  }
}

// One block per row.  MODE 0: sa = amax / 448 (fp32), a8 = RNE(x / sa) from fp32 -- one rounding.
// MODE 1: the arithmetic of a torch expression on bf16 tensors, `s = x.abs().max() / 448` (a bf16 value) and
// `(x / s).to(float8_e4m3fn)` (quotient rounded to bf16, then to fp8): sa = float(bf16(amax / 448)).
// Second launch of a K-split plain W8A8 GEMM (GemmArgs::split_reduce): thread (block tile, wave, tile, lane) sums its
// four register groups over the splits in split order -- the order and arithmetic of the last-arriving block of the
// one-launch form, so the same bits -- and finishes them like the scattered epilogue above, on every CU.
template <int MT>
__global__ __launch_bounds__(256) void w8a8_split_reduce_kernel(GemmArgs a, int nblk_m, int nthreads) {
  constexpr int TILES = MT * NT;
  const int gid = blockIdx.x * 256 + threadIdx.x;
  if (gid >= nthreads) return;
  const int lane = gid & 63, half = lane >> 5, l32 = lane & 31;
  const int t = (gid >> 6) % TILES;
  const int wave = (gid >> 6) / TILES % NW;
  const int blk_lin = (gid >> 6) / (TILES * NW);
  const int mblock = blk_lin % nblk_m, nblk = blk_lin / nblk_m;
  const int mt = t / NT, nt = t % NT;
  const int strip = nblk * NW + wave;
  const f32x4* src = (const f32x4*)a.partial + (size_t)blk_lin * a.ksplit * (NW * TILES * 4 * 64) + (size_t)wave * TILES * 4 * 64 + (size_t)t * 4 * 64 + lane;
  f32x4 sum[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) sum[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int s = 0; s < a.ksplit; ++s) {
    f32x4 p[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) p[g] = src[(size_t)s * (NW * TILES * 4 * 64) + g * 64];
#pragma unroll
    for (int g = 0; g < 4; ++g) sum[g] += p[g];
  }
  const int m = (mblock * MT + mt) * 32 + l32;
  if (m >= a.M) return;
  const float sa = a.row_scale[m];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int n0 = (strip * NT + nt) * 32 + 8 * g + 4 * half;
    if (n0 >= a.N) continue;
    const f32x4 sc = *(const f32x4*)(a.s0 + n0);
    f32x4 v = sum[g];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = mul_rn(mul_rn(v[j], sa), sc[j]);
    i32x2 r = pack_bf16x4(v);
    if (a.resid) {
      const f32x4 rv = a.resid_f32 ? *(const f32x4*)((const float*)a.resid + (size_t)m * a.ldr + n0)
                                   : unpack_bf16x4(*(const i32x2*)((const u16*)a.resid + (size_t)m * a.ldr + n0));
      r = pack_bf16x4(unpack_bf16x4(r) + rv);
    }
    *(i32x2*)(a.y + (size_t)m * a.ldy + n0) = r;
  }
}

constexpr int kQuantMaxPieces = 8;  // 16-byte pieces of a row per thread: K <= 8 * 256 * 8 = 16384
__global__ __launch_bounds__(256) void quant_act_rows_kernel(QuantActArgs a) {
  __shared__ float part[4];
  const int tid = threadIdx.x;
  const char* row = (const char*)a.x + (size_t)blockIdx.x * a.ldx * 2;
  const int pieces = a.K / 8;
  i32x4 v[kQuantMaxPieces];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < kQuantMaxPieces; ++i) {
    const int p = tid + i * 256;
    v[i] = i32x4{0, 0, 0, 0};
    if (p < pieces) v[i] = *(const i32x4*)(row + (size_t)p * 16);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const unsigned u = (unsigned)v[i][e];
      amax = fmaxf(amax, fmaxf(fabsf(__uint_as_float(u << 16)), fabsf(__uint_as_float(u & 0xffff0000u))));
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  if ((tid & 63) == 0) part[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
  float sa = amax / 448.0f;
  if (a.mode == 1) sa = round_bf16(sa);
  if (tid == 0) a.sa[blockIdx.x] = sa;
  unsigned char* dst = (unsigned char*)a.a8 + (size_t)blockIdx.x * a.lda;
#pragma unroll
  for (int i = 0; i < kQuantMaxPieces; ++i) {
    const int p = tid + i * 256;
    if (p >= pieces) continue;
    float q[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const unsigned u = (unsigned)v[i][e];
      q[2 * e] = __uint_as_float(u << 16);
      q[2 * e + 1] = __uint_as_float(u & 0xffff0000u);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float y = amax == 0.f ? 0.f : q[e] / sa;  // IEEE division, as the elementwise reference computes it
      if (a.mode == 1) y = round_bf16(y);
      q[e] = y;
    }
    // four fp32 -> four e4m3fn (RNE, saturating at +-448) per conversion pair
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], hi, true);
    *(i32x2*)(dst + (size_t)p * 8) = i32x2{lo, hi};
  }
}

}  // namespace

int tk_w8a8_cols() { return NW * NT * 32; }
int tk_quant_act_max_k() { return kQuantMaxPieces * 256 * 8; }

// a.mtiles: 32-row tiles per block, 2 or 4
int tk_launch_w8a8_gemm(GemmArgs a, hipStream_t st) {
  if (a.mtiles != 2 && a.mtiles != 4) return -1;
  const int nblk_m = (a.M + a.mtiles * 32 - 1) / (a.mtiles * 32);
  const int nblk_n = (a.ntiles + NW * NT - 1) / (NW * NT);
  const int ngroups = nblk_n * a.ksplit;
  const dim3 grid((unsigned)((ngroups + 7) / 8) * 8u * (unsigned)nblk_m), block(NW * 64);
  a.split_reduce = a.ksplit > 1 && !a.s1;  // partials out, then a reduction launch over all CUs
  if (a.s1) {
    if (a.mtiles == 4)
      hipLaunchKernelGGL((w8a8_wide_kernel<1, 4, 1>), grid, block, 0, st, a, nblk_m, ngroups);
    else
      hipLaunchKernelGGL((w8a8_wide_kernel<1, 2, 2>), grid, block, 0, st, a, nblk_m, ngroups);
  } else {
    if (a.mtiles == 4)
      hipLaunchKernelGGL((w8a8_wide_kernel<0, 4, 1>), grid, block, 0, st, a, nblk_m, ngroups);
    else
      hipLaunchKernelGGL((w8a8_wide_kernel<0, 2, 2>), grid, block, 0, st, a, nblk_m, ngroups);
  }
  if (a.split_reduce) {
    const int nthreads = nblk_n * nblk_m * NW * a.mtiles * NT * 64;
    if (a.mtiles == 4) hipLaunchKernelGGL((w8a8_split_reduce_kernel<4>), dim3((nthreads + 255) / 256), dim3(256), 0, st, a, nblk_m, nthreads);
    else hipLaunchKernelGGL((w8a8_split_reduce_kernel<2>), dim3((nthreads + 255) / 256), dim3(256), 0, st, a, nblk_m, nthreads);
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

int tk_launch_quant_act_rows(QuantActArgs a, hipStream_t st) {
  hipLaunchKernelGGL(quant_act_rows_kernel, dim3(a.M), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
