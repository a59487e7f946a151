// fp8-weight GEMM for skinny M on gfx950:  y[M,N] = bf16((x[M,K] . W8[N,K]^T) * scale[n]).
//
// Memory-bound (weight streaming), so the layout is built around the weight read:
//   * W8 is pre-packed into 32(n) x 32(k)-byte tiles in MFMA B-operand lane order; a wave reads a
//     tile with ONE coalesced 1 KiB global_load_dwordx4 straight into operand registers.
//   * e4m3 -> bf16 is exact and done in registers (v_cvt_scalef32_pk_bf16_fp8, scale 1.0), the
//     product runs on v_mfma_f32_32x32x16_bf16 with fp32 accumulation.
//   * A block owns NT n-tiles x MT m-tiles and a contiguous range of k-tiles; per round its NW
//     waves take NW*TPW consecutive k-tiles (TPW each).  The activations of a round
//     (MT*32 rows x NW*TPW*32 columns, bf16) are staged ONCE per block through LDS with fully
//     coalesced 16-byte loads (whole 128-byte lines per row) and read back in A-operand order:
//     reading them per lane from global memory costs one cache-line lookup per row and
//     instruction and caps a CU at a fraction of its L1 fill rate.
//   * Columns past the block's K range (K tail, next split) are zeroed in LDS, so the weight
//     loads need no masking: a zero activation column cancels whatever tile was read.
//   * Reductions are fixed-order: waves through LDS (w = 0..NW-1), K splits through an fp32
//     partial buffer summed by the last-arriving block in split order (no float atomics).
#include <type_traits>

#include "tk_common.h"
#include "tk_kernels.h"


#ifdef TK_PHASE_TIMING
// development aid (never built into the shipped library): per-block phase timestamps of the single-launch FFN,
// 10 ns units; [half][block][slot]
__device__ long long tk_phase_stamps[2 * 1024 * 8];
extern "C" int tk_debug_read_phases(void* host_out) {
  return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(tk_phase_stamps), sizeof(long long) * 2 * 1024 * 8);
}
#define TK_MARK(i)                                                                                                \
  do {                                                                                                            \
    if (FUSE != 0 && threadIdx.x == 0 && blockIdx.x < 1024) tk_phase_stamps[((FUSE - 1) * 1024 + blockIdx.x) * 8 + (i)] = wall_clock64(); \
  } while (0)
#else
#define TK_MARK(i)
#endif

namespace {

// LDS-only barrier: waits for this wave's LDS traffic, not for the global prefetch queue
// (a full __syncthreads() would drain vmcnt and serialise the weight stream every round).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// EPI: 0 plain (scale, optional per-column gate, optional residual), 1 gated (gate/up tile pairs ->
//      act(g)*u), 2 rope (tile pairs hold columns (i, i + D/2) of one head -> rotary embedding).
// W16: weights are bf16 (two 16-byte operand chunks per lane and k tile) instead of e4m3.
// PRO: 0 none, 1 RMSNorm of bf16 activations, 2 RMSNorm of fp32 activations, 3 adaptive RMSNorm of
//      bf16 activations: bf16((x * rstd) * (1 + scale[k]) + shift[k]) in fp32 -- applied while the
//      activations are staged into LDS, with the reference's rounding points:
//      bf16 input: bf16(w * bf16(x * rstd));  fp32 input: bf16(w * (x * rstd)).
//  NR: number of block rounds when the host knows it (every block walks the same number of k tiles), else 0:
//      with a constant count the pipeline below is straight-line code -- no tail conditions, exact wait counts.
// FUSE: 0 a launch of its own.  1 / 2: the two halves of the single-launch gated FFN -- 1 is a gate/up block, which
//      writes its 32 x 32 slice of the intermediate through to memory and raises its flag; 2 is a down block, which
//      requests its first weight rounds, THEN waits (bounded) for the flags of the gate/up strips its k range
//      covers, and reads their slices.  The intermediate is kept tile by tile -- slice (row block, strip) is 2 KiB
//      of its own, [32 rows][32 columns] -- so every 128-byte line of it has ONE writer: a down block's plain loads
//      then either miss in their L2 (nobody there touched the line since the launch began) and fetch what was
//      written through, or hit the copy the writer's own write-through stores left in the same L2.
// (strip, split, mblock): the block's position; nstrips: strips per row block (the arrival counters' pitch).
template <int MT, int NT, int NW, int EPI, int PF, int TPW, bool W16, int PRO, int NR, int FUSE>
__device__ __forceinline__ void gemm_block(const GemmArgs& a, const int strip, const int split, const int mblock, const int nstrips) {
  constexpr bool GATED = EPI == 1;
  // every round of the block in flight from the start (PF == NR) with the bf16 RMSNorm prologue (plain or adaptive):
  // the staged pieces stay in registers until the row statistics are known, so the statistics come from them -- no
  // second pass over the rows.  The host picks this only when a block walks the whole K (no K split).
  constexpr bool FULL = (PRO == 1 || PRO == 3) && NR > 0 && PF == NR;
  constexpr bool PAIRED = EPI != 0;  // both n tiles of a pair are finished by the same wave
  constexpr bool XF32 = PRO == 2;
  constexpr int TILES = MT * NT;
  constexpr int RKT = NW * TPW;               // k tiles per block round
  constexpr int ROWB = RKT * 64;              // bytes of one staged (bf16) activation row per round
  constexpr int PITCH = ROWB + 16;            // LDS row pitch (bytes), keeps 16-byte alignment
  constexpr int ROWS = MT * 32;
  constexpr int XBUF = ROWS * PITCH;          // bytes per staging buffer
  constexpr int PPR = ROWB / 16;              // 8-element pieces per row
  constexpr int XPT = ROWS * PPR / (NW * 64); // pieces per thread and round
  constexpr int RW = 4;                       // waves that reduce and finish (one per register group)
  constexpr int RED_BYTES = TILES * RW * 16 * 64 * 4;  // four waves' partial tiles at once
  constexpr int LDS_BYTES = 2 * XBUF > RED_BYTES ? 2 * XBUF : RED_BYTES;
  constexpr int WCH = W16 ? 2 : 1;            // 16-byte operand chunks per lane, n tile and k tile
  constexpr int WTILE = W16 ? 2048 : 1024;    // bytes of one packed 32x32 tile
  static_assert(ROWS * PPR % (NW * 64) == 0, "staging pieces must divide evenly");
  static_assert(!PAIRED || NT == 2, "paired epilogues need two n tiles per strip");
  __shared__ __align__(16) unsigned char lds[LDS_BYTES];
  __shared__ float rstd_s[ROWS];

  TK_MARK(0);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps k-tile indices scalar
  const int half = lane >> 5;
  const int l32 = lane & 31;
  // k tiles of this split: KT = ksplit * kt_q + kt_r, the first kt_r splits take one more (host-side
  // division: a 64-bit divide here costs some 300 scalar instructions before the first load)
  const int kt_lo = split * a.kt_q + (split < a.kt_r ? split : a.kt_r);
  const int kt_hi = kt_lo + a.kt_q + (split < a.kt_r ? 1 : 0);
  const int nrounds = NR > 0 ? NR : (kt_hi - kt_lo + RKT - 1) / RKT;
  const int k_end = kt_hi * 32 < a.K ? kt_hi * 32 : a.K;  // first activation column this block must not use

  // weight tile streams of this wave; a strip may hang over the last n tile: clamp to a valid
  // tile (its results are never stored) so every load is unconditional.
  const uint8_t* wbase[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int ntg = strip * NT + nt;
    if (ntg > a.ntiles - 1) ntg = a.ntiles - 1;
    wbase[nt] = a.w + ((size_t)ntg * a.KT) * WTILE + lane * 16;
  }

  // staging pieces of this thread: piece p -> (row p / PPR, 8-element column p % PPR).  Rows >= M
  // are clamped to M-1 (an output row depends only on its own activation row; rows >= M are
  // never stored).
  const char* xsrc[XPT];
  int xcol[XPT];   // first element (k index) of the piece within a round
  int xdst[XPT];   // LDS byte offset within a staging buffer
  int xrow[XPT];
#pragma unroll
  for (int i = 0; i < XPT; ++i) {
    const int p = tid + i * NW * 64;
    // FUSE == 2: consecutive threads walk a 2 KiB slice (k tile, row, 16-byte piece): whole lines per request
    const int r = FUSE == 2 ? (p % 128) / 4 : p / PPR, c = FUSE == 2 ? (p / 128) * 4 + p % 4 : p % PPR;
    int m = mblock * ROWS + r;
    if (m > a.M - 1) m = a.M - 1;
    if (FUSE == 2)
      xsrc[i] = (const char*)a.x + (((size_t)mblock * a.KT + kt_lo + c / 4) * 32 + r) * 64 + (c % 4) * 16;
    else
      xsrc[i] = (const char*)a.x + (size_t)m * a.ldx * (XF32 ? 4 : 2);
    xcol[i] = c * 8;
    xdst[i] = r * PITCH + c * 16;
    xrow[i] = r;
  }

  // rotary epilogue: the positions of this lane's rows, requested before anything else -- the table rows they
  // select are requested after the k loop, and would otherwise wait a second round trip for them there
  int rpos[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = (mblock * MT + mt) * 32 + l32;
    if (m > a.M - 1) m = a.M - 1;
    rpos[mt] = EPI == 2 ? a.rope_pos[m] : 0;
  }

  f32x16 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;

  struct WFrag {
    i32x4 w[TPW][NT][WCH];
  };
  auto wload = [&](WFrag& f, int r) {
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      int kt = kt_lo + r * RKT + wave * TPW + j;
      if (kt > a.KT - 1) kt = a.KT - 1;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int c = 0; c < WCH; ++c) f.w[j][nt][c] = *(const i32x4*)(wbase[nt] + (size_t)kt * WTILE + c * 1024);
    }
  };
  constexpr bool ADA = PRO == 3;
  // a thread's pieces of a round are the same 8 columns of XPT different rows (the block's threads are a multiple
  // of the pieces per row), so the norm weights of those columns are held once
  static_assert((NW * 64) % PPR == 0, "a thread's pieces share their columns");
  struct XFrag {
    i32x4 v[XPT][XF32 ? 2 : 1];
    i32x4 nw[ADA ? 4 : 1];  // norm weights of the pieces' 8 columns (ADA: fp32 scale, shift)
  };
  auto xload = [&](XFrag& f, int r) {
    const int k0 = (kt_lo + r * RKT) * 32;
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
      int k = k0 + xcol[i];
      if (k > a.K - 8) k = a.K - 8;  // keep the address inside the row; the value is dropped below
      if (XF32) {
        const i32x4* p = (const i32x4*)(xsrc[i] + (size_t)k * 4);
        f.v[i][0] = p[0];
        f.v[i][XF32 ? 1 : 0] = p[1];
      } else if (FUSE == 2) {
        f.v[i][0] = *(const i32x4*)(xsrc[i] + (size_t)r * (RKT * 2048));  // round r: RKT slices on
      } else {
        f.v[i][0] = *(const i32x4*)(xsrc[i] + (size_t)k * 2);
      }
      if (i == 0) {
        if (ADA) {
          f.nw[0] = *(const i32x4*)(a.ada_scale + k);
          f.nw[ADA ? 1 : 0] = *(const i32x4*)(a.ada_scale + k + 4);
          f.nw[ADA ? 2 : 0] = *(const i32x4*)(a.ada_shift + k);
          f.nw[ADA ? 3 : 0] = *(const i32x4*)(a.ada_shift + k + 4);
        } else if (PRO) {
          f.nw[0] = *(const i32x4*)(a.norm_w + k);
        }
      }
    }
  };
  float my_rstd[XPT];
#pragma unroll
  for (int i = 0; i < XPT; ++i) my_rstd[i] = 1.f;
  // MASKED: zero the columns past the block's k range.  Only a block's LAST round can reach past it (the
  // rounds before cover whole k tiles below kt_hi, and only the last k tile of the matrix is partial), so
  // every other round stages without the per-element selects -- they sit on each round's critical path.
  auto xstore = [&](const XFrag& f, int r, int b, auto masked_c) {
    constexpr bool MASKED = decltype(masked_c)::value;
    const int k0 = (kt_lo + r * RKT) * 32;
    const i32x4 z = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
      const bool ok = !MASKED || (k0 + xcol[i]) < k_end;
      i32x4 out;
      if (PRO == 0) {
        out = f.v[i][0];
      } else if (ADA) {
        union { i32x4 v; unsigned u[4]; } xu, o;
        union { i32x4 v[2]; float f[8]; } sc, sh;
        xu.v = f.v[i][0];
        sc.v[0] = f.nw[0];
        sc.v[1] = f.nw[ADA ? 1 : 0];
        sh.v[0] = f.nw[ADA ? 2 : 0];
        sh.v[1] = f.nw[ADA ? 3 : 0];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // separately rounded fp32 operations, as the elementwise reference computes them
          const float x0 = __uint_as_float(xu.u[e] << 16), x1 = __uint_as_float(xu.u[e] & 0xffff0000u);
          const float y0 = add_rn(mul_rn(mul_rn(x0, my_rstd[i]), add_rn(1.0f, sc.f[2 * e])), sh.f[2 * e]);
          const float y1 = add_rn(mul_rn(mul_rn(x1, my_rstd[i]), add_rn(1.0f, sc.f[2 * e + 1])), sh.f[2 * e + 1]);
          o.u[e] = pack_bf16x2(y0, y1);
        }
        out = o.v;
      } else {
        union { i32x4 v; unsigned u[4]; } nwu, o;
        nwu.v = f.nw[0];
        float xv[8];
        if (XF32) {
          union { i32x4 v; float f[4]; } lo, hi;
          lo.v = f.v[i][0];
          hi.v = f.v[i][XF32 ? 1 : 0];
#pragma unroll
          for (int e = 0; e < 4; ++e) { xv[e] = lo.f[e]; xv[4 + e] = hi.f[e]; }
        } else {
          union { i32x4 v; unsigned u[4]; } xu;
          xu.v = f.v[i][0];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            xv[2 * e] = __uint_as_float(xu.u[e] << 16);
            xv[2 * e + 1] = __uint_as_float(xu.u[e] & 0xffff0000u);
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float n0 = xv[2 * e] * my_rstd[i], n1 = xv[2 * e + 1] * my_rstd[i];
          if (!XF32) {  // a bf16 input is normalised back to bf16 before the weight multiply
            const unsigned u = pack_bf16x2(n0, n1);
            n0 = __uint_as_float(u << 16);
            n1 = __uint_as_float(u & 0xffff0000u);
          }
          o.u[e] = pack_bf16x2(__uint_as_float(nwu.u[e] << 16) * n0, __uint_as_float(nwu.u[e] & 0xffff0000u) * n1);
        }
        out = o.v;
      }
      *(i32x4*)(lds + b * XBUF + xdst[i]) = ok ? out : z;
    }
  };
  auto compute = [&](const WFrag& f, int b) {
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      i32x4 xa[MT][2];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const i32x4* p = (const i32x4*)(lds + b * XBUF + (mt * 32 + l32) * PITCH + ((wave * TPW + j) * 32 + 16 * half) * 2);
        xa[mt][0] = p[0];
        xa[mt][1] = p[1];
      }
      bf16x8 wb[NT][2];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        if (W16) {
          wb[nt][0] = as_bf16x8(f.w[j][nt][0]);
          wb[nt][1] = as_bf16x8(f.w[j][nt][W16 ? 1 : 0]);
        } else {
          wb[nt][0] = fp8x8_to_bf16x8(f.w[j][nt][0][0], f.w[j][nt][0][1]);
          wb[nt][1] = fp8x8_to_bf16x8(f.w[j][nt][0][2], f.w[j][nt][0][3]);
        }
      }
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[nt][h2], as_bf16x8(xa[mt][h2]), acc[mt][nt], 0, 0, 0);
    }
  };

  // Software pipeline over block rounds: PF rounds in flight.  A round's activations and weights
  // are requested together (memory returns in order, so waiting for one means waiting for
  // everything requested before it).  The steady-state loop runs while a whole group of PF rounds
  // can prefetch and has no branch, so the compiler keeps precise vmcnt waits; the tail (at most
  // 2*PF-1 rounds) uses block-uniform conditions and requests nothing that is not consumed.
  WFrag wbuf[PF];
  XFrag xbuf[PF];
  // (unconditional even when the block has fewer than PF rounds -- the addresses are clamped to
  // valid tiles: a branch here would make the compiler's wait-count analysis assume, at the head
  // of the steady-state loop, that the first stage's loads might be the youngest in flight, and
  // drain the whole queue once per pass)
  int fuse_ticket = -1;
  if (FUSE == 2) {
    static_assert(FUSE != 2 || (PRO == 0 && MT == 1), "the down half reads a finished intermediate, 32 rows of it");
    // the weights do not depend on the other half: on their way before the wait
#pragma unroll
    for (int p = 0; p < PF; ++p) wload(wbuf[p], p);
    if (wave == 0) {
      // lanes poll the flags of the strips [kt_lo, kt_hi) -- the slices this block's k range reads
      const int* flags = a.fuse + mblock * TK_FUSE_STRIPS;
      bool ready = false;
      for (int n = 0;; ++n) {
        bool mine = true;
        for (int sidx = kt_lo + lane; sidx < kt_hi; sidx += 64)
          mine = mine && __hip_atomic_load(flags + sidx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
        ready = __builtin_amdgcn_ballot_w64(!mine) == 0;
        if (ready || n >= a.fuse_spin) break;
        __builtin_amdgcn_s_sleep(2);
      }
      if (!ready && lane == 0)  // gave up: say so (this launch's output is then undefined) and go on, so that the grid drains
        __hip_atomic_store(a.fuse + TK_FUSE_ERROR, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    handoff_acquire();
    TK_MARK(1);
#pragma unroll
    for (int p = 0; p < PF; ++p) xload(xbuf[p], p);
    // count this block past its wait (behind the loads above: memory returns in order); the answer is looked at
    // after the k loop
    if (tid == 0) fuse_ticket = __hip_atomic_fetch_add(a.fuse + TK_FUSE_PAST + mblock, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    TK_MARK(2);
  } else if (FULL) {
    // the activations first: memory returns in order, and the statistics below need every piece of the rows
#pragma unroll
    for (int p = 0; p < PF; ++p) xload(xbuf[p], p);
#pragma unroll
    for (int p = 0; p < PF; ++p) wload(wbuf[p], p);
  } else {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      xload(xbuf[p], p);
      wload(wbuf[p], p);
    }
  }
  if (FULL) {
    // piece i of every round belongs to row xrow[i]; the PPR threads that share a row are consecutive lanes
    static_assert(!FULL || ((PPR == 16 || PPR == 32) && !XF32), "the row's pieces sit in PPR consecutive lanes");
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
      float ss0 = 0.f, ss1 = 0.f;
#pragma unroll
      for (int p = 0; p < PF; ++p) {
        if (p * RKT * 32 + xcol[i] < a.K) {  // pieces past K hold a repeated piece of the row
          union { i32x4 v; bf16x2 h[4]; } xu;
          xu.v = xbuf[p].v[i][0];
          ss0 = __builtin_amdgcn_fdot2_f32_bf16(xu.h[0], xu.h[0], ss0, false);
          ss1 = __builtin_amdgcn_fdot2_f32_bf16(xu.h[1], xu.h[1], ss1, false);
          ss0 = __builtin_amdgcn_fdot2_f32_bf16(xu.h[2], xu.h[2], ss0, false);
          ss1 = __builtin_amdgcn_fdot2_f32_bf16(xu.h[3], xu.h[3], ss1, false);
        }
      }
      float ss = ss0 + ss1;
#pragma unroll
      for (int o = PPR / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
      my_rstd[i] = rsqrtf(ss / (float)a.K + a.norm_eps);
    }
  } else if (PRO) {
    // per-row 1/rms over the whole K (every block needs it for its rows, whatever its k range)
    constexpr int TPR = NW * 64 / ROWS;  // threads per row
    const int r = tid / TPR, q = tid % TPR;
    const int m = mblock * ROWS + r;
    const char* row = (const char*)a.x + (size_t)(m < a.M ? m : 0) * a.ldx * (XF32 ? 4 : 2);
    const int npieces = m < a.M ? a.K / 8 : 0;  // rows past M are never stored: skip their reads
    float ss0 = 0.f, ss1 = 0.f;
#pragma unroll 8
    for (int p = q; p < npieces; p += TPR) {
      if (XF32) {
        const f32x4* p4 = (const f32x4*)(row + (size_t)p * 32);
        const f32x4 u0 = p4[0], u1 = p4[1];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          ss0 = fmaf(u0[e], u0[e], ss0);
          ss1 = fmaf(u1[e], u1[e], ss1);
        }
      } else {
        union { i32x4 v; bf16x2 h[4]; } xu;
        xu.v = *(const i32x4*)(row + (size_t)p * 16);
        ss0 = __builtin_amdgcn_fdot2_f32_bf16(xu.h[0], xu.h[0], ss0, false);
        ss1 = __builtin_amdgcn_fdot2_f32_bf16(xu.h[1], xu.h[1], ss1, false);
        ss0 = __builtin_amdgcn_fdot2_f32_bf16(xu.h[2], xu.h[2], ss0, false);
        ss1 = __builtin_amdgcn_fdot2_f32_bf16(xu.h[3], xu.h[3], ss1, false);
      }
    }
    float ss = ss0 + ss1;
#pragma unroll
    for (int o = TPR / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    if (q == 0) rstd_s[r] = rsqrtf(ss / (float)a.K + a.norm_eps);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < XPT; ++i) my_rstd[i] = rstd_s[xrow[i]];
  }
  if (nrounds > 0) {
    int it = 0;
    for (; it + 2 * PF <= nrounds; it += PF) {
#pragma unroll
      for (int p = 0; p < PF; ++p) {
        const int r = it + p;
        xstore(xbuf[p], r, r & 1, std::false_type{});
        lds_barrier();
        compute(wbuf[p], r & 1);
        xload(xbuf[p], r + PF);
        wload(wbuf[p], r + PF);
        __builtin_amdgcn_sched_barrier(0);  // keep the refill right behind its stage's MFMAs
      }
    }
    const int rem = nrounds - it;  // in [0, 2*PF)
#pragma unroll
    for (int q = 0; q < 2 * PF - 1; ++q) {
      if (q < rem) {  // block-uniform
        const int r = it + q;
        if (q == rem - 1) xstore(xbuf[q % PF], r, r & 1, std::true_type{});  // block-uniform
        else xstore(xbuf[q % PF], r, r & 1, std::false_type{});
        lds_barrier();
        compute(wbuf[q % PF], r & 1);
        if (q + PF < rem) {
          xload(xbuf[q % PF], r + PF);
          wload(wbuf[q % PF], r + PF);
        }
      }
    }
  }
  TK_MARK(3);
  if (FUSE == 2 && wave == 0) {
    // the last down block of the row block to get past its wait leaves the flags and the count ready for the next launch
    if (__builtin_amdgcn_readfirstlane(fuse_ticket) == a.fuse_consumers - 1) {
      for (int sidx = lane; sidx < a.KT; sidx += 64)
        __hip_atomic_store(a.fuse + mblock * TK_FUSE_STRIPS + sidx, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (lane == 0) __hip_atomic_store(a.fuse + TK_FUSE_PAST + mblock, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __syncthreads();  // staging buffers are dead; the reduction reuses the LDS

  // The accumulators hold C^T tiles: lane l of a tile owns activation row m = l % 32 and, in
  // register i, output column n = 8*(i/4) + 4*(l/32) + i%4 -- register group g = i/4 is four
  // consecutive columns.  From here on wave w owns group g = w of EVERY tile: all four waves take
  // part in the reductions and in the epilogue, and everything moves as 8- or 16-byte vectors.
  static_assert(NW == 4 || NW == 8, "one wave per register group, or two");
  if (NW == 8) {
    // eight waves walked the k tiles: waves 4..7 hand their accumulators to waves 0..3 (w + 4 -> w) and leave
    f32x4 (*fold)[RW][4][64] = (f32x4 (*)[RW][4][64])lds;  // [tile][wave - 4][group][lane]
    if (wave >= RW) {
#pragma unroll
      for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          fold[t][wave - RW][g][lane] = f32x4{acc[t / NT][t % NT][4 * g], acc[t / NT][t % NT][4 * g + 1], acc[t / NT][t % NT][4 * g + 2],
                                              acc[t / NT][t % NT][4 * g + 3]};
    }
    __syncthreads();
    if (wave >= RW) return;
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 v = fold[t][wave][g][lane];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[t / NT][t % NT][4 * g + j] += v[j];
      }
    __syncthreads();  // (the four remaining waves) the exchange below reuses the space
  }
  const int ng = wave * 8 + half * 4;  // first of this lane's four columns within an n tile

  // ---- epilogue operands: requested now, consumed after the reductions ----
  f32x4 e_sc[NT];     // EPI 0: column scales; EPI 1: e_sc[0] gate scale, e_sc[1] up scale
  f32x4 e_rv[TILES];  // EPI 0: residual values; EPI 2: [2*mt] cos, [2*mt+1] sin of this lane's row
  i32x2 e_gate[NT];   // EPI 0: per-column gate (bf16 x4)
  if (EPI == 0) {
    if (a.vec) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        int n0 = (strip * NT + nt) * 32 + ng;
        if (n0 > a.N - 4) n0 = a.N - 4;  // columns past N are never stored
        if (!W16) e_sc[nt] = *(const f32x4*)(a.s0 + n0);
        if (a.gate) e_gate[nt] = *(const i32x2*)(a.gate + n0);
        if (a.resid) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            int m = (mblock * MT + mt) * 32 + l32;
            if (m > a.M - 1) m = a.M - 1;
            e_rv[mt * NT + nt] = a.resid_f32 ? *(const f32x4*)((const float*)a.resid + (size_t)m * a.ldr + n0)
                                             : unpack_bf16x4(*(const i32x2*)((const u16*)a.resid + (size_t)m * a.ldr + n0));
          }
        }
      }
    }
  } else if (EPI == 1) {
    int col = strip * 32 + ng;
    if (col > a.N - 4) col = a.N - 4;
    e_sc[0] = *(const f32x4*)(a.s0 + col);
    e_sc[NT - 1] = *(const f32x4*)(a.s1 + col);
  } else {
    const int po = a.rope_half >> 5;
    const int fi = (((strip / po) * 2 * po + strip % po) * 32 + ng) % (2 * a.rope_half);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      int m = (mblock * MT + mt) * 32 + l32;
      if (m > a.M - 1) m = a.M - 1;
      int pos = rpos[mt];
      pos = pos < 0 ? 0 : (pos > a.rope_positions - 1 ? a.rope_positions - 1 : pos);
      e_rv[2 * mt] = *(const f32x4*)(a.rope_cos + (size_t)pos * a.rope_half + fi);
      e_rv[2 * mt + 1] = *(const f32x4*)(a.rope_sin + (size_t)pos * a.rope_half + fi);
    }
  }

  // ---- in-block reduction over waves (fixed order w = 0..3): one exchange for all tiles ----
  f32x4 (*red)[RW][4][64] = (f32x4 (*)[RW][4][64])lds;  // [tile][wave][group][lane]
  f32x4 own[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    const int mt = t / NT, nt = t % NT;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x4 v = {acc[mt][nt][4 * g], acc[mt][nt][4 * g + 1], acc[mt][nt][4 * g + 2], acc[mt][nt][4 * g + 3]};
      red[t][wave][g][lane] = v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    f32x4 sum = red[t][0][wave][lane];
#pragma unroll
    for (int w = 1; w < RW; ++w) sum += red[t][w][wave][lane];
    own[t] = sum;
  }

  // ---- K-split reduction through global partials, wave by wave: wave w of every split block leaves register
  // group w of its tiles and counts itself in on counter (block, w); the wave that arrives last for a group sums
  // that group in split order and finishes it.  No block barrier in the chain: a wave's store acknowledgement,
  // count and read-back overlap with the other waves'. ----
  const int blk_lin = mblock * nstrips + strip;
  if (a.ksplit > 1) {
    // partial layout: [(block, split)][tile][group][lane][4 floats], written and read as 8-byte
    // device-coherent accesses (write-through, so the hand-off needs no cache flush)
    unsigned long long* pbase = (unsigned long long*)a.partial + ((size_t)wave * 64 + lane) * 2;
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      unsigned long long* dst = pbase + (((size_t)blk_lin * a.ksplit + split) * TILES + t) * 512;
      st_agent64(dst, own[t][0], own[t][1]);
      st_agent64(dst + 1, own[t][2], own[t][3]);
    }
    // wait until this wave's partials are acknowledged, then count it in
    handoff_publish();
    int* counter = a.counters + (size_t)(blk_lin * RW + wave) * a.cstride;
    int old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (__builtin_amdgcn_readfirstlane(old) != a.ksplit - 1) return;  // wave-uniform
    handoff_acquire();
    if (lane == 0)  // leave the counter ready for the next launch
      __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int t = 0; t < TILES; ++t) own[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    // sum in split order; four splits' loads are in flight together
    constexpr int SB = 4;
    for (int s0 = 0; s0 < a.ksplit; s0 += SB) {
      unsigned long long raw[SB][TILES][2];
#pragma unroll
      for (int j = 0; j < SB; ++j) {
        const int sj = s0 + j < a.ksplit ? s0 + j : a.ksplit - 1;
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          const unsigned long long* src = pbase + (((size_t)blk_lin * a.ksplit + sj) * TILES + t) * 512;
          raw[j][t][0] = ld_agent64(src);
          raw[j][t][1] = ld_agent64(src + 1);
        }
      }
#pragma unroll
      for (int j = 0; j < SB; ++j) {
        if (s0 + j < a.ksplit) {
#pragma unroll
          for (int t = 0; t < TILES; ++t) {
            own[t][0] += __uint_as_float((unsigned)raw[j][t][0]);
            own[t][1] += __uint_as_float((unsigned)(raw[j][t][0] >> 32));
            own[t][2] += __uint_as_float((unsigned)raw[j][t][1]);
            own[t][3] += __uint_as_float((unsigned)(raw[j][t][1] >> 32));
          }
        }
      }
    }
  }

  TK_MARK(6);
  // ---- epilogue: this lane finishes row m (per m tile), columns n0 .. n0+3 of each n tile ----
  if (EPI == 0) {
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const int mt = t / NT, nt = t % NT;
      const int m = (mblock * MT + mt) * 32 + l32;
      const int n0 = (strip * NT + nt) * 32 + ng;
      if (m >= a.M || n0 >= a.N) continue;
      if (a.vec) {  // N % 4 == 0 and every row pitch / pointer allows 8-byte accesses
        f32x4 v = own[t];
        if (!W16) v *= e_sc[nt];
        i32x2 r = pack_bf16x4(v);
        if (a.gate) r = pack_bf16x4(unpack_bf16x4(r) * unpack_bf16x4(e_gate[nt]));
        if (a.resid) r = pack_bf16x4(unpack_bf16x4(r) + e_rv[t]);
        *(i32x2*)(a.y + (size_t)m * a.ldy + n0) = r;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = n0 + j;
          if (n >= a.N) continue;
          u16 r = f32_to_bf16_bits(own[t][j] * (W16 ? 1.0f : a.s0[n]));
          if (a.gate) r = f32_to_bf16_bits(bf16_bits_to_f32(r) * bf16_bits_to_f32(a.gate[n]));
          if (a.resid) {
            const float rv = a.resid_f32 ? ((const float*)a.resid)[(size_t)m * a.ldr + n]
                                         : bf16_bits_to_f32(((const u16*)a.resid)[(size_t)m * a.ldr + n]);
            r = f32_to_bf16_bits(bf16_bits_to_f32(r) + rv);
          }
          a.y[(size_t)m * a.ldy + n] = r;
        }
      }
    }
    TK_MARK(7);
  } else if (EPI == 1) {
    // tiles come in (gate, up) pairs over the same logical columns; I % 32 == 0
    const int col = strip * 32 + ng;  // logical column in [0, I)
    if (col < a.N) {
      const f32x4 scg = e_sc[0], scu = e_sc[NT - 1];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = (mblock * MT + mt) * 32 + l32;
        if (m >= a.M) continue;
        const f32x4 g = unpack_bf16x4(pack_bf16x4(own[mt * 2] * scg));
        const f32x4 up = unpack_bf16x4(pack_bf16x4(own[mt * 2 + 1] * scu));
        f32x4 act;
#pragma unroll
        for (int j = 0; j < 4; ++j) act[j] = a.act == 0 ? silu_f(g[j]) : gelu_tanh_f(g[j]);
        act = unpack_bf16x4(pack_bf16x4(act));
        const i32x2 hv = pack_bf16x4(act * up);
        if (FUSE == 1)  // slice (row block, strip), written through
          __hip_atomic_store((unsigned long long*)(a.y + (((size_t)mblock * nstrips + strip) * 32 + l32) * 32 + ng),
                             (unsigned long long)(unsigned)hv[0] | ((unsigned long long)(unsigned)hv[1] << 32), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        else
          *(i32x2*)(a.y + (size_t)m * a.ldy + col) = hv;
      }
    }
    if (FUSE == 1) {
      // this block's slice of the intermediate is written through: raise its flag
      TK_MARK(4);
      handoff_publish();
      __syncthreads();
      TK_MARK(5);
      if (threadIdx.x == 0) __hip_atomic_store(a.fuse + mblock * TK_FUSE_STRIPS + strip, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      TK_MARK(7);
    }
  } else {
    // the two tiles of a strip hold columns (c, c + rope_half) of one head: logical tile of
    // physical tile (strip, j) is (strip / PO) * 2 * PO + strip % PO + j * PO with PO = rope_half / 32
    const int po = a.rope_half >> 5;
    const int lt0 = (strip / po) * 2 * po + strip % po;
    const int ca = lt0 * 32 + ng, cb = ca + a.rope_half;
    const bool rot = ca < a.rope_cols;
    if (cb + 3 < a.N) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = (mblock * MT + mt) * 32 + l32;
        if (m >= a.M) continue;
        f32x4 va = unpack_bf16x4(pack_bf16x4(own[mt * 2]));
        f32x4 vb = unpack_bf16x4(pack_bf16x4(own[mt * 2 + 1]));
        if (rot) {
          const f32x4 cs = e_rv[2 * mt], sn = e_rv[2 * mt + 1];
          f32x4 ra, rb;
          if (a.rope_bf16) {
            // bf16 arithmetic (x * cos + rotate_half(x) * sin on bf16 tensors): every product and
            // the sum round to bf16; the tables hold bf16 values
            const f32x4 ac = unpack_bf16x4(pack_bf16x4(va * cs)), bs = unpack_bf16x4(pack_bf16x4(vb * sn));
            const f32x4 bc = unpack_bf16x4(pack_bf16x4(vb * cs)), as = unpack_bf16x4(pack_bf16x4(va * sn));
            ra = ac - bs;
            rb = bc + as;
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              // separately rounded products, as an elementwise fp32 implementation computes them
              ra[j] = sub_rn(mul_rn(va[j], cs[j]), mul_rn(vb[j], sn[j]));
              rb[j] = add_rn(mul_rn(vb[j], cs[j]), mul_rn(va[j], sn[j]));
            }
          }
          va = ra;
          vb = rb;
        }
        const i32x2 pa = pack_bf16x4(va), pbv = pack_bf16x4(vb);
        *(i32x2*)(a.y + (size_t)m * a.ldy + ca) = pa;
        *(i32x2*)(a.y + (size_t)m * a.ldy + cb) = pbv;
        if (a.vt && ca >= a.vt_col0) {  // tile-uniform: vt_col0 is a multiple of the head size
          // value columns, transposed for the attention kernel (lanes = consecutive rows m)
          u16* va_t = a.vt + (size_t)(ca - a.vt_col0) * a.vt_ld + m;
          u16* vb_t = a.vt + (size_t)(cb - a.vt_col0) * a.vt_ld + m;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            va_t[(size_t)j * a.vt_ld] = (u16)(((unsigned)pa[j >> 1]) >> (16 * (j & 1)));
            vb_t[(size_t)j * a.vt_ld] = (u16)(((unsigned)pbv[j >> 1]) >> (16 * (j & 1)));
          }
        }
      }
    }
  }
}

template <int MT, int NT, int NW, int EPI, int PF, int TPW, bool W16, int PRO, int NR = 0>
__global__ __launch_bounds__(NW * 64) void fp8w_gemm_kernel(GemmArgs a) {
  gemm_block<MT, NT, NW, EPI, PF, TPW, W16, PRO, NR, 0>(a, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.x);
}

// The gated FFN of the action chunk in ONE launch: blocks [0, nprod) are gate/up blocks (strip-major within a row
// block), the rest down blocks (strip, K split, row block).  Blocks are dispatched in index order, so every gate/up
// block is resident (or done) before a down block can wait for it; the wait is bounded all the same.
//   G*: the gate/up half's <NW, PF, PRO, NR>;  D*: the down half's <NT, NW, PF, NR>.
template <int GNW, int GPF, int GPRO, int GNR, int DNT, int DNW, int DPF, int DNR>
__global__ __launch_bounds__((GNW > DNW ? GNW : DNW) * 64) void ffn_fused_kernel(GemmArgs g, GemmArgs d, int nprod, int gstrips, int dstrips) {
  const int b = blockIdx.x;
  if (b < nprod) {
    if (GNW < DNW && threadIdx.x >= GNW * 64) return;
    gemm_block<1, 2, GNW, 1, GPF, 1, false, GPRO, GNR, 1>(g, b % gstrips, 0, b / gstrips, gstrips);
  } else {
    if (DNW < GNW && threadIdx.x >= DNW * 64) return;
    const int c = b - nprod;
    const int strip = c % dstrips, rest = c / dstrips;
    gemm_block<1, DNT, DNW, 0, DPF, 1, false, 0, DNR, 2>(d, strip, rest % d.ksplit, rest / d.ksplit, dstrips);
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

// bf16 [N, K] row-major -> 2 KiB tiles: chunk c (0/1) of lane l = 8 bf16 at k = 32*kt + 16*(l/32) + 8*c,
// stored as [c][lane] so each of the two loads of a tile is one coalesced 1 KiB read.  With
// pair_off = PO > 0, physical n tile (2p + j) holds logical n tile (p / PO) * 2 * PO + p % PO + j * PO,
// i.e. the two tiles of a strip hold columns (c, c + 32*PO) -- the rotary pairs of one head.
__global__ void pack_bf16_kernel(const unsigned short* __restrict__ w, uint8_t* __restrict__ out, int N, int K, int KT,
                                 long long nchunks, int pair_off) {
  long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= nchunks) return;
  const int lane = (int)(c & 63);
  const int ch = (int)((c >> 6) & 1);
  const long long tile = c >> 7;
  const int kt = (int)(tile % KT);
  const int ntp = (int)(tile / KT);
  int nt = ntp;
  if (pair_off > 0) {
    const int p = ntp >> 1, j = ntp & 1;
    nt = (p / pair_off) * 2 * pair_off + p % pair_off + j * pair_off;
  }
  const int n = nt * 32 + (lane & 31);
  const int k = kt * 32 + 16 * (lane >> 5) + 8 * ch;
  i32x4 v = {0, 0, 0, 0};
  if (n < N && k < K) v = *(const i32x4*)(w + (size_t)n * K + k);
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

// Pipeline depth (block rounds in flight) and k tiles per wave and round.  Measured on MI355X: 4 rounds
// cover the weight stream's latency at the 33.5 MB shapes (2, 6 and 8 are no faster); two k tiles per
// wave and round halve the barriers but lengthen every small launch of the denoise loop.
constexpr int kPF = 4;
constexpr int kTPW = 1;
constexpr int kPF8 = 3;  // rounds in flight of the eight-wave blocks (2 and 4 measured slower in whole requests)
template <int MT, int NT, int EPI, bool W16, int PRO, int NR, int NW>
int launch_nr(const GemmArgs& a, dim3 grid, hipStream_t st) {
  // the RMSNorm prologue over a short K that one block walks alone: all of its rounds in flight, the row
  // statistics taken from the staged pieces (SmolVLA's expert: K = 720, VLM: 960)
  constexpr bool CAN_FULL = (PRO == 1 || PRO == 3) && MT == 1 && NR > 0 && NR * NW <= 32;
  constexpr int PFN = NW == 8 ? kPF8 : kPF;
  if (CAN_FULL && a.ksplit == 1) {
    hipLaunchKernelGGL((fp8w_gemm_kernel<MT, NT, NW, EPI, CAN_FULL ? NR : PFN, kTPW, W16, PRO, NR>), grid, dim3(NW * 64), 0, st, a);
  } else {
    hipLaunchKernelGGL((fp8w_gemm_kernel<MT, NT, NW, EPI, PFN, kTPW, W16, PRO, NR>), grid, dim3(NW * 64), 0, st, a);
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
template <int MT, int NT, int EPI, bool W16, int PRO>
int launch(const GemmArgs& a, dim3 grid, int nw, hipStream_t st) {
  // the action chunk's launches (32-row blocks, every block the same number of k tiles) at the round counts
  // of the two models' expert layers.  Four waves: K = 720 -> 6, 960 / 1024 -> 8, 2048 -> 16, 4096 in four
  // splits -> 8; eight waves: 3, 4, 8, 4
  if (MT == 1 && a.kt_r == 0) {
    const int nr = (a.kt_q + nw * kTPW - 1) / (nw * kTPW);
    if (nw == 8) {
      if (nr == 3) return launch_nr<MT, NT, EPI, W16, PRO, MT == 1 ? 3 : 0, MT == 1 ? 8 : 4>(a, grid, st);
      if (nr == 4) return launch_nr<MT, NT, EPI, W16, PRO, MT == 1 ? 4 : 0, MT == 1 ? 8 : 4>(a, grid, st);
      if (nr == 8) return launch_nr<MT, NT, EPI, W16, PRO, MT == 1 ? 8 : 0, MT == 1 ? 8 : 4>(a, grid, st);
    } else {
      if (nr == 6) return launch_nr<MT, NT, EPI, W16, PRO, MT == 1 ? 6 : 0, 4>(a, grid, st);
      if (nr == 8) return launch_nr<MT, NT, EPI, W16, PRO, MT == 1 ? 8 : 0, 4>(a, grid, st);
      if (nr == 16) return launch_nr<MT, NT, EPI, W16, PRO, MT == 1 ? 16 : 0, 4>(a, grid, st);
    }
  }
  if (MT == 1 && nw == 8) return launch_nr<MT, NT, EPI, W16, PRO, 0, MT == 1 ? 8 : 4>(a, grid, st);
  return launch_nr<MT, NT, EPI, W16, PRO, 0, 4>(a, grid, st);
}

}  // namespace

int tk_launch_gemm(GemmArgs a, int MT, int NT, int mblocks, hipStream_t st) {
  dim3 grid((a.ntiles + NT - 1) / NT, a.ksplit, mblocks);
  // eight waves on a 32-row block where they pay (measured per launch and in whole requests, K = 720 .. 2048): a
  // long k range of fp8 tiles (half the rounds) or a norm prologue, plain or adaptive (half the normalisation work
  // per thread, and at K <= 1024 every round in flight with the row statistics taken from the staged pieces);
  // elsewhere four waves are as fast or faster (one LDS exchange less)
  const int pro_ = a.ada_scale != nullptr ? 3 : (a.norm_w == nullptr ? 0 : (a.x_f32 ? 2 : 1));
  const int nw = (MT == 1 && ((!a.w16 && a.kt_q >= 48) || pro_ == 1 || pro_ == 3)) ? 8 : 4;
  const int epi = a.s1 != nullptr ? 1 : (a.rope_pos != nullptr ? 2 : 0);
  const int pro = a.ada_scale != nullptr ? 3 : (a.norm_w == nullptr ? 0 : (a.x_f32 ? 2 : 1));
  if (a.w16) {
    // bf16-weight linears of the expert / VLM layers: 32- or 64-row blocks; one-tile strips for the plain epilogue only
    if (NT == 1) {
      if (epi != 0 || pro != 0) return -1;
      return MT == 1 ? launch<1, 1, 0, true, 0>(a, grid, nw, st) : launch<2, 1, 0, true, 0>(a, grid, nw, st);
    }
    if (epi == 2) {
      if (pro == 1) return MT == 1 ? launch<1, 2, 2, true, 1>(a, grid, nw, st) : launch<2, 2, 2, true, 1>(a, grid, nw, st);
      if (pro == 2) return MT == 1 ? launch<1, 2, 2, true, 2>(a, grid, nw, st) : launch<2, 2, 2, true, 2>(a, grid, nw, st);
      if (pro == 3) return MT == 1 ? launch<1, 2, 2, true, 3>(a, grid, nw, st) : launch<2, 2, 2, true, 3>(a, grid, nw, st);
      return MT == 1 ? launch<1, 2, 2, true, 0>(a, grid, nw, st) : launch<2, 2, 2, true, 0>(a, grid, nw, st);
    }
    if (epi == 0 && pro == 0) return MT == 1 ? launch<1, 2, 0, true, 0>(a, grid, nw, st) : launch<2, 2, 0, true, 0>(a, grid, nw, st);
    return -1;
  }
  if (epi == 2 || pro == 2) return -1;
  if (epi == 1) {
    if (NT != 2) return -1;
    if (pro == 1) return MT == 1 ? launch<1, 2, 1, false, 1>(a, grid, nw, st) : launch<2, 2, 1, false, 1>(a, grid, nw, st);
    if (pro == 3) return MT == 1 ? launch<1, 2, 1, false, 3>(a, grid, nw, st) : launch<2, 2, 1, false, 3>(a, grid, nw, st);
    return MT == 1 ? launch<1, 2, 1, false, 0>(a, grid, nw, st) : launch<2, 2, 1, false, 0>(a, grid, nw, st);
  }
  if (pro) return -1;
  if (NT == 1) return MT == 1 ? launch<1, 1, 0, false, 0>(a, grid, nw, st) : launch<2, 1, 0, false, 0>(a, grid, nw, st);
  return MT == 1 ? launch<1, 2, 0, false, 0>(a, grid, nw, st) : launch<2, 2, 0, false, 0>(a, grid, nw, st);
}

int tk_launch_ffn_fused(GemmArgs g, GemmArgs d, int d_nt, int mblocks, hipStream_t st) {
  // the same wave and round counts tk_launch_gemm would pick for the two launches (32-row blocks)
  if (g.w16 || d.w16 || g.s1 == nullptr || g.rope_pos != nullptr || d.s1 != nullptr || d.rope_pos != nullptr || g.ada_scale != nullptr ||
      g.x_f32 || d.norm_w != nullptr || d.ada_scale != nullptr || g.ksplit != 1 || g.kt_r != 0 || d.kt_r != 0 || mblocks > TK_FUSE_ROWBLOCKS || (g.ntiles + 1) / 2 > TK_FUSE_STRIPS ||
      d.KT != (g.ntiles + 1) / 2)
    return -1;
  const int gpro = g.norm_w != nullptr ? 1 : 0;
  const int gnw = (g.kt_q >= 48 || gpro == 1) ? 8 : 4, dnw = d.kt_q >= 48 ? 8 : 4;
  const int gnr = (g.kt_q + gnw - 1) / gnw, dnr = (d.kt_q + dnw - 1) / dnw;
  const int gstrips = (g.ntiles + 1) / 2, dstrips = (d.ntiles + d_nt - 1) / d_nt;
  const int nprod = gstrips * mblocks;
  const dim3 grid(nprod + dstrips * d.ksplit * mblocks);
#define TK_FUSED(GNW, GPF, GPRO, GNR, DNT, DNW, DPF, DNR)                                                                              \
  if (gnw == GNW && gpro == GPRO && gnr == GNR && d_nt == DNT && dnw == DNW && dnr == DNR) {                                           \
    hipLaunchKernelGGL((ffn_fused_kernel<GNW, GPF, GPRO, GNR, DNT, DNW, DPF, DNR>), grid, dim3((GNW > DNW ? GNW : DNW) * 64), 0, st, g, \
                       d, nprod, gstrips, dstrips);                                                                                    \
    return hipGetLastError() == hipSuccess ? 0 : -3;                                                                                   \
  }
  // K = 720 with the RMSNorm prologue -> I = 2048 -> 720 (SmolVLA's expert), the same without the prologue, and
  // K = 1024 -> I = 4096 -> 1024 with the down projection in four K splits (pi0.5's expert)
  TK_FUSED(8, 3, 1, 3, 1, 8, kPF8, 8)
  TK_FUSED(4, kPF, 0, 6, 1, 8, kPF8, 8)
  TK_FUSED(4, kPF, 0, 8, 1, 4, kPF, 8)
#undef TK_FUSED
  return -1;
}

int tk_launch_pack_bf16(const void* w, void* out, int N, int K, int pair_off, hipStream_t st) {
  const int KT = (K + 31) / 32;
  const int ntiles = (N + 31) / 32;
  const long long nchunks = (long long)ntiles * KT * 128;
  const long long blocks = (nchunks + 255) / 256;
  hipLaunchKernelGGL(pack_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const unsigned short*)w, (uint8_t*)out, N,
                     K, KT, nchunks, pair_off);
  return hipGetLastError() == hipSuccess ? 0 : -3;
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
