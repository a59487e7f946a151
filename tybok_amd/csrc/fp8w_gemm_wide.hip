// fp8-weight GEMM for many rows (M > 64: the VLM prefill) on gfx950.
//
// Same operands and packed weight tiles as the skinny kernel (fp8w_gemm.hip), other balance: with
// hundreds of rows the product is MFMA-bound, so the block tile is large enough that neither
// operand is re-read often:
//   * a block of 4 waves owns 128 rows x 8 packed n tiles (256 packed columns) and a range of k
//     tiles; wave w owns n tiles 2w, 2w+1 for all 128 rows: 8 accumulator tiles of 32x32, and per
//     k tile 16 MFMAs against 2 weight loads (straight from global memory into operand registers,
//     1 KiB coalesced per tile, e4m3 -> bf16 in registers) and 8 LDS operand reads;
//   * the activations of a round (128 rows x 64 columns) are staged once per block through LDS with
//     whole 128-byte lines per row, double buffered, one LDS barrier per round;
//   * blocks that share weights (same n tiles and k range, different rows) get consecutive slots of
//     ONE XCD, so the weight tiles are read from HBM once and served from that XCD's L2 afterwards;
//   * K splits (few column blocks, long K: the down projection) leave fp32 partials in the workspace and a
//     second launch over all CUs sums them in split order and runs the epilogue -- bit-deterministic.  (A
//     gated launch that is split keeps the one-launch form: the last-arriving block sums.  Measured at
//     M=712, K=16384, N=2048, 5 splits: 74 -> 52 + 7.7 us; one block per output tile -- 48 of 256 CUs -- pulling
//     31 MB of partials through 8-byte coherent loads, split after split, was a fifth of the launch.)
//   * where the grid would fill the device twice over (the gated 2048 -> 2 x 16384 launch) a block is EIGHT waves on
//     192 or 256 rows with the weights staged through LDS too (fp8w_tile_kernel below): half the bytes per matrix
//     instruction through the L2, the same accumulators, partials and epilogue, the same bits.
// The epilogues compute exactly what the skinny kernel's do (same rounding points).
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

constexpr int NT = 2;   // n tiles per wave
constexpr int NW = 4;   // waves per block
constexpr int RK = 2;   // k tiles per round

// LDS row pitch (bytes) of a wave's private 32-row output tile in wide_epilogue
__host__ __device__ constexpr int wide_ep_pitch(int epi) { return (epi == 0 ? NT * 32 : 32) * 2 + 16; }

// Epilogue of a wave that holds MT x NT accumulator tiles: rows row0 .. row0 + MT*32 - 1, packed n tiles strip*NT ..
// (EPI 1: the (gate, up) pair of output columns strip*32 ..).  wl: the wave's private LDS tile of 32 rows x
// wide_ep_pitch(EPI) bytes (used when the output is 16-byte aligned); the caller has made sure that no wave still
// reads what that space held before.
template <int EPI, int MT>
__device__ __forceinline__ void wide_epilogue(const GemmArgs& a, const f32x16 (&acc)[MT][NT], unsigned char* wl, int row0, int strip, int lane) {
  const int half = lane >> 5;
  const int l32 = lane & 31;
  // ---- epilogue: lane l of a tile owns row m = l % 32 and, per register group g, four
  // consecutive columns 8g + 4*(l/32) .. +3 (the accumulators hold C^T) ----
  if (a.vec16) {
    // Coalesced stores: a lane holds, per tile, row l % 32 and four 4-column pieces 16 bytes apart -- stored as
    // they are, one instruction would touch 32 rows with 16 bytes each.  Each wave therefore passes its 32 rows of
    // an m tile through a private LDS tile (a wave's LDS instructions execute in order, so it needs no barrier
    // of its own) and stores them as 16-byte chunks of consecutive columns: whole 64- or 128-byte row segments
    // per 4 or 8 lanes.
    constexpr int COLS = EPI == 0 ? NT * 32 : 32;  // output columns of a wave per row
    constexpr int EP = COLS * 2 + 16;              // LDS row pitch (bytes)
    constexpr int LPR = COLS / 8;                  // lanes (16-byte chunks) per row
    constexpr int RPI = 64 / LPR;                  // rows per store instruction
    static_assert(EP == wide_ep_pitch(EPI), "the callers size the LDS tiles by wide_ep_pitch");
    const int ncol0 = EPI == 0 ? strip * NT * 32 : strip * 32;  // first output column of this wave
    f32x4 sc0[EPI == 0 ? NT : 1][4], sc1[4], gt[EPI == 0 ? NT : 1][4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (EPI == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          int n0 = (strip * NT + nt) * 32 + 8 * g + 4 * half;
          if (n0 > a.N - 4) n0 = a.N - 4;  // columns past N are never stored
          sc0[EPI == 0 ? nt : 0][g] = *(const f32x4*)(a.s0 + n0);
          if (a.gate) gt[EPI == 0 ? nt : 0][g] = unpack_bf16x4(*(const i32x2*)(a.gate + n0));
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
            const f32x4 v = {c[4 * g], c[4 * g + 1], c[4 * g + 2], c[4 * g + 3]};
            i32x2 r = pack_bf16x4(v * sc0[EPI == 0 ? nt : 0][g]);
            if (a.gate) r = pack_bf16x4(unpack_bf16x4(r) * gt[EPI == 0 ? nt : 0][g]);
            *(i32x2*)(wl + l32 * EP + (nt * 32 + 8 * g + 4 * half) * 2) = r;
          }
        } else {
          const f32x16& cg = acc[mt][0];
          const f32x16& cu = acc[mt][1];
          const f32x4 vg = {cg[4 * g], cg[4 * g + 1], cg[4 * g + 2], cg[4 * g + 3]};
          const f32x4 vu = {cu[4 * g], cu[4 * g + 1], cu[4 * g + 2], cu[4 * g + 3]};
          const f32x4 gg = unpack_bf16x4(pack_bf16x4(vg * sc0[0][g]));
          const f32x4 up = unpack_bf16x4(pack_bf16x4(vu * sc1[g]));
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
        const int m = row0 + mt * 32 + row;
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
        f32x4 gt = {0.f, 0.f, 0.f, 0.f};
        if (a.gate) gt = unpack_bf16x4(*(const i32x2*)(a.gate + n0));
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int m = row0 + mt * 32 + l32;
          if (m >= a.M) continue;
          const f32x16& c = acc[mt][nt];
          f32x4 v = {c[4 * g], c[4 * g + 1], c[4 * g + 2], c[4 * g + 3]};
          i32x2 r = pack_bf16x4(v * sc);
          if (a.gate) r = pack_bf16x4(unpack_bf16x4(r) * gt);
          if (a.resid) {
            const f32x4 rv = a.resid_f32 ? *(const f32x4*)((const float*)a.resid + (size_t)m * a.ldr + n0)
                                         : unpack_bf16x4(*(const i32x2*)((const u16*)a.resid + (size_t)m * a.ldr + n0));
            r = pack_bf16x4(unpack_bf16x4(r) + rv);
          }
          *(i32x2*)(a.y + (size_t)m * a.ldy + n0) = r;
        }
      }
  } else {
    // tile pair (gate, up) of logical columns strip*32 ..; I % 32 == 0
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int col = strip * 32 + 8 * g + 4 * half;
      if (col >= a.N) continue;
      const f32x4 scg = *(const f32x4*)(a.s0 + col), scu = *(const f32x4*)(a.s1 + col);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = row0 + mt * 32 + l32;
        if (m >= a.M) continue;
        const f32x16& cg = acc[mt][0];
        const f32x16& cu = acc[mt][1];
        const f32x4 vg = {cg[4 * g], cg[4 * g + 1], cg[4 * g + 2], cg[4 * g + 3]};
        const f32x4 vu = {cu[4 * g], cu[4 * g + 1], cu[4 * g + 2], cu[4 * g + 3]};
        const f32x4 gg = unpack_bf16x4(pack_bf16x4(vg * scg));
        const f32x4 up = unpack_bf16x4(pack_bf16x4(vu * scu));
        f32x4 act;
#pragma unroll
        for (int j = 0; j < 4; ++j) act[j] = a.act == 0 ? silu_f(gg[j]) : gelu_tanh_f(gg[j]);
        act = unpack_bf16x4(pack_bf16x4(act));
        *(i32x2*)(a.y + (size_t)m * a.ldy + col) = pack_bf16x4(act * up);
      }
    }
  }
}

// EPI: 0 plain (scale, optional per-column gate, optional residual), 1 gated (gate/up tile pairs).
// MT: 32-row tiles per block (and per wave): 4 with one block per CU, 2 with two -- co-resident blocks cover each
// other's first loads and epilogue.  PF: rounds in flight (even: round r uses LDS buffer r % 2).
template <int EPI, int MT, int PF, int OCC>
__global__ __launch_bounds__(NW * 64, OCC) void fp8w_wide_kernel(GemmArgs a, int nblk_m, int ngroups) {
  constexpr int ROWS = MT * 32;
  constexpr int ROWB = RK * 64;            // bytes of one staged activation row per round
  constexpr int PITCH = ROWB + 16;         // conflict-free 16-byte operand reads, 16-byte aligned
  constexpr int XBUF = ROWS * PITCH;
  constexpr int PPR = ROWB / 16;           // 16-byte pieces per staged row
  constexpr int XPT = ROWS * PPR / (NW * 64);
  constexpr int TILES = MT * NT;
  constexpr int EPB = NW * 32 * ((EPI == 0 ? NT * 32 : 32) * 2 + 16);  // the epilogue's per-wave tiles
  __shared__ __align__(16) unsigned char lds[2 * XBUF > EPB ? 2 * XBUF : EPB];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5;
  const int l32 = lane & 31;

  // slot s of XCD x (blocks are dealt to the 8 XCDs round-robin) -> group (s / nblk_m) * 8 + x, m block
  // s % nblk_m: the nblk_m blocks of a group (same weights) run back to back on one XCD
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

  const int strip = nblk * NW + wave;  // this wave's pair of packed n tiles
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
    xsrc[i] = (const char*)a.x + (size_t)m * a.ldx * 2;
    xcol[i] = c * 8;
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
  auto wload1 = [&](WFrag& f, int r, int j, int nt) {  // k tile j of round r, n tile nt: one 1 KiB tile
    int kt = kt_lo + r * RK + j;
    if (kt > a.KT - 1) kt = a.KT - 1;  // its activation columns are zeroed
    f.w[j][nt] = *(const i32x4*)(wbase[nt] + (size_t)kt * 1024);
  };
  auto xload1 = [&](XFrag& f, int r, int i) {
    int k = (kt_lo + r * RK) * 32 + xcol[i];
    if (k > a.K - 8) k = a.K - 8;
    f.v[i] = *(const i32x4*)(xsrc[i] + (size_t)k * 2);
  };
  auto xstore1 = [&](const XFrag& f, int r, int b, int i) {
    const i32x4 z = {0, 0, 0, 0};
    *(i32x4*)(lds + b * XBUF + xdst[i]) = ((kt_lo + r * RK) * 32 + xcol[i]) < k_end ? f.v[i] : z;
  };
  // operand fragments and converted weights of two k tiles: while the MFMAs of one k tile run, the LDS reads and
  // the e4m3 -> bf16 conversions of the next one are issued between them
  i32x4 xa[2][MT][2];
  bf16x8 wb[2][NT][2];
  auto xread1 = [&](int set, int b, int j, int u) {  // u in [0, 2*MT): k step u%2 of m tile u/2, k tile j
    xa[set][u / 2][u % 2] = *(const i32x4*)(lds + b * XBUF + ((u / 2) * 32 + l32) * PITCH + (j * 32 + 16 * half) * 2 + 16 * (u % 2));
  };
  auto wcvt1 = [&](int set, const WFrag& f, int j, int q) {  // q in [0, 2*NT): k step q%2 of n tile q/2
    wb[set][q / 2][q % 2] = fp8x8_to_bf16x8(f.w[j][q / 2][2 * (q % 2)], f.w[j][q / 2][2 * (q % 2) + 1]);
  };
  auto mma1 = [&](int set, int t) {  // t in [0, 2*MT*NT): k step, m tile, n tile
    const int h2 = t / (MT * NT), mt = (t / NT) % MT, nt = t % NT;
    acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[set][nt][h2], as_bf16x8(xa[set][mt][h2]), acc[mt][nt], 0, 0, 0);
  };
  static_assert(RK == 2 && PF % 2 == 0, "a round is two phases; buffer parity follows the pipeline slot");

  // PF rounds in flight; every load is unconditional (clamped addresses; columns past the block's k range are
  // zeroed when staged), so the loop bodies have no branch and the compiler keeps precise wait counts.  Round r,
  // phase A: multiplies k tile 0 while k tile 1's operands are fetched from LDS and its weights converted (their
  // registers are refilled for round r+PF right after), and round r+1 is staged into the other LDS buffer; then
  // the round's only barrier (a wave can write buffer b for round r+2 only after every wave has passed the barrier
  // of round r+1, i.e. has its round-r operands in registers); phase B: fetches round r+1's first operands,
  // converts its first weights (and refills their registers) and multiplies k tile 1.  Each of a phase's
  // 2*MT*NT matrix instructions is followed by its share of the other work, fenced so that the order stands:
  // reads and conversions in the first half of the slots, the loads that refill converted registers in the second.
  constexpr int SLOTS = 2 * MT * NT;
  constexpr int HS = SLOTS / 2;
  static_assert(2 * MT <= SLOTS && 2 * NT <= HS && NT <= HS && XPT <= HS, "the pieces fit the slots");
  WFrag wbuf[PF];
  XFrag xbuf[PF];
#pragma unroll
  for (int p = 0; p < PF; ++p) {
#pragma unroll
    for (int i = 0; i < XPT; ++i) xload1(xbuf[p], p, i);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      wload1(wbuf[p], p, 0, nt);
      wload1(wbuf[p], p, 1, nt);
    }
  }
#pragma unroll
  for (int i = 0; i < XPT; ++i) xstore1(xbuf[0], 0, 0, i);
#pragma unroll
  for (int i = 0; i < XPT; ++i) xload1(xbuf[0], PF, i);
  lds_barrier();
#pragma unroll
  for (int u = 0; u < 2 * MT; ++u) xread1(0, 0, 0, u);
#pragma unroll
  for (int q = 0; q < 2 * NT; ++q) wcvt1(0, wbuf[0], 0, q);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) wload1(wbuf[0], PF, 0, nt);
  auto round = [&](int p, int r) {
    const int b = p & 1;  // == r & 1: rounds advance PF at a time
    const int pn = (p + 1) % PF;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      mma1(0, i);
#pragma unroll
      for (int u = 0; u < 2 * MT; ++u)
        if (u * SLOTS / (2 * MT) == i) xread1(1, b, 1, u);
#pragma unroll
      for (int q = 0; q < 2 * NT; ++q)
        if (q * HS / (2 * NT) == i) wcvt1(1, wbuf[p], 1, q);
#pragma unroll
      for (int x = 0; x < XPT; ++x) {
        if (x * HS / XPT == i) xstore1(xbuf[pn], r + 1, b ^ 1, x);
        if (HS + x * HS / XPT == i) xload1(xbuf[pn], r + 1 + PF, x);
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        if (HS + nt * HS / NT == i) wload1(wbuf[p], r + PF, 1, nt);  // converted above
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      mma1(1, i);
#pragma unroll
      for (int u = 0; u < 2 * MT; ++u)
        if (u * SLOTS / (2 * MT) == i) xread1(0, b ^ 1, 0, u);
#pragma unroll
      for (int q = 0; q < 2 * NT; ++q)
        if (q * HS / (2 * NT) == i) wcvt1(0, wbuf[pn], 0, q);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        if (HS + nt * HS / NT == i) wload1(wbuf[pn], r + 1 + PF, 0, nt);  // converted above
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

  // ---- K-split hand-off: fp32 partials [(block, split)][wave][tile][group][lane][4] ----
  const int blk_lin = nblk * nblk_m + mblock;
  if (a.ksplit > 1 && a.split_reduce) {
    // the partial leaves as it is (plain 16-byte stores: the kernel boundary publishes it); wide_split_reduce_kernel
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
    handoff_publish();
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
    for (int s = 0; s < a.ksplit; ++s) {  // split order, whoever arrived last
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

  // ---- epilogue ----
  constexpr int EP = wide_ep_pitch(EPI);
  static_assert(NW * 32 * EP == EPB, "the epilogue tiles fit the LDS array");
  if (a.vec16) lds_barrier();  // every wave has left the staged activations behind
  wide_epilogue<EPI, MT>(a, acc, lds + wave * 32 * EP, mblock * ROWS, strip, lane);
}

// The same product on a block of EIGHT waves that owns 2*WM*32 rows x 256 packed columns, with BOTH operands of a
// round staged through LDS: wave (wm, wn) = (wave / 4, wave % 4) owns rows wm*WM*32 .. of the block and the n tile
// pair wn, as a wave of the four-wave kernel does, so accumulators, partial layout and epilogue are the same -- but a
// weight tile is fetched (and converted to bf16) once per block and serves both wave rows, which halves the bytes
// that a CU pulls through the L2 per matrix instruction (the four-wave kernel's bound).  A round is four k steps of
// 16; operand registers of step s + 1 are read while step s multiplies; one barrier per round, before its last step:
// by then every wave has read the round's operands out of buffer b and written its share of round r + 1 into b ^ 1.
//   staging per thread and round: WM 16-byte pieces of x, 2 pieces of 16 fp8 weights (wave (wm, wn): k tile wm of
//   the round for its own n tile pair); each piece is requested again for round r + 1 + PF right after it is stored.
// LDS: 2 x (2*WM*32 rows x 144 B + 32 KiB of bf16 weight tiles) = 136 KB (WM = 4) / 118 KB (WM = 3), dynamic.
template <int EPI, int WM, int PF>
__global__ __launch_bounds__(512, 1) void fp8w_tile_kernel(GemmArgs a, int nblk_m, int ngroups) {
  constexpr int NWV = 8;
  constexpr int ROWS = 2 * WM * 32;
  constexpr int ROWB = RK * 64;
  constexpr int PITCH = ROWB + 16;
  constexpr int XBUF = ROWS * PITCH;
  constexpr int WBUF = NW * NT * RK * 2048;  // bf16 tiles of the round: [n tile][k tile][k step][lane][16 B]
  constexpr int STAGE = XBUF + WBUF;
  constexpr int XPT = ROWS * (ROWB / 16) / (NWV * 64);
  constexpr int TILES = WM * NT;
  constexpr int SL = WM * NT;  // matrix instructions per k step
  static_assert(XPT == WM && NWV * 32 * wide_ep_pitch(EPI) <= 2 * STAGE, "staging and epilogue tiles fit");
  extern __shared__ __align__(16) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int half = lane >> 5;
  const int l32 = lane & 31;

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

  const int strip = nblk * NW + wn;
  const uint8_t* wbase[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int ntg = strip * NT + nt;
    if (ntg > a.ntiles - 1) ntg = a.ntiles - 1;
    wbase[nt] = a.w + ((size_t)ntg * a.KT) * 1024 + lane * 16;
  }
  const char* xsrc[XPT];
  const int xcol = (tid & 7) * 8;
  const int xdst = (tid >> 3) * PITCH + (tid & 7) * 16;  // piece i: + i * 64 rows
#pragma unroll
  for (int i = 0; i < XPT; ++i) {
    int m = mblock * ROWS + i * 64 + (tid >> 3);
    if (m > a.M - 1) m = a.M - 1;
    xsrc[i] = (const char*)a.x + (size_t)m * a.ldx * 2;
  }

  f32x16 acc[WM][NT];
#pragma unroll
  for (int mt = 0; mt < WM; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;

  struct Stg {
    i32x4 x[XPT];
    i32x4 w[NT];
  };
  auto xload1 = [&](Stg& f, int r, int i) {
    int k = (kt_lo + r * RK) * 32 + xcol;
    if (k > a.K - 8) k = a.K - 8;
    f.x[i] = *(const i32x4*)(xsrc[i] + (size_t)k * 2);
  };
  auto wload1 = [&](Stg& f, int r, int nt) {
    int kt = kt_lo + r * RK + wm;
    if (kt > a.KT - 1) kt = a.KT - 1;  // its activation columns are zeroed
    f.w[nt] = *(const i32x4*)(wbase[nt] + (size_t)kt * 1024);
  };
  auto xstore1 = [&](const Stg& f, int r, int b, int i) {
    const i32x4 z = {0, 0, 0, 0};
    *(i32x4*)(lds + b * STAGE + xdst + i * 64 * PITCH) = ((kt_lo + r * RK) * 32 + xcol) < k_end ? f.x[i] : z;
  };
  auto wstore1 = [&](const Stg& f, int b, int q) {  // q in [0, 2*NT): k step q%2 of n tile q/2
    *(bf16x8*)(lds + b * STAGE + XBUF + ((((wn * NT + q / 2) * RK + wm) * 2 + q % 2) * 64 + lane) * 16) =
        fp8x8_to_bf16x8(f.w[q / 2][2 * (q % 2)], f.w[q / 2][2 * (q % 2) + 1]);
  };
  i32x4 fa[2][WM];
  bf16x8 fb[2][NT];
  auto fread1 = [&](int b, int s, int u) {  // operand u of k step s: u < WM the m tiles, then the n tiles
    const int set = s & 1, j = s >> 1, h2 = s & 1;
    if (u < WM)
      fa[set][u] = *(const i32x4*)(lds + b * STAGE + ((wm * WM + u) * 32 + l32) * PITCH + (j * 32 + 16 * half) * 2 + 16 * h2);
    else
      fb[set][u - WM] = *(const bf16x8*)(lds + b * STAGE + XBUF + ((((wn * NT + u - WM) * RK + j) * 2 + h2) * 64 + lane) * 16);
  };
  auto mma1 = [&](int set, int t) {
    const int mt = t / NT, nt = t % NT;
    acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[set][nt], as_bf16x8(fa[set][mt]), acc[mt][nt], 0, 0, 0);
  };

  Stg stg[PF];
#pragma unroll
  for (int q = 0; q < PF; ++q) {
#pragma unroll
    for (int i = 0; i < XPT; ++i) xload1(stg[q], q, i);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) wload1(stg[q], q, nt);
  }
#pragma unroll
  for (int i = 0; i < XPT; ++i) {
    xstore1(stg[0], 0, 0, i);
    xload1(stg[0], PF, i);
  }
#pragma unroll
  for (int q = 0; q < 2 * NT; ++q) wstore1(stg[0], 0, q);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) wload1(stg[0], PF, nt);
  lds_barrier();
#pragma unroll
  for (int u = 0; u < WM + NT; ++u) fread1(0, 0, u);

  auto round = [&](int p, int r) {  // p = r % 2 (the LDS buffer); round r + 1 waits in stg[(p + 1) % PF]
    const int b = p & 1;
    Stg& nx = stg[(p + 1) % PF];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if (s == 3) lds_barrier();
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < SL; ++i) {
        mma1(s & 1, i);
        if (i < WM + NT) fread1(s == 3 ? b ^ 1 : b, (s + 1) & 3, i);
        if (s == 0) {
#pragma unroll
          for (int x = 0; x < XPT; ++x)
            if (x * SL / XPT + 1 == i) {
              xstore1(nx, r + 1, b ^ 1, x);
              xload1(nx, r + 1 + PF, x);
            }
        }
        if (s == 1) {
#pragma unroll
          for (int q = 0; q < 2 * NT; ++q)
            if (q * SL / (2 * NT) + 1 == i) {
              wstore1(nx, b ^ 1, q);
              if (q % 2 == 1) wload1(nx, r + 1 + PF, q / 2);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  {
    int it = 0;
    for (; it + 2 <= nrounds; it += 2) {
      round(0, it);
      round(1, it + 1);
    }
    if (it < nrounds) round(0, it);
  }

  const int blk_lin = nblk * nblk_m + mblock;
  if (a.ksplit > 1) {  // always the two-launch form here: partials [(block, split)][wave][tile][group][lane][4]
    f32x4* mine = (f32x4*)a.partial + ((size_t)blk_lin * a.ksplit + split) * (NWV * TILES * 4 * 64) + (size_t)wave * TILES * 4 * 64 + lane;
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x16& c = acc[t / NT][t % NT];
        mine[(t * 4 + g) * 64] = f32x4{c[4 * g], c[4 * g + 1], c[4 * g + 2], c[4 * g + 3]};
      }
    return;
  }
  constexpr int EP = wide_ep_pitch(EPI);
  if (a.vec16) lds_barrier();
  wide_epilogue<EPI, WM>(a, acc, lds + wave * 32 * EP, mblock * ROWS + wm * WM * 32, strip, lane);
}

// Second launch of a K-split plain GEMM (GemmArgs::split_reduce): thread (block tile, wave, tile, lane) sums its four
// register groups over the splits in split order -- the order and the arithmetic of the last-arriving block of the
// one-launch form, so the same bits -- and finishes them like the scattered epilogue above.  Every CU takes part.
template <int MT, int NWV>
__global__ __launch_bounds__(256) void wide_split_reduce_kernel(GemmArgs a, int nblk_m, int nthreads) {
  constexpr int TILES = MT * NT;
  const int gid = blockIdx.x * 256 + threadIdx.x;
  if (gid >= nthreads) return;
  const int lane = gid & 63, half = lane >> 5, l32 = lane & 31;
  const int t = (gid >> 6) % TILES;
  const int wave = (gid >> 6) / TILES % NWV;
  const int blk_lin = (gid >> 6) / (TILES * NWV);
  const int mblock = blk_lin % nblk_m, nblk = blk_lin / nblk_m;
  const int mt = t / NT, nt = t % NT;
  const int strip = nblk * NW + wave % NW;
  const f32x4* src = (const f32x4*)a.partial + (size_t)blk_lin * a.ksplit * (NWV * TILES * 4 * 64) + (size_t)wave * TILES * 4 * 64 + (size_t)t * 4 * 64 + lane;
  f32x4 sum[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) sum[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int s = 0; s < a.ksplit; ++s) {
    f32x4 p[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) p[g] = src[(size_t)s * (NWV * TILES * 4 * 64) + g * 64];
#pragma unroll
    for (int g = 0; g < 4; ++g) sum[g] += p[g];
  }
  const int m = ((mblock * (NWV / NW) + wave / NW) * MT + mt) * 32 + l32;  // (eight waves: two wave rows of MT tiles)
  if (m >= a.M) return;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int n0 = (strip * NT + nt) * 32 + 8 * g + 4 * half;
    if (n0 >= a.N) continue;
    const f32x4 sc = *(const f32x4*)(a.s0 + n0);
    i32x2 r = pack_bf16x4(sum[g] * sc);
    if (a.gate) r = pack_bf16x4(unpack_bf16x4(r) * unpack_bf16x4(*(const i32x2*)(a.gate + n0)));
    if (a.resid) {
      const f32x4 rv = a.resid_f32 ? *(const f32x4*)((const float*)a.resid + (size_t)m * a.ldr + n0)
                                   : unpack_bf16x4(*(const i32x2*)((const u16*)a.resid + (size_t)m * a.ldr + n0));
      r = pack_bf16x4(unpack_bf16x4(r) + rv);
    }
    *(i32x2*)(a.y + (size_t)m * a.ldy + n0) = r;
  }
}

// One block per row: out = bf16 norm of the bf16 row, with the rounding points of the skinny
// kernel's prologues: RMSNorm bf16(w * bf16(x * rstd)); adaptive bf16((x * rstd) * (1 + scale) + shift).
// A thread's first piece of the row and the norm's operands for it are requested together up front and stay in
// registers (rows up to 2048 columns need nothing else): one memory round trip before the store, not three.
__global__ __launch_bounds__(256) void norm_rows_kernel(NormRowsArgs a) {
  __shared__ float part[4];
  const int tid = threadIdx.x;
  const char* row = (const char*)a.x + (size_t)blockIdx.x * a.ldx * 2;
  const int pieces = a.K / 8;
  const int p0 = tid < pieces ? tid : pieces - 1;  // past the row: a valid piece, not used
  union { i32x4 v; bf16x2 h[4]; unsigned u[4]; } x0;
  x0.v = *(const i32x4*)(row + (size_t)p0 * 16);
  union { i32x4 v[2]; float f[8]; } sc0, sh0;
  union { i32x4 v; unsigned u[4]; } nw0;
  if (a.ada_scale) {
    sc0.v[0] = *(const i32x4*)(a.ada_scale + p0 * 8);
    sc0.v[1] = *(const i32x4*)(a.ada_scale + p0 * 8 + 4);
    sh0.v[0] = *(const i32x4*)(a.ada_shift + p0 * 8);
    sh0.v[1] = *(const i32x4*)(a.ada_shift + p0 * 8 + 4);
  } else {
    nw0.v = *(const i32x4*)(a.norm_w + p0 * 8);
  }
  float ss0 = 0.f, ss1 = 0.f;
  auto square = [&](const bf16x2* h) {
    ss0 = __builtin_amdgcn_fdot2_f32_bf16(h[0], h[0], ss0, false);
    ss1 = __builtin_amdgcn_fdot2_f32_bf16(h[1], h[1], ss1, false);
    ss0 = __builtin_amdgcn_fdot2_f32_bf16(h[2], h[2], ss0, false);
    ss1 = __builtin_amdgcn_fdot2_f32_bf16(h[3], h[3], ss1, false);
  };
  if (tid < pieces) square(x0.h);
  for (int p = tid + 256; p < pieces; p += 256) {
    union { i32x4 v; bf16x2 h[4]; } xu;
    xu.v = *(const i32x4*)(row + (size_t)p * 16);
    square(xu.h);
  }
  float ss = ss0 + ss1;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  if ((tid & 63) == 0) part[tid >> 6] = ss;
  __syncthreads();
  ss = (part[0] + part[1]) + (part[2] + part[3]);
  const float rstd = rsqrtf(ss / (float)a.K + a.eps);
  char* dst = (char*)a.out + (size_t)blockIdx.x * a.ldo * 2;
  auto norm_piece = [&](const unsigned* xu, const float* sc, const float* sh, const unsigned* nw) {
    union { i32x4 v; unsigned u[4]; } o;
    if (a.ada_scale) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x0f = __uint_as_float(xu[e] << 16), x1f = __uint_as_float(xu[e] & 0xffff0000u);
        const float y0 = add_rn(mul_rn(mul_rn(x0f, rstd), add_rn(1.0f, sc[2 * e])), sh[2 * e]);
        const float y1 = add_rn(mul_rn(mul_rn(x1f, rstd), add_rn(1.0f, sc[2 * e + 1])), sh[2 * e + 1]);
        o.u[e] = pack_bf16x2(y0, y1);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const unsigned u = pack_bf16x2(__uint_as_float(xu[e] << 16) * rstd, __uint_as_float(xu[e] & 0xffff0000u) * rstd);
        o.u[e] = pack_bf16x2(__uint_as_float(nw[e] << 16) * __uint_as_float(u << 16),
                             __uint_as_float(nw[e] & 0xffff0000u) * __uint_as_float(u & 0xffff0000u));
      }
    }
    return o.v;
  };
  if (tid < pieces) *(i32x4*)(dst + (size_t)tid * 16) = norm_piece(x0.u, sc0.f, sh0.f, nw0.u);
  for (int p = tid + 256; p < pieces; p += 256) {
    union { i32x4 v; unsigned u[4]; } xu, nw;
    union { i32x4 v[2]; float f[8]; } sc, sh;
    xu.v = *(const i32x4*)(row + (size_t)p * 16);
    if (a.ada_scale) {
      sc.v[0] = *(const i32x4*)(a.ada_scale + p * 8);
      sc.v[1] = *(const i32x4*)(a.ada_scale + p * 8 + 4);
      sh.v[0] = *(const i32x4*)(a.ada_shift + p * 8);
      sh.v[1] = *(const i32x4*)(a.ada_shift + p * 8 + 4);
    } else {
      nw.v = *(const i32x4*)(a.norm_w + p * 8);
    }
    *(i32x4*)(dst + (size_t)p * 16) = norm_piece(xu.u, sc.f, sh.f, nw.u);
  }
}

}  // namespace

int tk_wide_cols() { return NW * NT * 32; }

namespace {
template <int EPI, int WM, int PF>
bool launch_tile(const GemmArgs& a, dim3 grid, int nblk_m, int ngroups, hipStream_t st) {
  constexpr int LDS = 2 * (2 * WM * 32 * (RK * 64 + 16) + NW * NT * RK * 2048);
  static bool sized = false;  // above 64 KiB of LDS a kernel has to be told once
  if (!sized) {
    if (hipFuncSetAttribute((const void*)fp8w_tile_kernel<EPI, WM, PF>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess) return false;
    sized = true;
  }
  hipLaunchKernelGGL((fp8w_tile_kernel<EPI, WM, PF>), grid, dim3(512), LDS, st, a, nblk_m, ngroups);
  return true;
}
}  // namespace

// a.mtiles: 32-row tiles per block: 2 or 4 (four waves, weights straight from memory), 6 or 8 (eight waves, both
// operands through LDS; a K split of those always finishes in the reduction launch)
int tk_launch_gemm_wide(GemmArgs a, hipStream_t st) {
  if (a.mtiles != 2 && a.mtiles != 4 && a.mtiles != 6 && a.mtiles != 8) return -1;
  const bool tile8 = a.mtiles > 4;
  const int nblk_m = (a.M + a.mtiles * 32 - 1) / (a.mtiles * 32);
  const int nblk_n = (a.ntiles + NW * NT - 1) / (NW * NT);
  const int ngroups = nblk_n * a.ksplit;
  const dim3 grid((unsigned)((ngroups + 7) / 8) * 8u * (unsigned)nblk_m), block(NW * 64);
  // K splits of a plain launch with 4-column alignment: partials out, then a reduction launch over all CUs
  a.split_reduce = a.ksplit > 1 && !a.s1 && a.vec && a.N % 4 == 0;
  if (tile8 && a.ksplit > 1 && !a.split_reduce) return -1;
  bool ok = true;
  if (a.s1) {
    if (a.mtiles == 8)
      ok = launch_tile<1, 4, 1>(a, grid, nblk_m, ngroups, st);
    else if (a.mtiles == 6)
      ok = launch_tile<1, 3, 1>(a, grid, nblk_m, ngroups, st);
    else if (a.mtiles == 4)
      hipLaunchKernelGGL((fp8w_wide_kernel<1, 4, 4, 1>), grid, block, 0, st, a, nblk_m, ngroups);
    else
      hipLaunchKernelGGL((fp8w_wide_kernel<1, 2, 4, 2>), grid, block, 0, st, a, nblk_m, ngroups);
  } else {
    if (a.mtiles == 8)
      ok = launch_tile<0, 4, 1>(a, grid, nblk_m, ngroups, st);
    else if (a.mtiles == 6)
      ok = launch_tile<0, 3, 1>(a, grid, nblk_m, ngroups, st);
    else if (a.mtiles == 4)
      hipLaunchKernelGGL((fp8w_wide_kernel<0, 4, 4, 1>), grid, block, 0, st, a, nblk_m, ngroups);
    else
      hipLaunchKernelGGL((fp8w_wide_kernel<0, 2, 4, 2>), grid, block, 0, st, a, nblk_m, ngroups);
  }
  if (!ok) return -3;
  if (a.split_reduce) {
    const int nthreads = nblk_n * nblk_m * NW * a.mtiles * NT * 64;  // one per (output tile, lane), whatever the waves
    const dim3 rg((nthreads + 255) / 256), rb(256);
    if (a.mtiles == 8) hipLaunchKernelGGL((wide_split_reduce_kernel<4, 8>), rg, rb, 0, st, a, nblk_m, nthreads);
    else if (a.mtiles == 6) hipLaunchKernelGGL((wide_split_reduce_kernel<3, 8>), rg, rb, 0, st, a, nblk_m, nthreads);
    else if (a.mtiles == 4) hipLaunchKernelGGL((wide_split_reduce_kernel<4, 4>), rg, rb, 0, st, a, nblk_m, nthreads);
    else hipLaunchKernelGGL((wide_split_reduce_kernel<2, 4>), rg, rb, 0, st, a, nblk_m, nthreads);
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

int tk_launch_norm_rows(NormRowsArgs a, hipStream_t st) {
  hipLaunchKernelGGL(norm_rows_kernel, dim3(a.M), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
