// bf16-weight GEMM for many rows with bias / GELU / residual epilogues on gfx950: the linears of the vision
// towers (q|k|v, out_proj, fc1, fc2 over 256 .. 1024 patches per camera) and the bf16 projections of the VLM
// prefill.
//
//   y[M, N] = bf16( resid + act( bf16( x[M, K] . W[N, K]^T + bias[N] ) ) )
//
// Operands: x bf16 row-major; W in the 2 KiB tile order of tk_pack_bf16_weight (tile (nt, kt): two 1 KiB chunks,
// chunk c of lane l = 8 bf16 of column nt*32 + l%32 at k = 32*kt + 16*(l/32) + 8*c), so a weight operand of
// v_mfma_f32_32x32x16_bf16 is one coalesced 16-byte load per lane straight into registers.
//   * a block of 4 waves owns MT*32 rows x 4*NT*32 columns and a range of k tiles; wave w owns n tiles
//     w*NT .. w*NT+NT-1 for all rows;
//   * the activations of a round (MT*32 rows x 64 columns) are staged once per block through LDS with whole
//     128-byte lines per row, double buffered, one LDS barrier per round;
//   * blocks that share weights (same n tiles and k range, different rows) get consecutive slots of ONE XCD, so
//     a weight tile comes from HBM once and from that XCD's L2 afterwards;
//   * K splits hand fp32 partials through the workspace; the last-arriving block sums them in split order:
//     bit-deterministic;
//   * the epilogue passes each wave's 32-row slices through a private LDS tile and stores 16-byte row segments.
// Tile shapes (MT, NT) from (4, 2) = 128 x 256, one block per CU, down to (1, 1) = 32 x 128 with four blocks per
// CU: the host picks the one whose blocks are all resident at once and load the CUs evenly (co-resident blocks
// overlap each other's first loads and epilogue, a second generation of blocks would pay both again).
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

constexpr int NW = 4;  // waves per block
constexpr int RK = 2;  // k tiles (of 32) per round

// F16: the operands are fp16 (v_mfma_f32_32x32x16_f16) instead of bf16; same tile order, same epilogues
// ROPE (NT == 2, bf16): the weights are packed in rotary pair order -- the two tiles of a wave hold columns
// (c, c + rope_half) of one head -- and the epilogue is the skinny kernel's rotary one: columns < rope_cols rotated
// by the table row of pos[m] (fp32 products rounded separately, or every product and sum rounded to bf16), columns
// >= vt_col0 also written transposed for the attention kernel.  No bias, activation or residual in this form.
template <int MT, int NT, int PF, int OCC, bool F16, bool ROPE = false>
__global__ __launch_bounds__(NW * 64, OCC) void bf16w_wide_kernel(GemmArgs a, int nblk_m, int ngroups) {
  static_assert(!ROPE || (NT == 2 && !F16), "the rotary epilogue needs both halves of a pair in one wave");
  constexpr int ROWS = MT * 32;
  constexpr int ROWB = RK * 64;     // bytes of one staged activation row per round
  constexpr int PITCH = ROWB + 16;  // conflict-free 16-byte operand reads, 16-byte aligned
  constexpr int XBUF = ROWS * PITCH;
  constexpr int PPR = ROWB / 16;    // 16-byte pieces per staged row
  constexpr int XPT = ROWS * PPR / (NW * 64);
  constexpr int TILES = MT * NT;
  static_assert(RK == 2 && PF % 2 == 0, "a round is two phases; buffer parity follows the pipeline slot");
  // epilogue: each wave's 32 x (NT*32) bf16 slice passes through a private LDS tile in the staging buffers' space
  constexpr int COLS = NT * 32;      // output columns of a wave per row
  constexpr int EP = COLS * 2 + 16;  // LDS row pitch (bytes)
  constexpr int LPR = COLS / 8;      // lanes (16-byte chunks) per row
  constexpr int RPI = 64 / LPR;      // rows per store instruction
  constexpr int LDSB = 2 * XBUF > NW * 32 * EP ? 2 * XBUF : NW * 32 * EP;
  __shared__ __align__(16) unsigned char lds[LDSB];

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

  const int strip = nblk * NW + wave;  // this wave's NT packed n tiles
  const uint8_t* wbase[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int ntg = strip * NT + nt;
    if (ntg > a.ntiles - 1) ntg = a.ntiles - 1;  // overhanging tiles are computed on valid data, never stored
    wbase[nt] = a.w + ((size_t)ntg * a.KT) * 2048 + lane * 16;
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
    i32x4 w[RK][NT][2];
  };
  struct XFrag {
    i32x4 v[XPT];
  };
  // One piece of each kind of work, so that a round can deal them out between its matrix instructions: a wave
  // cannot issue anything while it waits for the matrix pipe to take its next instruction, so whatever stands
  // between two groups of matrix instructions in program order runs with the pipe empty.
  auto wload1 = [&](WFrag& f, int r, int j, int q) {  // q in [0, 2*NT): chunk q%2 of n tile q/2, k tile j of round r
    int kt = kt_lo + r * RK + j;
    if (kt > a.KT - 1) kt = a.KT - 1;  // its activation columns are zeroed
    f.w[j][q / 2][q % 2] = *(const i32x4*)(wbase[q / 2] + (size_t)kt * 2048 + (q % 2) * 1024);
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
  // operand fragments of the round's two k tiles, as the 16-byte halves (k steps of 16) they are read in
  i32x4 xa[2][MT][2];
  auto xread1 = [&](int set, int b, int j, int u) {  // u in [0, 2*MT): k step u%2 of m tile u/2, k tile j
    xa[set][u / 2][u % 2] = *(const i32x4*)(lds + b * XBUF + ((u / 2) * 32 + l32) * PITCH + (j * 32 + 16 * half) * 2 + 16 * (u % 2));
  };
  auto mma1 = [&](int set, const WFrag& f, int j, int t) {  // t in [0, 2*MT*NT): k step, m tile, n tile
    const int h2 = t / (MT * NT), mt = (t / NT) % MT, nt = t % NT;
    if (F16)
      acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_f16x8(f.w[j][nt][h2]), as_f16x8(xa[set][mt][h2]), acc[mt][nt], 0, 0, 0);
    else
      acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(f.w[j][nt][h2]), as_bf16x8(xa[set][mt][h2]), acc[mt][nt], 0, 0, 0);
  };

  // PF rounds in flight; every load is unconditional (clamped addresses; columns past the block's k range are
  // zeroed when staged), so the loop bodies have no branch and the compiler keeps precise wait counts.  Round r,
  // phase A: multiplies k tile 0 while k tile 1's operands are fetched from LDS, round r+1 is staged into the
  // other LDS buffer and the weight registers that round r-1's k tile 1 has left are refilled; then the round's
  // only barrier (a wave can write buffer b for round r+2 only after every wave has passed the barrier of round
  // r+1, i.e. has its round-r operands in registers); phase B: fetches round r+1's first operands, multiplies k
  // tile 1 and refills k tile 0's weight registers.  A phase never reloads registers its own matrix instructions
  // read.  Each of a phase's 2*MT*NT matrix instructions is followed by its share of the other work (piece j of
  // n goes to slot j * SLOTS / n), fenced so that the order stands.
  constexpr int SLOTS = 2 * MT * NT;
  constexpr int HS = SLOTS / 2;  // staging: stores in the first half of phase A's slots, loads in the second
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
  for (int u = 0; u < 2 * MT; ++u) xread1(0, 0, 0, u);
  auto round = [&](int p, int r) {
    const int b = p & 1;  // == r & 1: rounds advance PF at a time
    const int pn = (p + 1) % PF, pp = (p + PF - 1) % PF;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      mma1(0, wbuf[p], 0, i);
#pragma unroll
      for (int u = 0; u < 2 * MT; ++u)
        if (u * SLOTS / (2 * MT) == i) xread1(1, b, 1, u);
#pragma unroll
      for (int x = 0; x < XPT; ++x) {
        if (x * HS / XPT == i) xstore1(xbuf[pn], r + 1, b ^ 1, x);
        if (HS + x * HS / XPT == i) xload1(xbuf[pn], r + 1 + PF, x);
      }
#pragma unroll
      for (int q = 0; q < 2 * NT; ++q)
        if (q * SLOTS / (2 * NT) == i) wload1(wbuf[pp], r - 1 + PF, 1, q);  // registers round r-1 finished with in its phase B
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      mma1(1, wbuf[p], 1, i);
#pragma unroll
      for (int u = 0; u < 2 * MT; ++u)
        if (u * SLOTS / (2 * MT) == i) xread1(0, b ^ 1, 0, u);
#pragma unroll
      for (int q = 0; q < 2 * NT; ++q)
        if (q * SLOTS / (2 * NT) == i) wload1(wbuf[p], r + PF, 0, q);  // k tile 0's registers: free since phase A
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
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        unsigned long long raw[4][2];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          raw[g][0] = ld_agent64(src + (size_t)(t * 4 + g) * 128);
          raw[g][1] = ld_agent64(src + (size_t)(t * 4 + g) * 128 + 1);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x16& c = acc[t / NT][t % NT];
          c[4 * g] += __uint_as_float((unsigned)raw[g][0]);
          c[4 * g + 1] += __uint_as_float((unsigned)(raw[g][0] >> 32));
          c[4 * g + 2] += __uint_as_float((unsigned)raw[g][1]);
          c[4 * g + 3] += __uint_as_float((unsigned)(raw[g][1] >> 32));
        }
      }
    }
  }

  // ---- epilogue: lane l of a tile owns row m = l % 32 and, per register group g, four consecutive columns
  // 8g + 4*(l/32) .. +3 (the accumulators hold C^T).  Stored as they are, one instruction would touch 32 rows with
  // 8 bytes each; each wave therefore passes its 32 rows of an m tile through a private LDS tile (a wave's LDS
  // instructions execute in order, so it needs no barrier of its own) and stores 16-byte chunks of consecutive
  // columns: whole row segments of NT*64 bytes per 4*NT lanes. ----
  lds_barrier();  // every wave has left the staged activations behind
  unsigned char* wl = lds + wave * 32 * EP;
  if constexpr (ROPE) {
    // logical tile of physical tile (strip, j): (strip / PO) * 2 * PO + strip % PO + j * PO, PO = rope_half / 32
    const int po = a.rope_half >> 5;
    const int ca0 = ((strip / po) * 2 * po + strip % po) * 32, cb0 = ca0 + a.rope_half;  // first columns of the two tiles
    const bool rot = ca0 < a.rope_cols;
    const int fi0 = ca0 % (2 * a.rope_half) + 4 * half;
    const int lrow = lane / LPR, lchunk = lane % LPR;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m0 = (mblock * MT + mt) * 32;
      int mr = m0 + l32;
      if (mr > a.M - 1) mr = a.M - 1;
      int pos = a.rope_pos[mr];
      pos = pos < 0 ? 0 : (pos > a.rope_positions - 1 ? a.rope_positions - 1 : pos);
      const float* cs_row = a.rope_cos + (size_t)pos * a.rope_half + fi0;
      const float* sn_row = a.rope_sin + (size_t)pos * a.rope_half + fi0;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x16& c0 = acc[mt][0];
        const f32x16& c1 = acc[mt][1];
        f32x4 va = unpack_bf16x4(pack_bf16x4(f32x4{c0[4 * g], c0[4 * g + 1], c0[4 * g + 2], c0[4 * g + 3]}));
        f32x4 vb = unpack_bf16x4(pack_bf16x4(f32x4{c1[4 * g], c1[4 * g + 1], c1[4 * g + 2], c1[4 * g + 3]}));
        if (rot) {
          const f32x4 cs = *(const f32x4*)(cs_row + 8 * g), sn = *(const f32x4*)(sn_row + 8 * g);
          f32x4 ra, rb;
          if (a.rope_bf16) {
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
          va = ra;
          vb = rb;
        }
        *(i32x2*)(wl + l32 * EP + (8 * g + 4 * half) * 2) = pack_bf16x4(va);
        *(i32x2*)(wl + l32 * EP + (32 + 8 * g + 4 * half) * 2) = pack_bf16x4(vb);
      }
#pragma unroll
      for (int j = 0; j < 32 / RPI; ++j) {
        const int row = j * RPI + lrow;
        const int m = m0 + row;
        const int n = (lchunk < 4 ? ca0 : cb0) + (lchunk & 3) * 8;
        const i32x4 t = *(const i32x4*)(wl + row * EP + lchunk * 16);
        if (m >= a.M || n >= a.N) continue;
        *(i32x4*)(a.y + (size_t)m * a.ldy + n) = t;  // N is a multiple of 64 in this form
      }
      if (a.vt && ca0 >= a.vt_col0) {  // wave-uniform: vt_col0 is a multiple of the head size
        // value columns, transposed for the attention kernel: lane = one of the wave's 64 columns, eight consecutive
        // rows per 16-byte store; rows past M stay zero (the attention kernel relies on zeros behind the last key)
        const int n = (lane < 32 ? ca0 : cb0) + (lane & 31);
        if (n < a.N) {
          u16* dst = a.vt + (size_t)(n - a.vt_col0) * a.vt_ld + m0;
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            unsigned e[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) e[r] = m0 + 8 * rg + r < a.M ? *(const u16*)(wl + (8 * rg + r) * EP + lane * 2) : 0u;
            if (m0 + 8 * rg < a.M)
              *(i32x4*)(dst + 8 * rg) = i32x4{(int)(e[0] | (e[1] << 16)), (int)(e[2] | (e[3] << 16)), (int)(e[4] | (e[5] << 16)), (int)(e[6] | (e[7] << 16))};
          }
        }
      }
    }
    return;
  }
  const int ncol0 = strip * COLS;  // first output column of this wave
  f32x4 bias[NT][4];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      int n0 = ncol0 + nt * 32 + 8 * g + 4 * half;
      if (n0 > a.N - 4) n0 = a.N - 4;  // columns past N are never stored
      bias[nt][g] = a.bias ? unpack_16x4<F16>(*(const i32x2*)(a.bias + n0)) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  const int lrow = lane / LPR, lchunk = lane % LPR;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x16& c = acc[mt][nt];
        f32x4 v = {c[4 * g], c[4 * g + 1], c[4 * g + 2], c[4 * g + 3]};
        v = v + bias[nt][g];
        if (a.act == 1) v = unpack_16x4<F16>(pack_16x4<F16>(v));  // the linear's 16-bit output, then the activation on it
        if (a.act) {
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = gelu_tanh_f(v[j]);
        }
        *(i32x2*)(wl + l32 * EP + (nt * 32 + 8 * g + 4 * half) * 2) = pack_16x4<F16>(v);
      }
#pragma unroll
    for (int j = 0; j < 32 / RPI; ++j) {
      const int row = j * RPI + lrow;
      const int m = (mblock * MT + mt) * 32 + row;
      const int n = ncol0 + lchunk * 8;
      i32x4 t = *(const i32x4*)(wl + row * EP + lchunk * 16);
      if (m >= a.M || n >= a.N) continue;
      if (a.resid) {
        f32x4 r0, r1 = {0.f, 0.f, 0.f, 0.f};
        if (a.resid_f32) {
          const f32x4* rp = (const f32x4*)((const float*)a.resid + (size_t)m * a.ldr + n);
          r0 = rp[0];
          if (n + 8 <= a.N) r1 = rp[1];
        } else if (n + 8 <= a.N) {
          const i32x4 rr = *(const i32x4*)((const u16*)a.resid + (size_t)m * a.ldr + n);
          r0 = unpack_16x4<F16>(i32x2{rr[0], rr[1]});
          r1 = unpack_16x4<F16>(i32x2{rr[2], rr[3]});
        } else {
          r0 = unpack_16x4<F16>(*(const i32x2*)((const u16*)a.resid + (size_t)m * a.ldr + n));
        }
        const i32x2 lo = pack_16x4<F16>(unpack_16x4<F16>(i32x2{t[0], t[1]}) + r0), hi = pack_16x4<F16>(unpack_16x4<F16>(i32x2{t[2], t[3]}) + r1);
        t = i32x4{lo[0], lo[1], hi[0], hi[1]};
      }
      u16* dst = a.y + (size_t)m * a.ldy + n;
      if (n + 8 <= a.N) *(i32x4*)dst = t;
      else *(i32x2*)dst = i32x2{t[0], t[1]};  // N % 8 == 4: the row's last four columns
    }
    if (a.vt && ncol0 >= a.vt_col0) {  // wave-uniform: vt_col0 is a multiple of the wave's COLS columns
      // value columns of a packed q|k|v projection, also written transposed for the attention kernel (no activation
      // or residual in this form, so the LDS tile holds the final values): a lane takes one of the wave's columns
      // and eight consecutive rows per 16-byte store.  The rows of an m tile belong to one problem (vt_rows is a
      // multiple of 32); rows past M are written as zeros.
      const int ccol = lane % COLS, n = ncol0 + ccol;
      const int m0 = (mblock * MT + mt) * 32;
      if (n < a.N && m0 < a.M) {
        const int prob = a.vt_rows ? m0 / a.vt_rows : 0, key0 = a.vt_rows ? m0 % a.vt_rows : m0;
        u16* dst = a.vt + (size_t)prob * a.vt_bs + (size_t)(n - a.vt_col0) * a.vt_ld + key0;
#pragma unroll
        for (int rg = lane / COLS; rg < 4; rg += 64 / COLS) {
          unsigned e[8];
#pragma unroll
          for (int r = 0; r < 8; ++r) e[r] = m0 + 8 * rg + r < a.M ? *(const u16*)(wl + (8 * rg + r) * EP + ccol * 2) : 0u;
          if (m0 + 8 * rg < a.M)
            *(i32x4*)(dst + 8 * rg) = i32x4{(int)(e[0] | (e[1] << 16)), (int)(e[2] | (e[3] << 16)), (int)(e[4] | (e[5] << 16)), (int)(e[6] | (e[7] << 16))};
        }
      }
    }
  }
}

template <int MT, int NT, int PF, int OCC>
int launch(const GemmArgs& a, hipStream_t st) {
  const int nblk_m = (a.M + MT * 32 - 1) / (MT * 32);
  const int nblk_n = (a.ntiles + NW * NT - 1) / (NW * NT);
  const int ngroups = nblk_n * a.ksplit;
  const unsigned blocks = (unsigned)((ngroups + 7) / 8) * 8u * (unsigned)nblk_m;
  if (a.rope_pos) {
    if constexpr (NT == 2) {
      if (a.f16) return -1;
      hipLaunchKernelGGL((bf16w_wide_kernel<MT, NT, PF, OCC, false, true>), dim3(blocks), dim3(NW * 64), 0, st, a, nblk_m, ngroups);
      return hipGetLastError() == hipSuccess ? 0 : -3;
    } else {
      return -1;
    }
  }
  if (a.f16)
    hipLaunchKernelGGL((bf16w_wide_kernel<MT, NT, PF, OCC, true>), dim3(blocks), dim3(NW * 64), 0, st, a, nblk_m, ngroups);
  else
    hipLaunchKernelGGL((bf16w_wide_kernel<MT, NT, PF, OCC, false>), dim3(blocks), dim3(NW * 64), 0, st, a, nblk_m, ngroups);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace

// tile = 10 * MT + NT
int tk_launch_bf16w_wide(const GemmArgs& a, int tile, hipStream_t st) {
  switch (tile) {
    case 42: return launch<4, 2, 4, 1>(a, st);
    case 41: return launch<4, 1, 2, 2>(a, st);
    case 32: return launch<3, 2, 2, 2>(a, st);
    case 31: return launch<3, 1, 2, 3>(a, st);
    case 22: return launch<2, 2, 2, 2>(a, st);
    case 21: return launch<2, 1, 2, 4>(a, st);
    case 12: return launch<1, 2, 2, 3>(a, st);
    case 11: return launch<1, 1, 2, 4>(a, st);
  }
  return -1;
}
