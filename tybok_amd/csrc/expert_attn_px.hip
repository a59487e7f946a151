// Action-expert attention for 64-wide heads when one block covers the whole key range (the SmolVLA
// self layers: 50 queries, 15 heads over 5 K/V heads, ~290 keys = 10 key tiles), same operands and
// masks as expert_attn.hip.
//
// One wave per 32-key tile computes S^T = K . Q^T for its tile and the tile's softmax terms against
// the block-wide maximum (one exchange of the tile maxima through LDS).  Q, K and V^T are read as whole
// rows with coalesced 16-byte loads and staged through LDS into MFMA operand order.  Instead of every wave also multiplying its probabilities with its V tile and
// the block then merging one partial output per wave (8 KiB each through LDS, summed by four owner
// waves -- the longest phase of that kernel), the waves park their P^T tiles in LDS as ready-made B
// operands (2 KiB each) and D/32 waves compute the whole O^T = V^T . P^T, one 32-row slice each, from
// V^T rows they requested at the very start: no partial outputs, no merge.
#include <math.h>
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

constexpr float kF32Min = -3.4028234663852886e38f;  // finfo(float32).min
constexpr float kOpenpiMask = -2.3819763e38f;       // additive mask of the pi0.5 path

// K row held by MFMA row r of a key tile (bits 2 and 3 of r swapped): accumulator registers 8s..8s+7
// of a lane are then eight consecutive keys, one 16-byte chunk of a V^T row and of the P^T operand
__device__ __forceinline__ int key_of_row(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

__device__ __forceinline__ i32x4 pack8(const float* v) {
  i32x4 r = {(int)pack_bf16x2(v[0], v[1]), (int)pack_bf16x2(v[2], v[3]), (int)pack_bf16x2(v[4], v[5]), (int)pack_bf16x2(v[6], v[7])};
  return r;
}

__device__ __forceinline__ void lds_only_barrier() {
  // waits for LDS traffic only: the V^T loads stay in flight across it
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// NWV waves, at most NWV key tiles (prefix tiles, then suffix tiles); grid (head, query tile)
template <int D, int NWV>
__global__ __launch_bounds__(NWV * 64) void expert_attn_px_kernel(AttnArgs a) {
  constexpr int DS = D / 16;  // k steps of Q.K^T
  constexpr int DT = D / 32;  // 32-row slices of O^T = waves of the second product
  static_assert(DT <= NWV, "one wave per output slice");
  constexpr int RCH = D / 8;            // 16-byte chunks of a Q or K row
  constexpr int KCH = 32 * RCH / 64;    // chunks of a K tile per lane
  constexpr int VCH = D * 4 / 64;       // chunks of the block's V^T (D rows x NWV tiles x 4) per thread
  constexpr int QPITCH = D * 2 + 16;    // staged Q / K rows: 16-byte operand reads of 32 rows stay conflict-free
  constexpr int VPITCH = NWV * 64 + 16; // staged V^T rows (NWV tiles x 32 keys)
  __shared__ float st_m[NWV][32], st_l[NWV][32];
  __shared__ __align__(16) i32x4 pt[NWV][2][64];  // P^T of every key tile as B operands [tile][k step][lane]
  __shared__ __align__(16) unsigned char qs[32 * QPITCH];
  __shared__ __align__(16) unsigned char kst[NWV][32 * QPITCH];
  __shared__ __align__(16) unsigned char vs[D * VPITCH];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int h = blockIdx.x;
  const int mtile = blockIdx.y;
  const int g = (h * a.gqa_mul) >> 16;
  const int tp = (a.P + 31) >> 5;  // prefix tiles; suffix tiles follow
  const int nt = tp + ((a.S + 31) >> 5);
  const int qi = mtile * 32 + l32;
  const bool q_ok = qi < a.M;
  const bool active = wave < nt;  // this wave has a key tile of its own
  unsigned char* const ks = kst[wave];

  // ---- every load up front, as whole rows (lane -> consecutive 16-byte chunks) staged through LDS:
  // read straight into operand registers (one row per lane) every load instruction touches 32 cache
  // lines for 1 KiB, and a block's 12 waves x 12 such loads are bound by the CU's tag-lookup rate ----
  const int tid = threadIdx.x;
  const int t = active ? wave : nt - 1;  // idle waves read a valid tile and drop it
  const bool pre = t < tp;
  const int tt = pre ? t : t - tp;
  const int len = pre ? a.P : a.S;
  i32x4 qreg, kreg[KCH], vreg[VCH];
  {
    // Q tile: 32 rows x D, one chunk per thread of the first waves
    const int c = tid < 32 * RCH ? tid : 0, row = c / RCH, col = c % RCH;
    int m = mtile * 32 + row;
    if (m > a.M - 1) m = a.M - 1;  // rows past M are never stored
    qreg = *(const i32x4*)(a.q + (size_t)m * a.q_sm + (size_t)h * a.q_sh + col * 8);
  }
  {
    const u16* kb = (pre ? a.k_pre : a.k_suf) + (size_t)g * (pre ? a.pre_sh : a.suf_sh);
    const size_t ksl = pre ? a.pre_sl : a.suf_sl;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = lane + 64 * i, row = c / RCH, col = c % RCH;
      int kr = tt * 32 + row;
      if (kr > len - 1) kr = len - 1;  // masked below; keeps the address valid and the value finite
      kreg[i] = *(const i32x4*)(kb + (size_t)kr * ksl + col * 8);
    }
  }
  // per-key visibility of the prefix (always requested, from a harmless address when unused)
  const bool use_pad = pre && a.mask2d == nullptr && a.pad != nullptr;
  const int key = tt * 32 + l32;
  const int padv = *((use_pad && key < a.P) ? a.pad + key : (const uint8_t*)a.q);
  const int pad_ok = use_pad ? (key < a.P ? padv : 0) : 1;
  // per-(query, key) visibility bytes of the tile (prefill): eight consecutive keys per word, the keys of
  // this lane's registers 0..7 and 8..15
  const bool use_m2 = pre && a.mask2d != nullptr;
  const uint8_t* mp = use_m2 ? a.mask2d + (size_t)(q_ok ? qi : a.M - 1) * a.mask_ld + tt * 32 + 8 * half : (const uint8_t*)a.q;
  const unsigned long long m2lo = *(const unsigned long long*)mp;
  const unsigned long long m2hi = *(const unsigned long long*)(mp + (use_m2 ? 16 : 8));
  // V^T: D rows x (NWV key tiles x 4 chunks), dealt to all threads; tiles past the range read a valid
  // tile (their P^T is zero)
#pragma unroll
  for (int i = 0; i < VCH; ++i) {
    const int c = tid + i * NWV * 64, row = c / (NWV * 4), col = c % (NWV * 4);
    const int j = col >> 2;
    const int tj = j < nt ? j : nt - 1;
    const bool pj = tj < tp;
    const int ttj = pj ? tj : tj - tp;
    const u16* vb = (pj ? a.vt_pre : a.vt_suf) + (size_t)g * (pj ? a.pre_vt_sh : a.suf_vt_sh) + (size_t)row * (pj ? a.pre_vt_sd : a.suf_vt_sd);
    vreg[i] = *(const i32x4*)(vb + ttj * 32 + (col & 3) * 8);
  }
  // keep the V^T requests above the first product: sunk below it they would leave a round trip later
  __builtin_amdgcn_sched_barrier(0);

  if (tid < 32 * RCH) *(i32x4*)(qs + (tid / RCH) * QPITCH + (tid % RCH) * 16) = qreg;
#pragma unroll
  for (int i = 0; i < KCH; ++i) {
    const int c = lane + 64 * i;
    *(i32x4*)(ks + key_of_row(c / RCH) * QPITCH + (c % RCH) * 16) = kreg[i];  // MFMA row r holds key key_of_row(r)
  }
  lds_only_barrier();  // the Q tile is complete (the K tile is this wave's own)

  // ---- S^T tile = K . Q^T (one query column per lane) ----
  f32x16 sT;
#pragma unroll
  for (int i = 0; i < 16; ++i) sT[i] = 0.f;
  {
    i32x4 ka[DS], qb[DS];
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int off = l32 * QPITCH + (16 * s + 8 * half) * 2;
      ka[s] = *(const i32x4*)(ks + off);
      qb[s] = *(const i32x4*)(qs + off);
    }
#pragma unroll
    for (int s = 0; s < DS; ++s) sT = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(ka[s]), as_bf16x8(qb[s]), sT, 0, 0, 0);
  }

  // ---- scale and mask.  Register i of this lane holds key 16*(i/8) + 8*half + i%8 of the tile;
  // visibility and range become two 16-bit masks (bit i = register i) ----
  unsigned vbits, ibits;
  {
    const int k0 = tt * 32 + 8 * half;
    const int left = len - k0;
    const unsigned lo8 = left >= 8 ? 0xffu : (left > 0 ? (1u << left) - 1u : 0u);
    const unsigned hi8 = left >= 24 ? 0xffu : (left > 16 ? (1u << (left - 16)) - 1u : 0u);
    ibits = active ? (lo8 | (hi8 << 8)) : 0u;
    if (!pre) {
      if (a.mask_mode == 1) {
        vbits = 0xffffu;
      } else {  // causal among the suffix tokens: key <= query
        const int c = qi - k0 + 1;
        const unsigned cl = c >= 8 ? 0xffu : (c > 0 ? (1u << c) - 1u : 0u);
        const unsigned ch = c >= 24 ? 0xffu : (c > 16 ? (1u << (c - 16)) - 1u : 0u);
        vbits = cl | (ch << 8);
      }
    } else if (a.mask2d) {
      // one byte (0 or 1) per key: gather bit 0 of the 8 bytes of each word
      const unsigned long long gather = 0x0102040810204080ull, ones = 0x0101010101010101ull;
      vbits = (unsigned)(((m2lo & ones) * gather) >> 56) | ((unsigned)(((m2hi & ones) * gather) >> 56) << 8);
    } else {
      const unsigned pmask = (unsigned)__ballot(pad_ok != 0);  // lanes 0..31: keys of this tile
      vbits = ((pmask >> (8 * half)) & 0xffu) | (((pmask >> (16 + 8 * half)) & 0xffu) << 8);
    }
  }
  const bool lb = a.logits_bf16 != 0;
  float p[16];
  float tmax = -INFINITY;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    float sv = sT[i];
    sv = lb ? round_bf16(sv) : sv;
    sv *= a.scale;
    const float masked = lb ? sv + kOpenpiMask : kF32Min;
    sv = (vbits >> i) & 1u ? sv : masked;
    sv = (ibits >> i) & 1u ? sv : -INFINITY;
    p[i] = sv;
    tmax = fmaxf(tmax, sv);
  }
  tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
  if (half == 0) st_m[wave][l32] = tmax;
  lds_only_barrier();
  float bm = st_m[0][l32];  // tile 0 always has a key in range: finite
#pragma unroll
  for (int w = 1; w < NWV; ++w) bm = fmaxf(bm, st_m[w][l32]);
  float lsum = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    p[i] = __expf(p[i] - bm);  // out-of-range keys give 0
    lsum += p[i];
  }
  lsum += __shfl_xor(lsum, 32);
  if (half == 0) st_l[wave][l32] = lsum;
  pt[wave][0][lane] = pack8(p);
  pt[wave][1][lane] = pack8(p + 8);
#pragma unroll
  for (int i = 0; i < VCH; ++i) {
    const int c = tid + i * NWV * 64;
    *(i32x4*)(vs + (c / (NWV * 4)) * VPITCH + (c % (NWV * 4)) * 16) = vreg[i];
  }
  lds_only_barrier();
  if (wave >= DT) return;

  // ---- O^T rows [32w, 32w + 32) = V^T . P^T over every key tile ----
  float bl = st_l[0][l32];
#pragma unroll
  for (int w = 1; w < NWV; ++w) bl += st_l[w][l32];
  i32x4 pb[NWV][2], vf[NWV][2];
#pragma unroll
  for (int j = 0; j < NWV; ++j)
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      pb[j][s] = pt[j][s][lane];
      vf[j][s] = *(const i32x4*)(vs + (32 * wave + l32) * VPITCH + (32 * j + 16 * s + 8 * half) * 2);
    }
  f32x16 o;
#pragma unroll
  for (int i = 0; i < 16; ++i) o[i] = 0.f;
#pragma unroll
  for (int j = 0; j < NWV; ++j)
#pragma unroll
    for (int s = 0; s < 2; ++s) o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vf[j][s]), as_bf16x8(pb[j][s]), o, 0, 0, 0);

  // this lane's output: query qi, columns 32w + 8g4 + 4*half + 0..3 for the four register groups g4
  if (q_ok) {
    u16* op = a.out + (size_t)qi * a.out_sm + (size_t)h * D + 32 * wave + 4 * half;
    const float inv = 1.0f / bl;
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const f32x4 v = {o[4 * g4], o[4 * g4 + 1], o[4 * g4 + 2], o[4 * g4 + 3]};
      *(i32x2*)(op + 8 * g4) = pack_bf16x4(v * inv);
    }
  }
}

// Cross layers of the SmolVLA action expert: the same exchange of probabilities, with the query tile
// computed in the launch (RMSNorm of the 32 hidden rows, projection with this head's 64 columns of the
// packed bf16 q weight -- k tiles dealt to the waves, fixed-order reduction through LDS -- and the rotary
// embedding) while the K / V^T loads are in flight, and with fp32 K / V given as bf16 hi + lo planes
// (x = hi + lo to 16 mantissa bits): S^T = (K_hi + K_lo) . Q^T, O^T = V_hi . P_hi + V_lo . P_hi + V_hi . P_lo.
// Prefix keys only (at most 8 key tiles), grid (head, query tile), 8 waves.
constexpr int kCrossWaves = 8;
constexpr int kCrossMaxK = 768;                        // widest hidden size the projection stages (SmolVLA expert: 720)
constexpr int kXPitch = kCrossMaxK * 2 + 16;           // staged hidden rows (bf16)
constexpr int kQPitch = 64 * 2 + 16;                   // staged Q / K rows
constexpr int kVPitch = kCrossWaves * 64 + 16;         // staged V^T rows (8 tiles x 32 keys)
constexpr int kKTile = 32 * kQPitch;                   // one staged K tile (one plane)
constexpr int kVPlane = 64 * kVPitch;                  // one staged V^T plane
constexpr int kPtPlane = kCrossWaves * 2 * 64 * 16;    // P^T operands of every key tile (one plane)
constexpr int kRedBytes = 2 * kCrossWaves * 4 * 64 * 16;  // the projection's partial tiles of every wave
// region A: hidden rows, later the K tiles, later the P^T operands; region B: projection partials, later V^T
constexpr int kRegionA = 2 * kCrossWaves * kKTile;
constexpr int kRegionB = 2 * kVPlane;
constexpr int kCrossLds = kRegionA + kRegionB + kKTile;
static_assert(32 * kXPitch <= kRegionA && 2 * kPtPlane <= kRegionA && kRedBytes <= kRegionB, "aliased regions must fit");

__global__ __launch_bounds__(kCrossWaves * 64) void expert_cross_px_kernel(AttnArgs a) {
  constexpr int D = 64, NWV = kCrossWaves, DS = 4, DT = 2;
  __shared__ float st_m[NWV][32], st_l[NWV][32];
  extern __shared__ __align__(16) unsigned char lds[];
  unsigned char* const xs = lds;                                       // region A
  unsigned char* const qs = lds + kRegionA + kRegionB;
  f32x4(*const red)[NWV][4][64] = (f32x4(*)[NWV][4][64])(lds + kRegionA);  // region B

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int h = blockIdx.x;
  const int mtile = blockIdx.y;
  const int g = (h * a.gqa_mul) >> 16;
  const int nt = (a.P + 31) >> 5;  // key tiles, 1..8
  const int qi = mtile * 32 + l32;
  const bool q_ok = qi < a.M;
  const bool active = wave < nt;
  unsigned char* const ks = lds + (size_t)wave * 2 * kKTile;           // this wave's K tile: hi plane, then lo

  // the rotary position of this lane's query row: asked for before anything else, so that its table rows can be
  // requested with the other operands below instead of two round trips after the projection
  int qpos = a.qp_rope_pos[qi < a.M ? qi : a.M - 1];
  // ---- requests in the order of use (memory returns in order): the block's 32 hidden rows and the norm weight
  // (16 threads per row, a thread's pieces requested together and kept in registers), the projection's weights,
  // then K / V^T (whole rows, lane -> consecutive chunks) ----
  constexpr int TPR = NWV * 2, XP = kCrossMaxK / 8 / TPR;  // threads per row, 16-byte pieces per thread
  const int xr = tid / TPR, xq = tid % TPR;
  const int xm = mtile * 32 + xr;
  const u16* xrow = a.qp_x + (size_t)(xm < a.M ? xm : a.M - 1) * a.qp_ldx;
  const int npieces = a.qp_K / 8;
  i32x4 xpc[XP], nwp[XP];
#pragma unroll
  for (int i = 0; i < XP; ++i) {
    const int p = xq + TPR * i;
    const int pc = p < npieces ? p : npieces - 1;  // past the row: a valid piece, not used
    xpc[i] = *(const i32x4*)(xrow + 8 * pc);
    nwp[i] = *(const i32x4*)(a.qp_norm_w + 8 * pc);
  }
  __builtin_amdgcn_sched_barrier(0);
  // this wave's weight tiles of the head's strip (packed n tiles 2h, 2h+1): k tiles wave, wave + 8, wave + 16
  constexpr int KPW = (kCrossMaxK / 32 + NWV - 1) / NWV;
  i32x4 wfr[KPW][2][2];
  {
    const uint8_t* wq = a.qp_w + ((size_t)(2 * h) * a.qp_KT) * 2048 + lane * 16;
#pragma unroll
    for (int i = 0; i < KPW; ++i) {
      int kt = wave + NWV * i;
      if (kt > a.qp_KT - 1) kt = a.qp_KT - 1;
#pragma unroll
      for (int n2 = 0; n2 < 2; ++n2)
#pragma unroll
        for (int c = 0; c < 2; ++c) wfr[i][n2][c] = *(const i32x4*)(wq + ((size_t)n2 * a.qp_KT + kt) * 2048 + c * 1024);
    }
  }
  const int tt = active ? wave : nt - 1;  // idle waves read a valid tile and drop it
  i32x4 kreg[2][4], vreg[2][4];
  {
    const size_t goff = (size_t)g * a.pre_sh;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = lane + 64 * i, row = c >> 3, col = c & 7;
      int kr = tt * 32 + row;
      if (kr > a.P - 1) kr = a.P - 1;  // masked below; keeps the address valid and the value finite
      const size_t off = (size_t)kr * a.pre_sl + goff + col * 8;
      kreg[0][i] = *(const i32x4*)(a.k_pre + off);
      kreg[1][i] = *(const i32x4*)(a.k_pre_lo + off);
    }
  }
  const int key = tt * 32 + l32;
  const int padv = *((a.pad != nullptr && key < a.P) ? a.pad + key : (const uint8_t*)a.qp_x);
  const int pad_ok = a.pad != nullptr ? (key < a.P ? padv : 0) : 1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + i * NWV * 64, row = c >> 5, col = c & 31;  // 32 chunks per V^T row: 8 tiles x 4
    const int j = col >> 2;
    const int tj = j < nt ? j : nt - 1;  // tiles past the range: a valid address, P^T is zero there
    const size_t off = (size_t)g * a.pre_vt_sh + (size_t)row * a.pre_vt_sd + tj * 32 + (col & 3) * 8;
    vreg[0][i] = *(const i32x4*)(a.vt_pre + off);
    vreg[1][i] = *(const i32x4*)(a.vt_pre_lo + off);
  }
  // the rotary table rows of the query (the lanes of waves 0..3 finish the projection: four consecutive columns
  // 8 wave + 4 half .. of both halves of the head)
  qpos = qpos < 0 ? 0 : (qpos > a.qp_positions - 1 ? a.qp_positions - 1 : qpos);
  const int rfi = 8 * (wave & 3) + 4 * half;
  const f32x4 rcs = *(const f32x4*)(a.qp_cos + (size_t)qpos * (D / 2) + rfi);
  const f32x4 rsn = *(const f32x4*)(a.qp_sin + (size_t)qpos * (D / 2) + rfi);
  __builtin_amdgcn_sched_barrier(0);

  // ---- the query tile: 1 / rms of its rows, normalised rows into LDS as bf16(w * bf16(x * rstd)), columns from K
  // to the end of the last k tile zero ----
  {
    float ss0 = 0.f, ss1 = 0.f;
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      if (xq + TPR * i < npieces) {
        union { i32x4 v; bf16x2 hh[4]; } xu;
        xu.v = xpc[i];
        ss0 = __builtin_amdgcn_fdot2_f32_bf16(xu.hh[0], xu.hh[0], ss0, false);
        ss1 = __builtin_amdgcn_fdot2_f32_bf16(xu.hh[1], xu.hh[1], ss1, false);
        ss0 = __builtin_amdgcn_fdot2_f32_bf16(xu.hh[2], xu.hh[2], ss0, false);
        ss1 = __builtin_amdgcn_fdot2_f32_bf16(xu.hh[3], xu.hh[3], ss1, false);
      }
    }
    float ss = ss0 + ss1;
#pragma unroll
    for (int o2 = TPR / 2; o2 > 0; o2 >>= 1) ss += __shfl_xor(ss, o2);
    const float rstd = rsqrtf(ss / (float)a.qp_K + a.qp_eps);
    const int kpieces = a.qp_KT * 4;
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      const int p = xq + TPR * i;
      if (p < kpieces) {
        union { i32x4 v; unsigned u[4]; } xu, nw, o4;
        o4.v = i32x4{0, 0, 0, 0};
        if (p < npieces) {
          xu.v = xpc[i];
          nw.v = nwp[i];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const unsigned u = pack_bf16x2(__uint_as_float(xu.u[e] << 16) * rstd, __uint_as_float(xu.u[e] & 0xffff0000u) * rstd);
            o4.u[e] = pack_bf16x2(__uint_as_float(nw.u[e] << 16) * __uint_as_float(u << 16),
                                  __uint_as_float(nw.u[e] & 0xffff0000u) * __uint_as_float(u & 0xffff0000u));
          }
        }
        *(i32x4*)(xs + xr * kXPitch + p * 16) = o4.v;
      }
    }
  }
  lds_only_barrier();
  {
    f32x16 qacc[2];
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2)
#pragma unroll
      for (int i = 0; i < 16; ++i) qacc[n2][i] = 0.f;
#pragma unroll
    for (int i = 0; i < KPW; ++i) {
      const int kt = wave + NWV * i;
      if (kt < a.qp_KT) {  // wave-uniform
        const i32x4* xp = (const i32x4*)(xs + l32 * kXPitch + (kt * 32 + 16 * half) * 2);
        const i32x4 xa0 = xp[0], xa1 = xp[1];
#pragma unroll
        for (int n2 = 0; n2 < 2; ++n2) {
          qacc[n2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(wfr[i][n2][0]), as_bf16x8(xa0), qacc[n2], 0, 0, 0);
          qacc[n2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(wfr[i][n2][1]), as_bf16x8(xa1), qacc[n2], 0, 0, 0);
        }
      }
    }
    // fixed-order reduction over the waves; waves 0..3 own register group w (query row l32, four
    // consecutive columns 8w + 4*half .. of both tiles = a rotary pair (c, c + 32))
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const f32x4 v = {qacc[n2][4 * gq], qacc[n2][4 * gq + 1], qacc[n2][4 * gq + 2], qacc[n2][4 * gq + 3]};
        red[n2][wave][gq][lane] = v;
      }
  }
  lds_only_barrier();
  if (wave < 4) {
    f32x4 sum[2];
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2) {
      sum[n2] = red[n2][0][wave][lane];
#pragma unroll
      for (int w = 1; w < NWV; ++w) sum[n2] += red[n2][w][wave][lane];
    }
    const int fi = rfi;  // first of this lane's four columns within the half head
    const f32x4 cs = rcs, sn = rsn;
    const f32x4 va = unpack_bf16x4(pack_bf16x4(sum[0])), vb = unpack_bf16x4(pack_bf16x4(sum[1]));
    f32x4 ra, rb;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // separately rounded products, as an elementwise fp32 implementation computes them
      ra[j] = sub_rn(mul_rn(va[j], cs[j]), mul_rn(vb[j], sn[j]));
      rb[j] = add_rn(mul_rn(vb[j], cs[j]), mul_rn(va[j], sn[j]));
    }
    *(i32x2*)(qs + l32 * kQPitch + fi * 2) = pack_bf16x4(ra);
    *(i32x2*)(qs + l32 * kQPitch + (D / 2 + fi) * 2) = pack_bf16x4(rb);
  }
  // K tiles over the hidden rows, V^T over the projection partials: every wave is past its reads of both
  // once the query tile is complete
  lds_only_barrier();
#pragma unroll
  for (int pl = 0; pl < 2; ++pl) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = lane + 64 * i;
      *(i32x4*)(ks + pl * kKTile + key_of_row(c >> 3) * kQPitch + (c & 7) * 16) = kreg[pl][i];  // MFMA row r holds key key_of_row(r)
      const int cv = tid + i * NWV * 64;
      *(i32x4*)(lds + kRegionA + pl * kVPlane + (cv >> 5) * kVPitch + (cv & 31) * 16) = vreg[pl][i];
    }
  }

  // ---- S^T tile = (K_hi + K_lo) . Q^T (one query column per lane) ----
  f32x16 sT;
#pragma unroll
  for (int i = 0; i < 16; ++i) sT[i] = 0.f;
  {
    i32x4 kh[DS], kl[DS], qb[DS];
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int off = l32 * kQPitch + (16 * s + 8 * half) * 2;
      kh[s] = *(const i32x4*)(ks + off);
      kl[s] = *(const i32x4*)(ks + kKTile + off);
      qb[s] = *(const i32x4*)(qs + off);
    }
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      sT = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kh[s]), as_bf16x8(qb[s]), sT, 0, 0, 0);
      sT = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kl[s]), as_bf16x8(qb[s]), sT, 0, 0, 0);
    }
  }
  // register i of this lane holds key 16*(i/8) + 8*half + i%8 of the tile
  unsigned vbits, ibits;
  {
    const int k0 = tt * 32 + 8 * half;
    const int left = a.P - k0;
    const unsigned lo8 = left >= 8 ? 0xffu : (left > 0 ? (1u << left) - 1u : 0u);
    const unsigned hi8 = left >= 24 ? 0xffu : (left > 16 ? (1u << (left - 16)) - 1u : 0u);
    ibits = active ? (lo8 | (hi8 << 8)) : 0u;
    const unsigned pmask = (unsigned)__ballot(pad_ok != 0);  // lanes 0..31: keys of this tile
    vbits = ((pmask >> (8 * half)) & 0xffu) | (((pmask >> (16 + 8 * half)) & 0xffu) << 8);
  }
  float p[16];
  float tmax = -INFINITY;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    float sv = sT[i] * a.scale;
    sv = (vbits >> i) & 1u ? sv : kF32Min;
    sv = (ibits >> i) & 1u ? sv : -INFINITY;
    p[i] = sv;
    tmax = fmaxf(tmax, sv);
  }
  tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
  if (half == 0) st_m[wave][l32] = tmax;
  lds_only_barrier();  // (every wave is past its K tile: the P^T operands go over them)
  float bm = st_m[0][l32];  // tile 0 always has a key in range: finite
#pragma unroll
  for (int w = 1; w < NWV; ++w) bm = fmaxf(bm, st_m[w][l32]);
  float lsum = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    p[i] = __expf(p[i] - bm);  // out-of-range keys give 0
    lsum += p[i];
  }
  lsum += __shfl_xor(lsum, 32);
  if (half == 0) st_l[wave][l32] = lsum;
  i32x4(*const pt)[NWV][2][64] = (i32x4(*)[NWV][2][64])lds;  // [plane][tile][k step][lane], region A
  {
    float lo[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) lo[i] = p[i] - round_bf16(p[i]);
    pt[0][wave][0][lane] = pack8(p);
    pt[0][wave][1][lane] = pack8(p + 8);
    pt[1][wave][0][lane] = pack8(lo);
    pt[1][wave][1][lane] = pack8(lo + 8);
  }
  lds_only_barrier();
  if (wave >= DT) return;

  // ---- O^T rows [32w, 32w + 32) = V_hi . P_hi + V_lo . P_hi + V_hi . P_lo over every key tile ----
  float bl = st_l[0][l32];
#pragma unroll
  for (int w = 1; w < NWV; ++w) bl += st_l[w][l32];
  f32x16 o;
#pragma unroll
  for (int i = 0; i < 16; ++i) o[i] = 0.f;
  const unsigned char* const vrow = lds + kRegionA + (32 * wave + l32) * kVPitch + 8 * half * 2;
#pragma unroll
  for (int j0 = 0; j0 < NWV; j0 += 4) {
    i32x4 vh[4][2], vl[4][2], ph[4][2], pl[4][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        vh[j][s] = *(const i32x4*)(vrow + (32 * (j0 + j) + 16 * s) * 2);
        vl[j][s] = *(const i32x4*)(vrow + kVPlane + (32 * (j0 + j) + 16 * s) * 2);
        ph[j][s] = pt[0][j0 + j][s][lane];
        pl[j][s] = pt[1][j0 + j][s][lane];
      }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vh[j][s]), as_bf16x8(ph[j][s]), o, 0, 0, 0);
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vl[j][s]), as_bf16x8(ph[j][s]), o, 0, 0, 0);
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vh[j][s]), as_bf16x8(pl[j][s]), o, 0, 0, 0);
      }
  }
  if (q_ok) {
    u16* op = a.out + (size_t)qi * a.out_sm + (size_t)h * D + 32 * wave + 4 * half;
    const float inv = 1.0f / bl;
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const f32x4 v = {o[4 * g4], o[4 * g4 + 1], o[4 * g4 + 2], o[4 * g4 + 3]};
      *(i32x2*)(op + 8 * g4) = pack_bf16x4(v * inv);
    }
  }
}

template <int NWV>
int launch_px(const AttnArgs& a, hipStream_t st) {
  hipLaunchKernelGGL((expert_attn_px_kernel<64, NWV>), dim3(a.H, (a.M + 31) / 32), dim3(NWV * 64), 0, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace

int tk_attn_px_max_tiles() { return 12; }

// head size 64, bf16 K/V (no hi/lo planes), one problem, at most 12 key tiles
int tk_launch_attn_px(AttnArgs a, int D, hipStream_t st) {
  const int nt = (a.P + 31) / 32 + (a.S + 31) / 32;
  if (D != 64 || a.k_pre_lo || a.batch > 0 || nt < 1 || nt > 12) return -1;
  if (nt <= 4) return launch_px<4>(a, st);
  if (nt <= 8) return launch_px<8>(a, st);
  return launch_px<12>(a, st);
}

// cross layers: hi / lo prefix K and V^T planes, head size 64, at most 8 key tiles, query projection in the launch
int tk_launch_attn_cross_px(AttnArgs a, hipStream_t st) {
  if (!a.k_pre_lo || !a.vt_pre_lo || !a.qp_x || a.P < 1 || (a.P + 31) / 32 > kCrossWaves || a.qp_K > kCrossMaxK) return -1;
  // more LDS than a launch gets by default: raise the kernel's limit once per process
  static int raised = 0;
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&expert_cross_px_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kCrossLds) != hipSuccess)
      return -3;
    raised = 1;
  }
  hipLaunchKernelGGL(expert_cross_px_kernel, dim3(a.H, (a.M + 31) / 32), dim3(kCrossWaves * 64), kCrossLds, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
