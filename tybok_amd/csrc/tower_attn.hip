// Unmasked self-attention of the vision towers on gfx950 (many query tiles per head, long key
// ranges):  out[b, m, h*D + d] = softmax(q . K^T * scale) . V  per (problem b, head h).
//
// A block owns 128 queries of one (problem, head) pair.  Its eight waves form two groups of four:
// group g walks half g of the key range in stages of 64 keys, and within a group each wave owns one
// 32-query tile.  A stage's K rows and V^T rows are fetched from global memory once per group
// (16-byte coalesced loads, one stage ahead, in registers), parked in a double-buffered LDS tile
// and read back by the group's waves in MFMA operand order -- a key or value byte crosses the
// L2 -> CU path once per 128 queries.  Two waves per SIMD: one's MFMAs run under the other's
// softmax arithmetic, which is what bounds this kernel.  Waves meet at one barrier per stage; each
// keeps the running max / sum / accumulator of its own queries and key half (online softmax,
// fp32), and the two halves of a query tile are merged once, through LDS, at the end.
//
// Orientation as in the expert attention kernel: S^T = K . Q^T puts one query per lane (max and sum
// are in-lane plus one cross-half exchange) and makes the probabilities the B operand of
// O^T += V^T . P^T without a transpose.  The accumulator is only rescaled when some lane's running
// max actually moved (wave-uniform test); after the first stages that is rare.
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

constexpr int kGroups = 2;   // key halves
constexpr int kStageKeys = 64;
// QT: query tiles (waves) per key-half group.  4: 128 queries a block, two blocks per CU.  5: 160 queries a block of
// ten waves, one block per CU (three waves on two of the SIMDs) -- for grids that four-tile blocks would spread as
// "one block on most CUs, two on some": the doubly loaded CUs then run four waves per SIMD and set the launch's
// duration (3 cameras x 12 heads x 1024 queries: 288 blocks on 256 CUs; 252 blocks of five tiles fit one per CU).

// S^T rows are dealt to keys so that accumulator register i of lane half `hf` holds key
// 16*(i/8) + 8*hf + i%8 of the tile: registers 8s..8s+7 are then the B operand of k step s.
__device__ __forceinline__ int key_of_row(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

// eight fp32 -> one 16-byte matrix operand of the kernel's flavour (bf16 or fp16), round to nearest even
template <bool F16>
__device__ __forceinline__ i32x4 pack8(const float* v) {
  i32x4 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = (int)(F16 ? pack_f16x2(v[2 * j], v[2 * j + 1]) : pack_bf16x2(v[2 * j], v[2 * j + 1]));
  return r;
}
// one 32 x 32 x 16 product with the operands read as bf16 or as fp16
template <bool F16>
__device__ __forceinline__ f32x16 mma16(i32x4 a, i32x4 b, f32x16 c) {
  if (F16) return __builtin_amdgcn_mfma_f32_32x32x16_f16(as_f16x8(a), as_f16x8(b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}

// max / sum of a value over the two lanes that share a query (lane l and l ^ 32), without an LDS trip:
// v_permlane32_swap hands each half the other half's registers
__device__ __forceinline__ float other_half_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float other_half_sum(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ void stage_barrier() {
  // LDS-only: the global prefetch of the next stage stays in flight across it
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int D, int QT>
struct TowerLds {
  static constexpr int KP = D * 2 + 16;             // pitch of a K row (bytes): rows 16 apart share banks, nothing closer
  static constexpr int VP = kStageKeys * 2 + 16;    // pitch of a V^T row
  static constexpr int KBYTES = kStageKeys * KP, VBYTES = D * VP;
  static constexpr int GROUP = 2 * (KBYTES + VBYTES);  // a group's double buffer; later its merge record
  static constexpr int TOTAL = kGroups * GROUP;
  static constexpr int MERGE_WAVE = (2 + (D / 32) * 16) * 64 * 4;  // m, l and O^T of one wave
  // the merge record lies in the second group's staging area and, if it is longer, runs back into the first one's
  // (every wave of the block is past its last staging read by then)
  static constexpr int MERGE_OFF = QT * MERGE_WAVE <= GROUP ? GROUP : TOTAL - QT * MERGE_WAVE;
  static_assert(QT * MERGE_WAVE <= TOTAL, "the merge record must fit the staging areas");
};

// LB: the logits are rounded to bf16 before the scale and the softmax (what a bf16 matmul hands to a
// fp32 softmax); otherwise they stay fp32.
// F16: q, K, V^T are fp16 and the probabilities are rounded to fp16 for P.V (both products on the fp16 matrix
// instruction); the output stays bf16.
// QT: query tiles per block (each group of QT waves walks one half of the keys): 4, 5 where four-tile blocks would put two
// blocks on some CUs and one on the rest, 2 where four-tile blocks would leave more than half of the CUs idle (pi0.5's
// tower: 2 x 256 tokens, 16 heads: 64 -> 128 blocks, 9.9 -> 7.0 us; one 1024-token camera: 17.9 -> 13.3 us); a wave's
// arithmetic does not depend on it, so every form gives the same bits.
// WPE: waves per SIMD the registers are budgeted for -- 4 lets two four-tile blocks of head size 64 share a CU (128
// registers per lane, a few of them spilled); 2 / 3 when the grid puts one block on a CU anyway.
template <int D, bool LB, bool F16, int QT, int WPE>
__global__ __launch_bounds__(QT * kGroups * 64, WPE) void tower_attn_kernel(AttnArgs a, int qblocks) {
  using L = TowerLds<D, QT>;
  constexpr int kQTiles = QT, kGroupThreads = QT * 64;
  constexpr int DS = D / 16;            // k steps of Q.K^T
  constexpr int DT = D / 32;            // 32-row tiles of O^T
  constexpr int KT = kStageKeys / 32;   // key tiles per stage
  constexpr int KP = L::KP, VP = L::VP, KBYTES = L::KBYTES, VBYTES = L::VBYTES;
  constexpr int KCH = D / 8;            // 16-byte chunks per K row
  constexpr int NCHUNK = kStageKeys * KCH;                              // 16-byte chunks of a stage, K and V^T alike
  constexpr int NLD = (NCHUNK + kGroupThreads - 1) / kGroupThreads;     // per thread and stage
  constexpr bool EVEN = NCHUNK % kGroupThreads == 0;                    // (five tiles: the last pass is partly empty)
  extern __shared__ __align__(16) unsigned char lds_all[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, l32 = lane & 31, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave / kQTiles, qt = wave % kQTiles;
  const int gtid = (kGroupThreads & (kGroupThreads - 1)) == 0 ? (tid & (kGroupThreads - 1)) : tid - grp * kGroupThreads;
  unsigned char* lds = lds_all + grp * L::GROUP;
  // 1-D grid dealt round-robin to the 8 XCDs: XCD x takes the x-th eighth of the (pair, query block) list in pair-major
  // order, so the query blocks of one (problem, head) pair run on one XCD (two where the pair straddles a boundary),
  // whose L2 then holds that pair's K / V^T for all of them, and every XCD gets the same number of blocks
  const int total = a.batch * a.H * qblocks, per_xcd = (total + 7) / 8;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int item = xcd * per_xcd + slot;
  if (slot >= per_xcd || item >= total) return;
  const int pair = item / qblocks;
  const int qb = item % qblocks;
  const int bi = pair / a.H, h = pair % a.H;
  const int g = (h * a.gqa_mul) >> 16;
  const u16* qp = a.q + (long long)bi * a.q_sb + (size_t)h * a.q_sh;
  const u16* kp = a.k_pre + (long long)bi * a.k_sb + (size_t)g * a.pre_sh;
  const u16* vp = a.vt_pre + (long long)bi * a.vt_sb + (size_t)g * a.pre_vt_sh;
  u16* op = a.out + (long long)bi * a.out_sb + (size_t)h * D;

  // stages of this group: the first group takes the extra one of an odd count (the host guarantees
  // at least two stages, so neither group is empty)
  const int nstages = (a.P + kStageKeys - 1) / kStageKeys;
  const int n0 = (nstages + 1) / 2;
  const int s_lo = grp ? n0 : 0;
  const int s_n = grp ? nstages - n0 : n0;
  const int qi = (qb * kQTiles + qt) * 32 + l32;
  const bool q_ok = qi < a.M;

  // this thread's staging chunks: K chunk c -> (key c / KCH, columns 8 * (c % KCH));
  // V^T chunk c -> (row d = c / 8, keys 8 * (c % 8))
  i32x4 kreg[NLD], vreg[NLD];
  auto gload = [&](int s) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      int c = gtid + i * kGroupThreads;
      if (!EVEN && c > NCHUNK - 1) c = NCHUNK - 1;  // loaded again, not stored
      int key = s * kStageKeys + c / KCH;
      if (key > a.P - 1) key = a.P - 1;  // rows past the end are masked below; keep the address valid
      kreg[i] = *(const i32x4*)(kp + (size_t)key * a.pre_sl + (c % KCH) * 8);
      // V^T rows are zero padded up to the next multiple of 32 keys; a stage may reach 32 further
      int k0 = s * kStageKeys + (c % 8) * 8;
      const int vmax = ((a.P + 31) & ~31) - 8;
      if (k0 > vmax) k0 = vmax;  // a fully masked key tile: its probabilities are exactly zero
      vreg[i] = *(const i32x4*)(vp + (size_t)(c / 8) * a.pre_vt_sd + k0);
    }
  };
  auto lstore = [&](int buf) {
    unsigned char* kb = lds + buf * (KBYTES + VBYTES);
    unsigned char* vb = kb + KBYTES;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int c = gtid + i * kGroupThreads;
      if (!EVEN && c >= NCHUNK) continue;
      *(i32x4*)(kb + (c / KCH) * KP + (c % KCH) * 16) = kreg[i];
      *(i32x4*)(vb + (c / 8) * VP + (c % 8) * 16) = vreg[i];
    }
  };

  gload(s_lo);
  // Q^T operands of this wave's tile: lane (query l32, half) holds columns 16 s + 8 half .. + 8
  i32x4 qf[DS];
  {
    const u16* qrow = qp + (size_t)(q_ok ? qi : a.M - 1) * a.q_sm;
#pragma unroll
    for (int s = 0; s < DS; ++s) qf[s] = *(const i32x4*)(qrow + 16 * s + 8 * half);
  }
  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  // exp(x * scale - m) = exp2(x * scale * log2(e) - m * log2(e)): the running max is kept in that unit.
  // The scale is positive, so the max is taken over the unscaled logits and scaled once.
  const float scale2 = a.scale * 1.4426950408889634f;
  float m_run = -INFINITY, l_run = 0.f;
  const int krow = key_of_row(l32);

  lstore(0);
  stage_barrier();
  for (int it = 0; it < n0; ++it) {  // block-uniform trip count; the second group may sit out the last pass
    const int buf = it & 1;
    if (it < s_n) {  // wave-uniform
      const int s = s_lo + it;
      if (it + 1 < s_n) gload(s + 1);
      const unsigned char* kb = lds + buf * (KBYTES + VBYTES);
      const unsigned char* vb = kb + KBYTES;
      // ---- S^T = K . Q^T for both 32-key tiles of the stage (two independent MFMA chains) ----
      f32x16 sT[KT];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sT[kt][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < DS; ++ks)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
          const i32x4 kop = *(const i32x4*)(kb + (kt * 32 + krow) * KP + (16 * ks + 8 * half) * 2);
          sT[kt] = mma16<F16>(kop, qf[ks], sT[kt]);
        }
      // ---- one online-softmax step over the stage's 64 keys, one query per lane; register i of tile
      //      kt = key 64 s + 32 kt + 16*(i/8) + 8*half + i%8 ----
      if ((s + 1) * kStageKeys > a.P) {
        // the last stage: keys past P (possibly its whole second tile) get probability exactly 0
        const int left = a.P - (s * kStageKeys + 8 * half);  // keys from this lane's first one on that exist
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int off = 32 * kt + 16 * (i >> 3) + (i & 7);
            sT[kt][i] = off < left ? sT[kt][i] : -INFINITY;
          }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          if (LB) {  // two roundings per conversion instruction
            const unsigned u = pack_bf16x2(sT[kt][i], sT[kt][i + 1]);
            sT[kt][i] = __uint_as_float(u << 16);
            sT[kt][i + 1] = __uint_as_float(u & 0xffff0000u);
          }
          tmax = fmaxf(tmax, fmaxf(sT[kt][i], sT[kt][i + 1]));
        }
      tmax = other_half_max(tmax) * scale2;
      if (__any(tmax > m_run)) {  // wave-uniform
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
        m_run = m_new;
      }
      float p[KT][16];
      float lsum0 = 0.f, lsum1 = 0.f;
      const float neg_m = -m_run;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          p[kt][i] = __builtin_amdgcn_exp2f(fmaf(sT[kt][i], scale2, neg_m));
          p[kt][i + 1] = __builtin_amdgcn_exp2f(fmaf(sT[kt][i + 1], scale2, neg_m));
          lsum0 += p[kt][i];
          lsum1 += p[kt][i + 1];
        }
      l_run += other_half_sum(lsum0 + lsum1);
      // ---- O^T += V^T . P^T (probabilities rounded to bf16, fp32 accumulation) ----
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const i32x4 pb = pack8<F16>(p[kt] + 8 * ks);
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const i32x4 vop = *(const i32x4*)(vb + (32 * dt + l32) * VP + (kt * 32 + 16 * ks + 8 * half) * 2);
            o[dt] = mma16<F16>(vop, pb, o[dt]);
          }
        }
      if (it + 1 < s_n) lstore(buf ^ 1);  // the other buffer: every wave of the group left it at the last barrier
    }
    stage_barrier();
  }

  // ---- merge the two key halves of each query tile: the second group hands (m, l, O^T) over through
  //      its staging area (all of its waves are past their last read of it: the barrier above) ----
  float* rec = (float*)(lds_all + L::MERGE_OFF + qt * L::MERGE_WAVE);
  if (grp == 1) {
    rec[lane] = m_run;
    rec[64 + lane] = l_run;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) rec[(2 + dt * 16 + i) * 64 + lane] = o[dt][i];
  }
  stage_barrier();
  if (grp == 0 && q_ok) {
    const float m1 = rec[lane], l1 = rec[64 + lane];
    const float m = fmaxf(m_run, m1);
    const float a0 = __builtin_amdgcn_exp2f(m_run - m), a1 = __builtin_amdgcn_exp2f(m1 - m);
    const float inv = 1.0f / (l_run * a0 + l1 * a1);
    const float c0 = a0 * inv, c1 = a1 * inv;
    // lane owns query column l32; register i of tile dt is row d = 32 dt + 8 (i/4) + 4 half + i%4
    u16* orow = op + (size_t)qi * a.out_sm;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = o[dt][4 * gq + e] * c0 + rec[(2 + dt * 16 + 4 * gq + e) * 64 + lane] * c1;
        *(i32x2*)(orow + 32 * dt + 8 * gq + 4 * half) = pack_bf16x4(v);
      }
  }
}

template <int D, bool LB, bool F16, int QT, int WPE>
int launch_tower_qt(const AttnArgs& a, hipStream_t st) {
  // more LDS than a launch gets by default: raise the kernel's limit once per process
  static int raised = 0;
  constexpr int lds_bytes = TowerLds<D, QT>::TOTAL;
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&tower_attn_kernel<D, LB, F16, QT, WPE>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            lds_bytes) != hipSuccess)
      return -3;
    raised = 1;
  }
  const int qblocks = (a.M + QT * 32 - 1) / (QT * 32);
  const int pairs = a.batch * a.H;
  dim3 grid(8 * ((pairs * qblocks + 7) / 8));
  hipLaunchKernelGGL((tower_attn_kernel<D, LB, F16, QT, WPE>), grid, dim3(QT * kGroups * 64), lds_bytes, st, a, qblocks);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <int D, bool LB, bool F16 = false>
int launch_tower(const AttnArgs& a, hipStream_t st, int cus) {
  if constexpr (D == 64 && !F16) {
    // one block per CU where the grid allows it: four-tile blocks with the whole register file to themselves, or
    // five-tile blocks where four-tile ones would double up on some CUs (see QT above); else two blocks per CU
    const int pairs = a.batch * a.H, tiles = (a.M + 31) / 32;
    const int b4 = pairs * ((tiles + 3) / 4), b5 = pairs * ((tiles + 4) / 5);
    if (2 * b4 <= cus && tiles >= 2) return launch_tower_qt<D, LB, F16, 2, 2>(a, st);  // few blocks: two-tile blocks on twice the CUs
    if (b4 <= cus) return launch_tower_qt<D, LB, F16, 4, 2>(a, st);
    if (b4 < 2 * cus && b5 <= cus) return launch_tower_qt<D, LB, F16, 5, 3>(a, st);
    return launch_tower_qt<D, LB, F16, 4, 4>(a, st);
  } else {
    const int pairs = a.batch * a.H, tiles = (a.M + 31) / 32;
    if (2 * pairs * ((tiles + 3) / 4) <= cus && tiles >= 2) return launch_tower_qt<D, LB, F16, 2, 2>(a, st);
    return launch_tower_qt<D, LB, F16, 4, 2>(a, st);
  }
}

// V [B, P, G, D] (d contiguous) -> V^T [B, G, D, ld] (keys contiguous), zero filled from P up to the end
// of its last 64-key tile (or ld): a block moves one 64-key x D tile of one (problem, kv head)
// through LDS -- 16-byte coalesced reads of the key rows, 16-byte coalesced writes of the d rows.
template <int D>
__global__ __launch_bounds__(256) void tower_vt_kernel(TransposeVArgs a) {
  constexpr int KCH = D / 8;
  constexpr int PITCH = D * 2 + 4;  // odd number of dwords: the column reads below touch every bank once
  constexpr int NCH = 64 * KCH / 256;
  __shared__ __align__(4) unsigned char tile[64 * PITCH];
  const int tid = threadIdx.x;
  const int key0 = blockIdx.x * 64, g = blockIdx.y, bi = blockIdx.z;
  const u16* v = a.v + (long long)bi * a.v_sb + (size_t)g * a.v_sh;
  u16* vt = a.vt + (long long)bi * a.vt_sb + (size_t)g * a.vt_sh;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = tid + i * 256;
    const int key = key0 + c / KCH;
    i32x4 x = {0, 0, 0, 0};
    if (key < a.P) x = *(const i32x4*)(v + (size_t)key * a.v_sl + (c % KCH) * 8);
    int* dst = (int*)(tile + (c / KCH) * PITCH + (c % KCH) * 16);
    dst[0] = x[0];
    dst[1] = x[1];
    dst[2] = x[2];
    dst[3] = x[3];
  }
  __syncthreads();
  // output chunk c -> (row d = c / 8, keys 8 * (c % 8) .. + 8)
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = tid + i * 256;
    const int d = c / 8, kc = c % 8;
    if (key0 + 8 * kc >= a.ld) continue;
    union { i32x4 q; u16 h[8]; } o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o.h[j] = *(const u16*)(tile + (8 * kc + j) * PITCH + d * 2);
    *(i32x4*)(vt + (size_t)d * a.vt_sd + key0 + 8 * kc) = o.q;
  }
}

}  // namespace

int tk_launch_transpose_v(TransposeVArgs a, int D, hipStream_t st) {
  dim3 grid((a.P + 63) / 64, a.G, a.B);
  if (D == 64)
    hipLaunchKernelGGL((tower_vt_kernel<64>), grid, dim3(256), 0, st, a);
  else if (D == 96)
    hipLaunchKernelGGL((tower_vt_kernel<96>), grid, dim3(256), 0, st, a);
  else
    return -1;
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

// Shapes this kernel is built for (checked by the caller): batched, unmasked, prefix-only, bf16 K / V^T,
// head size 64 or 96, at least 128 keys (two stages), strides and alignment as for the expert attention
// kernel.
int tk_launch_tower_attn(AttnArgs a, int D, int cus, hipStream_t st) {
  if (a.P <= kStageKeys) return -1;
  if (a.f16) return D == 96 && !a.logits_bf16 ? launch_tower<96, false, true>(a, st, cus) : -1;  // (pi0.5's tower)
  if (D == 64) return a.logits_bf16 ? launch_tower<64, true>(a, st, cus) : launch_tower<64, false>(a, st, cus);
  if (D == 96) return a.logits_bf16 ? launch_tower<96, true>(a, st, cus) : launch_tower<96, false>(a, st, cus);
  return -1;
}
