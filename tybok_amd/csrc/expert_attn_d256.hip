// Action-expert attention for 256-wide heads on gfx950 (the pi0.5 expert: 50 queries, 8 heads over one
// K/V head, ~760 keys), same operands, masks and hand-off buffers as expert_attn.hip.
//
// With D = 256 a wave that owns a key tile AND the whole output row (8 accumulator tiles) leaves no
// registers for anything else, and merging the waves means exchanging 32 KiB of partial output per wave.
// Here the two products are cut along different axes instead:
//   * S^T = K . Q^T : wave w owns key tile w of the block's range (32 keys, all 256 d) -- 16 MFMAs;
//   * O^T += V^T . P^T : wave w owns output rows d in [32w, 32w + 32) for ALL of the block's keys --
//     16 MFMAs over the up to 8 key tiles.
// What crosses waves is only the probabilities: every wave parks its P^T tile in LDS as ready-made B
// operands (1 KiB per k step), after one exchange of the tile maxima fixes the block's softmax base.
// Each wave requests everything it will read -- its Q tile, its K tile and the V^T rows of its 32
// output columns for the whole key range -- before the first MFMA, keeps one accumulator tile, and the
// eight waves finish (or hand to the last-arriving block of a key split) disjoint slices of the output.
// A block walks its key range in rounds of 8 key tiles (online softmax across rounds: one rescale of the
// accumulator tile per round).  Few query tiles (the denoise step): the key range is split over blocks
// of one round each, and the last-arriving block merges the fp32 partials in split order, as in the
// other attention kernel.  Many query tiles (the prefill): one block per query tile and head, no hand-off.
#include <math.h>
#include "tk_common.h"
#include "tk_kernels.h"


namespace {

constexpr float kF32Min = -3.4028234663852886e38f;  // finfo(float32).min
constexpr float kOpenpiMask = -2.3819763e38f;       // additive mask of the pi0.5 path
constexpr int kD = 256;
constexpr int kWaves = kD / 32;  // one 32-row slice of O^T per wave; also the key tiles of a block
constexpr int kMaxSplits = 8;
constexpr int kPitch = kD * 2 + 16;          // bytes between staged rows
constexpr int kTileBytes = 32 * kPitch;      // one staged 32-row tile
constexpr int kLdsBytes = (1 + kWaves) * kTileBytes;
static_assert(kWaves * 2 * 64 * 16 <= kTileBytes, "the P^T operands reuse the Q tile's space");

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

__global__ __launch_bounds__(kWaves * 64) void expert_attn_d256_kernel(AttnArgs a) {
  constexpr int DS = kD / 16;  // k steps of Q.K^T
  __shared__ float st_m[kWaves][32], st_l[kWaves][32];
  // dynamic LDS: the Q tile (later the P^T operands of every key tile), then one staging tile per wave
  // (its K tile, later its V^T rows); rows of 512 bytes at a pitch that keeps 16-byte operand reads of
  // 32 rows conflict-free
  extern __shared__ __align__(16) unsigned char lds[];
  unsigned char* const qs = lds;
  i32x4(*const pt)[2][64] = (i32x4(*)[2][64])lds;  // [key tile][k step][lane]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int h = blockIdx.x;
  const int mtile = blockIdx.y;
  const int split = blockIdx.z;
  const int g = (h * a.gqa_mul) >> 16;
  const int tp = (a.P + 31) >> 5;  // prefix tiles; suffix tiles follow
  const int t_lo = split * a.tile_q + (split < a.tile_r ? split : a.tile_r);
  const int ntb = a.tile_q + (split < a.tile_r ? 1 : 0);  // key tiles of this block, in rounds of kWaves
  const int qi = mtile * 32 + l32;
  const bool q_ok = qi < a.M;
  unsigned char* const mine = lds + (1 + wave) * kTileBytes;
  const int tid = threadIdx.x;

  // running softmax base / sum of this lane's query (the same in every wave) and this wave's slice of O^T
  float bm = -INFINITY, bl = 0.f;
  f32x16 o;
#pragma unroll
  for (int i = 0; i < 16; ++i) o[i] = 0.f;
  for (int r_lo = 0; r_lo < ntb; r_lo += kWaves) {
  const int nt = ntb - r_lo < kWaves ? ntb - r_lo : kWaves;  // key tiles of this round, 1..kWaves
  const int rt_lo = t_lo + r_lo;
  const bool active = wave < nt;  // this wave has a key tile of its own
  // (a further round: every wave must be past its reads of the last round's P^T, which the Q tile overwrites)
  if (r_lo > 0) lds_only_barrier();
  // ---- every load, back to back, as whole 512-byte rows (lane -> consecutive 16-byte chunks): Q by the
  // block, K (32 keys x 256 d) and V^T (this wave's 32 d rows x the block's 256 keys) per wave.  Read
  // straight into operand registers instead (one row per lane), every load instruction would touch
  // 32 cache lines for 1 KiB, and the CU's 8 waves x 48 such loads are bound by its tag-lookup rate. ----
  i32x4 qreg[2], kreg[16], vreg[16];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid + 512 * i, row = c >> 5, col = c & 31;
    int m = mtile * 32 + row;
    if (m > a.M - 1) m = a.M - 1;  // rows past M are never stored
    qreg[i] = *(const i32x4*)(a.q + (size_t)m * a.q_sm + (size_t)h * a.q_sh + col * 8);
  }
  const int t = rt_lo + (active ? wave : nt - 1);  // idle waves read a valid tile and drop it
  const bool pre = t < tp;
  const int tt = pre ? t : t - tp;
  const int len = pre ? a.P : a.S;
  {
    const u16* kb = (pre ? a.k_pre : a.k_suf) + (size_t)g * (pre ? a.pre_sh : a.suf_sh);
    const size_t ksl = pre ? a.pre_sl : a.suf_sl;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int c = lane + 64 * i, row = c >> 5, col = c & 31;
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
  {
    // chunk col of a staged V^T row: key tile col / 4 of the block (tiles past the range: a valid
    // address, P^T is zero there), keys 8 * (col % 4) .. + 7 of that tile
    const int col = lane & 31;
    const int j = col >> 2;
    const int tj = rt_lo + (j < nt ? j : nt - 1);
    const bool pj = tj < tp;
    const int ttj = pj ? tj : tj - tp;
    const size_t vsd = pj ? a.pre_vt_sd : a.suf_vt_sd;
    const u16* vb = (pj ? a.vt_pre : a.vt_suf) + (size_t)g * (pj ? a.pre_vt_sh : a.suf_vt_sh) + ttj * 32 + (col & 3) * 8;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = (lane + 64 * i) >> 5;
      vreg[i] = *(const i32x4*)(vb + (size_t)(32 * wave + row) * vsd);
    }
  }
  // keep the V^T requests here: sunk below the first product (to save registers) they would leave only
  // after Q and K have arrived, one memory round trip later
  __builtin_amdgcn_sched_barrier(0);
  // ---- S^T tile = K . Q^T (one query column per lane) ----
  f32x16 sT;
#pragma unroll
  for (int i = 0; i < 16; ++i) sT[i] = 0.f;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid + 512 * i;
    *(i32x4*)(qs + (c >> 5) * kPitch + (c & 31) * 16) = qreg[i];
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int c = lane + 64 * i;
    *(i32x4*)(mine + key_of_row(c >> 5) * kPitch + (c & 31) * 16) = kreg[i];  // MFMA row r holds key key_of_row(r)
  }
  lds_only_barrier();  // the Q tile is complete (the K tile is this wave's own)
  // operand reads in two batches of 8 k steps, each batch out before its first product waits for one
  // (all 16 at once would not leave registers for the V^T rows still held for the second product)
#pragma unroll
  for (int s0 = 0; s0 < DS; s0 += 8) {
    i32x4 ka[8], qb[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int off = l32 * kPitch + (16 * (s0 + s) + 8 * half) * 2;
      ka[s] = *(const i32x4*)(mine + off);
      qb[s] = *(const i32x4*)(qs + off);
    }
    __builtin_amdgcn_sched_barrier(0);  // (the scheduler would pair each read with its product again)
#pragma unroll
    for (int s = 0; s < 8; ++s) sT = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(ka[s]), as_bf16x8(qb[s]), sT, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
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
  float m_new = bm;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) m_new = fmaxf(m_new, st_m[w][l32]);
  // every round has a key in range, so m_new is finite; the first round's alpha is exp(-inf) = 0
  const float alpha = __expf(bm - m_new);
  bm = m_new;
  float lsum = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    p[i] = __expf(p[i] - bm);  // out-of-range keys give 0
    lsum += p[i];
  }
  lsum += __shfl_xor(lsum, 32);
  if (half == 0) st_l[wave][l32] = lsum;
  // (every wave is past its reads of the Q tile: they feed the maxima exchanged above)
  pt[wave][0][lane] = pack8(p);
  pt[wave][1][lane] = pack8(p + 8);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int c = lane + 64 * i;
    *(i32x4*)(mine + (c >> 5) * kPitch + (c & 31) * 16) = vreg[i];  // over this wave's K tile, which it has consumed
  }
  lds_only_barrier();
  {
    float rl = st_l[0][l32];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) rl += st_l[w][l32];
    bl = bl * alpha + rl;
  }
  // ---- O^T rows [32w, 32w + 32) += V^T . P^T over every key tile of the round ----
#pragma unroll
  for (int i = 0; i < 16; ++i) o[i] *= alpha;  // all of a lane's registers belong to its one query
  {
    i32x4 va[kWaves][2], pb[kWaves][2];
#pragma unroll
    for (int j = 0; j < kWaves; ++j)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        va[j][s] = *(const i32x4*)(mine + l32 * kPitch + (32 * j + 16 * s + 8 * half) * 2);
        pb[j][s] = pt[j][s][lane];
      }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < kWaves; ++j)
#pragma unroll
      for (int s = 0; s < 2; ++s) o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(va[j][s]), as_bf16x8(pb[j][s]), o, 0, 0, 0);
  }
  }  // rounds
  // this lane's output: query qi, columns 32w + 8g4 + 4*half + 0..3 for the four register groups g4
  u16* op = a.out + (size_t)(q_ok ? qi : 0) * a.out_sm + (size_t)h * kD + 32 * wave + 4 * half;
  if (a.kv_splits == 1) {
    if (q_ok) {
      const float inv = 1.0f / bl;
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const f32x4 v = {o[4 * g4], o[4 * g4 + 1], o[4 * g4 + 2], o[4 * g4 + 3]};
        *(i32x2*)(op + 8 * g4) = pack_bf16x4(v * inv);
      }
    }
    return;
  }

  // ---- key-split merge, wave by wave: wave w of every split block leaves its slice of O^T (with its own copy of
  // the statistics, which are the same in every wave) and counts itself in on counter (block, w); the wave that
  // arrives last for a slice merges that slice.  No block barrier in the chain: a wave's store acknowledgement,
  // count and read-back overlap with the other waves'. ----
  // partials per (block, split): [wave][2][32] statistics, then [wave][group][lane][4 floats]
  const int blk_lin = mtile * a.H + h;
  constexpr size_t PSTRIDE = (size_t)kWaves * 64 + (size_t)kWaves * 1024;  // floats
  float* pmine = a.partial + ((size_t)blk_lin * a.kv_splits + split) * PSTRIDE;
  if (half == 0) {
    st_agent(pmine + wave * 64 + l32, bm);
    st_agent(pmine + wave * 64 + 32 + l32, bl);
  }
  {
    unsigned long long* dst = (unsigned long long*)(pmine + kWaves * 64) + ((size_t)wave * 256 + lane) * 2;
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      st_agent64(dst + (size_t)g4 * 128, o[4 * g4], o[4 * g4 + 1]);
      st_agent64(dst + (size_t)g4 * 128 + 1, o[4 * g4 + 2], o[4 * g4 + 3]);
    }
  }
  handoff_publish();  // this wave's slice acknowledged (written through) before its count
  int old = 0;
  if (lane == 0) old = __hip_atomic_fetch_add(a.counters + (blk_lin * kWaves + wave) * 16, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  old = __builtin_amdgcn_readfirstlane(old);
  if (old != a.kv_splits - 1) return;  // wave-uniform
  handoff_acquire();
  if (lane == 0) __hip_atomic_store(a.counters + (blk_lin * kWaves + wave) * 16, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  const float* pblk = a.partial + (size_t)blk_lin * a.kv_splits * PSTRIDE;
  // every read of the hand-off goes out before the first one is consumed
  float ms[kMaxSplits], ls[kMaxSplits];
  unsigned long long raw[kMaxSplits][4][2];
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s) {
    ms[s] = -INFINITY;
    ls[s] = 0.f;
    if (s < a.kv_splits) {  // block-uniform
      ms[s] = ld_agent(pblk + (size_t)s * PSTRIDE + wave * 64 + l32);
      ls[s] = ld_agent(pblk + (size_t)s * PSTRIDE + wave * 64 + 32 + l32);
    }
  }
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s) {
    if (s < a.kv_splits) {
      const unsigned long long* src = (const unsigned long long*)(pblk + (size_t)s * PSTRIDE + kWaves * 64) + ((size_t)wave * 256 + lane) * 2;
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        raw[s][g4][0] = ld_agent64(src + (size_t)g4 * 128);
        raw[s][g4][1] = ld_agent64(src + (size_t)g4 * 128 + 1);
      }
    }
  }
  float mt = -INFINITY;
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s)
    if (s < a.kv_splits) mt = fmaxf(mt, ms[s]);
  float lt = 0.f, es[kMaxSplits];
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s) {
    es[s] = s < a.kv_splits ? __expf(ms[s] - mt) : 0.f;
    if (s < a.kv_splits) lt += ls[s] * es[s];
  }
  const float inv = 1.0f / lt;
#pragma unroll
  for (int g4 = 0; g4 < 4; ++g4) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < kMaxSplits; ++s) {
      if (s < a.kv_splits) {
        const f32x4 v = {__uint_as_float((unsigned)raw[s][g4][0]), __uint_as_float((unsigned)(raw[s][g4][0] >> 32)),
                         __uint_as_float((unsigned)raw[s][g4][1]), __uint_as_float((unsigned)(raw[s][g4][1] >> 32))};
        acc += v * es[s];
      }
    }
    if (q_ok) *(i32x2*)(op + 8 * g4) = pack_bf16x4(acc * inv);
  }
}

}  // namespace

int tk_attn_d256_max_splits() { return kMaxSplits; }
int tk_attn_d256_tiles_per_block() { return kWaves; }

// a.kv_splits blocks per (head, query tile), each over its share of the key tiles; no hi/lo planes, one problem
int tk_launch_attn_d256(AttnArgs a, hipStream_t st) {
  if (a.k_pre_lo || a.batch > 0 || a.kv_splits < 1 || a.kv_splits > kMaxSplits) return -1;
  if (a.tile_q < 1) return -1;
  // more LDS than a launch gets by default: raise the kernel's limit once per process
  static int raised = 0;
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&expert_attn_d256_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess)
      return -3;
    raised = 1;
  }
  dim3 grid(a.H, (a.M + 31) / 32, a.kv_splits);
  hipLaunchKernelGGL(expert_attn_d256_kernel, grid, dim3(kWaves * 64), kLdsBytes, st, a);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
