// extern "C" entry points of libtybok_hip.so (declared in include/tybok_hip.h).
// Host-side argument checks, launch geometry, workspace carving.  No allocation, no sync.
#include <atomic>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/tybok_hip.h"
#include "tk_common.h"
#include "tk_kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// workspace carving (bytes)
constexpr size_t kCounterBytes = TK_WS_COUNTER_BYTES;
constexpr size_t kPartialOff = kCounterBytes;
constexpr size_t kPartialBytes = 56ull << 20;  // split-K / kv-split fp32 partials
constexpr size_t kNormOff = kPartialOff + kPartialBytes;
constexpr size_t kNormBytes = 8ull << 20;  // normalised activations of a many-row GEMM
constexpr size_t kHiddenOff = kNormOff + kNormBytes;
constexpr size_t kHiddenBytes = TK_WS_TOTAL_BYTES - kHiddenOff;  // FFN [M, I] bf16 intermediate
// the last TK_FUSE_WORDS int32 of the counter region belong to the single-launch FFN's hand-off
constexpr int kMaxCounters = (int)(kCounterBytes / 4) - TK_FUSE_WORDS;
constexpr size_t kFuseOff = (size_t)kMaxCounters * 4;
// (off unless asked for: on MI355X the in-kernel hand-off -- write-through acknowledge, flag, poll round trip, first read of
// the intermediate: 2.6 us from the last flag raised to the flags seen -- costs more than the launch boundary it
// replaces; measured 10.9 against 8.6 us per FFN at (50, 720, 2048), 13.3 against 10.9 us at (50, 1024, 4096))
std::atomic<int> g_ffn_fusion{0};          // tk_set_ffn_fusion
std::atomic<int> g_handoff_spin{200000};   // tk_set_handoff_spin: polls a waiting block makes before it gives up

// Scratch of tk_fp8w_gemm_static (callers that cannot allocate): arrival counters followed by split-K
// partials, the head of the workspace layout above at a modest size.  Every device the library runs on
// holds its own copy until the process ends.  In host code the array's NAME is only a handle: the
// device address comes from hipGetSymbolAddress (static_scratch() below), once per device.
constexpr size_t kStaticPartialBytes = 8ull << 20;
constexpr size_t kStaticBytes = kCounterBytes + kStaticPartialBytes;
constexpr int kStaticMaxRows = 64;
static __device__ __align__(256) unsigned char scratch[kStaticBytes];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];  // device address of `scratch` per device ordinal, nullptr = not looked up yet

bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }
bool aligned8(const void* p) { return (((uintptr_t)p) & 7) == 0; }

int g_cus = -1;
int device_cus() {
  if (g_cus < 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    g_cus = n;
  }
  return g_cus;
}

// Device address of this device's copy of `scratch`: looked up on the first call per device, with that device
// current (concurrent first calls store the same value twice, atomically).  The lookup is a runtime call that
// does not belong inside a stream capture: a first call on a capturing stream is refused instead -- call
// tk_static_scratch_bytes() (which resolves the address for the current device) or run one launch before
// capturing.
int static_scratch(void** out, hipStream_t st, bool may_fail_capture) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(TK_ELAUNCH, "static scratch: no current device (or ordinal >= %d)", kMaxDevices);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (may_fail_capture) {
      hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
      if (hipStreamIsCapturing(st, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
        return fail(TK_EINVAL, "gemm_static: first call on this device under stream capture (call tk_static_scratch_bytes() before capturing)");
    }
    const hipError_t rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (rc != hipSuccess || !p) return fail(TK_ELAUNCH, "static scratch: hipGetSymbolAddress failed (%s)", hipGetErrorString(rc));
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return TK_OK;
}

// Optional pieces of a GEMM launch beyond y = bf16((x . W^T) * scale).
struct GemmExtra {
  int x_f32 = 0;                  // activations are fp32 (norm prologue only)
  int w16 = 0;                    // bf16 weight tiles
  const void* norm_w = nullptr;   // RMSNorm prologue
  float norm_eps = 0.f;
  const void* ada_scale = nullptr;  // adaptive RMSNorm prologue (fp32 [K] scale / shift)
  const void* ada_shift = nullptr;
  const int* rope_pos = nullptr;  // rotary epilogue
  const float* rope_cos = nullptr;
  const float* rope_sin = nullptr;
  int rope_positions = 0, rope_cols = 0, rope_half = 0, rope_bf16 = 0;
  void* vt = nullptr;  // transposed copy of the columns >= vt_col0 (rotary epilogue)
  int vt_col0 = 0, vt_ld = 0;
  int clear_counters = 0;  // zero the arrival counters a split launch uses right before it (shared static scratch)
};

// What gemm_common decided for a launch it was asked to plan instead of run.
struct GemmPlan {
  GemmArgs a;
  int MT = 0, NT = 0, mblocks = 0;
  bool skinny = false;  // fp8w_gemm_kernel (not the many-row or the weight-streaming kernel)
};

// One GEMM launch (plain, gated or rotary).  `N` is the logical output width.
int gemm_common(const void* x, int ldx, const void* w_packed, const float* s0, const float* s1, void* y, int ldy,
                const void* resid, int ldr, int resid_dtype, const void* gate, int M, int N, int K, int split_k,
                int act, void* ws, size_t ws_bytes, hipStream_t st, const GemmExtra& e = GemmExtra(), GemmPlan* plan = nullptr) {
  if (M <= 0 || N <= 0 || K <= 0) return fail(TK_EINVAL, "gemm: non-positive shape M=%d N=%d K=%d", M, N, K);
  if (K % 16) return fail(TK_EINVAL, "gemm: K=%d must be a multiple of 16", K);
  if (ldx % 8 || ldx < K) return fail(TK_EINVAL, "gemm: ldx=%d must be >= K and a multiple of 8", ldx);
  if (ldy < N) return fail(TK_EINVAL, "gemm: ldy=%d < N=%d", ldy, N);
  if (!x || !w_packed || (!s0 && !e.w16) || !y) return fail(TK_EINVAL, "gemm: null pointer");
  if (!aligned16(x) || !aligned16(w_packed)) return fail(TK_EINVAL, "gemm: x and w_packed must be 16-byte aligned");
  if (resid && resid_dtype != TK_BF16 && resid_dtype != TK_F32) return fail(TK_EINVAL, "gemm: bad resid_dtype");
  if (resid && ldr < N) return fail(TK_EINVAL, "gemm: ldr=%d < N=%d", ldr, N);
  const bool gated = s1 != nullptr;
  const bool rope = e.rope_pos != nullptr;
  if (gated && (N % 32)) return fail(TK_EINVAL, "gated gemm: I=%d must be a multiple of 32", N);
  if (e.x_f32 && !e.norm_w) return fail(TK_EINVAL, "gemm: fp32 activations need the norm prologue");
  if ((e.ada_scale != nullptr) != (e.ada_shift != nullptr)) return fail(TK_EINVAL, "gemm: adaptive norm needs both scale and shift");
  if (e.ada_scale && (e.norm_w || e.x_f32 || !aligned16(e.ada_scale) || !aligned16(e.ada_shift)))
    return fail(TK_EINVAL, "gemm: adaptive norm takes bf16 activations, no norm weight, 16-byte aligned scale / shift");
  if (e.norm_w && !aligned16(e.norm_w)) return fail(TK_EINVAL, "gemm: norm weight must be 16-byte aligned");
  if (rope) {
    if (gated || resid || gate) return fail(TK_EINVAL, "gemm: the rotary epilogue excludes gate/residual epilogues");
    if (!e.rope_cos || !e.rope_sin || e.rope_positions <= 0) return fail(TK_EINVAL, "gemm: null rotary table");
    if (e.rope_half < 32 || e.rope_half % 32) return fail(TK_EINVAL, "gemm: rope_half=%d must be a multiple of 32", e.rope_half);
    if (N % (2 * e.rope_half) || e.rope_cols % (2 * e.rope_half) || e.rope_cols > N)
      return fail(TK_EINVAL, "gemm: N=%d and rope_cols=%d must be multiples of the head size %d", N, e.rope_cols, 2 * e.rope_half);
  }

  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.x = x;
  a.ldx = ldx;
  a.x_f32 = e.x_f32;
  a.w16 = e.w16;
  a.w = (const uint8_t*)w_packed;
  a.s0 = s0;
  a.s1 = s1;
  a.y = (u16*)y;
  a.ldy = ldy;
  a.resid = resid;
  a.ldr = ldr;
  a.resid_f32 = resid_dtype == TK_F32;
  a.gate = (const u16*)gate;
  a.M = M;
  a.N = N;
  a.K = K;
  a.KT = (K + 31) / 32;
  a.ntiles = ((N + 31) / 32) * (gated ? 2 : 1);
  a.act = act;
  a.vec = N % 4 == 0 && ldy % 4 == 0 && aligned8(y) && (e.w16 || aligned16(s0)) && (!gate || aligned8(gate)) &&
          (!resid || (ldr % 4 == 0 && (resid_dtype == TK_F32 ? aligned16(resid) : aligned8(resid))));
  a.vec16 = ldy % 8 == 0 && aligned16(y) && (!resid || (aligned16(resid) && ldr % (resid_dtype == TK_F32 ? 4 : 8) == 0));
  if ((gated || rope) && (ldy % 4 || !aligned8(y) || (gated && (!aligned16(s0) || !aligned16(s1)))))
    return fail(TK_EINVAL, "gemm: this epilogue needs ldy %% 4 == 0, an 8-byte aligned y and 16-byte aligned scales");
  if (rope && (!aligned16(e.rope_cos) || !aligned16(e.rope_sin)))
    return fail(TK_EINVAL, "gemm: rotary tables must be 16-byte aligned");
  if (e.vt) {
    if (!rope) return fail(TK_EINVAL, "gemm: the transposed value output belongs to the rotary epilogue");
    if (e.vt_col0 < e.rope_cols || e.vt_col0 > N || e.vt_col0 % (2 * e.rope_half) || e.vt_ld < M)
      return fail(TK_EINVAL, "gemm: vt_col0=%d must be a head boundary in [rope_cols, N] and vt_ld=%d >= M", e.vt_col0, e.vt_ld);
  }
  a.norm_w = (const u16*)e.norm_w;
  a.norm_eps = e.norm_eps;
  a.ada_scale = (const float*)e.ada_scale;
  a.ada_shift = (const float*)e.ada_shift;
  a.rope_bf16 = e.rope_bf16;
  a.rope_pos = e.rope_pos;
  a.rope_cos = e.rope_cos;
  a.rope_sin = e.rope_sin;
  a.rope_positions = e.rope_positions;
  a.rope_cols = e.rope_cols;
  a.rope_half = e.rope_half;
  a.vt = (u16*)e.vt;
  a.vt_col0 = e.vt_col0;
  a.vt_ld = e.vt_ld;

  const int cus = device_cus();
  const bool has_norm = e.norm_w || e.ada_scale;
  // (from 256 rows on, or when its 128 x 256 tiles already fill the device; below that the skinny
  // kernel's finer blocks and K splits win)
  const int wide_blocks = ((a.ntiles * 32 + tk_wide_cols() - 1) / tk_wide_cols()) * ((M + 127) / 128);
  if (!e.w16 && !rope && !e.x_f32 && a.vec && (M >= 256 || (M > 64 && wide_blocks >= cus)) &&
      (!has_norm || (ws && ws_bytes >= kNormOff + (size_t)M * K * 2 && (size_t)M * K * 2 <= kNormBytes))) {
    // many rows: MFMA-bound kernel with a 128 x 256 block tile
    if (plan) return TK_OK;  // (plan->skinny stays false)
    if (has_norm) {
      NormRowsArgs nr;
      nr.x = (const u16*)x;
      nr.ldx = ldx;
      nr.norm_w = (const u16*)e.norm_w;
      nr.ada_scale = (const float*)e.ada_scale;
      nr.ada_shift = (const float*)e.ada_shift;
      nr.eps = e.norm_eps;
      nr.out = (u16*)((char*)ws + kNormOff);
      nr.ldo = K;
      nr.M = M;
      nr.K = K;
      if (tk_launch_norm_rows(nr, st)) return fail(TK_ELAUNCH, "gemm: norm launch failed");
      a.x = nr.out;
      a.ldx = K;
      a.norm_w = nullptr;
      a.ada_scale = a.ada_shift = nullptr;
    }
    // 64-row blocks, two per CU, once the 128-row grid would run in several generations anyway: co-resident
    // blocks cover each other's first loads and epilogue; few blocks keep the 128-row tile
    a.mtiles = wide_blocks >= 2 * cus ? 2 : 4;
    if (a.mtiles == 2 && split_k <= 1) {
      // eight-wave blocks of 192 / 256 rows with both operands through LDS, one per CU, where a CU's share of the rows
      // (blocks in a row on it x rows per block) is no larger than with the 64-row blocks (measured on the gated
      // 2048 -> 2 x 16384 launch: M=712 94 -> 90 us on 192 rows, 100 us on 256 -- its 384 blocks are one and a half
      // generations; M=512 / 968 / 1024: 256-row blocks take 6 / 8 / 9 us off the FFN)
      const int nb = (a.ntiles * 32 + tk_wide_cols() - 1) / tk_wide_cols();
      auto share = [&](int rows) { return ((nb * ((M + rows - 1) / rows) + cus - 1) / cus) * rows; };
      if (share(192) <= share(64)) a.mtiles = 6;
      if (share(256) < share(192) && share(256) <= share(64)) a.mtiles = 8;
    }
    const int nbn = (a.ntiles * 32 + tk_wide_cols() - 1) / tk_wide_cols();
    int ks = split_k;
    if (ks <= 0 && a.mtiles == 4 && !a.s1 && a.N % 4 == 0 && ws && a.KT >= 32) {
      // Few column blocks over a long K (the down projection): 64- or 128-row blocks and the split count by a cost
      // fitted to M = 296 .. 968 at K = 16384, N = 2048 -- the k loop of the blocks that share a CU (0.1 us per 1000
      // row x k products), the partials' trip through memory (0.5 us per MB), the weights pulled once per row block
      // (0.005 us per MB) and 8 us that a grid of lone four-wave 64-row blocks loses to 128-row ones.  At 296 rows
      // 64-row blocks x 6 splits take 31.8 us where 128-row blocks x 10 take 36.2; from 552 rows on 128-row blocks.
      double best = 1e30;
      for (int mt = 2; mt <= 4; mt += 2)
        for (int sp = 1; sp <= 16 && sp <= a.KT / 16; ++sp) {
          const int nbm = (M + mt * 32 - 1) / (mt * 32);
          const int gens = (nbn * nbm * sp + cus - 1) / cus;
          const double loop = 1e-4 * gens * (mt * 32) * ((double)K / sp);
          const double part = sp > 1 ? 0.5e-6 * 4.0 * sp * nbm * (mt * 32) * nbn * tk_wide_cols() : 0.0;
          const double cost = loop + part + (mt == 2 ? 8.0 : 0.0) + 0.005e-6 * nbm * (double)K * nbn * tk_wide_cols();
          if (cost < best) best = cost, a.mtiles = mt, ks = sp;
        }
    }
    const int brows = a.mtiles * 32;
    const int blocks0 = nbn * ((M + brows - 1) / brows);
    if (ks <= 0) {
      // fill the device once; a split keeps at least 16 k tiles and its partials must fit
      ks = cus / blocks0;
      if (ks > a.KT / 16) ks = a.KT / 16;
      if (ks < 1) ks = 1;
    }
    const size_t per_split = (size_t)brows * tk_wide_cols() * 4;
    if (ks > 1 && ws) {
      const size_t fit = kPartialBytes / (per_split * blocks0);
      const size_t have = ws_bytes > kPartialOff ? (ws_bytes - kPartialOff) / (per_split * blocks0) : 0;
      if ((size_t)ks > fit) ks = (int)fit;
      if ((size_t)ks > have) ks = (int)have;
      if (ks < 1) ks = 1;
    }
    if (ks > a.KT) ks = a.KT;
    if (ks > 1 && (!ws || blocks0 > kMaxCounters)) {
      if (split_k > 1) return fail(TK_EWORKSPACE, "gemm: split_k=%d needs a workspace", ks);
      ks = 1;
    }
    a.ksplit = ks;
    a.kt_q = a.KT / ks;
    a.kt_r = a.KT % ks;
    a.partial = ks > 1 ? (float*)((char*)ws + kPartialOff) : nullptr;
    a.counters = ks > 1 ? (int*)ws : nullptr;
    if (tk_launch_gemm_wide(a, st)) return fail(TK_ELAUNCH, "gemm: launch failed (%s)", hipGetErrorString(hipGetLastError()));
    return TK_OK;
  }
  int MT = M <= 32 ? 1 : 2;
  // The action chunk (33..64 rows) over a small weight matrix is a latency-bound launch: two blocks
  // of 32 rows per strip halve each block's staging, normalisation and product work and put twice
  // as many CUs on it (measured: FFN at K=720 12.6 -> 10.0 us, with the norm prologue 15.7 -> 12.6 us);
  // the weights are then read twice, which only a large matrix notices (the 33.5 MB shapes lose 5 %).
  if (M > 32 && M <= 64 && (size_t)a.ntiles * 32 * a.KT * 32 * (e.w16 ? 2 : 1) <= (16u << 20)) MT = 1;
  // A few hundred rows (the SmolVLA prefill: 241 / 177) over a small matrix: 32-row blocks too.  With the bf16
  // RMSNorm prologue over a short K they run the prologue that requests every round up front and takes the row
  // statistics from the staged pieces (-3 us per launch inside a request); the other launches gain 0.7 us from the
  // finer blocks
  if (M > 64 && e.norm_w && !e.x_f32 && a.KT <= 32) MT = 1;
  if (M > 64 && M <= 256 && !e.x_f32 && (size_t)a.ntiles * 32 * a.KT * 32 * (e.w16 ? 2 : 1) <= (16u << 20)) MT = 1;
  int NT = 2;
  // 33..64 rows over a large fp8 matrix with the plain epilogue: the weight-streaming schedule (two-tile strips,
  // every block 16 or 8 rounds of four k tiles) when a K split of that size about fills the device
  int stream_ks = 0;
  if (MT == 2 && M <= 64 && !gated && !rope && !e.w16 && !has_norm && !e.x_f32 && K % 32 == 0 && split_k <= 0) {
    const int strips2 = (a.ntiles + 1) / 2;
    for (int per = 64; per >= 32 && !stream_ks; per /= 2) {
      if (a.KT % per) continue;
      const int c = a.KT / per;
      const size_t need = (size_t)strips2 * c * 4 * 4096;
      const bool fits = c == 1 || (ws && strips2 <= kMaxCounters && need <= kPartialBytes && ws_bytes >= kPartialOff + need);
      if (fits && c <= 64 && strips2 * c >= cus / 2 && strips2 * c <= 2 * cus) stream_ks = c;
    }
  }
  if (!stream_ks && !gated && !rope && ((a.ntiles + 1) / 2) * ((M + 32 * MT - 1) / (32 * MT)) < cus / 2) {
    NT = 1;  // few columns: finer strips (the paired epilogues need both tiles of a strip in one wave)
  }
  const int mblocks = (M + 32 * MT - 1) / (32 * MT);
  const int strips = (a.ntiles + NT - 1) / NT;
  const int blocks0 = strips * mblocks;
  const int NW = 4;
  int ks = stream_ks ? stream_ks : split_k;
  if (ks <= 0) {
    // Launch-cost model (microseconds, fitted to graph-replayed launches on MI355X): the k loop costs
    // 0.35 per block round (NW k tiles) for 64-row blocks, 0.20 for 32-row blocks (0.27 with two bf16
    // weight tiles per wave and round), with a floor of one memory round trip; splitting K adds a partial write, an arrival
    // count and a read-back that grows with the number of splits and steps up with every batch of four
    // the finishing block has in flight (1.1 + 0.4 c + 1.0 per further batch), and only pays while the
    // grid still fits the device twice over.
    ks = 1;
    if (blocks0 < cus) {
      const float per_round = MT == 1 ? (e.w16 && NT == 2 ? 0.27f : 0.20f) : 0.35f;
      float best = 1e30f;
      // (an automatic choice never asks for more partial space than the workspace holds)
      const size_t cap = !ws || ws_bytes <= kPartialOff ? 0 : (ws_bytes - kPartialOff < kPartialBytes ? ws_bytes - kPartialOff : kPartialBytes);
      for (int c = 1; c <= 64 && c * NW <= a.KT && (c == 1 || (blocks0 * c <= 2 * cus && (size_t)blocks0 * c * MT * NT * 4096 <= cap && blocks0 * 4 <= kMaxCounters)); ++c) {
        const int rounds = (a.KT + c * NW - 1) / (c * NW);
        float t = rounds * per_round;
        if (t < 1.0f) t = 1.0f;
        if (c > 1) t += 1.1f + 0.4f * (float)c + 1.0f * (float)((c + 3) / 4 - 1);
        if (t < best - 1e-3f) {
          best = t;
          ks = c;
        }
      }
    }
  }
  if (ks > a.KT) ks = a.KT;
  if (ks > 64) ks = 64;
  a.ksplit = ks;
  a.kt_q = a.KT / ks;
  a.kt_r = a.KT % ks;
  a.partial = nullptr;
  a.counters = nullptr;
  if (ks > 1) {
    if (!ws) return fail(TK_EWORKSPACE, "gemm: split_k=%d needs a workspace", ks);
    const size_t need = (size_t)blocks0 * ks * MT * NT * 4096;
    // (an arrival counter per block and finishing wave: the four waves of a block hand over on their own)
    if (blocks0 * 4 > kMaxCounters || need > kPartialBytes || ws_bytes < kPartialOff + need)
      return fail(TK_EWORKSPACE, "gemm: workspace too small (need %zu partial bytes, %d counters)", need, blocks0 * 4);
    a.partial = (float*)((char*)ws + kPartialOff);
    a.counters = (int*)ws;
    // a 64-byte line per counter where the region holds that many: atomics on one line queue behind each other
    a.cstride = blocks0 * 4 * 16 <= kMaxCounters ? 16 : 1;
    if (!plan && e.clear_counters && tk_launch_fill_zero(a.counters, blocks0 * 4 * a.cstride, st)) return fail(TK_ELAUNCH, "gemm: counter fill launch failed");
  }
  // 33..64 rows over a large fp8 matrix: the weight-streaming schedule
  const bool stream = MT == 2 && NT == 2 && mblocks == 1 && tk_gemm_stream_takes(a);
  if (plan) {
    plan->a = a;
    plan->MT = MT;
    plan->NT = NT;
    plan->mblocks = mblocks;
    plan->skinny = !stream;
    return TK_OK;
  }
  int rc = stream ? tk_launch_gemm_stream(a, st) : tk_launch_gemm(a, MT, NT, mblocks, st);
  if (rc == -1) return fail(TK_EINVAL, "gemm: this combination of weight type, prologue and epilogue is not built");
  if (rc) return fail(TK_ELAUNCH, "gemm: launch failed (%s)", hipGetErrorString(hipGetLastError()));
  return TK_OK;
}

// gate/up (+ norm prologue) -> h [M, I] in the workspace -> down (+ gate, residual).  The action chunk (at most 64
// rows, 32-row blocks on both sides, a pair of shapes the fused kernel is built for) runs as ONE launch whose down
// blocks wait for the gate/up blocks inside the kernel; everything else as two launches.  Same arithmetic and
// summation order either way: the same bits.
int ffn_launches(const void* x, int ldx, const GemmExtra& e, const void* wgu_packed, const void* sg, const void* su, void* hbuf,
                 const void* wd_packed, const void* sd, void* y, int ldy, const void* resid, int ldr, int resid_dtype, const void* gate,
                 int M, int K, int I, int act, void* ws, size_t ws_bytes, hipStream_t st) {
  // (the fused form keeps the intermediate in 32-row slices: whole row blocks of it must fit)
  if (M <= 64 && g_ffn_fusion.load(std::memory_order_relaxed) && ws_bytes >= kHiddenOff + (size_t)((M + 31) / 32) * 32 * I * 2) {
    GemmPlan pg, pd;
    int rc = gemm_common(x, ldx, wgu_packed, (const float*)sg, (const float*)su, hbuf, I, nullptr, 0, 0, nullptr, M, I, K, 0, act, ws,
                         ws_bytes, st, e, &pg);
    if (rc) return rc;
    rc = gemm_common(hbuf, I, wd_packed, (const float*)sd, nullptr, y, ldy, resid, ldr, resid_dtype, gate, M, K, I, 0, 0, ws, ws_bytes, st,
                     GemmExtra(), &pd);
    if (rc) return rc;
    if (pg.skinny && pd.skinny && pg.MT == 1 && pd.MT == 1 && pg.NT == 2 && pg.a.ksplit == 1 && pg.mblocks == pd.mblocks) {
      int* fuse = (int*)((char*)ws + kFuseOff);
      pg.a.fuse = pd.a.fuse = fuse;
      pd.a.fuse_consumers = ((pd.a.ntiles + pd.NT - 1) / pd.NT) * pd.a.ksplit;
      pd.a.fuse_spin = g_handoff_spin.load(std::memory_order_relaxed);
      rc = tk_launch_ffn_fused(pg.a, pd.a, pd.NT, pg.mblocks, st);
      if (rc == 0) return TK_OK;
      if (rc != -1) return fail(TK_ELAUNCH, "ffn: launch failed (%s)", hipGetErrorString(hipGetLastError()));
    }
  }
  int rc = gemm_common(x, ldx, wgu_packed, (const float*)sg, (const float*)su, hbuf, I, nullptr, 0, 0, nullptr, M, I, K, 0, act, ws,
                       ws_bytes, st, e);
  if (rc) return rc;
  return gemm_common(hbuf, I, wd_packed, (const float*)sd, nullptr, y, ldy, resid, ldr, resid_dtype, gate, M, K, I, 0, 0, ws, ws_bytes, st);
}

}  // namespace

extern "C" {

int tk_version(void) { return 1; }
const char* tk_last_error(void) { return g_err; }
int tk_device_cus(void) { return device_cus(); }

size_t tk_workspace_bytes(void) { return TK_WS_TOTAL_BYTES; }

int tk_workspace_init(void* ws, size_t ws_bytes, void* stream) {
  if (!ws || ws_bytes < kCounterBytes) return fail(TK_EWORKSPACE, "workspace_init: need >= %zu bytes", kCounterBytes);
  if (tk_launch_fill_zero((int*)ws, (int)(kCounterBytes / 4), (hipStream_t)stream))
    return fail(TK_ELAUNCH, "workspace_init: launch failed");
  return TK_OK;
}

int tk_set_ffn_fusion(int on) { return g_ffn_fusion.exchange(on ? 1 : 0); }
int tk_set_handoff_spin(int polls) { return g_handoff_spin.exchange(polls < 0 ? 0 : polls); }
size_t tk_workspace_handoff_error_offset(void) { return kFuseOff + (size_t)TK_FUSE_ERROR * 4; }

size_t tk_fp8w_packed_bytes(int N, int K) {
  if (N <= 0 || K <= 0) return 0;
  return (size_t)((N + 31) / 32) * ((K + 31) / 32) * 1024;
}

int tk_pack_fp8_weight(const void* w8, void* packed, int N, int K, void* stream) {
  if (!w8 || !packed || N <= 0 || K <= 0) return fail(TK_EINVAL, "pack: bad argument");
  if (K % 16) return fail(TK_EINVAL, "pack: K=%d must be a multiple of 16", K);
  if (!aligned16(w8) || !aligned16(packed)) return fail(TK_EINVAL, "pack: pointers must be 16-byte aligned");
  if (tk_launch_pack(w8, nullptr, packed, N, K, 0, (hipStream_t)stream)) return fail(TK_ELAUNCH, "pack: launch failed");
  return TK_OK;
}

int tk_pack_fp8_gate_up(const void* wg8, const void* wu8, void* packed, int I, int K, void* stream) {
  if (!wg8 || !wu8 || !packed || I <= 0 || K <= 0) return fail(TK_EINVAL, "pack_gate_up: bad argument");
  if (K % 16 || I % 32) return fail(TK_EINVAL, "pack_gate_up: need K %% 16 == 0 and I %% 32 == 0 (K=%d I=%d)", K, I);
  if (!aligned16(wg8) || !aligned16(wu8) || !aligned16(packed))
    return fail(TK_EINVAL, "pack_gate_up: pointers must be 16-byte aligned");
  if (tk_launch_pack(wg8, wu8, packed, I, K, 1, (hipStream_t)stream))
    return fail(TK_ELAUNCH, "pack_gate_up: launch failed");
  return TK_OK;
}

int tk_fp8w_gemm(const void* x, int ldx, const void* w_packed, const void* scale, void* y, int ldy, const void* resid,
                 int ldr, int resid_dtype, const void* gate, int M, int N, int K, int split_k, void* ws, size_t ws_bytes,
                 void* stream) {
  return gemm_common(x, ldx, w_packed, (const float*)scale, nullptr, y, ldy, resid, ldr, resid_dtype, gate, M, N, K,
                     split_k, 0, ws, ws_bytes, (hipStream_t)stream);
}

int tk_fp8w_gemm_static(const void* x, int ldx, const void* w_packed, const void* scale, void* y, int ldy,
                        const void* resid, int ldr, int resid_dtype, const void* gate, int M, int N, int K, int split_k,
                        void* stream) {
  if (M > kStaticMaxRows)
    return fail(TK_EINVAL, "gemm_static: M=%d exceeds the %d rows this entry point is built for (use tk_fp8w_gemm with a workspace)",
                M, kStaticMaxRows);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws, (hipStream_t)stream, true)) return rc;
  GemmExtra e;
  e.clear_counters = 1;
  return gemm_common(x, ldx, w_packed, (const float*)scale, nullptr, y, ldy, resid, ldr, resid_dtype, gate, M, N, K, split_k,
                     0, ws, kStaticBytes, (hipStream_t)stream, e);
}

size_t tk_static_scratch_bytes(void) {
  // also resolves the array's address for the current device, so that no later call has to (stream capture)
  void* p = nullptr;
  (void)static_scratch(&p, nullptr, false);
  return kStaticBytes;
}

int tk_fp8w_gated_ffn(const void* x, int ldx, const void* wgu_packed, const void* sg, const void* su,
                      const void* wd_packed, const void* sd, void* y, int ldy, const void* resid, int ldr,
                      int resid_dtype, const void* gate, int M, int K, int I, int act, void* ws, size_t ws_bytes,
                      void* stream) {
  if (act != TK_ACT_SILU && act != TK_ACT_GELU_TANH) return fail(TK_EINVAL, "ffn: unknown activation %d", act);
  if (M <= 0 || K <= 0 || I <= 0) return fail(TK_EINVAL, "ffn: non-positive shape M=%d K=%d I=%d", M, K, I);
  if (!sg || !su || !sd) return fail(TK_EINVAL, "ffn: null scale pointer");
  if (I % 32) return fail(TK_EINVAL, "ffn: I=%d must be a multiple of 32", I);
  if (!ws) return fail(TK_EWORKSPACE, "ffn: needs a workspace");
  const size_t hbytes = (size_t)M * I * 2;
  if (hbytes > kHiddenBytes || ws_bytes < kHiddenOff + hbytes)
    return fail(TK_EWORKSPACE, "ffn: workspace too small for the [%d, %d] intermediate", M, I);
  void* hbuf = (char*)ws + kHiddenOff;
  // gate/up + activation-multiply -> h[M, I] (bf16, workspace)
  return ffn_launches(x, ldx, GemmExtra(), wgu_packed, sg, su, hbuf, wd_packed, sd, y, ldy, resid, ldr, resid_dtype, gate, M, K, I, act, ws,
                      ws_bytes, (hipStream_t)stream);
}

// ---- W8A8 tier ---------------------------------------------------------------------------------
namespace {
int w8a8_common(const void* a8, int lda, const float* sa, const void* w_packed, const float* s0, const float* s1, void* y, int ldy,
                const void* resid, int ldr, int resid_dtype, int M, int N, int K, int split_k, int act, void* ws, size_t ws_bytes,
                hipStream_t st) {
  if (M <= 0 || N <= 0 || K <= 0) return fail(TK_EINVAL, "w8a8: non-positive shape M=%d N=%d K=%d", M, N, K);
  if (K % 16) return fail(TK_EINVAL, "w8a8: K=%d must be a multiple of 16", K);
  if (lda % 16 || lda < K) return fail(TK_EINVAL, "w8a8: lda=%d must be >= K and a multiple of 16 (bytes)", lda);
  if (!a8 || !sa || !w_packed || !s0 || !y) return fail(TK_EINVAL, "w8a8: null pointer");
  if (!aligned16(a8) || !aligned16(w_packed) || !aligned16(s0) || (s1 && !aligned16(s1))) return fail(TK_EINVAL, "w8a8: a8, w_packed and the weight scales must be 16-byte aligned");
  if (N % 4 || ldy % 4 || ldy < N || !aligned8(y)) return fail(TK_EINVAL, "w8a8: N=%d and ldy=%d must be multiples of 4, ldy >= N, y 8-byte aligned", N, ldy);
  if (s1 && N % 32) return fail(TK_EINVAL, "w8a8 gated: I=%d must be a multiple of 32", N);
  if (resid && resid_dtype != TK_BF16 && resid_dtype != TK_F32) return fail(TK_EINVAL, "w8a8: bad resid_dtype");
  if (resid && (ldr < N || ldr % 4 || !(resid_dtype == TK_F32 ? aligned16(resid) : aligned8(resid)))) return fail(TK_EINVAL, "w8a8: residual pitch / alignment");
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.x = a8;
  a.ldx = lda;
  a.row_scale = sa;
  a.w = (const uint8_t*)w_packed;
  a.s0 = s0;
  a.s1 = s1;
  a.y = (u16*)y;
  a.ldy = ldy;
  a.resid = resid;
  a.ldr = ldr;
  a.resid_f32 = resid_dtype == TK_F32;
  a.M = M;
  a.N = N;
  a.K = K;
  a.KT = (K + 31) / 32;
  a.ntiles = ((N + 31) / 32) * (s1 ? 2 : 1);
  a.act = act;
  a.vec = 1;
  a.vec16 = ldy % 8 == 0 && aligned16(y) && (!resid || (aligned16(resid) && ldr % (resid_dtype == TK_F32 ? 4 : 8) == 0));
  // 64-row blocks, two per CU, once the 128-row grid would run in several generations anyway: co-resident blocks
  // cover each other's first loads and epilogue (gate/up at 712 rows: 73 -> 59 us); few blocks keep the 128-row tile
  const int blocks128 = ((a.ntiles * 32 + tk_w8a8_cols() - 1) / tk_w8a8_cols()) * ((M + 127) / 128);
  a.mtiles = blocks128 >= 2 * device_cus() ? 2 : 4;
  const int rows = a.mtiles * 32;
  const int blocks0 = ((a.ntiles * 32 + tk_w8a8_cols() - 1) / tk_w8a8_cols()) * ((M + rows - 1) / rows);
  int ks = split_k;
  if (ks <= 0) {
    // fill the device once; a split keeps at least 32 k tiles and its partials must fit
    ks = device_cus() / blocks0;
    if (ks > a.KT / 32) ks = a.KT / 32;
    if (ks < 1) ks = 1;
  }
  const size_t per_split = (size_t)rows * tk_w8a8_cols() * 4;
  if (ks > 1) {
    const size_t have = ws && ws_bytes > kPartialOff ? (ws_bytes - kPartialOff < kPartialBytes ? ws_bytes - kPartialOff : kPartialBytes) / (per_split * blocks0) : 0;
    if ((size_t)ks > have || blocks0 > kMaxCounters) {
      if (split_k > 1) return fail(TK_EWORKSPACE, "w8a8: split_k=%d needs %zu bytes of partial space", ks, per_split * blocks0 * ks);
      ks = have > 1 && blocks0 <= kMaxCounters ? (int)have : 1;
    }
  }
  if (ks > a.KT) ks = a.KT;
  a.ksplit = ks;
  a.kt_q = a.KT / ks;
  a.kt_r = a.KT % ks;
  a.partial = ks > 1 ? (float*)((char*)ws + kPartialOff) : nullptr;
  a.counters = ks > 1 ? (int*)ws : nullptr;
  if (tk_launch_w8a8_gemm(a, st)) return fail(TK_ELAUNCH, "w8a8: launch failed (%s)", hipGetErrorString(hipGetLastError()));
  return TK_OK;
}
}  // namespace

// ---- bf16-weight linears with bias / GELU / residual epilogues (vision towers) ---------------------------------
namespace {
struct DenseTile {
  int id, rows, cols;
  int occ;  // blocks of this shape that fit one CU (registers)
};
constexpr DenseTile kDenseTiles[] = {{42, 128, 256, 1}, {41, 128, 128, 2}, {32, 96, 256, 2}, {31, 96, 128, 3},
                                     {22, 64, 256, 2},  {21, 64, 128, 4},  {12, 32, 256, 3}, {11, 32, 128, 4}};

// Estimated duration (us) of a launch with this tile and K split; the constants are fitted to timings of the
// vision towers' and the prefill's shapes (the picked tile is within 1 % of the best one on average).  Blocks
// that are resident together share a CU's matrix pipes and overlap each other's first loads and epilogues; every
// further generation of blocks pays those again.  A wave issues (rows/32) * (cols/128) MFMAs per 16 columns of k
// (18.8 ns each under full load; 30 / 35 / 45 % of that rate reached with one / two / three or more waves per
// SIMD), and a block loads (rows + cols) * 128 bytes per 64 columns of k at about 60 KiB/us per CU.
float dense_cost(const DenseTile& t, int M, int N, int KT, int ks, int cus) {
  const long long blocks = (long long)((M + t.rows - 1) / t.rows) * ((N + t.cols - 1) / t.cols) * ks;
  const float kt = (float)((KT + ks - 1) / ks);
  const float eff = t.occ >= 3 ? 0.45f : t.occ == 2 ? 0.35f : 0.3f;
  const float mfma_us = (float)(t.rows / 32) * (float)(t.cols / 128) * 2.f * kt * 0.0188f / eff;
  const float load_us = 0.5f * kt * (float)(t.rows + t.cols) * 0.125f / 60.f;
  const float tile_us = mfma_us > load_us ? mfma_us : load_us;
  float us = 0.f;
  long long left = blocks;
  while (left > 0) {
    const long long gen = left < (long long)cus * t.occ ? left : (long long)cus * t.occ;
    us += 3.f + (float)((gen + cus - 1) / cus) * tile_us;
    left -= gen;
  }
  if (ks > 1) us += 1.5f + (float)blocks * (float)(t.rows * t.cols) * 8.f / 4e6f;  // fp32 partials out and back in
  return us;
}
}  // namespace

namespace {
// rotary form of the many-row linear: weights in rotary pair order, tables and positions as in tk_bf16w_linear
// transposed copy of the columns >= col0 of a packed q|k|v projection, one problem per `rows` rows
struct DenseVt {
  void* vt = nullptr;
  int col0 = 0, ld = 0, rows = 0;
  long long bs = 0;
};

struct DenseRope {
  const int* pos = nullptr;
  const float* cos = nullptr;
  const float* sin = nullptr;
  int positions = 0, cols = 0, half = 0, bf16 = 0;
  void* vt = nullptr;
  int vt_col0 = 0, vt_ld = 0;
};

int dense_common(const void* x, int ldx, const void* w_packed, const void* bias, int act, void* y, int ldy, const void* resid,
                 int ldr, int resid_dtype, int M, int N, int K, int tile, int split_k, void* ws, size_t ws_bytes, void* stream,
                 int f16, const DenseRope* rope = nullptr, const DenseVt* vt = nullptr) {
  if (M <= 0 || N <= 0 || K <= 0) return fail(TK_EINVAL, "bf16w_dense: non-positive shape M=%d N=%d K=%d", M, N, K);
  if (K % 16 || ldx % 8 || ldx < K) return fail(TK_EINVAL, "bf16w_dense: K=%d must be a multiple of 16 and ldx=%d a multiple of 8 >= K", K, ldx);
  if (!x || !w_packed || !y) return fail(TK_EINVAL, "bf16w_dense: null pointer");
  if (!aligned16(x) || !aligned16(w_packed) || !aligned16(y) || (bias && !aligned8(bias)))
    return fail(TK_EINVAL, "bf16w_dense: x, w_packed and y must be 16-byte aligned, bias 8-byte aligned");
  if (N % 4 || ldy % 8 || ldy < N) return fail(TK_EINVAL, "bf16w_dense: N=%d must be a multiple of 4 and ldy=%d a multiple of 8 >= N", N, ldy);
  if (act < 0 || act > 2) return fail(TK_EINVAL, "bf16w_dense: act=%d (0 none, 1 tanh-GELU of the bf16 output, 2 tanh-GELU in fp32)", act);
  if (resid && resid_dtype != TK_BF16 && resid_dtype != TK_F32) return fail(TK_EINVAL, "bf16w_dense: bad resid_dtype");
  if (resid && (ldr < N || ldr % (resid_dtype == TK_F32 ? 4 : 8) || !aligned16(resid)))
    return fail(TK_EINVAL, "bf16w_dense: residual must be 16-byte aligned with a pitch >= N that keeps rows 16-byte aligned");
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.x = x;
  a.ldx = ldx;
  a.w16 = 1;
  a.w = (const uint8_t*)w_packed;
  a.bias = (const u16*)bias;
  a.y = (u16*)y;
  a.ldy = ldy;
  a.resid = resid;
  a.ldr = ldr;
  a.resid_f32 = resid_dtype == TK_F32;
  a.M = M;
  a.N = N;
  a.K = K;
  a.KT = (K + 31) / 32;
  a.ntiles = (N + 31) / 32;
  a.act = act;
  a.f16 = f16;
  a.vec = a.vec16 = 1;
  if (rope) {
    if (f16 || bias || act || resid) return fail(TK_EINVAL, "bf16w_dense_rope: bf16 only, no bias, activation or residual");
    if (!rope->pos || !rope->cos || !rope->sin || rope->positions <= 0) return fail(TK_EINVAL, "bf16w_dense_rope: null table or position pointer");
    if (rope->half < 32 || rope->half % 32 || rope->cols <= 0 || rope->cols % (2 * rope->half) || rope->cols > N || N % (2 * rope->half))
      return fail(TK_EINVAL, "bf16w_dense_rope: rope_half=%d must be a multiple of 32, rope_cols=%d and N=%d whole heads of 2 * rope_half columns", rope->half, rope->cols, N);
    if (!aligned16(rope->cos) || !aligned16(rope->sin)) return fail(TK_EINVAL, "bf16w_dense_rope: tables must be 16-byte aligned");
    if (rope->vt && (rope->vt_col0 % (2 * rope->half) || rope->vt_col0 < 0 || rope->vt_col0 >= N || rope->vt_ld % 8 || rope->vt_ld < (M + 31) / 32 * 32 || !aligned16(rope->vt)))
      return fail(TK_EINVAL, "bf16w_dense_rope: vt_col0=%d must start a head, vt_ld=%d be a multiple of 8 >= M rounded up to 32, vt 16-byte aligned", rope->vt_col0, rope->vt_ld);
    a.rope_pos = rope->pos;
    a.rope_cos = rope->cos;
    a.rope_sin = rope->sin;
    a.rope_positions = rope->positions;
    a.rope_cols = rope->cols;
    a.rope_half = rope->half;
    a.rope_bf16 = rope->bf16;
    a.vt = (u16*)rope->vt;
    a.vt_col0 = rope->vt_col0;
    a.vt_ld = rope->vt_ld;
  }
  if (vt) {
    if (act || resid) return fail(TK_EINVAL, "bf16w_dense_vt: no activation or residual in this form");
    if (!vt->vt || !aligned16(vt->vt) || vt->col0 < 0 || vt->col0 >= N || vt->col0 % 64 || vt->ld % 8 || vt->rows < 0 || vt->rows % 32 || vt->bs % 8 ||
        vt->ld < (vt->rows ? vt->rows : (M + 31) / 32 * 32))
      return fail(TK_EINVAL, "bf16w_dense_vt: vt 16-byte aligned, vt_col0=%d a multiple of 64 below N, vt_rows=%d a multiple of 32, vt_ld=%d a multiple of 8 that holds a problem's rows, vt_bs a multiple of 8",
                  vt->col0, vt->rows, vt->ld);
    a.vt = (u16*)vt->vt;
    a.vt_col0 = vt->col0;
    a.vt_ld = vt->ld;
    a.vt_rows = vt->rows;
    a.vt_bs = vt->bs;
  }
  const int cus = device_cus();
  const DenseTile* best = nullptr;
  int ks = split_k > 0 ? split_k : 1;
  float best_cost = 0.f;
  for (const DenseTile& t : kDenseTiles) {
    if (tile && t.id != tile) continue;
    if (rope && t.id % 10 != 2) continue;  // the rotary epilogue needs two n tiles per wave
    const int blocks0 = ((M + t.rows - 1) / t.rows) * ((N + t.cols - 1) / t.cols);
    int k1 = 1;
    if (split_k > 0) {
      k1 = split_k;
    } else if (rope) {
      // measured at the prefill's q|k|v shape (712 x 2048 -> 2560): 64 x 256 blocks, unsplit, 20.7 us; 32 x 256:
      // 27.9, 96 x 256: 25.7, 128 x 256: 32.2; any K split 30-39 us (the partials weigh more than the idle CUs)
      if (!tile && t.id != (M > 32 ? 22 : 12)) continue;
    } else {
      // few blocks and a long K: split, keeping at least 32 k tiles per split
      k1 = cus / blocks0;
      if (k1 > a.KT / 32) k1 = a.KT / 32;
      if (k1 < 1) k1 = 1;
    }
    const float c = dense_cost(t, M, N, a.KT, k1, cus);
    if (!best || c < best_cost) best = &t, best_cost = c, ks = k1;
  }
  if (!best) return fail(TK_EINVAL, "bf16w_dense: tile=%d (0 = automatic, or 42, 41, 32, 31, 22, 21, 12, 11)", tile);
  const int blocks0 = ((M + best->rows - 1) / best->rows) * ((N + best->cols - 1) / best->cols);
  const size_t per_split = (size_t)best->rows * best->cols * 4;
  if (ks > 1) {
    const size_t have = ws && ws_bytes > kPartialOff ? (ws_bytes - kPartialOff < kPartialBytes ? ws_bytes - kPartialOff : kPartialBytes) / (per_split * blocks0) : 0;
    if ((size_t)ks > have || blocks0 > kMaxCounters) {
      if (split_k > 1) return fail(TK_EWORKSPACE, "bf16w_dense: split_k=%d needs %zu bytes of partial space", ks, per_split * blocks0 * ks);
      ks = have > 1 && blocks0 <= kMaxCounters ? (int)have : 1;
    }
  }
  if (ks > a.KT) ks = a.KT;
  a.ksplit = ks;
  a.kt_q = a.KT / ks;
  a.kt_r = a.KT % ks;
  a.partial = ks > 1 ? (float*)((char*)ws + kPartialOff) : nullptr;
  a.counters = ks > 1 ? (int*)ws : nullptr;
  if (tk_launch_bf16w_wide(a, best->id, (hipStream_t)stream)) return fail(TK_ELAUNCH, "bf16w_dense: launch failed (%s)", hipGetErrorString(hipGetLastError()));
  return TK_OK;
}
}  // namespace

int tk_bf16w_dense(const void* x, int ldx, const void* w_packed, const void* bias, int act, void* y, int ldy, const void* resid,
                   int ldr, int resid_dtype, int M, int N, int K, int tile, int split_k, void* ws, size_t ws_bytes, void* stream) {
  return dense_common(x, ldx, w_packed, bias, act, y, ldy, resid, ldr, resid_dtype, M, N, K, tile, split_k, ws, ws_bytes, stream, 0);
}

int tk_bf16w_dense_rope(const void* x, int ldx, const void* w_packed, void* y, int ldy, const void* rope_pos, const void* rope_cos,
                        const void* rope_sin, int rope_positions, int rope_cols, int rope_half, int rope_bf16, void* vt, int vt_col0,
                        int vt_ld, int M, int N, int K, int tile, int split_k, void* ws, size_t ws_bytes, void* stream) {
  DenseRope r;
  r.pos = (const int*)rope_pos;
  r.cos = (const float*)rope_cos;
  r.sin = (const float*)rope_sin;
  r.positions = rope_positions;
  r.cols = rope_cols;
  r.half = rope_half;
  r.bf16 = rope_bf16;
  r.vt = vt;
  r.vt_col0 = vt_col0;
  r.vt_ld = vt_ld;
  return dense_common(x, ldx, w_packed, nullptr, 0, y, ldy, nullptr, 0, 0, M, N, K, tile, split_k, ws, ws_bytes, stream, 0, &r);
}

int tk_bf16w_dense_vt(const void* x, int ldx, const void* w_packed, const void* bias, void* y, int ldy, void* vt, int vt_col0, int vt_ld,
                      int vt_rows, long long vt_bs, int f16, int M, int N, int K, int tile, int split_k, void* ws, size_t ws_bytes, void* stream) {
  DenseVt v;
  v.vt = vt;
  v.col0 = vt_col0;
  v.ld = vt_ld;
  v.rows = vt_rows;
  v.bs = vt_bs;
  return dense_common(x, ldx, w_packed, bias, 0, y, ldy, nullptr, 0, 0, M, N, K, tile, split_k, ws, ws_bytes, stream, f16 ? 1 : 0, nullptr, &v);
}

int tk_f16w_dense(const void* x, int ldx, const void* w_packed, const void* bias, int act, void* y, int ldy, const void* resid,
                  int ldr, int resid_dtype, int M, int N, int K, int tile, int split_k, void* ws, size_t ws_bytes, void* stream) {
  return dense_common(x, ldx, w_packed, bias, act, y, ldy, resid, ldr, resid_dtype, M, N, K, tile, split_k, ws, ws_bytes, stream, 1);
}

int tk_quant_act_rows(const void* x, int ldx, void* a8, int lda, void* sa, int M, int K, int mode, void* stream) {
  if (M <= 0 || K <= 0 || K % 8 || K > tk_quant_act_max_k()) return fail(TK_EINVAL, "quant_act_rows: bad shape M=%d K=%d (K a multiple of 8, at most %d)", M, K, tk_quant_act_max_k());
  if (!x || !a8 || !sa || ldx < K || ldx % 8 || lda < K || lda % 8) return fail(TK_EINVAL, "quant_act_rows: null pointer or row pitch not a multiple of 8 >= K");
  if (!aligned16(x) || !aligned8(a8)) return fail(TK_EINVAL, "quant_act_rows: x must be 16-byte and a8 8-byte aligned");
  if (mode != 0 && mode != 1) return fail(TK_EINVAL, "quant_act_rows: mode %d (0 = fp32 scale, 1 = bf16 scale and quotient)", mode);
  QuantActArgs q;
  q.x = (const u16*)x;
  q.ldx = ldx;
  q.a8 = (unsigned char*)a8;
  q.lda = lda;
  q.sa = (float*)sa;
  q.M = M;
  q.K = K;
  q.mode = mode;
  if (tk_launch_quant_act_rows(q, (hipStream_t)stream)) return fail(TK_ELAUNCH, "quant_act_rows: launch failed");
  return TK_OK;
}

int tk_w8a8_gemm(const void* a8, int lda, const void* sa, const void* w_packed, const void* w_scale, void* y, int ldy,
                 const void* resid, int ldr, int resid_dtype, int M, int N, int K, int split_k, void* ws, size_t ws_bytes,
                 void* stream) {
  return w8a8_common(a8, lda, (const float*)sa, w_packed, (const float*)w_scale, nullptr, y, ldy, resid, ldr, resid_dtype, M, N, K,
                     split_k, 0, ws, ws_bytes, (hipStream_t)stream);
}

int tk_w8a8_gated_ffn(const void* x, int ldx, const void* wgu_packed, const void* sg, const void* su, const void* wd_packed,
                      const void* sd, void* y, int ldy, const void* resid, int ldr, int resid_dtype, int M, int K, int I,
                      int act, int quant_mode, void* ws, size_t ws_bytes, void* stream) {
  if (act != TK_ACT_SILU && act != TK_ACT_GELU_TANH) return fail(TK_EINVAL, "w8a8 ffn: unknown activation %d", act);
  if (quant_mode != 0 && quant_mode != 1) return fail(TK_EINVAL, "w8a8 ffn: unknown quantisation mode %d", quant_mode);
  if (M <= 0 || K <= 0 || I <= 0 || I % 32 || K % 16) return fail(TK_EINVAL, "w8a8 ffn: bad shape M=%d K=%d I=%d (K a multiple of 16, I of 32)", M, K, I);
  if (!sg || !su || !sd) return fail(TK_EINVAL, "w8a8 ffn: null scale pointer");
  if (!ws) return fail(TK_EWORKSPACE, "w8a8 ffn: needs a workspace");
  // workspace: quantised input + its scales in the norm region; bf16 intermediate, its codes and scales in the hidden region
  const size_t a8_bytes = (size_t)M * K, sa_bytes = (((size_t)M * 4) + 255) / 256 * 256;
  const size_t h_bytes = (size_t)M * I * 2, h8_bytes = (size_t)M * I;
  if (a8_bytes + sa_bytes > kNormBytes || h_bytes + h8_bytes + sa_bytes > kHiddenBytes || ws_bytes < kHiddenOff + h_bytes + h8_bytes + sa_bytes)
    return fail(TK_EWORKSPACE, "w8a8 ffn: workspace too small for M=%d K=%d I=%d", M, K, I);
  char* base = (char*)ws;
  void* a8 = base + kNormOff;
  void* sa = base + kNormOff + (a8_bytes + 255) / 256 * 256;
  if ((a8_bytes + 255) / 256 * 256 + sa_bytes > kNormBytes) return fail(TK_EWORKSPACE, "w8a8 ffn: workspace too small for the quantised input");
  void* h = base + kHiddenOff;
  void* h8 = base + kHiddenOff + (h_bytes + 255) / 256 * 256;
  void* sh = base + kHiddenOff + (h_bytes + 255) / 256 * 256 + (h8_bytes + 255) / 256 * 256;
  if ((size_t)((char*)sh - base) + sa_bytes > ws_bytes) return fail(TK_EWORKSPACE, "w8a8 ffn: workspace too small for the intermediate");
  hipStream_t st = (hipStream_t)stream;
  int rc = tk_quant_act_rows(x, ldx, a8, K, sa, M, K, quant_mode, stream);
  if (rc) return rc;
  rc = w8a8_common(a8, K, (const float*)sa, wgu_packed, (const float*)sg, (const float*)su, h, I, nullptr, 0, 0, M, I, K, 0, act, ws, ws_bytes, st);
  if (rc) return rc;
  rc = tk_quant_act_rows(h, I, h8, I, sh, M, I, quant_mode, stream);
  if (rc) return rc;
  return w8a8_common(h8, I, (const float*)sh, wd_packed, (const float*)sd, nullptr, y, ldy, resid, ldr, resid_dtype, M, K, I, 0, 0, ws, ws_bytes, st);
}

int tk_w8a8_ffn_layout(int M, int K, int I, size_t* h_off, size_t* h8_off, size_t* sh_off) {
  if (M <= 0 || K <= 0 || I <= 0 || !h_off || !h8_off || !sh_off) return fail(TK_EINVAL, "w8a8 ffn layout: bad argument");
  const size_t h_bytes = (size_t)M * I * 2, h8_bytes = (size_t)M * I;
  *h_off = kHiddenOff;
  *h8_off = kHiddenOff + (h_bytes + 255) / 256 * 256;
  *sh_off = *h8_off + (h8_bytes + 255) / 256 * 256;
  return TK_OK;
}

size_t tk_bf16w_packed_bytes(int N, int K) {
  if (N <= 0 || K <= 0) return 0;
  return (size_t)((N + 31) / 32) * ((K + 31) / 32) * 2048;
}

int tk_pack_bf16_weight(const void* w, void* packed, int N, int K, int rope_half, void* stream) {
  if (!w || !packed || N <= 0 || K <= 0) return fail(TK_EINVAL, "pack_bf16: bad argument");
  if (K % 16) return fail(TK_EINVAL, "pack_bf16: K=%d must be a multiple of 16", K);
  if (!aligned16(w) || !aligned16(packed)) return fail(TK_EINVAL, "pack_bf16: pointers must be 16-byte aligned");
  if (rope_half && (rope_half % 32 || N % (2 * rope_half)))
    return fail(TK_EINVAL, "pack_bf16: rope_half=%d must be a multiple of 32 and 2*rope_half divide N=%d", rope_half, N);
  if (tk_launch_pack_bf16(w, packed, N, K, rope_half / 32, (hipStream_t)stream))
    return fail(TK_ELAUNCH, "pack_bf16: launch failed");
  return TK_OK;
}

int tk_bf16w_linear(const void* x, int ldx, int x_dtype, const void* w_packed, const void* norm_w, float norm_eps,
                    const void* ada_scale, const void* ada_shift, const void* rope_pos, const void* rope_cos,
                    const void* rope_sin, int rope_positions, int rope_cols, int rope_half, int rope_bf16, void* vt,
                    int vt_col0, int vt_ld, void* y, int ldy, const void* resid, int ldr, int resid_dtype, const void* gate,
                    int M, int N, int K, int split_k, void* ws, size_t ws_bytes, void* stream) {
  if (x_dtype != TK_BF16 && x_dtype != TK_F32) return fail(TK_EINVAL, "bf16w_linear: bad x_dtype");
  GemmExtra e;
  e.x_f32 = x_dtype == TK_F32;
  e.w16 = 1;
  e.norm_w = norm_w;
  e.norm_eps = norm_eps;
  e.ada_scale = ada_scale;
  e.ada_shift = ada_shift;
  e.rope_pos = (const int*)rope_pos;
  e.rope_cos = (const float*)rope_cos;
  e.rope_sin = (const float*)rope_sin;
  e.rope_positions = rope_positions;
  e.rope_cols = rope_cols;
  e.rope_half = rope_half;
  e.rope_bf16 = rope_bf16;
  e.vt = vt;
  e.vt_col0 = vt_col0;
  e.vt_ld = vt_ld;
  if (!rope_pos && (norm_w || ada_scale))
    return fail(TK_EINVAL, "bf16w_linear: the norm prologues are built for the rotary projection only");
  return gemm_common(x, ldx, w_packed, nullptr, nullptr, y, ldy, resid, ldr, resid_dtype, gate, M, N, K, split_k, 0, ws,
                     ws_bytes, (hipStream_t)stream, e);
}

int tk_fp8w_norm_gated_ffn(const void* x, int ldx, const void* norm_w, float norm_eps, const void* ada_scale,
                           const void* ada_shift, const void* wgu_packed,
                           const void* sg, const void* su, const void* wd_packed, const void* sd, void* y, int ldy,
                           const void* resid, int ldr, int resid_dtype, const void* gate, int M, int K, int I, int act,
                           void* ws, size_t ws_bytes, void* stream) {
  if (act != TK_ACT_SILU && act != TK_ACT_GELU_TANH) return fail(TK_EINVAL, "ffn: unknown activation %d", act);
  if (M <= 0 || K <= 0 || I <= 0) return fail(TK_EINVAL, "ffn: non-positive shape M=%d K=%d I=%d", M, K, I);
  if (!sg || !su || !sd || (!norm_w && !ada_scale)) return fail(TK_EINVAL, "ffn: null scale or norm pointer");
  if (I % 32) return fail(TK_EINVAL, "ffn: I=%d must be a multiple of 32", I);
  if (!ws) return fail(TK_EWORKSPACE, "ffn: needs a workspace");
  const size_t hbytes = (size_t)M * I * 2;
  if (hbytes > kHiddenBytes || ws_bytes < kHiddenOff + hbytes)
    return fail(TK_EWORKSPACE, "ffn: workspace too small for the [%d, %d] intermediate", M, I);
  void* hbuf = (char*)ws + kHiddenOff;
  GemmExtra e;
  e.norm_w = norm_w;
  e.norm_eps = norm_eps;
  e.ada_scale = ada_scale;
  e.ada_shift = ada_shift;
  return ffn_launches(x, ldx, e, wgu_packed, sg, su, hbuf, wd_packed, sd, y, ldy, resid, ldr, resid_dtype, gate, M, K, I, act, ws, ws_bytes,
                      (hipStream_t)stream);
}

int tk_attn_prepare_kv(const void* k, const void* v, int kv_dtype, int sl, int sh, int L, int G, int D, void* k_hi,
                       void* k_lo, void* vt_hi, void* vt_lo, int vt_ld, void* stream) {
  if (L <= 0 || G <= 0 || D <= 0 || D % 8) return fail(TK_EINVAL, "prepare_kv: bad shape L=%d G=%d D=%d", L, G, D);
  if (kv_dtype != TK_BF16 && kv_dtype != TK_F32) return fail(TK_EINVAL, "prepare_kv: bad kv_dtype");
  if (vt_ld < ((L + 31) / 32) * 32 || vt_ld % 8) return fail(TK_EINVAL, "prepare_kv: vt_ld=%d must be >= L rounded up to 32", vt_ld);
  if (!v || !vt_hi) return fail(TK_EINVAL, "prepare_kv: null pointer");
  if (kv_dtype == TK_F32 && (!k || !k_hi || !k_lo || !vt_lo)) return fail(TK_EINVAL, "prepare_kv: fp32 sources need all four planes");
  KvPrepArgs p;
  p.k = k;
  p.v = v;
  p.f32 = kv_dtype == TK_F32;
  p.sl = sl;
  p.sh = sh;
  p.L = L;
  p.G = G;
  p.D = D;
  p.k_hi = (u16*)k_hi;
  p.k_lo = (u16*)k_lo;
  p.vt_hi = (u16*)vt_hi;
  p.vt_lo = (u16*)vt_lo;
  p.ld = vt_ld;
  if (tk_launch_kv_prepare(p, (hipStream_t)stream)) return fail(TK_ELAUNCH, "prepare_kv: launch failed");
  return TK_OK;
}

static int kv_project_impl(int L, const void* const* k, const void* const* v, int sl, int P, int KV, const void* const* wk,
                           const void* const* wv, int N, void* k_hi, void* k_lo, void* vt_hi, void* vt_lo, int vt_ld, void* stream) {
  if (L < 1 || L > kKvProjMaxLayers) return fail(TK_EINVAL, "kv_project: %d layers in one launch (1..%d)", L, kKvProjMaxLayers);
  if (P <= 0 || KV <= 0 || N <= 0 || N % 32 || KV % 16)
    return fail(TK_EINVAL, "kv_project: bad shape P=%d KV=%d N=%d (N a multiple of 32, KV of 16)", P, KV, N);
  if (!k || !v || !wk || !wv || !k_hi || !k_lo || !vt_hi || !vt_lo) return fail(TK_EINVAL, "kv_project: null pointer");
  if (sl < KV || sl % 8) return fail(TK_EINVAL, "kv_project: row stride %d must be >= KV=%d and a multiple of 8", sl, KV);
  if (vt_ld < ((P + 31) / 32) * 32) return fail(TK_EINVAL, "kv_project: vt_ld=%d must hold P rounded up to 32", vt_ld);
  if (!aligned8(k_hi) || !aligned8(k_lo)) return fail(TK_EINVAL, "kv_project: K planes must be 8-byte aligned");
  KvProjArgs a;
  memset(&a, 0, sizeof(a));
  a.L = L;
  for (int l = 0; l < L; ++l) {
    if (!k[l] || !v[l] || !wk[l] || !wv[l]) return fail(TK_EINVAL, "kv_project: null pointer (layer %d)", l);
    if (!aligned16(k[l]) || !aligned16(v[l]) || !aligned16(wk[l]) || !aligned16(wv[l])) return fail(TK_EINVAL, "kv_project: inputs must be 16-byte aligned");
    a.k[l] = (const u16*)k[l];
    a.v[l] = (const u16*)v[l];
    a.wk[l] = (const float*)wk[l];
    a.wv[l] = (const float*)wv[l];
  }
  a.sl = sl;
  a.P = P;
  a.KV = KV;
  a.N = N;
  a.k_hi = (u16*)k_hi;
  a.k_lo = (u16*)k_lo;
  a.vt_hi = (u16*)vt_hi;
  a.vt_lo = (u16*)vt_lo;
  a.ld = vt_ld;
  if (tk_launch_kv_proj(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "kv_project: launch failed");
  return TK_OK;
}

int tk_expert_kv_project(const void* k, const void* v, int sl, int P, int KV, const void* wk, const void* wv, int N,
                         void* k_hi, void* k_lo, void* vt_hi, void* vt_lo, int vt_ld, void* stream) {
  return kv_project_impl(1, &k, &v, sl, P, KV, &wk, &wv, N, k_hi, k_lo, vt_hi, vt_lo, vt_ld, stream);
}

int tk_expert_kv_project_layers(int layers, const void* const* k, const void* const* v, int sl, int P, int KV, const void* const* wk,
                                const void* const* wv, int N, void* k_hi, void* k_lo, void* vt_hi, void* vt_lo, int vt_ld,
                                void* stream) {
  return kv_project_impl(layers, k, v, sl, P, KV, wk, wv, N, k_hi, k_lo, vt_hi, vt_lo, vt_ld, stream);
}

static int attn_impl(int batch, long long q_sb, long long k_sb, long long vt_sb, long long out_sb, const void* q, int q_sm, int q_sh, const void* k_pre, const void* k_pre_lo, int pre_sl, int pre_sh,
                   const void* vt_pre, const void* vt_pre_lo, int pre_vt_sd, int pre_vt_sh, const void* k_suf, int suf_sl,
                   int suf_sh, const void* vt_suf, int suf_vt_sd, int suf_vt_sh, const void* pad, const void* mask2d,
                   int mask_ld, void* out, int out_sm, int M, int P, int S, int H, int G, int D, int mask_mode,
                   int logits_bf16, float scale, void* ws, size_t ws_bytes, void* stream) {
  if (M <= 0 || P < 0 || S < 0 || P + S <= 0 || H <= 0 || G <= 0 || H % G)
    return fail(TK_EINVAL, "attn: bad shape M=%d P=%d S=%d H=%d G=%d", M, P, S, H, G);
  if (D != 64 && D != 96 && D != 128 && D != 256) return fail(TK_EINVAL, "attn: head_dim %d not in {64,96,128,256}", D);
  if (!(scale >= 0.f)) return fail(TK_EINVAL, "attn: negative or NaN scale");
  const bool split = k_pre_lo != nullptr || vt_pre_lo != nullptr;
  if (split && (!k_pre_lo || !vt_pre_lo)) return fail(TK_EINVAL, "attn: hi/lo planes need both K and V^T low planes");
  if (split && (S != 0 || D != 64))
    return fail(TK_EINVAL, "attn: hi/lo (fp32) K/V is supported for prefix-only attention with head_dim 64");
  if (mask_mode < 0 || mask_mode > 2) return fail(TK_EINVAL, "attn: bad mask_mode %d", mask_mode);
  if (S > 0 && mask_mode == TK_MASK_NONE) return fail(TK_EINVAL, "attn: suffix keys need a suffix mask mode");
  if (!q || !out || (P > 0 && (!k_pre || !vt_pre)) || (S > 0 && (!k_suf || !vt_suf)))
    return fail(TK_EINVAL, "attn: null pointer");
  if (q_sm % 8 || q_sh % 8 || (P > 0 && (pre_sl % 8 || pre_sh % 8 || pre_vt_sd % 8 || pre_vt_sh % 8)) ||
      (S > 0 && (suf_sl % 8 || suf_sh % 8 || suf_vt_sd % 8 || suf_vt_sh % 8)))
    return fail(TK_EINVAL, "attn: strides must be multiples of 8 elements");
  if (!aligned16(q) || !aligned16(k_pre) || !aligned16(vt_pre) || !aligned16(k_pre_lo) || !aligned16(vt_pre_lo) ||
      !aligned16(k_suf) || !aligned16(vt_suf))
    return fail(TK_EINVAL, "attn: q/k/v^T must be 16-byte aligned");
  if ((P > 0 && pre_vt_sd < ((P + 31) / 32) * 32) || (S > 0 && suf_vt_sd < ((S + 31) / 32) * 32))
    return fail(TK_EINVAL, "attn: a V^T row must hold the segment length rounded up to 32 keys (zero padded)");
  if (mask2d && (mask_ld % 8 || mask_ld < ((P + 31) / 32) * 32 || !aligned8(mask2d)))
    return fail(TK_EINVAL, "attn: mask2d rows must be 8-byte aligned and hold P rounded up to 32 bytes");
  if (out_sm < H * D || out_sm % 4 || !aligned8(out)) return fail(TK_EINVAL, "attn: out_sm=%d must be >= H*D, a multiple of 4, out 8-byte aligned", out_sm);

  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.q = (const u16*)q;
  a.q_sm = q_sm;
  a.q_sh = q_sh;
  a.k_pre = (const u16*)k_pre;
  a.k_pre_lo = (const u16*)k_pre_lo;
  a.vt_pre = (const u16*)vt_pre;
  a.vt_pre_lo = (const u16*)vt_pre_lo;
  a.pre_sl = pre_sl;
  a.pre_sh = pre_sh;
  a.pre_vt_sd = pre_vt_sd;
  a.pre_vt_sh = pre_vt_sh;
  a.k_suf = (const u16*)k_suf;
  a.vt_suf = (const u16*)vt_suf;
  a.suf_sl = suf_sl;
  a.suf_sh = suf_sh;
  a.suf_vt_sd = suf_vt_sd;
  a.suf_vt_sh = suf_vt_sh;
  a.pad = (const uint8_t*)pad;
  a.mask2d = (const uint8_t*)mask2d;
  a.mask_ld = mask_ld;
  a.out = (u16*)out;
  a.out_sm = out_sm;
  a.M = M;
  a.batch = batch;
  a.q_sb = q_sb;
  a.k_sb = k_sb;
  a.vt_sb = vt_sb;
  a.out_sb = out_sb;
  a.P = P;
  a.S = S;
  a.H = H;
  a.G = G;
  a.mask_mode = mask_mode;
  a.logits_bf16 = logits_bf16 == 1;
  a.f16 = logits_bf16 == 2;
  a.scale = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
  if (a.f16 && !(batch > 0 && !split && S == 0 && !mask2d && !pad && D == 96 && P >= 128 && M >= 128))
    return fail(TK_EINVAL, "attn: fp16 operands are built for the batched tower shape only (D = 96, >= 128 queries and keys)");

  if (batch > 0 && !split && S == 0 && !mask2d && !pad && (D == 64 || D == 96) && P >= 128 && M >= 128) {
    // vision towers: many query tiles over a long key range -- K / V^T staged through LDS once per 128 queries
    a.gqa_mul = (65536 + H / G - 1) / (H / G);
    int rc = tk_launch_tower_attn(a, D, device_cus(), (hipStream_t)stream);
    if (rc) return fail(TK_ELAUNCH, "attn: launch failed (%s)", hipGetErrorString(hipGetLastError()));
    return TK_OK;
  }
  const int ntiles = (P + 31) / 32 + (S + 31) / 32;
  const int mtiles = ((M + 31) / 32) * (batch > 0 ? batch : 1);
  // one 32-key tile per wave: split the keys over blocks of four waves (at most 8 splits, beyond
  // that a wave loops over several tiles)
  const int waves = tk_attn_waves(D, split ? 1 : 0, ntiles);
  int splits = (ntiles + waves - 1) / waves;
  if (splits < 1) splits = 1;
  if (splits > (D > 128 ? 7 : 8)) splits = D > 128 ? 7 : 8;
  // many query tiles already fill the device: keep whole key ranges in one block (no partials)
  while (splits > 1 && H * mtiles * splits > 2 * device_cus()) --splits;
  // 256-wide heads (pi0.5): blocks of 8 waves that cut the two products along different axes and walk the
  // keys 8 tiles at a time; one round per block while that leaves the device room, else several
  bool d256 = false;
  if (D == 256 && !split && batch == 0) {
    const int per = tk_attn_d256_tiles_per_block();
    int sp = (ntiles + per - 1) / per;
    if (sp > tk_attn_d256_max_splits()) sp = tk_attn_d256_max_splits();
    if (H * mtiles * 2 >= device_cus()) sp = 1;  // the query tiles alone fill half the device: no hand-off
    while (sp > 1 && H * mtiles * sp > 2 * device_cus()) --sp;
    // (a statistics record and an arrival counter per wave: the waves of a block hand over on their own)
    const size_t need = (size_t)H * mtiles * sp * (size_t)(D / 32) * (64 + 1024) * 4;
    if (sp > 1 && !(ws && H * mtiles * (D / 32) * 16 <= kMaxCounters && need <= kPartialBytes && ws_bytes >= kPartialOff + need)) sp = 1;
    d256 = true;
    splits = sp;
  }
  // 64-wide heads, whole key range in one block (the SmolVLA self layers and prefill)
  const bool px = D == 64 && !split && batch == 0 && ntiles <= tk_attn_px_max_tiles();
  if (px) splits = 1;
  a.kv_splits = splits;
  a.tile_q = ntiles / splits;
  a.tile_r = ntiles % splits;
  a.gqa_mul = (65536 + H / G - 1) / (H / G);
  a.xcd_remap = (batch > 0 && splits == 1 && H * mtiles >= 2 * device_cus()) ? 1 : 0;
  a.partial = nullptr;
  a.counters = nullptr;
  if (splits > 1) {
    const int blocks = H * mtiles * (d256 ? (D / 32) * 16 : 1);  // arrival counters (256-wide heads: one per wave, a 64-byte line each)
    const size_t need = d256 ? (size_t)H * mtiles * splits * (size_t)(D / 32) * (64 + 1024) * 4
                             : (size_t)blocks * splits * (64 + (size_t)(D / 32) * 1024) * 4;
    if (!ws || blocks > kMaxCounters || need > kPartialBytes || ws_bytes < kPartialOff + need)
      return fail(TK_EWORKSPACE, "attn: workspace too small (need %zu bytes)", need);
    a.partial = (float*)((char*)ws + kPartialOff);
    a.counters = (int*)ws;
  }
  int rc = d256 ? tk_launch_attn_d256(a, (hipStream_t)stream) : px ? tk_launch_attn_px(a, D, (hipStream_t)stream) : tk_launch_attn(a, D, waves, (hipStream_t)stream);
  if (rc) return fail(TK_ELAUNCH, "attn: launch failed (%s)", hipGetErrorString(hipGetLastError()));
  return TK_OK;
}

int tk_expert_attn(const void* q, int q_sm, int q_sh, const void* k_pre, const void* k_pre_lo, int pre_sl, int pre_sh,
                   const void* vt_pre, const void* vt_pre_lo, int pre_vt_sd, int pre_vt_sh, const void* k_suf, int suf_sl,
                   int suf_sh, const void* vt_suf, int suf_vt_sd, int suf_vt_sh, const void* pad, const void* mask2d,
                   int mask_ld, void* out, int out_sm, int M, int P, int S, int H, int G, int D, int mask_mode,
                   int logits_bf16, void* ws, size_t ws_bytes, void* stream) {
  return attn_impl(0, 0, 0, 0, 0, q, q_sm, q_sh, k_pre, k_pre_lo, pre_sl, pre_sh, vt_pre, vt_pre_lo, pre_vt_sd, pre_vt_sh, k_suf,
                   suf_sl, suf_sh, vt_suf, suf_vt_sd, suf_vt_sh, pad, mask2d, mask_ld, out, out_sm, M, P, S, H, G, D, mask_mode,
                   logits_bf16, 0.f, ws, ws_bytes, stream);
}

int tk_expert_cross_attn_fused(const void* x, int ldx, const void* norm_w, float norm_eps, const void* wq_packed, int K,
                               const void* rope_pos, const void* rope_cos, const void* rope_sin, int rope_positions,
                               const void* k_hi, const void* k_lo, int pre_sl, int pre_sh, const void* vt_hi,
                               const void* vt_lo, int pre_vt_sd, int pre_vt_sh, const void* pad, void* out, int out_sm,
                               int M, int P, int H, int G, int D, void* stream) {
  if (M <= 0 || P <= 0 || H <= 0 || G <= 0 || H % G) return fail(TK_EINVAL, "cross_attn_fused: bad shape M=%d P=%d H=%d G=%d", M, P, H, G);
  if (D != 64) return fail(TK_EINVAL, "cross_attn_fused: head_dim %d (built for 64)", D);
  if ((P + 31) / 32 > 8) return fail(TK_EINVAL, "cross_attn_fused: P=%d needs more than 8 key tiles (one block of 8 waves covers the prefix)", P);
  if (K <= 0 || K % 8 || K > 768 || ldx < K || ldx % 8) return fail(TK_EINVAL, "cross_attn_fused: K=%d must be a multiple of 8, at most 768, ldx=%d >= K and a multiple of 8", K, ldx);
  if (!x || !norm_w || !wq_packed || !rope_pos || !rope_cos || !rope_sin || rope_positions <= 0 || !k_hi || !k_lo || !vt_hi || !vt_lo || !out)
    return fail(TK_EINVAL, "cross_attn_fused: null pointer");
  if (pre_sl % 8 || pre_sh % 8 || pre_vt_sd % 8 || pre_vt_sh % 8) return fail(TK_EINVAL, "cross_attn_fused: strides must be multiples of 8 elements");
  if (!aligned16(x) || !aligned16(norm_w) || !aligned16(wq_packed) || !aligned16(rope_cos) || !aligned16(rope_sin) || !aligned16(k_hi) ||
      !aligned16(k_lo) || !aligned16(vt_hi) || !aligned16(vt_lo))
    return fail(TK_EINVAL, "cross_attn_fused: operands must be 16-byte aligned");
  if (pre_vt_sd < ((P + 31) / 32) * 32) return fail(TK_EINVAL, "cross_attn_fused: a V^T row must hold P rounded up to 32 keys (zero padded)");
  if (out_sm < H * D || out_sm % 4 || !aligned8(out)) return fail(TK_EINVAL, "cross_attn_fused: out_sm=%d must be >= H*D, a multiple of 4, out 8-byte aligned", out_sm);
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.q = (const u16*)x;  // never read as queries; keeps the kernel's dummy operand address valid
  a.k_pre = (const u16*)k_hi;
  a.k_pre_lo = (const u16*)k_lo;
  a.vt_pre = (const u16*)vt_hi;
  a.vt_pre_lo = (const u16*)vt_lo;
  a.pre_sl = pre_sl;
  a.pre_sh = pre_sh;
  a.pre_vt_sd = pre_vt_sd;
  a.pre_vt_sh = pre_vt_sh;
  a.pad = (const uint8_t*)pad;
  a.out = (u16*)out;
  a.out_sm = out_sm;
  a.M = M;
  a.P = P;
  a.H = H;
  a.G = G;
  a.mask_mode = TK_MASK_NONE;
  a.scale = 1.0f / sqrtf((float)D);
  a.kv_splits = 1;
  a.tile_q = (P + 31) / 32;
  a.gqa_mul = (65536 + H / G - 1) / (H / G);
  a.qp_x = (const u16*)x;
  a.qp_ldx = ldx;
  a.qp_norm_w = (const u16*)norm_w;
  a.qp_eps = norm_eps;
  a.qp_w = (const uint8_t*)wq_packed;
  a.qp_K = K;
  a.qp_KT = (K + 31) / 32;
  a.qp_rope_pos = (const int*)rope_pos;
  a.qp_cos = (const float*)rope_cos;
  a.qp_sin = (const float*)rope_sin;
  a.qp_positions = rope_positions;
  if (tk_launch_attn_cross_px(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "cross_attn_fused: launch failed (%s)", hipGetErrorString(hipGetLastError()));
  return TK_OK;
}

int tk_batched_attn(const void* q, long long q_sb, int q_sm, int q_sh, const void* k, long long k_sb, int k_sl, int k_sh,
                    const void* vt, long long vt_sb, int vt_sd, int vt_sh, void* out, long long out_sb, int out_sm, int B,
                    int M, int P, int H, int G, int D, int logits_bf16, float scale, void* ws, size_t ws_bytes, void* stream) {
  if (B <= 0) return fail(TK_EINVAL, "batched_attn: B=%d", B);
  if (q_sb % 8 || k_sb % 8 || vt_sb % 8 || out_sb % 4) return fail(TK_EINVAL, "batched_attn: batch strides must keep 16-byte alignment");
  return attn_impl(B, q_sb, k_sb, vt_sb, out_sb, q, q_sm, q_sh, k, nullptr, k_sl, k_sh, vt, nullptr, vt_sd, vt_sh, nullptr, 0, 0,
                   nullptr, 0, 0, nullptr, nullptr, 0, out, out_sm, M, P, 0, H, G, D, TK_MASK_NONE, logits_bf16, scale, ws,
                   ws_bytes, stream);
}

int tk_batched_transpose_v(const void* v, long long v_sb, int v_sl, int v_sh, void* vt, long long vt_sb, int vt_sh, int vt_sd,
                           int vt_keys, int B, int P, int G, int D, void* stream) {
  if (B <= 0 || P <= 0 || G <= 0) return fail(TK_EINVAL, "transpose_v: bad shape B=%d P=%d G=%d", B, P, G);
  if (D != 64 && D != 96) return fail(TK_EINVAL, "transpose_v: head_dim %d not in {64, 96}", D);
  if (!v || !vt || !aligned16(v) || !aligned16(vt)) return fail(TK_EINVAL, "transpose_v: null or unaligned pointer");
  if (v_sb % 8 || v_sl % 8 || v_sh % 8 || vt_sb % 8 || vt_sh % 8 || vt_sd % 8 || vt_keys % 8)
    return fail(TK_EINVAL, "transpose_v: strides must be multiples of 8 elements");
  if (vt_keys < ((P + 31) / 32) * 32 || vt_sd < vt_keys) return fail(TK_EINVAL, "transpose_v: a V^T row must hold P rounded up to 32 keys (vt_keys=%d, vt_sd=%d)", vt_keys, vt_sd);
  TransposeVArgs a;
  a.v = (const u16*)v;
  a.v_sb = v_sb;
  a.v_sl = v_sl;
  a.v_sh = v_sh;
  a.vt = (u16*)vt;
  a.vt_sb = vt_sb;
  a.vt_sh = vt_sh;
  a.vt_sd = vt_sd;
  a.ld = vt_keys;
  a.B = B;
  a.P = P;
  a.G = G;
  if (tk_launch_transpose_v(a, D, (hipStream_t)stream)) return fail(TK_ELAUNCH, "transpose_v: launch failed");
  return TK_OK;
}

static int tail_impl(const void* x, int ldx, const void* norm_w, const void* ada_scale, const void* ada_shift, float eps,
                     const void* w, const void* bias, void* v_out, const void* x_t, void* x_out, float dt, int M, int N, int K,
                     const void* emb_w, const void* emb_b, int emb_n, int emb_act, void* emb_out, int emb_ld, int emb_dtype,
                     void* stream) {
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K) return fail(TK_EINVAL, "tail: bad shape M=%d N=%d K=%d ldx=%d", M, N, K, ldx);
  if (N > 256 || 256 % N) return fail(TK_EINVAL, "tail: N=%d must divide 256", N);
  // (the normalised row lives in LDS as fp32: 32 KiB at the limit)
  if (K > 8192 || K % 4) return fail(TK_EINVAL, "tail: K=%d must be a multiple of 4 and at most 8192", K);
  if (!aligned16(w)) return fail(TK_EINVAL, "tail: w must be 16-byte aligned");
  if (!x || !w || (!norm_w && !(ada_scale && ada_shift)) || (norm_w && (ada_scale || ada_shift)))
    return fail(TK_EINVAL, "tail: needs x, w and exactly one of norm_w or ada_scale + ada_shift");
  if (x_out && !x_t) return fail(TK_EINVAL, "tail: x_out needs x_t");
  if (!v_out && !x_out) return fail(TK_EINVAL, "tail: no output requested");
  TailArgs a;
  a.x = (const u16*)x;
  a.ldx = ldx;
  a.norm_w = (const u16*)norm_w;
  a.ada_scale = (const float*)ada_scale;
  a.ada_shift = (const float*)ada_shift;
  a.eps = eps;
  a.w = (const float*)w;
  a.bias = (const float*)bias;
  a.v_out = (float*)v_out;
  a.x_t = (const float*)x_t;
  a.x_out = (float*)x_out;
  a.dt = dt;
  a.M = M;
  a.N = N;
  a.K = K;
  a.emb_w = nullptr;
  a.emb_b = nullptr;
  a.emb_out = nullptr;
  a.emb_J = a.emb_ld = a.emb_act = a.emb_bf16 = 0;
  if (emb_out) {
    if (!x_out) return fail(TK_EINVAL, "tail: the embedding is computed from x_out");
    if (N != tk_tail_embed_width()) return fail(TK_EINVAL, "tail: the embedding takes N=%d inputs, got %d", tk_tail_embed_width(), N);
    if (!emb_w || !aligned16(emb_w)) return fail(TK_EINVAL, "tail: emb_w must be a 16-byte aligned fp32 [emb_n, N] matrix");
    if (emb_n <= 0 || emb_ld < emb_n) return fail(TK_EINVAL, "tail: bad embedding shape emb_n=%d emb_ld=%d", emb_n, emb_ld);
    if (emb_act != 0 && emb_act != 1) return fail(TK_EINVAL, "tail: emb_act=%d must be 0 (none) or 1 (SiLU)", emb_act);
    if (emb_dtype != TK_BF16 && emb_dtype != TK_F32) return fail(TK_EINVAL, "tail: emb_dtype=%d", emb_dtype);
    a.emb_w = (const float*)emb_w;
    a.emb_b = (const float*)emb_b;
    a.emb_out = emb_out;
    a.emb_J = emb_n;
    a.emb_ld = emb_ld;
    a.emb_act = emb_act;
    a.emb_bf16 = emb_dtype == TK_BF16;
  }
  if (tk_launch_tail(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "tail: launch failed");
  return TK_OK;
}

int tk_expert_tail(const void* x, int ldx, const void* norm_w, const void* ada_scale, const void* ada_shift, float eps,
                   const void* w, const void* bias, void* v_out, const void* x_t, void* x_out, float dt, int M, int N, int K,
                   void* stream) {
  return tail_impl(x, ldx, norm_w, ada_scale, ada_shift, eps, w, bias, v_out, x_t, x_out, dt, M, N, K, nullptr, nullptr, 0, 0,
                   nullptr, 0, 0, stream);
}

int tk_expert_tail_embed(const void* x, int ldx, const void* norm_w, const void* ada_scale, const void* ada_shift, float eps,
                         const void* w, const void* bias, void* v_out, const void* x_t, void* x_out, float dt, int M, int N,
                         int K, const void* emb_w, const void* emb_b, int emb_n, int emb_act, void* emb_out, int emb_ld,
                         int emb_dtype, void* stream) {
  if (!emb_out) return fail(TK_EINVAL, "tail: emb_out is null");
  return tail_impl(x, ldx, norm_w, ada_scale, ada_shift, eps, w, bias, v_out, x_t, x_out, dt, M, N, K, emb_w, emb_b, emb_n, emb_act,
                   emb_out, emb_ld, emb_dtype, stream);
}

int tk_rms_norm_rows(const void* x, int ldx, const void* norm_w, const void* ada_scale, const void* ada_shift, float eps, void* y,
                     int ldy, int M, int K, void* stream) {
  if (M <= 0 || K <= 0 || K % 8) return fail(TK_EINVAL, "rms_norm_rows: bad shape M=%d K=%d (K a multiple of 8)", M, K);
  if (!x || !y || ldx < K || ldy < K || ldx % 8 || ldy % 8) return fail(TK_EINVAL, "rms_norm_rows: null pointer or row pitch not a multiple of 8 >= K");
  if ((norm_w != nullptr) == (ada_scale != nullptr) || (ada_scale != nullptr) != (ada_shift != nullptr))
    return fail(TK_EINVAL, "rms_norm_rows: needs exactly one of norm_w or ada_scale + ada_shift");
  if (!aligned16(x) || !aligned16(y) || !aligned16(norm_w) || !aligned16(ada_scale) || !aligned16(ada_shift))
    return fail(TK_EINVAL, "rms_norm_rows: operands must be 16-byte aligned");
  NormRowsArgs a;
  a.x = (const u16*)x;
  a.ldx = ldx;
  a.norm_w = (const u16*)norm_w;
  a.ada_scale = (const float*)ada_scale;
  a.ada_shift = (const float*)ada_shift;
  a.eps = eps;
  a.out = (u16*)y;
  a.ldo = ldy;
  a.M = M;
  a.K = K;
  if (tk_launch_norm_rows(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "rms_norm_rows: launch failed");
  return TK_OK;
}

int tk_rope_rows(void* y, int ldy, const void* rope_pos, const void* rope_cos, const void* rope_sin, int rope_positions,
                 int rope_cols, int rope_half, int rope_bf16, int M, void* stream) {
  if (M <= 0 || rope_cols <= 0 || rope_half < 8 || rope_half % 8 || rope_cols % (2 * rope_half))
    return fail(TK_EINVAL, "rope_rows: bad shape M=%d rope_cols=%d rope_half=%d (half a multiple of 8, cols of the head size)", M, rope_cols, rope_half);
  if (!y || !rope_pos || !rope_cos || !rope_sin || rope_positions <= 0) return fail(TK_EINVAL, "rope_rows: null pointer or empty table");
  if (ldy < rope_cols || ldy % 8 || !aligned16(y) || !aligned16(rope_cos) || !aligned16(rope_sin))
    return fail(TK_EINVAL, "rope_rows: ldy=%d must be >= rope_cols and a multiple of 8; y and the tables 16-byte aligned", ldy);
  RopeRowsArgs a;
  a.y = (u16*)y;
  a.ldy = ldy;
  a.pos = (const int*)rope_pos;
  a.cos = (const float*)rope_cos;
  a.sin = (const float*)rope_sin;
  a.positions = rope_positions;
  a.rope_cols = rope_cols;
  a.half = rope_half;
  a.bf16_math = rope_bf16;
  a.M = M;
  if (tk_launch_rope_rows(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "rope_rows: launch failed");
  return TK_OK;
}

int tk_prefix_meta(const void* pad, const void* att, int P, int p_pad, int rope_positions, int S, void* mask2d, void* pos32,
                   void* suf_pos, void* stream) {
  if (P <= 0 || P > tk_prefix_meta_max_tokens()) return fail(TK_EINVAL, "prefix_meta: P=%d must be in 1..%d", P, tk_prefix_meta_max_tokens());
  if (!pad || rope_positions <= 0 || S < 0 || (S > 0 && !suf_pos)) return fail(TK_EINVAL, "prefix_meta: null pad flags, empty position range or S without an output");
  if (mask2d && (p_pad < P || p_pad % 16 || !aligned16(mask2d))) return fail(TK_EINVAL, "prefix_meta: p_pad=%d must be a multiple of 16 >= P and the mask 16-byte aligned", p_pad);
  PrefixMetaArgs a;
  a.pad = (const unsigned char*)pad;
  a.att = (const unsigned char*)att;
  a.P = P;
  a.p_pad = p_pad;
  a.positions = rope_positions;
  a.S = S;
  a.mask2d = (unsigned char*)mask2d;
  a.pos = (int*)pos32;
  a.suf_pos = (int*)suf_pos;
  if (tk_launch_prefix_meta(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "prefix_meta: launch failed");
  return TK_OK;
}

static int patchify_impl(const void* const* imgs, int n, int H, int W, int patch, float scale, float shift, void* out, int out_f32,
                         void* stream) {
  const int unit = out_f32 ? 2 : 8;  // pixels per thread: a thread's pixels must not straddle two patches
  if (n < 1 || n > 4 || H <= 0 || W <= 0 || patch <= 0 || patch % unit || H % patch || W % patch)
    return fail(TK_EINVAL, "patchify: n=%d in 1..4, patch=%d a multiple of %d that divides H=%d and W=%d", n, patch, unit, H, W);
  if (!out || !aligned16(out)) return fail(TK_EINVAL, "patchify: the output must be 16-byte aligned");
  PatchifyArgs a;
  for (int i = 0; i < 4; ++i) {
    if (i < n && (!imgs[i] || !aligned16(imgs[i]))) return fail(TK_EINVAL, "patchify: image %d is null or not 16-byte aligned", i);
    a.img[i] = (const float*)imgs[i < n ? i : 0];
  }
  a.n = n;
  a.H = H;
  a.W = W;
  a.ps = patch;
  a.scale = scale;
  a.shift = shift;
  a.out = out;
  a.out_f32 = out_f32;
  if (tk_launch_patchify(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "patchify: launch failed");
  return TK_OK;
}

int tk_patchify_images(const void* img0, const void* img1, const void* img2, const void* img3, int n, int H, int W, int patch,
                       float scale, float shift, void* out, void* stream) {
  const void* imgs[4] = {img0, img1, img2, img3};
  return patchify_impl(imgs, n, H, W, patch, scale, shift, out, 0, stream);
}

int tk_patchify_images_f32(const void* img0, const void* img1, const void* img2, const void* img3, int n, int H, int W, int patch,
                           float scale, float shift, void* out, void* stream) {
  const void* imgs[4] = {img0, img1, img2, img3};
  return patchify_impl(imgs, n, H, W, patch, scale, shift, out, 1, stream);
}

int tk_prefix_rows(const void* img, int img_dtype, int n_img, float img_scale, const void* table, const void* tokens, int n_tok,
                   int vocab, float tok_scale, const void* last, int n_last, void* out, int out_dtype, int H, const void* cam_flag0,
                   const void* cam_flag1, const void* cam_flag2, const void* cam_flag3, int cams, const void* tok_flag, void* pad_out,
                   void* stream) {
  if ((img_dtype != TK_BF16 && img_dtype != TK_F32) || (out_dtype != TK_BF16 && out_dtype != TK_F32))
    return fail(TK_EINVAL, "prefix_rows: image rows and result are bf16 or fp32 (img_dtype=%d, out_dtype=%d)", img_dtype, out_dtype);
  if (n_img < 0 || n_tok < 0 || n_last < 0 || n_img + n_tok + n_last < 1 || H <= 0 || H % 8)
    return fail(TK_EINVAL, "prefix_rows: row counts %d + %d + %d must be non-negative with a row in all, H=%d a multiple of 8", n_img, n_tok,
                n_last, H);
  if (!out || !aligned16(out)) return fail(TK_EINVAL, "prefix_rows: the output is null or not 16-byte aligned");
  if ((n_img && (!img || !aligned16(img))) || (n_last && (!last || !aligned16(last))))
    return fail(TK_EINVAL, "prefix_rows: image rows and closing rows must be 16-byte aligned");
  if (n_tok && (!table || !aligned16(table) || !tokens || ((uintptr_t)tokens & 7) || vocab < 1))
    return fail(TK_EINVAL, "prefix_rows: the token rows need a 16-byte aligned table, vocab >= 1 and 8-byte aligned ids");
  const void* flags[4] = {cam_flag0, cam_flag1, cam_flag2, cam_flag3};
  PrefixRowsArgs a;
  memset(&a, 0, sizeof(a));
  if (pad_out) {
    if (n_img && (cams < 1 || cams > 4 || n_img % cams)) return fail(TK_EINVAL, "prefix_rows: %d image rows do not split over cams=%d (1..4)", n_img, cams);
    for (int i = 0; n_img && i < cams; ++i)
      if (!flags[i]) return fail(TK_EINVAL, "prefix_rows: the flag of camera %d is null", i);
    if (n_tok && !tok_flag) return fail(TK_EINVAL, "prefix_rows: pad flags asked for without the tokens' flags");
    a.cams = n_img ? cams : 1;
    a.per_cam = n_img ? n_img / cams : 1;
    for (int i = 0; i < 4; ++i) a.cam_flag[i] = (const unsigned char*)flags[(n_img && i < cams) ? i : 0];
  }
  a.img = img;
  a.img_f32 = img_dtype == TK_F32;
  a.n_img = n_img;
  a.img_scale = img_scale;
  a.table = (const u16*)table;
  a.tokens = (const long long*)tokens;
  a.n_tok = n_tok;
  a.vocab = vocab;
  a.tok_scale = tok_scale;
  a.last = (const float*)last;
  a.n_last = n_last;
  a.out = out;
  a.out_bf16 = out_dtype == TK_BF16;
  a.H = H;
  a.tok_flag = (const unsigned char*)tok_flag;
  a.pad_out = (unsigned char*)pad_out;
  if (tk_launch_prefix_rows(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "prefix_rows: launch failed");
  return TK_OK;
}

static int layer_norm_impl(const char* who, const void* x, int ldx, int x_dtype, const void* r, int ldr, void* xsum, int ldxs,
                           const void* w, const void* b, int wb_dtype, float eps, void* y, int ldy, int M, int K, void* stream,
                           int y_f16 = 0, const int* y_rows = nullptr) {
  if (M <= 0 || K <= 0 || K % 8 || K > tk_layer_norm_max_k()) return fail(TK_EINVAL, "%s: K=%d must be a multiple of 8, at most %d", who, K, tk_layer_norm_max_k());
  if ((x_dtype != TK_BF16 && x_dtype != TK_F32) || x_dtype != wb_dtype) return fail(TK_EINVAL, "%s: rows and parameters must both be bf16 or both fp32", who);
  if (!x || !w || !b || !y || ldx < K || ldy < K || ldx % 8 || ldy % 8) return fail(TK_EINVAL, "%s: null pointer or row pitch not a multiple of 8 >= K", who);
  if (!aligned16(x) || !aligned16(w) || !aligned16(b) || !aligned16(y)) return fail(TK_EINVAL, "%s: operands must be 16-byte aligned", who);
  if (r && (!xsum || ldr < K || ldxs < K || ldr % 8 || ldxs % 8 || !aligned16(r) || !aligned16(xsum)))
    return fail(TK_EINVAL, "%s: the residual branch and the sum need 16-byte aligned pointers and row pitches that are multiples of 8 >= K", who);
  LayerNormArgs a;
  a.x = x;
  a.ldx = ldx;
  a.x_f32 = x_dtype == TK_F32;
  a.w = w;
  a.b = b;
  a.wb_f32 = wb_dtype == TK_F32;
  a.eps = eps;
  a.y = (u16*)y;
  a.ldy = ldy;
  a.y_f16 = y_f16;
  a.M = M;
  a.K = K;
  a.r = (const u16*)r;
  a.ldr = ldr;
  a.xsum = xsum;
  a.ldxs = ldxs;
  a.y_rows = y_rows;
  if (tk_launch_layer_norm(a, (hipStream_t)stream)) return fail(TK_ELAUNCH, "%s: launch failed", who);
  return TK_OK;
}

int tk_layer_norm(const void* x, int ldx, int x_dtype, const void* w, const void* b, int wb_dtype, float eps, void* y, int ldy,
                  int M, int K, void* stream) {
  return layer_norm_impl("layer_norm", x, ldx, x_dtype, nullptr, 0, nullptr, 0, w, b, wb_dtype, eps, y, ldy, M, K, stream);
}

int tk_add_layer_norm(const void* x, int ldx, int x_dtype, const void* r, int ldr, void* xsum, int ldxs, const void* w,
                      const void* b, int wb_dtype, float eps, void* y, int ldy, int M, int K, void* stream) {
  if (!r) return fail(TK_EINVAL, "add_layer_norm: null residual branch");
  return layer_norm_impl("add_layer_norm", x, ldx, x_dtype, r, ldr, xsum, ldxs, w, b, wb_dtype, eps, y, ldy, M, K, stream);
}

int tk_add_layer_norm_rows(const void* x, int ldx, int x_dtype, const void* r, int ldr, void* xsum, int ldxs, const void* w,
                           const void* b, int wb_dtype, float eps, void* y, int ldy, const void* y_rows, int M, int K, void* stream) {
  if (!r) return fail(TK_EINVAL, "add_layer_norm_rows: null residual branch");
  if (!y_rows || ((uintptr_t)y_rows & 3)) return fail(TK_EINVAL, "add_layer_norm_rows: the row map is null or not 4-byte aligned");
  if (y == xsum || y == x) return fail(TK_EINVAL, "add_layer_norm_rows: rows move, so y must not be x or xsum");
  return layer_norm_impl("add_layer_norm_rows", x, ldx, x_dtype, r, ldr, xsum, ldxs, w, b, wb_dtype, eps, y, ldy, M, K, stream, 0,
                         (const int*)y_rows);
}

int tk_layer_norm_f16(const void* x, int ldx, const void* w, const void* b, float eps, void* y, int ldy, int M, int K, void* stream) {
  return layer_norm_impl("layer_norm_f16", x, ldx, TK_F32, nullptr, 0, nullptr, 0, w, b, TK_F32, eps, y, ldy, M, K, stream, 1);
}

int tk_add_layer_norm_f16(const void* x, int ldx, const void* r, int ldr, void* xsum, int ldxs, const void* w, const void* b, float eps,
                          void* y, int ldy, int M, int K, void* stream) {
  if (!r) return fail(TK_EINVAL, "add_layer_norm_f16: null residual branch");
  return layer_norm_impl("add_layer_norm_f16", x, ldx, TK_F32, r, ldr, xsum, ldxs, w, b, TK_F32, eps, y, ldy, M, K, stream, 1);
}

int tk_debug_stream_read(const void* src, size_t bytes, int blocks, void* sink, void* stream) {
  if (!src || !aligned16(src) || blocks <= 0 || blocks > 65536) return fail(TK_EINVAL, "stream_read: null or unaligned source, or blocks=%d out of range", blocks);
  if (bytes == 0 || bytes % ((size_t)blocks * 4096)) return fail(TK_EINVAL, "stream_read: bytes=%zu must be a positive multiple of blocks * 4096", bytes);
  if (tk_launch_stream_read(src, bytes, blocks, (int*)sink, (hipStream_t)stream)) return fail(TK_ELAUNCH, "stream_read: launch failed");
  return TK_OK;
}

int tk_debug_fp8w_gemm_cut(const void* x, int ldx, const void* w_packed, const void* scale, void* y, int ldy, int M, int N, int K,
                           int cut, void* stream) {
  GemmPlan plan;
  const int rc = gemm_common(x, ldx, w_packed, (const float*)scale, nullptr, y, ldy, nullptr, 0, 0, nullptr, M, N, K, 0, 0, nullptr, 0,
                             (hipStream_t)stream, GemmExtra(), &plan);
  if (rc) return rc;
  if (plan.skinny || plan.a.ksplit != 1 || tk_launch_gemm_stream_cut(plan.a, cut, (hipStream_t)stream))
    return fail(TK_EINVAL, "gemm_cut: only for shapes the 16-round weight-streaming kernel takes unsplit (K = 2048, at most 64 rows), cut 1..4");
  return TK_OK;
}

int tk_debug_decode_fp8(void* out_f32, void* stream) {
  if (!out_f32) return fail(TK_EINVAL, "decode: null pointer");
  if (tk_launch_decode_fp8((float*)out_f32, (hipStream_t)stream)) return fail(TK_ELAUNCH, "decode: launch failed");
  return TK_OK;
}

}  // extern "C"
