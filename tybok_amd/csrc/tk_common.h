// Shared device helpers for the gfx950 kernels (wave64, MFMA 32x32x16 bf16, OCP fp8).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16;

#define TK_WAVE 64

// Workspace layout (bytes): [counters][scratch ...]
#define TK_WS_COUNTER_BYTES (64 * 1024)  // 16384 int32 arrival counters
#define TK_WS_TOTAL_BYTES (128ull * 1024 * 1024)

__device__ __forceinline__ float bf16_bits_to_f32(u16 b) { return __uint_as_float(((unsigned)b) << 16); }

// two fp32 -> packed bf16 pair (lo = a, hi = b), round-to-nearest-even in one v_cvt_pk_bf16_f32
// (NaN stays a quiet NaN), same as torch's cast.
__device__ __forceinline__ unsigned pack_bf16x2(float a, float b) {
  f32x2 v = {a, b};
  union { bf16x2 h; unsigned u; } r;
  r.h = __builtin_convertvector(v, bf16x2);
  return r.u;
}
__device__ __forceinline__ u16 f32_to_bf16_bits(float f) { return (u16)pack_bf16x2(f, 0.f); }
// four fp32 <-> four bf16 in two dwords
__device__ __forceinline__ i32x2 pack_bf16x4(f32x4 v) {
  i32x2 r = {(int)pack_bf16x2(v[0], v[1]), (int)pack_bf16x2(v[2], v[3])};
  return r;
}
__device__ __forceinline__ f32x4 unpack_bf16x4(i32x2 r) {
  f32x4 v = {__uint_as_float((unsigned)r[0] << 16), __uint_as_float((unsigned)r[0] & 0xffff0000u),
             __uint_as_float((unsigned)r[1] << 16), __uint_as_float((unsigned)r[1] & 0xffff0000u)};
  return v;
}
// Products, sums and differences that round on their own, as separate elementwise launches of the
// reference round them: without the pragma the compiler is free to fuse `a * b + c` into one fma
// (the __f*_rn intrinsics are plain operators to it).
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float add_rn(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}
__device__ __forceinline__ float sub_rn(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}
// fp16 counterparts (round-to-nearest-even conversions), for the kernels that also come in an fp16 flavour
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ unsigned pack_f16x2(float a, float b) {
  f32x2 v = {a, b};
  union { f16x2 h; unsigned u; } r;
  r.h = __builtin_convertvector(v, f16x2);
  return r.u;
}
__device__ __forceinline__ i32x2 pack_f16x4(f32x4 v) {
  i32x2 r = {(int)pack_f16x2(v[0], v[1]), (int)pack_f16x2(v[2], v[3])};
  return r;
}
__device__ __forceinline__ f32x4 unpack_f16x4(i32x2 r) {
  union { i32x2 i; f16x2 h[2]; } u;
  u.i = r;
  f32x4 v = {(float)u.h[0][0], (float)u.h[0][1], (float)u.h[1][0], (float)u.h[1][1]};
  return v;
}
__device__ __forceinline__ f16x8 as_f16x8(i32x4 v) {
  union { i32x4 i; f16x8 h; } u;
  u.i = v;
  return u.h;
}
// four fp32 <-> four 16-bit floats of the kernel's flavour
template <bool F16>
__device__ __forceinline__ i32x2 pack_16x4(f32x4 v) {
  return F16 ? pack_f16x4(v) : pack_bf16x4(v);
}
template <bool F16>
__device__ __forceinline__ f32x4 unpack_16x4(i32x2 r) {
  return F16 ? unpack_f16x4(r) : unpack_bf16x4(r);
}

__device__ __forceinline__ float round_bf16(float f) { return __uint_as_float(pack_bf16x2(f, 0.f) << 16); }

// 4 e4m3fn bytes (one dword) -> 4 bf16 (exact: every e4m3 value is a bf16 value).
__device__ __forceinline__ void fp8x4_to_bf16x4(int v, bf16x2& lo, bf16x2& hi) {
  lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v, 1.0f, false);
  hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v, 1.0f, true);
}

// 8 e4m3fn bytes (two dwords) -> one MFMA operand of 8 bf16.
__device__ __forceinline__ bf16x8 fp8x8_to_bf16x8(int a, int b) {
  bf16x2 p0, p1, p2, p3;
  fp8x4_to_bf16x4(a, p0, p1);
  fp8x4_to_bf16x4(b, p2, p3);
  bf16x8 r;
  r[0] = p0[0]; r[1] = p0[1]; r[2] = p1[0]; r[3] = p1[1];
  r[4] = p2[0]; r[5] = p2[1]; r[6] = p3[0]; r[7] = p3[1];
  return r;
}

__device__ __forceinline__ bf16x8 as_bf16x8(i32x4 v) {
  union { i32x4 i; bf16x8 b; } u;
  u.i = v;
  return u.b;
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }
// gelu(x, approximate="tanh") = 0.5 x (1 + tanh(z)) = x / (1 + exp(-2z)), z = sqrt(2/pi) (x + 0.044715 x^3):
// the same function through one exponential instead of a tanh expansion.
__device__ __forceinline__ float gelu_tanh_f(float x) {
  const float c0 = 0.7978845608028654f;  // sqrt(2/pi)
  const float inner = c0 * (x + 0.044715f * x * x * x);
  return x / (1.0f + __expf(-2.0f * inner));
}

// Device-coherent (agent-scope, cache write-through / cache-bypassing) accesses used for data that
// one block hands to another inside a kernel: with them the hand-off needs no L2 flush.
__device__ __forceinline__ void st_agent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_agent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// two floats as one 8-byte device-coherent access
__device__ __forceinline__ void st_agent64(unsigned long long* p, float lo, float hi) {
  const unsigned long long v = (unsigned long long)__float_as_uint(lo) | ((unsigned long long)__float_as_uint(hi) << 32);
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long ld_agent64(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Ordering of such a hand-off.  RULE: every byte one block hands to another is written with st_agent* and read
// with ld_agent* -- a plain store would sit in this XCD's L2 and a plain load could hit a stale line there; the
// scheme below orders the accesses, it does not make ordinary ones coherent.
// The writer's partials are write-through stores, visible to every block once
// the wave's memory counters have drained; handoff_publish() drains them and pins the compiler on both sides
// (no memory access may be moved across it), and the arrival count that follows it publishes the data.  On the
// reader's side handoff_acquire() pins the compiler between seeing the count and reading the partials (the
// reads themselves bypass the non-coherent caches).
__device__ __forceinline__ void handoff_publish() {
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0);
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
}
__device__ __forceinline__ void handoff_acquire() { __atomic_signal_fence(__ATOMIC_SEQ_CST); }

// C layout of v_mfma_f32_32x32x16: lane l, register i holds
//   column = l % 32, row = 8*(i/4) + 4*(l/32) + (i%4).
__device__ __forceinline__ int mfma32_row(int lane, int i) { return 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3); }
