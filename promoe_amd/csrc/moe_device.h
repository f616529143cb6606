// Device-side helpers shared by the kernel sources (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "moe_kernels.h"

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned int u32;

// ---------------------------------------------------------------------------
// small device helpers
// ---------------------------------------------------------------------------
static __device__ __forceinline__ float bf16lo(u32 v) { return __uint_as_float(v << 16); }
static __device__ __forceinline__ float bf16hi(u32 v) { return __uint_as_float(v & 0xffff0000u); }
static __device__ __forceinline__ uint16_t f32_to_bf16(float f) {  // round to nearest even
  u32 u = __float_as_uint(f);
  u32 r = ((u >> 16) & 1u) + 0x7fffu;
  return (uint16_t)((u + r) >> 16);
}
static __device__ __forceinline__ float dot2bf(u32 a, u32 b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                         __builtin_bit_cast(bf16x2_t, b), c, false);
}
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;
// buffer resource over [p, p+bytes): loads past the end return 0 instead of faulting
static __device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, (int)bytes, 0x00020000);
}
// A unit list for the host: stores with both scope bits set go past the caches straight to the pinned
// host buffer; once they have completed (host_stores_done) the sequence word the host polls may follow.
// No cache write-back or invalidate is involved, unlike a system-scope fence.
static __device__ __forceinline__ void host_store_unit(moe_unit *dst, int i, int expert, int m, int row0) {
  const u32x4_t v = {(u32)expert, (u32)m, (u32)row0, 0u};
  __builtin_amdgcn_raw_buffer_store_b128(v, make_rsrc(dst, 0x7fffffffu), i * 16, 0, 17 /* sc0 | sc1 */);
}
static __device__ __forceinline__ void host_store_i32(int *dst, int v) {
  __builtin_amdgcn_raw_buffer_store_b32((u32)v, make_rsrc(dst, 0x7fffffffu), 0, 0, 17);
}
static __device__ __forceinline__ void host_stores_done() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);  // every outstanding memory operation of this wave has completed
}
static __device__ __forceinline__ float half_bits_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
// 8 int4 weights (interleaved nibble order) x 8 bf16 activations; the weights
// enter as the exact bf16 values 128+q (0x4300 | q), the caller removes 128*sum(x).
// Mask and exponent pattern of dot8_q4 held in vector registers, made once per kernel: (w & M) | C is then ONE
// v_and_or_b32 (a VOP3 instruction takes no literal and one scalar operand on this target, so with the constants
// as literals the compiler emits an and and an or: 12 instead of 8 operations per 8 weights).
struct Q4Consts { u32 M, C; };
static __device__ __forceinline__ Q4Consts q4_consts() {
  Q4Consts q{0x000f000fu, 0x43004300u};
  asm volatile("" : "+v"(q.M), "+v"(q.C));
  return q;
}
static __device__ __forceinline__ float dot8_q4(u32 w, const uint4 &x, float acc, const Q4Consts &q) {
  const u32 M = q.M, C = q.C;
  acc = dot2bf((w & M) | C, x.x, acc);
  acc = dot2bf(((w >> 4) & M) | C, x.y, acc);
  acc = dot2bf(((w >> 8) & M) | C, x.z, acc);
  acc = dot2bf(((w >> 12) & M) | C, x.w, acc);
  return acc;
}

// maximum over the 64 lanes of a wave, built from DPP row shifts and broadcasts (no LDS traffic)
static __device__ __forceinline__ float wave_max_f32(float x) {
  // inclusive max-scan inside each row of 16 lanes, then rows 0->1, 2->3, then 1->3: lane 63 holds the result
#define WMAX_STEP(ctrl, rmask)                                                                          \
  {                                                                                                     \
    const int xi = __builtin_bit_cast(int, x);                                                          \
    x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(xi, xi, ctrl, rmask, 0xf, false))); \
  }
  WMAX_STEP(0x111, 0xf)  // row_shr:1
  WMAX_STEP(0x112, 0xf)  // row_shr:2
  WMAX_STEP(0x114, 0xf)  // row_shr:4
  WMAX_STEP(0x118, 0xf)  // row_shr:8
  WMAX_STEP(0x142, 0xa)  // row_bcast:15 into rows 1 and 3
  WMAX_STEP(0x143, 0xc)  // row_bcast:31 into rows 2 and 3
#undef WMAX_STEP
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

// global-address-space loads (pointers that come out of the slot table are generic
// to the compiler and would otherwise become flat_load)
typedef __attribute__((address_space(1))) const u32x4_t g_uint4;
typedef __attribute__((address_space(1))) const unsigned int g_u32;
static __device__ __forceinline__ uint4 ldg_u4(const void *p) {
  const u32x4_t v = *(g_uint4 *)(unsigned long long)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}
static __device__ __forceinline__ u32 ldg_u32(const void *p) { return *(g_u32 *)(unsigned long long)p; }
static __device__ __forceinline__ float sum8_bf16(const uint4 &v) {
  return bf16lo(v.x) + bf16hi(v.x) + bf16lo(v.y) + bf16hi(v.y) + bf16lo(v.z) + bf16hi(v.z) + bf16lo(v.w) +
         bf16hi(v.w);
}

static __device__ __forceinline__ uint4 bload16(rsrc_t r, int voff, int soff) {
  const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
// the same marked non-temporal: for weight tiles that a launch reads exactly once (the decode kernels below 16
// tokens).  A 7.8 GB stack streams through the caches anyway; told so, they keep what is read again (activation
// rows, scale sections, the next kernel's inputs): one-token w13 launch 8.16 -> 7.6 us, Mixtral-shaped one-token layer
// 49.3 -> 45.9 us, q4_K three-token layer 152.5 -> 143.7 us.
static __device__ __forceinline__ uint4 bload16_nt(rsrc_t r, int voff, int soff) {
  const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 2);
  return make_uint4(v.x, v.y, v.z, v.w);
}
static __device__ __forceinline__ u32 bload4(rsrc_t r, int voff, int soff) {
  return __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0);
}
static __device__ __forceinline__ u32 bload2(rsrc_t r, int voff, int soff) {
  return (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0);
}
static __device__ __forceinline__ u32 bload1(rsrc_t r, int voff, int soff) {
  return (u32)(unsigned char)__builtin_amdgcn_raw_buffer_load_b8(r, voff, soff, 0);
}

// ---------------------------------------------------------------------------
// fp16 operands for the matrix cores from nibble formats (int4-g128 and q4_K tile kernels, q4_K decode)
// ---------------------------------------------------------------------------
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
static __device__ __forceinline__ u32 bf16x2_to_f16x2(u32 d) {
  // both halves are bf16; fp16 has more mantissa bits, so round-to-zero conversion is exact
  auto h = __builtin_amdgcn_cvt_pkrtz(__uint_as_float(d << 16), __uint_as_float(d & 0xffff0000u));
  return __builtin_bit_cast(u32, h);
}
// Dequantisation of 8 nibbles of a dword into 8 fp16 weights with ONE packed fma per pair: a nibble is masked into
// mantissa bits 6..9 of an fp16 with the exponent of 1.0, which makes the exact value h = 1 + q/16; with S = 16 s and
// C = -(16 + zero) s (int4) or C = -(16 s + m) (q4_K), both prepared once per group and row, h S + C = (q - zero) s
// or q s - m.  The product is exact inside the fma; C carries the one extra rounding (2^-11 of at most 31 s, i.e.
// 0.015 of a quantisation step, a bias common to the 128 weights of a group row).  The form before this one
// ((h - (1024 + zero)) s with h = 1024 + q) was exact up to the final rounding and cost a packed subtract and
// a packed multiply per pair (three operations for q4_K), in kernels that are bound by these operations.
// Mask and exponent pattern are held in vector registers, made once per kernel: (x & M) | C is then ONE
// v_and_or_b32 (a VOP3 instruction takes no literal and one scalar operand on this target).
struct DeqF16Consts { u32 M, C; };
static __device__ __forceinline__ DeqF16Consts deq_f16_consts() {
  DeqF16Consts q{0x03c003c0u, 0x3c003c00u};
  asm volatile("" : "+v"(q.M), "+v"(q.C));
  return q;
}
// s2 / c2: fp16 bit patterns of S and C replicated in both halves
static __device__ __forceinline__ f16x8_t deq8_f16(u32 d, u32 s2, u32 c2, const DeqF16Consts &q) {
  const u32 M = q.M, C = q.C;
  u32x4_t v;
  v.x = ((d << 6) & M) | C; v.y = ((d << 2) & M) | C; v.z = ((d >> 2) & M) | C; v.w = ((d >> 6) & M) | C;
  const f16x8_t h = __builtin_bit_cast(f16x8_t, v);   // 1 + q/16, exact
  const f16x8_t s8 = __builtin_bit_cast(f16x8_t, u32x4_t{s2, s2, s2, s2});
  const f16x8_t c8 = __builtin_bit_cast(f16x8_t, u32x4_t{c2, c2, c2, c2});
  return __builtin_elementwise_fma(h, s8, c8);
}

static __device__ __forceinline__ u32 h2f_bits(u32 hbits) {  // fp16 bits -> fp32 bits
  const _Float16 h = __builtin_bit_cast(_Float16, (uint16_t)hbits);
  return __builtin_bit_cast(u32, (float)h);
}
static __device__ __forceinline__ u32 f2h_bits(float f) {  // fp32 -> fp16 bits (round to nearest)
  return (u32)__builtin_bit_cast(uint16_t, (_Float16)f);
}

