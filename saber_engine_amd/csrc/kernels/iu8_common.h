// Shared device helpers of the gfx950 W4A8-iu8 kernels: operand orders, the int8 MFMA,
// the nibble unpack, bf16 rounding and the epilogue contract.
//
// OPERAND ORDERS (gfx950 device-final; a wave64 lane reads 16 bytes = one MFMA operand).
//   A   int8 activations, rows padded to 16. Fragment (mt, kt) = 1024 B at
//       (mt * K/64 + kt) * 1024; lane l's 16 bytes at l*16 = row mt*16 + l%16,
//       k = kt*64 + (l/16)*16 + 0..15. Rows past M are never stored from.
//   W4  int4 [-8,7] two's-complement nibbles. Fragment (nt, kt) = 1024 B at
//       (nt * K/128 + kt) * 1024; lane l's 4 dwords d0..d3 at l*16 belong to row
//       nt*16 + l%16; dword j, byte b: low nibble = k0 + b, high nibble = k0 + 4 + b with
//       k0 = kt*128 + (j/2)*64 + (l/16)*16 + (j%2)*8. Unpacked to the exact int8 16*w
//       (lo = (d << 4) & 0xF0F0F0F0, hi = d & 0xF0F0F0F0), so {lo(d0),hi(d0),lo(d1),hi(d1)}
//       is the operand of k-step 2*kt and {lo(d2),hi(d2),lo(d3),hi(d3)} of 2*kt+1, both in
//       natural k order, and the int32 accumulator holds 16 * sum(a*w).
//   W8  int8 [-127,127]: the A order by rows of W (fragment (nt, kt) of 16 rows x 64 k).
// The reference's gfx12 orders (crates/saber-kernels/hip/macaq_iu8.hip:8-18) are wave32 WMMA
// fragment orders; these are their wave64 MFMA counterparts and keep the same sizes.
//
// THE CONTRACT (crates/saber-kernels/hip/macaq_iu8.hip:20-24): acc = exact int32 sum over all
// of K; y = bf16_rne((f32(acc) * as[m]) * (ws[n] * U)), U = 1/16 for W4 and 1 for W8, each `*`
// one IEEE f32 multiply. Every translation unit including this header is compiled with
// -ffp-contract=off.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int iu8_v4i __attribute__((ext_vector_type(4)));
typedef unsigned iu8_v4u __attribute__((ext_vector_type(4)));
typedef unsigned iu8_v2u __attribute__((ext_vector_type(2)));
typedef float iu8_v4f __attribute__((ext_vector_type(4)));
typedef unsigned char iu8_u8;

// D[n][m] += sum_k W[n][k] * A[m][k] over 64 k: src0 = weight operand (lane: row n = l%16),
// src1 = activation operand (lane: row m = l%16); D lane l holds n = 4*(l/16) + 0..3, m = l%16.
static __device__ __forceinline__ iu8_v4i iu8_mfma(iu8_v4i w, iu8_v4i a, iu8_v4i c) {
  return __builtin_amdgcn_mfma_i32_16x16x64_i8(w, a, c, 0, 0, 0);
}

// 16 B of a W4 fragment -> the two k-step operands (int8 = 16 * code).
static __device__ __forceinline__ void iu8_unpack_w4(iu8_v4u d, iu8_v4i &s0, iu8_v4i &s1) {
  s0 = iu8_v4i{(int)((d.x << 4) & 0xF0F0F0F0u), (int)(d.x & 0xF0F0F0F0u), (int)((d.y << 4) & 0xF0F0F0F0u),
               (int)(d.y & 0xF0F0F0F0u)};
  s1 = iu8_v4i{(int)((d.z << 4) & 0xF0F0F0F0u), (int)(d.z & 0xF0F0F0F0u), (int)((d.w << 4) & 0xF0F0F0F0u),
               (int)(d.w & 0xF0F0F0F0u)};
}

// f32 -> bf16 bits, round to nearest even (finite inputs; NaN stays a quiet NaN).
static __device__ __forceinline__ unsigned iu8_bf16_bits(float x) {
  const unsigned u = __float_as_uint(x);
  if (x != x) return (u >> 16) | 0x40u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
static __device__ __forceinline__ float iu8_bf16_f32(unsigned short b) { return __uint_as_float((unsigned)b << 16); }
typedef float iu8_v2f __attribute__((ext_vector_type(2)));
typedef __bf16 iu8_v2bf __attribute__((ext_vector_type(2)));

// two f32 -> packed bf16, round to nearest even (v_cvt_pk_bf16_f32); lo in bits 0..15
static __device__ __forceinline__ unsigned iu8_bf16_pack(float lo, float hi) {
  const iu8_v2bf r = __builtin_convertvector(iu8_v2f{lo, hi}, iu8_v2bf);
  return *(const unsigned *)&r;
}
// bf16(silu(x)) as the producer kernels compute it (macaq_i8q: i8q_silu_bf16; the law
// crates/saber-kernels/hip/mxfp4_hadi8.hip:118-146): x / (1 + expf(-x)), IEEE divide, one bf16 rounding.
static __device__ __forceinline__ float iu8_silu_bf16(float x) {
#pragma clang fp contract(off)
  return iu8_bf16_f32((unsigned short)iu8_bf16_bits(x / (1.f + expf(-x))));
}

template <bool W8>
static __device__ __forceinline__ float iu8_wsu(const float *__restrict__ ws, int n) {
#pragma clang fp contract(off)
  return W8 ? ws[n] : ws[n] * 0.0625f;
}
static __device__ __forceinline__ float iu8_epi(int acc, float a_scale, float w_scale_u) {
#pragma clang fp contract(off)
  const float t = (float)acc * a_scale;
  return t * w_scale_u;
}

// The per-token int8 code (crates/saber-kernels/hip/macaq_i8.h:10-13): IEEE divide, clamp,
// round half to even.
static __device__ __forceinline__ unsigned iu8_code(float x, float sc) {
  const float y = fminf(fmaxf(__fdiv_rn(x, sc), -127.f), 127.f);
  return ((unsigned)(int)__builtin_rintf(y)) & 0xffu;
}

// The same codes without a divide per element: rcp = __fdiv_rn(1, sc) once a row, t = x * rcp is
// within 1.6e-5 of x / sc for |x / sc| <= 127 (two roundings of 2^-24 relative), the IEEE quotient
// within 7.6e-6. If t sits at least 1e-4 inside its rounding interval, the IEEE quotient rounds to
// the same integer; otherwise (a tie or next to one, rare) the divide decides. NaN and infinite
// rows come out as through the divide: NaN clamps to -127 on both paths.
//
// Four codes at once, packed little-endian into a dword, by the same law. The fast path rounds by
// adding 1.5 * 2^23: for |t| <= 127 the sum's unit in the last place is 1, so the IEEE addition itself
// rounds t to the nearest integer, ties to even, and leaves that integer's two's-complement low byte
// in the low byte of the sum's bit pattern; subtracting the constant again (exact) gives the rounded
// value for the tie test. v_med3_f32 returns the minimum of its operands when one is NaN, which is
// the -127 of fminf(fmaxf(NaN, -127), 127). Any element next to a tie sends its four to the divide.
static __device__ __forceinline__ unsigned iu8_code4_rcp(float x0, float x1, float x2, float x3, float sc, float rcp) {
#pragma clang fp contract(off)
  const float MAGIC = 12582912.f;
  const float t0 = __builtin_amdgcn_fmed3f(x0 * rcp, -127.f, 127.f), t1 = __builtin_amdgcn_fmed3f(x1 * rcp, -127.f, 127.f);
  const float t2 = __builtin_amdgcn_fmed3f(x2 * rcp, -127.f, 127.f), t3 = __builtin_amdgcn_fmed3f(x3 * rcp, -127.f, 127.f);
  const float u0 = t0 + MAGIC, u1 = t1 + MAGIC, u2 = t2 + MAGIC, u3 = t3 + MAGIC;
  // one test for the four: the largest distance of a t from its rounded value
  const float off = fmaxf(fmaxf(fabsf(t0 - (u0 - MAGIC)), fabsf(t1 - (u1 - MAGIC))),
                          fmaxf(fabsf(t2 - (u2 - MAGIC)), fabsf(t3 - (u3 - MAGIC))));
  const bool near_tie = !(off <= 0.4999f);  // NaN goes to the divide as well
  if (__builtin_expect(near_tie, 0)) {
    // stays a branch: without this statement the compiler now and then runs the four divides for every
    // quad and selects afterwards (seen as a third more VALU work in a row producer)
    asm volatile("");
    return iu8_code(x0, sc) | (iu8_code(x1, sc) << 8) | (iu8_code(x2, sc) << 16) | (iu8_code(x3, sc) << 24);
  }
  // bytes 0,1 from (u0, u1), bytes 2,3 from (u2, u3); selector 0x0c yields a zero byte
  return __builtin_amdgcn_perm(__float_as_uint(u1), __float_as_uint(u0), 0x0c0c0400u) |
         __builtin_amdgcn_perm(__float_as_uint(u3), __float_as_uint(u2), 0x04000c0cu);
}

// The per-token law from a row kept as packed bf16 pairs (pk[g][w]: elements 2w and 2w + 1 of 16-element group g, as
// loaded; a thread's groups past the row's end are zeros). The largest magnitude of finite bf16 values is
// the largest of their bit patterns without the sign, two a packed 16-bit maximum; a thread that holds a
// NaN (a pattern above infinity's) takes the f32 maximum instead, which passes NaNs over.
template <int NG>
static __device__ __forceinline__ float iu8_pk_amax(const unsigned (&pk)[NG][8]) {
  typedef unsigned short us2 __attribute__((ext_vector_type(2)));
  us2 m2 = {0, 0};
#pragma unroll
  for (int i = 0; i < NG; ++i)
#pragma unroll
    for (int w = 0; w < 8; ++w) m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(us2, pk[i][w] & 0x7FFF7FFFu));
  const unsigned top = m2.x > m2.y ? m2.x : m2.y;
  float amax = __uint_as_float(top << 16);
  if (top > 0x7F80u) {
    amax = 0.f;
#pragma unroll
    for (int i = 0; i < NG; ++i)
#pragma unroll
      for (int w = 0; w < 8; ++w) {
        unsigned r = pk[i][w];
        asm volatile("" : "+v"(r));  // a value of its own: nothing of the fast path is kept alive for this one
        amax = fmaxf(amax, fabsf(__uint_as_float(r << 16)));
        amax = fmaxf(amax, fabsf(__uint_as_float(r & 0xFFFF0000u)));
      }
  }
  return amax;
}
static __device__ __forceinline__ iu8_v4u iu8_pk_codes(const unsigned (&g)[8], float sc, float rcp) {
  unsigned d[4];
#pragma unroll
  for (int w = 0; w < 4; ++w)
    d[w] = iu8_code4_rcp(__uint_as_float(g[2 * w] << 16), __uint_as_float(g[2 * w] & 0xFFFF0000u),
                         __uint_as_float(g[2 * w + 1] << 16), __uint_as_float(g[2 * w + 1] & 0xFFFF0000u), sc, rcp);
  return iu8_v4u{d[0], d[1], d[2], d[3]};
}
// Maximum over the 64 lanes of a wave of values that are non-negative and never NaN (row maxima of
// |x|): DPP inside each 16-lane row (partners xor 1, xor 2, the half-row and the row mirror), then the
// four rows' values through scalar registers, where the unsigned order of the bit patterns is the
// values' order. The result is wave-uniform. A butterfly of six exchanges through the LDS crossbar
// costs most of a microsecond in a kernel that is a latency chain.
static __device__ __forceinline__ float iu8_wave_max_nonneg(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, false)));
  const int u = __float_as_int(v);
  const unsigned m01 = max((unsigned)__builtin_amdgcn_readlane(u, 0), (unsigned)__builtin_amdgcn_readlane(u, 16));
  const unsigned m23 = max((unsigned)__builtin_amdgcn_readlane(u, 32), (unsigned)__builtin_amdgcn_readlane(u, 48));
  return __uint_as_float(max(m01, m23));
}

// Cross-workgroup hand-over without a cache flush. The card has one L2 per XCD, so a device-scope
// release fence writes an L2's dirty lines back and an acquire fence invalidates it; with hundreds of
// workgroups doing that the fences alone cost 15-60 us a launch (measured with and without dirty
// data). Accesses with both scope bits set are coherent by themselves: such a store goes through to
// memory and its completion (vmcnt) means it is visible there, such a load comes from there. So a
// producer stores its partials this way, waits for their completion, meets its workgroup and bumps a
// device-scope atomic counter; the consumer that finds the counter full loads the partials this way.
// The order is the hardware's in-order completion count, not a language-level fence: these helpers
// are asm for that reason.
static __device__ __forceinline__ void iu8_store_through(int *p, iu8_v4i v) {
  // the wait states behind it: a store of more than 8 bytes reads its data registers for two more
  // cycles, and the compiler's hazard recognizer does not look inside an asm statement
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 2" ::"v"(p), "v"(v) : "memory");
}
static __device__ __forceinline__ iu8_v4i iu8_load_through(const int *p) {
  iu8_v4i v;
  asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  return v;
}
static __device__ __forceinline__ void iu8_stores_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// one lane, after the workgroup met behind its completed stores: count the arrival
static __device__ __forceinline__ int iu8_arrive(int *counter) {
  return __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

static __device__ __forceinline__ iu8_v4u iu8_ldg_nt(const iu8_u8 *p) {
  return __builtin_nontemporal_load((const iu8_v4u *)p);
}
