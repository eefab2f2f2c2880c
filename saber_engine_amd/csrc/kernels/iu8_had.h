// Shared pieces of the Hadamard-basis int8 producers (code objects `mxfp4_hadi8` and
// `attn_glue_hadi8`): the 32-point transform of crates/saber-kernels/hip/macaq_had.h:47-83 on the
// reference's lane map, the row order of a launch, and the per-token int8 tail.
//
// THE LANE MAP is the reference's: thread tid owns the 8-element groups g = tid + i*T (T a multiple of
// 4), so a 32-block = 4 adjacent lanes x 8 registers; stages on element bits 0, 1, 2 in registers, then
// bit 3 (lane xor 1) and bit 4 (lane xor 2) by DPP quad_perm, which moves registers exactly and works
// the same in a 64-wide wave. Contraction is off in every object that includes this.
#pragma once
#include "iu8_common.h"

#define HAD_MAXG 5  // 8-element groups a thread: K <= 40 * T

static __device__ __forceinline__ float had_dpp_xor1(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));
}
static __device__ __forceinline__ float had_dpp_xor2(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));
}

// v[8]: this lane's 8 values of its group; t8: the group's 8 entries of t. In place.
static __device__ __forceinline__ void had32(float (&v)[8], const float *__restrict__ t8, int lane) {
#pragma clang fp contract(off)
  const float4 ta = ((const float4 *)t8)[0], tb = ((const float4 *)t8)[1];
  v[0] = v[0] * ta.x, v[1] = v[1] * ta.y, v[2] = v[2] * ta.z, v[3] = v[3] * ta.w;
  v[4] = v[4] * tb.x, v[5] = v[5] * tb.y, v[6] = v[6] * tb.z, v[7] = v[7] * tb.w;
#pragma unroll
  for (int s = 1; s < 8; s <<= 1) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j & s) continue;
      const float lo = v[j], hi = v[j | s];
      v[j] = lo + hi;
      v[j | s] = lo - hi;
    }
  }
  const bool b0 = (lane & 1) != 0, b1 = (lane & 2) != 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float p = had_dpp_xor1(v[j]);
    v[j] = b0 ? (p - v[j]) : (v[j] + p);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float p = had_dpp_xor2(v[j]);
    v[j] = b1 ? (p - v[j]) : (v[j] + p);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = v[j] * __uint_as_float(0x3E3504F3u);
}

// The row of workgroup b: the 8 A tiles of a full group of 128 rows go one to an XCD (consecutive
// workgroups are dealt round-robin over the 8 XCDs), so an XCD's L2 sees whole lines of the tiles.
static __device__ __forceinline__ int had_row() {
  const int b = blockIdx.x, full = (int)gridDim.x & ~127;
  if (b >= full) return b;
  return (b & ~127) + (b & 7) * 16 + ((b & 127) >> 3);
}

// the int8 tail: row maximum (order-free), scale, codes, 8-byte stores in A fragment order
template <int T>
static __device__ __forceinline__ void had_tail(float (&sv)[HAD_MAXG][8], int NV, iu8_u8 *__restrict__ q,
                                                float *__restrict__ scale, int row, int K) {
  __shared__ float s_max[T / 64];
  const int tid = threadIdx.x;
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    if (tid + i * T >= NV) continue;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(sv[i][j]));
  }
  amax = iu8_wave_max_nonneg(amax);
  if ((tid & 63) == 0) s_max[tid >> 6] = amax;
  __syncthreads();
  amax = s_max[0];
#pragma unroll
  for (int w = 1; w < T / 64; ++w) amax = fmaxf(amax, s_max[w]);
  const float sc = fmaxf(__fdiv_rn(amax, 127.f), 1e-30f);
  const float rcp = __fdiv_rn(1.f, sc);
  if (tid == 0) scale[row] = sc;
  iu8_u8 *qrow = q + (size_t)(row >> 4) * (K >> 6) * 1024 + (row & 15) * 16;
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    const int g = tid + i * T;
    if (g >= NV) continue;
    const unsigned lo = iu8_code4_rcp(sv[i][0], sv[i][1], sv[i][2], sv[i][3], sc, rcp);
    const unsigned hi = iu8_code4_rcp(sv[i][4], sv[i][5], sv[i][6], sv[i][7], sc, rcp);
    // group g = elements 8g..8g+7: fragment kt = g/8, 16-byte piece (g/2)%4 of the row, half g%2
    *(iu8_v2u *)(qrow + (size_t)(g >> 3) * 1024 + ((g >> 1) & 3) * 256 + (g & 1) * 8) = iu8_v2u{lo, hi};
  }
}

static __device__ __forceinline__ void had_load8(const unsigned short *p, float (&v)[8]) {
  const iu8_v4u u = *(const iu8_v4u *)p;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    v[2 * w] = __uint_as_float(u[w] << 16);
    v[2 * w + 1] = __uint_as_float(u[w] & 0xFFFF0000u);
  }
}

// The two gates of the producers above that carry the device's expf. Both are functions of a bf16
// input, so a checker can table them over all 65,536 inputs (the tap kernels of `iu8_taps`).
// silu in f32 (the GDN norm's gate, crates/saber-kernels/hip/mxfp4_hadi8.hip:148-186):
static __device__ __forceinline__ float had_silu_f32(float z) {
#pragma clang fp contract(off)
  return z / (1.f + expf(-z));
}
// sigmoid rounded to bf16 (the attention output gate, crates/saber-kernels/hip/attn_glue_hadi8.hip:23-79):
static __device__ __forceinline__ float glue_sigmoid_bf16(float g) {
#pragma clang fp contract(off)
  return iu8_bf16_f32((unsigned short)iu8_bf16_bits(1.f / (1.f + expf(-g))));
}
