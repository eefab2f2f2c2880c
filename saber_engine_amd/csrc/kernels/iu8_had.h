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

// One butterfly stage across lanes: the pair is (this lane, the lane CTRL's quad permute brings in);
// the lane whose bit is clear holds the pair's low element and keeps the sum, the other the difference
// low - high. A DPP move copies registers exactly, in a 64-wide wave as in a 32-wide one.
template <int CTRL>
static __device__ __forceinline__ void had_lane_stage(float (&v)[8], bool holds_high) {
#pragma clang fp contract(off)
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float other = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v[j]), CTRL, 0xF, 0xF, false));
    v[j] = holds_high ? other - v[j] : v[j] + other;
  }
}

// The 32-point transform (crates/saber-kernels/hip/macaq_had.h:47-83) of the block whose elements
// 8*(lane & 3) .. + 7 this lane holds in v: multiply by the block's t, the unnormalised Sylvester
// butterfly over element bits 0..4 in that order -- bits 0..2 pair registers, bits 3 and 4 pair lanes
// (xor 1, xor 2) -- each stage (low, high) -> (low + high, low - high), then one multiply by
// (float)(1 / sqrt(32)). t8: the 8 entries of t for this lane's elements. In place.
static __device__ __forceinline__ void had32(float (&v)[8], iu8_v4f t_lo, iu8_v4f t_hi, int lane) {
#pragma clang fp contract(off)
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = v[j] * t_lo[j], v[j + 4] = v[j + 4] * t_hi[j];
#pragma unroll
  for (int bit = 0; bit < 3; ++bit) {
    const int span = 1 << bit;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j & span) continue;  // j is the pair's low element
      const float low = v[j], high = v[j + span];
      v[j] = low + high;
      v[j + span] = low - high;
    }
  }
  had_lane_stage<0xB1>(v, (lane & 1) != 0);  // quad_perm [1,0,3,2]: element bit 3
  had_lane_stage<0x4E>(v, (lane & 2) != 0);  // quad_perm [2,3,0,1]: element bit 4
  const float inv_sqrt32 = __uint_as_float(0x3E3504F3u);
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = v[j] * inv_sqrt32;
}

static __device__ __forceinline__ void had32(float (&v)[8], const float *__restrict__ t8, int lane) {
  had32(v, *(const iu8_v4f *)t8, *(const iu8_v4f *)(t8 + 4), lane);
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

// A table of a gate over all 65,536 bf16 bit patterns (bf16 or f32 entries, as a table kernel of these
// objects wrote it with the gate's own expression) serves a producer through its middle: the patterns of
// magnitudes 2^-17 up to 2^15, both signs, 2 x HAD_LUT_N entries, which a workgroup copies into LDS (16 KiB of
// bf16 entries, 32 KiB of f32). A lookup returns the computed gate's bits by construction; a pattern
// outside (zeros, denormals, huge values, infinities, NaN: one in some hundred thousand of unit-scale
// values) is computed.
#define HAD_LUT_LO (110 << 7)  // first pattern without sign in the table: 2^-17
#define HAD_LUT_N 4096         // patterns a sign: 32 exponents
// requests this thread's 16-byte pieces of the middle (T threads; E = unsigned short or float)
template <class E, int T>
struct had_lut_copy {
  static constexpr int PER = 16 / sizeof(E), NP = 2 * HAD_LUT_N / PER / T;
  iu8_v4u tb[NP];
  __device__ __forceinline__ void request(const E *__restrict__ lut, int tid) {
#pragma unroll
    for (int c = 0; c < NP; ++c) {
      const int i = (c * T + tid) * PER;  // entry: sign i / HAD_LUT_N, pattern HAD_LUT_LO + i % HAD_LUT_N
      tb[c] = *(const iu8_v4u *)(lut + (i / HAD_LUT_N) * 32768 + HAD_LUT_LO + (i & (HAD_LUT_N - 1)));
    }
  }
  __device__ __forceinline__ void commit(E *s_lut, int tid) const {  // the caller's barrier follows
#pragma unroll
    for (int c = 0; c < NP; ++c) ((iu8_v4u *)s_lut)[c * T + tid] = tb[c];
  }
};
// the LDS index of pattern b (low 16 bits), or false when b is outside the middle
static __device__ __forceinline__ bool had_lut_index(unsigned b, unsigned &at) {
  const unsigned idx = (b & 0x7FFFu) - HAD_LUT_LO;
  at = ((b >> 15) << 12) | idx;
  return idx < (unsigned)HAD_LUT_N;
}
