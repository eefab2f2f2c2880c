// The Hadamard-basis int8 producers for gfx950: the code object `mxfp4_hadi8`, standing in for the
// reference's object of the same name (crates/saber-kernels/hip/mxfp4_hadi8.hip, symbols
// crates/saber-kernels/src/macaq_iu8.rs:864-875) with the same kernel symbols and kernarg layouts
// (`had_t` last). A producer's final bf16-rounded values v become u = v * t, x = H32 u per 32-block
// along K, x = x * (1/sqrt(32)) (crates/saber-kernels/hip/macaq_had.h:1-19), and the per-token int8
// law runs on x (iu8_common.h); codes are stored in the gfx950 A fragment order.
//
//   add_rms_quant_hadi8_t{256,512}_tiled1   v = bf16((f32(y) + f32(res)) * inv * (f32(w) + 1)), res_out = bf16(y + res)
//   silu_mul_quant_hadi8_t{256,512}_tiled1  v = bf16(bf16(silu(gate)) * up)
//   quant_hadi8_t{256,512}_tiled1           v = x (no counterpart among the reference's symbols: the
//                                           transform in front of the plain producer)
// Not built: gdn_norm_quant_hadi8 and attn_gate_quant_hadi8 (their parents belong to layer kinds the
// benchmark configurations do not have).
//
// THE LANE MAP is the reference's: thread tid owns the 8-element groups g = tid + i*T (T a multiple of
// 4), so a 32-block = 4 adjacent lanes x 8 registers; stages on element bits 0, 1, 2 in registers, then
// bit 3 (lane xor 1) and bit 4 (lane xor 2) by DPP quad_perm, which moves registers exactly and works
// the same in a 64-wide wave. Contraction is off in this whole object.
//
// The sum of squares of add_rms keeps the reference's order (per-thread fma over its groups, then
// shfl_down 16..1 inside each 32 lanes, then over the T/32 partials). Its `rsqrtf` is the one thing
// not taken over: the device's approximate reciprocal square root cannot be restated on a host, so
// inv = 1 / sqrt(x) here uses the IEEE square root and divide.
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
#pragma unroll
  for (int o = 32; o; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
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
    unsigned lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo |= iu8_code_rcp(sv[i][j], sc, rcp) << (8 * j);
      hi |= iu8_code_rcp(sv[i][4 + j], sc, rcp) << (8 * j);
    }
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

template <int T>
static __device__ __forceinline__ void had_quant_body(const unsigned short *__restrict__ x, iu8_u8 *__restrict__ q,
                                                      float *__restrict__ scale, int K,
                                                      const float *__restrict__ had_t) {
  const int row = had_row(), tid = threadIdx.x, NV = K >> 3;
  x += (size_t)row * K;
  float sv[HAD_MAXG][8];
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    const int g = tid + i * T;
    if (g >= NV) continue;
    had_load8(x + g * 8, sv[i]);
    had32(sv[i], had_t + 8 * g, tid);
  }
  had_tail<T>(sv, NV, q, scale, row, K);
}

template <int T>
static __device__ __forceinline__ void had_silu_body(const unsigned short *__restrict__ gu, iu8_u8 *__restrict__ q,
                                                     float *__restrict__ scale, int N,
                                                     const float *__restrict__ had_t) {
#pragma clang fp contract(off)
  const int row = had_row(), tid = threadIdx.x, NV = N >> 3;
  gu += (size_t)row * 2 * N;
  float sv[HAD_MAXG][8];
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    const int g = tid + i * T;
    if (g >= NV) continue;
    float vg[8], vu[8];
    had_load8(gu + g * 8, vg);
    had_load8(gu + N + g * 8, vu);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float t = iu8_bf16_f32((unsigned short)iu8_bf16_bits(vg[j] / (1.f + expf(-vg[j]))));
      sv[i][j] = iu8_bf16_f32((unsigned short)iu8_bf16_bits(t * vu[j]));
    }
    had32(sv[i], had_t + 8 * g, tid);
  }
  had_tail<T>(sv, NV, q, scale, row, N);
}

template <int T>
static __device__ __forceinline__ void had_add_rms_body(const unsigned short *__restrict__ y,
                                                        const unsigned short *__restrict__ res,
                                                        const unsigned short *__restrict__ w, iu8_u8 *__restrict__ q,
                                                        float *__restrict__ scale, unsigned short *__restrict__ res_out,
                                                        int K, float eps, const float *__restrict__ had_t) {
#pragma clang fp contract(off)
  __shared__ float s_sum[T / 32];
  const int row = had_row(), tid = threadIdx.x, NV = K >> 3;
  y += (size_t)row * K, res += (size_t)row * K, res_out += (size_t)row * K;
  float sv[HAD_MAXG][8];
  float ssq = 0.f;
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    const int g = tid + i * T;
    if (g >= NV) continue;
    float vy[8], vr[8];
    had_load8(y + g * 8, vy);
    had_load8(res + g * 8, vr);
    unsigned o[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = vy[j] + vr[j];
      sv[i][j] = v;
      ssq = __builtin_fmaf(v, v, ssq);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = iu8_bf16_bits(sv[i][2 * j]) | (iu8_bf16_bits(sv[i][2 * j + 1]) << 16);
    *(iu8_v4u *)(res_out + g * 8) = iu8_v4u{o[0], o[1], o[2], o[3]};
  }
  // the reference's trees (32 lanes, then the T/32 partials), so the sum's bits are its own
#pragma unroll
  for (int o = 16; o; o >>= 1) ssq = ssq + __shfl_down(ssq, o, 32);
  if ((tid & 31) == 0) s_sum[tid >> 5] = ssq;
  __syncthreads();
  if (tid < T / 32) {
    float v = s_sum[tid];
#pragma unroll
    for (int o = T / 64; o; o >>= 1) v = v + __shfl_down(v, o, 32);
    if (tid == 0) s_sum[0] = v;
  }
  __syncthreads();
  const float inv = __fdiv_rn(1.f, __fsqrt_rn(__fdiv_rn(s_sum[0], (float)K) + eps));
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    const int g = tid + i * T;
    if (g >= NV) continue;
    float vw[8];
    had_load8(w + g * 8, vw);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      sv[i][j] = iu8_bf16_f32((unsigned short)iu8_bf16_bits((sv[i][j] * inv) * (vw[j] + 1.f)));
    had32(sv[i], had_t + 8 * g, tid);
  }
  had_tail<T>(sv, NV, q, scale, row, K);
}

#define HAD_ARQ(name, T)                                                                                          \
  extern "C" __global__ __launch_bounds__(T) void name(                                                          \
      const unsigned short *__restrict__ y, const unsigned short *__restrict__ res,                              \
      const unsigned short *__restrict__ w, unsigned char *__restrict__ q, float *__restrict__ scale,            \
      unsigned short *__restrict__ res_out, int K, float eps, const float *__restrict__ had_t) {                 \
    had_add_rms_body<T>(y, res, w, q, scale, res_out, K, eps, had_t);                                            \
  }
HAD_ARQ(add_rms_quant_hadi8_t256_tiled1, 256)
HAD_ARQ(add_rms_quant_hadi8_t512_tiled1, 512)
#undef HAD_ARQ

#define HAD_SMQ(name, T)                                                                                          \
  extern "C" __global__ __launch_bounds__(T) void name(const unsigned short *__restrict__ gu,                    \
                                                       unsigned char *__restrict__ q, float *__restrict__ scale, \
                                                       int N, const float *__restrict__ had_t) {                 \
    had_silu_body<T>(gu, q, scale, N, had_t);                                                                    \
  }
HAD_SMQ(silu_mul_quant_hadi8_t256_tiled1, 256)
HAD_SMQ(silu_mul_quant_hadi8_t512_tiled1, 512)
#undef HAD_SMQ

#define HAD_Q(name, T)                                                                                            \
  extern "C" __global__ __launch_bounds__(T) void name(const unsigned short *__restrict__ x,                     \
                                                       unsigned char *__restrict__ q, float *__restrict__ scale, \
                                                       int k, const float *__restrict__ had_t) {                 \
    had_quant_body<T>(x, q, scale, k, had_t);                                                                    \
  }
HAD_Q(quant_hadi8_t256_tiled1, 256)
HAD_Q(quant_hadi8_t512_tiled1, 512)
#undef HAD_Q
