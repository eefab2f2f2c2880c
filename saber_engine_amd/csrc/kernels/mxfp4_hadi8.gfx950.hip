// The Hadamard-basis int8 producers for gfx950: the code object `mxfp4_hadi8`, standing in for the
// reference's object of the same name (crates/saber-kernels/hip/mxfp4_hadi8.hip, symbols
// crates/saber-kernels/src/macaq_iu8.rs:864-875) with the same kernel symbols and kernarg layouts
// (`had_t` last). A producer's final bf16-rounded values v become u = v * t, x = H32 u per 32-block
// along K, x = x * (1/sqrt(32)) (crates/saber-kernels/hip/macaq_had.h:1-19), and the per-token int8
// law runs on x (iu8_common.h); codes are stored in the gfx950 A fragment order.
//
//   add_rms_quant_hadi8_t{256,512}_tiled1   v = bf16((f32(y) + f32(res)) * inv * (f32(w) + 1)), res_out = bf16(y + res)
//   silu_mul_quant_hadi8_t{256,512}_tiled1  v = bf16(bf16(silu(gate)) * up)
//   silu_mul_quant_hadi8_lut_t{256,512}     the same with bf16(silu(gate)) read from a table (LDS)
//   quant_hadi8_t{256,512}_tiled1           v = x (no counterpart among the reference's symbols: the
//                                           transform in front of the plain producer)
//   gdn_norm_quant_hadi8_t256_tiled1        v = bf16(((x * inv_head) * w) * silu_f32(z)), per 128-element head
//
// The sums of squares keep the reference's order: add_rms per-thread fma over its groups, then
// shfl_down 16..1 inside each 32 lanes, then over the T/32 partials; gdn_norm per group
// (x1*x1, fma x0, fma x2..x7), then the xor butterfly 8, 4, 2, 1 over the head's 16 lanes. Their
// `rsqrtf` is the one thing not taken over: the device's approximate reciprocal square root cannot be
// restated on a host, so inv = 1 / sqrt(x) here uses the IEEE square root and divide (`__builtin_sqrtf`, which
// this toolchain expands to the correctly rounded sequence; its `__fsqrt_rn` is the native approximation, an
// ulp off now and then, which showed as a bf16 value of a row flipped once in a few million elements). gdn_norm's
// gate silu_f32(z) = z / (1 + expf(-z)) stays in f32 and so carries the device's expf: a function of
// a bf16 input, it is tabled by a tap kernel of the test-only object `iu8_taps` (had_silu_f32 lives
// in iu8_had.h for both) for a checker to hold against a host's.
#include "iu8_had.h"

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
  const float inv = __fdiv_rn(1.f, __builtin_sqrtf(__fdiv_rn(s_sum[0], (float)K) + eps));
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

// add_rms for few rows of up to 8,192 elements, 16 waves a row, with the sum of squares in the 256-thread form's order
// (which is part of its law: thread t of 256 runs one fma chain over its groups t, t + 256, t + 512, t + 768 in turn, then
// the 32-lane and 8-partial trees). Here thread tid owns group tid, and the chain of "thread" t = tid % 256 is handed
// from slice tid / 256 to the next through LDS -- four short turns -- while everything else (the loads, y + res and its
// store, the weights, the transform, the codes) runs on four times the threads. Same bits as
// add_rms_quant_hadi8_t256_tiled1.
static __device__ __forceinline__ void had_add_rms_v256_body(const unsigned short *__restrict__ y,
                                                             const unsigned short *__restrict__ res,
                                                             const unsigned short *__restrict__ w, iu8_u8 *__restrict__ q,
                                                             float *__restrict__ scale, unsigned short *__restrict__ res_out,
                                                             int K, float eps, const float *__restrict__ had_t) {
#pragma clang fp contract(off)
  constexpr int T = 1024, V = 256;
  __shared__ float s_chain[V];
  __shared__ float s_sum[V / 32];
  const int row = had_row(), tid = threadIdx.x, NV = K >> 3, g = tid, t = tid & (V - 1), slice = tid >> 8;
  const bool live = g < NV;
  y += (size_t)row * K, res += (size_t)row * K, res_out += (size_t)row * K;
  float sv[HAD_MAXG][8];
  float vw[8];
  if (live) {
    float vy[8], vr[8];
    had_load8(y + g * 8, vy);
    had_load8(res + g * 8, vr);
    had_load8(w + g * 8, vw);
    unsigned o[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) sv[0][j] = vy[j] + vr[j];
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = iu8_bf16_bits(sv[0][2 * j]) | (iu8_bf16_bits(sv[0][2 * j + 1]) << 16);
    *(iu8_v4u *)(res_out + g * 8) = iu8_v4u{o[0], o[1], o[2], o[3]};
  }
  for (int turn = 0; turn < T / V; ++turn) {
    if (slice == turn) {
      float ssq = turn ? s_chain[t] : 0.f;
      if (live) {
#pragma unroll
        for (int j = 0; j < 8; ++j) ssq = __builtin_fmaf(sv[0][j], sv[0][j], ssq);
      }
      s_chain[t] = ssq;
    }
    __syncthreads();
  }
  if (tid < V) {
    float ssq = s_chain[tid];
#pragma unroll
    for (int o = 16; o; o >>= 1) ssq = ssq + __shfl_down(ssq, o, 32);
    if ((tid & 31) == 0) s_sum[tid >> 5] = ssq;
  }
  __syncthreads();
  if (tid < V / 32) {
    float v = s_sum[tid];
#pragma unroll
    for (int o = V / 64; o; o >>= 1) v = v + __shfl_down(v, o, 32);
    if (tid == 0) s_sum[0] = v;
  }
  __syncthreads();
  const float inv = __fdiv_rn(1.f, __builtin_sqrtf(__fdiv_rn(s_sum[0], (float)K) + eps));
  if (live) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      sv[0][j] = iu8_bf16_f32((unsigned short)iu8_bf16_bits((sv[0][j] * inv) * (vw[j] + 1.f)));
    had32(sv[0], had_t + 8 * g, tid);
  }
  had_tail<T>(sv, NV, q, scale, row, K);
}
extern "C" __global__ __launch_bounds__(1024) void add_rms_quant_hadi8_t1024(
    const unsigned short *__restrict__ y, const unsigned short *__restrict__ res, const unsigned short *__restrict__ w,
    unsigned char *__restrict__ q, float *__restrict__ scale, unsigned short *__restrict__ res_out, int K, float eps,
    const float *__restrict__ had_t) {
  had_add_rms_v256_body(y, res, w, q, scale, res_out, K, eps, had_t);
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
HAD_SMQ(silu_mul_quant_hadi8_t1024, 1024)  // 16 waves a row: few long rows (no counterpart among the reference's symbols)
#undef HAD_SMQ

// silu_mul_quant with the bf16 silu read from a table: `lut` holds bf16(silu(x)) of every bf16 bit pattern x as
// macaq_silu_bf16_table (code object `macaq_i8q`) wrote it, i.e. this file's own expression
// vg / (1 + expf(-vg)) rounded to bf16, so the bytes are those of the computed form, which spends about 30 of
// its 55 VALU operations an element on the exp and the divide and is bound by them. A workgroup copies the
// table's middle -- magnitudes from 2^-17 up to 2^15, both signs: 2 x 4,096 entries, 16 KiB -- into LDS beside
// its row's loads; a gate outside (one in some hundred thousand of unit-scale rows) is computed as before.
// The kernel is the computed form otherwise (a workgroup a row, the same lane map). No counterpart among
// the reference's symbols (`lut` behind its kernarg list).
template <int T>
static __device__ __forceinline__ void had_silu_lut_body(const unsigned short *__restrict__ gu, iu8_u8 *__restrict__ q,
                                                         float *__restrict__ scale, int N,
                                                         const float *__restrict__ had_t,
                                                         const unsigned short *__restrict__ lut) {
#pragma clang fp contract(off)
  __shared__ __attribute__((aligned(16))) unsigned short s_lut[2 * HAD_LUT_N];
  const int row = had_row(), tid = threadIdx.x, NV = N >> 3;
  gu += (size_t)row * 2 * N;
  // the row's pieces and the table are requested together, nothing is used before the last request has left
  iu8_v4u rg[HAD_MAXG], ru[HAD_MAXG];
  had_lut_copy<unsigned short, T> tb;
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    const int g = tid + i * T;
    rg[i] = ru[i] = iu8_v4u{0u, 0u, 0u, 0u};
    if (g < NV) rg[i] = *(const iu8_v4u *)(gu + (unsigned)(g * 8)), ru[i] = *(const iu8_v4u *)(gu + N + (unsigned)(g * 8));
  }
  tb.request(lut, tid);
  tb.commit(s_lut, tid);
  __syncthreads();
  auto silu = [&](unsigned b) {  // bf16 pattern (low 16 bits) -> bf16(silu) as f32
    unsigned at;
    if (__builtin_expect(had_lut_index(b, at), 1)) return iu8_bf16_f32(s_lut[at]);
    const float x = iu8_bf16_f32((unsigned short)b);
    return iu8_bf16_f32((unsigned short)iu8_bf16_bits(x / (1.f + expf(-x))));
  };
  float sv[HAD_MAXG][8];
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    const int g = tid + i * T;
    if (g >= NV) continue;
#pragma unroll
    for (int w = 0; w < 4; ++w) {  // two products a v_cvt_pk_bf16_f32
      const float t0 = silu(rg[i][w] & 0xFFFFu), t1 = silu(rg[i][w] >> 16);
      const unsigned p2 = iu8_bf16_pack(t0 * __uint_as_float(ru[i][w] << 16), t1 * __uint_as_float(ru[i][w] & 0xFFFF0000u));
      sv[i][2 * w] = __uint_as_float(p2 << 16);
      sv[i][2 * w + 1] = __uint_as_float(p2 & 0xFFFF0000u);
    }
    had32(sv[i], had_t + 8 * g, tid);
  }
  had_tail<T>(sv, NV, q, scale, row, N);
}
#define HAD_SMQ_LUT(name, T)                                                                                      \
  extern "C" __global__ __launch_bounds__(T) void name(                                                          \
      const unsigned short *__restrict__ gu, unsigned char *__restrict__ q, float *__restrict__ scale, int N,    \
      const float *__restrict__ had_t, const unsigned short *__restrict__ lut) {                                 \
    had_silu_lut_body<T>(gu, q, scale, N, had_t, lut);                                                           \
  }
HAD_SMQ_LUT(silu_mul_quant_hadi8_lut_t256, 256)
HAD_SMQ_LUT(silu_mul_quant_hadi8_lut_t512, 512)
HAD_SMQ_LUT(silu_mul_quant_hadi8_lut_t1024, 1024)
#undef HAD_SMQ_LUT

#define HAD_Q(name, T)                                                                                            \
  extern "C" __global__ __launch_bounds__(T) void name(const unsigned short *__restrict__ x,                     \
                                                       unsigned char *__restrict__ q, float *__restrict__ scale, \
                                                       int k, const float *__restrict__ had_t) {                 \
    had_quant_body<T>(x, q, scale, k, had_t);                                                                    \
  }
HAD_Q(quant_hadi8_t256_tiled1, 256)
HAD_Q(quant_hadi8_t512_tiled1, 512)
HAD_Q(quant_hadi8_t1024, 1024)
#undef HAD_Q

// One workgroup a row of N = heads * 128 elements; z rows `zs` elements apart; w the head's 128 weights.
template <int T>
static __device__ __forceinline__ void had_gdn_norm_body(const unsigned short *__restrict__ x,
                                                         const unsigned short *__restrict__ z, long zs,
                                                         const unsigned short *__restrict__ w, iu8_u8 *__restrict__ q,
                                                         float *__restrict__ scale, int N, float eps,
                                                         const float *__restrict__ had_t) {
#pragma clang fp contract(off)
  const int row = had_row(), tid = threadIdx.x, NV = N >> 3;
  x += (size_t)row * N, z += (size_t)row * zs;
  float sv[HAD_MAXG][8];
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    // whole heads (16 lanes) are live or not together: NV is a multiple of 16, T a multiple of 16
    const int g = tid + i * T;
    const bool on = g < NV;
    const int gl = on ? g : 0;
    float vz[8], vw[8];
    had_load8(x + gl * 8, sv[i]);
    float ssq = sv[i][1] * sv[i][1];
    ssq = __builtin_fmaf(sv[i][0], sv[i][0], ssq);
#pragma unroll
    for (int j = 2; j < 8; ++j) ssq = __builtin_fmaf(sv[i][j], sv[i][j], ssq);
#pragma unroll
    for (int o = 8; o; o >>= 1) ssq = ssq + __shfl_xor(ssq, o, 16);
    if (!on) continue;
    const float inv = __fdiv_rn(1.f, __builtin_sqrtf(ssq * (1.f / 128.f) + eps));
    had_load8(z + g * 8, vz);
    had_load8(w + (g & 15) * 8, vw);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      sv[i][j] = iu8_bf16_f32((unsigned short)iu8_bf16_bits(((sv[i][j] * inv) * vw[j]) * had_silu_f32(vz[j])));
    had32(sv[i], had_t + 8 * g, tid);
  }
  had_tail<T>(sv, NV, q, scale, row, N);
}

extern "C" __global__ __launch_bounds__(256) void gdn_norm_quant_hadi8_t256_tiled1(
    const unsigned short *__restrict__ x, const unsigned short *__restrict__ z, long zs,
    const unsigned short *__restrict__ w, unsigned char *__restrict__ q, float *__restrict__ scale, int N, float eps,
    const float *__restrict__ had_t) {
  had_gdn_norm_body<256>(x, z, zs, w, q, scale, N, eps, had_t);
}
// 16 waves a row: few rows (a head's sum is the 16 lanes' whatever the workgroup's size, so the bits are the same)
extern "C" __global__ __launch_bounds__(1024) void gdn_norm_quant_hadi8_t1024(
    const unsigned short *__restrict__ x, const unsigned short *__restrict__ z, long zs,
    const unsigned short *__restrict__ w, unsigned char *__restrict__ q, float *__restrict__ scale, int N, float eps,
    const float *__restrict__ had_t) {
  had_gdn_norm_body<1024>(x, z, zs, w, q, scale, N, eps, had_t);
}
