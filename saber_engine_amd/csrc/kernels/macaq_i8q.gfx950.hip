// The per-token int8 activation producers for gfx950: the code object `macaq_i8q`.
// The law is the reference's int8 tail (crates/saber-kernels/hip/macaq_i8.h:1-13,
// crates/saber-kernels/hip/mxfp4_hadi8.hip:21-58): amax over the row, sc = max(amax/127, 1e-30)
// with an IEEE divide, q = rint(clamp(x/sc, +-127)) half-to-even; codes stored in the gfx950
// A fragment order (iu8_common.h), scale f32 per row.
//
//   macaq_i8_quant_t256           x bf16 [M,K] -> q, scale                 (grid M, block 256)
//   macaq_i8_silu_mul_quant_t256  gu bf16 [M, 2N] (gate | up) -> p = bf16(bf16(silu(g)) * u)
//                                 -> q, scale over N                       (grid M, block 256)
//                                 (crates/saber-kernels/hip/mxfp4_hadi8.hip:118-146 without the
//                                 Hadamard; signature crates/saber-kernels/src/abi.rs:315-320)
//   macaq_silu_bf16_table         the bf16 silu of all 65,536 bf16 inputs (a checker's tap)
//
// One workgroup a row; a thread owns 16-element groups g = tid + i*256 (one 16-byte store each).
#include "iu8_common.h"

#define I8Q_T 256
#define I8Q_MAXG 8  // K <= 16 * 256 * 8 = 32,768

static __device__ __forceinline__ float i8q_block_max(float v) {
  __shared__ float s_w[I8Q_T / 64];
#pragma unroll
  for (int o = 32; o; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  if ((threadIdx.x & 63) == 0) s_w[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = s_w[0];
#pragma unroll
  for (int w = 1; w < I8Q_T / 64; ++w) r = fmaxf(r, s_w[w]);
  return r;
}

// codes of one row from v[g][16] (f32 values), written in A fragment order
static __device__ __forceinline__ void i8q_tail(float (&v)[I8Q_MAXG][16], int G, iu8_u8 *__restrict__ q,
                                                float *__restrict__ scale, int row, int K) {
  const int tid = threadIdx.x;
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < I8Q_MAXG; ++i) {
    if (tid + i * I8Q_T >= G) break;
#pragma unroll
    for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
  }
  amax = i8q_block_max(amax);
  const float sc = fmaxf(__fdiv_rn(amax, 127.f), 1e-30f);
  if (tid == 0) scale[row] = sc;
  iu8_u8 *qrow = q + (size_t)(row >> 4) * (K >> 6) * 1024 + (row & 15) * 16;
#pragma unroll
  for (int i = 0; i < I8Q_MAXG; ++i) {
    const int g = tid + i * I8Q_T;
    if (g >= G) break;
    unsigned d[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      d[w] = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) d[w] |= iu8_code(v[i][w * 4 + b], sc) << (8 * b);
    }
    *(iu8_v4u *)(qrow + (size_t)(g >> 2) * 1024 + (g & 3) * 256) = iu8_v4u{d[0], d[1], d[2], d[3]};
  }
}

extern "C" __global__ __launch_bounds__(I8Q_T) void macaq_i8_quant_t256(const unsigned short *__restrict__ x,
                                                                        unsigned char *__restrict__ q,
                                                                        float *__restrict__ scale, int k) {
  const int row = blockIdx.x, G = k >> 4;
  const unsigned short *xr = x + (size_t)row * k;
  float v[I8Q_MAXG][16];
#pragma unroll
  for (int i = 0; i < I8Q_MAXG; ++i) {
    const int g = threadIdx.x + i * I8Q_T;
    if (g >= G) break;
    const iu8_v4u lo = *(const iu8_v4u *)(xr + g * 16), hi = *(const iu8_v4u *)(xr + g * 16 + 8);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      v[i][2 * w] = __uint_as_float(lo[w] << 16);
      v[i][2 * w + 1] = __uint_as_float(lo[w] & 0xFFFF0000u);
      v[i][8 + 2 * w] = __uint_as_float(hi[w] << 16);
      v[i][8 + 2 * w + 1] = __uint_as_float(hi[w] & 0xFFFF0000u);
    }
  }
  i8q_tail(v, G, q, scale, row, k);
}

static __device__ __forceinline__ float i8q_silu_bf16(float x) {
#pragma clang fp contract(off)
  return iu8_bf16_f32((unsigned short)iu8_bf16_bits(x / (1.f + expf(-x))));
}

// `row_tok` / `meta` are optional (may be null): with them the kernel runs on the expert-major
// rows of a routed layer and skips pad rows (row_tok < 0) and rows past meta[1]
// (signature crates/saber-kernels/src/abi.rs:344-351).
extern "C" __global__ __launch_bounds__(I8Q_T) void macaq_i8_silu_mul_quant_t256(
    const unsigned short *__restrict__ gu, unsigned char *__restrict__ q, float *__restrict__ scale, int n,
    const int *__restrict__ row_tok, const int *__restrict__ meta) {
#pragma clang fp contract(off)
  const int row = blockIdx.x, G = n >> 4;
  if (meta != nullptr && row >= meta[1]) return;
  if (row_tok != nullptr && row_tok[row] < 0) return;
  const unsigned short *gr = gu + (size_t)row * 2 * n;
  float v[I8Q_MAXG][16];
#pragma unroll
  for (int i = 0; i < I8Q_MAXG; ++i) {
    const int g = threadIdx.x + i * I8Q_T;
    if (g >= G) break;
    union { iu8_v4u u[2]; unsigned short h[16]; } vg, vu;
    vg.u[0] = *(const iu8_v4u *)(gr + g * 16);
    vg.u[1] = *(const iu8_v4u *)(gr + g * 16 + 8);
    vu.u[0] = *(const iu8_v4u *)(gr + n + g * 16);
    vu.u[1] = *(const iu8_v4u *)(gr + n + g * 16 + 8);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float t = i8q_silu_bf16(iu8_bf16_f32(vg.h[j]));
      v[i][j] = iu8_bf16_f32((unsigned short)iu8_bf16_bits(t * iu8_bf16_f32(vu.h[j])));
    }
  }
  i8q_tail(v, G, q, scale, row, n);
}

extern "C" __global__ __launch_bounds__(256) void macaq_silu_bf16_table(unsigned short *__restrict__ out) {
  const unsigned i = blockIdx.x * 256 + threadIdx.x;
  out[i] = (unsigned short)iu8_bf16_bits(i8q_silu_bf16(iu8_bf16_f32((unsigned short)i)));
}
