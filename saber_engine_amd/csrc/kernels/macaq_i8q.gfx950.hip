// The per-token int8 activation producers for gfx950: the code object `macaq_i8q`.
// The law is the reference's int8 tail (crates/saber-kernels/hip/macaq_i8.h:1-13,
// crates/saber-kernels/hip/mxfp4_hadi8.hip:21-58): amax over the row, sc = max(amax/127, 1e-30)
// with an IEEE divide, q = rint(clamp(x/sc, +-127)) half-to-even; codes stored in the gfx950
// A fragment order (iu8_common.h), scale f32 per row.
//
//   macaq_i8_quant_t256           x bf16 [M,K] -> q, scale                 (grid M, block 256)
//   macaq_i8_rowscale_t256        the rows' scales alone (the pass in front of macaq_iu8_pfq_*)
//   macaq_i8_quant_rm_t256        the same with the codes row-major, q[row * K + col] (the operand a
//                                 grouped GEMM gathers whole token rows from)
//   macaq_i8_quant_rows_t256      the first through a row map: output row r = input row row_tok[r]
//                                 (the gathered, expert-major activations of a routed layer)
//   macaq_i8_silu_mul_quant_t256  gu bf16 [M, 2N] (gate | up) -> p = bf16(bf16(silu(g)) * u)
//                                 -> q, scale over N                       (grid M, block 256)
//                                 (crates/saber-kernels/hip/mxfp4_hadi8.hip:118-146 without the
//                                 Hadamard; signature crates/saber-kernels/src/abi.rs:315-320)
//   macaq_i8_quant_t1024, macaq_i8_silu_mul_quant_t1024   the first and the fifth with 16 waves a row (block
//                                 1024): few rows of more than 4,096 elements
//   macaq_i8_quant_w64, macaq_i8_silu_mul_quant_w64   the same two for rows of up to 4,096 elements,
//                                 a wave a row, four rows a workgroup (grid M/4, block 256)
//   macaq_i8_silu_mul_quant_lut_w64   the second with the bf16 silu read from a 65,536-entry table in
//                                 LDS: persistent, 16 waves, a wave a row (grid <= 256, block 1024)
//   macaq_silu_bf16_table         the bf16 silu of all 65,536 bf16 inputs (a checker's tap)
//
// One workgroup a row; a thread owns 16-element groups g = tid + i*256 (one 16-byte store each).
// A kernel holds its row in registers, so each comes in forms for rows of up to 4,096 (_g1), 8,192
// (_g2), 20,480 (_g5) and 32,768 (no suffix) elements: the narrow forms keep the register count low
// enough for eight waves a SIMD, which is what hides the load latency of a one-pass row kernel.
#include "iu8_common.h"

#define I8Q_T 256

// The row of workgroup b. The hardware deals consecutive workgroups round-robin over the 8 XCDs, and
// the 16 rows of an A tile interleave their 16-byte pieces inside 256-byte runs: so the 8 tiles of
// every full group of 128 rows go one to an XCD, and an XCD's L2 sees whole lines before it writes
// them back. Rows past the last full group keep their order.
static __device__ __forceinline__ int i8q_row() {
  const int b = blockIdx.x, full = (int)gridDim.x & ~127;
  if (b >= full) return b;
  return (b & ~127) + (b & 7) * 16 + ((b & 127) >> 3);
}

template <int T = I8Q_T>
static __device__ __forceinline__ float i8q_block_max(float v) {
  __shared__ float s_w[T / 64];
  v = iu8_wave_max_nonneg(v);
  if ((threadIdx.x & 63) == 0) s_w[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = s_w[0];
#pragma unroll
  for (int w = 1; w < T / 64; ++w) r = fmaxf(r, s_w[w]);
  return r;
}

// codes of one row from v[g][16] (f32 values), written in A fragment order (RM: row-major, K bytes a row)
// SCALE_ONLY: the row's scale alone (the row-maximum pass in front of a GEMM that makes the codes itself)
template <int I8Q_MAXG, bool RM = false, bool SCALE_ONLY = false, int T = I8Q_T>
static __device__ __forceinline__ void i8q_tail(float (&v)[I8Q_MAXG][16], int G, iu8_u8 *__restrict__ q,
                                                float *__restrict__ scale, int row, int K) {
  const int tid = threadIdx.x;
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < I8Q_MAXG; ++i) {
    if (tid + i * T >= G) continue;
#pragma unroll
    for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
  }
  amax = i8q_block_max<T>(amax);
  const float sc = fmaxf(__fdiv_rn(amax, 127.f), 1e-30f);
  const float rcp = __fdiv_rn(1.f, sc);
  if (tid == 0) scale[row] = sc;
  if constexpr (SCALE_ONLY) return;
  iu8_u8 *qrow = q + (size_t)(row >> 4) * (K >> 6) * 1024 + (row & 15) * 16;
#pragma unroll
  for (int i = 0; i < I8Q_MAXG; ++i) {
    const int g = tid + i * T;
    if (g >= G) continue;
    unsigned d[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      d[w] = iu8_code4_rcp(v[i][w * 4], v[i][w * 4 + 1], v[i][w * 4 + 2], v[i][w * 4 + 3], sc, rcp);
    }
    if constexpr (RM) *(iu8_v4u *)(q + (size_t)row * K + g * 16) = iu8_v4u{d[0], d[1], d[2], d[3]};
    else *(iu8_v4u *)(qrow + (size_t)(g >> 2) * 1024 + (g & 3) * 256) = iu8_v4u{d[0], d[1], d[2], d[3]};
  }
}

// A group's 16 elements, zeros when the group is past the row's end. Nothing uses the registers before
// every group of the row has been requested: a load whose data is used under the same test is waited
// for before the next is requested -- MAXG memory latencies a row instead of one.
static __device__ __forceinline__ void i8q_pk_load(unsigned (&g)[8], const unsigned short *p, bool live) {
  iu8_v4u lo = {0u, 0u, 0u, 0u}, hi = {0u, 0u, 0u, 0u};
  if (live) lo = *(const iu8_v4u *)p, hi = *(const iu8_v4u *)(p + 8);
#pragma unroll
  for (int w = 0; w < 4; ++w) g[w] = lo[w], g[4 + w] = hi[w];
}
template <int I8Q_MAXG, bool RM, bool SCALE_ONLY>
static __device__ __forceinline__ void i8q_tail_pk(const unsigned (&pk)[I8Q_MAXG][8], int G, iu8_u8 *__restrict__ q,
                                                   float *__restrict__ scale, int row, int K) {
  const int tid = threadIdx.x;
  const float amax = i8q_block_max(iu8_pk_amax(pk));
  const float sc = fmaxf(__fdiv_rn(amax, 127.f), 1e-30f);
  const float rcp = __fdiv_rn(1.f, sc);
  if (tid == 0) scale[row] = sc;
  if constexpr (SCALE_ONLY) return;
  iu8_u8 *qrow = q + (size_t)(row >> 4) * (K >> 6) * 1024 + (row & 15) * 16;
#pragma unroll
  for (int i = 0; i < I8Q_MAXG; ++i) {
    const int g = tid + i * I8Q_T;
    if (g >= G) continue;
    const iu8_v4u d = iu8_pk_codes(pk[i], sc, rcp);
    if constexpr (RM) *(iu8_v4u *)(q + (size_t)row * K + g * 16) = d;
    else *(iu8_v4u *)(qrow + (size_t)(g >> 2) * 1024 + (g & 3) * 256) = d;
    __builtin_amdgcn_sched_barrier(0);  // a group's codes at a time: their temporaries are what fills the registers
  }
}

// `row_tok` / `meta` (optional, may be null): with them output row r is the quantised input row
// row_tok[r] (the expert-major rows of a routed layer, gathered here once so that the grouped GEMM
// reads whole fragments); pad rows (row_tok < 0) and rows past meta[1] are skipped.
template <int I8Q_MAXG, bool RM = false, bool SCALE_ONLY = false, int T = I8Q_T>
static __device__ __forceinline__ void i8q_quant_body(const unsigned short *__restrict__ x, unsigned char *__restrict__ q,
                                                      float *__restrict__ scale, int k,
                                                      const int *__restrict__ row_tok = nullptr,
                                                      const int *__restrict__ meta = nullptr) {
  const int row = i8q_row(), G = k >> 4;
  if (meta != nullptr && row >= meta[1]) return;
  int src = row;
  if (row_tok != nullptr) {
    src = row_tok[row];
    if (src < 0) return;
  }
  const unsigned short *xr = x + (size_t)src * k;
  if constexpr (I8Q_MAXG >= 5) {
    static_assert(I8Q_MAXG < 5 || T == I8Q_T, "the packed forms are the 256-thread ones");
    // The long forms request a row's pieces all at once (i8q_pk_load) and keep them packed as they came, 8
    // registers a group instead of 16: the form for up to 20,480 elements then runs eight waves a SIMD
    // (2,048 rows of 17,408: 26.0 -> 21.9 us). The forms of one or two groups measured 4-8 % slower this way.
    unsigned pk[I8Q_MAXG][8];
#pragma unroll
    for (int i = 0; i < I8Q_MAXG; ++i) i8q_pk_load(pk[i], xr + (threadIdx.x + i * I8Q_T) * 16, (int)threadIdx.x + i * I8Q_T < G);
    i8q_tail_pk<I8Q_MAXG, RM, SCALE_ONLY>(pk, G, q, scale, row, k);
  } else {
    float v[I8Q_MAXG][16];
#pragma unroll
    for (int i = 0; i < I8Q_MAXG; ++i) {
      const int g = threadIdx.x + i * T;
      if (g >= G) continue;
      const iu8_v4u lo = *(const iu8_v4u *)(xr + g * 16), hi = *(const iu8_v4u *)(xr + g * 16 + 8);
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        v[i][2 * w] = __uint_as_float(lo[w] << 16);
        v[i][2 * w + 1] = __uint_as_float(lo[w] & 0xFFFF0000u);
        v[i][8 + 2 * w] = __uint_as_float(hi[w] << 16);
        v[i][8 + 2 * w + 1] = __uint_as_float(hi[w] & 0xFFFF0000u);
      }
    }
    i8q_tail<I8Q_MAXG, RM, SCALE_ONLY, T>(v, G, q, scale, row, k);
  }
}
#define I8Q_QUANT(name, MAXG, WPE)                                                                              \
  extern "C" __global__ __launch_bounds__(I8Q_T) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void name(      \
      const unsigned short *__restrict__ x, unsigned char *__restrict__ q, float *__restrict__ scale, int k) {  \
    i8q_quant_body<MAXG>(x, q, scale, k);                                                                       \
  }
I8Q_QUANT(macaq_i8_quant_t256, 8, 5)
I8Q_QUANT(macaq_i8_quant_t256_g5, 5, 8)
I8Q_QUANT(macaq_i8_quant_t256_g2, 2, 8)
I8Q_QUANT(macaq_i8_quant_t256_g1, 1, 8)
#undef I8Q_QUANT
// the rows' scales alone: x bf16 [M, K] -> scale f32 [M] (what macaq_i8_quant_* stores beside its codes)
#define I8Q_ROWSCALE(name, MAXG)                                                                                \
  extern "C" __global__ __launch_bounds__(I8Q_T) void name(const unsigned short *__restrict__ x,                \
                                                           float *__restrict__ scale, int k) {                  \
    i8q_quant_body<MAXG, false, true>(x, nullptr, scale, k);                                                    \
  }
I8Q_ROWSCALE(macaq_i8_rowscale_t256, 8)
I8Q_ROWSCALE(macaq_i8_rowscale_t256_g2, 2)
I8Q_ROWSCALE(macaq_i8_rowscale_t256_g1, 1)
#undef I8Q_ROWSCALE
// row-major codes (q[row * k + col]): the operand a routed layer's grouped GEMM gathers token rows from
#define I8Q_QUANT_RM(name, MAXG)                                                                                \
  extern "C" __global__ __launch_bounds__(I8Q_T) void name(const unsigned short *__restrict__ x,                \
                                                           unsigned char *__restrict__ q, float *__restrict__ scale, \
                                                           int k) {                                             \
    i8q_quant_body<MAXG, true>(x, q, scale, k);                                                                 \
  }
I8Q_QUANT_RM(macaq_i8_quant_rm_t256, 8)
I8Q_QUANT_RM(macaq_i8_quant_rm_t256_g2, 2)
I8Q_QUANT_RM(macaq_i8_quant_rm_t256_g1, 1)
#undef I8Q_QUANT_RM
#define I8Q_QUANT_ROWS(name, MAXG)                                                                               \
  extern "C" __global__ __launch_bounds__(I8Q_T) void name(                                                      \
      const unsigned short *__restrict__ x, unsigned char *__restrict__ q, float *__restrict__ scale, int k,     \
      const int *__restrict__ row_tok, const int *__restrict__ meta) {                                           \
    i8q_quant_body<MAXG>(x, q, scale, k, row_tok, meta);                                                         \
  }
I8Q_QUANT_ROWS(macaq_i8_quant_rows_t256, 8)
I8Q_QUANT_ROWS(macaq_i8_quant_rows_t256_g2, 2)
I8Q_QUANT_ROWS(macaq_i8_quant_rows_t256_g1, 1)
#undef I8Q_QUANT_ROWS

static __device__ __forceinline__ float i8q_silu_bf16(float x) {
#pragma clang fp contract(off)
  return iu8_bf16_f32((unsigned short)iu8_bf16_bits(x / (1.f + expf(-x))));
}

// `row_tok` / `meta` are optional (may be null): with them the kernel runs on the expert-major
// rows of a routed layer and skips pad rows (row_tok < 0) and rows past meta[1]
// (signature crates/saber-kernels/src/abi.rs:344-351).
template <int I8Q_MAXG, int T = I8Q_T>
static __device__ __forceinline__ void i8q_silu_body(const unsigned short *__restrict__ gu, unsigned char *__restrict__ q,
                                                     float *__restrict__ scale, int n, const int *__restrict__ row_tok,
                                                     const int *__restrict__ meta) {
#pragma clang fp contract(off)
  const int row = i8q_row(), G = n >> 4;
  if (meta != nullptr && row >= meta[1]) return;
  if (row_tok != nullptr && row_tok[row] < 0) return;
  const unsigned short *gr = gu + (size_t)row * 2 * n;
  float v[I8Q_MAXG][16];
#pragma unroll
  for (int i = 0; i < I8Q_MAXG; ++i) {
    const int g = threadIdx.x + i * T;
    if (g >= G) continue;
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
  i8q_tail<I8Q_MAXG, false, false, T>(v, G, q, scale, row, n);
}
#define I8Q_SILU(name, MAXG)                                                                                     \
  extern "C" __global__ __launch_bounds__(I8Q_T) void name(                                                      \
      const unsigned short *__restrict__ gu, unsigned char *__restrict__ q, float *__restrict__ scale, int n,    \
      const int *__restrict__ row_tok, const int *__restrict__ meta) {                                           \
    i8q_silu_body<MAXG>(gu, q, scale, n, row_tok, meta);                                                         \
  }
I8Q_SILU(macaq_i8_silu_mul_quant_t256, 8)
I8Q_SILU(macaq_i8_silu_mul_quant_t256_g5, 5)
I8Q_SILU(macaq_i8_silu_mul_quant_t256_g2, 2)
I8Q_SILU(macaq_i8_silu_mul_quant_t256_g1, 1)
#undef I8Q_SILU

// Few long rows: 16 waves a row, a thread owns groups g = tid + i*1024 (rows of up to 32,768 elements).
// With fewer rows than CUs a row's time is one workgroup's, and a 256-thread workgroup walks a row of
// 17,408 in five dependent steps a thread (5 groups of loads, conversions, exps); here it is two at most.
extern "C" __global__ __launch_bounds__(1024) void macaq_i8_quant_t1024(const unsigned short *__restrict__ x,
                                                                        unsigned char *__restrict__ q,
                                                                        float *__restrict__ scale, int k) {
  i8q_quant_body<2, false, false, 1024>(x, q, scale, k);
}
extern "C" __global__ __launch_bounds__(1024) void macaq_i8_silu_mul_quant_t1024(
    const unsigned short *__restrict__ gu, unsigned char *__restrict__ q, float *__restrict__ scale, int n,
    const int *__restrict__ row_tok, const int *__restrict__ meta) {
  i8q_silu_body<2, 1024>(gu, q, scale, n, row_tok, meta);
}

// ---------------------------------------------------------------------------- a wave a row
// Rows of up to 4,096 elements: four rows a workgroup, one wave each, a lane owns groups
// g = lane + i*64. No LDS and no barrier: the row maximum is a wave butterfly. The launch covers
// 4 * gridDim.x rows (the caller's row count is a multiple of 4).
#define I8Q_WG 4  // groups a lane
static __device__ __forceinline__ int i8q_row4() {
  const int b = blockIdx.x, full = (int)gridDim.x & ~31;  // 32 workgroups = 128 rows = 8 tiles, one an XCD
  const int u = b >= full ? b : (b & ~31) + (b & 7) * 4 + ((b & 31) >> 3);
  return u * 4 + (threadIdx.x >> 6);
}
static __device__ __forceinline__ void i8q_tail_w64(float (&v)[I8Q_WG][16], int G, iu8_u8 *__restrict__ q,
                                                    float *__restrict__ scale, int row, int K) {
  const int lane = threadIdx.x & 63;
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < I8Q_WG; ++i) {
    if (lane + i * 64 >= G) continue;
#pragma unroll
    for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
  }
  amax = iu8_wave_max_nonneg(amax);
  const float sc = fmaxf(__fdiv_rn(amax, 127.f), 1e-30f);
  const float rcp = __fdiv_rn(1.f, sc);
  if (lane == 0) scale[row] = sc;
  iu8_u8 *qrow = q + (size_t)(row >> 4) * (K >> 6) * 1024 + (row & 15) * 16;
#pragma unroll
  for (int i = 0; i < I8Q_WG; ++i) {
    const int g = lane + i * 64;
    if (g >= G) continue;
    unsigned d[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      d[w] = iu8_code4_rcp(v[i][w * 4], v[i][w * 4 + 1], v[i][w * 4 + 2], v[i][w * 4 + 3], sc, rcp);
    }
    *(iu8_v4u *)(qrow + (size_t)(g >> 2) * 1024 + (g & 3) * 256) = iu8_v4u{d[0], d[1], d[2], d[3]};
  }
}

extern "C" __global__ __launch_bounds__(256) void macaq_i8_quant_w64(const unsigned short *__restrict__ x,
                                                                     unsigned char *__restrict__ q,
                                                                     float *__restrict__ scale, int k) {
  const int row = i8q_row4(), G = k >> 4, lane = threadIdx.x & 63;
  const unsigned short *xr = x + (size_t)row * k;
  float v[I8Q_WG][16];
#pragma unroll
  for (int i = 0; i < I8Q_WG; ++i) {
    const int g = lane + i * 64;
    if (g >= G) continue;
    const iu8_v4u lo = *(const iu8_v4u *)(xr + g * 16), hi = *(const iu8_v4u *)(xr + g * 16 + 8);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      v[i][2 * w] = __uint_as_float(lo[w] << 16);
      v[i][2 * w + 1] = __uint_as_float(lo[w] & 0xFFFF0000u);
      v[i][8 + 2 * w] = __uint_as_float(hi[w] << 16);
      v[i][8 + 2 * w + 1] = __uint_as_float(hi[w] & 0xFFFF0000u);
    }
  }
  i8q_tail_w64(v, G, q, scale, row, k);
}

extern "C" __global__ __launch_bounds__(256) void macaq_i8_silu_mul_quant_w64(
    const unsigned short *__restrict__ gu, unsigned char *__restrict__ q, float *__restrict__ scale, int n,
    const int *__restrict__ row_tok, const int *__restrict__ meta) {
#pragma clang fp contract(off)
  const int row = i8q_row4(), G = n >> 4, lane = threadIdx.x & 63;
  if (meta != nullptr && row >= meta[1]) return;
  if (row_tok != nullptr && row_tok[row] < 0) return;
  const unsigned short *gr = gu + (size_t)row * 2 * n;
  float v[I8Q_WG][16];
#pragma unroll
  for (int i = 0; i < I8Q_WG; ++i) {
    const int g = lane + i * 64;
    if (g >= G) continue;
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
  i8q_tail_w64(v, G, q, scale, row, n);
}

// The same op for many rows, with the bf16 silu read from a table: `lut` holds the silu of every
// bf16 bit pattern as macaq_silu_bf16_table wrote it (128 KiB), each workgroup copies it into LDS
// once and its 16 waves then walk the rows, a wave a row, the 16 rows of an A tile on one workgroup
// (tile = blockIdx.x + r * gridDim.x) so that the tile's 256-byte runs fill in one L2. The computed
// form spends about 60 VALU operations an element on exp and the IEEE divide and is bound by them;
// this one is bound by memory. Same bytes: the table is that form's own output.
extern "C" __global__ __launch_bounds__(1024) void macaq_i8_silu_mul_quant_lut_w64(
    const unsigned short *__restrict__ gu, unsigned char *__restrict__ q, float *__restrict__ scale, int n,
    const int *__restrict__ row_tok, const int *__restrict__ meta, const unsigned short *__restrict__ lut) {
#pragma clang fp contract(off)
  __shared__ __attribute__((aligned(16))) unsigned short s_lut[65536];
  for (int i = threadIdx.x; i < 65536 / 8; i += 1024) ((iu8_v4u *)s_lut)[i] = ((const iu8_v4u *)lut)[i];
  __syncthreads();
  const int G = n >> 4, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rows = meta != nullptr ? meta[1] : 0x7FFFFFFF;
  for (int tile = blockIdx.x;; tile += gridDim.x) {
    const int row = tile * 16 + wave;
    if (tile * 16 >= rows) break;
    if (row >= rows || (row_tok != nullptr && row_tok[row] < 0)) continue;
    const unsigned short *gr = gu + (size_t)row * 2 * n;
    float v[I8Q_WG][16];
#pragma unroll
    for (int i = 0; i < I8Q_WG; ++i) {
      const int g = lane + i * 64;
      if (g >= G) continue;
      union { iu8_v4u u[2]; unsigned short h[16]; } vg, vu;
      vg.u[0] = *(const iu8_v4u *)(gr + g * 16);
      vg.u[1] = *(const iu8_v4u *)(gr + g * 16 + 8);
      vu.u[0] = *(const iu8_v4u *)(gr + n + g * 16);
      vu.u[1] = *(const iu8_v4u *)(gr + n + g * 16 + 8);
#pragma unroll
      for (int j = 0; j < 16; j += 2) {  // two products a v_cvt_pk_bf16_f32
        const float t0 = iu8_bf16_f32(s_lut[vg.h[j]]), t1 = iu8_bf16_f32(s_lut[vg.h[j + 1]]);
        const unsigned p2 = iu8_bf16_pack(t0 * iu8_bf16_f32(vu.h[j]), t1 * iu8_bf16_f32(vu.h[j + 1]));
        v[i][j] = __uint_as_float(p2 << 16);
        v[i][j + 1] = __uint_as_float(p2 & 0xFFFF0000u);
      }
    }
    i8q_tail_w64(v, G, q, scale, row, n);
  }
}

extern "C" __global__ __launch_bounds__(256) void macaq_silu_bf16_table(unsigned short *__restrict__ out) {
  const unsigned i = blockIdx.x * 256 + threadIdx.x;
  out[i] = (unsigned short)iu8_bf16_bits(i8q_silu_bf16(iu8_bf16_f32((unsigned short)i)));
}
