// The attention output gate's Hadamard-basis int8 producer for gfx950: the code object
// `attn_glue_hadi8`, standing in for the reference's object of the same name
// (crates/saber-kernels/hip/attn_glue_hadi8.hip, symbol crates/saber-kernels/src/macaq_iu8.rs:870)
// with the same kernel symbol and kernarg layout (`had_t` last).
//
//   attn_gate_quant_hadi8_t256_tiled1   v = bf16(core * bf16(sigmoid(gate))), the o_proj's A producer.
//       core bf16 [rows, n]; gate is the projection's [q | gate] block, row stride `gs`, head stride
//       2*hd, the gate half at +hd (crates/saber-kernels/src/abi.rs:2683-2694); n <= 6144.
//
// Then u = v * t, x = H32 u per 32-block, x * (1/sqrt(32)), and the per-token int8 law on x; codes
// in the gfx950 A fragment order. sigmoid = 1 / (1 + expf(-g)) is rounded to bf16 before use, so the
// device's expf shows only through a bf16 -> bf16 function (glue_sigmoid_bf16, iu8_had.h), which a
// tap kernel of the test-only object `iu8_taps` tables.
#include "iu8_had.h"

// `lut` (the table form, may be null): bf16(sigmoid) of every bf16 pattern as attn_gate_sigmoid_bf16_table wrote
// it; the gate is then read from the table's middle in LDS (iu8_had.h) instead of computed.
template <bool LUT, int T = 256>
static __device__ __forceinline__ void attn_gate_body(const unsigned short *__restrict__ core,
                                                      const unsigned short *__restrict__ gate, unsigned char *__restrict__ q,
                                                      float *__restrict__ scale, int n, int hd, int gs,
                                                      const float *__restrict__ had_t,
                                                      const unsigned short *__restrict__ lut) {
#pragma clang fp contract(off)
  const int row = had_row(), tid = threadIdx.x, NV = n >> 3;
  core += (size_t)row * n, gate += (size_t)row * gs;
  __shared__ __attribute__((aligned(16))) unsigned short s_lut[LUT ? 2 * HAD_LUT_N : 8];
  if constexpr (LUT) {
    had_lut_copy<unsigned short, T> tb;
    tb.request(lut, tid);
    tb.commit(s_lut, tid);
    __syncthreads();
  }
  auto sig = [&](float g) {
    if constexpr (LUT) {
      unsigned at;
      if (__builtin_expect(had_lut_index(__float_as_uint(g) >> 16, at), 1)) return iu8_bf16_f32(s_lut[at]);
    }
    return glue_sigmoid_bf16(g);
  };
  float sv[HAD_MAXG][8];
#pragma unroll
  for (int i = 0; i < HAD_MAXG; ++i) {
    const int g = tid + i * T;
    if (g >= NV) continue;
    const int e = g << 3, h = e / hd, o = e - h * hd;
    float vc[8], vg[8];
    had_load8(core + e, vc);
    had_load8(gate + (size_t)h * 2 * hd + hd + o, vg);
#pragma unroll
    for (int j = 0; j < 8; ++j) sv[i][j] = iu8_bf16_f32((unsigned short)iu8_bf16_bits(vc[j] * sig(vg[j])));
    had32(sv[i], had_t + 8 * g, tid);
  }
  had_tail<T>(sv, NV, q, scale, row, n);
}
extern "C" __global__ __launch_bounds__(256) void attn_gate_quant_hadi8_t256_tiled1(
    const unsigned short *__restrict__ core, const unsigned short *__restrict__ gate, unsigned char *__restrict__ q,
    float *__restrict__ scale, int n, int hd, int gs, const float *__restrict__ had_t) {
  attn_gate_body<false>(core, gate, q, scale, n, hd, gs, had_t, nullptr);
}
// the table form (no counterpart among the reference's symbols: `lut` behind its kernarg list)
extern "C" __global__ __launch_bounds__(256) void attn_gate_quant_hadi8_lut_t256(
    const unsigned short *__restrict__ core, const unsigned short *__restrict__ gate, unsigned char *__restrict__ q,
    float *__restrict__ scale, int n, int hd, int gs, const float *__restrict__ had_t,
    const unsigned short *__restrict__ lut) {
  attn_gate_body<true>(core, gate, q, scale, n, hd, gs, had_t, lut);
}
// 16 waves a row, for few rows (no counterpart among the reference's symbols)
extern "C" __global__ __launch_bounds__(1024) void attn_gate_quant_hadi8_t1024(
    const unsigned short *__restrict__ core, const unsigned short *__restrict__ gate, unsigned char *__restrict__ q,
    float *__restrict__ scale, int n, int hd, int gs, const float *__restrict__ had_t) {
  attn_gate_body<false, 1024>(core, gate, q, scale, n, hd, gs, had_t, nullptr);
}
extern "C" __global__ __launch_bounds__(1024) void attn_gate_quant_hadi8_lut_t1024(
    const unsigned short *__restrict__ core, const unsigned short *__restrict__ gate, unsigned char *__restrict__ q,
    float *__restrict__ scale, int n, int hd, int gs, const float *__restrict__ had_t,
    const unsigned short *__restrict__ lut) {
  attn_gate_body<true, 1024>(core, gate, q, scale, n, hd, gs, had_t, lut);
}
// bf16(sigmoid) of all 65,536 bf16 inputs (bf16 bits [65536]): the table of attn_gate_quant_hadi8_lut_t256.
// grid 256, block 256.
extern "C" __global__ __launch_bounds__(256) void attn_gate_sigmoid_bf16_table(unsigned short *__restrict__ out) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  out[i] = (unsigned short)iu8_bf16_bits(glue_sigmoid_bf16(iu8_bf16_f32((unsigned short)i)));
}
