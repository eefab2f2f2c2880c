// The parity suite's taps: the code object `iu8_taps`. Test infrastructure, not part of the plugin
// set a host loads: it is built beside the plugin directory (in `taps/`) and a checker adds it to a
// context by its manifest.
//
//   macaq_iu8_dec_{w4,w8}_tm1_acc, macaq_iu8_dec_w4_tm4_acc, macaq_iu8_pf_{w4,w8}_acc
//       the GEMM bodies of `macaq_iu8` with the raw int32 accumulators stored instead of the bf16
//       epilogue (`c` is int32 [M,N]; 16 * sum(a*w) for W4, sum(a*w) for W8): the product kernels'
//       argument lists, so the same descriptors launch them
//   mxfp4_hadi8_silu_f32_table          had_silu_f32 of all 65,536 bf16 inputs (f32 out)
//   attn_glue_hadi8_sigmoid_bf16_table  glue_sigmoid_bf16 of all 65,536 bf16 inputs (bf16 bits out)
#include "iu8_dense_defs.h"
#include "iu8_had.h"

#define IU8_DEC_TAP(name, TM, W8, NT, KW, WPB, D, ALDS, ACC) IU8_DEC(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)
#define IU8_PF_TAP(name, W8, WMW, WNW, TM, TN, ACC, ST, OCC, DEEP) IU8_PF32(name, W8, WMW, WNW, TM, TN, ACC, ST, OCC, DEEP)
#include "iu8_variants.def"

extern "C" __global__ __launch_bounds__(256) void mxfp4_hadi8_silu_f32_table(float *__restrict__ out) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  out[i] = had_silu_f32(iu8_bf16_f32((unsigned short)i));
}

extern "C" __global__ __launch_bounds__(256) void attn_glue_hadi8_sigmoid_bf16_table(unsigned short *__restrict__ out) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  out[i] = (unsigned short)iu8_bf16_bits(glue_sigmoid_bf16(iu8_bf16_f32((unsigned short)i)));
}
