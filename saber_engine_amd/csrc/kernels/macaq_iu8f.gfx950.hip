// The fused decode forms of the W4A8-iu8 GEMM for gfx950: the code object `macaq_iu8f`, standing in
// for the reference's object of the same name (crates/saber-kernels/hip/macaq_iu8f.hip:148-178,
// symbols crates/saber-kernels/src/macaq_iu8.rs:508-515, kernarg list
// crates/saber-kernels/src/abi.rs:3411-3432).
//
// THE DECODE PAIR: two W4 decode GEMMs that read one activation operand (one A, one per-token
// scale; the same M and K) in one dispatch. Problem 0's grid -- nb column blocks x ks shares of K,
// column block fastest -- then problem 1's, end to end in gridDim.x; each workgroup runs the plain
// decode body (iu8_gemm.h) on its problem's operands, so the bytes of c and c_b are those of two
// separate launches. What it saves is a launch: on this card a decode GEMV launch costs several
// microseconds of start and drain beside its streaming time. The `pairb` symbols lay the second
// problem's workgroups in front of problem 0's (the reference's ba-first order,
// crates/saber-kernels/src/macaq_iu8.rs:549-553): the same bytes, the small half not in the tail.
#include "iu8_gemm.h"
#include "iu8_chain.h"

#define IU8F_PAIR(name, TM, NT, KW, WPB, D, ALDS, BFIRST)                                                                \
  extern "C" __global__ __launch_bounds__(WPB * 64) void name(                                                      \
      const unsigned char *__restrict__ a, const float *__restrict__ as, const unsigned char *__restrict__ w,       \
      const float *__restrict__ ws, int *__restrict__ decode_partial, int *__restrict__ decode_counter,             \
      unsigned short *__restrict__ c, const unsigned char *__restrict__ w_b, const float *__restrict__ ws_b,        \
      int *__restrict__ decode_partial_b, int *__restrict__ decode_counter_b, unsigned short *__restrict__ c_b,     \
      int m, int k, int n, int ks, int nb, int n_b, int ks_b, int nb_b) {                                           \
    const int b0 = nb * ks, b1 = nb_b * ks_b, bx = (int)blockIdx.x;                                                 \
    const bool p1 = BFIRST ? bx < b1 : bx >= b0;                                                                    \
    const int bl = BFIRST ? (p1 ? bx : bx - b1) : (p1 ? bx - b0 : bx), nbp = p1 ? nb_b : nb;                        \
    iu8_dec_body<TM, false, NT, KW, WPB, D, ALDS, false>(                                                           \
        a, p1 ? w_b : w, as, p1 ? ws_b : ws, p1 ? decode_partial_b : decode_partial,                                \
        p1 ? decode_counter_b : decode_counter, p1 ? c_b : c, iu8_rows{nullptr, 0, m}, p1 ? n_b : n, k,             \
        iu8_blk{bl % nbp, bl / nbp, p1 ? ks_b : ks});                                                               \
  }
#define IU8_PAIR_VARIANT(name, TM, NT, KW, WPB, D, ALDS, BFIRST) IU8F_PAIR(name, TM, NT, KW, WPB, D, ALDS, BFIRST)
#include "iu8_variants.def"
#undef IU8F_PAIR

// THE DECODE MLP CHAIN: gate+up linear -> SiLU(gate) * up with its per-token requantisation -> down
// linear, one persistent launch for at most 4 rows (iu8_chain.h). `w` / `ws` are the gate and up
// weights as one [2n, k] operand (gate rows first), `w_b` / `ws_b` the down weights [k, n]; `gu`
// (bf16 [m, 2n]) and `p` (bf16 [m, n]) are the launch's working rows; `state` is the 13 KiB block
// the workgroups meet through (zero before the first launch, left zero past its first 8 KiB by a launch
// that completes; the word at 12 KiB non-zero: a wait timed out, c is not valid).
// The grid is the host's: every workgroup resident at once (one a CU: 16 waves), at most 512 of them,
// at most 8 column blocks of either linear a workgroup.
extern "C" __global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4))) void macaq_iu8f_mlp_w4_tm1(
    const unsigned short *__restrict__ x, const unsigned char *__restrict__ w, const float *__restrict__ ws,
    const unsigned char *__restrict__ w_b, const float *__restrict__ ws_b, unsigned short *__restrict__ gu,
    unsigned short *__restrict__ p, unsigned char *__restrict__ state, unsigned short *__restrict__ c, int m, int k, int n,
    int spin) {
  iu8_chain_mlp<1, 8, 16, 4>(x, w, ws, w_b, ws_b, gu, p, state, c, m, k, n, spin);
}
// `_a80`: the same launch with the second linear on the 80 KiB form -- up to 4 rows whose intermediate codes
// (rows rounded up to a power of two) fit 80 KiB: 2 to 4 rows of the benchmark layer's 17,408.
extern "C" __global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4))) void macaq_iu8f_mlp_w4_tm1_a80(
    const unsigned short *__restrict__ x, const unsigned char *__restrict__ w, const float *__restrict__ ws,
    const unsigned char *__restrict__ w_b, const float *__restrict__ ws_b, unsigned short *__restrict__ gu,
    unsigned short *__restrict__ p, unsigned char *__restrict__ state, unsigned short *__restrict__ c, int m, int k, int n,
    int spin) {
  iu8_chain_mlp<1, 8, 16, 4, 80>(x, w, ws, w_b, ws_b, gu, p, state, c, m, k, n, spin);
}

// THE GATE+UP LINEAR OF A DECODE MLP WITH ITS ACTIVATION, 5 to 16 rows: a [m, k] = the rows' int8 codes (one 16-row
// tile, K <= 5120, staged once a workgroup as in macaq_iu8_dec_w4_tm1_s80) x w [2n, k] (gate rows, then up rows) ->
// p bf16 [m, n] = bf16(bf16(silu(gate)) * up), the gate and up tiles of a 16-column block computed side by side by
// the two halves of a workgroup's waves and met in its epilogue; gu (bf16 [m, 2n], may be null) is a tap of
// [gate | up]. The dense twin of the routed layer's moe_iu8_grouped_w4_decpa_*: in place of linear ->
// macaq_i8_silu_mul_quant_* the MLP runs this launch and the plain quantiser on p, which reads half the bytes
// and computes no exp. Grid: the fused forms' (n / 16 column blocks, at most 8 a workgroup), block 1024.
extern "C" __global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4))) void macaq_iu8f_gateup_act_w4_s80(
    const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,
    const float *__restrict__ ws, unsigned short *__restrict__ gu, unsigned short *__restrict__ p, int m, int n, int k) {
  __shared__ iu8_decq_lds<1, 8, 16, 4, 80> lds;
  if (m > 8)
    iu8_decq_body<false, 1, 8, 16, 4, 4, iu8_decq_codes_pair, 80, 4>(lds, (const unsigned short *)a, w, ws, nullptr, nullptr, gu, m, n,
                                                                      k, iu8_decq_codes_pair{as, p, nullptr});
  else
    iu8_decq_body<false, 1, 8, 16, 4, 4, iu8_decq_codes_pair, 80>(lds, (const unsigned short *)a, w, ws, nullptr, nullptr, gu, m, n, k,
                                                                   iu8_decq_codes_pair{as, p, nullptr});
}
