// The W4A8-iu8 GEMMs for gfx950 (CDNA4, wave64, int8 MFMA): the code object `macaq_iu8`.
// It stands in for the reference's gfx1201 object of the same name
// (crates/saber-kernels/hip/macaq_iu8.hip; symbols crates/saber-kernels/src/macaq_iu8.rs:51-62)
// with the same kernel symbols and the same kernarg layouts
// (crates/saber-kernels/src/abi.rs:3349-3372), so the host side that packs kernargs and
// launches by name does not change. Operand orders and the contract: iu8_common.h.
//
// Two regimes, two designs.
//   decode  (M <= 64)  HBM-bound weight streaming. A workgroup owns WN*NT 16-row weight tiles;
//           its KW "k-waves" interleave over 128-deep K steps of the same tiles. Every wave keeps
//           a ring of D steps of 128-bit nontemporal loads of packed int4 in flight (one 1-KiB
//           fragment per wave-load): a step is consumed (nibble unpack in registers,
//           v_mfma_i32_16x16x64_i8) and its ring slot re-issued D steps ahead. For M <= 16 the
//           workgroup's activation rows are staged once in LDS (only the live rows, behind the
//           first ring of weight loads); lanes of dead rows read row 0, which is harmless: a
//           row of A only reaches its own row of C, and dead rows are never stored. The k-waves'
//           partials are reduced through LDS (exact int32). An optional grid-level split
//           (gridDim.z) goes through the `decode_partial` / `decode_counter` workspaces with the
//           last-arriving workgroup summing; it costs device-scope fences across the 8 XCDs' L2s
//           and the launch law does not use it by default.
//   prefill (M > 64)   MFMA-bound tile GEMM. A workgroup of WMW x WNW waves owns a
//           (WMW*TM*16) x (WNW*TN*16) output tile; A and W fragments of one 128-deep K step are
//           staged in LDS in fragment order (W4 stays packed; the unpack happens after the LDS
//           read, once per fragment, and is reused across the wave's TM row tiles), with the next
//           step's global loads in flight during the MFMAs.
#include "iu8_gemm.h"

#define IU8_DEC(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)                                                         \
  extern "C" __global__ __launch_bounds__(WPB * 64) void name(                                                    \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, int *__restrict__ decode_partial, int *__restrict__ decode_counter,           \
      unsigned short *__restrict__ c, int m, int n, int k) {                                                       \
    iu8_dec_body<TM, W8, NT, KW, WPB, D, ALDS, ACC>(a, w, as, ws, decode_partial, decode_counter, c,          \
                                                    iu8_rows{nullptr, 0, m}, n, k);     \
  }
#define IU8_DEC_VARIANT(name, TM, W8, NT, KW, WPB, D, ALDS, ACC) IU8_DEC(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)
#define IU8_PF_VARIANT(name, W8, WMW, WNW, TM, TN, ACC)
#include "iu8_variants.def"
#undef IU8_DEC_VARIANT
#undef IU8_PF_VARIANT
#undef IU8_DEC

#define IU8_PF(name, W8, WMW, WNW, TM, TN, ACC)                                                                  \
  extern "C" __global__ __launch_bounds__(WMW * WNW * 64) void name(                                              \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, unsigned short *__restrict__ c, int m, int n, int k) {                         \
    iu8_pf_body<W8, WMW, WNW, TM, TN, ACC>(a, w, as, ws, c, iu8_rows{nullptr, 0, m},                            \
                                           (int)blockIdx.y * (WMW * TM * 16), n, k);                                              \
  }
#define IU8_DEC_VARIANT(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)
#define IU8_PF_VARIANT(name, W8, WMW, WNW, TM, TN, ACC) IU8_PF(name, W8, WMW, WNW, TM, TN, ACC)
#include "iu8_variants.def"
#undef IU8_DEC_VARIANT
#undef IU8_PF_VARIANT
#undef IU8_PF
