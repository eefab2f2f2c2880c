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
//           last-arriving workgroup summing (partials handed over straight through memory, no
//           cache flush); the launch law does not use it by default.
//   prefill (M > 64)   MFMA-bound tile GEMM on v_mfma_i32_32x32x32_i8 (iu8_pf32.h): persistent
//           workgroups of 8 waves (two a SIMD) walk an XCD-aware tile order; the fragments of a
//           128-deep K step go from HBM/L2 into one of three LDS stages by LDS-DMA loads, two steps
//           ahead of the MFMAs and across tile boundaries; W4 stays packed in LDS and is unpacked
//           in registers just in time; the output tile goes out through LDS as whole row segments.
#include "iu8_gemm.h"
#include "iu8_decq.h"
#include "iu8_decq1.h"
#include "iu8_pf32.h"
#include "iu8_dense_defs.h"

#define IU8_DEC_VARIANT(name, TM, W8, NT, KW, WPB, D, ALDS, ACC) IU8_DEC(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)
#include "iu8_variants.def"

// The decode linear with the per-token quantisation fused into the activation staging (M <= 4 rows
// that fit the staged form): x is the bf16 activation matrix; `q` / `scale` (optional, may be null)
// receive the int8 codes in A fragment order and the row scales, written by workgroup 0. One launch
// instead of producer + GEMM; the bytes of c, q and scale are those of the two-launch path. The
// reference fuses producers the other way round (norm/activation + quant in front of an int8 GEMM,
// crates/saber-kernels/hip/mxfp4_hadi8.hip); this is the same law inside the GEMV's prologue, where
// it hides behind the first weight loads.
// Geometry: 16 waves a workgroup (one workgroup a CU, 4 waves a SIMD) as 8 k-waves x 2 column tiles, a
// ring of 4 steps a wave. Measured against 8 waves (4 k-waves x 2 tiles, two workgroups a CU) with a ring
// of 8 -- the same bytes in flight a CU: QKV 5.99 -> 5.56 us, O 5.57 -> 5.20, gate+up 16.4 -> 15.8, down
// 12.8 -> 10.7 at one row: the rows' quantisation, which every workgroup repeats in front of its first
// MFMA, is spread over twice the lanes, and a CU's waves all see one set of staged codes. Ring depths
// 2/3/5/6 and 16 k-waves on 16-column blocks measured slower on every shape.
// `_a80`: the same launch for up to 16 rows whose codes (rows rounded up to a power of two) fit 80 KiB of
// LDS -- 16 rows of K = 5120, 4 rows of K = 17408 -- in place of a producer launch + GEMV.
#define IU8_DECQX(name, W8, NT, KW, WPB, D) IU8_DECQA(name, W8, NT, KW, WPB, D, 20)
#define IU8_DECQA(name, W8, NT, KW, WPB, D, AKB)                                                                       \
  extern "C" __global__ __launch_bounds__(WPB * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void name(              \
      const unsigned short *__restrict__ x, const unsigned char *__restrict__ w, const float *__restrict__ ws,     \
      unsigned char *__restrict__ q, float *__restrict__ scale, unsigned short *__restrict__ c, int m, int n,      \
      int k) {                                                                                                     \
    __shared__ iu8_decq_lds<NT, KW, WPB, 0, AKB> lds;                                                              \
    iu8_decq_body<W8, NT, KW, WPB, D, 0, iu8_decq_nohook, AKB>(lds, x, w, ws, q, scale, c, m, n, k);               \
  }
IU8_DECQX(macaq_iu8_decq_w4_tm1, false, 1, 8, 16, 4)
IU8_DECQX(macaq_iu8_decq_w8_tm1, true, 1, 8, 16, 2)
IU8_DECQA(macaq_iu8_decq_w4_tm1_a80, false, 1, 8, 16, 4, 80)
IU8_DECQA(macaq_iu8_decq_w8_tm1_a80, true, 1, 8, 16, 2, 80)
#undef IU8_DECQX
#undef IU8_DECQA

// The GEMV of up to 16 quantised rows whose 16-row tile fits 80 KiB of LDS (K <= 5120), persistent like the
// fused forms: a workgroup copies the tile into LDS once and streams its column blocks against it. The
// streamed form (`_a0`) reads the tile from L2 once a 32-column block -- at 16 rows of K = 5120 as many bytes
// through L2 as the weights bring from memory. `_s80r`: the same for fewer live rows of a longer K (the rows
// rounded up to a power of two x K <= 80 KiB: 4 rows of 20,480), whose copy takes the live rows' pieces of the
// tile; a kernel of its own because the row shift is then a register in every LDS index of the K loop, which
// costs the whole-tile launches 0.1-0.4 us.
#define IU8_DECS(name, W8, NT, KW, WPB, D, MRS)                                                                    \
  extern "C" __global__ __launch_bounds__(WPB * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void name(          \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, int *__restrict__ decode_partial, int *__restrict__ decode_counter,           \
      unsigned short *__restrict__ c, int m, int n, int k) {                                                       \
    __shared__ iu8_decq_lds<NT, KW, WPB, 3, 80> lds;                                                               \
    iu8_decq_body<W8, NT, KW, WPB, D, 3, iu8_decq_codes, 80, MRS>(lds, (const unsigned short *)a, w, ws, nullptr, nullptr, c, m, n, \
                                                                  k, iu8_decq_codes{as});                          \
  }
IU8_DECS(macaq_iu8_dec_w4_tm1_s80, false, 1, 8, 16, 4, 4)
IU8_DECS(macaq_iu8_dec_w8_tm1_s80, true, 1, 8, 16, 2, 4)
IU8_DECS(macaq_iu8_dec_w4_tm1_s80r, false, 1, 8, 16, 4, -1)
IU8_DECS(macaq_iu8_dec_w8_tm1_s80r, true, 1, 8, 16, 2, -1)
#undef IU8_DECS

// One row (`_r1`, the GEMV of a single token): the same launch with the row's codes made just in time --
// a wave converts only the K steps it multiplies, a chunk of 4 steps ahead of their use, inside the weight
// stream (iu8_decq1.h). In front of the first MFMA stand the row's arrival, one meeting of the waves'
// maxima and one chunk's conversion instead of the whole row's conversion behind two barriers.
#define IU8_DECQ1(name, W8, KW, WPB, D)                                                                            \
  extern "C" __global__ __launch_bounds__(WPB * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void name(          \
      const unsigned short *__restrict__ x, const unsigned char *__restrict__ w, const float *__restrict__ ws,     \
      unsigned char *__restrict__ q, float *__restrict__ scale, unsigned short *__restrict__ c, int m, int n,      \
      int k) {                                                                                                     \
    iu8_decq1_body<W8, KW, WPB, D>(x, w, ws, q, scale, c, n, k);                                                   \
  }
IU8_DECQ1(macaq_iu8_decq_w4_r1, false, 8, 16, 4)
IU8_DECQ1(macaq_iu8_decq_w8_r1, true, 8, 16, 2)
#undef IU8_DECQ1

// Cells with K split over gridDim.z (symbol suffix `_ks`, the decode kernarg list: the two workspaces
// in front of c), for the rows between the regimes, where few tiles leave CUs idle. Measured, the
// partials' way through memory (ks * M * N * 4 bytes out and back) costs more than the idle CUs on
// every shape but deep, narrow linears at 49-128 rows, the one band where the launch law picks a
// split form (the 64 x 128 cell); the others are kept, tested and reachable by name like the decode split.
#define IU8_PF32K(name, W8, WMW, WNW, TM, TN, ST, OCC, DEEP)                                                       \
  extern "C" __global__ __launch_bounds__(WMW * WNW * 64)                                                         \
      __attribute__((amdgpu_waves_per_eu(WMW * WNW * OCC / 4, WMW * WNW * OCC / 4))) void name(                    \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, int *__restrict__ decode_partial, int *__restrict__ decode_counter,           \
      unsigned short *__restrict__ c, int m, int n, int k) {                                                       \
    constexpr int BM = WMW * TM * 32, BN = WNW * TN * 32;                                                          \
    const int gx = (n + BN - 1) / BN, gy = (m + BM - 1) / BM;                                                      \
    const iu8_rows R{nullptr, 0, m};                                                                               \
    iu8_pf32_run<W8, WMW, WNW, TM, TN, false, ST, DEEP>(                                                           \
        a, as, c, n, k,                                                                                            \
        [&](int r, iu8_tile &t) {                                                                                  \
          int bx, by;                                                                                              \
          if (!iu8_dense_tile_at(r, gx, gy, bx, by)) return false;                                                 \
          t = iu8_tile{R, by * BM, bx * (BN / 16), w, ws, by * gx + bx};                                           \
          return true;                                                                                             \
        },                                                                                                         \
        gridDim.z > 1 ? decode_partial : nullptr, decode_counter);                                                 \
  }
IU8_PF32K(macaq_iu8_pf_w4_t128x128_ks, false, 4, 2, 1, 2, 3, 1, false)
IU8_PF32K(macaq_iu8_pf_w8_t128x128_ks, true, 4, 2, 1, 2, 3, 1, false)
IU8_PF32K(macaq_iu8_pf_w4_t256x160_ks, false, 8, 1, 1, 5, 3, 1, false)
IU8_PF32K(macaq_iu8_pf_w8_t256x160_ks, true, 8, 1, 1, 5, 3, 1, false)
IU8_PF32K(macaq_iu8_pf_w4_t64x128_s_ks, false, 2, 2, 1, 2, 5, 2, true)
#undef IU8_PF32K
#define IU8_PF_VARIANT(name, W8, WMW, WNW, TM, TN, ACC, ST, OCC, DEEP) IU8_PF32(name, W8, WMW, WNW, TM, TN, ACC, ST, OCC, DEEP)
#include "iu8_variants.def"

// The tile GEMM with the per-token quantisation fused into its A-tile load (symbols `macaq_iu8_pfq_*`,
// the cell named by the suffix): `x` is the bf16 activation matrix [m, k] itself, `as` the rows' scales
// (macaq_i8_rowscale_*, or carried from the producer of the rows); the codes are made on the way into
// the A stage by the routine the producer kernel uses, so c holds the bytes of producer + GEMM. No
// counterpart among the reference's symbols: its prefill reads codes a producer stored
// (crates/saber-kernels/hip/macaq_iu8.hip:174-280). The conversion is VALU work that shares the
// CU with the MFMAs -- about 11 * BM wave instructions a step against BM * BN / 32 MFMA cycles a SIMD --
// and measured on this card the fused cells take 2.3-3.1x the time of their plain twins (1.8-3.8x of
// producer + the law's GEMM over the four 27B-class shapes at 256, 2048 and 8192 rows), so the launch law
// does not pick them: they are kept, tested and reachable by name. The 256 x 256 cell has no registers
// left for the pieces in flight (it spilt, and still was the least slow at 2.05-2.3x), so it has no
// fused form here.
#define IU8_PFQ(name, W8, WMW, WNW, TM, TN, ST, OCC)                                                               \
  extern "C" __global__ __launch_bounds__(WMW * WNW * 64)                                                         \
      __attribute__((amdgpu_waves_per_eu(WMW * WNW * OCC / 4, WMW * WNW * OCC / 4))) void name(                    \
      const unsigned short *__restrict__ x, const unsigned char *__restrict__ w, const float *__restrict__ as,    \
      const float *__restrict__ ws, unsigned short *__restrict__ c, int m, int n, int k) {                         \
    constexpr int BM = WMW * TM * 32, BN = WNW * TN * 32;                                                          \
    const int gx = (n + BN - 1) / BN, gy = (m + BM - 1) / BM;                                                      \
    const iu8_rows R{nullptr, 0, m};                                                                               \
    iu8_pf32_run<W8, WMW, WNW, TM, TN, false, ST, false, false, false, false, true>(                               \
        (const iu8_u8 *)x, as, c, n, k, [&](int r, iu8_tile &t) {                                                  \
          int bx, by;                                                                                              \
          if (!iu8_dense_tile_at(r, gx, gy, bx, by)) return false;                                                 \
          t = iu8_tile{R, by * BM, bx * (BN / 16), w, ws, by * gx + bx};                                           \
          return true;                                                                                             \
        });                                                                                                        \
  }
IU8_PFQ(macaq_iu8_pfq_w4_t128x128, false, 4, 2, 1, 2, 3, 1)
IU8_PFQ(macaq_iu8_pfq_w8_t128x128, true, 4, 2, 1, 2, 3, 1)
IU8_PFQ(macaq_iu8_pfq_w4_t128x128_o2, false, 2, 2, 2, 2, 3, 2)
IU8_PFQ(macaq_iu8_pfq_w4_t256x160, false, 8, 1, 1, 5, 3, 1)
IU8_PFQ(macaq_iu8_pfq_w8_t256x160, true, 8, 1, 1, 5, 3, 1)
#undef IU8_PFQ
