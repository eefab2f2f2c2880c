// The kernel definitions of the dense W4A8-iu8 GEMMs, as macros over the bodies in iu8_gemm.h and
// iu8_pf32.h: one place for the argument lists (crates/saber-kernels/src/abi.rs:3349-3372) shared by
// the product object `macaq_iu8` and the parity suite's accumulator taps (`iu8_taps`).
#pragma once
#include "iu8_gemm.h"
#include "iu8_pf32.h"

#define IU8_DEC(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)                                                         \
  extern "C" __global__ __launch_bounds__(WPB * 64) void name(                                                    \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, int *__restrict__ decode_partial, int *__restrict__ decode_counter,           \
      unsigned short *__restrict__ c, int m, int n, int k) {                                                       \
    iu8_dec_body<TM, W8, NT, KW, WPB, D, ALDS, ACC>(a, w, as, ws, decode_partial, decode_counter, c,          \
                                                    iu8_rows{nullptr, 0, m}, n, k);     \
  }

// Persistent launch: gridDim.x workgroups (one or OCC a CU) walk the tiles of the m x n output.
//
// The 256 x 256 cell's last round. With G workgroups and q * G + rem tiles, the last round keeps rem
// workgroups busy and the others idle for a whole tile (a fifth of the launch at 1,088 tiles on 256
// workgroups). When rem <= G / 2 those rem tiles are cut into quarters and run on the 128 x 128 cell
// instead: 4 * rem quarter tiles over all G workgroups take 0.42 (one round) or 0.84 (two) of a big
// tile's time. Same bytes: every output element is one exact integer sum and one epilogue, whichever
// cell computes it.
#define IU8_PF32(name, W8, WMW, WNW, TM, TN, ACC, ST, OCC, DEEP)                                                        \
  extern "C" __global__ __launch_bounds__(WMW * WNW * 64)                                                         \
      __attribute__((amdgpu_waves_per_eu(WMW * WNW * OCC / 4, WMW * WNW * OCC / 4))) void name(                    \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, unsigned short *__restrict__ c, int m, int n, int k) {                         \
    constexpr int BM = WMW * TM * 32, BN = WNW * TN * 32;                                                          \
    constexpr bool TAIL = WMW == 2 && WNW == 4 && TM == 4 && TN == 2 && !ACC && !DEEP;                             \
    const int gx = (n + BN - 1) / BN, gy = (m + BM - 1) / BM;                                                      \
    const iu8_rows R{nullptr, 0, m};                                                                               \
    if constexpr (TAIL) {                                                                                          \
      constexpr int LB = iu8_pf32_lds_bytes<W8, WMW, WNW, TM, TN, ST>(), LS = iu8_pf32_lds_bytes<W8, 4, 2, 1, 2, 3>(); \
      __shared__ __attribute__((aligned(1024))) iu8_u8 lds[LB > LS ? LB : LS];                                     \
      const int G = gridDim.x, total = gx * gy, q = total / G, rem = total - q * G;                                \
      const bool tail = q >= 1 && rem > 0 && 2 * rem <= G;                                                         \
      iu8_pf32_run<W8, WMW, WNW, TM, TN, ACC, ST, DEEP, false, false, true>(                                       \
          a, as, c, n, k,                                                                                          \
          [&](int r, iu8_tile &t) {                                                                                \
            int bx, by;                                                                                            \
            if ((tail && r >= q) || !iu8_dense_tile_at(r, gx, gy, bx, by)) return false;                           \
            t = iu8_tile{R, by * BM, bx * (BN / 16), w, ws, by * gx + bx};                                         \
            return true;                                                                                           \
          },                                                                                                       \
          nullptr, nullptr, lds);                                                                                  \
      if (tail) {                                                                                                  \
        __syncthreads();                                                                                           \
        iu8_pf32_run<W8, 4, 2, 1, 2, ACC, 3, false, false, false, true>(                                           \
            a, as, c, n, k,                                                                                        \
            [&](int r, iu8_tile &t) {                                                                              \
              const int j = (int)blockIdx.x + r * G;                                                               \
              if (j >= 4 * rem) return false;                                                                      \
              int bx, by;                                                                                          \
              iu8_dense_tile_of(q * G + (j >> 2), gx, gy, bx, by);                                                 \
              t = iu8_tile{R, by * BM + ((j >> 1) & 1) * 128, (bx * BN + (j & 1) * 128) / 16, w, ws, 0};           \
              return true;                                                                                         \
            },                                                                                                     \
            nullptr, nullptr, lds);                                                                                \
      }                                                                                                            \
    } else {                                                                                                       \
      iu8_pf32_run<W8, WMW, WNW, TM, TN, ACC, ST, DEEP>(a, as, c, n, k, [&](int r, iu8_tile &t) {                  \
        int bx, by;                                                                                                \
        if (!iu8_dense_tile_at(r, gx, gy, bx, by)) return false;                                                   \
        t = iu8_tile{R, by * BM, bx * (BN / 16), w, ws, by * gx + bx};                                             \
        return true;                                                                                               \
      });                                                                                                          \
    }                                                                                                              \
  }
