// The W4A8-iu8 GEMMs for gfx950 (CDNA4, wave64, int8 MFMA): the code object `macaq_iu8`.
// It stands in for the reference's gfx1201 object of the same name
// (crates/saber-kernels/hip/macaq_iu8.hip; symbols crates/saber-kernels/src/macaq_iu8.rs:51-62)
// with the same kernel symbols and the same kernarg layouts
// (crates/saber-kernels/src/abi.rs:3349-3372), so the host side that packs kernargs and
// launches by name does not change. Operand orders and the contract: iu8_common.h.
//
// Two regimes, two designs.
//   decode  (M <= 64)  HBM-bound weight streaming. A workgroup owns WN*NT 16-row weight tiles;
//           its KW "k-waves" interleave over 128-deep K steps of the same tiles, each issuing
//           128-bit nontemporal loads of packed int4 (one 1-KiB fragment per wave-load), with the
//           next batch of loads in flight while the current one is unpacked in registers and fed
//           to v_mfma_i32_16x16x64_i8. The split-K partials of the k-waves are reduced through
//           LDS (exact int32); an optional grid-level split (gridDim.z) goes through the
//           `decode_partial` / `decode_counter` workspaces, the last-arriving workgroup summing.
//   prefill (M > 64)   MFMA-bound tile GEMM. A workgroup of WMW x WNW waves owns a
//           (WMW*TM*16) x (WNW*TN*16) output tile; A and W fragments of one 128-deep K step are
//           staged in LDS in fragment order (W4 stays packed; the unpack happens after the LDS
//           read, once per fragment, and is reused across the wave's TM row tiles), with the next
//           step's global loads in flight during the MFMAs.
#include "iu8_common.h"

// ============================================================================ decode band
template <int TM, bool W8, int NT, int KW, int WPB, int U, bool ACC>
__device__ __forceinline__ void iu8_dec_body(const iu8_u8 *__restrict__ A, const iu8_u8 *__restrict__ W,
                                             const float *__restrict__ as, const float *__restrict__ ws,
                                             int *__restrict__ P, int *__restrict__ cnt, void *__restrict__ Cv,
                                             int M, int N, int K) {
  static_assert(WPB % KW == 0, "k-waves divide the workgroup");
  constexpr int WN = WPB / KW;
  constexpr int WSTEP = W8 ? 2048 : 1024;  // bytes of one 16-row weight tile per 128-deep K step
  constexpr int WV = W8 ? 2 : 1;           // 16-byte loads a lane per step per tile
  constexpr int BN = WN * NT * 16;         // columns a workgroup
  __shared__ int s_red[(KW > 1 ? KW - 1 : 1) * WN * TM * NT * 256];
  __shared__ int s_last;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wk = wave % KW, wn = wave / KW;
  const int ntiles = N >> 4, steps = K >> 7, ktiles = K >> 6;
  const int Z = gridDim.z, z = blockIdx.z;
  const int spb = (steps + Z - 1) / Z;
  const int s_lo = z * spb, s_hi = min(steps, s_lo + spb);
  const int nt0 = (blockIdx.x * WN + wn) * NT;

  const iu8_u8 *wp[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int ntj = min(nt0 + j, ntiles - 1);  // a tile past N re-reads the last one and stores nothing
    wp[j] = W + (size_t)ntj * steps * WSTEP + lane * 16;
  }
  bool live[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) live[i] = i * 16 + (lane & 15) < M;
  const iu8_u8 *ap = A + lane * 16;

  iu8_v4i acc[TM][NT];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = iu8_v4i{0, 0, 0, 0};

  struct Batch {
    iu8_v4u w[U][NT][WV];
    iu8_v4i a[U][TM][2];
  };
  auto load = [&](Batch &b, int s) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int su = s + u * KW;
      if (su < s_hi) {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int v = 0; v < WV; ++v) b.w[u][j][v] = iu8_ldg_nt(wp[j] + (size_t)su * WSTEP + v * 1024);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            b.a[u][i][h] = iu8_v4i{0, 0, 0, 0};
            if (live[i]) b.a[u][i][h] = *(const iu8_v4i *)(ap + ((size_t)i * ktiles + 2 * su + h) * 1024);
          }
      } else {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int v = 0; v < WV; ++v) b.w[u][j][v] = iu8_v4u{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int h = 0; h < 2; ++h) b.a[u][i][h] = iu8_v4i{0, 0, 0, 0};
      }
    }
  };
  auto compute = [&](const Batch &b) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        iu8_v4i w0, w1;
        if constexpr (W8) {
          w0 = (iu8_v4i)b.w[u][j][0];
          w1 = (iu8_v4i)b.w[u][j][WV - 1];
        } else {
          iu8_unpack_w4(b.w[u][j][0], w0, w1);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          acc[i][j] = iu8_mfma(w0, b.a[u][i][0], acc[i][j]);
          acc[i][j] = iu8_mfma(w1, b.a[u][i][1], acc[i][j]);
        }
      }
  };

  {
    int s = s_lo + wk;
    if (s < s_hi) {
      Batch b0;
      load(b0, s);
      for (; s < s_hi; s += KW * U) {
        Batch b1;
        load(b1, s + KW * U);  // past the end: zeros, no memory touched
        compute(b0);
        b0 = b1;
      }
    }
  }

  // ---- the k-waves' partials meet in LDS (exact int32 adds)
  if constexpr (KW > 1) {
    if (wk > 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
          *(iu8_v4i *)&s_red[((((wk - 1) * WN + wn) * TM + i) * NT + j) * 256 + lane * 4] = acc[i][j];
    }
    __syncthreads();
    if (wk == 0) {
#pragma unroll
      for (int q = 0; q < KW - 1; ++q)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j)
            acc[i][j] += *(const iu8_v4i *)&s_red[(((q * WN + wn) * TM + i) * NT + j) * 256 + lane * 4];
    }
  }

  const int ml = lane & 15, nq = (lane >> 4) * 4;
  if (Z == 1) {
    if (wk != 0) return;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      if (nt0 + j >= ntiles) continue;
      const int n = (nt0 + j) * 16 + nq;
      float wsu[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) wsu[r] = iu8_wsu<W8>(ws, n + r);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = i * 16 + ml;
        if (m >= M) continue;
        if constexpr (ACC) {
          *(iu8_v4i *)((int *)Cv + (size_t)m * N + n) = acc[i][j];
        } else {
          const float am = as[m];
          unsigned h[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) h[r] = iu8_bf16_bits(iu8_epi(acc[i][j][r], am, wsu[r]));
          *(iu8_v2u *)((unsigned short *)Cv + (size_t)m * N + n) = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        }
      }
    }
    return;
  }

  // ---- grid-level split: partials to `decode_partial`, the last-arriving workgroup of this
  // column block sums them and runs the epilogue; the counter is left at zero.
  if (wk == 0) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      if (nt0 + j >= ntiles) continue;
      const int n = (nt0 + j) * 16 + nq;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = i * 16 + ml;
        if (m < M) *(iu8_v4i *)&P[((size_t)z * M + m) * N + n] = acc[i][j];
      }
    }
  }
  __syncthreads();
  if (tid == 0) {
    __threadfence();
    s_last = (atomicAdd(&cnt[blockIdx.x], 1) == Z - 1);
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  if (tid == 0) cnt[blockIdx.x] = 0;
  const int nb = blockIdx.x * BN, nw4 = min(BN, N - nb) >> 2;
  for (int idx = tid; idx < nw4 * M; idx += WPB * 64) {
    const int m = idx / nw4, n = nb + (idx % nw4) * 4;
    iu8_v4i sum = iu8_v4i{0, 0, 0, 0};
    for (int q = 0; q < Z; ++q) sum += __builtin_nontemporal_load((const iu8_v4i *)&P[((size_t)q * M + m) * N + n]);
    if constexpr (ACC) {
      *(iu8_v4i *)((int *)Cv + (size_t)m * N + n) = sum;
    } else {
      const float am = as[m];
      unsigned h[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) h[r] = iu8_bf16_bits(iu8_epi(sum[r], am, iu8_wsu<W8>(ws, n + r)));
      *(iu8_v2u *)((unsigned short *)Cv + (size_t)m * N + n) = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
    }
  }
}

#define IU8_DEC(name, TM, W8, NT, KW, WPB, U, ACC)                                                               \
  extern "C" __global__ __launch_bounds__(WPB * 64) void name(                                                    \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, int *__restrict__ decode_partial, int *__restrict__ decode_counter,           \
      unsigned short *__restrict__ c, int m, int n, int k) {                                                       \
    iu8_dec_body<TM, W8, NT, KW, WPB, U, ACC>(a, w, as, ws, decode_partial, decode_counter, c, m, n, k);           \
  }

#define IU8_DEC_VARIANT(name, TM, W8, NT, KW, WPB, U, ACC) IU8_DEC(name, TM, W8, NT, KW, WPB, U, ACC)
#define IU8_PF_VARIANT(name, W8, WMW, WNW, TM, TN, ACC)
#include "iu8_variants.def"
#undef IU8_DEC_VARIANT
#undef IU8_PF_VARIANT
#undef IU8_DEC

// ============================================================================ prefill tile
template <bool W8, int WMW, int WNW, int TM, int TN, bool ACC>
__device__ __forceinline__ void iu8_pf_body(const iu8_u8 *__restrict__ A, const iu8_u8 *__restrict__ W,
                                            const float *__restrict__ as, const float *__restrict__ ws,
                                            void *__restrict__ Cv, int M, int N, int K) {
  constexpr int NTHR = WMW * WNW * 64;
  constexpr int BMT = WMW * TM, BNT = WNW * TN;  // 16-row tiles a workgroup, both ways
  constexpr int WSTEP = W8 ? 2048 : 1024;
  constexpr int A_PIECES = BMT * 128, W_PIECES = BNT * (WSTEP / 16);  // 16-byte pieces a K step
  constexpr int A_PER = (A_PIECES + NTHR - 1) / NTHR, W_PER = (W_PIECES + NTHR - 1) / NTHR;
  __shared__ __attribute__((aligned(16))) iu8_u8 sA[BMT * 2048];
  __shared__ __attribute__((aligned(16))) iu8_u8 sW[BNT * WSTEP];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WNW, wn = wave % WNW;
  const int mtiles = (M + 15) >> 4, ntiles = N >> 4, steps = K >> 7, ktiles = K >> 6;
  const int mt0 = blockIdx.y * BMT, nt0 = blockIdx.x * BNT;

  // the global side of every piece this thread stages (tiles past the edge re-read the last one)
  const iu8_u8 *ga[A_PER];
  const iu8_u8 *gw[W_PER];
#pragma unroll
  for (int p = 0; p < A_PER; ++p) {
    const int piece = p * NTHR + tid;
    const int mt = min(mt0 + piece / 128, mtiles - 1);
    ga[p] = A + (size_t)mt * ktiles * 1024 + (piece % 128) * 16;
  }
#pragma unroll
  for (int p = 0; p < W_PER; ++p) {
    const int piece = p * NTHR + tid;
    const int nt = min(nt0 + piece / (WSTEP / 16), ntiles - 1);
    gw[p] = W + (size_t)nt * steps * WSTEP + (piece % (WSTEP / 16)) * 16;
  }

  iu8_v4i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = iu8_v4i{0, 0, 0, 0};

  iu8_v4u ra[A_PER], rw[W_PER];
  auto gload = [&](int s) {
#pragma unroll
    for (int p = 0; p < A_PER; ++p)
      if (A_PIECES % NTHR == 0 || p * NTHR + tid < A_PIECES) ra[p] = *(const iu8_v4u *)(ga[p] + (size_t)s * 2048);
#pragma unroll
    for (int p = 0; p < W_PER; ++p)
      if (W_PIECES % NTHR == 0 || p * NTHR + tid < W_PIECES) rw[p] = iu8_ldg_nt(gw[p] + (size_t)s * WSTEP);
  };
  gload(0);
  for (int s = 0; s < steps; ++s) {
    __syncthreads();  // every wave is done reading the previous step's fragments
#pragma unroll
    for (int p = 0; p < A_PER; ++p)
      if (A_PIECES % NTHR == 0 || p * NTHR + tid < A_PIECES) *(iu8_v4u *)&sA[(p * NTHR + tid) * 16] = ra[p];
#pragma unroll
    for (int p = 0; p < W_PER; ++p)
      if (W_PIECES % NTHR == 0 || p * NTHR + tid < W_PIECES) *(iu8_v4u *)&sW[(p * NTHR + tid) * 16] = rw[p];
    __syncthreads();
    if (s + 1 < steps) gload(s + 1);

    iu8_v4i wf[TN][2];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if constexpr (W8) {
        wf[j][0] = *(const iu8_v4i *)&sW[((wn * TN + j) * 2 + 0) * 1024 + lane * 16];
        wf[j][1] = *(const iu8_v4i *)&sW[((wn * TN + j) * 2 + 1) * 1024 + lane * 16];
      } else {
        iu8_unpack_w4(*(const iu8_v4u *)&sW[(wn * TN + j) * 1024 + lane * 16], wf[j][0], wf[j][1]);
      }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const iu8_v4i af = *(const iu8_v4i *)&sA[((wm * TM + i) * 2 + h) * 1024 + lane * 16];
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = iu8_mfma(wf[j][h], af, acc[i][j]);
      }
  }

  const int ml = lane & 15, nq = (lane >> 4) * 4;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int nt = nt0 + wn * TN + j;
    if (nt >= ntiles) continue;
    const int n = nt * 16 + nq;
    float wsu[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) wsu[r] = iu8_wsu<W8>(ws, n + r);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = (mt0 + wm * TM + i) * 16 + ml;
      if (m >= M) continue;
      if constexpr (ACC) {
        *(iu8_v4i *)((int *)Cv + (size_t)m * N + n) = acc[i][j];
      } else {
        const float am = as[m];
        unsigned h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) h[r] = iu8_bf16_bits(iu8_epi(acc[i][j][r], am, wsu[r]));
        *(iu8_v2u *)((unsigned short *)Cv + (size_t)m * N + n) = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
      }
    }
  }
}

#define IU8_PF(name, W8, WMW, WNW, TM, TN, ACC)                                                                  \
  extern "C" __global__ __launch_bounds__(WMW * WNW * 64) void name(                                              \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, unsigned short *__restrict__ c, int m, int n, int k) {                         \
    iu8_pf_body<W8, WMW, WNW, TM, TN, ACC>(a, w, as, ws, c, m, n, k);                                              \
  }
#define IU8_DEC_VARIANT(name, TM, W8, NT, KW, WPB, U, ACC)
#define IU8_PF_VARIANT(name, W8, WMW, WNW, TM, TN, ACC) IU8_PF(name, W8, WMW, WNW, TM, TN, ACC)
#include "iu8_variants.def"
#undef IU8_DEC_VARIANT
#undef IU8_PF_VARIANT
#undef IU8_PF
