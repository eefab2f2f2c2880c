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
#include "iu8_common.h"

// ============================================================================ decode band
template <int TM, bool W8, int NT, int KW, int WPB, int D, int ALDS, bool ACC>
__device__ __forceinline__ void iu8_dec_body(const iu8_u8 *__restrict__ A, const iu8_u8 *__restrict__ W,
                                             const float *__restrict__ as, const float *__restrict__ ws,
                                             int *__restrict__ P, int *__restrict__ cnt, void *__restrict__ Cv,
                                             int M, int N, int K) {
  static_assert(WPB % KW == 0, "k-waves divide the workgroup");
  static_assert(ALDS == 0 || TM == 1, "LDS staging of A is the M <= 16 form");
  constexpr int WN = WPB / KW;
  constexpr int NTHR = WPB * 64;
  constexpr int WSTEP = W8 ? 2048 : 1024;  // bytes of one 16-row weight tile per 128-deep K step
  constexpr int WV = W8 ? 2 : 1;           // 16-byte loads a lane per step per tile
  constexpr int BN = WN * NT * 16;         // columns a workgroup
  constexpr int RED = (KW > 1 ? KW - 1 : 1) * WN * TM * NT * 1024;
  constexpr int ABYTES = ALDS * 1024;
  // one LDS block: the staged activation rows, re-used for the k-waves' partials at the end
  __shared__ __attribute__((aligned(16))) iu8_u8 s_mem[ABYTES > RED ? ABYTES : RED];
  __shared__ int s_last;
  int *s_red = (int *)s_mem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wk = wave % KW, wn = wave / KW;
  const int ntiles = N >> 4, steps = K >> 7, ktiles = K >> 6;
  const int Z = gridDim.z, z = blockIdx.z;
  const int spb = (steps + Z - 1) / Z;
  const int s_lo = z * spb, s_hi = min(steps, s_lo + spb);
  const int nt0 = (blockIdx.x * WN + wn) * NT;
  const int ml = lane & 15, lg = lane >> 4;
  // this wave's steps: s_lo + wk + t*KW, t in [0, T)
  const int T = s_lo + wk < s_hi ? (s_hi - s_lo - wk + KW - 1) / KW : 0;

  const iu8_u8 *wp[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int ntj = min(nt0 + j, ntiles - 1);  // a tile past N re-reads the last one and stores nothing
    wp[j] = W + ((size_t)ntj * steps + s_lo + wk) * WSTEP + lane * 16;
  }

  iu8_v4i acc[TM][NT];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = iu8_v4i{0, 0, 0, 0};

  // ---- LDS staging of the live activation rows (issued before the weight ring, waited after it)
  // MR = staged rows (a power of two >= M); piece p = ((kt*4 + g)*MR + r) holds row r's 16 bytes
  // of k = (2*s_lo + kt)*64 + g*16.
  bool staged = false;
  int mr_shift = 0;
  constexpr int A_PER = ALDS ? (ABYTES / 16 + NTHR - 1) / NTHR : 1;
  constexpr bool A_INREG = A_PER <= 8;
  iu8_v4u areg[A_INREG ? A_PER : 1];
  int a_pieces = 0;
  if constexpr (ALDS > 0) {
    while ((1 << mr_shift) < M) ++mr_shift;
    a_pieces = ((s_hi - s_lo) * 2 * 4) << mr_shift;
    staged = M <= 16 && a_pieces * 16 <= ABYTES;
    if (staged) {
      auto a_src = [&](int piece) {
        const int r = piece & ((1 << mr_shift) - 1), g = (piece >> mr_shift) & 3, kt = piece >> (mr_shift + 2);
        return (const iu8_v4u *)(A + ((size_t)(2 * s_lo + kt) * 1024 + (r + 16 * g) * 16));
      };
      if constexpr (A_INREG) {  // few pieces a thread: loads now, LDS stores behind the first weight ring
#pragma unroll
        for (int p = 0; p < A_PER; ++p)
          if (p * NTHR + tid < a_pieces) areg[p] = *a_src(p * NTHR + tid);
      } else {                  // many: copy before the ring starts
        for (int piece = tid; piece < a_pieces; piece += NTHR) *(iu8_v4u *)&s_mem[piece * 16] = *a_src(piece);
      }
    }
  }

  // ---- the weight ring
  iu8_v4u ring[D][NT][WV];
  iu8_v4i ringa[ALDS ? 1 : D][TM][2];  // direct-from-L2 activation operands when not staged
  bool live[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) live[i] = i * 16 + ml < M;
  const iu8_u8 *ap = A + (size_t)(s_lo + wk) * 2048 + lane * 16;
  auto issue = [&](int slot, int t) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int v = 0; v < WV; ++v) ring[slot][j][v] = iu8_ldg_nt(wp[j] + (size_t)t * (KW * WSTEP) + v * 1024);
    if (!staged) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          ringa[ALDS ? 0 : slot][i][h] = iu8_v4i{0, 0, 0, 0};
          if (live[i])
            ringa[ALDS ? 0 : slot][i][h] =
                *(const iu8_v4i *)(ap + ((size_t)i * ktiles + (size_t)t * (2 * KW) + h) * 1024);
        }
    }
  };
  const int a_lane = (((lg << mr_shift) + min(ml, (1 << mr_shift) - 1)) << 4);
  auto consume = [&](int slot, int t) {
    iu8_v4i a0[TM], a1[TM];
    if (ALDS > 0 && staged) {
      const int kt = 2 * (wk + t * KW);
      a0[0] = *(const iu8_v4i *)&s_mem[((kt * 4) << (mr_shift + 4)) + a_lane];
      a1[0] = *(const iu8_v4i *)&s_mem[(((kt + 1) * 4) << (mr_shift + 4)) + a_lane];
    } else {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        a0[i] = ringa[ALDS ? 0 : slot][i][0];
        a1[i] = ringa[ALDS ? 0 : slot][i][1];
      }
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      iu8_v4i w0, w1;
      if constexpr (W8) {
        w0 = (iu8_v4i)ring[slot][j][0];
        w1 = (iu8_v4i)ring[slot][j][WV - 1];
      } else {
        iu8_unpack_w4(ring[slot][j][0], w0, w1);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        acc[i][j] = iu8_mfma(w0, a0[i], acc[i][j]);
        acc[i][j] = iu8_mfma(w1, a1[i], acc[i][j]);
      }
    }
  };

  if constexpr (ALDS > 0) {
    // staged form: the ring never holds activations, so the not-staged fallback of an ALDS kernel
    // (shape too large for its LDS) loads them at consume time through the one-slot `ringa`
    if (!staged) {
      for (int t = 0; t < T; ++t) {
        issue(0, t);
        consume(0, t);
      }
    } else {
#pragma unroll
      for (int i = 0; i < D; ++i)
        if (i < T) issue(i, i);
      if constexpr (A_INREG) {
#pragma unroll
        for (int p = 0; p < A_PER; ++p)
          if (p * NTHR + tid < a_pieces) *(iu8_v4u *)&s_mem[(p * NTHR + tid) * 16] = areg[p];
      }
      __syncthreads();
      int t0 = 0;
      for (; t0 + 2 * D <= T; t0 += D) {  // steady state: every slot consumed and re-issued
#pragma unroll
        for (int i = 0; i < D; ++i) {
          consume(i, t0 + i);
          issue(i, t0 + i + D);
        }
      }
      for (; t0 < T; t0 += D) {  // drain
#pragma unroll
        for (int i = 0; i < D; ++i)
          if (t0 + i < T) {
            consume(i, t0 + i);
            if (t0 + i + D < T) issue(i, t0 + i + D);
          }
      }
      __syncthreads();  // every wave is done with the staged rows before s_mem holds partials
    }
  } else {
#pragma unroll
    for (int i = 0; i < D; ++i)
      if (i < T) issue(i, i);
    int t0 = 0;
    for (; t0 + 2 * D <= T; t0 += D) {
#pragma unroll
      for (int i = 0; i < D; ++i) {
        consume(i, t0 + i);
        issue(i, t0 + i + D);
      }
    }
    for (; t0 < T; t0 += D) {
#pragma unroll
      for (int i = 0; i < D; ++i)
        if (t0 + i < T) {
          consume(i, t0 + i);
          if (t0 + i + D < T) issue(i, t0 + i + D);
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

  const int nq = lg * 4;
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
  for (int idx = tid; idx < nw4 * M; idx += NTHR) {
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

#define IU8_DEC(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)                                                         \
  extern "C" __global__ __launch_bounds__(WPB * 64) void name(                                                    \
      const unsigned char *__restrict__ a, const unsigned char *__restrict__ w, const float *__restrict__ as,     \
      const float *__restrict__ ws, int *__restrict__ decode_partial, int *__restrict__ decode_counter,           \
      unsigned short *__restrict__ c, int m, int n, int k) {                                                       \
    iu8_dec_body<TM, W8, NT, KW, WPB, D, ALDS, ACC>(a, w, as, ws, decode_partial, decode_counter, c, m, n, k);     \
  }
#define IU8_DEC_VARIANT(name, TM, W8, NT, KW, WPB, D, ALDS, ACC) IU8_DEC(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)
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
#define IU8_DEC_VARIANT(name, TM, W8, NT, KW, WPB, D, ALDS, ACC)
#define IU8_PF_VARIANT(name, W8, WMW, WNW, TM, TN, ACC) IU8_PF(name, W8, WMW, WNW, TM, TN, ACC)
#include "iu8_variants.def"
#undef IU8_DEC_VARIANT
#undef IU8_PF_VARIANT
#undef IU8_PF
