// The two GEMM bodies of the gfx950 W4A8-iu8 path, shared by the dense code object (`macaq_iu8`)
// and the grouped, expert-routed one (`moe_iu8`). Operand orders and the contract: iu8_common.h.
//
// Both bodies see the rows they work on through an `iu8_rows` map: a dense launch owns rows
// [0, M) of A / as / C; a grouped launch owns, per tile of the router's tile table, `rows` rows of
// one expert starting at expert-major row `row0`, whose activations are either those rows of a
// compact A (down projection) or gathered through `row_tok` from the token-major A (gate+up),
// the reference's schedule (crates/saber-kernels/hip/moe_grouped.hip:33-120). Rows past the live
// ones are clamped, never predicated, and never stored.
#pragma once
#include "iu8_common.h"
#include <type_traits>

struct iu8_rows {
  const int *row_tok;  // gather map: expert-major row -> row of A and `as`; nullptr = in place
  int row0;            // first row (a multiple of 16) of the tile in C and in a compact A
  int rows;            // live rows from row0
};
// The row of A (and of `as`) behind tile-local row m.
static __device__ __forceinline__ int iu8_arow(const iu8_rows &R, int m) {
  if (R.row_tok != nullptr) return max(R.row_tok[R.row0 + min(m, R.rows - 1)], 0);
  return R.row0 + min(m, ((R.rows + 15) & ~15) - 1);
}

// Where a workgroup stands in a decode launch: its column block, its share of a grid-level split
// of K and the number of shares. A plain launch reads them off the grid; a launch that lays
// several problems' grids end to end hands each workgroup its own.
struct iu8_blk {
  int bx, z, Z;
};
static __device__ __forceinline__ iu8_blk iu8_blk_of_grid() {
  return iu8_blk{(int)blockIdx.x, (int)blockIdx.z, (int)gridDim.z};
}

// ============================================================================ decode band
// MODE 1, the gate+up projection of an MLP with the activation in its epilogue: W holds N/2 gate rows
// and then N/2 up rows, a wave's NT tiles are NT/2 gate tiles and the up tiles of the same columns,
// and C is p = bf16(bf16(silu(gate)) * up), bf16 [rows, N/2] -- what the three steps (this GEMM to
// bf16, SiLU * up, bf16) write (crates/saber-kernels/hip/mxfp4_hadi8.hip:118-146), without the
// [gate | up] matrix in memory. A column block is WN * NT/2 * 16 columns of p.
// MODE 2, the projection behind it: A is those bf16 rows themselves ([rows, K], in place), quantised
// here by the per-token law (crates/saber-kernels/hip/macaq_i8.h:10-13) into the staged LDS form, the
// scales kept in LDS for the epilogue; `as` is not read. The tile's rows must fit: pow2(rows) * K <=
// ALDS KiB (the host's rule). Every workgroup of a tile repeats its rows' quantisation, which is what
// a producer launch in front would cost once -- worth it for the few rows an expert has in decode.
// EXACT (the staged forms): the first ring issued by every wave and the last steps as straight-line code, so that
// the compiler counts the loads in flight at each consume (see the streamed form's ring below). It costs registers:
// the grouped launches, held to 64 a lane for eight waves a SIMD, keep the plain loops.
template <int TM, bool W8, int NT, int KW, int WPB, int D, int ALDS, bool ACC, int MODE = 0, bool EXACT = true>
__device__ __forceinline__ void iu8_dec_body(const iu8_u8 *__restrict__ A, const iu8_u8 *__restrict__ W,
                                             const float *__restrict__ as, const float *__restrict__ ws,
                                             int *__restrict__ P, int *__restrict__ cnt, void *__restrict__ Cv,
                                             const iu8_rows R, int N, int K, const iu8_blk B = iu8_blk_of_grid()) {
  const int M = R.rows;
  static_assert(WPB % KW == 0, "k-waves divide the workgroup");
  static_assert(ALDS == 0 || TM == 1, "LDS staging of A is the M <= 16 form");
  constexpr bool PAIR = MODE == 1, AQ = MODE == 2;
  static_assert(!PAIR || (NT % 2 == 0 && TM == 1 && !W8 && !ACC), "the paired form: gate tiles and their up tiles a wave");
  constexpr int NP = PAIR ? NT / 2 : 1;  // tiles of p a wave (paired: tiles [0, NP) are gate tiles, [NP, NT) their up tiles)
  static_assert(!AQ || (ALDS > 0 && !ACC), "rows quantised here are staged in LDS");
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
  const int Z = B.Z, z = B.z;
  const int spb = (steps + Z - 1) / Z;
  const int s_lo = z * spb, s_hi = min(steps, s_lo + spb);
  const int nt0 = (B.bx * WN + wn) * NT;
  const int ml = lane & 15, lg = lane >> 4;
  // this wave's steps: s_lo + wk + t*KW, t in [0, T)
  const int T = s_lo + wk < s_hi ? (s_hi - s_lo - wk + KW - 1) / KW : 0;

  const iu8_u8 *wp[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    // a tile past N re-reads the last one and stores nothing; paired: tile j = 0 of the gate rows, 1 of the up rows
    const int ntj = PAIR ? (j / NP) * (ntiles >> 1) + min((B.bx * WN + wn) * NP + j % NP, (ntiles >> 1) - 1) : min(nt0 + j, ntiles - 1);
    // (EXACT: a k-wave past a short K issues the first ring all the same, on the share's last step, and drops it)
    wp[j] = W + ((size_t)ntj * steps + (EXACT && ALDS > 0 ? min(s_lo + wk, steps - 1) : s_lo + wk)) * WSTEP + lane * 16;
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
  // rows quantised here (AQ): 16-element groups of the bf16 rows, group i = row * K/16 + k/16; a thread's
  // first group stays in registers (all of them for up to NTHR groups: 5 rows of 1,536), later ones are
  // read again for the codes, out of the cache
  iu8_v4u xraw[2];
  __shared__ unsigned s_rmax[AQ ? 16 : 1];
  __shared__ float s_rsc[AQ ? 16 : 1], s_rrcp[AQ ? 16 : 1];
  const int k16 = K >> 4, q_groups = M * k16;
  auto q_src = [&](int i) {
    const int row = i / k16, g = i - row * k16;
    return (const iu8_v4u *)((const unsigned short *)A + (size_t)iu8_arow(R, row) * K + g * 16);
  };
  if constexpr (ALDS > 0) {
    while ((1 << mr_shift) < M) ++mr_shift;
    a_pieces = ((s_hi - s_lo) * 2 * 4) << mr_shift;
    staged = M <= 16 && a_pieces * 16 <= ABYTES;
    if constexpr (AQ) {
      if (!staged || Z != 1) return;  // the host's rule keeps such a launch out; nothing is stored
      if (tid < 16) s_rmax[tid] = 0u;
      if (tid < q_groups) {
        const iu8_v4u *src = q_src(tid);
        xraw[0] = src[0];
        xraw[1] = src[1];
      }
    } else if (staged) {
      auto a_src = [&](int piece) {
        const int r = piece & ((1 << mr_shift) - 1), g = (piece >> mr_shift) & 3, kt = piece >> (mr_shift + 2);
        const int ar = iu8_arow(R, r);
        return (const iu8_v4u *)(A + (((size_t)(ar >> 4) * ktiles + 2 * s_lo + kt) * 1024 + ((ar & 15) + 16 * g) * 16));
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
  // this lane's row of every activation tile, at the wave's first K step. A lane past the live rows reads the
  // last live row again (the piece a live lane of the same load already touches: no line more from L2), and
  // what it multiplies lands in output rows that are never stored. The loads are unconditional on purpose:
  // under a per-lane test the compiler cannot count them and waits for every load in flight (`vmcnt(0)`) at
  // each consume, which makes a ring of any depth a ring of one.
  const iu8_u8 *ap[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int ar = iu8_arow(R, min(i * 16 + ml, M - 1));
    ap[i] = A + ((size_t)(ar >> 4) * ktiles + (size_t)(s_lo + wk) * 2) * 1024 + ((ar & 15) + 16 * lg) * 16;
  }
  auto issue = [&](int slot, int t) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int v = 0; v < WV; ++v) ring[slot][j][v] = iu8_ldg_nt(wp[j] + (size_t)t * (KW * WSTEP) + v * 1024);
    if (!staged) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          ringa[ALDS ? 0 : slot][i][h] = *(const iu8_v4i *)(ap[i] + ((size_t)t * (2 * KW) + h) * 1024);
    }
  };
  auto issue_w = [&](int slot, int t) {  // the staged ring: weights alone, no run-time test around a load
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int v = 0; v < WV; ++v) ring[slot][j][v] = iu8_ldg_nt(wp[j] + (size_t)t * (KW * WSTEP) + v * 1024);
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
      if constexpr (EXACT) {
#pragma unroll
        for (int i = 0; i < D; ++i) issue_w(i, max(min(i, T - 1), 0));
      } else {
#pragma unroll
        for (int i = 0; i < D; ++i)
          if (i < T) issue(i, i);
      }
      if constexpr (AQ) {
#pragma clang fp contract(off)
        // the rows' maxima (f32 maxima of |x| as the producers take them, met by an integer max in LDS:
        // non-negative floats order as their bit patterns), scales by 16 lanes, codes into the staged form
        auto val = [&](const iu8_v4u (&x)[2], int j) {
          const unsigned w = x[j >> 3][(j >> 1) & 3];
          return __uint_as_float((j & 1) ? (w & 0xFFFF0000u) : (w << 16));
        };
        auto group_max = [&](const iu8_v4u (&x)[2], int i) {
          float mx = 0.f;
#pragma unroll
          for (int j = 0; j < 16; ++j) mx = fmaxf(mx, fabsf(val(x, j)));
          atomicMax(&s_rmax[i / k16], __float_as_uint(mx));
        };
        auto group_codes = [&](const iu8_v4u (&x)[2], int i) {
          const int row = i / k16, g = i - row * k16;
          const float sc = s_rsc[row], rcp = s_rrcp[row];
          unsigned d[4];
#pragma unroll
          for (int w = 0; w < 4; ++w) d[w] = iu8_code4_rcp(val(x, w * 4), val(x, w * 4 + 1), val(x, w * 4 + 2), val(x, w * 4 + 3), sc, rcp);
          // staged piece ((kt * 4 + chunk) * MR + row): the 16 codes of k = kt * 64 + chunk * 16, i.e. group g = kt * 4 + chunk
          *(iu8_v4u *)&s_mem[((g << mr_shift) + row) << 4] = iu8_v4u{d[0], d[1], d[2], d[3]};
        };
        __syncthreads();
        if (tid < q_groups) group_max(xraw, tid);
        for (int i = tid + NTHR; i < q_groups; i += NTHR) {
          const iu8_v4u *src = q_src(i);
          const iu8_v4u x[2] = {src[0], src[1]};
          group_max(x, i);
        }
        __syncthreads();
        if (tid < 16) {
          const float sc = fmaxf(__fdiv_rn(__uint_as_float(s_rmax[tid]), 127.f), 1e-30f);
          s_rsc[tid] = sc;
          s_rrcp[tid] = __fdiv_rn(1.f, sc);
        }
        __syncthreads();
        if (tid < q_groups) group_codes(xraw, tid);
        for (int i = tid + NTHR; i < q_groups; i += NTHR) {
          const iu8_v4u *src = q_src(i);
          const iu8_v4u x[2] = {src[0], src[1]};
          group_codes(x, i);
        }
      } else if constexpr (A_INREG) {
#pragma unroll
        for (int p = 0; p < A_PER; ++p)
          if (p * NTHR + tid < a_pieces) *(iu8_v4u *)&s_mem[(p * NTHR + tid) * 16] = areg[p];
      }
      __syncthreads();
      int t0 = 0;
      if constexpr (EXACT) {
        for (; t0 + 2 * D <= T; t0 += D) {
#pragma unroll
          for (int i = 0; i < D; ++i) {
            consume(i, t0 + i);
            __builtin_amdgcn_sched_barrier(0);
            issue_w(i, t0 + i + D);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        const int rest = T - t0;  // up to 2D - 1 steps left, min(rest, D) of them in the ring
#pragma unroll
        for (int e = 0; e < D; ++e) {
          if (rest - D != e) continue;  // rest = D + e: e more steps to issue
#pragma unroll
          for (int i = 0; i < D; ++i) {
            consume(i, t0 + i);
            __builtin_amdgcn_sched_barrier(0);
            if (i < e) issue_w(i, t0 + i + D);
            __builtin_amdgcn_sched_barrier(0);
          }
#pragma unroll
          for (int i = 0; i < e; ++i) consume(i, t0 + D + i);
        }
        if (rest < D) {
#pragma unroll
          for (int i = 0; i < D; ++i)
            if (i < rest) consume(i, t0 + i);
        }
      } else {
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
      }
      __syncthreads();  // every wave is done with the staged rows before s_mem holds partials
    }
  } else {
    // Every load of the ring is issued unconditionally and the tail is straight-line code a case, so that the
    // compiler can count the loads in flight at each consume (`vmcnt(n)` for the slot's own loads, the rest stay
    // in flight). Under a test -- a first ring of fewer than D steps, a drain loop that asks `is there a step D
    // ahead` -- it cannot, and waits for every load in flight at each consume. The scheduling fences keep a
    // slot's re-issue behind its own consume and in front of the next slot's: without them the compiler gathers
    // the D consumes and then the D issues, i.e. waits for everything, multiplies, and only then asks for more.
    // A wave with fewer than D steps loads its last step again into the spare slots and does not consume them.
    if (T > 0) {
#pragma unroll
      for (int i = 0; i < D; ++i) issue(i, min(i, T - 1));
    }
    int t0 = 0;
    auto round = [&](int t) {
#pragma unroll
      for (int i = 0; i < D; ++i) {
        consume(i, t + i);
        __builtin_amdgcn_sched_barrier(0);
        issue(i, t + i + D);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    for (; t0 + 2 * D <= T; t0 += D) round(t0);
    const int rest = T - t0;  // up to 2D - 1 steps left, min(rest, D) of them in the ring
#pragma unroll
    for (int e = 0; e < D; ++e) {
      if (rest - D != e) continue;  // rest = D + e: e more steps to issue
#pragma unroll
      for (int i = 0; i < D; ++i) {
        consume(i, t0 + i);
        __builtin_amdgcn_sched_barrier(0);
        if (i < e) issue(i, t0 + i + D);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int i = 0; i < e; ++i) consume(i, t0 + D + i);
    }
    if (rest < D) {
#pragma unroll
      for (int i = 0; i < D; ++i)
        if (i < rest) consume(i, i);
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
  if constexpr (PAIR) {
#pragma clang fp contract(off)
    const int half = N >> 1;
    if (wk != 0 || ml >= M) return;
    const float am = as[iu8_arow(R, ml)];
#pragma unroll
    for (int jj = 0; jj < NP; ++jj) {
      const int tp = (B.bx * WN + wn) * NP + jj;  // this wave's jj-th tile of p
      if (tp >= (ntiles >> 1)) continue;
      const int n = tp * 16 + nq;
      unsigned h[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float g = iu8_bf16_f32((unsigned short)iu8_bf16_bits(iu8_epi(acc[0][jj][r], am, iu8_wsu<W8>(ws, n + r))));
        const float u = iu8_bf16_f32((unsigned short)iu8_bf16_bits(iu8_epi(acc[0][NP + jj][r], am, iu8_wsu<W8>(ws, half + n + r))));
        h[r] = iu8_bf16_bits(iu8_silu_bf16(g) * u);
      }
      *(iu8_v2u *)((unsigned short *)Cv + (size_t)(R.row0 + ml) * half + n) = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
    }
    return;
  }
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
        const size_t crow = (size_t)(R.row0 + m) * N;
        if constexpr (ACC) {
          *(iu8_v4i *)((int *)Cv + crow + n) = acc[i][j];
        } else {
          const float am = AQ ? s_rsc[m] : as[iu8_arow(R, m)];
          unsigned h[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) h[r] = iu8_bf16_bits(iu8_epi(acc[i][j][r], am, wsu[r]));
          *(iu8_v2u *)((unsigned short *)Cv + crow + n) = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
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
        if (m < M) iu8_store_through(&P[((size_t)z * M + m) * N + n], acc[i][j]);
      }
    }
    iu8_stores_done();
  }
  __syncthreads();
  if (tid == 0) s_last = (iu8_arrive(&cnt[B.bx]) == Z - 1);
  __syncthreads();
  if (!s_last) return;
  if (tid == 0) __hip_atomic_store(&cnt[B.bx], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int nb = B.bx * BN, nw4 = min(BN, N - nb) >> 2;
  for (int idx = tid; idx < nw4 * M; idx += NTHR) {
    const int m = idx / nw4, n = nb + (idx % nw4) * 4;
    iu8_v4i sum = iu8_v4i{0, 0, 0, 0};
    for (int q = 0; q < Z; ++q) sum += iu8_load_through(&P[((size_t)q * M + m) * N + n]);
    const size_t crow = (size_t)(R.row0 + m) * N;
    if constexpr (ACC) {
      *(iu8_v4i *)((int *)Cv + crow + n) = sum;
    } else {
      const float am = as[iu8_arow(R, m)];
      unsigned h[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) h[r] = iu8_bf16_bits(iu8_epi(sum[r], am, iu8_wsu<W8>(ws, n + r)));
      *(iu8_v2u *)((unsigned short *)Cv + crow + n) = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
    }
  }
}
