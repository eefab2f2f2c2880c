// The fused decode linear of the gfx950 W4A8-iu8 path: per-token int8 quantisation of at most 4 bf16
// rows + the GEMV against them, one persistent launch. Operand orders and the contract: iu8_common.h.
//
// A workgroup (WPB waves: WN column groups x KW k-waves, as in the plain decode body) owns the
// column blocks blockIdx.x, blockIdx.x + gridDim.x, ... of WN*NT*16 columns each. It loads the rows,
// starts its weight loads as soon as they are in, quantises the rows once (row amax, IEEE divide law,
// codes into LDS in staged order) while those loads fly, then streams its blocks' weights against the
// staged codes. The weight ring (D 128-deep K steps of 128-bit nontemporal loads a wave) runs ACROSS
// block boundaries: when a wave consumes the last step of a block its loads for the next block are
// already in flight, so the memory pipe never drains inside the launch. A block ends with the
// k-waves' partials meeting in LDS (exact int32, two alternating areas so one barrier a block
// suffices) and the bf16 epilogue, whose weight scales were requested at the start and put in LDS
// behind the ring's issue: loads return in order, so a scale load issued at a block's end would only
// come back behind the whole ring. A launch gives a workgroup at most IU8_DECQ_MAXB blocks (the
// host's grid law).
#pragma once
#include "iu8_common.h"

#define IU8_DECQ_MAXB 8  // column blocks a workgroup: gridDim.x >= ceil(blocks / 8)

// CH (a launch that chains the MLP's two linears through memory, iu8_chain.h): 0 = a launch of its own.
// 1 = the chain's first linear, gate and up PAIRED: W holds 2N rows (N gate rows, then N up rows), a
// column block is ONE 16-column tile of the product p = bf16(bf16(silu(gate)) * up), whose gate tile
// goes to the waves wn = 0 and whose up tile to the waves wn = 1 (WN = 2, NT = 1). The up wave leaves
// its bf16 values in LDS, the gate wave combines them a block later (behind that block's own
// meeting, so the exchange costs no barrier of its own), stores p straight through to memory
// (coherent for the other workgroups of the launch, whatever XCD they run on) and keeps the rows'
// maxima of |p|, which end in `hook.slot` (4 floats, this workgroup's). C, if not null, receives
// [gate | up] as a launch of its own would store them (bf16 [M, 2N]).
// 2 = the chain's second linear: its rows are the first's output, so the weight ring starts first,
// then `hook.wait()` returns when every workgroup's share of the rows is in memory, the rows are
// loaded coherently, and their maxima come from `hook.amax(out)` (found by the producers) instead of a
// pass over the rows.
struct iu8_decq_pairhook {
  unsigned short *p;  // bf16 [M, N]
  float *slot;        // this workgroup's 4 maxima
};
struct iu8_decq_nohook {
  __device__ bool wait() const { return true; }
  __device__ void amax(float[4]) const {}
};
// CH 3: the rows arrive quantised (`X` is the A operand of up to 16 rows, int8 codes in fragment order, which
// is the staged order at 16 rows a tile: a straight copy into LDS; with fewer live rows, rounded up to a power of
// two, the copy takes those rows' pieces of every 256-byte run) with their scales in `hook.as`.
struct iu8_decq_codes {
  const float *as;
  __device__ bool wait() const { return true; }
  __device__ void amax(float[4]) const {}
};
// CH 4: both -- quantised rows in (CH 3), gate and up paired with p = bf16(bf16(silu(gate)) * up) out (CH 1): the
// gate+up linear of a decode MLP at 5 to 16 rows with the activation in its epilogue. `slot` null: no maxima kept
// (the rows' requantisation is a producer launch of its own behind this one).
struct iu8_decq_codes_pair {
  const float *as;
  unsigned short *p;
  float *slot;
  __device__ bool wait() const { return true; }
  __device__ void amax(float[4]) const {}
};
static __device__ __forceinline__ iu8_v4u iu8_decq_ld_coherent(const iu8_v4u *p) {
  const unsigned long long lo = __hip_atomic_load((const unsigned long long *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const unsigned long long hi = __hip_atomic_load((const unsigned long long *)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  return iu8_v4u{(unsigned)lo, (unsigned)(lo >> 32), (unsigned)hi, (unsigned)(hi >> 32)};
}
// The body's LDS, as one object: a kernel that runs two bodies one after the other (the MLP chain) lays both
// objects over one block of LDS; a kernel with one body declares one.
template <int NT, int KW, int WPB, int CH, int AKB>
struct iu8_decq_lds {
  static constexpr int WN = WPB / KW, RED = (KW - 1) * WN * NT * 256;
  static constexpr bool BIG = AKB > 20, PAIRED = CH == 1 || CH == 4;
  __attribute__((aligned(16))) iu8_u8 s_a[AKB * 1024];  // staged codes: pow2(M) * K bytes
  __attribute__((aligned(16))) int s_red[2][RED];       // the k-waves' partials, two alternating areas
  float s_amax[WPB][4];
  float s_sq[2][4];  // scale and reciprocal a row, made once a workgroup
  unsigned s_rowmax[BIG ? 16 : 1];
  float s_rsc[BIG ? 16 : 1], s_rrcp[BIG ? 16 : 1];
  float s_ws[IU8_DECQ_MAXB][WN * NT * 16];  // the epilogue's weight scales (W4: already / 16)
  __attribute__((aligned(8))) unsigned s_up[PAIRED ? 2 : 1][PAIRED ? 128 : 2];  // the up wave's bf16 values, two blocks
};
// MRS: the staged rows' power-of-two count as a shift when the kernel knows it (4: a whole 16-row tile), else -1: from M.
// Known, every LDS index of the K loop is a constant plus a register; the launches of 9 to 16 rows are 0.25-0.4 us
// faster for it.
template <bool W8, int NT, int KW, int WPB, int D, int CH = 0, class Hook = iu8_decq_nohook, int AKB = 20, int MRS = -1>
__device__ __forceinline__ void iu8_decq_body(iu8_decq_lds<NT, KW, WPB, CH, AKB> &S, const unsigned short *__restrict__ X,
                                              const iu8_u8 *__restrict__ W, const float *__restrict__ ws,
                                              iu8_u8 *__restrict__ qout, float *__restrict__ sout,
                                              unsigned short *__restrict__ C, int M, int N, int K,
                                              const Hook hook = Hook{}) {
  static_assert(KW > 1 && WPB % KW == 0, "k-waves divide the workgroup");
  constexpr int WN = WPB / KW;
  constexpr bool PAIRED = CH == 1 || CH == 4;
  static_assert(!PAIRED || (WN == 2 && NT == 1 && !W8), "the paired form: a gate wave and an up wave a tile");
  constexpr int WNB = PAIRED ? 1 : WN;  // column-tile groups of the OUTPUT a block
  constexpr int NTHR = WPB * 64;
  constexpr int WSTEP = W8 ? 2048 : 1024;  // bytes of one 16-row weight tile per 128-deep K step
  constexpr int WV = W8 ? 2 : 1;           // 16-byte loads a lane per step per tile
  constexpr int ABYTES = AKB * 1024;       // staged codes: pow2(M) * K bytes
  // BIG (more than 20 KiB staged): up to 16 rows. The rows' maxima meet by LDS integer max (a wave's
  // pieces of one load lie in one row when K is a multiple of 512: then one lane a wave), scales and
  // reciprocals are made once a row by 16 lanes, and a lane reads its row's scale for the epilogue.
  constexpr bool BIG = AKB > 20;
  static_assert(!BIG || CH != 1, "the chain's first linear stages at most 20 KiB");
  constexpr bool CODES = CH == 3 || CH == 4;
  auto &s_a = S.s_a;
  auto &s_red = S.s_red;
  auto &s_amax = S.s_amax;
  auto &s_sq = S.s_sq;
  auto &s_rowmax = S.s_rowmax;
  auto &s_rsc = S.s_rsc;
  auto &s_rrcp = S.s_rrcp;
  auto &s_ws = S.s_ws;
  auto &s_up = S.s_up;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wk = wave % KW, wn = wave / KW;
  const int ntiles = N >> 4, steps = K >> 7;
  const int ml = lane & 15, lg = lane >> 4;
  const int G = gridDim.x;
  const int T = wk < steps ? (steps - wk + KW - 1) / KW : 0;  // this wave's steps of a block: wk + t*KW
  const int nblk = (ntiles + WNB * NT - 1) / (WNB * NT);
  // the weight tile of this wave's j-th tile in the workgroup's block b (paired: the up rows follow the N gate rows)
  auto tile_of = [&](int b, int j) {
    if constexpr (PAIRED) return wn * ntiles + min((int)blockIdx.x + b * G, ntiles - 1);
    else return min((((int)blockIdx.x + b * G) * WN + wn) * NT + j, ntiles - 1);  // a tile past N re-reads the last one and stores nothing
  };
  const int nb = (int)blockIdx.x < nblk ? (nblk - (int)blockIdx.x + G - 1) / G : 0;  // this workgroup's blocks
  const int TT = nb * T;

  // ---- the rows' bf16 pieces (8 elements = 16 bytes; piece p = row * K/8 + k/8), loaded first
  int mr_shift = 0;
  if constexpr (MRS >= 0) mr_shift = MRS;
  else
    while ((1 << mr_shift) < M) ++mr_shift;
  constexpr int X_PER = CODES ? (ABYTES / 16 + NTHR - 1) / NTHR : (ABYTES / 8 + NTHR - 1) / NTHR;
  iu8_v4u xreg[X_PER];
  // CODES: the live rows' 16-byte pieces of the 16-row tile, (K / 16) << mr_shift of them: staged piece i is the tile's
  // piece (i >> mr_shift) * 16 + (i & (MR - 1)) -- the tile itself at 9 to 16 rows
  const int k8 = K >> 3, x_pieces = CODES ? (K >> 4) << mr_shift : M * k8;
  if constexpr (CODES) {
#pragma unroll
    for (int p = 0; p < X_PER; ++p) {
      const int i = p * NTHR + tid;
      if (i < x_pieces) xreg[p] = *((const iu8_v4u *)X + ((i >> mr_shift) << 4) + (i & ((1 << mr_shift) - 1)));
    }
  } else if constexpr (CH != 2) {
#pragma unroll
    for (int p = 0; p < X_PER; ++p)
      if (p * NTHR + tid < x_pieces) xreg[p] = *((const iu8_v4u *)X + p * NTHR + tid);
  }

  // ---- this workgroup's weight scales, all blocks: loaded now, put in LDS behind the ring's issue
  // (a store here would wait out the load's whole latency in front of the weight loads)
  constexpr int WS_ALL = IU8_DECQ_MAXB * (WN * NT * 16), WS_PER = (WS_ALL + NTHR - 1) / NTHR;
  float wsreg[WS_PER];
#pragma unroll
  for (int p = 0; p < WS_PER; ++p) {
    const int i = p * NTHR + tid, b = i / (WN * NT * 16), c = i - b * (WN * NT * 16);
    int n;
    bool in;
    if constexpr (PAIRED) {
      const int t = (int)blockIdx.x + b * G;
      n = (c >> 4) * N + t * 16 + (c & 15), in = t < ntiles;
    } else {
      n = ((int)blockIdx.x + b * G) * (WN * NT * 16) + c, in = n < N;
    }
    wsreg[p] = (i < min(nb, IU8_DECQ_MAXB) * (WN * NT * 16) && in) ? iu8_wsu<W8>(ws, n) : 0.f;
  }

  // ---- the issue side of the ring: block ib, step it, this lane's address in every tile
  int ib = 0, it = 0;
  const iu8_u8 *ip[NT];
  auto set_ip = [&](int b) {
#pragma unroll
    for (int j = 0; j < NT; ++j) ip[j] = W + ((size_t)tile_of(b, j) * steps + wk) * WSTEP + lane * 16;
  };
  set_ip(0);
  iu8_v4u ring[D][NT][WV];
  auto issue = [&](int slot) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int v = 0; v < WV; ++v) ring[slot][j][v] = iu8_ldg_nt(ip[j] + v * 1024);
    if (++it == T) {
      it = 0;
      if (++ib < nb) set_ip(ib);
    } else {
#pragma unroll
      for (int j = 0; j < NT; ++j) ip[j] += KW * WSTEP;
    }
  };

  // A launch of the chain that cannot complete (a producer never arrived, or the state block still carries an
  // earlier launch's raised status) gives up as a whole and says so where the caller looks: every output this
  // workgroup owns becomes a bf16 NaN (0x7FC0), so a replayed graph that can no longer complete does not hand
  // back stale or half-written rows as if they were results. (The status word says the same to a host that
  // reads the state block.)
  auto give_up = [&]() {
    constexpr int BC = WNB * NT * 16;
    for (int i = tid; i < nb * BC * M; i += NTHR) {
      const int b = i / (BC * M), r = (i / BC) % M, cc = i % BC;
      const int n = ((int)blockIdx.x + b * G) * BC + cc;
      if (n < N) C[(size_t)r * N + n] = 0x7FC0;
    }
  };
  // ---- quantise the rows: amax lane -> wave (butterfly) -> workgroup (LDS),
  // all order-free maxima; sc = max(amax / 127, 1e-30); codes by the exact reciprocal path
  float qsc[4] = {1.f, 1.f, 1.f, 1.f};
  float my_sc = 1.f;  // BIG: the scale of this lane's row (ml)
  if constexpr (CODES) {
    static_assert(!CODES || BIG, "the codes form reads its row's scale like the 80 KiB form");
    my_sc = hook.as[min(ml, M - 1)];
#pragma unroll
    for (int i = 0; i < D; ++i)
      if (i < TT) issue(i);
#pragma unroll
    for (int p = 0; p < WS_PER; ++p)
      if (p * NTHR + tid < WS_ALL) (&s_ws[0][0])[p * NTHR + tid] = wsreg[p];
#pragma unroll
    for (int p = 0; p < X_PER; ++p)
      if (p * NTHR + tid < x_pieces) *(iu8_v4u *)&s_a[(p * NTHR + tid) << 4] = xreg[p];
    __syncthreads();
  } else if constexpr (BIG) {
    // piece p * NTHR + tid = (row, col) in pieces of 8: two divides here, then steps of NTHR pieces
    const int row_step = NTHR / k8, col_step = NTHR - row_step * k8;
    int row = tid / k8, col = tid - row * k8;
    auto next_piece = [&]() {
      row += row_step, col += col_step;
      if (col >= k8) col -= k8, ++row;
    };
    if constexpr (CH == 2) {
      // the chain's second linear on the 80 KiB form (up to 4 rows): weights first (they do not depend on the
      // first linear), then the rows once every producer's share is in memory; the rows' maxima are the
      // producers' (hook.amax), no pass over the rows
#pragma unroll
      for (int i = 0; i < D; ++i)
        if (i < TT) issue(i);
      if (!hook.wait()) {
        give_up();
        return;
      }
#pragma unroll
      for (int p = 0; p < X_PER; ++p)
        if (p * NTHR + tid < x_pieces) xreg[p] = iu8_decq_ld_coherent((const iu8_v4u *)X + p * NTHR + tid);
#pragma unroll
      for (int p = 0; p < WS_PER; ++p)
        if (p * NTHR + tid < WS_ALL) (&s_ws[0][0])[p * NTHR + tid] = wsreg[p];
      float a4[4];
      hook.amax(a4);  // the whole workgroup: the maxima over the producers' shares
      if (tid < 16) s_rowmax[tid] = tid < 4 ? __float_as_uint(tid == 0 ? a4[0] : tid == 1 ? a4[1] : tid == 2 ? a4[2] : a4[3]) : 0u;
    } else {
    if (tid < 16) s_rowmax[tid] = 0u;
    __syncthreads();
    const bool wave_rows = (k8 & 63) == 0;  // a wave's 64 pieces of one load lie in one row
#pragma unroll
    for (int p = 0; p < X_PER; ++p, next_piece()) {
      const int piece = p * NTHR + tid;
      const bool live = piece < x_pieces;
      float m8 = 0.f;
      if (live) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          m8 = fmaxf(m8, fabsf(__uint_as_float(xreg[p][w] << 16)));
          m8 = fmaxf(m8, fabsf(__uint_as_float(xreg[p][w] & 0xFFFF0000u)));
        }
      }
      if (wave_rows) {  // x_pieces is then a multiple of 64: a wave is live or not as a whole
        m8 = iu8_wave_max_nonneg(m8);
        if (lane == 0 && live) __hip_atomic_fetch_max(&s_rowmax[row & 15], __float_as_uint(m8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      } else if (live) {
        __hip_atomic_fetch_max(&s_rowmax[row & 15], __float_as_uint(m8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
    row = tid / k8, col = tid - row * k8;
    asm volatile("" : "+v"(row), "+v"(col));  // walked again from here: not ten (row, col) pairs kept in registers
#pragma unroll
    for (int i = 0; i < D; ++i)
      if (i < TT) issue(i);
#pragma unroll
    for (int p = 0; p < WS_PER; ++p)
      if (p * NTHR + tid < WS_ALL) (&s_ws[0][0])[p * NTHR + tid] = wsreg[p];
    }
    __syncthreads();
    if (tid < 16) {
      const float sc = fmaxf(__fdiv_rn(__uint_as_float(s_rowmax[tid]), 127.f), 1e-30f);
      s_rsc[tid] = sc;
      s_rrcp[tid] = __fdiv_rn(1.f, sc);
    }
    __syncthreads();
    const bool out0 = blockIdx.x == 0 && qout != nullptr;
    if (blockIdx.x == 0 && sout != nullptr && tid < M) sout[tid] = s_rsc[tid];
    my_sc = s_rsc[ml];
#pragma unroll
    for (int p = 0; p < X_PER; ++p, next_piece()) {
      const int piece = p * NTHR + tid;
      if (piece >= x_pieces) continue;
      const int k = col << 3;
      const float sc = s_rsc[row], rcp = s_rrcp[row];
      float f[8];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        f[2 * w] = __uint_as_float(xreg[p][w] << 16);
        f[2 * w + 1] = __uint_as_float(xreg[p][w] & 0xFFFF0000u);
      }
      const unsigned d0 = iu8_code4_rcp(f[0], f[1], f[2], f[3], sc, rcp);
      const unsigned d1 = iu8_code4_rcp(f[4], f[5], f[6], f[7], sc, rcp);
      const int kt = k >> 6, g = (k >> 4) & 3, half = (k >> 3) & 1;
      *(iu8_v2u *)&s_a[((((kt * 4 + g) << mr_shift) + row) << 4) + half * 8] = iu8_v2u{d0, d1};
      if (out0) *(iu8_v2u *)(qout + (size_t)kt * 1024 + (row + 16 * g) * 16 + half * 8) = iu8_v2u{d0, d1};
    }
    __syncthreads();
  } else
  {
    if constexpr (CH == 2) {
      // the chain's second linear: weights first (they do not depend on the first linear), then the
      // rows once every producer's share is in memory; no pass for the maxima
#pragma unroll
      for (int i = 0; i < D; ++i)
        if (i < TT) issue(i);
      if (!hook.wait()) {
        give_up();
        return;
      }
#pragma unroll
      for (int p = 0; p < X_PER; ++p)
        if (p * NTHR + tid < x_pieces) xreg[p] = iu8_decq_ld_coherent((const iu8_v4u *)X + p * NTHR + tid);
#pragma unroll
      for (int p = 0; p < WS_PER; ++p)
        if (p * NTHR + tid < WS_ALL) (&s_ws[0][0])[p * NTHR + tid] = wsreg[p];
      float a4[4];
      hook.amax(a4);  // the whole workgroup: the maxima over the producers' shares
#pragma unroll
      for (int r = 0; r < 4; ++r) s_amax[0][r] = a4[r];
    } else {
    float am[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < X_PER; ++p) {
      const int piece = p * NTHR + tid;
      if (piece >= x_pieces) continue;
      const int row = (piece >= k8) + (piece >= 2 * k8) + (piece >= 3 * k8);  // M <= 4: no divide
      float m8 = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        m8 = fmaxf(m8, fabsf(__uint_as_float(xreg[p][w] << 16)));
        m8 = fmaxf(m8, fabsf(__uint_as_float(xreg[p][w] & 0xFFFF0000u)));
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) am[r] = r == row ? fmaxf(am[r], m8) : am[r];
    }
    // The weight ring starts here, behind the first use of the rows, not at the kernel's top: every
    // workgroup of the launch fires its ring at once, and rows requested in front of that burst took
    // 2.5 us to arrive instead of one -- the whole quantisation chain waited on them, while the
    // weights are not needed before the codes exist (QKV 7.7 -> 6.4 us, O 6.8 -> 5.9, down 13.7 -> 12.5;
    // gate+up, bound by its bytes, unchanged).
#pragma unroll
    for (int i = 0; i < D; ++i)
      if (i < TT) issue(i);
    // wave maximum of the live rows
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (r >= M) break;
      am[r] = iu8_wave_max_nonneg(am[r]);
    }
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r) s_amax[wave][r] = am[r];
    }
    // the weight scales have long arrived behind the rows' loads
#pragma unroll
    for (int p = 0; p < WS_PER; ++p)
      if (p * NTHR + tid < WS_ALL) (&s_ws[0][0])[p * NTHR + tid] = wsreg[p];
    }
    __syncthreads();
    float qrcp[4] = {1.f, 1.f, 1.f, 1.f};
    // lane r makes row r's scale and reciprocal (two IEEE divides) once a workgroup; every lane making them
    // for itself cost more than this hand-over: 16 partial maxima to read and 20 instructions a row and lane
    // (one row: QKV 5.75 -> 5.56 us, O 5.53 -> 5.34, gate+up 16.9 -> 16.5; four rows: QKV 7.8 -> 6.9)
    if (tid < 4) {
      float a = s_amax[0][tid];
      if constexpr (CH != 2) {
#pragma unroll
        for (int w = 1; w < WPB; ++w) a = fmaxf(a, s_amax[w][tid]);
      }
      const float sc = fmaxf(__fdiv_rn(a, 127.f), 1e-30f);
      s_sq[0][tid] = sc;
      s_sq[1][tid] = __fdiv_rn(1.f, sc);
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) qsc[r] = s_sq[0][r], qrcp[r] = s_sq[1][r];
    const bool out0 = blockIdx.x == 0 && qout != nullptr;
    if (blockIdx.x == 0 && sout != nullptr && tid < M)
      sout[tid] = tid == 0 ? qsc[0] : tid == 1 ? qsc[1] : tid == 2 ? qsc[2] : qsc[3];
#pragma unroll
    for (int p = 0; p < X_PER; ++p) {
      const int piece = p * NTHR + tid;
      if (piece >= x_pieces) continue;
      const int row = (piece >= k8) + (piece >= 2 * k8) + (piece >= 3 * k8), k = (piece - row * k8) << 3;
      const float sc = row == 0 ? qsc[0] : row == 1 ? qsc[1] : row == 2 ? qsc[2] : qsc[3];
      const float rcp = row == 0 ? qrcp[0] : row == 1 ? qrcp[1] : row == 2 ? qrcp[2] : qrcp[3];
      float f[8];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        f[2 * w] = __uint_as_float(xreg[p][w] << 16);
        f[2 * w + 1] = __uint_as_float(xreg[p][w] & 0xFFFF0000u);
      }
      const unsigned d0 = iu8_code4_rcp(f[0], f[1], f[2], f[3], sc, rcp);
      const unsigned d1 = iu8_code4_rcp(f[4], f[5], f[6], f[7], sc, rcp);
      // staged order: piece ((kt*4 + g) * MR + row) holds the row's 16 bytes of k = kt*64 + g*16
      const int kt = k >> 6, g = (k >> 4) & 3, half = (k >> 3) & 1;
      *(iu8_v2u *)&s_a[((((kt * 4 + g) << mr_shift) + row) << 4) + half * 8] = iu8_v2u{d0, d1};
      if (out0) *(iu8_v2u *)(qout + (size_t)kt * 1024 + (row + 16 * g) * 16 + half * 8) = iu8_v2u{d0, d1};
    }
    __syncthreads();
  }

  // ---- the consume side: block cb, step ct
  iu8_v4i acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = iu8_v4i{0, 0, 0, 0};
  int cb = 0, ct = 0;
  const int a_lane = (((lg << mr_shift) + min(ml, (1 << mr_shift) - 1)) << 4);
  // LDS writes of this wave are done, then the workgroup meets; loads in flight stay in flight
  auto meet = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
  };
  // the paired form's gate wave: its bf16 gate values of the block before, the rows' running maxima
  iu8_v2u g_prev = iu8_v2u{0, 0};
  float pmax = 0.f;
  auto pair_done = [&](int b) {  // p of the workgroup's block b: the gate wave's values x the up wave's, out of LDS
#pragma clang fp contract(off)
    if constexpr (PAIRED) {
      const iu8_v2u u = *(const iu8_v2u *)&s_up[b & 1][lane * 2];
      const int tile = (int)blockIdx.x + b * G;
      if (tile >= ntiles || ml >= M) return;
      const unsigned gw[2] = {g_prev.x, g_prev.y}, uw[2] = {u.x, u.y};
      unsigned o[2];
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const float g0 = __uint_as_float(gw[w] << 16), g1 = __uint_as_float(gw[w] & 0xFFFF0000u);
        const float u0 = __uint_as_float(uw[w] << 16), u1 = __uint_as_float(uw[w] & 0xFFFF0000u);
        const unsigned b0 = iu8_bf16_bits(iu8_silu_bf16(g0) * u0), b1 = iu8_bf16_bits(iu8_silu_bf16(g1) * u1);
        o[w] = b0 | (b1 << 16);
        pmax = fmaxf(pmax, fmaxf(fabsf(iu8_bf16_f32((unsigned short)b0)), fabsf(iu8_bf16_f32((unsigned short)b1))));
      }
      __hip_atomic_store((unsigned long long *)(hook.p + (size_t)ml * N + tile * 16 + lg * 4),
                         (unsigned long long)o[0] | ((unsigned long long)o[1] << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  };
  auto block_end = [&]() {
    int *red = s_red[cb & 1];
    if (wk > 0) {
#pragma unroll
      for (int j = 0; j < NT; ++j) *(iu8_v4i *)&red[(((wk - 1) * WN + wn) * NT + j) * 256 + lane * 4] = acc[j];
    }
    meet();
    if (wk == 0) {
#pragma unroll
      for (int q = 0; q < KW - 1; ++q)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[j] += *(const iu8_v4i *)&red[((q * WN + wn) * NT + j) * 256 + lane * 4];
      const float am = BIG ? my_sc : ml == 0 ? qsc[0] : ml == 1 ? qsc[1] : ml == 2 ? qsc[2] : qsc[3];
      if constexpr (PAIRED) {
        const int tile = (int)blockIdx.x + cb * G;
        const float *wsu = &s_ws[min(cb, IU8_DECQ_MAXB - 1)][wn * 16 + lg * 4];
        unsigned h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) h[r] = iu8_bf16_bits(iu8_epi(acc[0][r], am, wsu[r]));
        const iu8_v2u out = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        if (C != nullptr && tile < ntiles && ml < M) *(iu8_v2u *)(C + (size_t)ml * 2 * N + wn * N + tile * 16 + lg * 4) = out;
        if (wn == 1) {
          *(iu8_v2u *)&s_up[cb & 1][lane * 2] = out;  // read by the gate wave behind the NEXT meeting
        } else {
          if (cb > 0) pair_done(cb - 1);  // the up wave stored these before the meeting just passed
          g_prev = out;
        }
      } else {
        const int nt0 = (((int)blockIdx.x + cb * G) * WN + wn) * NT;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          if (nt0 + j >= ntiles || ml >= M) continue;
          const int n = (nt0 + j) * 16 + lg * 4;
          const float *wsu = &s_ws[min(cb, IU8_DECQ_MAXB - 1)][(wn * NT + j) * 16 + lg * 4];
          unsigned h[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) h[r] = iu8_bf16_bits(iu8_epi(acc[j][r], am, wsu[r]));
          *(iu8_v2u *)(C + (size_t)ml * N + n) = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        }
      }
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[j] = iu8_v4i{0, 0, 0, 0};
    ++cb;
  };
  auto consume = [&](int slot) {
    const int kt = 2 * (wk + ct * KW);
    const iu8_v4i a0 = *(const iu8_v4i *)&s_a[((kt * 4) << (mr_shift + 4)) + a_lane];
    const iu8_v4i a1 = *(const iu8_v4i *)&s_a[(((kt + 1) * 4) << (mr_shift + 4)) + a_lane];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      iu8_v4i w0, w1;
      if constexpr (W8) {
        w0 = (iu8_v4i)ring[slot][j][0];
        w1 = (iu8_v4i)ring[slot][j][WV - 1];
      } else {
        iu8_unpack_w4(ring[slot][j][0], w0, w1);
      }
      acc[j] = iu8_mfma(w0, a0, acc[j]);
      acc[j] = iu8_mfma(w1, a1, acc[j]);
    }
    if (++ct == T) {
      ct = 0;
      block_end();
    }
  };

  if (T == 0) {  // a k-wave past a short K: no steps, but it meets the others once a block
    for (int b = 0; b < nb; ++b) block_end();
  } else {
    int L0 = 0;
    for (; L0 + 2 * D <= TT; L0 += D) {  // steady state: every slot consumed and re-issued
#pragma unroll
      for (int i = 0; i < D; ++i) {
        consume(i);
        issue(i);
      }
    }
    for (; L0 < TT; L0 += D) {  // drain
#pragma unroll
      for (int i = 0; i < D; ++i) {
        if (L0 + i < TT) {
          consume(i);
          if (L0 + i + D < TT) issue(i);
        }
      }
    }
  }
  if constexpr (PAIRED) {
    // the last block's pair, behind one more meeting; then this workgroup's maxima: a lane holds row
    // ml's over its 4 columns of every block, the four lanes of a row meet by two exchanges
    meet();
    if (wk == 0 && wn == 0) {
      if (nb > 0) pair_done(nb - 1);
      pmax = fmaxf(pmax, __shfl_xor(pmax, 16));
      pmax = fmaxf(pmax, __shfl_xor(pmax, 32));
      if (lane < 4 && hook.slot != nullptr)  // all four words, every launch: nothing of an earlier launch survives
        __hip_atomic_store((unsigned *)hook.slot + lane, lane < M ? __float_as_uint(pmax) : 0u, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}
