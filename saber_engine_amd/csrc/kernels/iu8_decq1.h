// The fused decode linear for ONE row (M = 1): per-token int8 quantisation of a bf16 row + the GEMV
// against it, one persistent launch, with the row's codes made just in time inside the weight stream.
// Operand orders and the contract: iu8_common.h; the several-row form and the geometry: iu8_decq.h.
//
// In the several-row form every workgroup turns the whole row into codes in front of its first MFMA:
// that is VALU work for the whole CU (about 11 operations an element, 1.2-1.4 us at K = 17,408)
// behind two workgroup barriers, while the weight loads it has started wait to be consumed. Here a
// wave touches only the K steps it will multiply (k-wave wk owns steps wk, wk + KW, ...):
//   * it loads the bf16 pieces of its own steps (a lane a piece of 8 elements, 4 steps a wave-load),
//     takes their maximum (packed 16-bit maxima on the bit patterns) and parks them in its own LDS
//     region -- no other wave reads that region, so no barrier covers it;
//   * the waves' maxima meet once (one barrier; every wave then makes the row's scale and
//     reciprocal itself: two IEEE divides cost less than a second barrier);
//   * the codes of a chunk of 4 steps are made from the parked pieces one chunk ahead of their use,
//     in place (a step's 256 bytes of bf16 become its 128 bytes of codes), by the law's own routine
//     (iu8_code4_rcp), while the wave would otherwise wait for its weight loads; only the first
//     chunk stands in front of the first MFMA. The two column groups of a k step convert the same
//     pieces twice: the VALU has the room (the launch is bound by its weight bytes), a hand-over
//     between waves would cost a barrier a chunk.
// Later column blocks of the workgroup find all codes in place. The weight ring, the partials' meeting
// in LDS and the epilogue are those of iu8_decq.h.
#pragma once
#include "iu8_common.h"

#define IU8_DECQ1_MAXB 8       // column blocks a workgroup: gridDim.x >= ceil(blocks / 8)
#define IU8_DECQ1_KMAX 20480   // the row's K: KMAX / 128 / KW steps a k-wave, 256 bytes of LDS each

template <bool W8, int KW, int WPB, int D>
__device__ __forceinline__ void iu8_decq1_body(const unsigned short *__restrict__ X, const iu8_u8 *__restrict__ W,
                                               const float *__restrict__ ws, iu8_u8 *__restrict__ qout,
                                               float *__restrict__ sout, unsigned short *__restrict__ C, int N, int K) {
  static_assert(KW > 1 && WPB % KW == 0, "k-waves divide the workgroup");
  static_assert(4 % D == 0, "a chunk of 4 steps is whole rounds of the ring");
  constexpr int WN = WPB / KW;
  constexpr int NTHR = WPB * 64;
  constexpr int WSTEP = W8 ? 2048 : 1024;  // bytes of one 16-row weight tile per 128-deep K step
  constexpr int WV = W8 ? 2 : 1;           // 16-byte loads a lane per step
  constexpr int TMAX = IU8_DECQ1_KMAX / 128 / KW, NCH = (TMAX + 3) / 4;  // steps and chunks of a k-wave
  constexpr int RED = (KW - 1) * WN * 256;  // ints of one partial area
  __shared__ __attribute__((aligned(16))) iu8_u8 s_x[WPB][TMAX * 256];  // a wave's pieces, then its codes, a step every 256 bytes
  __shared__ __attribute__((aligned(16))) int s_red[2][RED];
  __shared__ __attribute__((aligned(16))) float s_amax[WPB];
  __shared__ float s_ws[IU8_DECQ1_MAXB][WN * 16];  // the epilogue's weight scales (W4: already / 16)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wk = wave % KW, wn = wave / KW;
  const int ntiles = N >> 4, steps = K >> 7;
  const int ml = lane & 15, lg = lane >> 4;
  const int G = gridDim.x;
  const int T = wk < steps ? (steps - wk + KW - 1) / KW : 0;  // this wave's steps of a block: wk + t*KW
  const int nblk = (ntiles + WN - 1) / WN;
  auto tile_of = [&](int b) { return min(((int)blockIdx.x + b * G) * WN + wn, ntiles - 1); };  // a tile past N re-reads the last one and stores nothing
  const int nb = (int)blockIdx.x < nblk ? (nblk - (int)blockIdx.x + G - 1) / G : 0;  // this workgroup's blocks
  const int TT = nb * T;
  iu8_u8 *mine = s_x[wave];

  // ---- this wave's pieces of the row: chunk c, lane (lg, ml) = piece ml of step 4c + lg
  // (every load unconditional -- a lane past the wave's steps re-reads the row's first step and drops it:
  // a load under a test is waited for before the next one is requested, a memory latency a chunk)
  iu8_v4u xreg[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int t = 4 * c + lg;
    xreg[c] = *(const iu8_v4u *)(X + (size_t)(t < T ? wk + t * KW : 0) * 128 + ml * 8);
  }
#pragma unroll
  for (int c = 0; c < NCH; ++c)
    if (4 * c + lg >= T) xreg[c] = iu8_v4u{0, 0, 0, 0};

  // ---- this workgroup's weight scales, all blocks: loaded now, put in LDS behind the ring's issue
  constexpr int WS_ALL = IU8_DECQ1_MAXB * (WN * 16), WS_PER = (WS_ALL + NTHR - 1) / NTHR;
  float wsreg[WS_PER];
#pragma unroll
  for (int p = 0; p < WS_PER; ++p) {
    const int i = p * NTHR + tid, b = i / (WN * 16), c = i - b * (WN * 16);
    const int n = ((int)blockIdx.x + b * G) * (WN * 16) + c;
    wsreg[p] = (i < min(nb, IU8_DECQ1_MAXB) * (WN * 16) && n < N) ? iu8_wsu<W8>(ws, n) : 0.f;
  }

  // ---- the issue side of the ring: block ib, step it, this lane's address
  int ib = 0, it = 0;
  const iu8_u8 *ip = W + ((size_t)tile_of(0) * steps + wk) * WSTEP + lane * 16;
  iu8_v4u ring[D][WV];
  auto issue = [&](int slot) {
#pragma unroll
    for (int v = 0; v < WV; ++v) ring[slot][v] = iu8_ldg_nt(ip + v * 1024);
    if (++it == T) {
      it = 0;
      if (++ib < nb) ip = W + ((size_t)tile_of(ib) * steps + wk) * WSTEP + lane * 16;
    } else {
      ip += KW * WSTEP;
    }
  };

  // ---- the pieces' maximum (bit patterns without the sign, two a packed 16-bit maximum; a lane that holds
  // a NaN takes the f32 maximum, which passes NaNs over) and the pieces into this wave's region
  typedef unsigned short us2 __attribute__((ext_vector_type(2)));
  us2 m2 = {0, 0};
#pragma unroll
  for (int c = 0; c < NCH; ++c)
    if (4 * c < T) {  // (wave-uniform: a short row's wave skips the chunks it does not have)
#pragma unroll
      for (int w = 0; w < 4; ++w) m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(us2, xreg[c][w] & 0x7FFF7FFFu));
    }
  const unsigned top = m2.x > m2.y ? m2.x : m2.y;
  float am = __uint_as_float(top << 16);
  if (top > 0x7F80u) {
    am = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        am = fmaxf(am, fabsf(__uint_as_float(xreg[c][w] << 16)));
        am = fmaxf(am, fabsf(__uint_as_float(xreg[c][w] & 0xFFFF0000u)));
      }
  }
#pragma unroll
  for (int c = 0; c < NCH; ++c)
    if (4 * c < T) *(iu8_v4u *)&mine[(4 * c + lg) * 256 + ml * 16] = xreg[c];  // (zeros past the wave's steps of its last chunk)
  // The weight ring starts here, behind the first use of the row's pieces (requested in front of the
  // whole launch's burst of weight loads, they would arrive a microsecond later).
#pragma unroll
  for (int i = 0; i < D; ++i)
    if (i < TT) issue(i);
  am = iu8_wave_max_nonneg(am);
  if (lane == 0) s_amax[wave] = am;
#pragma unroll
  for (int p = 0; p < WS_PER; ++p)
    if (p * NTHR + tid < WS_ALL) (&s_ws[0][0])[p * NTHR + tid] = wsreg[p];
  __syncthreads();
  float amax = 0.f;
#pragma unroll
  for (int w = 0; w < WPB; w += 4) {
    const iu8_v4f a4 = *(const iu8_v4f *)&s_amax[w];
    amax = fmaxf(fmaxf(amax, a4.x), fmaxf(fmaxf(a4.y, a4.z), a4.w));
  }
  const float sc = fmaxf(__fdiv_rn(amax, 127.f), 1e-30f), rcp = __fdiv_rn(1.f, sc);
  if (blockIdx.x == 0 && sout != nullptr && tid == 0) sout[0] = sc;

  // ---- chunk c of this wave's steps: pieces -> codes, in place (steps past the wave's hold zeros). No access
  // to memory in here: a store inside the weight stream would have the ring's loads waited out around it.
  auto convert = [&](int c) {
    const int t = 4 * c + lg;
    const iu8_v4u r = *(const iu8_v4u *)&mine[t * 256 + ml * 16];
    const unsigned d0 = iu8_code4_rcp(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xFFFF0000u), __uint_as_float(r.y << 16),
                                      __uint_as_float(r.y & 0xFFFF0000u), sc, rcp);
    const unsigned d1 = iu8_code4_rcp(__uint_as_float(r.z << 16), __uint_as_float(r.z & 0xFFFF0000u), __uint_as_float(r.w << 16),
                                      __uint_as_float(r.w & 0xFFFF0000u), sc, rcp);
    *(iu8_v2u *)&mine[t * 256 + ml * 8] = iu8_v2u{d0, d1};
  };
  convert(0);

  // ---- the consume side: block cb, step ct
  iu8_v4i acc = iu8_v4i{0, 0, 0, 0};
  int cb = 0, ct = 0;
  auto block_end = [&]() {
    int *red = s_red[cb & 1];
    if (wk > 0) *(iu8_v4i *)&red[((wk - 1) * WN + wn) * 256 + lane * 4] = acc;
    // LDS writes of this wave are done, then the workgroup meets; loads in flight stay in flight
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    if (wk == 0) {
#pragma unroll
      for (int q = 0; q < KW - 1; ++q) acc += *(const iu8_v4i *)&red[(q * WN + wn) * 256 + lane * 4];
      const int nt = ((int)blockIdx.x + cb * G) * WN + wn;
      if (nt < ntiles && ml == 0) {
        const float *wsu = &s_ws[min(cb, IU8_DECQ1_MAXB - 1)][wn * 16 + lg * 4];
        unsigned h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) h[r] = iu8_bf16_bits(iu8_epi(acc[r], sc, wsu[r]));
        *(iu8_v2u *)(C + nt * 16 + lg * 4) = iu8_v2u{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
      }
    }
    acc = iu8_v4i{0, 0, 0, 0};
    ++cb;
  };
  auto consume = [&](int slot) {
    const iu8_v4i a0 = *(const iu8_v4i *)&mine[ct * 256 + lg * 16];
    const iu8_v4i a1 = *(const iu8_v4i *)&mine[ct * 256 + 64 + lg * 16];
    iu8_v4i w0, w1;
    if constexpr (W8) {
      w0 = (iu8_v4i)ring[slot][0];
      w1 = (iu8_v4i)ring[slot][WV - 1];
    } else {
      iu8_unpack_w4(ring[slot][0], w0, w1);
    }
    acc = iu8_mfma(w0, a0, acc);
    acc = iu8_mfma(w1, a1, acc);
    if (++ct == T) {
      ct = 0;
      block_end();
    }
  };
  // flat step L0 (a multiple of 4 in the first block): the chunk after the one about to be consumed
  auto ahead = [&](int L0) {
    if ((L0 & 3) == 0 && L0 + 4 < T) convert((L0 >> 2) + 1);
  };

  if (T == 0) {  // a k-wave past a short K: no steps, but it meets the others once a block
    for (int b = 0; b < nb; ++b) block_end();
  } else {
    int L0 = 0;
    // (the next chunk's conversion sits behind the round's first re-issued loads, not in front of its first MFMA)
    for (; L0 + 2 * D <= TT; L0 += D) {  // steady state: every slot consumed and re-issued
#pragma unroll
      for (int i = 0; i < D; ++i) {
        consume(i);
        issue(i);
        if (i == (D - 1) / 2) ahead(L0);
      }
    }
    for (; L0 < TT; L0 += D) {  // drain
#pragma unroll
      for (int i = 0; i < D; ++i) {
        if (L0 + i < TT) {
          consume(i);
          if (L0 + i + D < TT) issue(i);
        }
        if (i == (D - 1) / 2) ahead(L0);
      }
    }
  }
  // ---- the optional code output, by workgroup 0 behind its stream: every k-wave of the first column group
  // holds the codes of its steps; A fragment order, row 0 of fragment kt, 16-byte group g
  if (blockIdx.x == 0 && qout != nullptr && wn == 0) {
    for (int t = lg; t < T; t += 4) {
      const int k = (wk + t * KW) * 128 + ml * 8;
      *(iu8_v2u *)(qout + (size_t)(k >> 6) * 1024 + (16 * ((k >> 4) & 3)) * 16 + ((k >> 3) & 1) * 8) = *(const iu8_v2u *)&mine[t * 256 + ml * 8];
    }
  }
}
