// The MFMA-bound tile GEMM of the gfx950 W4A8-iu8 path on v_mfma_i32_32x32x32_i8, the int8 MFMA
// shape that sustains the card's matrix rate. Shared by the dense code object (`macaq_iu8`,
// persistent workgroups walking an XCD-aware tile order) and the grouped, expert-routed one
// (`moe_iu8`, one tile of the router's table a workgroup). Operand orders and the contract:
// iu8_common.h; the row map `iu8_rows`: iu8_gemm.h.
//
// A workgroup of WMW x WNW waves owns a (WMW*TM*32) x (WNW*TN*32) output tile and runs its tiles
// one after another. Each 128-deep K step lives in one of NST LDS stages (A fragments, then W
// fragments, in their HBM fragment order; W4 stays packed). global_load_lds_dwordx4 moves a
// fragment per wave-load from HBM/L2 into LDS without touching registers, NST-1 steps ahead of the
// MFMAs, and the stream of steps runs across tile boundaries: the first steps of the next tile are
// in flight while the current tile finishes and stores its output.
//
// Operand K order. An MFMA contracts over 32 k; lanes 0..31 carry one 16-byte k chunk and lanes
// 32..63 another, and the sum does not care which chunks as long as both operands agree. A step
// has 8 chunks c = 4*(k64 half) + (16-byte group); sub-step f = 2p + kt2, lane half h use chunk
// c = 4*kt2 + 2*p + h. A lane's 16-byte W4 piece then holds the operands of sub-steps 2p (dwords
// 0,1) and 2p+1 (dwords 2,3), so one LDS read serves two sub-steps.
//
// DEEP (small wave tiles). With TM*TN MFMAs a sub-step there is too little matrix work between an
// LDS read and its use to hide the read, and a lone workgroup a CU has no other wave to run. The
// deep form reads the operands of a whole K step (all four sub-steps) into registers one step
// ahead of its MFMAs, double-buffered a step: one barrier a step at its top, behind it the loads
// for NST-1 steps ahead leave, the next step's operands are read from its stage and this step's
// MFMAs run from registers filled a step ago.
//
// D[n][m]: src0 = weight operand (lane: row n = l%32), src1 = activation operand (lane: row
// m = l%32); lane l, register e holds n = 8*(e/4) + 4*(l/32) + e%4, m = l%32.
#pragma once
#include <type_traits>

#include "iu8_gemm.h"

typedef int iu8_v16i __attribute__((ext_vector_type(16)));

// One tile of work: rows [mbase, mbase + BM) of the row map R against the 16-row weight tiles from
// nt0 of W (with row scales ws).
struct iu8_tile {
  iu8_rows R;
  int mbase, nt0;
  const iu8_u8 *W;
  const float *ws;
  int id;  // the tile's index in the launch (its arrival counter under a split of K)
  // The tile's K steps run from step `rot` of the workgroup's share round to rot - 1 (0 <= rot < steps of
  // the share). The int32 sum does not depend on the order; tiles that start at different depths do
  // not all ask the same memory channels for the same K at the same time.
  int rot = 0;
};

// Dense tile order of a persistent launch of G workgroups over gx x gy tiles. The hardware deals
// consecutive workgroup ids round-robin over the 8 XCDs (each with its own L2): in every round an
// XCD's G/8 workgroups take one run of consecutive tile ids, and ids walk M-fastest in groups of
// 8 row blocks, so co-resident workgroups share W columns and A rows in their L2.
static __device__ __forceinline__ void iu8_dense_tile_of(int id, int gx, int gy, int &bx, int &by) {
  constexpr int GM = 8;
  const int group = id / (GM * gx), first = group * GM, gm = min(GM, gy - first);
  const int rr = id - group * (GM * gx);
  by = first + rr % gm;
  bx = rr / gm;
}
static __device__ __forceinline__ bool iu8_dense_tile_at(int r, int gx, int gy, int &bx, int &by) {
  const int G = gridDim.x, w = blockIdx.x, total = gx * gy;
  const int id = (G & 7) == 0 ? ((r * 8 + (w & 7)) * (G >> 3) + (w >> 3)) : (w + r * G);
  if (id >= total) return false;
  iu8_dense_tile_of(id, gx, gy, bx, by);
  return true;
}

// The grouped launches' tile cells (the sparse forms, at least 128 x 256) hand a tile's epilogue scales over
// through LDS (below): their items are short in K (an expert's down projection: 12 steps) and many a
// workgroup. A dense launch has long tiles and often one a workgroup: there the hand-over measured 3 % slower.
template <bool SPARSE, int WMW, int WNW, int TM, int TN>
constexpr bool iu8_pf32_stashes() {
  return SPARSE && WMW * TM * 32 * WNW * TN * 32 >= 128 * 256;
}
// LDS bytes of a cell (what iu8_pf32_run declares, or expects from its caller): its stages and, where the
// cell stashes them (STASH: iu8_pf32_stashes), two sets of a tile's epilogue scales (BM + BN floats each)
// behind them.
template <bool W8, int WMW, int WNW, int TM, int TN, int STMAX, bool STASH = false>
constexpr int iu8_pf32_lds_bytes() {
  constexpr int STAGE = WMW * TM * 2 * 2048 + WNW * TN * 2 * (W8 ? 2048 : 1024);
  constexpr int NFIT = 160 * 1024 / STAGE;
  constexpr int NST = STMAX < 2 ? 2 : (STMAX < NFIT ? STMAX : (NFIT < 2 ? 2 : NFIT));
  return NST * STAGE + (STASH ? 2 * (WMW * TM * 32 + WNW * TN * 32) * 4 : 0);
}

// A split of K over gridDim.z (P, cnt not null): the workgroups of share z run steps [z*spb, (z+1)*spb)
// of every tile and hand their int32 partials over through memory, the last to arrive at a tile's
// counter sums the shares and runs the epilogue (the flush-free hand-over of iu8_common.h; the counter
// is left at zero).
//
// ARM (the A operand row-major, K bytes a row, rows through the tile's row map): a wave-load still
// lands one fragment in LDS in fragment order -- lane l fetches the 16 bytes of row l % 16, k chunk
// l / 16 -- from 16 rows' 64-byte runs instead of one contiguous KiB.
//
// SPARSE (tiles of a routed layer, often nearly empty): a wave whose 32-row blocks of the tile are
// all past the tile's rows, or all but the first, runs the K loop in a form with none, or one, of
// its TM row blocks -- the same loads, barriers and stage walk, a fraction of the MFMAs and LDS reads
// -- so such a tile costs its operand traffic instead of a full tile's matrix work.
//
// AQ (the per-token quantisation fused into the A-tile load): A is the bf16 activation matrix itself,
// row-major [M, K], and `as` holds the rows' scales (max(amax / 127, 1e-30), from a row-maximum pass
// or carried from the producer of the rows). The A fragments of a step cannot go to LDS by LDS-DMA
// then: each wave loads the bf16 pieces of its fragments into registers a step ahead (32 bytes a lane
// a fragment), turns them into codes by the law's own routine (iu8_code4_rcp: the bytes of the
// producer kernel) one step later and writes the fragment into its stage; the weights keep their
// LDS-DMA stream. One conversion a workgroup and step, whatever the columns of the tile.
template <bool W8, int WMW, int WNW, int TM, int TN, bool ACC, int STMAX, bool DEEP = false, bool SPARSE = false, bool ARM = false, bool EXT_LDS = false, bool AQ = false, class TileAt>
__device__ __forceinline__ void iu8_pf32_run(const iu8_u8 *__restrict__ A, const float *__restrict__ as,
                                             void *__restrict__ Cv, int N, int K, TileAt tile_at,
                                             int *__restrict__ P = nullptr, int *__restrict__ cnt = nullptr,
                                             iu8_u8 *ext_lds = nullptr) {
  // tile_at(r, t): fills the workgroup's r-th tile, false when it has none
  constexpr int NWAVE = WMW * WNW;
  constexpr int BMT = WMW * TM * 2, BNT = WNW * TN * 2;  // 16-row tiles a workgroup, both ways
  constexpr int WSTEP = W8 ? 2048 : 1024;                // bytes of a 16-row weight tile per K step
  constexpr int A_BYTES = BMT * 2048, W_BYTES = BNT * WSTEP, STAGE = A_BYTES + W_BYTES;
  // a wave moves whole 1-KiB fragments: wave w moves fragments w, w + NWAVE, ... of A and of W
  constexpr int A_FR = A_BYTES / 1024, W_FR = W_BYTES / 1024;
  constexpr int A_PER = (A_FR + NWAVE - 1) / NWAVE, W_PER = (W_FR + NWAVE - 1) / NWAVE;
  // wave-loads every wave issues a step (some issue one more); AQ: two 16-byte loads a fragment of A
  constexpr int PER = (AQ ? 2 : 1) * (A_FR / NWAVE) + W_FR / NWAVE;
  // as many stages as asked for and as fit the 160 KiB of LDS, at least two
  constexpr int NFIT = 160 * 1024 / STAGE;
  constexpr int NST = STMAX < 2 ? 2 : (STMAX < NFIT ? STMAX : (NFIT < 2 ? 2 : NFIT));
  // waves below these issue one more wave-load a step (a cell whose fragments do not divide by its waves)
  constexpr int A_X = A_FR % NWAVE, W_X = W_FR % NWAVE;
  static_assert((NST - 2) * (PER + (A_X > 0) + (W_X > 0)) <= 63, "the in-flight count fits s_waitcnt's vmcnt field");
  static_assert(!DEEP || NST >= 3, "the deep form reads a stage a step ahead of its MFMAs");
  static_assert(!(DEEP && SPARSE), "the sparse forms exist for the phased loop only");
  static_assert(!AQ || (!DEEP && !SPARSE && !ARM && A_FR % NWAVE == 0), "the fused-quant form: phased loop, whole A fragments a wave");
  // EXT_LDS: the stages live in the caller's LDS block (1-KiB aligned, iu8_pf32_lds_bytes of this cell),
  // for a kernel that runs two cells one after the other in the same memory
  iu8_u8 *smem;
  if constexpr (EXT_LDS) {
    smem = ext_lds;
  } else {
    __shared__ __attribute__((aligned(1024))) iu8_u8 own_lds[iu8_pf32_lds_bytes<W8, WMW, WNW, TM, TN, STMAX, iu8_pf32_stashes<SPARSE, WMW, WNW, TM, TN>()>()];
    smem = own_lds;
  }

  // The epilogue's scales of a tile (its rows' activation scales, its columns' weight scales in the
  // weight scales) are put in LDS when the load stream enters the tile, a tile ahead of their use:
  // fetched in the epilogue they were a dependent load or two (a gathered row's scale hangs on its
  // row_tok entry) in front of the first output, with both waves of every SIMD waiting on them -- some
  // 1.7 us an item, a tenth of an item of the routed down projection (K = 1536). Two sets: the tile being
  // computed and the one the stream is in.
  constexpr int BM = BMT * 16, BN = BNT * 16;
  float(*s_am)[BM] = (float(*)[BM])(smem + NST * STAGE);
  float(*s_wsu)[BN] = (float(*)[BN])(smem + NST * STAGE + 2 * BM * 4);

  // Opaque to the optimiser: a kernel that runs cells in a loop must not carry one cell's per-lane
  // addresses in registers through the other cell's K loop.
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WNW, wn = wave % WNW;
  const int ntiles = N >> 4, ksteps = K >> 7, ktiles = K >> 6;
  // this workgroup's share of the K steps
  const int Z = P != nullptr ? (int)gridDim.z : 1, z = P != nullptr ? (int)blockIdx.z : 0;
  const int spb = (ksteps + Z - 1) / Z;
  const int s_lo = min(z * spb, ksteps - 1), s_hi = max(min(ksteps, z * spb + spb), s_lo + 1);
  const bool share_empty = z * spb >= ksteps;  // more shares than steps: this one re-runs a step and adds nothing
  const int steps = s_hi - s_lo;
  __shared__ int s_last;

  // ---- the load stream: (tile L, step ls), NST-1 steps ahead of the MFMAs
  // Global -> LDS without registers: global_load_lds_dwordx4 writes lane l's 16 bytes at
  // (wave-uniform LDS base in m0) + 16*l, so one wave-load lands one fragment in fragment order.
  // Per lane: the 32-bit byte offset of its piece at K step 0 of the load stream's tile.
  iu8_tile L, Nx;  // the stream's tile and the one after it
  if (!tile_at(0, L)) return;
  int lr = 0, ls = s_lo;
  unsigned ga[A_PER], gw[W_PER], gaN[A_PER], gwN[W_PER];
  // AQ: the scale of this lane's row in every fragment, for the stream's tile and the one after it
  float qs[AQ ? A_PER : 1], qsN[AQ ? A_PER : 1];
  auto addr_of = [&](const iu8_tile &t, unsigned (&oa)[A_PER], unsigned (&ow)[W_PER], float (&os)[AQ ? A_PER : 1]) {
#pragma unroll
    for (int p = 0; p < A_PER; ++p) {
      const int f = min(p * NWAVE + wave, A_FR - 1);  // fragment (mt = f/2, kt2 = f%2) of the step
      // rows past the edge: the last one of the padded 16-row tile (the int8 operand is padded to whole tiles); the
      // fused-quant form reads the caller's bf16 rows and their scales, which hold exactly `rows` rows: the last live one
      const int mrow = t.mbase + (f >> 1) * 16 + (lane & 15);
      const int ar = iu8_arow(t.R, AQ ? min(mrow, t.R.rows - 1) : mrow);
      if constexpr (AQ) {  // bf16 rows: 2 bytes an element
        oa[p] = (unsigned)(((size_t)ar * K + (f & 1) * 64 + (lane >> 4) * 16) * 2);
        os[p] = as[ar];
      } else if constexpr (ARM) oa[p] = (unsigned)((size_t)ar * K + (f & 1) * 64 + (lane >> 4) * 16);
      else oa[p] = (unsigned)(((size_t)(ar >> 4) * ktiles + (f & 1)) * 1024 + ((ar & 15) + 16 * (lane >> 4)) * 16);
    }
#pragma unroll
    for (int p = 0; p < W_PER; ++p) {
      const int f = min(p * NWAVE + wave, W_FR - 1);
      const int nt = min(t.nt0 + f / (WSTEP / 1024), ntiles - 1);  // tiles past N: the last one
      ow[p] = (unsigned)((size_t)nt * ksteps * WSTEP + (f % (WSTEP / 1024)) * 1024 + lane * 16);
    }
  };
  addr_of(L, ga, gw, qs);
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) iu8_u8 *)smem;
  // (with fewer K steps a tile than the stream runs ahead, it would be more than one tile ahead of the MFMAs and
  // two sets would not do: such a launch fetches the scales in the epilogue)
  const bool stashed = iu8_pf32_stashes<SPARSE, WMW, WNW, TM, TN>() && steps >= NST + (DEEP ? 1 : 0);  // the stream's lead in steps (the deep form fetches a step ahead of its MFMAs), and one to spare
  // Rows in place: both tables come by LDS-DMA like the operands (a dword a lane, 64 consecutive entries a
  // wave-load), so nothing waits for them at the crossing. Gathered rows: the row's scale hangs on its
  // row_tok entry, an ordinary dependent load -- the crossing of such a tile waits for that entry anyway,
  // for the operand addresses.
  auto dma4 = [&](const void *base, unsigned off, unsigned lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(lds), "v"(off), "s"(base) : "memory", "m0");
  };
  auto stash_scales = [&](const iu8_tile &t, int set) {
    if (!stashed) return;
    const unsigned l_am = lds0 + NST * STAGE + set * BM * 4, l_ws = lds0 + NST * STAGE + 2 * BM * 4 + set * BN * 4;
    if (t.R.row_tok == nullptr) {
      if (wave < BM / 64) dma4(as, (unsigned)iu8_arow(t.R, min(t.mbase + tid, t.R.rows - 1)) * 4u, l_am + wave * 256);
    } else if (tid < BM) {
      s_am[set][tid] = as[iu8_arow(t.R, min(t.mbase + tid, t.R.rows - 1))];
    }
#pragma unroll
    for (int c0 = 0; c0 < BN; c0 += NWAVE * 64)
      if (c0 + tid < BN) dma4(t.ws, (unsigned)min(t.nt0 * 16 + c0 + tid, N - 1) * 4u, l_ws + (c0 + wave * 64) * 4);  // (a lane an entry: none past the set)
  };
  stash_scales(L, 0);
  // The next tile's descriptor and addresses (a gathered tile reads its row map for them) are
  // fetched a whole tile ahead, so the stream never waits for them when it crosses into that tile.
  bool haveN = tile_at(1, Nx);
  if (haveN) addr_of(Nx, gaN, gwN, qsN);
  // The load is written as asm: the compiler models an LDS-DMA load as touching both memories and
  // then drains every counter to zero at each later LDS read, which would serialise the operand
  // pipeline below. Its completion is tracked by hand (vmcnt, before the step's barrier).
  // m0 = LDS address of the wave's fragment; one wait state between the m0 write and its use.
  auto dma = [&](const iu8_u8 *base, unsigned off, unsigned lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds), "v"(off), "s"(base)
                 : "memory", "m0");
  };
  // AQ: the bf16 pieces of every fragment of A this wave owns (two 16-byte loads a fragment) and the
  // scale of their rows. Fragment p is loaded in phase p % 3 of a step, right behind the conversion of
  // the pieces it replaces, and converted a whole step later: a step of latency cover, one register
  // set. Loads return in order, so the compiler's own wait for a fragment's pieces also vouches for
  // every DMA issued before them.
  iu8_v4u aq[AQ ? A_PER : 1][2];
  float aq_sc[AQ ? A_PER : 1];
  auto step_k = [&]() {
    int kk = ls + L.rot;
    if (kk >= s_hi) kk -= s_hi - s_lo;
    return kk;
  };
  auto issue = [&](int stage) {  // the load stream's step -> LDS stage
    const unsigned sA = lds0 + stage * STAGE, sW = sA + A_BYTES;
    const int kk = step_k();
    const iu8_u8 *As = A + (size_t)kk * (ARM ? 128 : 2048), *Ws = L.W + (size_t)kk * WSTEP;
    if constexpr (!AQ) {
#pragma unroll
      for (int p = 0; p < A_PER; ++p)
        if (A_FR % NWAVE == 0 || p * NWAVE + wave < A_FR) dma(As, ga[p], sA + (p * NWAVE + wave) * 1024);
    }
#pragma unroll
    for (int p = 0; p < W_PER; ++p)
      if (W_FR % NWAVE == 0 || p * NWAVE + wave < W_FR) dma(Ws, gw[p], sW + (p * NWAVE + wave) * 1024);
  };
  auto aq_load = [&](int p) {  // fragment p of the load stream's step into registers
    if constexpr (AQ) {
      const iu8_u8 *As = A + (size_t)step_k() * 256;
      aq[p][0] = *(const iu8_v4u *)(As + ga[p]);
      aq[p][1] = *(const iu8_v4u *)(As + ga[p] + 16);
      aq_sc[p] = qs[p];
    }
  };
  auto aq_commit = [&](int p, int stage) {  // the pieces of fragment p -> codes -> the fragment in `stage`
    if constexpr (AQ) {
      const float sc = aq_sc[p], rcp = __fdiv_rn(1.f, sc);
      unsigned d[4];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const unsigned u0 = aq[p][h][2 * w], u1 = aq[p][h][2 * w + 1];
          d[h * 2 + w] = iu8_code4_rcp(__uint_as_float(u0 << 16), __uint_as_float(u0 & 0xFFFF0000u), __uint_as_float(u1 << 16),
                                       __uint_as_float(u1 & 0xFFFF0000u), sc, rcp);
        }
      *(iu8_v4u *)&smem[stage * STAGE + (p * NWAVE + wave) * 1024 + lane * 16] = iu8_v4u{d[0], d[1], d[2], d[3]};
    }
  };
  // phase ph of a step: the fragments p = ph, ph + 3, ... are converted into stage `cst`, then re-loaded
  auto aq_phase = [&](int ph, int cst) {
    if constexpr (AQ) {
#pragma unroll
      for (int p = ph; p < A_PER; p += 3) {
        aq_commit(p, cst);
        aq_load(p);
      }
    }
  };
  auto advance = [&]() {  // next step of the stream; past the last tile it keeps re-loading the last step
    if (++ls == s_hi) {
      if (haveN) {
        ++lr, ls = s_lo, L = Nx;
#pragma unroll
        for (int p = 0; p < A_PER; ++p) ga[p] = gaN[p];
#pragma unroll
        for (int p = 0; p < W_PER; ++p) gw[p] = gwN[p];
        if constexpr (AQ) {
#pragma unroll
          for (int p = 0; p < A_PER; ++p) qs[p] = qsN[p];
        }
        stash_scales(L, lr & 1);
        haveN = tile_at(lr + 1, Nx);
        if (haveN) addr_of(Nx, gaN, gwN, qsN);
      } else {
        ls = s_hi - 1;
      }
    }
  };
  // s_waitcnt vmcnt(n) [lgkmcnt(0)] (gfx9 encoding: vmcnt = imm[3:0] | imm[15:14] << 4, expcnt open)
  auto wait_vm = [&](auto n, bool lgkm0) {
    constexpr int NN = decltype(n)::value;
    if (lgkm0) __builtin_amdgcn_s_waitcnt((NN & 15) | ((NN >> 4) << 14) | (7 << 4) | (0 << 8));
    else __builtin_amdgcn_s_waitcnt((NN & 15) | ((NN >> 4) << 14) | (7 << 4) | (15 << 8));
  };
  // Loads that may still fly at a step's barrier: those of the newest NST-2 steps, counted with what
  // this wave issues a step.
  const int xtra = (wave < A_X) + (wave < W_X);
  auto wait_step = [&](bool lgkm0) {
    if constexpr (A_X == 0 && W_X == 0) {
      wait_vm(std::integral_constant<int, (NST - 2) * PER>{}, lgkm0);
    } else {
      if (xtra == 0) wait_vm(std::integral_constant<int, (NST - 2) * PER>{}, lgkm0);
      else if (xtra == 1) wait_vm(std::integral_constant<int, (NST - 2) * (PER + 1)>{}, lgkm0);
      else wait_vm(std::integral_constant<int, (NST - 2) * (PER + (A_X > 0) + (W_X > 0))>{}, lgkm0);
    }
  };

  // this lane's operand addresses inside a stage, at sub-step 0
  const int r32 = lane & 31, h = lane >> 5;
  // A: fragment (mt, kt2) at (mt*2 + kt2) KiB; piece (chunk*16 + row%16)
  const int a_lane = (((wm * TM * 2 + (r32 >> 4)) * 2) * 64 + h * 16 + (r32 & 15)) * 16;
  // W4: fragment nt at nt KiB; W8: the A form
  const int w_lane = W8 ? (((wn * TN * 2 + (r32 >> 4)) * 2) * 64 + h * 16 + (r32 & 15)) * 16
                        : ((wn * TN * 2 + (r32 >> 4)) * 64 + h * 16 + (r32 & 15)) * 16;

  // ---- the pipelined K loop. A step is four phases (sub-steps) f = 2p + kt2. Nothing is consumed
  // in the phase that fetched it: a phase's MFMAs multiply A operands read from LDS one phase
  // earlier (register set f&1) with W operands unpacked just in time from packed pieces read at
  // least one phase earlier (wpk[p]; 16-byte reads of consecutive lanes are free of bank conflicts,
  // 8-byte reads at this stride are not). The unpack of column tile j+1 issues while the MFMAs of
  // column tile j run. The step's one barrier sits before the last phase, whose operands are
  // already in registers: behind it the first operands of the next step are read from the next
  // stage, and the stage just drained is free for the loads of NST-1 steps ahead.
  iu8_v16i acc[TM][TN];
  iu8_v4i af[2][TM] = {};
  iu8_v4i wf[W8 ? 2 : 1][TN] = {};
  iu8_v4u wpk[2][W8 ? 1 : TN] = {};
  using Full = std::integral_constant<int, TM>;
  auto fetch_a = [&](const iu8_u8 *sA, int buf, int p, int kt2, auto nl) {  // the first nl row blocks
#pragma unroll
    for (int i = 0; i < decltype(nl)::value; ++i) af[buf][i] = *(const iu8_v4i *)&sA[a_lane + i * 4096 + kt2 * 1024 + p * 512];
  };
  auto fetch_w8 = [&](const iu8_u8 *sW, int buf, int p, int kt2) {  // W8: a whole operand a phase
    if constexpr (W8) {
#pragma unroll
      for (int j = 0; j < TN; ++j) wf[buf][j] = *(const iu8_v4i *)&sW[w_lane + j * 4096 + kt2 * 1024 + p * 512];
    }
  };
  auto fetch_w4 = [&](const iu8_u8 *sW, int p) {  // W4: the packed pieces of sub-steps 2p, 2p+1
    if constexpr (!W8) {
#pragma unroll
      for (int j = 0; j < TN; ++j) wpk[p][j] = *(const iu8_v4u *)&sW[w_lane + j * 2048 + p * 512];
    }
  };
  auto mfmas = [&](int buf, int p, int kt2, auto nl) {
    if constexpr (decltype(nl)::value > 0)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if constexpr (!W8) {
        const unsigned d0 = kt2 ? wpk[p][j].z : wpk[p][j].x, d1 = kt2 ? wpk[p][j].w : wpk[p][j].y;
        wf[0][j] = iu8_v4i{(int)((d0 << 4) & 0xF0F0F0F0u), (int)(d0 & 0xF0F0F0F0u), (int)((d1 << 4) & 0xF0F0F0F0u),
                           (int)(d1 & 0xF0F0F0F0u)};
      }
#pragma unroll
      for (int i = 0; i < decltype(nl)::value; ++i)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[W8 ? buf : 0][j], af[buf][i], acc[i][j], 0, 0, 0);
    }
  };
  // Instruction order inside a phase (the machine scheduler follows these groups): the phase's LDS
  // reads, the first column tile's unpack, then per column tile its MFMAs with the next one's unpack
  // issued behind them.
  constexpr int UNPK = W8 ? 0 : 6;  // VALU ops of one piece-half unpack
#define IU8_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define IU8_PHASE_ORDER(NDS, NM)                        \
  if constexpr ((NDS) > 0) IU8_SGB(0x100, NDS);         \
  if constexpr ((NM) > 0) {                             \
    if (UNPK) IU8_SGB(0x002, UNPK);                     \
    _Pragma("unroll") for (int j_ = 0; j_ < TN; ++j_) { \
      IU8_SGB(0x008, NM);                               \
      if (UNPK && j_ + 1 < TN) IU8_SGB(0x002, UNPK);    \
    }                                                   \
  }                                                     \
  __builtin_amdgcn_sched_barrier(0)

#pragma unroll
  for (int s0 = 0; s0 < NST - 1; ++s0) {
    issue(s0);
    if constexpr (AQ) {  // the last step issued here stays in registers for the first step's phases
#pragma unroll
      for (int p = 0; p < A_PER; ++p) aq_load(p);
      if (s0 < NST - 2) {
#pragma unroll
        for (int p = 0; p < A_PER; ++p) aq_commit(p, s0);
      }
    }
    advance();
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  wait_step(false);
  __builtin_amdgcn_s_barrier();
  // deep form: register sets of one whole step, [set][sub-step f = 2p + kt2]
  iu8_v4i afd[DEEP ? 2 : 1][DEEP ? 4 : 1][TM] = {};
  iu8_v4i wfd[DEEP && W8 ? 2 : 1][DEEP && W8 ? 4 : 1][TN] = {};
  iu8_v4u wpd[DEEP && !W8 ? 2 : 1][DEEP && !W8 ? 2 : 1][TN] = {};
  auto fetch_step = [&](const iu8_u8 *sA, int set) {  // all operands of the step in stage sA
    const iu8_u8 *sW = sA + A_BYTES;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
      for (int kt2 = 0; kt2 < 2; ++kt2) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
          afd[set][2 * p + kt2][i] = *(const iu8_v4i *)&sA[a_lane + i * 4096 + kt2 * 1024 + p * 512];
        if constexpr (W8) {
#pragma unroll
          for (int j = 0; j < TN; ++j)
            wfd[set][2 * p + kt2][j] = *(const iu8_v4i *)&sW[w_lane + j * 4096 + kt2 * 1024 + p * 512];
        }
      }
      if constexpr (!W8) {
#pragma unroll
        for (int j = 0; j < TN; ++j) wpd[set][p][j] = *(const iu8_v4u *)&sW[w_lane + j * 2048 + p * 512];
      }
    }
  };
  if constexpr (DEEP) {
    fetch_step(smem, 0);
  } else {
    fetch_a(smem, 0, 0, 0, Full{});
    fetch_w8(smem + A_BYTES, 0, 0, 0);
    fetch_w4(smem + A_BYTES, 0);
  }
  __builtin_amdgcn_sched_barrier(0);

  iu8_tile C = L;
  tile_at(0, C);
  int st = 0;  // stage of the MFMAs' step
  for (int r = 0;; ++r) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    if constexpr (DEEP) {
      auto mfma_step = [&](int set) {
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
              iu8_v4i wv;
              if constexpr (W8) {
                wv = wfd[set][2 * p + kt2][j];
              } else {
                const unsigned d0 = kt2 ? wpd[set][p][j].z : wpd[set][p][j].x, d1 = kt2 ? wpd[set][p][j].w : wpd[set][p][j].y;
                wv = iu8_v4i{(int)((d0 << 4) & 0xF0F0F0F0u), (int)(d0 & 0xF0F0F0F0u), (int)((d1 << 4) & 0xF0F0F0F0u),
                             (int)(d1 & 0xF0F0F0F0u)};
              }
#pragma unroll
              for (int i = 0; i < TM; ++i)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wv, afd[set][2 * p + kt2][i], acc[i][j], 0, 0, 0);
            }
      };
      auto deep_step = [&](int set) {  // the MFMAs of the step in register set `set`; the next step's into the other
        const int st1 = st == NST - 1 ? 0 : st + 1, stl = st == 0 ? NST - 1 : st - 1;
        // The stage of the step before this one was read two steps ago (the last barrier vouches for
        // every wave), so the loads for NST-1 steps ahead leave first; then the next step's fragments
        // must have landed: all but the newest NST-2 steps' loads.
        issue(stl);
        advance();
        wait_step(true);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        fetch_step(smem + st1 * STAGE, set ^ 1);
        mfma_step(set);
        st = st1;
      };
      int s = 0;
      for (; s + 2 <= steps; s += 2) {
        deep_step(0);
        deep_step(1);
      }
      if (s < steps) {  // an odd step count: one more step, then the sets are renamed back
        deep_step(0);
#pragma unroll
        for (int f = 0; f < 4; ++f) {
#pragma unroll
          for (int i = 0; i < TM; ++i) afd[0][f][i] = afd[1][f][i];
          if constexpr (W8) {
#pragma unroll
            for (int j = 0; j < TN; ++j) wfd[0][f][j] = wfd[1][f][j];
          }
        }
        if constexpr (!W8) {
#pragma unroll
          for (int p = 0; p < 2; ++p)
#pragma unroll
            for (int j = 0; j < TN; ++j) wpd[0][p][j] = wpd[1][p][j];
        }
      }
    } else {
      // the phased loop with the first `nl` of this wave's TM row blocks live
      auto run_steps = [&](auto nl) {
        constexpr int NL = decltype(nl)::value;
        constexpr int NW = NL > 0 ? TN : 0;  // weight reads a phase that has MFMAs
        for (int s = 0; s < steps; ++s) {
          const int st1 = st == NST - 1 ? 0 : st + 1, stl = st == 0 ? NST - 1 : st - 1;  // next, last
          const iu8_u8 *sA = smem + st * STAGE, *sW = sA + A_BYTES;
          const iu8_u8 *nA = smem + st1 * STAGE, *nW = nA + A_BYTES;
          // phase 0; the load stream's step leaves HBM for the stage drained last
          fetch_a(sA, 1, 0, 1, nl);
          if constexpr (NL > 0) {
            fetch_w8(sW, 1, 0, 1);
            fetch_w4(sW, 1);
          }
          // AQ: the pieces loaded a step ago become fragments of the stage NST-1 steps ahead (the one
          // this step's DMA of the weights is for... a step later: the loads ran one step behind it)
          const int cst = st + NST - 2 >= NST ? st - 2 : st + NST - 2;
          if constexpr (!AQ) issue(stl);
          aq_phase(0, cst);
          mfmas(0, 0, 0, nl);
          IU8_PHASE_ORDER(NL + NW, NL);
          // phase 1
          fetch_a(sA, 0, 1, 0, nl);
          if constexpr (NL > 0) fetch_w8(sW, 0, 1, 0);
          aq_phase(1, cst);
          mfmas(1, 0, 1, nl);
          IU8_PHASE_ORDER(NL + (W8 ? NW : 0), NL);
          // phase 2
          fetch_a(sA, 1, 1, 1, nl);
          if constexpr (NL > 0) fetch_w8(sW, 1, 1, 1);
          aq_phase(2, cst);
          // AQ: the weights' DMA leaves behind the step's last register load. The compiler counts its own
          // loads only, so its wait for a fragment's pieces asks for as many more of the oldest loads as
          // DMAs were issued since; in this order those are register loads of a step ago, not a fresh DMA.
          if constexpr (AQ) issue(stl);
          mfmas(0, 1, 0, nl);
          IU8_PHASE_ORDER(NL + (W8 ? NW : 0), NL);
          // phase 3, behind the barrier: every wave's reads of this stage are done and the next step's
          // fragments have landed. The next step may be another tile's first, with every row block
          // live: its first operands are read in full whatever this tile's form.
          wait_step(true);
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_sched_barrier(0);
          fetch_a(nA, 0, 0, 0, Full{});
          fetch_w8(nW, 0, 0, 0);
          fetch_w4(nW, 0);
          mfmas(1, 1, 1, nl);
          IU8_PHASE_ORDER(TM + TN, NL);
          advance();
          st = st1;
        }
      };
      int nlw = TM;
      if constexpr (SPARSE) {
        const int blocks = (min(C.R.rows - C.mbase, WMW * TM * 32) + 31) >> 5;
        nlw = max(0, min(TM, blocks - wm * TM));
      }
      if (!SPARSE || nlw >= 2 || TM == 1) run_steps(Full{});
      else if (nlw == 1) run_steps(std::integral_constant<int, 1>{});
      else run_steps(std::integral_constant<int, 0>{});
    }

    // ---- epilogue of tile C. The stage the last step drained is free (the barrier of that step's
    // last phase came after every wave's reads of it); the other stages hold the next tile's first
    // steps.
    const int M = C.R.rows;
    const int nq = h * 4;
    const int ncol0 = (C.nt0 + wn * TN * 2) * 16;  // first column of the wave tile
    if (Z > 1) {
      // ---- a share of K: the partial goes out straight through memory, the last share to arrive at
      // the tile's counter sums all of them in share order (exact in int32) and runs the epilogue
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = C.mbase + (wm * TM + i) * 32 + r32;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = ncol0 + j * 32 + g * 8 + nq;
            if (m >= M || n >= N) continue;
            const iu8_v4i v = share_empty ? iu8_v4i{0, 0, 0, 0}
                                          : iu8_v4i{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
            iu8_store_through(&P[((size_t)z * M + C.R.row0 + m) * N + n], v);
          }
      }
      iu8_stores_done();
      __builtin_amdgcn_s_barrier();
      if (tid == 0) s_last = (iu8_arrive(&cnt[C.id]) == Z - 1);
      wait_vm(std::integral_constant<int, 63>{}, true);
      __builtin_amdgcn_s_barrier();
      if (s_last) {
              if (tid == 0) __hip_atomic_store(&cnt[C.id], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        constexpr int BM = WMW * TM * 32, BN = WNW * TN * 32;
        const int nb = C.nt0 * 16, rows = min(BM, M - C.mbase), cols4 = min(BN, N - nb) >> 2;
        for (int idx = tid; idx < rows * cols4; idx += NWAVE * 64) {
          const int r = idx / cols4, m = C.mbase + r, n = nb + (idx - r * cols4) * 4;
          iu8_v4i sum = iu8_v4i{0, 0, 0, 0};
          for (int q = 0; q < Z; ++q) sum += iu8_load_through(&P[((size_t)q * M + C.R.row0 + m) * N + n]);
          const size_t crow = (size_t)(C.R.row0 + m) * N;
          if constexpr (ACC) {
            *(iu8_v4i *)((int *)Cv + crow + n) = sum;
          } else {
            const float am = as[iu8_arow(C.R, m)];
            const float4 w4 = *(const float4 *)(C.ws + n);
            const float u = W8 ? 1.f : 0.0625f;
            const unsigned lo = iu8_bf16_pack(iu8_epi(sum[0], am, w4.x * u), iu8_epi(sum[1], am, w4.y * u));
            const unsigned hi = iu8_bf16_pack(iu8_epi(sum[2], am, w4.z * u), iu8_epi(sum[3], am, w4.w * u));
            *(iu8_v2u *)((unsigned short *)Cv + crow + n) = iu8_v2u{lo, hi};
          }
        }
      }
    } else if constexpr (ACC) {
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = ncol0 + j * 32 + g * 8 + nq;
          if (n >= N) continue;
#pragma unroll
          for (int i = 0; i < TM; ++i) {
            const int m = C.mbase + (wm * TM + i) * 32 + r32;
            if (m >= M) continue;
            *(iu8_v4i *)((int *)Cv + (size_t)(C.R.row0 + m) * N + n) =
                iu8_v4i{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
          }
        }
    } else if constexpr (NWAVE * 32 * (64 + 16) > STAGE) {
      // A cell of few rows, whose stage is too small for the transposing form below: every lane stores
      // its 4 consecutive columns of a row (8 bytes; lane halves side by side) -- such a tile's output
      // is small.
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = C.mbase + (wm * TM + i) * 32 + r32;
        const float am = as[iu8_arow(C.R, min(m, M - 1))];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int n = ncol0 + j * 32 + g * 8 + nq;
            const float4 w4 = *(const float4 *)(C.ws + min(n, N - 4));
            const float u = W8 ? 1.f : 0.0625f;  // exact: a power of two
            const unsigned lo = iu8_bf16_pack(iu8_epi(acc[i][j][g * 4], am, w4.x * u), iu8_epi(acc[i][j][g * 4 + 1], am, w4.y * u));
            const unsigned hi = iu8_bf16_pack(iu8_epi(acc[i][j][g * 4 + 2], am, w4.z * u), iu8_epi(acc[i][j][g * 4 + 3], am, w4.w * u));
            if (m < M && n < N) *(iu8_v2u *)((unsigned short *)Cv + (size_t)(C.R.row0 + m) * N + n) = iu8_v2u{lo, hi};
          }
      }
    } else {
      // Through LDS: a lane holds 4 consecutive columns of one row, so direct stores would touch 32
      // rows with 16 bytes each. Each wave turns a block of 32 rows x CB*32 columns at a time into
      // row-major bf16 in its own LDS region (rows padded by 16 bytes) and stores whole row
      // segments, 16 bytes a lane.
      constexpr int CB = TN % 2 == 0 && NWAVE * 32 * (2 * 64 + 16) <= STAGE ? 2 : 1;  // 32-column tiles a block
      constexpr int ROWB = CB * 64 + 16, LPR = CB * 4, PIECES = 32 * LPR;
      static_assert(NWAVE * 32 * ROWB <= STAGE, "the epilogue region fits one stage");
      iu8_u8 *reg = smem + (st == 0 ? NST - 1 : st - 1) * STAGE + wave * (32 * ROWB);
      float am[TM];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        am[i] = stashed ? s_am[r & 1][(wm * TM + i) * 32 + r32] : as[iu8_arow(C.R, min(C.mbase + (wm * TM + i) * 32 + r32, M - 1))];
      // a column block's weight scales are read once, for all the wave's row blocks
#pragma unroll
      for (int jb = 0; jb < TN / CB; ++jb) {
        float4 wsu[CB][4];
#pragma unroll
        for (int jj = 0; jj < CB; ++jj)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float4 w4 = stashed ? *(const float4 *)&s_wsu[r & 1][wn * TN * 32 + jb * (CB * 32) + jj * 32 + g * 8 + nq]
                                      : *(const float4 *)(C.ws + min(ncol0 + jb * (CB * 32) + jj * 32 + g * 8 + nq, N - 4));
            const float u = W8 ? 1.f : 0.0625f;  // exact: a power of two
            wsu[jj][g] = float4{w4.x * u, w4.y * u, w4.z * u, w4.w * u};
          }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          if (C.mbase + (wm * TM + i) * 32 >= M) continue;  // a row block past the tile's rows (the whole wave)
#pragma unroll
          for (int jj = 0; jj < CB; ++jj) {
            const int j = jb * CB + jj;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const int nl = jj * 32 + g * 8 + nq;
              const float4 w4 = wsu[jj][g];
              const unsigned lo = iu8_bf16_pack(iu8_epi(acc[i][j][g * 4], am[i], w4.x), iu8_epi(acc[i][j][g * 4 + 1], am[i], w4.y));
              const unsigned hi = iu8_bf16_pack(iu8_epi(acc[i][j][g * 4 + 2], am[i], w4.z), iu8_epi(acc[i][j][g * 4 + 3], am[i], w4.w));
              *(iu8_v2u *)&reg[r32 * ROWB + nl * 2] = iu8_v2u{lo, hi};
            }
          }
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int q0 = 0; q0 < PIECES; q0 += 64) {
            const int q = q0 + lane, row = q / LPR, pc = q % LPR;
            const int mm = C.mbase + (wm * TM + i) * 32 + row, nn = ncol0 + jb * (CB * 32) + pc * 8;
            if ((PIECES % 64 == 0 || q < PIECES) && mm < M && nn < N)
              *(iu8_v4u *)((unsigned short *)Cv + (size_t)(C.R.row0 + mm) * N + nn) =
                  *(const iu8_v4u *)&reg[row * ROWB + pc * 16];
          }
          __builtin_amdgcn_wave_barrier();
        }
      }
    }
    if (!tile_at(r + 1, C)) break;
    // every wave is done with the epilogue region before the next step's loads land in that stage
    wait_vm(std::integral_constant<int, 63>{}, true);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
#undef IU8_PHASE_ORDER
#undef IU8_SGB
  wait_vm(std::integral_constant<int, 0>{}, true);
}
