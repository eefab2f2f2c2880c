// The expert-routed (MoE) form of the W4A8-iu8 linear for gfx950: the code object `moe_iu8`.
// The reference has no iu8 MoE (its grouped GEMM is MXFP4 x e4m3, crates/saber-kernels/hip/
// moe_grouped.hip); this object composes the reference's routing / tile / combine LAW
// (crates/saber-kernels/hip/moe_route.hip:1-24,108-329, crates/saber-kernels/src/moe.rs:691-865)
// with the iu8 GEMM contract (iu8_common.h) at 128 experts, top-8:
//
//   moe_iu8_route_topk8_sort_e128   logits bf16 [T,128] -> f32 softmax (IEEE-only exp) -> top-8,
//        the LOWER expert id wins a tie -> w = p * (1 / (sum > 0 ? sum : 1)), sum in k order ->
//        expert-major sort of the local experts [e_lo, e_lo + e_loc) into 16-row blocks, cut into
//        tiles of `tile_blocks` blocks. One launch: a workgroup routes 128 tokens and counts its
//        routes per expert; the last workgroup to arrive scans and places every route. No atomic
//        decides an output byte: a route's row = expert offset + earlier workgroups' count + its
//        rank among this workgroup's earlier tokens, i.e. token order.
//        Signature: crates/saber-kernels/src/abi.rs:354-374.
//   moe_iu8_grouped_w4_{dec,pf}_g{0,1}   per tile of the table: one expert's weights through
//        xptr[2e] (W4 fragments) / xptr[2e+1] (f32 row scales), activation rows gathered through
//        row_tok (g1: from token-major A fragments; g2: from row-major codes, the reference's form,
//        crates/saber-kernels/hip/moe_grouped.hip:67-74) or in place (g0: down), C rows at the tile's row0. `dec` streams the
//        weights for tiles of <= 16 rows (few tokens: HBM-bound), `pf` is the MFMA tile for tiles of
//        up to 256 rows of one expert. Signature: crates/saber-kernels/src/abi.rs:325-340 (p / cnt /
//        pmax are the split-K workspaces of the reference's cells; this object does not split).
//   moe_iu8_combine_bf16   out[t] = bf16(sum_k w[t,k] * f32(Y[pos(t,k)])), f32 adds in top-k order,
//        one rounding (crates/saber-kernels/hip/moe_route.hip:287-329; abi.rs:377-385).
#include "iu8_gemm.h"
#include "iu8_pf32.h"

#define MOE_E 128
#define MOE_TOPK 8
#define MOE_TPB 128
#define MOE_PTPB 32  // tokens a routing workgroup of the part launches (256 threads)
#define MOE_THREADS 1024
#define MOE_CHUNK 36864  // rows of the placement tables held in LDS at a time (144 KiB)

// e^x for x <= 0 from IEEE-rounded multiply / add / rint / ldexp only, so that every implementation of
// the router gives the same bits (the law of crates/saber-kernels/hip/moe_route.hip:43-57):
// n = rint(x * log2(e)); r = x - n * ln2 in two Cody-Waite pieces; e^r by the degree-7 Taylor
// polynomial in Horner form (coefficients 1/7! ... 1/2!, 1, 1 as f32 bit patterns); result * 2^n.
// x <= -80 or NaN gives 0.
static __device__ __forceinline__ float moe_exp_nonpos(float x) {
#pragma clang fp contract(off)
  constexpr unsigned LOG2E = 0x3FB8AA3Bu, LN2_HEAD = 0x3F317200u, LN2_TAIL = 0x35BFBE8Eu;
  constexpr unsigned TAYLOR[8] = {0x39500D01u, 0x3AB60B61u, 0x3C088889u, 0x3D2AAAABu, 0x3E2AAAABu, 0x3F000000u, 0x3F800000u, 0x3F800000u};
  if (!(x > -80.f)) return 0.f;
  const float n = __builtin_rintf(x * __uint_as_float(LOG2E));
  float r = x - n * __uint_as_float(LN2_HEAD);
  r = r - n * __uint_as_float(LN2_TAIL);
  float poly = __uint_as_float(TAYLOR[0]);
#pragma unroll
  for (int i = 1; i < 8; ++i) poly = poly * r + __uint_as_float(TAYLOR[i]);
  return __builtin_ldexpf(poly, (int)n);
}

// Lane exchanges inside a token's 8 lanes without the LDS crossbar's latency: DPP quad permutes for
// the partners xor 1 and xor 2, and the half-row mirror (lane i <-> 7 - i), which after those two
// brings in the other quad. Only for order-free reductions (max, arg-max under a total order).
#define MOE_DPP_XOR1 0xB1    // quad_perm [1,0,3,2]
#define MOE_DPP_XOR2 0x4E    // quad_perm [2,3,0,1]
#define MOE_DPP_MIRROR8 0x141  // row_half_mirror
template <int CTRL>
static __device__ __forceinline__ int moe_dpp(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xF, 0xF, false);
}
template <int CTRL>
static __device__ __forceinline__ float moe_dppf(float v) {
  return __int_as_float(moe_dpp<CTRL>(__float_as_int(v)));
}

// The layout's four scans over the experts (rows, tiles, touched experts, routes) in one pass: one round of
// shuffles and one pair of barriers for all four. base[] = the exclusive prefixes, total[] = the sums, in that order.
static __device__ __forceinline__ void moe_exscan4(int rows, int tiles, int touched, int routes, int (*s_wave4)[4],
                                                   int (&base)[4], int (&total)[4]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int v[4] = {rows, tiles, touched, routes};
  int x[4] = {rows, tiles, touched, routes};
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      const int y = __shfl_up(x[f], o, 64);
      if (lane >= o) x[f] += y;
    }
  }
  if (lane == 63) {
#pragma unroll
    for (int f = 0; f < 4; ++f) s_wave4[wave][f] = x[f];
  }
  __syncthreads();
#pragma unroll
  for (int f = 0; f < 4; ++f) base[f] = x[f] - v[f], total[f] = 0;
#pragma unroll
  for (int w = 0; w < MOE_THREADS / 64; ++w) {
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      const int t = s_wave4[w][f];
      if (w < wave) base[f] += t;
      total[f] += t;
    }
  }
  __syncthreads();
}

// The router's workgroup `blk` of `nblk` (128 tokens each). PART: the workgroup stops behind its own
// counts and ranks (phases 1 and 2); the tables are then laid out by moe_iu8_route_place_e128, a launch
// of its own in which every workgroup places its own routes.
// TPB: tokens a workgroup, on TPB * 8 threads. The one-launch forms take 128 (the layout's scans and its placement
// are written for 1,024 threads); the part launches take MOE_PTPB = 32: the routing of a token is a long chain of
// dependent arithmetic (128 exps, eight rounds of arg-max), and with 128 tokens a workgroup it runs four waves a
// SIMD deep on T / 128 CUs while the rest of the card idles or quantises -- 32 tokens a workgroup put a wave a SIMD
// on four times the CUs.
template <bool PART = false, int TPB = MOE_TPB>
static __device__ __forceinline__ void moe_route_body(
    const unsigned short *__restrict__ logits, int T, int e_lo, int e_loc, int tile_blocks, int with_shared,
    int *__restrict__ topk_ids, float *__restrict__ topk_w, int *__restrict__ route_pos, int *__restrict__ row_tok,
    int *__restrict__ row_route, int *__restrict__ tile_expert, int *__restrict__ tile_row0,
    int *__restrict__ tile_rows, int *__restrict__ expert_cnt, int *__restrict__ meta, int *__restrict__ blk_cnt,
    int *__restrict__ rank, int *__restrict__ arrive, const int nblk, const int blk) {
#pragma clang fp contract(off)
  constexpr int NTHR = TPB * MOE_TOPK;
  static_assert(PART || TPB == MOE_TPB, "the layout behind the routing runs on 1,024 threads");
  __shared__ __attribute__((aligned(16))) int s_ids[TPB * MOE_TOPK];
  __shared__ int s_part[MOE_THREADS / MOE_E][MOE_E];
  __shared__ int s_rows[MOE_CHUNK];
  __shared__ unsigned s_mask[MOE_E][TPB / 32];
  __shared__ int s_cnt[MOE_E];
  __shared__ int s_off[MOE_E], s_toff[MOE_E];
  __shared__ int s_wave[MOE_THREADS / 64][4];
  __shared__ int s_last;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t0 = blk * TPB;

  for (int e = tid; e < MOE_E; e += NTHR) s_cnt[e] = 0;
  for (int i = tid; i < MOE_E * (TPB / 32); i += NTHR) s_mask[i / (TPB / 32)][i % (TPB / 32)] = 0u;
  for (int i = tid; i < TPB * MOE_TOPK; i += NTHR) s_ids[i] = -1;
  __syncthreads();

  // ---- phase 1: 8 lanes a token (a wave = 8 tokens); lane group g owns experts [16g, 16g + 16).
  // Sum order: a group's 16 in index order, then the xor butterfly 4, 2, 1 over the 8 group sums.
  {
    const int g = lane & 7, tl = wave * 8 + (lane >> 3), t = t0 + tl;
    if (t < T) {
      float p[16];
      const iu8_v4u *src = (const iu8_v4u *)(logits + (size_t)t * MOE_E + g * 16);
      const iu8_v4u v0 = src[0], v1 = src[1];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        p[2 * w] = __uint_as_float(v0[w] << 16);
        p[2 * w + 1] = __uint_as_float(v0[w] & 0xFFFF0000u);
        p[8 + 2 * w] = __uint_as_float(v1[w] << 16);
        p[8 + 2 * w + 1] = __uint_as_float(v1[w] & 0xFFFF0000u);
      }
      float mx = p[0];
#pragma unroll
      for (int j = 1; j < 16; ++j) mx = fmaxf(mx, p[j]);
      mx = fmaxf(mx, moe_dppf<MOE_DPP_XOR1>(mx));
      mx = fmaxf(mx, moe_dppf<MOE_DPP_XOR2>(mx));
      mx = fmaxf(mx, moe_dppf<MOE_DPP_MIRROR8>(mx));
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        p[j] = moe_exp_nonpos(p[j] - mx);
        s = s + p[j];
      }
      // the sum's order is part of the law: partner xor 4 (a swizzle), then xor 2, then xor 1
      s = s + __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(s), 0x101F));
      s = s + moe_dppf<MOE_DPP_XOR2>(s);
      s = s + moe_dppf<MOE_DPP_XOR1>(s);
      const float inv = 1.f / s;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        float q = p[j] * inv;
        if (!__builtin_isfinite(q)) q = 0.f;
        p[j] = q;
      }
      float sel = 0.f, mine_w = 0.f;
      int mine_i = 0;
#pragma unroll
      for (int k = 0; k < MOE_TOPK; ++k) {
        float bv = p[0];
        int bj = 0;
#pragma unroll
        for (int j = 1; j < 16; ++j)
          if (p[j] > bv) {  // strict: the lower index keeps a tie
            bv = p[j];
            bj = j;
          }
        int bi = g * 16 + bj;
        auto take = [&](float ov, int oi) {
          if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
          }
        };
        take(moe_dppf<MOE_DPP_XOR1>(bv), moe_dpp<MOE_DPP_XOR1>(bi));
        take(moe_dppf<MOE_DPP_XOR2>(bv), moe_dpp<MOE_DPP_XOR2>(bi));
        take(moe_dppf<MOE_DPP_MIRROR8>(bv), moe_dpp<MOE_DPP_MIRROR8>(bi));
        if ((bi >> 4) == g) {
#pragma unroll
          for (int j = 0; j < 16; ++j)
            if (j == (bi & 15)) p[j] = -1.f;  // probabilities are >= 0
        }
        if (k == g) {
          mine_w = bv;
          mine_i = bi;
        }
        sel = sel + bv;  // k order
      }
      const float scale = 1.f / (sel > 0.f ? sel : 1.f);
      // lane g of the token's group holds route k = g
      topk_ids[(size_t)t * MOE_TOPK + g] = mine_i;
      topk_w[(size_t)t * MOE_TOPK + g] = mine_w * scale;
      s_ids[tl * MOE_TOPK + g] = mine_i;
    }
  }
  __syncthreads();

  // ---- phase 2: this workgroup's per-expert counts and each route's rank among the earlier
  // tokens of this workgroup routed to the same expert (a token's experts are distinct): a bit a
  // token in the expert's 128-bit mask, the rank is the count of the bits below the token's
  for (int i = tid; i < TPB * MOE_TOPK; i += NTHR) {
    const int e = s_ids[i], le = e - e_lo, tl = i / MOE_TOPK;
    if (e >= 0 && le >= 0 && le < e_loc) atomicOr(&s_mask[le][tl >> 5], 1u << (tl & 31));
  }
  __syncthreads();
  for (int i = tid; i < TPB * MOE_TOPK; i += NTHR) {
    const int e = s_ids[i], le = e - e_lo, tl = i / MOE_TOPK;
    if (e < 0 || le < 0 || le >= e_loc) continue;
    int rk = 0;
#pragma unroll
    for (int w = 0; w < TPB / 32; ++w) {
      const unsigned m = s_mask[le][w];
      rk += __popc(w < (tl >> 5) ? m : w == (tl >> 5) ? m & ((1u << (tl & 31)) - 1u) : 0u);
    }
    rank[(size_t)t0 * MOE_TOPK + i] = rk;
  }
  for (int e = tid; e < e_loc; e += NTHR) {
    int c = 0;
#pragma unroll
    for (int w = 0; w < TPB / 32; ++w) c += __popc(s_mask[e][w]);
    s_cnt[e] = c;
  }
  __syncthreads();
  // A lone workgroup (up to 128 tokens) is its own last arriver: its counts are the totals, its
  // routes' bases are zero, and no hand-over through memory is needed.
  if constexpr (PART) {
    // (also with one workgroup: the placement launch sums the counts whatever their number, and a launch that
    // ends here holds none of the layout's LDS -- 144 KiB of row tables that would leave one workgroup a CU to
    // the quantising workgroups of the same launch)
    for (int e = tid; e < e_loc; e += NTHR) blk_cnt[(size_t)blk * e_loc + e] = s_cnt[e];
    return;
  }
  const bool solo = nblk == 1;
  if (!solo) {
    for (int e = tid; e < e_loc; e += MOE_THREADS) blk_cnt[(size_t)blk * e_loc + e] = s_cnt[e];
    __syncthreads();
    if (tid == 0) {
      __threadfence();
      s_last = atomicAdd(arrive, 1) == nblk - 1;
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();  // acquire: every workgroup's topk_ids, rank and blk_cnt
    if (tid == 0) *arrive = 0;
  }

  // ---- phase 3 (the last workgroup): totals, each workgroup's base, offsets, tiles, placement.
  // It works alone, so its time is load latency: eight threads an expert scan an eighth of the
  // workgroups' counts each, loads in batches of 8.
  if (solo) {
    for (int e = tid; e < e_loc; e += MOE_THREADS) expert_cnt[e] = s_cnt[e];
  } else {
    constexpr int PARTS = MOE_THREADS / MOE_E;
    const int e = tid % MOE_E, part = tid / MOE_E;
    const int chunk = (nblk + PARTS - 1) / PARTS, b_lo = min(part * chunk, nblk), b_hi = min(b_lo + chunk, nblk);
    int sum = 0;
    if (e < e_loc)
      for (int b0 = b_lo; b0 < b_hi; b0 += 8) {
        int c[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) c[u] = b0 + u < b_hi ? __builtin_nontemporal_load(&blk_cnt[(size_t)(b0 + u) * e_loc + e]) : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += c[u];
      }
    s_part[part][e] = sum;
    __syncthreads();
    int run = 0, all = 0;
#pragma unroll
    for (int q = 0; q < PARTS; ++q) {
      const int v = s_part[q][e];
      run += q < part ? v : 0;
      all += v;
    }
    if (e < e_loc) {
      for (int b0 = b_lo; b0 < b_hi; b0 += 8) {
        int c[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) c[u] = b0 + u < b_hi ? __builtin_nontemporal_load(&blk_cnt[(size_t)(b0 + u) * e_loc + e]) : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (b0 + u < b_hi) {
            blk_cnt[(size_t)(b0 + u) * e_loc + e] = run;
            run += c[u];
          }
      }
      if (part == 0) {
        s_cnt[e] = all;
        expert_cnt[e] = all;
      }
    }
  }
  __syncthreads();
  const int G = tile_blocks, TR = 16 * tile_blocks;
  int my_rows = 0, my_tiles = 0, my_touched = 0, my_routes = 0;
  if (tid < e_loc) {
    const int c = s_cnt[tid], nb = (c + 15) / 16;
    my_rows = nb * 16;
    my_tiles = (nb + G - 1) / G;
    my_touched = c > 0;
    my_routes = c;
  }
  int sbase[4], stotal[4];
  moe_exscan4(my_rows, my_tiles, my_touched, my_routes, s_wave, sbase, stotal);
  const int rbase = sbase[0], tbase = sbase[1];
  const int rows_total = stotal[0], tiles_total = stotal[1], touched_total = stotal[2], routes_total = stotal[3];
  if (tid < e_loc) {
    s_off[tid] = rbase;
    s_toff[tid] = tbase;
  }
  __syncthreads();
  const int sh_row0 = rows_total;
  const int sh_blocks = with_shared ? (T + 15) / 16 : 0;
  const int sh_tiles = (sh_blocks + G - 1) / G;
  if (tid == 0) {
    meta[0] = tiles_total + sh_tiles;
    meta[1] = rows_total + sh_blocks * 16;
    meta[2] = with_shared ? sh_row0 : -1;
    meta[3] = routes_total;
    meta[4] = touched_total;
    meta[5] = rows_total;
  }
  for (int e = tid; e < e_loc; e += MOE_THREADS) {
    const int c = s_cnt[e], nb = (c + 15) / 16, nt = (nb + G - 1) / G;
    for (int j = 0; j < nt; ++j) {
      tile_expert[s_toff[e] + j] = e;
      tile_row0[s_toff[e] + j] = s_off[e] + j * TR;
      tile_rows[s_toff[e] + j] = min(TR, c - j * TR);
    }
  }
  for (int j = tid; j < sh_tiles; j += MOE_THREADS) {
    tile_expert[tiles_total + j] = e_loc;
    tile_row0[tiles_total + j] = sh_row0 + j * TR;
    tile_rows[tiles_total + j] = min(TR, T - j * TR);
  }
  for (int r = tid; r < sh_blocks * 16; r += MOE_THREADS) {
    row_tok[sh_row0 + r] = r < T ? r : -1;
    row_route[sh_row0 + r] = -1;
  }
  __syncthreads();  // every expert's blk_cnt bases are written
  // Placement. A route's row is a scattered 4-byte store, and one workgroup scattering every route
  // straight to memory is bound by that (about 3 ns a route). So the row tables are built in LDS, a
  // chunk of MOE_CHUNK rows at a time (every slot starts as a pad, -1; each pass walks all routes
  // and keeps those that land in the chunk), and go out in whole lines.
  const int R = T * MOE_TOPK;
  for (int c0 = 0; c0 < rows_total; c0 += MOE_CHUNK) {
    const int cn = min(MOE_CHUNK, rows_total - c0);
    for (int i = tid; i < cn; i += MOE_THREADS) s_rows[i] = -1;
    __syncthreads();
    for (int r0 = tid; r0 < R; r0 += 16 * MOE_THREADS) {
      int e[16], rk[16], base[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int r = r0 + u * MOE_THREADS;
        e[u] = r < R ? __builtin_nontemporal_load(&topk_ids[r]) : -1;
        rk[u] = r < R ? __builtin_nontemporal_load(&rank[r]) : 0;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int r = r0 + u * MOE_THREADS, le = e[u] - e_lo;
        base[u] = (!solo && r < R && le >= 0 && le < e_loc) ? blk_cnt[(size_t)(r / MOE_TOPK / MOE_TPB) * e_loc + le] : 0;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int r = r0 + u * MOE_THREADS, le = e[u] - e_lo;
        if (r >= R) continue;
        const bool local = le >= 0 && le < e_loc;
        const int p = local ? s_off[le] + base[u] + rk[u] : -1;
        if (c0 == 0) route_pos[r] = p;
        if (local && p >= c0 && p < c0 + cn) s_rows[p - c0] = r;
      }
    }
    __syncthreads();
    for (int i = tid; i < cn; i += MOE_THREADS) {
      const int r = s_rows[i];
      row_route[c0 + i] = r;
      row_tok[c0 + i] = r < 0 ? -1 : r / MOE_TOPK;
    }
    __syncthreads();
  }
  if (rows_total == 0)  // no local route at all: the positions still have to be written
    for (int r = tid; r < R; r += MOE_THREADS) route_pos[r] = -1;
}
extern "C" __global__ __launch_bounds__(MOE_THREADS) void moe_iu8_route_topk8_sort_e128(
    const unsigned short *__restrict__ logits, int T, int e_lo, int e_loc, int tile_blocks, int with_shared,
    int *__restrict__ topk_ids, float *__restrict__ topk_w, int *__restrict__ route_pos, int *__restrict__ row_tok,
    int *__restrict__ row_route, int *__restrict__ tile_expert, int *__restrict__ tile_row0,
    int *__restrict__ tile_rows, int *__restrict__ expert_cnt, int *__restrict__ meta, int *__restrict__ blk_cnt,
    int *__restrict__ rank, int *__restrict__ arrive) {
  moe_route_body(logits, T, e_lo, e_loc, tile_blocks, with_shared, topk_ids, topk_w, route_pos, row_tok, row_route,
                 tile_expert, tile_row0, tile_rows, expert_cnt, meta, blk_cnt, rank, arrive, gridDim.x, blockIdx.x);
}

extern "C" __global__ __launch_bounds__(MOE_PTPB * MOE_TOPK) void moe_iu8_route_part_topk8_sort_e128(
    const unsigned short *__restrict__ logits, int T, int e_lo, int e_loc, int tile_blocks, int with_shared,
    int *__restrict__ topk_ids, float *__restrict__ topk_w, int *__restrict__ route_pos, int *__restrict__ row_tok,
    int *__restrict__ row_route, int *__restrict__ tile_expert, int *__restrict__ tile_row0,
    int *__restrict__ tile_rows, int *__restrict__ expert_cnt, int *__restrict__ meta, int *__restrict__ blk_cnt,
    int *__restrict__ rank, int *__restrict__ arrive) {
  moe_route_body<true, MOE_PTPB>(logits, T, e_lo, e_loc, tile_blocks, with_shared, topk_ids, topk_w, route_pos, row_tok, row_route,
                                 tile_expert, tile_row0, tile_rows, expert_cnt, meta, blk_cnt, rank, arrive, gridDim.x, blockIdx.x);
}

// The tables behind moe_iu8_route*_part_*: workgroup b (of ceil(T / 128), the part launch's routing
// workgroups) sums the workgroups' per-expert counts -- every workgroup the totals, and the counts of
// the workgroups in front of it as its own base -- lays out the experts' offsets like the one-launch
// router, and places its own 1,024 routes; workgroup 0 also writes the tile table, the counts, meta,
// the pad rows and a shared expert's rows. No workgroup waits for another: with more than one routing
// workgroup the one-launch form's last arriver lays out and places everything alone (4,096 tokens:
// 22 of its 38 us). Same tables: a route's row is the same sum. Kernarg list of the router (logits,
// topk_w and arrive are not touched). grid [ceil(T / 128), 1, 1].
extern "C" __global__ __launch_bounds__(MOE_THREADS) void moe_iu8_route_place_e128(
    const unsigned short *__restrict__ logits, int T, int e_lo, int e_loc, int tile_blocks, int with_shared,
    int *__restrict__ topk_ids, float *__restrict__ topk_w, int *__restrict__ route_pos, int *__restrict__ row_tok,
    int *__restrict__ row_route, int *__restrict__ tile_expert, int *__restrict__ tile_row0,
    int *__restrict__ tile_rows, int *__restrict__ expert_cnt, int *__restrict__ meta, int *__restrict__ blk_cnt,
    int *__restrict__ rank, int *__restrict__ arrive) {
  constexpr int PARTS = MOE_THREADS / MOE_E;
  __shared__ int s_all[PARTS][MOE_E], s_mine[PARTS][MOE_E];
  __shared__ int s_cnt[MOE_E], s_base[MOE_E], s_off[MOE_E], s_toff[MOE_E];
  __shared__ int s_wave[MOE_THREADS / 64][4];
  // the part launch counted and ranked in blocks of MOE_PTPB tokens: SUB of them make this workgroup's 128 tokens
  constexpr int SUB = MOE_TPB / MOE_PTPB;
  static_assert(SUB <= PARTS, "a thread group a sub-block");
  __shared__ int s_sub[SUB][MOE_E];
  const int tid = threadIdx.x, nblk = (T + MOE_PTPB - 1) / MOE_PTPB, blk = blockIdx.x * SUB;
  // this thread's route: its expert and rank are requested now, beside the count table, not behind the scans
  const int r = blockIdx.x * (MOE_TPB * MOE_TOPK) + tid;
  const bool mine = r < T * MOE_TOPK;
  const int my_e = mine ? topk_ids[r] : -1, my_rank = mine ? rank[r] : 0;
  {
    const int e = tid % MOE_E, part = tid / MOE_E;
    if (part < SUB) s_sub[part][e] = (e < e_loc && blk + part < nblk) ? blk_cnt[(size_t)(blk + part) * e_loc + e] : 0;
    const int chunk = (nblk + PARTS - 1) / PARTS, b_lo = min(part * chunk, nblk), b_hi = min(b_lo + chunk, nblk);
    int all = 0, mine = 0;
    if (e < e_loc)
      for (int b0 = b_lo; b0 < b_hi; b0 += 8) {
        int c[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) c[u] = b0 + u < b_hi ? blk_cnt[(size_t)(b0 + u) * e_loc + e] : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          all += c[u];
          mine += b0 + u < blk ? c[u] : 0;
        }
      }
    s_all[part][e] = all;
    s_mine[part][e] = mine;
    __syncthreads();
    if (part == 0) {
      int a = 0, m = 0;
#pragma unroll
      for (int q = 0; q < PARTS; ++q) {
        a += s_all[q][e];
        m += s_mine[q][e];
      }
      s_cnt[e] = e < e_loc ? a : 0;
      s_base[e] = m;
    }
    __syncthreads();
  }
  const int G = tile_blocks, TR = 16 * tile_blocks;
  int my_rows = 0, my_tiles = 0, my_touched = 0, my_routes = 0;
  if (tid < e_loc) {
    const int c = s_cnt[tid], nb = (c + 15) / 16;
    my_rows = nb * 16;
    my_tiles = (nb + G - 1) / G;
    my_touched = c > 0;
    my_routes = c;
  }
  int sbase[4], stotal[4];
  moe_exscan4(my_rows, my_tiles, my_touched, my_routes, s_wave, sbase, stotal);
  const int rbase = sbase[0], tbase = sbase[1];
  const int rows_total = stotal[0], tiles_total = stotal[1], touched_total = stotal[2], routes_total = stotal[3];
  if (tid < e_loc) {
    s_off[tid] = rbase;
    s_toff[tid] = tbase;
  }
  __syncthreads();
  if (blockIdx.x == 0) {
    const int sh_row0 = rows_total;
    const int sh_blocks = with_shared ? (T + 15) / 16 : 0;
    const int sh_tiles = (sh_blocks + G - 1) / G;
    if (tid == 0) {
      meta[0] = tiles_total + sh_tiles;
      meta[1] = rows_total + sh_blocks * 16;
      meta[2] = with_shared ? sh_row0 : -1;
      meta[3] = routes_total;
      meta[4] = touched_total;
      meta[5] = rows_total;
    }
    for (int e = tid; e < e_loc; e += MOE_THREADS) {
      const int c = s_cnt[e], nb = (c + 15) / 16, nt = (nb + G - 1) / G;
      expert_cnt[e] = c;
      for (int j = 0; j < nt; ++j) {
        tile_expert[s_toff[e] + j] = e;
        tile_row0[s_toff[e] + j] = s_off[e] + j * TR;
        tile_rows[s_toff[e] + j] = min(TR, c - j * TR);
      }
      for (int i = c; i < nb * 16; ++i) {  // the pad rows behind the expert's routes
        row_tok[s_off[e] + i] = -1;
        row_route[s_off[e] + i] = -1;
      }
    }
    for (int j = tid; j < sh_tiles; j += MOE_THREADS) {
      tile_expert[tiles_total + j] = e_loc;
      tile_row0[tiles_total + j] = sh_row0 + j * TR;
      tile_rows[tiles_total + j] = min(TR, T - j * TR);
    }
    for (int r = tid; r < sh_blocks * 16; r += MOE_THREADS) {
      row_tok[sh_row0 + r] = r < T ? r : -1;
      row_route[sh_row0 + r] = -1;
    }
  }
  if (mine) {  // this workgroup's routes: a thread a route
    const int le = my_e - e_lo;
    const bool local = le >= 0 && le < e_loc;
    int p = -1;
    if (local) {  // the experts' offset, the routes of the blocks in front of this route's 32-token block, its rank there
      p = s_off[le] + s_base[le] + my_rank;
#pragma unroll
      for (int j = 0; j + 1 < SUB; ++j) p += j < tid / (MOE_PTPB * MOE_TOPK) ? s_sub[j][le] : 0;
    }
    route_pos[r] = p;
    if (local) {
      row_route[p] = r;
      row_tok[p] = r / MOE_TOPK;
    }
  }
}

// The router and the tokens' quantisation in one launch: the two do not depend on each other, so the
// first ceil(T / 128) workgroups route and the ones behind them quantise the tokens (x bf16 [T, k] ->
// codes + scale[t]; macaq_i8.h:10-13, one 16-element group a thread, k <= 16,384), a row on 256, 512
// or 1,024 threads by its length, so 4, 2 or 1 rows a workgroup. With few tokens a layer's time is
// its launches; with many the router's tail (one workgroup lays out the tables) runs beside the
// quantisation instead of in front of it. Codes in the A fragment order (RM false, for the streaming
// cell) or row-major (RM true, for the MFMA cells' gather). grid [ceil(T/128) + ceil(T / rows a
// workgroup), 1, 1].
template <bool RM>
static __device__ __forceinline__ void moe_routeq_body(
    const unsigned short *__restrict__ logits, int T, int e_lo, int e_loc, int tile_blocks, int with_shared,
    int *__restrict__ topk_ids, float *__restrict__ topk_w, int *__restrict__ route_pos, int *__restrict__ row_tok,
    int *__restrict__ row_route, int *__restrict__ tile_expert, int *__restrict__ tile_row0,
    int *__restrict__ tile_rows, int *__restrict__ expert_cnt, int *__restrict__ meta, int *__restrict__ blk_cnt,
    int *__restrict__ rank, int *__restrict__ arrive, const unsigned short *__restrict__ x,
    unsigned char *__restrict__ q, float *__restrict__ scale, int k) {
#pragma clang fp contract(off)
  const int nblk = (T + MOE_TPB - 1) / MOE_TPB;
  if ((int)blockIdx.x < nblk) {
    moe_route_body<false>(logits, T, e_lo, e_loc, tile_blocks, with_shared, topk_ids, topk_w, route_pos, row_tok, row_route,
                          tile_expert, tile_row0, tile_rows, expert_cnt, meta, blk_cnt, rank, arrive, nblk, blockIdx.x);
    return;
  }
  __shared__ float s_max[MOE_THREADS / 64];
  const int G = k >> 4, span = G <= 256 ? 256 : G <= 512 ? 512 : 1024;  // threads a row
  const int sub = threadIdx.x / span, g = threadIdx.x - sub * span;
  const int row = ((int)blockIdx.x - nblk) * (MOE_THREADS / span) + sub;
  const bool mine = row < T && g < G;
  float v[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) v[j] = 0.f;
  if (mine) {
    const unsigned short *xr = x + (size_t)row * k + g * 16;
    const iu8_v4u lo = *(const iu8_v4u *)xr, hi = *(const iu8_v4u *)(xr + 8);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      v[2 * w] = __uint_as_float(lo[w] << 16);
      v[2 * w + 1] = __uint_as_float(lo[w] & 0xFFFF0000u);
      v[8 + 2 * w] = __uint_as_float(hi[w] << 16);
      v[8 + 2 * w + 1] = __uint_as_float(hi[w] & 0xFFFF0000u);
    }
  }
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(v[j]));
  amax = iu8_wave_max_nonneg(amax);
  if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  const int w0 = sub * (span >> 6);  // the waves of this row
  amax = s_max[w0];
  for (int w = 1; w < (span >> 6); ++w) amax = fmaxf(amax, s_max[w0 + w]);
  const float sc = fmaxf(__fdiv_rn(amax, 127.f), 1e-30f), rcp = __fdiv_rn(1.f, sc);
  if (g == 0 && row < T) scale[row] = sc;
  if (mine) {
    unsigned d[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) d[w] = iu8_code4_rcp(v[w * 4], v[w * 4 + 1], v[w * 4 + 2], v[w * 4 + 3], sc, rcp);
    if constexpr (RM) {
      *(iu8_v4u *)(q + (size_t)row * k + g * 16) = iu8_v4u{d[0], d[1], d[2], d[3]};
    } else {
      // fragment (row / 16, k / 64): 1 KiB; the 16 bytes of (row % 16, k chunk (g & 3)) at (row % 16 + 16 * chunk) * 16
      *(iu8_v4u *)(q + ((size_t)(row >> 4) * (k >> 6) + (g >> 2)) * 1024 + (g & 3) * 256 + (row & 15) * 16) =
          iu8_v4u{d[0], d[1], d[2], d[3]};
    }
  }
}
#define MOE_ROUTEQ(name, RM)                                                                                                \
  extern "C" __global__ __launch_bounds__(MOE_THREADS) void name(                                                      \
      const unsigned short *__restrict__ logits, int T, int e_lo, int e_loc, int tile_blocks, int with_shared,          \
      int *__restrict__ topk_ids, float *__restrict__ topk_w, int *__restrict__ route_pos, int *__restrict__ row_tok,   \
      int *__restrict__ row_route, int *__restrict__ tile_expert, int *__restrict__ tile_row0,                          \
      int *__restrict__ tile_rows, int *__restrict__ expert_cnt, int *__restrict__ meta, int *__restrict__ blk_cnt,     \
      int *__restrict__ rank, int *__restrict__ arrive, const unsigned short *__restrict__ x,                           \
      unsigned char *__restrict__ q, float *__restrict__ scale, int k) {                                                \
    moe_routeq_body<RM>(logits, T, e_lo, e_loc, tile_blocks, with_shared, topk_ids, topk_w, route_pos, row_tok,               \
                        row_route, tile_expert, tile_row0, tile_rows, expert_cnt, meta, blk_cnt, rank, arrive, x, q,    \
                        scale, k);                                                                                      \
  }
MOE_ROUTEQ(moe_iu8_routeq_topk8_sort_e128, false)
MOE_ROUTEQ(moe_iu8_routeq_rm_topk8_sort_e128, true)
#undef MOE_ROUTEQ
// The part form of the same launch (above 128 tokens, row-major codes): workgroups of 256 threads, the first
// ceil(T / 32) route 32 tokens each (moe_route_body), each of the T behind them quantises one token row, a thread
// up to four 16-element groups (k <= 16,384). grid [ceil(T / 32) + T, 1, 1]; moe_iu8_route_place_e128 follows.
extern "C" __global__ __launch_bounds__(MOE_PTPB * MOE_TOPK) void moe_iu8_routeq_rm_part_topk8_sort_e128(
    const unsigned short *__restrict__ logits, int T, int e_lo, int e_loc, int tile_blocks, int with_shared,
    int *__restrict__ topk_ids, float *__restrict__ topk_w, int *__restrict__ route_pos, int *__restrict__ row_tok,
    int *__restrict__ row_route, int *__restrict__ tile_expert, int *__restrict__ tile_row0,
    int *__restrict__ tile_rows, int *__restrict__ expert_cnt, int *__restrict__ meta, int *__restrict__ blk_cnt,
    int *__restrict__ rank, int *__restrict__ arrive, const unsigned short *__restrict__ x,
    unsigned char *__restrict__ q, float *__restrict__ scale, int k) {
#pragma clang fp contract(off)
  constexpr int NTHR = MOE_PTPB * MOE_TOPK, NG = 4;
  const int nblk = (T + MOE_PTPB - 1) / MOE_PTPB;
  if ((int)blockIdx.x < nblk) {
    moe_route_body<true, MOE_PTPB>(logits, T, e_lo, e_loc, tile_blocks, with_shared, topk_ids, topk_w, route_pos, row_tok, row_route,
                                   tile_expert, tile_row0, tile_rows, expert_cnt, meta, blk_cnt, rank, arrive, nblk, blockIdx.x);
    return;
  }
  __shared__ float s_max[NTHR / 64];
  const int row = (int)blockIdx.x - nblk, tid = threadIdx.x, G = k >> 4;
  if (row >= T) return;
  const unsigned short *xr = x + (size_t)row * k;
  // the row's pieces are requested all at once and stay packed as they came; groups past the row's end are zeros
  unsigned pk[NG][8];
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int g = tid + i * NTHR;
    iu8_v4u lo = {0u, 0u, 0u, 0u}, hi = {0u, 0u, 0u, 0u};
    if (g < G) lo = *(const iu8_v4u *)(xr + (unsigned)(g * 16)), hi = *(const iu8_v4u *)(xr + (unsigned)(g * 16) + 8);
#pragma unroll
    for (int w = 0; w < 4; ++w) pk[i][w] = lo[w], pk[i][4 + w] = hi[w];
  }
  float amax = iu8_pk_amax(pk);
  amax = iu8_wave_max_nonneg(amax);
  if ((tid & 63) == 0) s_max[tid >> 6] = amax;
  __syncthreads();
  amax = s_max[0];
#pragma unroll
  for (int w = 1; w < NTHR / 64; ++w) amax = fmaxf(amax, s_max[w]);
  const float sc = fmaxf(__fdiv_rn(amax, 127.f), 1e-30f), rcp = __fdiv_rn(1.f, sc);
  if (tid == 0) scale[row] = sc;
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int g = tid + i * NTHR;
    if (g >= G) continue;
    *(iu8_v4u *)(q + (size_t)row * k + (unsigned)(g * 16)) = iu8_pk_codes(pk[i], sc, rcp);
    __builtin_amdgcn_sched_barrier(0);  // a group's codes at a time (registers)
  }
}

// ---------------------------------------------------------------------------- grouped GEMMs
// grid [ceil(N / BN), tiles_cap, 1]: blockIdx.y is a tile; a workgroup whose tile is past the live
// count exits whole.
#define MOE_GROUPED_DEC(name, GATHER, NT, KW, WPB, D, ALDS, MODE, WPE)                                              \
  extern "C" __global__ __launch_bounds__(WPB * 64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void name(        \
      const unsigned char *__restrict__ a, const unsigned long long *__restrict__ xptr,                           \
      const int *__restrict__ tile_expert, const int *__restrict__ tile_row0, const int *__restrict__ tile_rows,  \
      const int *__restrict__ row_tok, const int *__restrict__ meta, const float *__restrict__ as,                \
      int *__restrict__ p, int *__restrict__ cnt, unsigned short *__restrict__ c, int n, int k, int pmax) {        \
    /* the tile's table entries are requested beside the live count, not behind it (the tables hold gridDim.y     \
       entries): one link less in the chain of dependent loads in front of the first weight load */               \
    const int tile = blockIdx.y;                                                                                   \
    const int live = meta[0], e = tile_expert[tile], row0 = tile_row0[tile], rows = tile_rows[tile];               \
    if (tile >= live) return;                                                                                      \
    const iu8_rows R{GATHER ? row_tok : nullptr, row0, min(rows, 16)};                                             \
    iu8_dec_body<1, false, NT, KW, WPB, D, ALDS, false, MODE, false>(a, (const unsigned char *)xptr[2 * e], as,    \
                                                              (const float *)xptr[2 * e + 1], p, cnt, c, R, n, k); \
  }
MOE_GROUPED_DEC(moe_iu8_grouped_w4_dec_g1, true, 1, 4, 8, 8, 20, 0, 8)
MOE_GROUPED_DEC(moe_iu8_grouped_w4_dec_g0, false, 1, 4, 8, 8, 20, 0, 8)
// The same cell with the activation rows streamed from L2 beside the weights instead of staged in
// LDS: the staged form holds pow2(rows) * K <= 20 KiB (4 rows at K = 4096) and runs a tile that
// does not fit without its load ring; this one keeps the ring for any tile.
// Short K (up to 16 steps): two k-waves a tile instead of four, so a workgroup covers 64 columns and a
// wave's ring holds its whole share (an expert's down projection, K = 1536: 50 -> 45 us at 16 tokens)
MOE_GROUPED_DEC(moe_iu8_grouped_w4_deck_g1, true, 1, 2, 8, 6, 20, 0, 8)
MOE_GROUPED_DEC(moe_iu8_grouped_w4_deck_g0, false, 1, 2, 8, 6, 20, 0, 8)
MOE_GROUPED_DEC(moe_iu8_grouped_w4_deca_g1, true, 2, 8, 8, 2, 0, 0, 8)
MOE_GROUPED_DEC(moe_iu8_grouped_w4_deca_g0, false, 2, 8, 8, 2, 0, 0, 8)
// The back half of a routed layer with few tokens as two launches instead of three: gate+up with the
// activation in its epilogue (a wave owns the gate tile and the up tile of 16 columns and writes
// p = bf16(bf16(silu(gate)) * up), bf16 [rows_cap, n / 2]; the reference chains the same three steps
// inside its persistent back half, crates/saber-kernels/hip/moe_grouped.hip:1656-1765), then down
// with p's per-token quantisation in front of its K loop (every workgroup of a tile converts the
// tile's few rows itself). Same bytes as gate+up -> macaq_i8_silu_mul_quant_* -> down: the same
// routines on the same values. gate+up on the row-streaming cell: the staged forms of this epilogue
// (its exp and divide on top of the staged rows' registers) spill inside the K loop at eight waves a
// SIMD and measured 5 to 60 % slower.
MOE_GROUPED_DEC(moe_iu8_grouped_w4_decpa_g1, true, 2, 8, 8, 2, 0, 1, 8)

MOE_GROUPED_DEC(moe_iu8_grouped_w4_deckq_g0, false, 1, 2, 8, 6, 24, 2, 8)
// two tiles of p a wave (32 columns a workgroup): the rows streamed beside the weights feed twice the
// columns, which pays from about 1.5 routes an expert (layer at 32 tokens 187 -> 183 us, at 64 246 -> 227,
// at 112 316 -> 272; at 8 tokens 100 -> 104)
MOE_GROUPED_DEC(moe_iu8_grouped_w4_decpb_g1, true, 4, 8, 8, 2, 0, 1, 5)
#undef MOE_GROUPED_DEC

// The MFMA-bound cells: a persistent launch of one workgroup a CU walks the work items
// (tile, column block) of the live tiles, column blocks of one tile on neighbouring workgroups, the
// load stream running across items (iu8_pf32.h). grid [256, 1, 1]. Every workgroup first sorts the
// tiles the same way, those of more than MOE_LIGHT_ROWS rows first in table order, the light ones
// after them; the walk is static (item = workgroup + r * gridDim.x), so each kind is dealt evenly.
//
// An expert's last tile is often nearly empty. On the tile cell such a tile still moves whole stages
// of mostly dead rows behind a barrier a step: measured, some 70 % of a full tile's time for a
// twentieth of its work. The two-cell form (LIGHT) runs the light tiles on a second cell in the same
// LDS, 64 rows x 256 columns (2 x 4 waves, the deep form of iu8_pf32.h), whose small stages keep five
// steps of loads in flight and move no dead rows; its K steps start at a depth that differs from
// item to item (iu8_tile::rot), which spreads the weight streams of the light items over the memory
// channels (512 tokens, gate+up: 187 -> 160 us). Light tiles together are bound by the memory rate,
// the heavy ones by the matrix pipes, so a workgroup runs its light items between two parts of its
// heavy ones, after (workgroup / 8) mod (rounds + 1) rounds, the light walk dealt from the last
// workgroup down: at any time a slice of every XCD's CUs streams light tiles under the others'
// matrix work (2,048 tokens on 128-row tiles: 633 -> 577 us a layer against 639 with the light items
// last). An item's descriptor hangs on a chain of dependent loads (order -> tile table -> expert
// pointers), so a workgroup resolves its items up front, one lane an item, into a table in LDS.
// The 128-row kernels are two-cell (256 to 2,048 tokens: 3 to 9 % a layer). The 256-row kernels are
// not: at 4,096 tokens the light tiles' weights come from memory a second time whichever cell asks
// (timestamps: a light item takes 20-28 us there against 4 with its weights cached, a heavy round
// 62-82 us with light items beside it against 63 without), the layer gained 2 %, and launches with no
// light tile (1,536 to 2,048 tokens) lost 2 to 4 % to the two-cell kernel's heavier item switch.
#define MOE_ORDER_CAP 4096  // tiles the ordering holds in LDS; beyond, table order on the big cell
#define MOE_LIGHT_ROWS 64
#define MOE_LIGHT_ST 6
#define MOE_HEAVY_ROUNDS 8  // rounds of items a workgroup resolves at a time: the item table in LDS
#define MOE_LIGHT_ROUNDS 8
struct moe_item {
  int row0, rows, nt0, rot;  // rows < 0: no item
  const unsigned char *W;
  const float *ws;
};
template <int NTHR>
static __device__ __forceinline__ int moe_tile_order(const int *__restrict__ tile_rows, int nt, unsigned short *s_order) {
  __shared__ int s_w[NTHR / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  auto block_sum = [&](int v, int &before) {  // sum over the workgroup; `before` = the waves ahead of this one
    if (lane == 0) s_w[wave] = v;
    __syncthreads();
    int all = 0;
    before = 0;
#pragma unroll
    for (int w = 0; w < NTHR / 64; ++w) {
      const int x = s_w[w];
      before += w < wave ? x : 0;
      all += x;
    }
    __syncthreads();
    return all;
  };
  int mine = 0, unused;
  for (int t = tid; t < nt; t += NTHR) mine += tile_rows[t] > MOE_LIGHT_ROWS;
#pragma unroll
  for (int o = 32; o; o >>= 1) mine += __shfl_xor(mine, o, 64);
  const int heavy_total = block_sum(mine, unused);
  int run = 0;  // heavy tiles before this chunk
  for (int base = 0; base < nt; base += NTHR) {
    const int t = base + tid;
    const bool h = t < nt && tile_rows[t] > MOE_LIGHT_ROWS;
    const unsigned long long b = __ballot(h);
    int wave_before;
    const int chunk = block_sum(__popcll(b), wave_before);
    const int hb = run + wave_before + __popcll(b & ((1ull << lane) - 1ull));  // heavy tiles before t
    if (t < nt) s_order[h ? hb : heavy_total + (t - hb)] = (unsigned short)t;
    run += chunk;
  }
  __syncthreads();
  return heavy_total;
}
// one cell, items in the sorted order
// Workgroup b of a grid of G in the order in which an XCD's workgroups follow each other: b % 8 is the XCD (the
// hardware deals consecutive ids round-robin), so XCD x holds positions x * G/8 ... of the walk. A grid that is not
// whole eighths keeps its ids.
static __device__ __forceinline__ int moe_xcd_run(unsigned b, int G) {
  return (G & 7) == 0 ? (int)(b & 7) * (G >> 3) + (int)(b >> 3) : (int)b;
}
#define MOE_ONE_ITEMS 64  // items a workgroup resolves up front (16,384 items a launch of 256 workgroups)
template <int GATHER, int WMW, int WNW, int TM, int TN, int ST>
static __device__ __forceinline__ void moe_grouped_pf_one(
    const unsigned char *__restrict__ a, const unsigned long long *__restrict__ xptr, const int *__restrict__ tile_expert,
    const int *__restrict__ tile_row0, const int *__restrict__ tile_rows, const int *__restrict__ row_tok,
    const int *__restrict__ meta, const float *__restrict__ as, unsigned short *__restrict__ c, int n, int k) {
  constexpr int BN = WNW * TN * 32;
  static_assert(BN == 256 && WMW * WNW == 8, "both cells are 8 waves and 256 columns wide");
  __shared__ unsigned short s_order[MOE_ORDER_CAP];
  __shared__ moe_item s_item[MOE_ONE_ITEMS];
  __shared__ __attribute__((aligned(1024))) iu8_u8 lds[iu8_pf32_lds_bytes<false, WMW, WNW, TM, TN, ST, true>()];  // one block for both walks below
  const int nt = meta[0], gx = (n + BN - 1) / BN, total = nt * gx;
  const bool ordered = nt <= MOE_ORDER_CAP;
  if (ordered) moe_tile_order<WMW * WNW * 64>(tile_rows, nt, s_order);
  // Consecutive workgroup ids are dealt round-robin over the 8 XCDs, consecutive item ids are the column blocks of
  // one tile. With a grid of whole eighths an XCD's workgroups take a run of item ids (`moe_xcd_run`), so a tile's
  // column blocks share the tile's rows in one L2, or two (dealt by workgroup id they spread over all eight and
  // every XCD fetched the rows for itself: the L2-miss fetch of a launch at 4,096 tokens was twice its operands).
  const int G = gridDim.x, wv = moe_xcd_run(blockIdx.x, G);
  const int rounds = (total + G - 1) / G;
  auto resolve = [&](int q, moe_item &it) {  // this workgroup's item of round q; false past its last
    const int j = wv + q * G;
    const int slot = j / gx, bx = j % gx;
    if (slot >= nt) return false;
    const int tile = ordered ? (int)s_order[slot] : slot;
    const int e = tile_expert[tile];
    it = moe_item{tile_row0[tile], min(tile_rows[tile], WMW * TM * 32), bx * (BN / 16), 0,
                  (const unsigned char *)xptr[2 * e], (const float *)xptr[2 * e + 1]};
    return true;
  };
  if (rounds <= MOE_ONE_ITEMS) {
    // An item's descriptor hangs on a chain of dependent loads (order -> tile table -> expert pointers);
    // fetched where the load stream crosses into the item, every link drains the stream. The
    // workgroup's items are resolved here instead, one lane an item, into a table in LDS.
    const int q = threadIdx.x;
    if (q < rounds) {
      moe_item it{0, -1, 0, 0, nullptr, nullptr};
      resolve(q, it);
      s_item[q] = it;
    }
    __syncthreads();
    iu8_pf32_run<false, WMW, WNW, TM, TN, false, ST, false, true, GATHER == 2, true>(a, as, c, n, k, [&](int r, iu8_tile &t) {
      if (r >= rounds) return false;
      const volatile int *p32 = (const volatile int *)&s_item[r];
      auto u = [&](int i) { return __builtin_amdgcn_readfirstlane(p32[i]); };
      if (u(1) < 0) return false;
      const unsigned long long wp = (unsigned)u(4) | ((unsigned long long)(unsigned)u(5) << 32);
      const unsigned long long sp = (unsigned)u(6) | ((unsigned long long)(unsigned)u(7) << 32);
      t = iu8_tile{iu8_rows{GATHER ? row_tok : nullptr, u(0), u(1)}, 0, u(2), (const unsigned char *)wp, (const float *)sp};
      return true;
    }, nullptr, nullptr, lds);
    return;
  }
  iu8_pf32_run<false, WMW, WNW, TM, TN, false, ST, false, true, GATHER == 2, true>(a, as, c, n, k, [&](int r, iu8_tile &t) {
    moe_item it;
    if (r >= rounds || !resolve(r, it)) return false;
    t = iu8_tile{iu8_rows{GATHER ? row_tok : nullptr, it.row0, it.rows}, 0, it.nt0, it.W, it.ws};
    return true;
  }, nullptr, nullptr, lds);
}
// two cells: heavy items on the tile cell, light ones on the small cell between two parts of them
template <int GATHER, int WMW, int WNW, int TM, int TN, int ST>
static __device__ __forceinline__ void moe_grouped_pf_two(
    const unsigned char *__restrict__ a, const unsigned long long *__restrict__ xptr, const int *__restrict__ tile_expert,
    const int *__restrict__ tile_row0, const int *__restrict__ tile_rows, const int *__restrict__ row_tok,
    const int *__restrict__ meta, const float *__restrict__ as, unsigned short *__restrict__ c, int n, int k) {
  constexpr int BN = WNW * TN * 32;
  static_assert(BN == 256 && WMW * WNW == 8, "both cells are 8 waves and 256 columns wide");
  constexpr int LB = iu8_pf32_lds_bytes<false, WMW, WNW, TM, TN, ST, true>();
  constexpr int LL = iu8_pf32_lds_bytes<false, 2, 4, 1, 2, MOE_LIGHT_ST>();
  __shared__ __attribute__((aligned(1024))) iu8_u8 lds[LB > LL ? LB : LL];
  __shared__ unsigned short s_order[MOE_ORDER_CAP];
  /* the walk's numbers and this workgroup's resolved items live in LDS */
  __shared__ int s_par[4];
  __shared__ moe_item s_item[MOE_HEAVY_ROUNDS + MOE_LIGHT_ROUNDS];
  auto par = [&](int i) { return __builtin_amdgcn_readfirstlane(((volatile int *)s_par)[i]); };
  auto item = [&](int q, iu8_tile &t) {
    const volatile int *p32 = (const volatile int *)&s_item[q];
    auto u = [&](int i) { return __builtin_amdgcn_readfirstlane(p32[i]); };
    if (u(1) < 0) return false;
    const unsigned long long wp = (unsigned)u(4) | ((unsigned long long)(unsigned)u(5) << 32);
    const unsigned long long sp = (unsigned)u(6) | ((unsigned long long)(unsigned)u(7) << 32);
    t = iu8_tile{iu8_rows{GATHER ? row_tok : nullptr, u(0), u(1)}, 0, u(2), (const unsigned char *)wp, (const float *)sp, 0, u(3)};
    return true;
  };
  const int nt = meta[0];
  const bool ordered = nt <= MOE_ORDER_CAP;
  const int heavy = ordered ? moe_tile_order<WMW * WNW * 64>(tile_rows, nt, s_order) : nt;
  /* a launch of more rounds than the item table holds runs in epochs of that many */
  for (int ep = 0;; ++ep) {
    {
      const int gx = (n + BN - 1) / BN, G = gridDim.x, w = moe_xcd_run(blockIdx.x, G);
      const int hi = heavy * gx, li = (nt - heavy) * gx;
      const int h0 = ep * MOE_HEAVY_ROUNDS, l0 = ep * MOE_LIGHT_ROUNDS;
      const int rounds = max(0, min((hi + G - 1) / G - h0, MOE_HEAVY_ROUNDS));
      const int lrounds = max(0, min((li + G - 1) / G - l0, MOE_LIGHT_ROUNDS));
      if (rounds + lrounds == 0) break;
      /* a workgroup's heavy items run in two parts, its light items between them, after `first` rounds */
      if (threadIdx.x == 0) {
        s_par[0] = rounds, s_par[1] = lrounds;
        s_par[2] = lrounds > 0 ? (w >> 3) % (rounds + 1) : rounds;
      }
      const int q = threadIdx.x;
      if (q < rounds + lrounds) {
        const bool light = q >= rounds;
        const int id = light ? G - 1 - w + (l0 + q - rounds) * G : w + (h0 + q) * G;
        moe_item it{0, -1, 0, 0, nullptr, nullptr};
        if (id < (light ? li : hi)) {
          const int slot = (light ? heavy : 0) + id / gx, tile = ordered ? (int)s_order[slot] : slot;
          const int e = tile_expert[tile];
          it = moe_item{tile_row0[tile], min(tile_rows[tile], light ? MOE_LIGHT_ROWS : WMW * TM * 32),
                        id % gx * (BN / 16), light ? (int)(((unsigned)id * 2654435761u >> 10) % (unsigned)(k >> 7)) : 0,
                        (const unsigned char *)xptr[2 * e], (const float *)xptr[2 * e + 1]};
        }
        s_item[q] = it;
      }
      __syncthreads();
    }
    for (int part = 0; part < 2; ++part) {
      if (part == 1) {
        if (par(1) == 0) break;
        iu8_pf32_run<false, 2, 4, 1, 2, false, MOE_LIGHT_ST, true, false, GATHER == 2, true>(
            a, as, c, n, k, [&](int r, iu8_tile &t) { return r < par(1) && item(par(0) + r, t); }, nullptr, nullptr, lds);
        __syncthreads();
      }
      iu8_pf32_run<false, WMW, WNW, TM, TN, false, ST, false, true, GATHER == 2, true>(
          a, as, c, n, k,
          [&](int r, iu8_tile &t) {
            const int first = par(2), rr = part ? first + r : r;
            return rr < (part ? par(0) : first) && item(rr, t);
          },
          nullptr, nullptr, lds);
      __syncthreads();
    }
  }
}
#define MOE_GROUPED_PF(name, BODY, GATHER, WMW, WNW, TM, TN, ST)                                                     \
  extern "C" __global__ __launch_bounds__(WMW * WNW * 64) void name(                                              \
      const unsigned char *__restrict__ a, const unsigned long long *__restrict__ xptr,                           \
      const int *__restrict__ tile_expert, const int *__restrict__ tile_row0, const int *__restrict__ tile_rows,  \
      const int *__restrict__ row_tok, const int *__restrict__ meta, const float *__restrict__ as,                \
      int *__restrict__ p, int *__restrict__ cnt, unsigned short *__restrict__ c, int n, int k, int pmax) {        \
    BODY<GATHER, WMW, WNW, TM, TN, ST>(a, xptr, tile_expert, tile_row0, tile_rows, row_tok, meta, as, c, n, k);    \
  }
// tiles of up to 128 rows (tile_blocks 8) on the 128 x 256 tile of 2 x 4 waves
MOE_GROUPED_PF(moe_iu8_grouped_w4_pf_g2, moe_grouped_pf_two, 2, 2, 4, 2, 2, 4)
MOE_GROUPED_PF(moe_iu8_grouped_w4_pf_g1, moe_grouped_pf_two, 1, 2, 4, 2, 2, 4)
MOE_GROUPED_PF(moe_iu8_grouped_w4_pf_g0, moe_grouped_pf_two, 0, 2, 4, 2, 2, 4)
// tiles of up to 256 rows (tile_blocks 16) on the 256 x 256 tile, the dense GEMM's fastest cell
MOE_GROUPED_PF(moe_iu8_grouped_w4_pf16_g2, moe_grouped_pf_one, 2, 2, 4, 4, 2, 3)
MOE_GROUPED_PF(moe_iu8_grouped_w4_pf16_g1, moe_grouped_pf_one, 1, 2, 4, 4, 2, 3)
MOE_GROUPED_PF(moe_iu8_grouped_w4_pf16_g0, moe_grouped_pf_one, 0, 2, 4, 4, 2, 3)
#undef MOE_GROUPED_PF

// ---------------------------------------------------------------------------- combine
// sigmoid(g) from the router's IEEE-only exp (crates/saber-kernels/hip/moe_route.hip:59-63): e = exp(-|g|),
// 1 / (1 + e) for g >= 0, e / (1 + e) below; IEEE divides.
static __device__ __forceinline__ float moe_sigmoid(float g) {
#pragma clang fp contract(off)
  const float e = moe_exp_nonpos(-fabsf(g));
  const float d = 1.f + e;
  return g >= 0.f ? __fdiv_rn(1.f, d) : __fdiv_rn(e, d);
}
// One workgroup a token, 8 bf16 a thread-step: out[t] = bf16(sum over the token's routes in top-k order of
// w * Y[route's row], then + sigmoid(sgate[t]) * Y[shared row t] when the layer has a shared expert
// (meta[2] >= 0 and sgate given), f32, one bf16 rounding (crates/saber-kernels/hip/moe_route.hip:287-329).
extern "C" __global__ __launch_bounds__(256) void moe_iu8_combine_bf16(
    const unsigned short *__restrict__ y, const float *__restrict__ topk_w, const int *__restrict__ route_pos,
    const unsigned short *__restrict__ sgate, const int *__restrict__ meta, unsigned short *__restrict__ out, int h) {
#pragma clang fp contract(off)
  const int t = blockIdx.x;
  __shared__ int s_pos[MOE_TOPK];
  __shared__ float s_w[MOE_TOPK];
  if (threadIdx.x < MOE_TOPK) {
    s_pos[threadIdx.x] = route_pos[(size_t)t * MOE_TOPK + threadIdx.x];
    s_w[threadIdx.x] = topk_w[(size_t)t * MOE_TOPK + threadIdx.x];
  }
  __syncthreads();
  const int sh0 = meta[2];
  const bool shared = sh0 >= 0 && sgate != nullptr;
  const float sg = shared ? moe_sigmoid(iu8_bf16_f32(sgate[t])) : 0.f;
  for (int g = threadIdx.x; g < h / 8; g += 256) {
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    // the routes' rows are requested together (a route that is not local, p < 0, reads row 0 and is not added):
    // one latency a group instead of eight in a row; the adds keep the top-k order
    iu8_v4u rows[MOE_TOPK];
#pragma unroll
    for (int k = 0; k < MOE_TOPK; ++k) rows[k] = ((const iu8_v4u *)(y + (size_t)max(s_pos[k], 0) * h))[g];
#pragma unroll
    for (int k = 0; k < MOE_TOPK; ++k) {
      if (s_pos[k] < 0) continue;
      const float w = s_w[k];
      const iu8_v4u v = rows[k];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[2 * q] = acc[2 * q] + w * __uint_as_float(v[q] << 16);
        acc[2 * q + 1] = acc[2 * q + 1] + w * __uint_as_float(v[q] & 0xFFFF0000u);
      }
    }
    if (shared) {
      const iu8_v4u v = ((const iu8_v4u *)(y + (size_t)(sh0 + t) * h))[g];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[2 * q] = acc[2 * q] + sg * __uint_as_float(v[q] << 16);
        acc[2 * q + 1] = acc[2 * q + 1] + sg * __uint_as_float(v[q] & 0xFFFF0000u);
      }
    }
    iu8_v4u o;
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = iu8_bf16_bits(acc[2 * q]) | (iu8_bf16_bits(acc[2 * q + 1]) << 16);
    ((iu8_v4u *)(out + (size_t)t * h))[g] = o;
  }
}
