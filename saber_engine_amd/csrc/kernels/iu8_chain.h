// The dense decode MLP as ONE persistent launch of the gfx950 W4A8-iu8 path: gate+up linear ->
// SiLU(gate) * up + per-token requantisation -> down linear, for the few rows of a decode step
// (M <= 4 and pow2(M) * I <= 20 KiB of staged codes). The reference chains its routed experts' back
// half this way (`moe_back_*`: gate_up -> silu-quant -> down -> combine in one persistent launch,
// phases handed over through device counters, crates/saber-kernels/hip/moe_grouped.hip:1656-1765,
// crates/saber-kernels/src/moe.rs:341-345); this is the dense twin for the iu8 decode band.
//
// Every workgroup of the launch is resident at once (the host refuses a grid the card cannot hold),
// so the two linears can meet inside the launch:
//   phase 1  the fused decode linear (iu8_decq.h) in its paired form: a column block is one 16-column
//            tile of p, its gate tile computed by one half of the workgroup's waves and its up tile by
//            the other, p = bf16(bf16(silu(gate)) * up) in the epilogue, stored straight through to
//            memory, the workgroup's maxima of |p| a row into its own slot;
//   meeting  arrived at once, waited for only after the down linear's first weight loads have left:
//            the weights do not depend on p, so their latency hides behind the meeting;
//   phase 2  the fused decode linear again, p -> c, the rows' scales from the maximum over all slots
//            (order-free, so the scale is the one a pass over the whole row finds).
// The bytes are those of the three launches (linear, macaq_i8_silu_mul_quant_*, linear): every piece
// is the same routine on the same values, maxima are order-free, and the int32 sums are exact.
// Measured: a meeting costs 4-5 us on this card (the data stores' completion, the word's store, a
// poll's round trip, all to memory: the XCDs share no cache), more than the 2.4 us between two
// launches -- a chain with the activation as a phase of its own between two meetings ran no faster
// than the three launches, which is why the activation sits in the first linear's epilogue.
//
// The meeting is a word a workgroup, not a shared counter: a workgroup that arrives stores 1 into its
// own word (straight through to memory, behind its completed data stores); the LAST workgroup of the
// grid collects -- it reads all the words at once, one a lane, and when all are set stores the `go`
// word, which every waiting workgroup polls with one lane. (512 read-modify-writes of one counter a
// meeting, which the memory system performs one after another at about 20 ns each, cost 10 us a
// meeting; every workgroup reading all the words itself -- 512 x 2 KB a microsecond out of one memory
// channel -- held the workgroups still streaming weights back by 3-5 us. Both measured.)
// The state block is a Persistent workspace in the reference's sense (include/saber_abi.h:163-174:
// zeroed once when allocated, left zero by the kernel): a workgroup that has seen `go` sets its
// `passed` word, and the collector -- at once when it has no column block of the second linear, else
// behind its own -- waits until every waiting workgroup has passed and then clears the words, the
// passed words and `go`. A launch that completes leaves every word it wrote at zero except the
// maxima slots, which every launch rewrites in full before reading them.
//
// A wait polls at most `spin` times (a bounded wait: about a microsecond a poll); past that the
// workgroup raises the status word and leaves, and so does every other one at its next look, so a
// launch that cannot complete ends instead of hanging; nothing is cleared then, and the host zeroes
// the state block before it is used again. Such a launch -- and every later one on a state block whose
// status is still raised -- fills its output rows with bf16 NaNs (0x7FC0), so the failure shows in `c`
// itself, also to a caller that replays a captured graph and never reads the state block.
//
// The state block (IU8_CHAIN_STATE_BYTES, zero before the first launch):
//   [0, 8 KiB)        512 slots of 4 floats: a workgroup's maxima of |p|, a row
//   [8 KiB, 10 KiB)   512 arrival words          [10 KiB, 12 KiB)  512 passed words
//   [12 KiB]          status (non-zero: a wait timed out);  [12 KiB + 4]  go
#pragma once
#include "iu8_decq.h"

#define IU8_CHAIN_MAXG 512
#define IU8_CHAIN_STATE_BYTES (13 * 1024)
#define IU8_CHAIN_WORDS_OFF (8 * 1024)
#define IU8_CHAIN_PASSED_OFF (10 * 1024)
#define IU8_CHAIN_STATUS_OFF (12 * 1024)

struct iu8_chain_sync {
  unsigned *words;   // arrival words, one a workgroup
  unsigned *passed;  // a waiting workgroup has seen `go`
  int *status;       // status[0] != 0: a wait timed out; status[1]: the collector's `go` word (an 8-byte aligned pair)
  int nwait;         // workgroups that wait at the meeting: those with a column block of the second linear
  int spin;          // polls a wait lasts at most
};
static __device__ __forceinline__ unsigned iu8_chain_ld(const unsigned *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
static __device__ __forceinline__ void iu8_chain_st(unsigned *p, unsigned v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// This workgroup's stores are in memory, then its word says so.
static __device__ __forceinline__ void iu8_chain_arrive(const iu8_chain_sync &S) {
  iu8_stores_done();
  __syncthreads();
  if (threadIdx.x == 0) iu8_chain_st(S.words + blockIdx.x, 1u);
}
// The whole workgroup: true once `n` words from `w` on are all set, false when the polls ran out or a
// wait elsewhere did (status raised). n <= blockDim.x: one word a lane.
static __device__ __forceinline__ bool iu8_chain_all_set(const iu8_chain_sync &S, const unsigned *w, int n) {
  bool ok = false;
  for (int i = 0; i < S.spin; ++i) {
    int pending = (int)threadIdx.x < n && iu8_chain_ld(w + threadIdx.x) == 0u;
    if (threadIdx.x == blockDim.x - 1) pending |= 2 * (iu8_chain_ld((const unsigned *)S.status) != 0u);
    const int any = __syncthreads_or(pending);
    if (any & 2) break;
    if (any == 0) {
      ok = true;
      break;
    }
  }
  if (!ok && threadIdx.x == 0) iu8_chain_st((unsigned *)S.status, 1u);
  return ok;
}
// The collector's first half: every workgroup has arrived -> `go`.
static __device__ __forceinline__ bool iu8_chain_collect(const iu8_chain_sync &S) {
  const bool ok = iu8_chain_all_set(S, S.words, (int)gridDim.x);
  if (ok && threadIdx.x == 0) iu8_chain_st((unsigned *)S.status + 1, 1u);
  return ok;
}
// The collector's second half: every waiting workgroup has seen `go` -> everything back to zero.
static __device__ __forceinline__ void iu8_chain_clear(const iu8_chain_sync &S) {
  if (!iu8_chain_all_set(S, S.passed, S.nwait)) return;
  if ((int)threadIdx.x < (int)gridDim.x) iu8_chain_st(S.words + threadIdx.x, 0u);
  if ((int)threadIdx.x < S.nwait) iu8_chain_st(S.passed + threadIdx.x, 0u);
  if (threadIdx.x == 0) iu8_chain_st((unsigned *)S.status + 1, 0u);
}
// A waiting workgroup: true once `go` is set (and says that it has seen it), false when the polls ran
// out or a wait elsewhere did. The collector itself collects here.
static __device__ __forceinline__ bool iu8_chain_wait(const iu8_chain_sync &S) {
  if (blockIdx.x == gridDim.x - 1) {
    const bool ok = iu8_chain_collect(S);
    if (ok && threadIdx.x == 0) iu8_chain_st(S.passed + blockIdx.x, 1u);
    return ok;
  }
  __shared__ int s_ok;
  if (threadIdx.x == 0) {
    int good = 0;
    for (int i = 0; i < S.spin; ++i) {
      // status and go, one 8-byte load
      const unsigned long long v = __hip_atomic_load((const unsigned long long *)S.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      if ((unsigned)v != 0u) break;
      if ((unsigned)(v >> 32) != 0u) {
        good = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
    if (good) iu8_chain_st(S.passed + blockIdx.x, 1u);
    else iu8_chain_st((unsigned *)S.status, 1u);
    s_ok = good;
  }
  __syncthreads();
  const bool ok = s_ok != 0;
  __syncthreads();
  return ok;
}

// The second linear's view of the chain: wait for the meeting, then the rows' maxima over all slots.
struct iu8_chain_hook {
  iu8_chain_sync S;
  const float *slots;
  __device__ bool wait() const { return iu8_chain_wait(S); }
  __device__ void amax(float out[4]) const {
    __shared__ float s_m[16][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (tid < (int)gridDim.x) {
      const iu8_v4u raw = iu8_decq_ld_coherent((const iu8_v4u *)slots + tid);
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = __uint_as_float(raw[r]);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v[r] = iu8_wave_max_nonneg(v[r]);
      if (lane == 0) s_m[wave][r] = v[r];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float a = s_m[0][r];
      for (int w = 1; w < (int)(blockDim.x >> 6); ++w) a = fmaxf(a, s_m[w][r]);
      out[r] = a;
    }
  }
};

// AKB2: KiB of staged codes of the second linear -- 20 (pow2(M) * I <= 20 KiB) or 80 (up to 4 rows of an
// intermediate width whose codes fit 80 KiB: the benchmark layer's 17,408 at 2 to 4 rows). The two linears
// run one after the other, so their LDS objects lie over one block.
template <int NT, int KW, int WPB, int D, int AKB2 = 20>
__device__ __forceinline__ void iu8_chain_mlp(const unsigned short *__restrict__ x, const iu8_u8 *__restrict__ w_gu,
                                              const float *__restrict__ ws_gu, const iu8_u8 *__restrict__ w_dn,
                                              const float *__restrict__ ws_dn, unsigned short *__restrict__ gu,
                                              unsigned short *__restrict__ p, unsigned char *__restrict__ state,
                                              unsigned short *__restrict__ c, int M, int H, int I, int spin) {
  static_assert(WPB * 64 >= IU8_CHAIN_MAXG, "a lane an arrival word");
  float *slots = (float *)state;
  constexpr int BLK2 = (WPB / KW) * NT * 16;  // columns of the second linear a workgroup and block
  const int G = gridDim.x;
  const iu8_chain_sync S{(unsigned *)(state + IU8_CHAIN_WORDS_OFF), (unsigned *)(state + IU8_CHAIN_PASSED_OFF),
                         (int *)(state + IU8_CHAIN_STATUS_OFF), min(G, (H + BLK2 - 1) / BLK2), spin};
  const bool collector = (int)blockIdx.x == G - 1;
  // phase 1: [gate | up] = x . Wgu^T (quantisation of x fused), p and this workgroup's maxima from its
  // epilogue, stored through; gu (may be null) is a tap
  __shared__ union Lds {
    iu8_decq_lds<NT, KW, WPB, 1, 20> first;
    iu8_decq_lds<NT, KW, WPB, 2, AKB2> second;
  } lds;
  iu8_decq_body<false, NT, KW, WPB, D, 1>(lds.first, x, w_gu, ws_gu, nullptr, nullptr, gu, M, I, H,
                                          iu8_decq_pairhook{p, slots + blockIdx.x * 4});
  iu8_chain_arrive(S);
  if ((int)blockIdx.x >= S.nwait) {
    // no column block of the second linear: done -- but the collector collects, and clears at once
    if (collector && iu8_chain_collect(S)) iu8_chain_clear(S);
    return;
  }
  // phase 2: c = p . Wdn^T; the hook waits for the meeting behind the first weight loads
  // (the first linear's LDS is dead: every wave of this workgroup is past iu8_chain_arrive's barrier)
  iu8_decq_body<false, NT, KW, WPB, D, 2, iu8_chain_hook, AKB2>(lds.second, p, w_dn, ws_dn, nullptr, nullptr, c, M, H, I,
                                                                iu8_chain_hook{S, slots});
  // (one answer for the whole workgroup: the clear holds barriers)
  if (collector && __syncthreads_or(iu8_chain_ld((const unsigned *)S.status) != 0u) == 0) iu8_chain_clear(S);
}
