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
// A meeting is a word a workgroup, not a shared counter: a workgroup that arrives stores the
// launch's generation and the phase into its own word (straight through to memory, behind its
// completed data stores), and a waiting workgroup reads all the words at once, one a lane. 512
// read-modify-writes of one counter a meeting, which the memory system performs one after another
// (about 20 ns each), cost 10 us a meeting (measured); the words cost a store and a load. The generation lives
// in the state block and is advanced by workgroup 0 once every workgroup has read it, so the words
// never need clearing: a launch that completes leaves the state block ready for the next one.
//
// A meeting polls at most `spin` times (a bounded wait: about a microsecond a poll); past that the
// workgroup raises the status word and leaves, and so does every other one at its next meeting, so
// a launch that cannot complete ends instead of hanging. The host then zeroes the state block
// before it is used again.
//
// The state block (IU8_CHAIN_STATE_BYTES, zero before the first launch):
//   [0, 8 KiB)        512 slots of 4 floats: a workgroup's maxima of |p|, a row
//   [8 KiB, 10 KiB)   512 arrival words
//   [10 KiB]          generation;  [10 KiB + 8]  status (non-zero: a meeting timed out);  [10 KiB + 12]  go
#pragma once
#include "iu8_decq.h"

#define IU8_CHAIN_MAXG 512
#define IU8_CHAIN_STATE_BYTES (12 * 1024)
#define IU8_CHAIN_WORDS_OFF (8 * 1024)
#define IU8_CHAIN_GEN_OFF (10 * 1024)

struct iu8_chain_sync {
  unsigned *words;  // arrival words, one a workgroup
  int *status;      // status[0] != 0: a meeting timed out; status[1]: the collector's `go` word (8-byte aligned pair)
  unsigned base;    // 4 * the launch's generation: phase ph of this launch is the value base + ph
  int spin;         // polls a meeting waits at most
};

// This workgroup's stores are in memory, then its word says so.
static __device__ __forceinline__ void iu8_chain_arrive(const iu8_chain_sync &S, unsigned phase) {
  iu8_stores_done();
  __syncthreads();
  if (threadIdx.x == 0) __hip_atomic_store(S.words + blockIdx.x, S.base + phase, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
// Returns true once every workgroup's word has reached `phase`, false when the wait ran out or
// another workgroup's did (status raised). Workgroup 0 collects: it reads all the words at once, one
// a lane (gridDim.x <= blockDim.x), and when all have arrived stores the `go` word; every other
// workgroup polls that one word with one lane. (Every workgroup reading all the words -- 512 x 2 KB a
// microsecond out of one memory channel -- held back the workgroups still streaming their weights
// through that channel by 3-5 us, measured from timestamps inside the kernel.)
static __device__ __forceinline__ bool iu8_chain_wait(const iu8_chain_sync &S, unsigned phase) {
  const unsigned target = S.base + phase;
  unsigned *go = (unsigned *)S.status + 1;
  bool ok = false;
  if (blockIdx.x == 0) {
    const bool mine = threadIdx.x < gridDim.x;
    for (int n = 0; n < S.spin; ++n) {
      int pending = 0;
      if (mine) pending = (int)(__hip_atomic_load(S.words + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) - target) < 0;
      if (threadIdx.x == blockDim.x - 1) pending |= 2 * (__hip_atomic_load(S.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0);
      const int any = __syncthreads_or(pending);
      if (any & 2) break;
      if (any == 0) {
        ok = true;
        break;
      }
    }
    if (threadIdx.x == 0) {
      if (ok) __hip_atomic_store(go, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      else __hip_atomic_store(S.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    return ok;
  }
  __shared__ int s_ok;
  if (threadIdx.x == 0) {
    int good = 0;
    for (int n = 0; n < S.spin; ++n) {
      // status and go, one 8-byte load
      const unsigned long long v = __hip_atomic_load((const unsigned long long *)S.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      if ((unsigned)v != 0u) break;
      if ((int)((unsigned)(v >> 32) - target) >= 0) {
        good = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
    if (!good) __hip_atomic_store(S.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    s_ok = good;
  }
  __syncthreads();
  ok = s_ok != 0;
  __syncthreads();
  return ok;
}

// The second linear's view of the chain: wait for the meeting, then the rows' maxima over all slots.
struct iu8_chain_hook {
  iu8_chain_sync S;
  const float *slots;
  __device__ bool wait() const { return iu8_chain_wait(S, 1u); }
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

template <int NT, int KW, int WPB, int D>
__device__ __forceinline__ void iu8_chain_mlp(const unsigned short *__restrict__ x, const iu8_u8 *__restrict__ w_gu,
                                              const float *__restrict__ ws_gu, const iu8_u8 *__restrict__ w_dn,
                                              const float *__restrict__ ws_dn, unsigned short *__restrict__ gu,
                                              unsigned short *__restrict__ p, unsigned char *__restrict__ state,
                                              unsigned short *__restrict__ c, int M, int H, int I, int spin) {
  static_assert(WPB * 64 >= IU8_CHAIN_MAXG, "a lane an arrival word");
  float *slots = (float *)state;
  unsigned *gen = (unsigned *)(state + IU8_CHAIN_GEN_OFF);
  // the generation: read by every workgroup before it arrives, advanced by workgroup 0 behind the
  // meeting -- when every workgroup has arrived and so has read it
  const unsigned g = __hip_atomic_load(gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const iu8_chain_sync S{(unsigned *)(state + IU8_CHAIN_WORDS_OFF), (int *)(gen + 2), 4u * g, spin};
  // phase 1: [gate | up] = x . Wgu^T (quantisation of x fused), p and this workgroup's maxima from its
  // epilogue, stored through; gu (may be null) is a tap
  iu8_decq_body<false, NT, KW, WPB, D, 1>(x, w_gu, ws_gu, nullptr, nullptr, gu, M, I, H,
                                          iu8_decq_pairhook{p, slots + blockIdx.x * 4});
  iu8_chain_arrive(S, 1u);
  // a workgroup with no column block of the second linear is done (workgroup 0 always has one)
  constexpr int BLK2 = (WPB / KW) * NT * 16;
  if ((int)blockIdx.x * BLK2 >= H) return;
  // phase 2: c = p . Wdn^T; the hook waits for the meeting behind the first weight loads
  iu8_decq_body<false, NT, KW, WPB, D, 2>(p, w_dn, ws_dn, nullptr, nullptr, c, M, H, I, iu8_chain_hook{S, slots});
  if (blockIdx.x == 0 && threadIdx.x == 0 && __hip_atomic_load(S.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == 0)
    __hip_atomic_store(gen, g + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
