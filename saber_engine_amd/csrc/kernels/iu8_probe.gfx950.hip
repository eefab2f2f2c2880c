// Roofline denominators measured on the card, next to the published ones: the code object
// `iu8_probe`. A streaming read, a plain copy of known size (the scale factor of the HBM byte
// counters), an empty launch (the per-launch floor of back-to-back timing) and a register-resident
// int8 MFMA loop (the matrix peak the clocks actually sustain).
#include "iu8_common.h"

// reads n16 16-byte pieces once; grid-stride, 8 loads in flight a lane; the xor lands in out[0]
// only for an impossible value, so the loads cannot be dropped
extern "C" __global__ __launch_bounds__(256) void iu8_probe_read(const unsigned char *__restrict__ src,
                                                                 unsigned *__restrict__ out, int n16) {
  const iu8_v4u *p = (const iu8_v4u *)src;
  const long stride = (long)gridDim.x * 256;
  long i = (long)blockIdx.x * 256 + threadIdx.x;
  iu8_v4u x = iu8_v4u{0, 0, 0, 0};
  for (; i + 7 * stride < n16; i += 8 * stride) {
    iu8_v4u v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) x ^= v[u];
  }
  for (; i < n16; i += stride) x ^= __builtin_nontemporal_load(p + i);
  if ((x.x ^ x.y ^ x.z ^ x.w) == 0x9E3779B9u) out[0] = x.x;
}

extern "C" __global__ __launch_bounds__(256) void iu8_probe_copy(const unsigned char *__restrict__ src,
                                                                 unsigned char *__restrict__ dst, int n16) {
  const iu8_v4u *p = (const iu8_v4u *)src;
  iu8_v4u *q = (iu8_v4u *)dst;
  const long stride = (long)gridDim.x * 256;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) q[i] = p[i];
}

extern "C" __global__ __launch_bounds__(256) void iu8_probe_empty(unsigned *__restrict__ out) {
  if (out == nullptr && threadIdx.x == 1023) __builtin_trap();
}

// n = iterations; every wave runs 8 independent accumulator chains of v_mfma_i32_16x16x64_i8
// (32,768 int8 ops each) per iteration
extern "C" __global__ __launch_bounds__(256) void iu8_probe_mfma(unsigned *__restrict__ out, int n) {
  iu8_v4i a = iu8_v4i{(int)threadIdx.x, 1, 2, 3}, b = iu8_v4i{4, 5, (int)blockIdx.x, 7};
  iu8_v4i c[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) c[j] = iu8_v4i{j, 0, 0, 0};
  for (int i = 0; i < n; ++i) {
#pragma unroll
    for (int j = 0; j < 8; ++j) c[j] = iu8_mfma(a, b, c[j]);
  }
  iu8_v4i s = c[0];
#pragma unroll
  for (int j = 1; j < 8; ++j) s += c[j];
  if ((s.x ^ s.y ^ s.z ^ s.w) == 0x12345679) out[0] = s.x;
}

// the same with v_mfma_i32_32x32x32_i8 (65,536 int8 ops each), 4 independent chains
typedef int iu8_v16i __attribute__((ext_vector_type(16)));
extern "C" __global__ __launch_bounds__(256) void iu8_probe_mfma32(unsigned *__restrict__ out, int n) {
  iu8_v4i a = iu8_v4i{(int)threadIdx.x, 1, 2, 3}, b = iu8_v4i{4, 5, (int)blockIdx.x, 7};
  iu8_v16i c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) c[j][e] = j + e;
  for (int i = 0; i < n; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c[j], 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) s ^= c[j][e];
  if (s == 0x12345679) out[0] = s;
}

// The matrix rate with real operands: every lane loads 4 + 4 operands from `src` once (random
// bytes or zeros, the caller's choice) and runs the 4 x 4 tile pattern of the prefill GEMM,
// 16 v_mfma_i32_32x32x32_i8 an iteration on 16 accumulator tiles. Same code, different data:
// the difference is what the card's power management takes off the clock.
extern "C" __global__ __launch_bounds__(256) void iu8_probe_mfma32d(const unsigned char *__restrict__ src,
                                                                    unsigned *__restrict__ out, int n) {
  const iu8_v4i *p = (const iu8_v4i *)src + (size_t)(blockIdx.x * 256 + threadIdx.x) * 8;
  iu8_v4i a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = p[i], b[i] = p[4 + i];
  iu8_v16i c[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) c[i][j][e] = 0;
  for (int it = 0; it < n; ++it) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) c[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[j], a[i], c[i][j], 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) s ^= c[i][j][e];
  if (s == 0x12345679) out[0] = s;
}

// What a launch pays before its first bytes: every wave stamps the 100 MHz constant clock at its
// start and after each of n dependent 1 KiB wave-loads (16 bytes a lane, nontemporal, one in flight
// at a time) of its own region of src; lane 0 stores the n + 1 stamps to out[(wave id) * (n + 1) ...]
// as 64-bit values. The first interval holds the start-of-kernel cost on top of the memory latency
// the later intervals show.
extern "C" __global__ __launch_bounds__(512) void iu8_probe_first(const unsigned char *__restrict__ src,
                                                                  unsigned *__restrict__ out, int n) {
  const int wave = (int)blockIdx.x * 8 + (int)(threadIdx.x >> 6), lane = threadIdx.x & 63;
  unsigned long long *o = (unsigned long long *)out + (size_t)wave * (n + 1);
  unsigned long long t = __builtin_amdgcn_s_memrealtime();
  if (lane == 0) o[0] = t;
  const unsigned char *p = src + ((size_t)wave * n) * 1024 + lane * 16;
  for (int r = 0; r < n; ++r) {
    iu8_v4u v;
    const unsigned char *q = p + (size_t)r * 1024;
    // load and wait in one volatile statement, so the stamp that follows is taken after the data
    asm volatile("global_load_dwordx4 %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(q) : "memory");
    t = __builtin_amdgcn_s_memrealtime() + (v.x == 0x9E3779B9u && v.y == 1u);
    if (lane == 0) o[r + 1] = t;
  }
}
