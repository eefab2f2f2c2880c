// The GEMM entry point that allocates nothing: the split-K workspaces of a launch (`decode_partial`,
// int32 partial sums of every K share, and `decode_counter`, the per-tile arrival counters) live in
// one file-scope device array of fixed size instead of buffers the caller allocates. For callers
// that cannot call hipMalloc between launches: code under HIP graph capture, tight serving loops.
//
// The array exists once per GPU the library is loaded on and is held until the process ends. Host
// code never uses the array's name as an address: its device address is asked for once per device
// (hipGetSymbolAddress, with that device current) when a context is opened, and kept. Every call on
// a GPU shares that GPU's array: calls that overlap in time on one GPU (two streams) race on it;
// calls on one stream, or ordered by events, do not. The partials are written before they are read
// (scratch semantics: the last call's contents do not matter); the counters start at zero -- the
// array is zero-filled when its address is taken, by a fill kernel, and every kernel that counts
// arrivals resets its counters before it ends -- so nothing is cleared per call and no memset node
// enters a captured graph.
#include <hip/hip_runtime.h>

#include <mutex>

#include "../../../include/saber_iu8.h"
#include "static_ws.h"
#include "util.h"

namespace {

static __device__ __align__(256) unsigned char scratch[iu8::STATIC_WS_BYTES];

__global__ void static_ws_fill(unsigned *p, size_t n4) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) p[i] = 0u;
}

constexpr int MAX_DEVICES = 64;
void *g_ptr[MAX_DEVICES];  // the array's address on each device, 0 = not asked for yet
std::mutex g_mu;           // two threads opening contexts on one device: one of them sets the array up, the other waits

}  // namespace

namespace iu8 {

int static_ws_init(int device) {
  if (device < 0 || device >= MAX_DEVICES) return fail(SABER_IU8_E_ARG, fmt("static workspace: device %d out of range", device));
  // held over the fill: a second opener must not see the address before the zeros are there, nor fill again
  // under a launch of the first that is counting arrivals
  std::lock_guard<std::mutex> lock(g_mu);
  if (g_ptr[device]) return 0;
  // the caller has made `device` current
  void *p = nullptr;
  hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p)
    return fail(SABER_IU8_E_HIP, fmt("hipGetSymbolAddress(scratch) on device %d: HIP status %d (%s)", device, (int)e, hipGetErrorString(e)));
  // zero it once through its address (a fill kernel, not a memset)
  hipLaunchKernelGGL(static_ws_fill, dim3(256), dim3(256), 0, (hipStream_t) nullptr, (unsigned *)p, STATIC_WS_BYTES / 4);
  if ((e = hipGetLastError()) != hipSuccess || (e = hipStreamSynchronize(nullptr)) != hipSuccess)
    return fail(SABER_IU8_E_HIP, fmt("static workspace fill on device %d: HIP status %d (%s)", device, (int)e, hipGetErrorString(e)));
  g_ptr[device] = p;
  return 0;
}

// The arrival counters back to zero, on the caller's stream, by the fill kernel (no memset: a caller may be
// capturing): for a process that had a launch cut short (a device error, a killed stream) between a tile's
// first arrival and its last, which leaves counters that no later launch would bring back to zero.
int static_ws_reset(int device, void *stream) {
  void *p = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_mu);
    p = device >= 0 && device < MAX_DEVICES ? g_ptr[device] : nullptr;
  }
  if (!p) return fail(SABER_IU8_E_NOTLOADED, fmt("static workspace of device %d was not set up", device));
  hipLaunchKernelGGL(static_ws_fill, dim3(16), dim3(256), 0, (hipStream_t)stream, (unsigned *)p, STATIC_WS_COUNTER_BYTES / 4);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(SABER_IU8_E_HIP, fmt("static workspace reset on device %d: HIP status %d (%s)", device, (int)e, hipGetErrorString(e)));
  return 0;
}

void *static_ws_partial(int device) {
  return device >= 0 && device < MAX_DEVICES && g_ptr[device] ? (unsigned char *)g_ptr[device] + STATIC_WS_COUNTER_BYTES : nullptr;
}
void *static_ws_counter(int device) { return device >= 0 && device < MAX_DEVICES ? g_ptr[device] : nullptr; }

}  // namespace iu8
