// The library's static split-K workspace (static_ws.hip): one device array a GPU, its address taken
// once per device when a context is opened.
#pragma once
#include <cstddef>

namespace iu8 {

// Arrival counters first (64 KiB: 16,384 tiles or column blocks), then the int32 partials (8 MiB:
// ks * M * N * 4 bytes of the largest launch the law splits today is 7.5 MiB).
constexpr size_t STATIC_WS_COUNTER_BYTES = 64 * 1024;
constexpr size_t STATIC_WS_PARTIAL_BYTES = 8 * 1024 * 1024;
constexpr size_t STATIC_WS_BYTES = STATIC_WS_COUNTER_BYTES + STATIC_WS_PARTIAL_BYTES;

// With `device` current: takes the array's address on it (once) and zero-fills it. 0 or an error code.
int static_ws_init(int device);
// Zero-fills the arrival counters on `stream` with a kernel (capture-legal). 0 or an error code.
int static_ws_reset(int device, void *stream);
void *static_ws_partial(int device);  // nullptr before static_ws_init(device)
void *static_ws_counter(int device);

}  // namespace iu8
