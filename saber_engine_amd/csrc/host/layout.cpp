// Host-side operand orders and the offline repack (canonical export forms and the reference's
// gfx12 fragment orders -> the gfx950 fragment orders documented in kernels/iu8_common.h).
#include <cstring>

#include "../../../include/saber_iu8.h"
#include "util.h"

using namespace iu8;

extern "C" {

size_t saber_iu8_a_bytes(uint32_t m, uint32_t k) { return (size_t)((m + 15) / 16 * 16) * k; }

uint64_t saber_iu8_a_offset(uint32_t m, uint32_t k, uint32_t K) {
  return ((uint64_t)(m >> 4) * (K / 64) + (k >> 6)) * 1024 + ((m & 15) + 16 * ((k >> 4) & 3)) * 16 + (k & 15);
}

uint64_t saber_iu8_w4_offset(uint32_t n, uint32_t k, uint32_t K, uint32_t *high) {
  const uint32_t r = k & 127, g = (r >> 4) & 3, j = (r >> 6) * 2 + ((r >> 3) & 1), within = r & 7;
  if (high) *high = within >> 2;
  return ((uint64_t)(n >> 4) * (K / 128) + (k >> 7)) * 1024 + ((n & 15) + 16 * g) * 16 + j * 4 + (within & 3);
}

static int shape_ok(const char *what, uint32_t n, uint32_t k) {
  if (n == 0 || k == 0 || n % 16 != 0 || k % 128 != 0)
    return fail(SABER_IU8_E_RULE, fmt("%s: N=%u must be a multiple of 16 and K=%u of 128", what, n, k));
  return 0;
}

int saber_iu8_repack_w4(const uint8_t *canonical, uint32_t n, uint32_t k, uint8_t *frag) {
  if (!canonical || !frag) return fail(SABER_IU8_E_ARG, "repack_w4: null buffer");
  if (int rc = shape_ok("repack_w4", n, k)) return rc;
  auto code = [&](uint32_t row, uint32_t kk) -> uint8_t {
    const uint8_t b = canonical[(size_t)row * (k / 2) + (kk >> 1)];
    return (kk & 1) ? (b >> 4) : (b & 15);
  };
  for (uint32_t nt = 0; nt < n / 16; ++nt)
    for (uint32_t kt = 0; kt < k / 128; ++kt) {
      uint8_t *tile = frag + ((size_t)nt * (k / 128) + kt) * 1024;
      for (uint32_t lane = 0; lane < 64; ++lane) {
        const uint32_t row = nt * 16 + (lane & 15), g = lane >> 4;
        for (uint32_t j = 0; j < 4; ++j) {
          const uint32_t k0 = kt * 128 + (j >> 1) * 64 + g * 16 + (j & 1) * 8;
          for (uint32_t b = 0; b < 4; ++b)
            tile[lane * 16 + j * 4 + b] = (uint8_t)(code(row, k0 + b) | (code(row, k0 + 4 + b) << 4));
        }
      }
    }
  return 0;
}

static void repack_rows(const int8_t *rowmajor, uint32_t rows, uint32_t rows_pad, uint32_t k, uint8_t *frag) {
  for (uint32_t rt = 0; rt < rows_pad / 16; ++rt)
    for (uint32_t kt = 0; kt < k / 64; ++kt) {
      uint8_t *tile = frag + ((size_t)rt * (k / 64) + kt) * 1024;
      for (uint32_t lane = 0; lane < 64; ++lane) {
        const uint32_t row = rt * 16 + (lane & 15), k0 = kt * 64 + (lane >> 4) * 16;
        if (row < rows) memcpy(tile + lane * 16, rowmajor + (size_t)row * k + k0, 16);
        else memset(tile + lane * 16, 0, 16);
      }
    }
}

int saber_iu8_repack_w8(const int8_t *rowmajor, uint32_t n, uint32_t k, uint8_t *frag) {
  if (!rowmajor || !frag) return fail(SABER_IU8_E_ARG, "repack_w8: null buffer");
  if (int rc = shape_ok("repack_w8", n, k)) return rc;
  repack_rows(rowmajor, n, n, k, frag);
  return 0;
}

int saber_iu8_repack_a(const int8_t *rowmajor, uint32_t m, uint32_t k, uint8_t *frag) {
  if (!rowmajor || !frag) return fail(SABER_IU8_E_ARG, "repack_a: null buffer");
  if (m == 0 || k == 0 || k % 64 != 0) return fail(SABER_IU8_E_RULE, fmt("repack_a: M=%u, K=%u must be a multiple of 64", m, k));
  repack_rows(rowmajor, m, (m + 15) / 16 * 16, k, frag);
  return 0;
}

int saber_iu8_unpack_a(const uint8_t *frag, uint32_t m, uint32_t k, int8_t *rowmajor) {
  if (!rowmajor || !frag) return fail(SABER_IU8_E_ARG, "unpack_a: null buffer");
  if (m == 0 || k == 0 || k % 64 != 0) return fail(SABER_IU8_E_RULE, fmt("unpack_a: M=%u, K=%u must be a multiple of 64", m, k));
  for (uint32_t row = 0; row < m; ++row)
    for (uint32_t k0 = 0; k0 < k; k0 += 16) memcpy(rowmajor + (size_t)row * k + k0, frag + saber_iu8_a_offset(row, k0, k), 16);
  return 0;
}

// gfx12 W4 fragment (nt, kk) = 128 B at (nt*K/16 + kk)*128; lane l (0..31) dword at l*4, byte b:
// low nibble = W[nt*16 + l%16][kk*16 + (l/16)*8 + b], high nibble = the same row at k + 4
// (crates/saber-kernels/hip/macaq_iu8.hip:12-15).
int saber_iu8_repack_w4_from_gfx12(const uint8_t *frag12, uint32_t n, uint32_t k, uint8_t *frag) {
  if (!frag12 || !frag) return fail(SABER_IU8_E_ARG, "repack_w4_from_gfx12: null buffer");
  if (int rc = shape_ok("repack_w4_from_gfx12", n, k)) return rc;
  memset(frag, 0, (size_t)n * k / 2);
  for (uint32_t row = 0; row < n; ++row)
    for (uint32_t kk = 0; kk < k; ++kk) {
      const uint32_t r = kk & 15, lane = (row & 15) + 16 * (r >> 3), j = r & 7;
      const uint8_t src = frag12[((size_t)(row >> 4) * (k / 16) + (kk >> 4)) * 128 + lane * 4 + (j & 3)];
      const uint8_t code = (j >> 2) ? (src >> 4) : (src & 15);
      uint32_t high = 0;
      const uint64_t dst = saber_iu8_w4_offset(row, kk, k, &high);
      frag[dst] |= high ? (uint8_t)(code << 4) : code;
    }
  return 0;
}

// gfx12 W8 fragment (nt, kk) = 256 B: lane l's 8 bytes = row nt*16 + l%16, k = kk*16 + (l/16)*8 + 0..7
// (crates/saber-kernels/hip/macaq_iu8.hip:16-17).
int saber_iu8_repack_w8_from_gfx12(const uint8_t *frag12, uint32_t n, uint32_t k, uint8_t *frag) {
  if (!frag12 || !frag) return fail(SABER_IU8_E_ARG, "repack_w8_from_gfx12: null buffer");
  if (int rc = shape_ok("repack_w8_from_gfx12", n, k)) return rc;
  for (uint32_t row = 0; row < n; ++row)
    for (uint32_t kk = 0; kk < k; ++kk) {
      const uint32_t r = kk & 15, lane = (row & 15) + 16 * (r >> 3);
      frag[saber_iu8_a_offset(row, kk, k)] = frag12[((size_t)(row >> 4) * (k / 16) + (kk >> 4)) * 256 + lane * 8 + (r & 7)];
    }
  return 0;
}

}  // extern "C"
