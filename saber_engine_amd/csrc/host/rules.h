// The gfx950 launch law of the iu8 path: which kernel, grid, block, split and workspaces a
// GEMM of m x n x k runs. The counterpart of crates/saber-kernels/src/macaq_iu8.rs
// (cell :286-358, decode_split :267-279, describe :429-489); the tables are this object's own
// speed data (256 CUs in 8 XCDs instead of the reference's 64-CU card).
#pragma once
#include <string>

#include "../../../include/saber_iu8.h"

namespace iu8 {

struct DecVariant {
  const char *name;
  int tm, w8, nt, kw, wpb, depth, alds, acc;
  int block_n() const { return wpb / kw * nt * 16; }
  int threads() const { return wpb * 64; }
};
struct PfVariant {
  const char *name;
  int w8, wmw, wnw, tm, tn, acc, occ;  // waves, 32 x 32 MFMA tiles a wave, workgroups a CU
  int block_m() const { return wmw * tm * 32; }
  int block_n() const { return wnw * tn * 32; }
  int threads() const { return wmw * wnw * 64; }
};

const DecVariant *dec_variant(const std::string &name);
const PfVariant *pf_variant(const std::string &name);
// The prefill cell (tile shape) the launch law picks for a shape.
const PfVariant *pf_cell(bool w8, uint32_t m, uint32_t n, uint32_t k);
uint32_t pf_split(bool w8, uint32_t m, uint32_t n, uint32_t k, const PfVariant **cell);

constexpr uint32_t DECODE_MAX_M = 64;  // the decode band's last row count (macaq_iu8.rs:31)
constexpr uint32_t KS_MAX = 8;         // the largest grid-level split (macaq_iu8.rs:44)
constexpr uint32_t CU_COUNT = 256;     // MI355X compute units
constexpr uint32_t FUSED_A80_MIN_K = 16384;  // two rows at least this long take the 80 KiB fused form
constexpr uint32_t FUSED_R1_MIN_K = 8192;   // rows at least this long take the one-row fused decode form
// the activation producers' 1024-thread forms: rows wider than one group a thread of the 256-thread form, up
// to `ROWS` of them (the quantiser / the activation), or any number of rows at least `WIDE` wide for the activation
constexpr uint32_t MLP_CHAIN_PAYS_INTER_1 = 12288, MLP_CHAIN_PAYS_INTER_2 = 13824;  // one / two rows: the chain beats the three launches from here
constexpr uint32_t S80_MIN_N = 24576;            // the staged persistent GEMV: columns from here at any row count
constexpr uint64_t S80_MIN_BYTES = 64ull << 20;  // the staged persistent GEMV: weights from here at up to 8 rows, and for int8 weights
constexpr uint32_t HAD_T1024_ROWS = 256, HAD_T1024_WIDTH = 4096;  // the Hadamard-basis producers' 16-wave forms: up to / from
constexpr uint32_t T1024_WIDTH_OVER = 4096;
constexpr uint32_t T1024_QUANT_ROWS = 256, T1024_QUANT_ROWS_WIDE = 512;
constexpr uint32_t T1024_SILU_ROWS = 512;
constexpr uint32_t T1024_WIDE = 12288;

// Grid-level split of a decode GEMM whose grid has `nblk` column blocks.
uint32_t decode_split(uint32_t m, uint32_t n, uint32_t k, uint32_t nblk, uint32_t kw);

int resolve(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out);
int describe(const std::string &kernel, uint32_t m, uint32_t n, uint32_t k, uint32_t ks, saber_iu8_desc *out);
// Two W4 decode descriptors of one M, K and kernel -> the one-dispatch pair (macaq_iu8.rs:632-704).
// order: -1 the law's block order, 0 problem 0 first (`pair`), 1 the second problem first (`pairb`).
int pair(const saber_iu8_desc &first, const saber_iu8_desc &second, saber_iu8_desc *out, int order = -1);
const DecVariant *pair_variant(const std::string &name);
int resolve_quant(uint32_t m, uint32_t k, saber_iu8_desc *out);
// The fused quant + GEMV of a decode linear; refuses (by name) shapes it does not hold.
bool fused_holds(uint32_t m, uint32_t k);        // the law: a fused launch is what runs (the 20 KiB form where it holds; the 80 KiB form at 2 rows of K >= 16384)
bool fused_form_holds(bool a80, uint32_t m, uint32_t k);  // what the kernel itself holds: `_tm1` 4 rows / 20 KiB, `_tm1_a80` 16 rows / 80 KiB
bool fused_small_holds(uint32_t m, uint32_t k);  // the 20 KiB form: up to 4 rows (`_tm1`, and the MLP chain's first linear)
bool mlp_chain_pays(uint32_t m, uint32_t hidden, uint32_t inter);        // ... and measured faster than the three launches
bool mlp_chain_form_holds(uint32_t m, uint32_t hidden, uint32_t inter);  // the chain: 20 KiB at the hidden width, 20 or 80 KiB at the intermediate
bool gate_up_act_holds(uint32_t m, uint32_t hidden, uint32_t inter);  // the gate+up linear with the activation in its epilogue
int resolve_gate_up_act(uint32_t m, uint32_t hidden, uint32_t inter, saber_iu8_desc *out);
bool staged80_holds(uint32_t m, uint32_t k);  // up to 16 rows whose codes (rows rounded up to a power of two) fit 80 KiB
uint32_t fused_grid(uint32_t nblk);  // workgroups for nblk column blocks: one a CU, then equal shares of at most 8
int resolve_fused(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out);
// The decode MLP (gate+up -> SiLU * up + requant -> down) as one persistent launch; spin 0 = the default.
constexpr uint32_t MLP_CHAIN_STATE_BYTES = 13 * 1024;  // the kernel's state block (kernels/iu8_chain.h)
constexpr uint32_t MLP_CHAIN_MAX_GRID = 512;           // arrival words and maxima slots in the state block
constexpr uint32_t MLP_CHAIN_SPIN = 1u << 20;  // polls a meeting waits at most (about a microsecond each)
int resolve_mlp_chain(uint32_t m, uint32_t hidden, uint32_t inter, uint32_t spin, saber_iu8_desc *out);
int resolve_silu_mul_quant(uint32_t rows, uint32_t n, saber_iu8_desc *out);
// The rows' scales alone, and the tile GEMM that makes the codes itself from bf16 rows + scales.
int resolve_rowscale(uint32_t m, uint32_t k, saber_iu8_desc *out);
int resolve_prefill_fused(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out);
// Quantisation to row-major codes (q[row * k + col]).
int resolve_quant_rowmajor(uint32_t m, uint32_t k, saber_iu8_desc *out);
// Quantisation through a row map (output row r = input row row_tok[r]).
int resolve_quant_rows(uint32_t rows, uint32_t k, saber_iu8_desc *out);

// The reference's symbol names this object answers through its launch law (band.cpp).
int ref_symbol_by_law(const std::string &kernel, int *w8, const char **note);
std::string band_toml();
std::string device_profile_toml();

// Fills name/offset/size of every slot from the kernel's signature; kinds default to BUFFER.
int fill_slots(const std::string &kernel, saber_iu8_desc *d);
void set_i32(saber_iu8_desc *d, const char *name, int64_t v);
void set_null(saber_iu8_desc *d, const char *name);
void set_buffer(saber_iu8_desc *d, const char *name);

}  // namespace iu8
