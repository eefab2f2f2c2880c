// The gfx950 launch law as data. The reference keeps its iu8 band as tables of its Rust module
// (PF_BAND / PF_TILES / DRAFT_TILES, KS_TARGET_BLOCKS, PAIR_BA_FIRST:
// crates/saber-kernels/src/macaq_iu8.rs:39-48,150-212,549-553) and its device as
// DeviceProfile::gfx1201_reference (crates/saber-plan/src/device.rs:208-258). A host that binds the
// gfx950 objects needs this card's counterparts of those tables; this file writes them out of the
// launch law itself (rules.cpp), so the data cannot drift from what `resolve` does: the cells'
// geometry, the (shape, M range) -> kernel bands over the 27B-class linears, the names of the
// reference's symbol set and what each resolves to here, the routed layer's tile thresholds, the
// pair's block order and the fused decode linear's limits.
#include <cstring>
#include <string>
#include <vector>

#include "../../../include/saber_iu8.h"
#include "abi.h"
#include "rules.h"
#include "util.h"

namespace iu8 {

// The reference's symbol set for this path (macaq_iu8.rs:51-62, 508-547). `same` = this object
// carries a kernel of that name (launched under this object's law); the others name gfx1201 tile
// shapes and resolve to whatever cell the gfx950 law picks for the shape they are asked at.
struct RefSymbol {
  const char *name;
  int w8;        // weight kind the name carries
  bool same;     // a kernel of this name ships in the gfx950 objects
  const char *note;
};
static const RefSymbol REF_SYMBOLS[] = {
    {"macaq_iu8_dec_w4_tm1", 0, true, ""},
    {"macaq_iu8_dec_w4_tm2", 0, true, ""},
    {"macaq_iu8_dec_w4_tm3", 0, true, ""},
    {"macaq_iu8_dec_w4_tm4", 0, true, ""},
    {"macaq_iu8_dec_w8_tm1", 1, true, ""},
    {"macaq_iu8_dec_w8_tm2", 1, true, ""},
    {"macaq_iu8_dec_w8_tm3", 1, true, ""},
    {"macaq_iu8_dec_w8_tm4", 1, true, ""},
    {"macaq_iu8_pf_w4_tn4_lbk64", 0, true, ""},
    {"macaq_iu8_pf_w8_tn4_lbk64", 1, true, ""},
    {"macaq_iu8f_pair_w4_tm1", 0, true, ""},
    {"macaq_iu8f_pair_w4_tm2", 0, true, ""},
    {"macaq_iu8f_pair_w4_tm3", 0, true, ""},
    {"macaq_iu8f_pair_w4_tm4", 0, true, ""},
    {"macaq_iu8f_pairb_w4_tm1", 0, true, ""},
    {"macaq_iu8f_pairb_w4_tm2", 0, true, ""},
    {"macaq_iu8f_pairb_w4_tm3", 0, true, ""},
    {"macaq_iu8f_pairb_w4_tm4", 0, true, ""},
    {"macaq_iu8f_arnq_hadi8_w4_tm1", 0, false, "two-rank all-reduce epilogue: not built (one GPU)"},
    {"macaq_iu8f_arnq_hadi8_w8_tm1", 1, false, "two-rank all-reduce epilogue: not built (one GPU)"},
    {"macaq_iu8f_dec_w4_tm5", 0, false, "law"},
    {"macaq_iu8f_dec_w4_tm6", 0, false, "law"},
    {"macaq_iu8f_dec_w4_tm7", 0, false, "law"},
    {"macaq_iu8f_dec_w4_tm8", 0, false, "law"},
    {"macaq_iu8f_dec_w8_tm5", 1, false, "law"},
    {"macaq_iu8f_dec_w8_tm6", 1, false, "law"},
    {"macaq_iu8f_dec_w8_tm7", 1, false, "law"},
    {"macaq_iu8f_dec_w8_tm8", 1, false, "law"},
    {"macaq_iu8f_pf_w4_bm128", 0, false, "law"},
    {"macaq_iu8f_pf_w4_bm64", 0, false, "law"},
    {"macaq_iu8f_pf_w8_bm128", 1, false, "law"},
    {"macaq_iu8f_pf_w8_bm64", 1, false, "law"},
    {"macaq_iu8f_pf_w4_t1w4n2k128p", 0, false, "law"},
    {"macaq_iu8f_pf_w4_t3w4n4k64p", 0, false, "law"},
    {"macaq_iu8f_pf_w4_t4w4n4k64p", 0, false, "law"},
    {"macaq_iu8f_pf_w4_t5w4n4k64p", 0, false, "law"},
    {"macaq_iu8f_pf_w4_t4w4n2k128p", 0, false, "law"},
    {"macaq_iu8f_pf_w4_t5w2n2k64p", 0, false, "law"},
    {"macaq_iu8f_pf_w8_t1w4n2k128", 1, false, "law"},
    {"macaq_iu8f_pf_w4_t3w2n2k128p", 0, false, "law"},
    {"macaq_iu8f_pf_w4_t3w2n4k64p", 0, false, "law"},
    {"macaq_iu8f_pf_w4_t2w2n2k128p", 0, false, "law"},
    {"macaq_iu8f_pf_w4_t2w4n4k128p", 0, false, "law"},
    {"macaq_iu8f_pf_w8_t3w4n2k64p", 1, false, "law"},
    {"macaq_iu8f_pf_w4_t3w8n4k128p", 0, false, "law"},
};

// 1 when `kernel` is one of the reference's names that this object answers through its launch law
// (*w8 = the weight kind the name carries), 0 when it is not such a name, -1 when the reference's
// symbol has no counterpart here (*note says why).
int ref_symbol_by_law(const std::string &kernel, int *w8, const char **note) {
  for (const RefSymbol &r : REF_SYMBOLS)
    if (kernel == r.name) {
      if (r.same) return 0;
      if (w8) *w8 = r.w8;
      if (note) *note = r.note;
      return strcmp(r.note, "law") == 0 ? 1 : -1;
    }
  return 0;
}

// The linears the bands are written out for: BASELINE's 27B-class layer set, the reference's own
// 27B shapes at TP=1 and TP=2 (macaq_iu8.rs:931-947) and the routed layer's expert shapes.
struct Shape {
  const char *op;
  uint32_t n, k;
};
static const Shape SHAPES[] = {
    {"qkv", 7168, 5120},          {"o", 5120, 5120},          {"gate_up", 34816, 5120},    {"down", 5120, 17408},
    {"gdn_in_proj_qkvz", 16384, 5120}, {"gdn_in_proj_ba", 96, 5120}, {"attn_qkv_gated", 14336, 5120}, {"out_proj", 5120, 6144},
    {"tp2_qkvz", 8192, 5120},     {"tp2_ba", 48, 5120},       {"tp2_out_proj", 5120, 3072}, {"tp2_gate_up", 17408, 5120},
    {"tp2_down", 5120, 8704},     {"expert_gate_up", 3072, 4096}, {"expert_down", 4096, 1536},
};
static const uint32_t M_LAST = 8192;

static void put(std::string &o, const char *key, const std::string &v) { o += std::string(key) + " = \"" + v + "\"\n"; }
static void put(std::string &o, const char *key, uint64_t v) { o += std::string(key) + " = " + std::to_string(v) + "\n"; }
static void putb(std::string &o, const char *key, bool v) { o += std::string(key) + (v ? " = true\n" : " = false\n"); }

std::string band_toml() {
  std::string o;
  o += "# The gfx950 launch law of the W4A8-iu8 GEMMs as data: written by saber_iu8_band_toml (the\n";
  o += "# build step regenerates it; a host test holds it against saber_iu8_resolve). Speed data of one\n";
  o += "# MI355X: every cell gives the same bytes for the same rows.\n";
  put(o, "schema_version", 1);
  put(o, "arch", std::string("gfx950"));
  put(o, "plugin", std::string("macaq_iu8"));
  put(o, "fused_plugin", std::string("macaq_iu8f"));
  put(o, "cu_count", CU_COUNT);
  put(o, "wavefront_size", 64);
  put(o, "decode_max_m", DECODE_MAX_M);
  put(o, "decode_split", 1);
  put(o, "ks_max", KS_MAX);
  put(o, "a_layout_id", SABER_IU8_LAYOUT_A_TILED_I8_64);
  put(o, "w4_layout_id", SABER_IU8_LAYOUT_I4_ROW_FRAG64);
  put(o, "w8_layout_id", SABER_IU8_LAYOUT_I8_ROW_FRAG64);
  put(o, "band_last_m", M_LAST);
  o += "\n[fused_decode_linear]\n";
  o += "# macaq_iu8_decq_{w4,w8}_tm1: quantisation + GEMV in one launch while the rows fit\n";
  put(o, "rows_max", 4);
  put(o, "staged_code_bytes", 20 * 1024);
  put(o, "column_blocks_per_workgroup_max", 8);
  o += "# macaq_iu8_decq_{w4,w8}_r1: one row; the row's codes are made just in time inside the weight stream\n";
  put(o, "r1_rows", 1);
  put(o, "r1_k_min", FUSED_R1_MIN_K);
  put(o, "r1_k_max", 20 * 1024);
  o += "# macaq_iu8_decq_{w4,w8}_tm1_a80: the same launch with 80 KiB of staged codes; the kernel holds up to 16\n";
  o += "# rows, the law launches it for 2 rows of K >= 16384 (every workgroup repeats the quantisation: more rows,\n";
  o += "# and shorter ones, lose to producer + GEMV)\n";
  put(o, "a80_staged_code_bytes", 80 * 1024);
  put(o, "a80_rows_max", 16);
  put(o, "a80_rows_by_law", 2);
  put(o, "a80_k_min_by_law", FUSED_A80_MIN_K);
  put(o, "threads", 1024);
  put(o, "column_block", 32);
  o += "# workgroups for b = ceil(n / 32) column blocks: b while b <= cu_count, else equal shares\n";
  o += "# ceil(b / min(8, ceil(b / cu_count))); the layer shapes:\n";
  for (const Shape &sh : SHAPES) {
    saber_iu8_desc d;
    if (resolve_fused(SABER_IU8_W4, 1, sh.n, sh.k, &d)) continue;
    o += fmt("grid.%s = %u\n", sh.op, d.grid[0]);
  }
  o += "\n[row_producers]\n# macaq_i8_quant_* / macaq_i8_silu_mul_quant_*: 16 waves a row (_t1024) for rows wider than\n";
  o += "# width_over while the row count leaves the card part idle, else the narrowest 256-thread form\n";
  put(o, "t1024_width_over", T1024_WIDTH_OVER);
  put(o, "t1024_quant_rows_max", T1024_QUANT_ROWS);
  put(o, "t1024_quant_rows_max_wide", T1024_QUANT_ROWS_WIDE);
  put(o, "t1024_silu_rows_max", T1024_SILU_ROWS);
  put(o, "t1024_wide", T1024_WIDE);
  o += "\n[mlp_chain]\n";
  o += "# macaq_iu8f_mlp_w4_tm1: gate+up -> SiLU * up + requantisation -> down in one persistent launch while\n";
  o += "# the rows fit the fused form at both widths; every workgroup resident (one a CU).\n";
  o += "# macaq_iu8f_mlp_w4_tm1_a80: the same with the second linear's rows in 80 KiB of staged codes (up to 4 rows)\n";
  put(o, "threads", 1024);
  put(o, "state_bytes", MLP_CHAIN_STATE_BYTES);
  put(o, "spin_default", MLP_CHAIN_SPIN);
  put(o, "workgroups_max", MLP_CHAIN_MAX_GRID);
  o += "# where the one launch measured faster than the three: rows -> least intermediate width\n";
  put(o, "pays_one_row_inter_min", MLP_CHAIN_PAYS_INTER_1);
  put(o, "pays_two_rows_inter_min", MLP_CHAIN_PAYS_INTER_2);
  {
    saber_iu8_desc d;
    if (!resolve_mlp_chain(1, 5120, 17408, 0, &d)) o += fmt("grid.hidden5120_inter17408 = %u\n", d.grid[0]);
    if (!resolve_mlp_chain(4, 5120, 5120, 0, &d)) o += fmt("grid.hidden5120_inter5120 = %u\n", d.grid[0]);
    if (!resolve_mlp_chain(4, 5120, 17408, 0, &d)) o += fmt("a80.grid.hidden5120_inter17408_rows4 = %u\n", d.grid[0]);
  }
  o += "\n[pair]\n# block order by tm: true = the second problem's workgroups first (macaq_iu8f_pairb_*)\n";
  {
    saber_iu8_desc a, b, p;
    o += "second_first = [";
    for (uint32_t tm = 1; tm <= 4; ++tm) {
      const uint32_t m = tm * 16;
      bool bf = false;
      if (!describe(fmt("macaq_iu8_dec_w4_tm%u", tm), m, 12288, 5120, 1, &a) && !describe(fmt("macaq_iu8_dec_w4_tm%u", tm), m, 96, 5120, 1, &b) &&
          !pair(a, b, &p))
        bf = strstr(p.kernel, "pairb") != nullptr;
      o += std::string(bf ? "true" : "false") + (tm < 4 ? ", " : "");
    }
    o += "]\n";
  }
  o += "\n[moe]\n# rows a tile = 16 * tile_blocks by routes an expert (tokens * topk / experts), 128 experts, top-8\n";
  {
    // the thresholds are read off the law itself
    uint32_t t1 = 0, t8 = 0;
    for (uint32_t t = 1; t <= 8192; ++t) {
      const uint32_t tb = saber_iu8_moe_tile_blocks(t, 8, 128);
      if (tb == 1) t1 = t;
      if (tb <= 8) t8 = t;
    }
    put(o, "tile_blocks_1_last_tokens", t1);
    put(o, "tile_blocks_8_last_tokens", t8);
    put(o, "tile_blocks_above", 16);
    // the back half as two launches (activation in gate+up's epilogue, requantisation in front of down's K loop)
    uint32_t tf = 0;
    for (uint32_t t = 1; t <= t1; ++t)
      if (saber_iu8_moe_back_pays(t, 8, 128, 1, 1536)) tf = t;
    put(o, "fused_back_last_tokens", tf);
    uint32_t imax = 0;
    for (uint32_t i = 128; i <= 8192; i += 128)
      if (saber_iu8_moe_back_holds(1, i)) imax = i;
    put(o, "fused_back_inter_max", imax);
  }

  // ---- cells
  std::vector<std::string> seen;
  auto cell_row = [&](const std::string &name) {
    for (const std::string &s : seen)
      if (s == name) return;
    seen.push_back(name);
  };
  // ---- bands
  std::string bands;
  for (int w8 = 0; w8 < 2; ++w8)
    for (const Shape &sh : SHAPES) {
      if (w8 && strncmp(sh.op, "expert", 6) == 0) continue;
      saber_iu8_desc d, first;
      uint32_t run0 = 0;
      auto flush = [&](uint32_t last, const saber_iu8_desc &f, const saber_iu8_desc &l) {
        bands += "\n[[band]]\n";
        put(bands, "op", std::string(sh.op));
        putb(bands, "w8", w8 != 0);
        put(bands, "n", sh.n);
        put(bands, "k", sh.k);
        put(bands, "first_m", run0);
        put(bands, "last_m", last);
        put(bands, "kernel", std::string(f.kernel));
        put(bands, "ks", f.ks);
        put(bands, "block", f.block[0]);
        bands += fmt("grid_first = [%u, %u, %u]\n", f.grid[0], f.grid[1], f.grid[2]);
        bands += fmt("grid_last = [%u, %u, %u]\n", l.grid[0], l.grid[1], l.grid[2]);
        cell_row(f.kernel);
      };
      saber_iu8_desc prev;
      for (uint32_t m = 1; m <= M_LAST; ++m) {
        if (resolve(w8, m, sh.n, sh.k, &d)) continue;
        if (run0 == 0) {
          run0 = m, first = d;
        } else if (strcmp(d.kernel, first.kernel) != 0 || d.ks != first.ks) {
          flush(m - 1, first, prev);
          run0 = m, first = d;
        }
        prev = d;
      }
      if (run0) flush(M_LAST, first, prev);
    }
  o += "\n# ---- the cells the bands name: geometry of a workgroup and how its grid is laid\n";
  for (const std::string &name : seen) {
    o += "\n[[cell]]\n";
    put(o, "kernel", name);
    const bool ks_form = name.size() > 3 && name.compare(name.size() - 3, 3, "_ks") == 0;
    if (const DecVariant *v = dec_variant(name)) {
      put(o, "regime", std::string("decode"));
      putb(o, "w8", v->w8 != 0);
      put(o, "rows_max", (uint64_t)v->tm * 16);
      put(o, "block_n", v->block_n());
      put(o, "threads", v->threads());
      put(o, "grid", std::string("[ceil(n / block_n), 1, ks]"));
      put(o, "kernarg", std::string("dec"));
    } else if (name.rfind("macaq_iu8_dec_w4_tm1_s80", 0) == 0 || name.rfind("macaq_iu8_dec_w8_tm1_s80", 0) == 0) {
      put(o, "regime", std::string("decode"));
      putb(o, "w8", name[15] == '8');
      put(o, "rows_max", 16);
      if (name.back() == 'r') put(o, "staged_code_bytes_max", 80 * 1024);  // rows rounded up to a power of two x K
      else put(o, "k_max", 5120);
      put(o, "block_n", 32);
      put(o, "threads", 1024);
      put(o, "grid", std::string("[blocks = ceil(n / 32); blocks <= cu_count ? blocks : ceil(blocks / min(8, ceil(blocks / cu_count))), 1, 1] persistent"));
      put(o, "kernarg", std::string("dec"));
    } else if (const PfVariant *v = pf_variant(ks_form ? name.substr(0, name.size() - 3) : name)) {
      put(o, "regime", std::string("prefill"));
      putb(o, "w8", v->w8 != 0);
      put(o, "block_m", v->block_m());
      put(o, "block_n", v->block_n());
      put(o, "threads", v->threads());
      put(o, "workgroups_per_cu", v->occ);
      put(o, "grid", std::string(ks_form ? "[min(tiles, cu_count * workgroups_per_cu / ks), 1, ks] persistent"
                                         : "[min(tiles, cu_count * workgroups_per_cu), 1, 1] persistent"));
      put(o, "kernarg", std::string(ks_form ? "dec" : "pf"));
    }
  }
  o += "\n# ---- (op, weight kind, n, k) x rows first_m..last_m -> kernel; grids at both ends of the run\n";
  o += bands;
  o += "\n# ---- the reference's symbol set (macaq_iu8.rs:51-62, 508-547) and what answers it here\n";
  for (const RefSymbol &r : REF_SYMBOLS) {
    o += "\n[[reference_symbol]]\n";
    put(o, "name", std::string(r.name));
    put(o, "answer", std::string(r.same ? "same name, this object's grid and block" : strcmp(r.note, "law") == 0 ? "the law's cell at the shape" : "none"));
    if (!r.same && strcmp(r.note, "law") != 0) put(o, "why", std::string(r.note));
  }
  return o;
}

// The target as the planner's DeviceProfile would hold it (crates/saber-plan/src/device.rs:168-193; the
// gfx1201 instance: device.rs:208-258), in that struct's field names and its serde shape (an enum
// variant with fields is a one-key table, a unit variant a string), so the Rust side can read it with
// the derive it already has. The matrix shapes are this target's MFMA forms under the struct's WMMA name.
std::string device_profile_toml() {
  std::string o;
  o += "# gfx950 (MI355X) as crates/saber-plan/src/device.rs::DeviceProfile: field names and serde shape of that\n";
  o += "# struct. Written by saber_iu8_device_profile_toml; the build step regenerates it.\n";
  put(o, "gfx_target", std::string("gfx950"));
  put(o, "name", std::string("AMD Instinct MI355X"));
  put(o, "cu_count", CU_COUNT);
  put(o, "lds_bytes", 160 * 1024);
  o += "wave_sizes = [64]\n";
  put(o, "infinity_cache_bytes", 256ull << 20);
  put(o, "vram_bytes", 288ull << 30);
  o += "\n[caps]\n";
  putb(o, "fp8_wmma", true);
  putb(o, "int8_wmma", true);
  putb(o, "int4_wmma", false);  // no int4 matrix form: W4 is unpacked to int8 in registers
  putb(o, "sparse_2_4_swmmac", true);
  putb(o, "lds_dma", true);
  putb(o, "nontemporal_loads", true);
  putb(o, "lds_transpose_read", true);
  o += "\n[bandwidths.dram]\n";
  o += "# a streaming read of 1 GiB (four times the Infinity Cache), every workgroup a contiguous span; a\n";
  o += "# grid-stride walk reads 5,000-6,800; the published figure is 8,000\n";
  o += "gbs = 7050.0\n";
  o += "source = { measured_here = { harness = \"iu8_probe_read, 1 GiB in contiguous spans\", when = \"2026-11-25\" } }\n";
  o += "\n[bandwidths.pcie_h2d]\ngbs = 64.0\nsource = \"nominal\"\n";
  o += "\n[bandwidths.p2p]\n# one xGMI link; this build runs on one GPU and never measured it\ngbs = 153.6\nsource = \"nominal\"\n";
  struct Shape { uint32_t m, n, k; const char *ab, *acc; bool sparse; };
  static const Shape MFMA[] = {
      {16, 16, 64, "iu8", "i32", false},      {32, 32, 32, "iu8", "i32", false},     {16, 16, 32, "bf16", "f32", false},
      {32, 32, 16, "bf16", "f32", false},     {16, 16, 32, "fp16", "f32", false},    {32, 32, 16, "fp16", "f32", false},
      {16, 16, 128, "fp8_e4m3", "f32", false}, {32, 32, 64, "fp8_e4m3", "f32", false}, {16, 16, 128, "fp8_e5m2", "f32", false},
      {32, 32, 64, "fp8_e5m2", "f32", false},  {16, 16, 128, "iu8", "i32", true},      {32, 32, 64, "iu8", "i32", true}};
  for (const Shape &w : MFMA) {
    o += "\n[[wmma_shapes]]\n";
    put(o, "m", w.m);
    put(o, "n", w.n);
    put(o, "k", w.k);
    put(o, "a_dtype", std::string(w.ab));
    put(o, "b_dtype", std::string(w.ab));
    put(o, "acc_dtype", std::string(w.acc));
    putb(o, "sparse_2_4", w.sparse);
  }
  return o;
}

}  // namespace iu8

static int text_out(const std::string &t, const char *what, char *buf, size_t cap, size_t *need) {
  if (need) *need = t.size() + 1;
  if (!buf || cap < t.size() + 1) return buf ? iu8::fail(SABER_IU8_E_ARG, std::string(what) + ": buffer too small") : 0;
  memcpy(buf, t.c_str(), t.size() + 1);
  return 0;
}

extern "C" int saber_iu8_device_profile_toml(char *buf, size_t cap, size_t *need) {
  return text_out(iu8::device_profile_toml(), "device_profile_toml", buf, cap, need);
}

extern "C" int saber_iu8_band_toml(char *buf, size_t cap, size_t *need) {
  const std::string t = iu8::band_toml();
  if (need) *need = t.size() + 1;
  if (!buf || cap < t.size() + 1) return buf ? iu8::fail(SABER_IU8_E_ARG, "band_toml: buffer too small") : 0;
  memcpy(buf, t.c_str(), t.size() + 1);
  return 0;
}
