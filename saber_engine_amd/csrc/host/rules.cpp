#include "rules.h"

#include <cmath>
#include <cstring>

#include "abi.h"
#include "util.h"

namespace iu8 {

static const DecVariant DEC_VARIANTS[] = {
#define IU8_DEC_VARIANT(name, TM, W8, NT, KW, WPB, D, ALDS, ACC) {#name, TM, W8, NT, KW, WPB, D, ALDS, ACC},
#define IU8_DEC_TAP(name, TM, W8, NT, KW, WPB, D, ALDS, ACC) {#name, TM, W8, NT, KW, WPB, D, ALDS, ACC},
#include "../kernels/iu8_variants.def"
};
static const PfVariant PF_VARIANTS[] = {
#define IU8_PF_VARIANT(name, W8, WMW, WNW, TM, TN, ACC, ST, OCC, DEEP) {#name, W8, WMW, WNW, TM, TN, ACC, OCC},
#define IU8_PF_TAP(name, W8, WMW, WNW, TM, TN, ACC, ST, OCC, DEEP) {#name, W8, WMW, WNW, TM, TN, ACC, OCC},
#include "../kernels/iu8_variants.def"
};
static const DecVariant PAIR_VARIANTS[] = {
#define IU8_PAIR_VARIANT(name, TM, NT, KW, WPB, D, ALDS, BFIRST) {#name, TM, false, NT, KW, WPB, D, ALDS, false},
#include "../kernels/iu8_variants.def"
};

const DecVariant *dec_variant(const std::string &name) {
  for (const DecVariant &v : DEC_VARIANTS)
    if (name == v.name) return &v;
  return nullptr;
}
const DecVariant *pair_variant(const std::string &name) {
  for (const DecVariant &v : PAIR_VARIANTS)
    if (name == v.name) return &v;
  return nullptr;
}
const PfVariant *pf_variant(const std::string &name) {
  for (const PfVariant &v : PF_VARIANTS)
    if (name == v.name) return &v;
  return nullptr;
}

static void copy_name(char *dst, size_t cap, const std::string &s) {
  snprintf(dst, cap, "%s", s.c_str());
}

int fill_slots(const std::string &kernel, saber_iu8_desc *d) {
  const Signature *sig = signature_for(kernel);
  if (!sig) return fail(SABER_IU8_E_RULE, kernel + ": no declared signature");
  std::vector<std::pair<uint32_t, uint32_t>> packed;
  d->kernarg_bytes = pack(*sig, packed);
  if (sig->size() > sizeof(d->args) / sizeof(d->args[0])) return fail(SABER_IU8_E_RULE, kernel + ": too many arguments");
  d->n_args = (uint32_t)sig->size();
  for (size_t i = 0; i < sig->size(); ++i) {
    saber_iu8_slot &s = d->args[i];
    memset(&s, 0, sizeof s);
    copy_name(s.name, sizeof s.name, (*sig)[i].name);
    s.offset = packed[i].first;
    s.size = packed[i].second;
    s.kind = (*sig)[i].kind == ArgKind::Buffer ? SABER_IU8_ARG_BUFFER
             : (*sig)[i].kind == ArgKind::F32  ? SABER_IU8_ARG_F32
             : (*sig)[i].kind == ArgKind::I64  ? SABER_IU8_ARG_I64
                                               : SABER_IU8_ARG_I32;
  }
  return 0;
}

void set_i32(saber_iu8_desc *d, const char *name, int64_t v) {
  for (uint32_t i = 0; i < d->n_args; ++i)
    if (!strcmp(d->args[i].name, name)) {
      d->args[i].kind = d->args[i].size == 8 ? SABER_IU8_ARG_I64 : SABER_IU8_ARG_I32;
      d->args[i].ival = v;
    }
}
void set_buffer(saber_iu8_desc *d, const char *name) {
  for (uint32_t i = 0; i < d->n_args; ++i)
    if (!strcmp(d->args[i].name, name)) d->args[i].kind = SABER_IU8_ARG_BUFFER;
}
void set_null(saber_iu8_desc *d, const char *name) {
  for (uint32_t i = 0; i < d->n_args; ++i)
    if (!strcmp(d->args[i].name, name)) d->args[i].kind = SABER_IU8_ARG_NULL_BUFFER;
}

static void add_ws(saber_iu8_desc *d, const char *name, uint32_t kind, uint64_t bytes, uint32_t zero_once) {
  saber_iu8_workspace &w = d->workspaces[d->n_workspaces++];
  memset(&w, 0, sizeof w);
  copy_name(w.name, sizeof w.name, name);
  w.kind = kind;
  w.bytes = bytes;
  w.zero_once = zero_once;
}

static int check_shape(const char *op, uint32_t m, uint32_t n, uint32_t k) {
  // the reference's refusals (macaq_iu8.rs:288-297), by name
  if (m == 0 || n == 0 || k == 0)
    return fail(SABER_IU8_E_RULE, fmt("%s: %u x %u x %u has nothing to do; an empty launch is a caller bug", op, m, n, k));
  if (n % 16 != 0 || k % 128 != 0)
    return fail(SABER_IU8_E_RULE,
                fmt("%s: N=%u must be a multiple of 16 (whole fragments) and K=%u of 128 (the slab)", op, n, k));
  return 0;
}

// The grid-level split of a decode GEMM. The k-waves of a workgroup already split K through LDS, and
// a split across workgroups adds 1.5-2 us of hand-over (partials through memory, a device-scope
// counter) to launches whose fixed cost dominates: measured on the 27B-class shapes it never wins
// by more than the noise, so the law does not split; `describe` still takes an explicit count.
uint32_t decode_split(uint32_t, uint32_t, uint32_t, uint32_t, uint32_t) { return 1; }

static int describe_dec(const DecVariant &v, uint32_t m, uint32_t n, uint32_t k, uint32_t ks, saber_iu8_desc *d) {
  const char *op = v.w8 ? "gemm_i8a8" : "gemm_i4a8";
  if (int rc = check_shape(op, m, n, k)) return rc;
  if (m > (uint32_t)v.tm * 16) return fail(SABER_IU8_E_RULE, fmt("%s: %s holds %d rows, M=%u", op, v.name, v.tm * 16, m));
  if (ks == 0 || ks > k / 128) return fail(SABER_IU8_E_RULE, fmt("%s: split %u of %u K steps", op, ks, k / 128));
  memset(d, 0, sizeof *d);
  copy_name(d->op, sizeof d->op, op);
  copy_name(d->plugin, sizeof d->plugin, "macaq_iu8");
  copy_name(d->kernel, sizeof d->kernel, v.name);
  const uint32_t nblk = (n + v.block_n() - 1) / v.block_n();
  d->grid[0] = nblk, d->grid[1] = 1, d->grid[2] = ks;
  d->block[0] = v.threads(), d->block[1] = 1, d->block[2] = 1;
  d->n_launches = 1;
  d->ks = ks;
  if (int rc = fill_slots(v.name, d)) return rc;
  set_i32(d, "m", m);
  set_i32(d, "n", n);
  set_i32(d, "k", k);
  if (ks == 1) {
    // named-null at ks 1: the kernel must not dereference them (macaq_iu8.rs:447-451)
    set_null(d, "decode_partial");
    set_null(d, "decode_counter");
  } else {
    add_ws(d, "decode_partial", SABER_IU8_WS_SCRATCH, (uint64_t)ks * m * n * 4, 0);
    add_ws(d, "decode_counter", SABER_IU8_WS_PERSISTENT, (uint64_t)nblk * 4, 1);
  }
  return 0;
}

// `ks` > 0 names the cell's split form (`<cell>_ks`, the decode kernarg list): gridDim.z shares of the
// K steps, none of them empty, `grid[0]` persistent workgroups a share.
static int describe_pf(const PfVariant &v, uint32_t m, uint32_t n, uint32_t k, uint32_t ks, saber_iu8_desc *d) {
  const char *op = v.w8 ? "gemm_i8a8" : "gemm_i4a8";
  if (int rc = check_shape(op, m, n, k)) return rc;
  // the tile GEMM addresses its operands with 32-bit byte offsets from a per-step base
  const uint64_t a_bytes = (uint64_t)((m + 15) / 16 * 16) * k, w_bytes = (uint64_t)n * k / (v.w8 ? 1 : 2);
  if (a_bytes > 0xFFFFFFFFull || w_bytes > 0xFFFFFFFFull)
    return fail(SABER_IU8_E_RULE, fmt("%s: %u x %u x %u puts an operand past 4 GiB (A %llu B, W %llu B), more than the tile GEMM addresses",
                                      op, m, n, k, (unsigned long long)a_bytes, (unsigned long long)w_bytes));
  const std::string name = std::string(v.name) + (ks ? "_ks" : "");
  if (ks) {
    const uint32_t steps = k / 128, spb = (steps + ks - 1) / ks;
    if (ks > steps || (uint64_t)spb * (ks - 1) >= steps)
      return fail(SABER_IU8_E_RULE, fmt("%s: %u shares of %u K steps would leave one empty", op, ks, steps));
  }
  memset(d, 0, sizeof *d);
  copy_name(d->op, sizeof d->op, op);
  copy_name(d->plugin, sizeof d->plugin, "macaq_iu8");
  copy_name(d->kernel, sizeof d->kernel, name);
  const uint32_t gx = (n + v.block_n() - 1) / v.block_n(), gy = (m + v.block_m() - 1) / v.block_m();
  // persistent: OCC workgroups a CU walk the tiles (the kernel derives gx, gy from m, n)
  const uint64_t tiles = (uint64_t)gx * gy, slots = std::max<uint64_t>(1, (uint64_t)CU_COUNT * v.occ / std::max(ks, 1u));
  d->grid[0] = (uint32_t)(tiles < slots ? tiles : slots), d->grid[1] = 1, d->grid[2] = std::max(ks, 1u);
  d->block[0] = v.threads(), d->block[1] = 1, d->block[2] = 1;
  d->n_launches = 1;
  d->ks = std::max(ks, 1u);
  if (int rc = fill_slots(name, d)) return rc;
  set_i32(d, "m", m);
  set_i32(d, "n", n);
  set_i32(d, "k", k);
  if (ks == 1) {
    set_null(d, "decode_partial");
    set_null(d, "decode_counter");
  } else if (ks > 1) {
    add_ws(d, "decode_partial", SABER_IU8_WS_SCRATCH, (uint64_t)ks * m * n * 4, 0);
    add_ws(d, "decode_counter", SABER_IU8_WS_PERSISTENT, tiles * 4, 1);
  }
  return 0;
}

static uint64_t staged_bytes(uint32_t m, uint32_t k);
// The streaming decode cell of M rows: tm 16-row tiles; one tile's live rows staged in LDS when they fit the 20 KiB
// form, else streamed from L2 beside the weights.
static std::string dec_stream_name(const char *tag, uint32_t m, uint32_t k) {
  const uint32_t tm = (m + 15) / 16;
  std::string name = fmt("macaq_iu8_dec_%s_tm%u", tag, tm);
  if (tm == 1) {
    uint32_t mr = 1;
    while (mr < m) mr *= 2;
    if ((uint64_t)mr * k > 20 * 1024) name += "_a0";
  }
  return name;
}

// The persistent GEMV of up to 16 quantised rows whose 16-row tile is staged once a workgroup in 80 KiB of LDS
// (`macaq_iu8_dec_{w4,w8}_tm1_s80`): the fused forms' geometry (16 waves, 32 columns a block, at most 8 blocks a
// workgroup) on the decode kernarg list.
bool staged80_holds(uint32_t m, uint32_t k) { return m >= 1 && m <= 16 && staged_bytes(m, k) <= 80 * 1024; }
static bool staged80_tile_holds(uint32_t m, uint32_t k) { return m >= 1 && m <= 16 && (uint64_t)k * 16 <= 80 * 1024; }
// `rows_form`: the kernel that takes the live rows' pieces of the tile (`_s80r`: few rows of a long K); else the
// whole-tile kernel (`_s80`, K <= 5120 at any row count)
static int describe_s80(bool w8, bool rows_form, uint32_t m, uint32_t n, uint32_t k, uint32_t ks, saber_iu8_desc *d) {
  const char *op = w8 ? "gemm_i8a8" : "gemm_i4a8";
  const std::string name = fmt("macaq_iu8_dec_%s_tm1_s80%s", w8 ? "w8" : "w4", rows_form ? "r" : "");
  if (int rc = check_shape(op, m, n, k)) return rc;
  if (ks != 1) return fail(SABER_IU8_E_RULE, name + ": the staged form does not split K");
  if (rows_form ? !staged80_holds(m, k) : !staged80_tile_holds(m, k))
    return fail(SABER_IU8_E_RULE, rows_form ? fmt("%s: %u rows (rounded up to a power of two) of %u do not fit 80 KiB", name.c_str(), m, k)
                                            : fmt("%s: %u rows of %u do not fit one 16-row tile in 80 KiB (K <= 5120)", name.c_str(), m, k));
  memset(d, 0, sizeof *d);
  copy_name(d->op, sizeof d->op, op);
  copy_name(d->plugin, sizeof d->plugin, "macaq_iu8");
  copy_name(d->kernel, sizeof d->kernel, name);
  d->grid[0] = fused_grid((n + 31) / 32), d->grid[1] = 1, d->grid[2] = 1;
  d->block[0] = 1024, d->block[1] = 1, d->block[2] = 1;
  d->n_launches = 1;
  d->ks = 1;
  if (int rc = fill_slots(name, d)) return rc;
  set_i32(d, "m", m);
  set_i32(d, "n", n);
  set_i32(d, "k", k);
  set_null(d, "decode_partial");
  set_null(d, "decode_counter");
  return 0;
}

int describe(const std::string &kernel, uint32_t m, uint32_t n, uint32_t k, uint32_t ks, saber_iu8_desc *out) {
  if (kernel == "macaq_iu8_dec_w4_tm1_s80" || kernel == "macaq_iu8_dec_w8_tm1_s80") return describe_s80(kernel[15] == '8', false, m, n, k, ks, out);
  if (kernel == "macaq_iu8_dec_w4_tm1_s80r" || kernel == "macaq_iu8_dec_w8_tm1_s80r") return describe_s80(kernel[15] == '8', true, m, n, k, ks, out);
  if (const DecVariant *v = dec_variant(kernel)) return describe_dec(*v, m, n, k, ks, out);
  if (const PfVariant *v = pf_variant(kernel)) {
    if (ks != 1) return fail(SABER_IU8_E_RULE, kernel + ": the prefill tile does not split K (its `_ks` form does)");
    return describe_pf(*v, m, n, k, 0, out);
  }
  if (kernel.size() > 3 && kernel.compare(kernel.size() - 3, 3, "_ks") == 0)
    if (const PfVariant *v = pf_variant(kernel.substr(0, kernel.size() - 3))) {
      if (!signature_for(kernel)) return fail(SABER_IU8_E_RULE, kernel + ": no such split form");
      return describe_pf(*v, m, n, k, ks, out);
    }
  // the tile GEMM with the quantisation fused into its A-tile load: the geometry of the cell it names
  if (kernel.rfind("macaq_iu8_pfq_", 0) == 0)
    if (const PfVariant *v = pf_variant("macaq_iu8_pf_" + kernel.substr(14))) {
      // the cells that have a fused-quant form (registers for the bf16 pieces in flight, whole A fragments a wave)
      static const char *const PFQ[] = {"w4_t128x128", "w8_t128x128", "w4_t128x128_o2", "w4_t256x160", "w8_t256x160"};
      bool has = false;
      for (const char *c : PFQ) has = has || kernel.substr(14) == c;
      if (!has || ks != 1) return fail(SABER_IU8_E_RULE, kernel + ": no such fused-quant form");
      if ((uint64_t)m * k * 2 > 0xFFFFFFFFull) return fail(SABER_IU8_E_RULE, fmt("%s: %u rows of %u bf16 pass 4 GiB", kernel.c_str(), m, k));
      if (int rc = describe_pf(*v, m, n, k, 0, out)) return rc;
      copy_name(out->kernel, sizeof out->kernel, kernel);
      copy_name(out->op, sizeof out->op, v->w8 ? "linear_i8a8_pfq" : "linear_i4a8_pfq");
      if (int rc = fill_slots(kernel, out)) return rc;
      set_i32(out, "m", m), set_i32(out, "n", n), set_i32(out, "k", k);
      return 0;
    }
  // a name of the reference's symbol set that this object does not carry (gfx1201 tile shapes): the
  // request is for the op at this shape, and the gfx950 law picks the cell
  int w8 = 0;
  const char *note = "";
  const int r = ref_symbol_by_law(kernel, &w8, &note);
  if (r > 0) {
    if (ks != 1) return fail(SABER_IU8_E_RULE, kernel + ": answered by the launch law, which picks the split itself");
    return resolve(w8 ? SABER_IU8_W8 : SABER_IU8_W4, m, n, k, out);
  }
  if (r < 0) return fail(SABER_IU8_E_RULE, kernel + ": " + note);
  return fail(SABER_IU8_E_RULE, kernel + ": not a kernel of the macaq_iu8 object");
}

static bool int_arg(const saber_iu8_desc &d, const char *name, int64_t *v) {
  for (uint32_t i = 0; i < d.n_args; ++i)
    if (!strcmp(d.args[i].name, name) && (d.args[i].kind == SABER_IU8_ARG_I32 || d.args[i].kind == SABER_IU8_ARG_I64)) {
      *v = d.args[i].ival;
      return true;
    }
  return false;
}

// The decode pair: each half is exactly the descriptor `resolve` / `describe` gave it alone (its
// split count, its partial slab and counters), the two grids end to end, problem 0 first
// (macaq_iu8.rs:632-704). Refused unless both halves are W4 decode cells of one kernel (so one row
// tiling and one staging form), M and K.
int pair(const saber_iu8_desc &first, const saber_iu8_desc &second, saber_iu8_desc *out, int order) {
  static const char PREFIX[] = "macaq_iu8_dec_w4_";
  // a half the law gave the staged persistent form is paired as its streamed form: the pair kernels are that geometry
  for (const saber_iu8_desc *h : {&first, &second})
    if (!strncmp(h->kernel, "macaq_iu8_dec_w4_tm1_s80", 24)) {
      saber_iu8_desc s[2];
      const saber_iu8_desc *in[2] = {&first, &second};
      for (int i = 0; i < 2; ++i) {
        int64_t hm = 0, hn = 0, hk = 0;
        s[i] = *in[i];
        if (!strncmp(in[i]->kernel, "macaq_iu8_dec_w4_tm1_s80", 24)) {
          if (!int_arg(*in[i], "m", &hm) || !int_arg(*in[i], "n", &hn) || !int_arg(*in[i], "k", &hk))
            return fail(SABER_IU8_E_RULE, "macaq iu8 pair: a half without its m, n, k");
          if (int rc = describe(dec_stream_name("w4", (uint32_t)hm, (uint32_t)hk), (uint32_t)hm, (uint32_t)hn, (uint32_t)hk, 1, &s[i])) return rc;
        }
      }
      return pair(s[0], s[1], out, order);
    }
  const std::string k0 = first.kernel, k1 = second.kernel;
  const DecVariant *v0 = dec_variant(k0), *v1 = dec_variant(k1);
  int64_t m0 = 0, kk0 = 0, n0 = 0, m1 = 0, kk1 = 0, n1 = 0;
  const bool ints = int_arg(first, "m", &m0) && int_arg(first, "k", &kk0) && int_arg(first, "n", &n0) &&
                    int_arg(second, "m", &m1) && int_arg(second, "k", &kk1) && int_arg(second, "n", &n1);
  if (!v0 || !v1 || !ints || v0->w8 || v1->w8 || v0->acc || v1->acc || k0 != k1 || m0 != m1 || kk0 != kk1)
    return fail(SABER_IU8_E_RULE, fmt("macaq iu8 pair: halves `%s` M %lld K %lld and `%s` M %lld K %lld are not two W4 cells of one M, K",
                                      k0.c_str(), (long long)m0, (long long)kk0, k1.c_str(), (long long)m1, (long long)kk1));
  // The block order by tm (speed data; both orders give the same bytes): the second problem's
  // workgroups first (`pairb`), as the reference's PAIR_BA_FIRST has it at every tm
  // (macaq_iu8.rs:549-553) -- the small half then does not sit in the launch's tail.
  static const bool PAIR_B_FIRST[4] = {true, true, true, true};
  const bool b_first = order < 0 ? PAIR_B_FIRST[std::min(std::max(v0->tm, 1), 4) - 1] : order > 0;
  const char *form = b_first ? "pairb" : "pair";
  const std::string name = std::string("macaq_iu8f_") + form + "_w4_" + k0.substr(sizeof PREFIX - 1);
  const DecVariant *pv = pair_variant(name);
  if (!pv) return fail(SABER_IU8_E_RULE, name + ": the fused object carries no such pair");
  const uint32_t nb0 = first.grid[0], nb1 = second.grid[0], ks0 = first.ks, ks1 = second.ks;
  memset(out, 0, sizeof *out);
  copy_name(out->op, sizeof out->op, "gemm_i4a8_pair");
  copy_name(out->plugin, sizeof out->plugin, "macaq_iu8f");
  copy_name(out->kernel, sizeof out->kernel, name);
  out->grid[0] = nb0 * ks0 + nb1 * ks1, out->grid[1] = 1, out->grid[2] = 1;
  out->block[0] = pv->threads(), out->block[1] = 1, out->block[2] = 1;
  out->n_launches = 1;
  out->ks = 1;
  if (int rc = fill_slots(name, out)) return rc;
  set_i32(out, "m", m0), set_i32(out, "k", kk0);
  set_i32(out, "n", n0), set_i32(out, "ks", ks0), set_i32(out, "nb", nb0);
  set_i32(out, "n_b", n1), set_i32(out, "ks_b", ks1), set_i32(out, "nb_b", nb1);
  const saber_iu8_desc *half[2] = {&first, &second};
  for (int h = 0; h < 2; ++h) {
    const char *sfx = h ? "_b" : "";
    const std::string p = std::string("decode_partial") + sfx, c = std::string("decode_counter") + sfx;
    if (half[h]->ks == 1) {
      set_null(out, p.c_str()), set_null(out, c.c_str());
    } else {
      for (uint32_t i = 0; i < half[h]->n_workspaces; ++i) {
        const saber_iu8_workspace &w = half[h]->workspaces[i];
        add_ws(out, (std::string(w.name) + sfx).c_str(), w.kind, w.bytes, w.zero_once);
      }
    }
  }
  return 0;
}

int resolve(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out) {
  if (wkind != SABER_IU8_W4 && wkind != SABER_IU8_W8) return fail(SABER_IU8_E_ARG, "unknown weight kind");
  const char *tag = wkind == SABER_IU8_W8 ? "w8" : "w4";
  if (int rc = check_shape(wkind == SABER_IU8_W8 ? "gemm_i8a8" : "gemm_i4a8", m, n, k)) return rc;
  // The decode band ends where the tile GEMM's small cells overtake the streaming form (speed data of
  // this card: 17..32 rows stream unless the output is very wide, 33..48 unless it is wide, from 49
  // rows the tiles win on every shape measured).
  // A deep, narrow linear leaves the band at 33 rows already: where the tile law shares K over workgroups
  // (pf_split), its 64 x 128 cell overtakes the three-tile streaming form (5120 x 17408 at 33 / 40 / 48 rows:
  // 23.7 / 23.9 / 25.8 us on four shares against 28.2 / 28.3 / 31.3; up to 32 rows streaming wins, 18.0 against 22.4).
  const PfVariant *split_cell = nullptr;
  const uint32_t tile_ks = pf_split(wkind == SABER_IU8_W8, m, n, k, &split_cell);
  const bool stream = m <= 16 || (m <= 32 && n <= 16384) || (m <= 48 && n <= 8192 && tile_ks == 0);
  if (m <= DECODE_MAX_M && stream) {
    // Up to 16 rows of K <= 5120: the persistent form that stages the 16-row tile once a workgroup (`_s80`) where
    // it measured faster than the streamed one, which re-reads the tile from L2 once a 32-column block. W4, 9-16
    // rows: everywhere (gate+up 34816 x 5120 19.1 -> 16.6 us, 28672 x 4096 13.2 -> 12.1, 14336 x 5120 9.4 -> 9.0,
    // QKV / O 6.1 / 5.9 -> 6.05 / 5.8); up to 8 rows, and int8 weights at any row count, from 64 MiB of weights
    // (W4 5-8 rows: gate+up 16.6-17.9 -> 16.4-17.2, 28672 x 4096 even, 14336 x 5120 8.5 -> 9.0 the other way;
    // W8: gate+up 31.3 -> 28.4, 28672 x 4096 21.0 -> 19.9, 14336 x 5120 14.3 -> 13.6, QKV 8.1 -> 8.4 the other way).
    // A wide N (from 24,576 columns: three and more column blocks a workgroup) takes it at any row count, also against the
    // staged 20 KiB form of 1-4 rows, which starts a workgroup a block (W4 gate+up at 1 / 2 / 4 rows 17.6 / 16.4 / 16.7 ->
    // 16.6 / 15.8 / 16.35, 24576 x 2048 7.5-7.6 -> 6.85-6.9, 28672 x 4096 12.1-12.25 -> 11.2-11.9; W8 gate+up 29.2-30.8 ->
    // 27.9-29.0; at 14336 columns and fewer it loses 0.1-0.7 us there).
    if (k <= 5120 && staged80_holds(m, k) &&
        ((m > 8 && wkind == SABER_IU8_W4) || n >= S80_MIN_N ||
         (m > 4 && (uint64_t)n * k / (wkind == SABER_IU8_W8 ? 1 : 2) >= S80_MIN_BYTES)))
      return describe_s80(wkind == SABER_IU8_W8, false, m, n, k, 1, out);
    // ... and 2 to 4 rows of a long K, whose live rows' codes fit the same 80 KiB (the copy takes their pieces of the
    // tile): 5120 x 17408 at 2 / 3 / 4 rows 11.0 -> 10.5 / 10.7 / 10.7 us; at K = 6144 and 8704 (5.7 -> 5.8, 6.9 -> 6.9)
    // and on 16384 x 8192 (12.4 -> 12.8) the streamed form stays
    if (m >= 2 && m <= 4 && k >= 16384 && wkind == SABER_IU8_W4 && staged80_holds(m, k))
      return describe_s80(false, true, m, n, k, 1, out);
    const std::string name = dec_stream_name(tag, m, k);
    const DecVariant *v = dec_variant(name);
    if (!v) return fail(SABER_IU8_E_RULE, name + ": no such variant");
    const uint32_t nblk = (n + v->block_n() - 1) / v->block_n();
    return describe_dec(*v, m, n, k, decode_split(m, n, k, nblk, v->kw), out);
  }
  if (tile_ks) return describe_pf(*split_cell, m, n, k, tile_ks, out);
  return describe_pf(*pf_cell(wkind == SABER_IU8_W8, m, n, k), m, n, k, 0, out);
}

// K shares of a tile launch (0: none). A deep, narrow linear at a few dozen rows gives the unsplit
// law so few tiles that half to two thirds of the CUs idle through hundreds of K steps; there, 2-4 workgroups
// a tile of the 64x128 cell, each on a share of K, measured 9-19 % faster although the partials
// travel through memory (5120 x 17408: M=64 34.1 -> 28.6 us, M=128 33.6 -> 30.7 us). On every other
// shape timed (K <= 6144 at any M, more than 128 tiles at any K, 256 rows and more) the unsplit cell won --
// the partials cost ks*M*N*4 bytes each way and the last arriver sums alone -- so the rule is this
// narrow. The launch then needs the `decode_partial` / `decode_counter` workspaces the descriptor lists.
uint32_t pf_split(bool w8, uint32_t m, uint32_t n, uint32_t k, const PfVariant **cell) {
  // measured at 33..192 rows; above, the partials (ks * M * N * 4 bytes each way) grow with M (at 256 rows the unsplit
  // cell is level or ahead: 5120 x 17408 43.9 against 43.9-58.6 us). Up to 128 tiles, i.e. two shares at least:
  // 81-128 tiles on two shares against the law's unsplit pick, us -- 5120 x 17408 at 129 / 160 / 192 rows 33.7 / 34.1 /
  // 35.3 against 35.4 / 36.7 / 36.5, 5120 x 20480 38.2 / 38.8 / 38.4 against 40.4 / 42.1 / 42.5, 4096 x 16384 31.0 / 31.4 /
  // 32.0 against 32.3 / 33.4 / 33.6; 8192 x 16384 at 96 / 128 rows 33.0 / 34.6 against 36.4 / 37.9, 12288 x 16384 at
  // 49 / 64 rows 33.3 / 34.6 against 35.8 / 35.5; 72 tiles on three shares (3072 x 16384 at 129-192 rows) 28.1-28.7
  // against 31.7-32.0.
  if (w8 || k < 16384 || m > 192) return 0;
  const PfVariant *v = pf_variant("macaq_iu8_pf_w4_t64x128_s");
  if (!v || !signature_for(std::string(v->name) + "_ks")) return 0;
  const uint64_t tiles = (uint64_t)((n + v->block_n() - 1) / v->block_n()) * ((m + v->block_m() - 1) / v->block_m());
  if (tiles > 128) return 0;
  *cell = v;
  return (uint32_t)std::min<uint64_t>(4, CU_COUNT / tiles);
}

// The prefill cell of a shape: the tile whose estimated time is least. A launch's time is a fixed
// cost, a cost a tile the busiest workgroup runs (pipeline fill, epilogue, tile switch: what a cell pays
// whatever K is) and the largest of three: the matrix work of the busiest CU over the cell's measured rate
// (co-resident workgroups of a two-a-CU cell share the CU's matrix units), the bytes that CU pulls in
// (its tiles' A rows and W columns, K deep) over what one CU takes from L2, and all tiles' bytes over
// what the L2s deliver together -- the last two are what bind for M up to about 512, where the A rows
// are re-read once a column block, so small tiles that put every CU to work win there and the large
// ones take over as the matrix work grows -- or the weights' way from memory, once for every row tile
// that runs beside another on the same column block (the wide gate+up at 256 rows on 128-row tiles). The constants are this card's speed data, one table a weight
// kind (int8 weights are twice the bytes a tile and have no unpack: the cells rank differently), fitted to
// sustained timings of every cell on the four 27B-class shapes x 14 row counts from 65 to 8,192, weights
// cold (successive launches walk copies that exceed the memory-side cache; with warm weights the 64 x 64
// cell overtakes the 64 x 128 one at 256 rows, which no layer of a model sees), and checked on shapes the fit had
// not seen -- the served 27B graph's own 16384 x 5120, 14336 x 5120, 5120 x 6144 and 96 x 5120 at eight row counts,
// which moved three small-cell rates and took the side-by-side term off the 64-row cells. W4: 850 timings, the
// pick is within 0.6 % of the fastest measured cell on all 88 shape x M points; W8, output-side shapes: every
// pick the fastest. The reference keeps its band tables the same way
// (crates/saber-kernels/src/macaq_iu8.rs:150-212). One table for both kinds had sent the int8-weight
// O and down projections at 2,048 rows to the 128 x 320 cell, 17-22 % behind the 256 x 160 cell there.
const PfVariant *pf_cell(bool w8, uint32_t m, uint32_t n, uint32_t k) {
  struct Cell { const char *tile; double tops_per_cu, tile_us; };
  struct Law { double fixed_us, cu_gbps, l2_tbps, lone, hbm_tbps, side_cap; Cell cells[11]; };
  static const Law W4 = {0.974, 90.000, 19.875, 1.422, 3.113, 2.116,
                         {{"tn4_lbk64", 14.007, 3.223}, {"t256x320", 13.568, 4.138}, {"t256x224", 13.814, 14.000}, {"t128x320", 11.147, 7.968}, {"t256x160", 11.173, 8.857}, {"t128x256", 9.046, 1.844}, {"t128x128", 8.799, 2.045}, {"t128x128_o2", 9.622, 3.231}, {"t128x64_s", 4.711, 1.952}, {"t64x128_s", 6.085, 2.027}, {"t64x64_s", 5.582, 1.829}}};
  static const Law W8 = {4.419, 75.175, 18.116, 1.782, 5.234, 1.935,
                         {{"tn4_lbk64", 13.145, 0.244}, {"t256x320", 12.800, 0.000}, {"t256x224", 11.270, 0.000}, {"t128x320", 6.328, 2.194}, {"t256x160", 11.499, 0.000}, {"t128x256", 10.761, 3.251}, {"t128x128", 8.069, 0.427}, {"t128x128_o2", 8.619, 0.229}, {"t128x64_s", 4.123, 0.073}, {"t64x128_s", 6.003, 2.817}, {"t64x64_s", 5.960, 0.000}}};
  const Law &law = w8 ? W8 : W4;
  double quarter_rate = 0;
  for (const auto &c : law.cells)
    if (!strcmp(c.tile, "t128x128")) quarter_rate = c.tops_per_cu;
  const PfVariant *best = nullptr;
  double best_t = 0;
  for (const auto &c : law.cells) {
    const PfVariant *v = pf_variant(fmt("macaq_iu8_pf_%s_%s", w8 ? "w8" : "w4", c.tile));
    if (!v) continue;
    const double bm = v->block_m(), bn = v->block_n();
    const uint64_t tiles = (uint64_t)((n + v->block_n() - 1) / v->block_n()) * ((m + v->block_m() - 1) / v->block_m());
    const uint64_t grid = std::min<uint64_t>(tiles, (uint64_t)CU_COUNT * v->occ);
    const uint64_t per_wg = (tiles + grid - 1) / grid;
    double cu_tiles = (double)per_wg * std::min<uint64_t>(v->occ, (grid + CU_COUNT - 1) / CU_COUNT);
    // the 256 x 256 cell runs a thin last round (at most half the workgroups) as quarter tiles on the
    // 128 x 128 cell, each a quarter of the work at that cell's rate
    const uint64_t q = tiles / grid, rem = tiles - q * grid;
    if (!strcmp(c.tile, "tn4_lbk64") && q >= 1 && rem > 0 && 2 * rem <= grid)
      cu_tiles = (double)q + (double)((4 * rem + grid - 1) / grid) * 0.25 * (c.tops_per_cu / quarter_rate);
    const double tile_bytes = bm * k + bn * k * (w8 ? 1.0 : 0.5);
    const double t_mfma = cu_tiles * bm * bn * k * 2.0 / (c.tops_per_cu * 1e6);
    const double t_cu = cu_tiles * tile_bytes / (law.cu_gbps * 1e3);
    const double t_l2 = (double)tiles * tile_bytes / (law.l2_tbps * 1e6);
    // the two-a-CU 128 x 128 cell alone on a CU (no more workgroups than CUs) has four waves to hide
    // its latencies with and measured well behind the eight-wave 128 x 128 cell there
    const double lone = (!strcmp(c.tile, "t128x128_o2") && grid <= CU_COUNT) ? law.lone : 1.0;
    // cold weights: the row tiles that run side by side on one column block each fetch it from memory -- those of the
    // 128- and 256-row cells; the 64-row cells' neighbours share a column block's lines (fetch over operands 1.5-1.65 at
    // four row tiles by the counters, and the wide projections of the served graph at 65-128 rows: 16.5-18.8 us on
    // 64 x 128 where a doubled fetch would make it 27)
    const uint64_t gx = (n + v->block_n() - 1) / v->block_n(), gy = (m + v->block_m() - 1) / v->block_m();
    const double side = v->block_m() == 64 ? 1.0 : std::min<double>((double)std::min<uint64_t>(gy, std::max<uint64_t>(1, grid / gx)), law.side_cap);
    const double t_hbm = ((double)n * k * (w8 ? 1.0 : 0.5) * side + (double)m * k) / (law.hbm_tbps * 1e6);
    const double t = law.fixed_us + (double)per_wg * c.tile_us + lone * std::max(std::max(t_mfma, t_hbm), std::max(t_cu, t_l2));
    if (!best || t < best_t) best = v, best_t = t;
  }
  return best;
}

static int describe_rows(const char *op, const char *kernel, uint32_t rows, uint32_t width, const char *wname,
                         saber_iu8_desc *d) {
  if (rows == 0 || width == 0) return fail(SABER_IU8_E_RULE, fmt("%s: %u rows of %u has nothing to do", op, rows, width));
  if (width % 64 != 0 || width > 32768)
    return fail(SABER_IU8_E_RULE, fmt("%s: row width %u must be a multiple of 64 (whole A fragments), at most 32768", op, width));
  memset(d, 0, sizeof *d);
  copy_name(d->op, sizeof d->op, op);
  copy_name(d->plugin, sizeof d->plugin, "macaq_i8q");
  copy_name(d->kernel, sizeof d->kernel, kernel);
  // the wave-a-row forms take four rows a workgroup
  const bool w64 = strlen(kernel) > 4 && !strcmp(kernel + strlen(kernel) - 4, "_w64");
  if (w64 && (rows % 4 != 0 || width > 4096))
    return fail(SABER_IU8_E_RULE, fmt("%s: %s takes a multiple of 4 rows of at most 4096, got %u of %u", op, kernel, rows, width));
  const bool t1024 = strlen(kernel) > 6 && !strcmp(kernel + strlen(kernel) - 6, "_t1024");
  d->grid[0] = w64 ? rows / 4 : rows, d->grid[1] = 1, d->grid[2] = 1;
  d->block[0] = t1024 ? 1024 : 256, d->block[1] = 1, d->block[2] = 1;
  d->n_launches = 1;
  d->ks = 1;
  if (int rc = fill_slots(kernel, d)) return rc;
  set_i32(d, wname, width);
  return 0;
}

// The fused forms quantise rows whose int8 codes (rows rounded up to a power of two) fit the kernel's
// staging area: up to 4 rows in 20 KiB (`_tm1`), up to 16 rows in 80 KiB (`_tm1_a80`). Every workgroup
// repeats the rows' quantisation (about 0.5 us a row of 5,120 on this card), a producer launch costs
// about 3 us once. The kernel itself holds what `fused_form_holds` says, by name; what the law launches is
// `fused_holds` below.
static uint64_t staged_bytes(uint32_t m, uint32_t k) {
  uint32_t mr = 1;
  while (mr < m) mr *= 2;
  return (uint64_t)mr * k;
}
bool fused_small_holds(uint32_t m, uint32_t k) { return m >= 1 && m <= 4 && staged_bytes(m, k) <= 20 * 1024; }
bool fused_form_holds(bool a80, uint32_t m, uint32_t k) {
  return a80 ? m >= 1 && m <= 16 && staged_bytes(m, k) <= 80 * 1024 : fused_small_holds(m, k);
}
// the MLP chain: the first linear's rows (hidden wide) in the 20 KiB form, the second's (intermediate wide) in
// the 20 KiB form or, for up to 4 rows, the 80 KiB one
bool mlp_chain_form_holds(uint32_t m, uint32_t hidden, uint32_t inter) {
  return fused_small_holds(m, hidden) && (fused_small_holds(m, inter) || (m <= 4 && fused_form_holds(true, m, inter)));
}
// Where the one launch beats the three (fused gate+up linear, 16-wave activation producer, streamed down GEMV), graph
// replay on cold weights, hidden / intermediate in us chain / three: one row 5120/17408 32.9/34.2, 5120/13824 27.4/29.2,
// 4096/14336 25.5/27.0, 4096/12288 23.0/24.2, 8192/8192 25.9/25.8, 5120/5120 18.9/17.5; two rows 5120/17408 35.3/36.0,
// 5120/13824 29.9/30.9, 4096/14336 28.0/28.7, 4096/12288 25.7/25.4; three rows 36.5-36.8/36.6-37.4 and 31.9/31.6; four
// rows 38.2/37.3, 33.7/32.6, 28.6/26.2. (A meeting inside the launch costs more than the gap between two launches;
// what the chain saves is the activation's pass over memory and one launch.)
bool mlp_chain_pays(uint32_t m, uint32_t hidden, uint32_t inter) {
  if (inter > 20 * 1024) return false;  // not measured past the one-row form's 20 KiB of codes
  return mlp_chain_form_holds(m, hidden, inter) && ((m == 1 && inter >= MLP_CHAIN_PAYS_INTER_1) || (m == 2 && inter >= MLP_CHAIN_PAYS_INTER_2));
}
// The law: the 20 KiB form wherever it holds (1-4 rows: 5.7 / 5.3 / 16.7 us against 7.8 / 7.2 / 19.7 as two launches
// at one row of the 27B layer's K = 5120 shapes, 6.9 / 6.7 / 17.2 against 8.0 / 7.5 / 19.2 at four); the 80 KiB form at
// two rows of K >= 16384 (K = 17408: 13.85 against 13.98 us, and a launch fewer); elsewhere it loses to the 16-wave
// producer + the streamed or staged GEMV (two rows of K = 12288: 11.4 / 11.2; three rows of K = 17408: 14.8 / 14.1, of
// 8192: 10.0 / 9.5; four rows: 16.0 / 14.8 at K = 17408, 10.5 / 9.5 at 8192, 9.2 / 8.5 at 6144).
bool fused_holds(uint32_t m, uint32_t k) {
  return fused_small_holds(m, k) || (m == 2 && k >= FUSED_A80_MIN_K && fused_form_holds(true, m, k));
}

uint32_t fused_grid(uint32_t nblk) {
  if (nblk <= CU_COUNT) return nblk;
  const uint32_t per = std::min<uint32_t>(8, (nblk + CU_COUNT - 1) / CU_COUNT);
  return (nblk + per - 1) / per;
}

int resolve_fused(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *d) {
  if (wkind != SABER_IU8_W4 && wkind != SABER_IU8_W8) return fail(SABER_IU8_E_ARG, "unknown weight kind");
  const char *op = wkind == SABER_IU8_W8 ? "linear_i8a8_fused" : "linear_i4a8_fused";
  if (int rc = check_shape(op, m, n, k)) return rc;
  if (!fused_holds(m, k))
    return fail(SABER_IU8_E_RULE, fmt("%s: %u rows of %u are not a fused launch (up to 4 rows in 20 KiB of codes; 2 rows of K >= 16384 in 80 KiB)", op, m, k));
  // one long row: the form that makes the row's codes just in time inside the weight stream (`_r1`). Measured on
  // this card against the several-row form at one row (cold weights, graph replay, N = 5120): K = 8,192 6.47
  // against 6.91 us, 12,288 7.82 against 8.38, 17,408 9.88 against 10.7-11.4, 20,480 10.97 against 11.83; at
  // K = 5,120 it loses (5.64 against 5.17: there a thread of the several-row form converts one piece at most,
  // which is what this form's first chunk costs, and its two column groups convert every piece twice)
  const std::string name = m == 1 && k >= FUSED_R1_MIN_K && fused_small_holds(m, k)
                               ? fmt("macaq_iu8_decq_%s_r1", wkind == SABER_IU8_W8 ? "w8" : "w4")
                               : fmt("macaq_iu8_decq_%s_tm1%s", wkind == SABER_IU8_W8 ? "w8" : "w4", fused_small_holds(m, k) ? "" : "_a80");
  memset(d, 0, sizeof *d);
  copy_name(d->op, sizeof d->op, op);
  copy_name(d->plugin, sizeof d->plugin, "macaq_iu8");
  copy_name(d->kernel, sizeof d->kernel, name);
  // 16 waves: 8 k-waves x 2 weight tiles = 32 columns a block, one workgroup a CU. Past one block a
  // CU the workgroups walk the blocks in equal shares (1,088 blocks: 218 workgroups x 5, measured 15.8 us
  // against 16.2 on 256 workgroups with 4 or 5), at most 8 each (the kernel's scale table).
  d->grid[0] = fused_grid((n + 31) / 32), d->grid[1] = 1, d->grid[2] = 1;
  d->block[0] = 1024, d->block[1] = 1, d->block[2] = 1;
  d->n_launches = 1;
  d->ks = 1;
  if (int rc = fill_slots(name, d)) return rc;
  set_i32(d, "m", m);
  set_i32(d, "n", n);
  set_i32(d, "k", k);
  return 0;
}

// The decode MLP as one persistent launch (kernels/iu8_chain.h): both linears in the fused form's
// bounds, every workgroup resident at once (two a CU: the runtime checks what the card really
// holds), at most 8 column blocks of either linear a workgroup.
int resolve_mlp_chain(uint32_t m, uint32_t hidden, uint32_t inter, uint32_t spin, saber_iu8_desc *d) {
  const char *op = "mlp_chain_i4a8";
  if (inter > 0x3FFFFFFFu) return fail(SABER_IU8_E_RULE, fmt("%s: intermediate width %u", op, inter));
  if (int rc = check_shape(op, m, 2 * inter, hidden)) return rc;
  if (int rc = check_shape(op, m, hidden, inter)) return rc;
  if (!mlp_chain_form_holds(m, hidden, inter))
    return fail(SABER_IU8_E_RULE, fmt("%s: %u rows of %u / %u do not fit the fused form (at most 4 rows, 20 KiB of codes at the hidden "
                                      "width, 80 KiB at the intermediate)", op, m, hidden, inter));
  // the first linear walks inter / 16 paired tiles, the second hidden / 32 column blocks; one workgroup a CU
  const uint32_t nblk = std::max(inter / 16, (hidden + 31) / 32);
  if (nblk > 8 * CU_COUNT)
    return fail(SABER_IU8_E_RULE, fmt("%s: %u column blocks are more than the %u resident workgroups walk (8 each)", op, nblk, CU_COUNT));
  const uint32_t grid = std::max(fused_grid(inter / 16), fused_grid((hidden + 31) / 32));
  // the second linear's rows in 20 KiB of staged codes, else in 80 KiB (`_a80`: 2 to 4 rows of the 27B layer's 17,408)
  const char *name = fused_small_holds(m, inter) ? "macaq_iu8f_mlp_w4_tm1" : "macaq_iu8f_mlp_w4_tm1_a80";
  memset(d, 0, sizeof *d);
  copy_name(d->op, sizeof d->op, op);
  copy_name(d->plugin, sizeof d->plugin, "macaq_iu8f");
  copy_name(d->kernel, sizeof d->kernel, name);
  d->grid[0] = grid, d->grid[1] = 1, d->grid[2] = 1;
  d->block[0] = 1024, d->block[1] = 1, d->block[2] = 1;
  d->n_launches = 1;
  d->ks = 1;
  if (int rc = fill_slots(name, d)) return rc;
  set_i32(d, "m", m);
  set_i32(d, "k", hidden);
  set_i32(d, "n", inter);
  set_i32(d, "spin", spin ? spin : MLP_CHAIN_SPIN);
  add_ws(d, "p", SABER_IU8_WS_SCRATCH, (uint64_t)m * inter * 2, 0);
  add_ws(d, "state", SABER_IU8_WS_PERSISTENT, MLP_CHAIN_STATE_BYTES, 1);
  return 0;
}

// The gate+up linear of a decode MLP with SiLU(gate) * up in its epilogue (`macaq_iu8f_gateup_act_w4_s80`): the rows'
// 16-row tile staged once a workgroup (what `_s80` holds), a column block = one 16-column tile of p.
bool gate_up_act_holds(uint32_t m, uint32_t hidden, uint32_t inter) {
  return m >= 1 && m <= 16 && hidden % 128 == 0 && inter % 16 == 0 && inter > 0 && staged80_holds(m, hidden) && inter / 16 <= 8 * CU_COUNT;
}
int resolve_gate_up_act(uint32_t m, uint32_t hidden, uint32_t inter, saber_iu8_desc *d) {
  const char *op = "linear_i4a8_gate_up_act";
  if (inter > 0x3FFFFFFFu) return fail(SABER_IU8_E_RULE, fmt("%s: intermediate width %u", op, inter));
  if (int rc = check_shape(op, m, 2 * inter, hidden)) return rc;
  if (!gate_up_act_holds(m, hidden, inter))
    return fail(SABER_IU8_E_RULE, fmt("%s: %u rows of %u / %u: at most 16 rows whose codes (rows rounded up to a power of two) fit 80 KiB, "
                                      "at most %u tiles of 16 columns", op, m, hidden, inter, 8 * CU_COUNT));
  const char *name = "macaq_iu8f_gateup_act_w4_s80";
  memset(d, 0, sizeof *d);
  copy_name(d->op, sizeof d->op, op);
  copy_name(d->plugin, sizeof d->plugin, "macaq_iu8f");
  copy_name(d->kernel, sizeof d->kernel, name);
  d->grid[0] = fused_grid(inter / 16), d->grid[1] = 1, d->grid[2] = 1;
  d->block[0] = 1024, d->block[1] = 1, d->block[2] = 1;
  d->n_launches = 1;
  d->ks = 1;
  if (int rc = fill_slots(name, d)) return rc;
  set_i32(d, "m", m);
  set_i32(d, "n", inter);
  set_i32(d, "k", hidden);
  return 0;
}

// The row kernels' register forms: the narrowest that holds the row (4,096 elements a group slot).
// Many narrow rows go a wave a row (`base`_w64), the rest a workgroup a row (`base`_t256...).
// Rows wider than 4,096 whose count leaves the card part idle go 16 waves a row (`base`_t1024): measured on this
// card, graph replay, 256-thread form / 1024-thread form in us -- the quantiser at 1 / 16 / 256 rows of 5,120:
// 2.57/2.34, 2.98/2.74, 3.41/3.20; of 17,408: 3.90/2.91, 5.09/3.92, 6.72/5.49; at 512 rows 3.98/4.52 and 7.92/7.09, at
// 1,024 4.84/6.32 and 13.3/14.3. The activation (exp and an IEEE divide an element) at 1 / 16 / 512 rows of 5,120:
// 6.36/4.64, 6.75/5.02, 8.22/7.13; of 17,408: 13.6/7.50, 14.3/8.06, 18.8/14.9, and 47.0/42.4 at 2,048 rows (5,120
// there: 17.5/22.1). Rows of 4,096: the two forms are within 3 % (a thread of either owns one group).
static std::string row_form(const char *base, uint32_t rows, uint32_t width, bool silu = false) {
  if (width <= 2048 && rows % 4 == 0 && rows >= 64) return std::string(base) + "_w64";  // up to two groups a lane
  if (width > T1024_WIDTH_OVER &&
      (silu ? rows <= T1024_SILU_ROWS || width >= T1024_WIDE
            : rows <= (width >= T1024_WIDE ? T1024_QUANT_ROWS_WIDE : T1024_QUANT_ROWS)))
    return std::string(base) + "_t1024";
  const uint32_t slots = (width + 4095) / 4096;
  return std::string(base) + "_t256" + (slots <= 1 ? "_g1" : slots <= 2 ? "_g2" : slots <= 5 ? "_g5" : "");
}

int resolve_quant(uint32_t m, uint32_t k, saber_iu8_desc *out) {
  return describe_rows("quant_i8", row_form("macaq_i8_quant", m, k).c_str(), m, k, "k", out);
}

int resolve_rowscale(uint32_t m, uint32_t k, saber_iu8_desc *out) {
  const uint32_t slots = (k + 4095) / 4096;
  const std::string name = std::string("macaq_i8_rowscale_t256") + (slots <= 1 ? "_g1" : slots <= 2 ? "_g2" : "");
  return describe_rows("rowscale_i8", name.c_str(), m, k, "k", out);
}

// The fused-quant tile GEMM of a shape: the 128 x 128 cell while few tiles would leave CUs idle on the
// larger one, else the 256 x 160 cell (the widest whose registers hold the bf16 pieces in flight).
int resolve_prefill_fused(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out) {
  if (wkind != SABER_IU8_W4 && wkind != SABER_IU8_W8) return fail(SABER_IU8_E_ARG, "unknown weight kind");
  const char *tag = wkind == SABER_IU8_W8 ? "w8" : "w4";
  const uint64_t big = (uint64_t)((m + 255) / 256) * ((n + 159) / 160);
  return describe(fmt("macaq_iu8_pfq_%s_%s", tag, big >= CU_COUNT ? "t256x160" : "t128x128"), m, n, k, 1, out);
}

int resolve_quant_rowmajor(uint32_t m, uint32_t k, saber_iu8_desc *out) {
  const uint32_t slots = (k + 4095) / 4096;
  const std::string name = std::string("macaq_i8_quant_rm_t256") + (slots <= 1 ? "_g1" : slots <= 2 ? "_g2" : "");
  return describe_rows("quant_i8_rowmajor", name.c_str(), m, k, "k", out);
}

int resolve_quant_rows(uint32_t rows, uint32_t k, saber_iu8_desc *out) {
  const uint32_t slots = (k + 4095) / 4096;
  const std::string name = std::string("macaq_i8_quant_rows_t256") + (slots <= 1 ? "_g1" : slots <= 2 ? "_g2" : "");
  return describe_rows("quant_rows_i8", name.c_str(), rows, k, "k", out);
}

int resolve_silu_mul_quant(uint32_t rows, uint32_t n, saber_iu8_desc *out) {
  if (int rc = describe_rows("silu_mul_quant_i8", row_form("macaq_i8_silu_mul_quant", rows, n, true).c_str(), rows, n, "n", out)) return rc;
  // the dense form has no row map; the routed form binds both (set_buffer)
  set_null(out, "row_tok");
  set_null(out, "meta");
  return 0;
}

}  // namespace iu8
