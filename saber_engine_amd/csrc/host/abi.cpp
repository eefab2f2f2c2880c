#include "abi.h"

namespace iu8 {

using K = ArgKind;

static const Signature SIG_DEC = {{"a", K::Buffer},  {"w", K::Buffer},
                                  {"as", K::Buffer}, {"ws", K::Buffer},
                                  {"decode_partial", K::Buffer}, {"decode_counter", K::Buffer},
                                  {"c", K::Buffer},  {"m", K::I32},
                                  {"n", K::I32},     {"k", K::I32}};
static const Signature SIG_DECQ = {{"x", K::Buffer},     {"w", K::Buffer}, {"ws", K::Buffer}, {"q", K::Buffer},
                                   {"scale", K::Buffer}, {"c", K::Buffer}, {"m", K::I32},     {"n", K::I32},
                                   {"k", K::I32}};
// the decode pair (crates/saber-kernels/src/abi.rs:3411-3432)
static const Signature SIG_PAIR = {{"a", K::Buffer},  {"as", K::Buffer}, {"w", K::Buffer},  {"ws", K::Buffer},
                                   {"decode_partial", K::Buffer},   {"decode_counter", K::Buffer},
                                   {"c", K::Buffer},  {"w_b", K::Buffer}, {"ws_b", K::Buffer},
                                   {"decode_partial_b", K::Buffer}, {"decode_counter_b", K::Buffer},
                                   {"c_b", K::Buffer}, {"m", K::I32},    {"k", K::I32},     {"n", K::I32},
                                   {"ks", K::I32},    {"nb", K::I32},    {"n_b", K::I32},   {"ks_b", K::I32},
                                   {"nb_b", K::I32}};
// the decode MLP chain (no counterpart list in the reference: its dense MLP is three launches)
static const Signature SIG_MLP = {{"x", K::Buffer},    {"w", K::Buffer},      {"ws", K::Buffer}, {"w_b", K::Buffer},
                                  {"ws_b", K::Buffer}, {"gu", K::Buffer},     {"p", K::Buffer},  {"state", K::Buffer},
                                  {"c", K::Buffer},    {"m", K::I32},         {"k", K::I32},     {"n", K::I32},
                                  {"spin", K::I32}};
// the gate+up linear with its activation in the epilogue (no counterpart list in the reference)
static const Signature SIG_GATEUP_ACT = {{"a", K::Buffer},  {"w", K::Buffer}, {"as", K::Buffer}, {"ws", K::Buffer}, {"gu", K::Buffer},
                                         {"p", K::Buffer},  {"m", K::I32},    {"n", K::I32},     {"k", K::I32}};
static const Signature SIG_PF = {{"a", K::Buffer}, {"w", K::Buffer}, {"as", K::Buffer}, {"ws", K::Buffer},
                                 {"c", K::Buffer}, {"m", K::I32},    {"n", K::I32},     {"k", K::I32}};
static const Signature SIG_PFQ = {{"x", K::Buffer}, {"w", K::Buffer}, {"as", K::Buffer}, {"ws", K::Buffer},
                                  {"c", K::Buffer}, {"m", K::I32},    {"n", K::I32},     {"k", K::I32}};
static const Signature SIG_ROWSCALE = {{"x", K::Buffer}, {"scale", K::Buffer}, {"k", K::I32}};
static const Signature SIG_QUANT = {{"x", K::Buffer}, {"q", K::Buffer}, {"scale", K::Buffer}, {"k", K::I32}};
static const Signature SIG_QUANT_ROWS = {{"x", K::Buffer}, {"q", K::Buffer},       {"scale", K::Buffer},
                                         {"k", K::I32},    {"row_tok", K::Buffer}, {"meta", K::Buffer}};
// the Hadamard-basis producers: the reference's lists, `had_t` last
// (prebuilt/gfx1201/mxfp4_hadi8.manifest.toml: 64 and 40 bytes)
static const Signature SIG_HAD_ARQ = {{"y", K::Buffer},     {"res", K::Buffer},     {"w", K::Buffer},
                                      {"q", K::Buffer},     {"scale", K::Buffer},   {"res_out", K::Buffer},
                                      {"k", K::I32},        {"eps", K::F32},        {"had_t", K::Buffer}};
static const Signature SIG_HAD_SMQ = {{"gu", K::Buffer}, {"q", K::Buffer}, {"scale", K::Buffer}, {"n", K::I32}, {"had_t", K::Buffer}};
static const Signature SIG_HAD_SMQ_LUT = {{"gu", K::Buffer}, {"q", K::Buffer}, {"scale", K::Buffer}, {"n", K::I32},
                                          {"had_t", K::Buffer}, {"lut", K::Buffer}};
static const Signature SIG_HAD_Q = {{"x", K::Buffer}, {"q", K::Buffer}, {"scale", K::Buffer}, {"k", K::I32}, {"had_t", K::Buffer}};
// crates/saber-kernels/src/abi.rs:652-662 and :2683-2694, `had_t` appended last
static const Signature SIG_HAD_GNQ = {{"x", K::Buffer}, {"z", K::Buffer},     {"zs", K::I64}, {"w", K::Buffer},
                                      {"q", K::Buffer}, {"scale", K::Buffer}, {"n", K::I32},  {"eps", K::F32},
                                      {"had_t", K::Buffer}};
static const Signature SIG_HAD_AGQ = {{"core", K::Buffer}, {"gate", K::Buffer}, {"q", K::Buffer}, {"scale", K::Buffer},
                                      {"n", K::I32},       {"hd", K::I32},      {"gs", K::I32},   {"had_t", K::Buffer}};
static const Signature SIG_HAD_AGQ_LUT = {{"core", K::Buffer}, {"gate", K::Buffer}, {"q", K::Buffer}, {"scale", K::Buffer},
                                          {"n", K::I32},       {"hd", K::I32},      {"gs", K::I32},   {"had_t", K::Buffer},
                                          {"lut", K::Buffer}};
static const Signature SIG_SILU = {{"gu", K::Buffer}, {"q", K::Buffer},       {"scale", K::Buffer},
                                   {"n", K::I32},     {"row_tok", K::Buffer}, {"meta", K::Buffer}};
static const Signature SIG_SILU_LUT = {{"gu", K::Buffer}, {"q", K::Buffer},       {"scale", K::Buffer}, {"n", K::I32},
                                       {"row_tok", K::Buffer}, {"meta", K::Buffer}, {"lut", K::Buffer}};
static const Signature SIG_TABLE = {{"out", K::Buffer}};
static const Signature SIG_MOE_ROUTE = {
    {"logits", K::Buffer},      {"t", K::I32},           {"e_lo", K::I32},        {"e_loc", K::I32},
    {"tile_blocks", K::I32},    {"with_shared", K::I32}, {"topk_ids", K::Buffer}, {"topk_w", K::Buffer},
    {"route_pos", K::Buffer},   {"row_tok", K::Buffer},  {"row_route", K::Buffer}, {"tile_expert", K::Buffer},
    {"tile_row0", K::Buffer},   {"tile_rows", K::Buffer}, {"expert_cnt", K::Buffer}, {"meta", K::Buffer},
    {"blk_cnt", K::Buffer},     {"rank", K::Buffer},     {"arrive", K::Buffer}};
static const Signature SIG_MOE_ROUTEQ = {
    {"logits", K::Buffer},      {"t", K::I32},           {"e_lo", K::I32},        {"e_loc", K::I32},
    {"tile_blocks", K::I32},    {"with_shared", K::I32}, {"topk_ids", K::Buffer}, {"topk_w", K::Buffer},
    {"route_pos", K::Buffer},   {"row_tok", K::Buffer},  {"row_route", K::Buffer}, {"tile_expert", K::Buffer},
    {"tile_row0", K::Buffer},   {"tile_rows", K::Buffer}, {"expert_cnt", K::Buffer}, {"meta", K::Buffer},
    {"blk_cnt", K::Buffer},     {"rank", K::Buffer},     {"arrive", K::Buffer},   {"x", K::Buffer},
    {"q", K::Buffer},           {"scale", K::Buffer},    {"k", K::I32}};
static const Signature SIG_MOE_GROUPED = {
    {"a", K::Buffer},       {"xptr", K::Buffer}, {"tile_expert", K::Buffer}, {"tile_row0", K::Buffer},
    {"tile_rows", K::Buffer}, {"row_tok", K::Buffer}, {"meta", K::Buffer},   {"as", K::Buffer},
    {"p", K::Buffer},       {"cnt", K::Buffer},  {"c", K::Buffer},           {"n", K::I32},
    {"k", K::I32},          {"pmax", K::I32}};
static const Signature SIG_MOE_COMBINE = {{"y", K::Buffer},    {"topk_w", K::Buffer}, {"route_pos", K::Buffer},
                                          {"sgate", K::Buffer}, {"meta", K::Buffer},  {"out", K::Buffer},
                                          {"h", K::I32}};

static const Signature SIG_PROBE_READ = {{"src", K::Buffer}, {"out", K::Buffer}, {"n", K::I32}};
static const Signature SIG_PROBE_COPY = {{"src", K::Buffer}, {"dst", K::Buffer}, {"n", K::I32}};

static bool starts(const std::string &s, const char *p) { return s.rfind(p, 0) == 0; }

const Signature *signature_for(const std::string &k) {
  if (starts(k, "macaq_iu8_dec_")) return &SIG_DEC;
  if (starts(k, "macaq_iu8_decq_")) return &SIG_DECQ;
  if (starts(k, "macaq_iu8_pfq_")) return &SIG_PFQ;
  if (starts(k, "macaq_i8_rowscale_")) return &SIG_ROWSCALE;
  if (starts(k, "macaq_iu8_pf_")) return k.size() > 3 && k.compare(k.size() - 3, 3, "_ks") == 0 ? &SIG_DEC : &SIG_PF;
  if (starts(k, "macaq_iu8f_pair_") || starts(k, "macaq_iu8f_pairb_")) return &SIG_PAIR;
  if (starts(k, "macaq_iu8f_mlp_")) return &SIG_MLP;
  if (starts(k, "macaq_iu8f_gateup_act_")) return &SIG_GATEUP_ACT;
  if (starts(k, "add_rms_quant_hadi8_")) return &SIG_HAD_ARQ;
  if (starts(k, "silu_mul_quant_hadi8_lut_")) return &SIG_HAD_SMQ_LUT;
  if (starts(k, "silu_mul_quant_hadi8_")) return &SIG_HAD_SMQ;
  if (starts(k, "quant_hadi8_")) return &SIG_HAD_Q;
  if (starts(k, "gdn_norm_quant_hadi8_")) return &SIG_HAD_GNQ;
  if (starts(k, "attn_gate_quant_hadi8_lut_")) return &SIG_HAD_AGQ_LUT;
  if (starts(k, "attn_gate_quant_hadi8_")) return &SIG_HAD_AGQ;
  if (k == "mxfp4_hadi8_silu_f32_table" || k == "attn_glue_hadi8_sigmoid_bf16_table") return &SIG_TABLE;
  if (k == "attn_gate_sigmoid_bf16_table") return &SIG_TABLE;
  if (starts(k, "macaq_i8_quant_rows_")) return &SIG_QUANT_ROWS;
  if (starts(k, "macaq_i8_quant_")) return &SIG_QUANT;
  if (starts(k, "macaq_i8_silu_mul_quant_lut_")) return &SIG_SILU_LUT;
  if (starts(k, "macaq_i8_silu_mul_quant_")) return &SIG_SILU;
  if (k == "macaq_silu_bf16_table") return &SIG_TABLE;
  if (k == "iu8_probe_read" || k == "iu8_probe_mfma32d") return &SIG_PROBE_READ;
  if (k == "iu8_probe_copy") return &SIG_PROBE_COPY;
  if (starts(k, "moe_iu8_route_")) return &SIG_MOE_ROUTE;
  if (starts(k, "moe_iu8_routeq_")) return &SIG_MOE_ROUTEQ;
  if (starts(k, "moe_iu8_grouped_")) return &SIG_MOE_GROUPED;
  if (starts(k, "moe_iu8_combine_")) return &SIG_MOE_COMBINE;
  return nullptr;
}

uint32_t pack(const Signature &sig, std::vector<std::pair<uint32_t, uint32_t>> &out) {
  out.clear();
  uint32_t off = 0;
  for (const SigArg &a : sig) {
    off = (off + a.align() - 1) / a.align() * a.align();
    out.emplace_back(off, a.size());
    off += a.size();
  }
  return off;
}

}  // namespace iu8
