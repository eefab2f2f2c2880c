#include "manifest.h"

#include <cstdlib>
#include <sstream>

#include "abi.h"
#include "util.h"

namespace iu8 {

const KernelDecl *Manifest::find(const std::string &name) const {
  for (auto &k : kernel)
    if (k.name == name) return &k;
  return nullptr;
}

Manifest manifest_from_code_object(const CodeObject &co, const std::string &plugin, const std::string &arch,
                                   const std::string &source, const std::string &source_sha256,
                                   const std::string &flags, const std::string &build_hash,
                                   const std::string &hsaco_name, const std::string &hsaco_sha256) {
  Manifest m;
  m.plugin = plugin, m.arch = arch, m.source = source, m.source_sha256 = source_sha256, m.flags = flags;
  m.build_hash = build_hash, m.hsaco = hsaco_name, m.hsaco_sha256 = hsaco_sha256;
  for (const CoKernel &k : co.kernels) {
    KernelDecl d;
    d.name = k.name, d.symbol = k.symbol;
    d.kernarg_segment_size = k.kernarg_segment_size, d.kernarg_segment_align = k.kernarg_segment_align;
    d.group_segment_fixed_size = k.group_segment_fixed_size, d.private_segment_fixed_size = k.private_segment_fixed_size;
    d.vgpr_count = k.vgpr_count, d.sgpr_count = k.sgpr_count, d.wavefront_size = k.wavefront_size;
    d.max_flat_workgroup_size = k.max_flat_workgroup_size;
    for (const CoArg &a : k.args) d.arg.push_back({a.offset, a.size, a.value_kind, a.name});
    m.kernel.push_back(std::move(d));
  }
  return m;
}

static std::string q(const std::string &s) {
  std::string o = "\"";
  for (char c : s) {
    if (c == '"' || c == '\\') o += '\\';
    o += c;
  }
  return o + "\"";
}

std::string manifest_to_toml(const Manifest &m) {
  std::ostringstream o;
  o << "schema_version = " << m.schema_version << "\n";
  o << "plugin = " << q(m.plugin) << "\narch = " << q(m.arch) << "\nsource = " << q(m.source) << "\n";
  o << "source_sha256 = " << q(m.source_sha256) << "\nflags = " << q(m.flags) << "\nbuild_hash = " << q(m.build_hash) << "\n";
  o << "hsaco = " << q(m.hsaco) << "\nhsaco_sha256 = " << q(m.hsaco_sha256) << "\n";
  for (const KernelDecl &k : m.kernel) {
    o << "\n[[kernel]]\nname = " << q(k.name) << "\nsymbol = " << q(k.symbol) << "\n";
    o << "kernarg_segment_size = " << k.kernarg_segment_size << "\nkernarg_segment_align = " << k.kernarg_segment_align << "\n";
    o << "group_segment_fixed_size = " << k.group_segment_fixed_size << "\nprivate_segment_fixed_size = "
      << k.private_segment_fixed_size << "\n";
    o << "vgpr_count = " << k.vgpr_count << "\nsgpr_count = " << k.sgpr_count << "\nwavefront_size = " << k.wavefront_size
      << "\nmax_flat_workgroup_size = " << k.max_flat_workgroup_size << "\n";
    for (const ArgDecl &a : k.arg) {
      o << "\n[[kernel.arg]]\noffset = " << a.offset << "\nsize = " << a.size << "\nvalue_kind = " << q(a.value_kind) << "\n";
      if (!a.name.empty()) o << "name = " << q(a.name) << "\n";
    }
  }
  return o.str();
}

// The TOML subset the manifest uses: `key = "string" | integer`, `[[kernel]]`, `[[kernel.arg]]`,
// comments and blank lines.
bool manifest_parse_toml(const std::string &text, Manifest &out, std::string *why) {
  out = Manifest();
  out.schema_version = 0;
  enum { Top, Kernel, Arg } where = Top;
  std::istringstream in(text);
  std::string line;
  int ln = 0;
  auto bad = [&](const std::string &m) {
    if (why) *why = fmt("manifest line %d: %s", ln, m.c_str());
    return false;
  };
  while (std::getline(in, line)) {
    ++ln;
    size_t a = line.find_first_not_of(" \t\r");
    if (a == std::string::npos || line[a] == '#') continue;
    size_t b = line.find_last_not_of(" \t\r");
    line = line.substr(a, b - a + 1);
    if (line == "[[kernel]]") {
      out.kernel.emplace_back();
      where = Kernel;
      continue;
    }
    if (line == "[[kernel.arg]]") {
      if (out.kernel.empty()) return bad("[[kernel.arg]] before any [[kernel]]");
      out.kernel.back().arg.emplace_back();
      where = Arg;
      continue;
    }
    if (line[0] == '[') return bad("unknown table " + line);
    const size_t eq = line.find('=');
    if (eq == std::string::npos) return bad("expected key = value");
    std::string key = line.substr(0, eq), val = line.substr(eq + 1);
    key.erase(key.find_last_not_of(" \t") + 1);
    val.erase(0, val.find_first_not_of(" \t"));
    bool is_str = false;
    std::string sval;
    uint32_t ival = 0;
    if (!val.empty() && val[0] == '"') {
      is_str = true;
      for (size_t i = 1; i < val.size(); ++i) {
        if (val[i] == '\\' && i + 1 < val.size()) sval += val[++i];
        else if (val[i] == '"') break;
        else sval += val[i];
      }
    } else {
      char *endp = nullptr;
      ival = (uint32_t)strtoul(val.c_str(), &endp, 10);
      if (endp == val.c_str()) return bad("value of `" + key + "` is neither a string nor an integer");
    }
    auto want_s = [&](std::string &dst) { if (!is_str) return false; dst = sval; return true; };
    auto want_i = [&](uint32_t &dst) { if (is_str) return false; dst = ival; return true; };
    bool ok = true;
    if (where == Top) {
      if (key == "schema_version") ok = want_i(out.schema_version);
      else if (key == "plugin") ok = want_s(out.plugin);
      else if (key == "arch") ok = want_s(out.arch);
      else if (key == "source") ok = want_s(out.source);
      else if (key == "source_sha256") ok = want_s(out.source_sha256);
      else if (key == "flags") ok = want_s(out.flags);
      else if (key == "build_hash") ok = want_s(out.build_hash);
      else if (key == "hsaco") ok = want_s(out.hsaco);
      else if (key == "hsaco_sha256") ok = want_s(out.hsaco_sha256);
      else return bad("unknown key `" + key + "`");
    } else if (where == Kernel) {
      KernelDecl &k = out.kernel.back();
      if (key == "name") ok = want_s(k.name);
      else if (key == "symbol") ok = want_s(k.symbol);
      else if (key == "kernarg_segment_size") ok = want_i(k.kernarg_segment_size);
      else if (key == "kernarg_segment_align") ok = want_i(k.kernarg_segment_align);
      else if (key == "group_segment_fixed_size") ok = want_i(k.group_segment_fixed_size);
      else if (key == "private_segment_fixed_size") ok = want_i(k.private_segment_fixed_size);
      else if (key == "vgpr_count") ok = want_i(k.vgpr_count);
      else if (key == "sgpr_count") ok = want_i(k.sgpr_count);
      else if (key == "wavefront_size") ok = want_i(k.wavefront_size);
      else if (key == "max_flat_workgroup_size") ok = want_i(k.max_flat_workgroup_size);
      else return bad("unknown kernel key `" + key + "`");
    } else {
      ArgDecl &g = out.kernel.back().arg.back();
      if (key == "offset") ok = want_i(g.offset);
      else if (key == "size") ok = want_i(g.size);
      else if (key == "value_kind") ok = want_s(g.value_kind);
      else if (key == "name") ok = want_s(g.name);
      else return bad("unknown arg key `" + key + "`");
    }
    if (!ok) return bad("wrong value type for `" + key + "`");
  }
  if (out.schema_version != SCHEMA_VERSION) {
    if (why) *why = fmt("manifest schema %u, this build speaks %u", out.schema_version, SCHEMA_VERSION);
    return false;
  }
  return true;
}

bool check_kernarg_layout(const Manifest &m, std::string *why) {
  for (const KernelDecl &k : m.kernel) {
    const Signature *sig = signature_for(k.name);
    if (!sig) continue;  // a kernel the host never launches by signature
    std::vector<std::pair<uint32_t, uint32_t>> packed;
    pack(*sig, packed);
    if (k.arg.size() != sig->size()) {
      if (why) *why = fmt("%s: %zu arguments declared, the signature has %zu", k.name.c_str(), k.arg.size(), sig->size());
      return false;
    }
    for (size_t i = 0; i < sig->size(); ++i) {
      const ArgDecl &a = k.arg[i];
      if (a.offset != packed[i].first || a.size != packed[i].second || a.value_kind != (*sig)[i].value_kind() ||
          (!a.name.empty() && a.name != (*sig)[i].name)) {
        if (why)
          *why = fmt("%s: argument %zu `%s` at %u size %u kind %s, the signature has `%s` at %u size %u kind %s",
                     k.name.c_str(), i, a.name.c_str(), a.offset, a.size, a.value_kind.c_str(), (*sig)[i].name,
                     packed[i].first, packed[i].second, (*sig)[i].value_kind());
        return false;
      }
    }
  }
  return true;
}

bool check_wave_size(const Manifest &m, std::string *why) {
  uint32_t seen = 0;
  for (const KernelDecl &k : m.kernel) {
    if (k.wavefront_size != 32 && k.wavefront_size != 64) {
      if (why) *why = fmt("%s: wavefront size %u", k.name.c_str(), k.wavefront_size);
      return false;
    }
    if (seen && seen != k.wavefront_size) {
      if (why) *why = fmt("%s: wavefront size %u in a plugin of wave%u kernels", k.name.c_str(), k.wavefront_size, seen);
      return false;
    }
    seen = k.wavefront_size;
  }
  return true;
}

bool validate_against_hsaco(const Manifest &m, const std::vector<uint8_t> &hsaco, const CodeObject &co,
                            const std::string &arch, std::string *why) {
  auto bad = [&](const std::string &s) {
    if (why) *why = m.plugin + ": " + s;
    return false;
  };
  if (sha256_hex(hsaco.data(), hsaco.size()) != m.hsaco_sha256) return bad("code object sha256 differs from the manifest's");
  if (!arch.empty() && m.arch != arch) return bad("manifest arch " + m.arch + ", loading for " + arch);
  if (co.target.find(m.arch) == std::string::npos) return bad("code object target " + co.target + " is not " + m.arch);
  for (const KernelDecl &k : m.kernel) {
    const CoKernel *c = co.kernel(k.name);
    if (!c) return bad(k.name + ": not in the code object");
#define IU8_SAME(field)                                                                                         \
  if (k.field != c->field) return bad(fmt("%s: %s %u declared, %u in the code object", k.name.c_str(), #field, k.field, c->field))
    IU8_SAME(kernarg_segment_size);
    IU8_SAME(kernarg_segment_align);
    IU8_SAME(group_segment_fixed_size);
    IU8_SAME(private_segment_fixed_size);
    IU8_SAME(vgpr_count);
    IU8_SAME(sgpr_count);
    IU8_SAME(wavefront_size);
    IU8_SAME(max_flat_workgroup_size);
#undef IU8_SAME
    if (k.symbol != c->symbol) return bad(k.name + ": symbol " + k.symbol + " declared, " + c->symbol + " in the code object");
    if (k.arg.size() != c->args.size())
      return bad(fmt("%s: %zu arguments declared, %zu in the code object", k.name.c_str(), k.arg.size(), c->args.size()));
    for (size_t i = 0; i < k.arg.size(); ++i)
      if (k.arg[i].offset != c->args[i].offset || k.arg[i].size != c->args[i].size ||
          k.arg[i].value_kind != c->args[i].value_kind)
        return bad(fmt("%s: argument %zu is %u/%u/%s declared, %u/%u/%s in the code object", k.name.c_str(), i,
                       k.arg[i].offset, k.arg[i].size, k.arg[i].value_kind.c_str(), c->args[i].offset, c->args[i].size,
                       c->args[i].value_kind.c_str()));
  }
  return true;
}

}  // namespace iu8
