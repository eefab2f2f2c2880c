#include "codeobj.h"

#include <cstring>
#include <map>

namespace iu8 {

// ---------------------------------------------------------------- msgpack (the subset LLVM emits)
namespace {
struct MpVal {
  enum Kind { Nil, Bool, Int, Str, Arr, Map, Other } kind = Nil;
  int64_t i = 0;
  std::string s;
  std::vector<MpVal> arr;
  std::vector<std::pair<MpVal, MpVal>> map;
  const MpVal *get(const char *key) const {
    for (auto &kv : map)
      if (kv.first.kind == Str && kv.first.s == key) return &kv.second;
    return nullptr;
  }
};

struct MpReader {
  const uint8_t *p, *end;
  bool ok = true;
  int depth = 0;  // containers open: a note nests four or five deep; a crafted one must not eat the stack
  uint64_t be(int n) {
    if (end - p < n) {
      ok = false;
      return 0;
    }
    uint64_t v = 0;
    for (int i = 0; i < n; ++i) v = v << 8 | *p++;
    return v;
  }
  void str(MpVal &v, size_t n) {
    if ((size_t)(end - p) < n) {
      ok = false;
      return;
    }
    v.kind = MpVal::Str;
    v.s.assign((const char *)p, n);
    p += n;
  }
  void arr(MpVal &v, size_t n) {
    v.kind = MpVal::Arr;
    for (size_t i = 0; i < n && ok; ++i) v.arr.push_back(value());
  }
  void map(MpVal &v, size_t n) {
    v.kind = MpVal::Map;
    for (size_t i = 0; i < n && ok; ++i) {
      MpVal k = value();
      MpVal x = value();
      v.map.emplace_back(std::move(k), std::move(x));
    }
  }
  MpVal value() {
    MpVal v;
    if (p >= end || depth > 32) {
      ok = false;
      return v;
    }
    struct Nest {
      int &d;
      explicit Nest(int &x) : d(x) { ++d; }
      ~Nest() { --d; }
    } nest(depth);
    const uint8_t t = *p++;
    if (t <= 0x7f) { v.kind = MpVal::Int; v.i = t; }
    else if (t >= 0xe0) { v.kind = MpVal::Int; v.i = (int8_t)t; }
    else if ((t & 0xe0) == 0xa0) str(v, t & 0x1f);
    else if ((t & 0xf0) == 0x90) arr(v, t & 0x0f);
    else if ((t & 0xf0) == 0x80) map(v, t & 0x0f);
    else switch (t) {
      case 0xc0: v.kind = MpVal::Nil; break;
      case 0xc2: v.kind = MpVal::Bool; v.i = 0; break;
      case 0xc3: v.kind = MpVal::Bool; v.i = 1; break;
      case 0xcc: v.kind = MpVal::Int; v.i = (int64_t)be(1); break;
      case 0xcd: v.kind = MpVal::Int; v.i = (int64_t)be(2); break;
      case 0xce: v.kind = MpVal::Int; v.i = (int64_t)be(4); break;
      case 0xcf: v.kind = MpVal::Int; v.i = (int64_t)be(8); break;
      case 0xd0: v.kind = MpVal::Int; v.i = (int8_t)be(1); break;
      case 0xd1: v.kind = MpVal::Int; v.i = (int16_t)be(2); break;
      case 0xd2: v.kind = MpVal::Int; v.i = (int32_t)be(4); break;
      case 0xd3: v.kind = MpVal::Int; v.i = (int64_t)be(8); break;
      case 0xd9: str(v, be(1)); break;
      case 0xda: str(v, be(2)); break;
      case 0xdb: str(v, be(4)); break;
      case 0xdc: arr(v, be(2)); break;
      case 0xdd: arr(v, be(4)); break;
      case 0xde: map(v, be(2)); break;
      case 0xdf: map(v, be(4)); break;
      case 0xc4: { const size_t n = be(1); v.kind = MpVal::Other; if ((size_t)(end - p) < n) ok = false; else p += n; break; }
      case 0xc5: { const size_t n = be(2); v.kind = MpVal::Other; if ((size_t)(end - p) < n) ok = false; else p += n; break; }
      case 0xca: be(4); v.kind = MpVal::Other; break;
      case 0xcb: be(8); v.kind = MpVal::Other; break;
      default: ok = false;
    }
    return v;
  }
};

uint32_t u32_of(const MpVal &m, const char *key) {
  const MpVal *v = m.get(key);
  return v && v->kind == MpVal::Int ? (uint32_t)v->i : 0;
}
std::string str_of(const MpVal &m, const char *key) {
  const MpVal *v = m.get(key);
  return v && v->kind == MpVal::Str ? v->s : std::string();
}

template <typename T>
bool rd(const std::vector<uint8_t> &b, size_t off, T &out) {
  if (off + sizeof(T) > b.size()) return false;
  memcpy(&out, b.data() + off, sizeof(T));
  return true;
}
}  // namespace

const CoKernel *CodeObject::kernel(const std::string &name) const {
  for (auto &k : kernels)
    if (k.name == name) return &k;
  return nullptr;
}

static bool parse_elf(const std::vector<uint8_t> &b, size_t base, size_t size, CodeObject &out, std::string *why) {
  auto bad = [&](const char *m) {
    if (why) *why = m;
    return false;
  };
  if (size < 64 || memcmp(b.data() + base, "\177ELF", 4) != 0) return bad("not an ELF");
  if (b[base + 4] != 2 || b[base + 5] != 1) return bad("not a little-endian ELF64");
  uint16_t machine = 0, shentsize = 0, shnum = 0;
  uint64_t shoff = 0;
  rd(b, base + 18, machine);
  rd(b, base + 40, shoff);
  rd(b, base + 58, shentsize);
  rd(b, base + 60, shnum);
  if (machine != 224) return bad("ELF machine is not EM_AMDGPU");
  uint64_t sh_end = 0;
  if (shoff == 0 || shentsize < 64 || __builtin_add_overflow(shoff, (uint64_t)shentsize * shnum, &sh_end) || sh_end > size)
    return bad("bad section table");
  for (uint16_t i = 0; i < shnum; ++i) {
    const size_t sh = base + shoff + (size_t)i * shentsize;
    uint32_t type = 0;
    uint64_t off = 0, sz = 0;
    rd(b, sh + 4, type);
    rd(b, sh + 24, off);
    rd(b, sh + 32, sz);
    uint64_t sec_end = 0;
    if (type != 7 /* SHT_NOTE */ || __builtin_add_overflow(off, sz, &sec_end) || sec_end > size) continue;
    size_t p = base + off;
    const size_t end = p + sz;
    while (p + 12 <= end) {
      uint32_t namesz = 0, descsz = 0, ntype = 0;
      rd(b, p, namesz);
      rd(b, p + 4, descsz);
      rd(b, p + 8, ntype);
      const size_t name_at = p + 12, desc_at = name_at + ((namesz + 3) & ~3u);
      if (desc_at + descsz > end) break;
      if (ntype == 32 /* NT_AMDGPU_METADATA */ && namesz >= 6 && memcmp(b.data() + name_at, "AMDGPU", 6) == 0) {
        MpReader r{b.data() + desc_at, b.data() + desc_at + descsz};
        const MpVal root = r.value();
        if (!r.ok || root.kind != MpVal::Map) return bad("metadata note is not a msgpack map");
        out.target = str_of(root, "amdhsa.target");
        const MpVal *ks = root.get("amdhsa.kernels");
        if (!ks || ks->kind != MpVal::Arr) return bad("metadata has no amdhsa.kernels");
        for (const MpVal &k : ks->arr) {
          CoKernel ck;
          ck.name = str_of(k, ".name");
          ck.symbol = str_of(k, ".symbol");
          ck.kernarg_segment_size = u32_of(k, ".kernarg_segment_size");
          ck.kernarg_segment_align = u32_of(k, ".kernarg_segment_align");
          ck.group_segment_fixed_size = u32_of(k, ".group_segment_fixed_size");
          ck.private_segment_fixed_size = u32_of(k, ".private_segment_fixed_size");
          ck.vgpr_count = u32_of(k, ".vgpr_count");
          ck.agpr_count = u32_of(k, ".agpr_count");
          ck.sgpr_count = u32_of(k, ".sgpr_count");
          ck.wavefront_size = u32_of(k, ".wavefront_size");
          ck.max_flat_workgroup_size = u32_of(k, ".max_flat_workgroup_size");
          if (const MpVal *as = k.get(".args"))
            for (const MpVal &a : as->arr) {
              CoArg ca;
              ca.offset = u32_of(a, ".offset");
              ca.size = u32_of(a, ".size");
              ca.value_kind = str_of(a, ".value_kind");
              ca.name = str_of(a, ".name");
              if (ca.value_kind.rfind("hidden_", 0) == 0) continue;
              ck.args.push_back(ca);
            }
          out.kernels.push_back(std::move(ck));
        }
        out.elf_offset = base;
        out.elf_size = size;
        return true;
      }
      p = desc_at + ((descsz + 3) & ~3u);
    }
  }
  return bad("no NT_AMDGPU_METADATA note (code object v3+ required)");
}

bool parse_code_object(const std::vector<uint8_t> &bytes, CodeObject &out, std::string *why) {
  static const char MAGIC[] = "__CLANG_OFFLOAD_BUNDLE__";
  out = CodeObject();
  if (bytes.size() >= 32 && memcmp(bytes.data(), MAGIC, 24) == 0) {
    uint64_t n = 0;
    rd(bytes, 24, n);
    size_t p = 32;
    int found = 0;
    size_t eoff = 0, esize = 0;
    for (uint64_t i = 0; i < n; ++i) {
      uint64_t off = 0, size = 0, ts = 0;
      if (!rd(bytes, p, off) || !rd(bytes, p + 8, size) || !rd(bytes, p + 16, ts) || p + 24 + ts > bytes.size()) {
        if (why) *why = "truncated offload bundle header";
        return false;
      }
      const std::string triple((const char *)bytes.data() + p + 24, ts);
      p += 24 + ts;
      if (triple.find("amdgcn") != std::string::npos && size > 0) {
        ++found;
        eoff = off;
        esize = size;
      }
    }
    // exactly one amdgcn entry a bundle (crates/saber-kernels/src/codeobj.rs:86-114)
    if (found != 1 || eoff + esize > bytes.size()) {
      if (why) *why = "offload bundle must hold exactly one amdgcn entry";
      return false;
    }
    return parse_elf(bytes, eoff, esize, out, why);
  }
  return parse_elf(bytes, 0, bytes.size(), out, why);
}

}  // namespace iu8
