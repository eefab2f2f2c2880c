// The per-plugin manifest (schema 1): what a code object contains, declared, hashed and
// checkable. Counterpart of crates/saber-kernels/src/manifest.rs (schema :17,63-79, generation
// :136-226, validation :228-324) and of the loader's checks in crates/saber-exec/src/loader.rs
// (:192-290).
#pragma once
#include <string>
#include <vector>

#include "codeobj.h"

namespace iu8 {

struct ArgDecl {
  uint32_t offset = 0, size = 0;
  std::string value_kind, name;
};
struct KernelDecl {
  std::string name, symbol;
  uint32_t kernarg_segment_size = 0, kernarg_segment_align = 0, group_segment_fixed_size = 0,
           private_segment_fixed_size = 0, vgpr_count = 0, sgpr_count = 0, wavefront_size = 0,
           max_flat_workgroup_size = 0;
  std::vector<ArgDecl> arg;
};
struct Manifest {
  uint32_t schema_version = 1;
  std::string plugin, arch, source, source_sha256, flags, build_hash, hsaco, hsaco_sha256;
  std::vector<KernelDecl> kernel;
  const KernelDecl *find(const std::string &name) const;
};

constexpr uint32_t SCHEMA_VERSION = 1;

Manifest manifest_from_code_object(const CodeObject &co, const std::string &plugin, const std::string &arch,
                                   const std::string &source, const std::string &source_sha256,
                                   const std::string &flags, const std::string &build_hash,
                                   const std::string &hsaco_name, const std::string &hsaco_sha256);
std::string manifest_to_toml(const Manifest &m);
bool manifest_parse_toml(const std::string &text, Manifest &out, std::string *why);

// The three loader validations. Each returns true when it passes; otherwise *why says what.
bool check_kernarg_layout(const Manifest &m, std::string *why);  // manifest args vs the declared signatures
bool check_wave_size(const Manifest &m, std::string *why);       // 32 or 64, one size a plugin
bool validate_against_hsaco(const Manifest &m, const std::vector<uint8_t> &hsaco, const CodeObject &co,
                            const std::string &arch, std::string *why);

}  // namespace iu8
