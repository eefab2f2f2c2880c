// Code-object reader: clang offload bundle -> amdgcn ELF -> NT_AMDGPU_METADATA (msgpack) ->
// per-kernel facts. The counterpart of crates/saber-kernels/src/codeobj.rs and msgpack.rs of the
// reference: what the manifest is generated from and what the loader re-derives at load time.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace iu8 {

struct CoArg {
  uint32_t offset = 0, size = 0;
  std::string value_kind, name;
};

struct CoKernel {
  std::string name, symbol;
  uint32_t kernarg_segment_size = 0, kernarg_segment_align = 0;
  uint32_t group_segment_fixed_size = 0, private_segment_fixed_size = 0;
  uint32_t vgpr_count = 0, agpr_count = 0, sgpr_count = 0;
  uint32_t wavefront_size = 0, max_flat_workgroup_size = 0;
  std::vector<CoArg> args;  // explicit arguments only (hidden_* dropped)
};

struct CodeObject {
  std::string target;  // e.g. amdgcn-amd-amdhsa--gfx950
  std::vector<CoKernel> kernels;
  // the amdgcn ELF inside `bytes` (the whole input when it is a bare ELF)
  size_t elf_offset = 0, elf_size = 0;
  const CoKernel *kernel(const std::string &name) const;
};

// Parses a bundle or bare ELF. On failure returns false and sets *why.
bool parse_code_object(const std::vector<uint8_t> &bytes, CodeObject &out, std::string *why);

}  // namespace iu8
