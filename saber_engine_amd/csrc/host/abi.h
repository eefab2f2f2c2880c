// Kernel signatures and the kernarg packing law: the counterpart of
// crates/saber-kernels/src/abi.rs (SigArg, pack at :111-130, SIG_MACAQ_IU8_* at :3349-3372,
// the MoE signatures at :325-385, signature_for at :3495).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace iu8 {

enum class ArgKind { Buffer, I32, F32, I64 };

struct SigArg {
  const char *name;
  ArgKind kind;
  uint32_t size() const { return kind == ArgKind::Buffer || kind == ArgKind::I64 ? 8 : 4; }
  uint32_t align() const { return size(); }
  const char *value_kind() const { return kind == ArgKind::Buffer ? "global_buffer" : "by_value"; }
};

using Signature = std::vector<SigArg>;

// The declared signature of a kernel symbol of the gfx950 objects, or nullptr.
const Signature *signature_for(const std::string &kernel);

// (offset, size) per argument by natural alignment; returns the explicit kernarg bytes.
uint32_t pack(const Signature &sig, std::vector<std::pair<uint32_t, uint32_t>> &out);

}  // namespace iu8
