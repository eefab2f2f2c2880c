// Loader, launcher and the operator-level entry points: the counterpart of
// crates/saber-exec/src/loader.rs (PluginSet::load_dir, :318-396), crates/saber-exec/src/launch.rs
// (pack_kernarg :123, Launcher::launch_op :590-660) and the HIP calls of crates/saber-hip
// (hipModuleLoadData / hipModuleGetFunction / hipModuleLaunchKernel with a packed-kernarg
// `extra`, src/ffi.rs:917-995).
#include <dirent.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstring>
#include <map>

#include "../../../include/saber_iu8.h"
#include "abi.h"
#include "manifest.h"
#include "rules.h"
#include "static_ws.h"
#include "util.h"

using namespace iu8;

struct LoadedKernel {
  hipFunction_t fn;
  uint32_t max_threads;  // the code object's max_flat_workgroup_size: the block its indexing is written for
  int64_t resident;      // workgroups of that size the device holds at once (kernels that meet inside a launch), else 0
};
struct saber_iu8_ctx {
  int device = 0;
  std::string arch;
  std::vector<hipModule_t> modules;
  std::map<std::string, LoadedKernel> fn;
  saber_iu8_counters counters{};
  std::string static_ws_error;  // why this device has no static workspace (empty: it has one)
};

static int hip_fail(const char *what, hipError_t e) {
  return fail(SABER_IU8_E_HIP, fmt("%s: HIP status %d (%s)", what, (int)e, hipGetErrorString(e)));
}

// Runs the loader's validations on one manifest; fills manifest, blob; names the refusal.
static int load_and_validate(const std::string &manifest_path, const std::string &arch, Manifest &m,
                             std::vector<uint8_t> &blob, int *refusal) {
  if (refusal) *refusal = 0;
  std::vector<uint8_t> text;
  if (!read_file(manifest_path, text)) return fail(SABER_IU8_E_IO, manifest_path + ": cannot read");
  std::string why;
  if (!manifest_parse_toml(std::string(text.begin(), text.end()), m, &why)) return fail(SABER_IU8_E_PARSE, manifest_path + ": " + why);
  if (!check_kernarg_layout(m, &why)) {
    if (refusal) *refusal = SABER_IU8_REFUSED_KERNARG;
    return fail(SABER_IU8_E_VALIDATE, "refused (kernarg): " + why);
  }
  const size_t slash = manifest_path.find_last_of('/');
  const std::string dir = slash == std::string::npos ? "." : manifest_path.substr(0, slash);
  if (!read_file(dir + "/" + m.hsaco, blob)) return fail(SABER_IU8_E_IO, dir + "/" + m.hsaco + ": cannot read");
  CodeObject co;
  if (!parse_code_object(blob, co, &why)) return fail(SABER_IU8_E_PARSE, m.hsaco + ": " + why);
  if (!check_wave_size(m, &why)) {
    if (refusal) *refusal = SABER_IU8_REFUSED_WAVE;
    return fail(SABER_IU8_E_VALIDATE, "refused (wave): " + why);
  }
  if (!validate_against_hsaco(m, blob, co, arch, &why)) {
    if (refusal) *refusal = SABER_IU8_REFUSED_METADATA;
    return fail(SABER_IU8_E_VALIDATE, "refused (metadata): " + why);
  }
  return 0;
}

static const void *find_binding(const saber_iu8_binding *bufs, uint32_t n, const char *name, bool *found) {
  for (uint32_t i = 0; i < n; ++i)
    if (bufs[i].name && !strcmp(bufs[i].name, name)) {
      *found = true;
      return bufs[i].ptr;
    }
  *found = false;
  return nullptr;
}

// Validates one manifest + code object and adds its kernels to the context. A refusal moves the
// counter it names and leaves the context as it was (the plugin is skipped, loader.rs:249-270); a HIP
// failure is returned as such.
static int load_one(saber_iu8_ctx *ctx, const std::string &manifest_path) {
  Manifest m;
  std::vector<uint8_t> blob;
  int refusal = 0;
  const int rc = load_and_validate(manifest_path, ctx->arch, m, blob, &refusal);
  if (rc != 0) {
    if (refusal == SABER_IU8_REFUSED_KERNARG) ctx->counters.refused_kernarg++;
    else if (refusal == SABER_IU8_REFUSED_WAVE) ctx->counters.refused_wave++;
    else ctx->counters.refused_metadata++;
    return rc;
  }
  hipModule_t mod;
  hipError_t e;
  if ((e = hipModuleLoadData(&mod, blob.data())) != hipSuccess) return hip_fail(("hipModuleLoadData " + m.hsaco).c_str(), e);
  ctx->modules.push_back(mod);
  ctx->counters.plugins_loaded++;
  for (const KernelDecl &k : m.kernel) {
    hipFunction_t fn;
    if ((e = hipModuleGetFunction(&fn, mod, k.name.c_str())) != hipSuccess) return hip_fail(("hipModuleGetFunction " + k.name).c_str(), e);
    int64_t resident = 0;
    if (k.name.rfind("macaq_iu8f_mlp_", 0) == 0) {
      // asked once, at load: the launch itself may run under stream capture
      int per_cu = 0, cus = 0;
      if ((e = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, (int)k.max_flat_workgroup_size, 0)) != hipSuccess)
        return hip_fail("hipModuleOccupancyMaxActiveBlocksPerMultiprocessor", e);
      if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, ctx->device)) != hipSuccess)
        return hip_fail("hipDeviceGetAttribute", e);
      resident = (int64_t)per_cu * cus;
    }
    ctx->fn[k.name] = LoadedKernel{fn, k.max_flat_workgroup_size, resident};
    ctx->counters.kernels_loaded++;
  }
  return 0;
}

extern "C" {

const char *saber_iu8_last_error(void) { return last_error(); }
int saber_iu8_abi_version(void) { return SABER_IU8_ABI_VERSION; }

int saber_iu8_resolve(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out) {
  if (!out) return fail(SABER_IU8_E_ARG, "resolve: null descriptor");
  return resolve(wkind, m, n, k, out);
}
int saber_iu8_describe(const char *kernel, uint32_t m, uint32_t n, uint32_t k, uint32_t ks, saber_iu8_desc *out) {
  if (!out || !kernel) return fail(SABER_IU8_E_ARG, "describe: null argument");
  return describe(kernel, m, n, k, ks, out);
}
int saber_iu8_resolve_quant(uint32_t m, uint32_t k, saber_iu8_desc *out) {
  if (!out) return fail(SABER_IU8_E_ARG, "resolve_quant: null descriptor");
  return resolve_quant(m, k, out);
}
int saber_iu8_pair(const saber_iu8_desc *first, const saber_iu8_desc *second, saber_iu8_desc *out) {
  if (!first || !second || !out) return fail(SABER_IU8_E_ARG, "pair: null descriptor");
  return pair(*first, *second, out);
}
int saber_iu8_pair_ordered(const saber_iu8_desc *first, const saber_iu8_desc *second, int second_first, saber_iu8_desc *out) {
  if (!first || !second || !out) return fail(SABER_IU8_E_ARG, "pair: null descriptor");
  return pair(*first, *second, out, second_first ? 1 : 0);
}
int saber_iu8_fused_holds(uint32_t m, uint32_t k) { return fused_holds(m, k) ? 1 : 0; }
int saber_iu8_mlp_chain_holds(uint32_t m, uint32_t hidden, uint32_t inter) {
  return mlp_chain_form_holds(m, hidden, inter) ? 1 : 0;
}
int saber_iu8_mlp_chain_pays(uint32_t m, uint32_t hidden, uint32_t inter) {
  return mlp_chain_pays(m, hidden, inter) ? 1 : 0;
}
int saber_iu8_resolve_fused(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out) {
  if (!out) return fail(SABER_IU8_E_ARG, "resolve_fused: null descriptor");
  return resolve_fused(wkind, m, n, k, out);
}
int saber_iu8_resolve_silu_mul_quant(uint32_t rows, uint32_t n, saber_iu8_desc *out) {
  if (!out) return fail(SABER_IU8_E_ARG, "resolve_silu_mul_quant: null descriptor");
  return resolve_silu_mul_quant(rows, n, out);
}

int saber_iu8_describe_raw(const char *kernel, const char *plugin, const uint32_t grid[3], uint32_t block,
                           saber_iu8_desc *out) {
  if (!kernel || !grid || !out) return fail(SABER_IU8_E_ARG, "describe_raw: null argument");
  if (!grid[0] || !grid[1] || !grid[2] || !block || block > 1024) return fail(SABER_IU8_E_RULE, std::string(kernel) + ": empty or oversized launch");
  memset(out, 0, sizeof *out);
  snprintf(out->op, sizeof out->op, "raw");
  snprintf(out->plugin, sizeof out->plugin, "%s", plugin ? plugin : "");
  snprintf(out->kernel, sizeof out->kernel, "%s", kernel);
  for (int i = 0; i < 3; ++i) out->grid[i] = grid[i];
  out->block[0] = block, out->block[1] = 1, out->block[2] = 1;
  out->n_launches = 1;
  out->ks = 1;
  return fill_slots(kernel, out);
}

int saber_iu8_desc_set_i32(saber_iu8_desc *desc, const char *name, int64_t value) {
  if (!desc || !name) return fail(SABER_IU8_E_ARG, "desc_set_i32: null argument");
  for (uint32_t i = 0; i < desc->n_args; ++i)
    if (!strcmp(desc->args[i].name, name)) {
      if (desc->args[i].kind == SABER_IU8_ARG_BUFFER || desc->args[i].kind == SABER_IU8_ARG_NULL_BUFFER)
        return fail(SABER_IU8_E_ARG, std::string(name) + ": a buffer slot, not a scalar");
      desc->args[i].kind = desc->args[i].size == 8 ? SABER_IU8_ARG_I64 : SABER_IU8_ARG_I32;
      desc->args[i].ival = value;
      return 0;
    }
  return fail(SABER_IU8_E_ARG, std::string(desc->kernel) + ": no argument `" + name + "`");
}

int saber_iu8_signature(const char *kernel, saber_iu8_slot *slots, uint32_t cap, uint32_t *n_slots, uint32_t *bytes) {
  if (!kernel || !slots || !n_slots || !bytes) return fail(SABER_IU8_E_ARG, "signature: null argument");
  saber_iu8_desc d;
  memset(&d, 0, sizeof d);
  if (int rc = fill_slots(kernel, &d)) return rc;
  if (d.n_args > cap) return fail(SABER_IU8_E_ARG, "signature: slot array too small");
  memcpy(slots, d.args, sizeof(saber_iu8_slot) * d.n_args);
  *n_slots = d.n_args;
  *bytes = d.kernarg_bytes;
  return 0;
}

int saber_iu8_pack_kernarg(const saber_iu8_desc *d, const saber_iu8_binding *bufs, uint32_t n_bufs, uint8_t *image,
                           uint32_t cap, uint32_t *bytes) {
  if (!d || !image || (!bufs && n_bufs)) return fail(SABER_IU8_E_ARG, "pack_kernarg: null argument");
  if (cap < d->kernarg_bytes) return fail(SABER_IU8_E_ARG, fmt("pack_kernarg: image of %u B, the kernel takes %u", cap, d->kernarg_bytes));
  memset(image, 0, d->kernarg_bytes);  // padding is zero-filled (launch.rs:120-122)
  for (uint32_t i = 0; i < d->n_args; ++i) {
    const saber_iu8_slot &s = d->args[i];
    if (s.offset + s.size > d->kernarg_bytes) return fail(SABER_IU8_E_ARG, fmt("%s: slot `%s` past the kernarg block", d->kernel, s.name));
    switch (s.kind) {
      case SABER_IU8_ARG_BUFFER: {
        bool found;
        const void *p = find_binding(bufs, n_bufs, s.name, &found);
        if (!found) return fail(SABER_IU8_E_ARG, fmt("%s: buffer `%s` is not bound", d->kernel, s.name));
        if (!p) return fail(SABER_IU8_E_ARG, fmt("%s: buffer `%s` is bound to NULL", d->kernel, s.name));
        memcpy(image + s.offset, &p, 8);
        break;
      }
      case SABER_IU8_ARG_NULL_BUFFER:
        break;
      case SABER_IU8_ARG_I32: {
        const int32_t v = (int32_t)s.ival;
        memcpy(image + s.offset, &v, 4);
        break;
      }
      case SABER_IU8_ARG_I64:
        memcpy(image + s.offset, &s.ival, 8);
        break;
      case SABER_IU8_ARG_F32:
        memcpy(image + s.offset, &s.fval, 4);
        break;
      default:
        return fail(SABER_IU8_E_ARG, fmt("%s: slot `%s` has unknown kind %u", d->kernel, s.name, s.kind));
    }
  }
  if (bytes) *bytes = d->kernarg_bytes;
  return 0;
}

int saber_iu8_sha256_file(const char *path, char *out65) {
  if (!path || !out65) return fail(SABER_IU8_E_ARG, "sha256_file: null argument");
  std::vector<uint8_t> b;
  if (!read_file(path, b)) return fail(SABER_IU8_E_IO, std::string(path) + ": cannot read");
  snprintf(out65, 65, "%s", sha256_hex(b.data(), b.size()).c_str());
  return 0;
}

int saber_iu8_manifest_write(const char *hsaco_path, const char *plugin, const char *arch, const char *source,
                             const char *source_sha256, const char *flags, const char *build_hash, const char *out_path) {
  if (!hsaco_path || !plugin || !arch || !source || !source_sha256 || !flags || !build_hash || !out_path)
    return fail(SABER_IU8_E_ARG, "manifest_write: null argument");
  std::vector<uint8_t> blob;
  if (!read_file(hsaco_path, blob)) return fail(SABER_IU8_E_IO, std::string(hsaco_path) + ": cannot read");
  CodeObject co;
  std::string why;
  if (!parse_code_object(blob, co, &why)) return fail(SABER_IU8_E_PARSE, std::string(hsaco_path) + ": " + why);
  if (co.target.find(arch) == std::string::npos)
    return fail(SABER_IU8_E_VALIDATE, "code object target " + co.target + " is not " + arch);
  const std::string hp(hsaco_path);
  const size_t slash = hp.find_last_of('/');
  Manifest m = manifest_from_code_object(co, plugin, arch, source, source_sha256, flags, build_hash,
                                         slash == std::string::npos ? hp : hp.substr(slash + 1),
                                         sha256_hex(blob.data(), blob.size()));
  // Name the arguments from the declared signatures (the code object has offsets but no names) and
  // refuse a kernel that has no signature or does not pack the way it does (manifest.rs:170-207).
  std::sort(m.kernel.begin(), m.kernel.end(), [](const KernelDecl &x, const KernelDecl &y) { return x.name < y.name; });
  for (KernelDecl &k : m.kernel) {
    const Signature *sig = signature_for(k.name);
    if (!sig) return fail(SABER_IU8_E_VALIDATE, k.name + ": no declared signature for this symbol");
    if (sig->size() != k.arg.size())
      return fail(SABER_IU8_E_VALIDATE, fmt("%s: signature has %zu args, code object %zu", k.name.c_str(), sig->size(), k.arg.size()));
    for (size_t i = 0; i < sig->size(); ++i) k.arg[i].name = (*sig)[i].name;
  }
  if (!check_kernarg_layout(m, &why)) return fail(SABER_IU8_E_VALIDATE, why);
  if (!write_file(out_path, manifest_to_toml(m))) return fail(SABER_IU8_E_IO, std::string(out_path) + ": cannot write");
  return 0;
}

int saber_iu8_manifest_validate(const char *manifest_path, const char *arch, int *refusal) {
  if (!manifest_path) return fail(SABER_IU8_E_ARG, "manifest_validate: null path");
  Manifest m;
  std::vector<uint8_t> blob;
  return load_and_validate(manifest_path, arch ? arch : "", m, blob, refusal);
}

int saber_iu8_open(const char *prebuilt_dir, int device, saber_iu8_ctx **out) {
  if (!prebuilt_dir || !out) return fail(SABER_IU8_E_ARG, "open: null argument");
  *out = nullptr;
  int ndev = 0;
  hipError_t e = hipGetDeviceCount(&ndev);
  if (e != hipSuccess || ndev <= 0) return hip_fail("hipGetDeviceCount (no GPU visible: this path has no CPU fallback)", e);
  if ((e = hipSetDevice(device)) != hipSuccess) return hip_fail("hipSetDevice", e);
  hipDeviceProp_t prop;
  if ((e = hipGetDeviceProperties(&prop, device)) != hipSuccess) return hip_fail("hipGetDeviceProperties", e);
  std::string arch(prop.gcnArchName);
  arch = arch.substr(0, arch.find(':'));
  DIR *dp = opendir(prebuilt_dir);
  if (!dp) return fail(SABER_IU8_E_IO, std::string(prebuilt_dir) + ": cannot open directory");
  std::vector<std::string> manifests;
  while (dirent *de = readdir(dp)) {
    const std::string f = de->d_name;
    const std::string suf = ".manifest.toml";
    if (f.size() > suf.size() && f.compare(f.size() - suf.size(), suf.size(), suf) == 0) manifests.push_back(f);
  }
  closedir(dp);
  std::sort(manifests.begin(), manifests.end());
  saber_iu8_ctx *ctx = new saber_iu8_ctx();
  ctx->device = device;
  ctx->arch = arch;
  std::string first_refusal;
  for (const std::string &f : manifests) {
    const int rc = load_one(ctx, std::string(prebuilt_dir) + "/" + f);
    if (rc == SABER_IU8_E_HIP) {
      saber_iu8_close(ctx);
      return rc;
    }
    if (rc != 0 && first_refusal.empty()) first_refusal = f + ": " + last_error();
  }
  if (ctx->modules.empty()) {
    const std::string msg = std::string(prebuilt_dir) + ": no plugin loaded for " + arch +
                            (first_refusal.empty() ? " (no *.manifest.toml)" : " (" + first_refusal + ")");
    saber_iu8_close(ctx);
    return fail(SABER_IU8_E_NOTLOADED, msg);
  }
  // The library's static split-K workspace on this device (saber_iu8_gemm_static): its address is taken here,
  // once a device, with the device current and behind the plugin set, whose refusals say more about a device
  // this library is not built for than a failed symbol look-up would. A failure is kept, not returned: only
  // saber_iu8_gemm_static needs the array, and it then says why it has none.
  if (static_ws_init(device) != 0) ctx->static_ws_error = last_error();
  *out = ctx;
  return 0;
}

int saber_iu8_load_plugin(saber_iu8_ctx *ctx, const char *manifest_path) {
  if (!ctx || !manifest_path) return fail(SABER_IU8_E_ARG, "load_plugin: null argument");
  hipError_t e;
  if ((e = hipSetDevice(ctx->device)) != hipSuccess) return hip_fail("hipSetDevice", e);
  return load_one(ctx, manifest_path);
}

void saber_iu8_close(saber_iu8_ctx *ctx) {
  if (!ctx) return;
  for (hipModule_t m : ctx->modules) (void)hipModuleUnload(m);
  delete ctx;
}

int saber_iu8_get_counters(const saber_iu8_ctx *ctx, saber_iu8_counters *out) {
  if (!ctx || !out) return fail(SABER_IU8_E_ARG, "get_counters: null argument");
  *out = ctx->counters;
  return 0;
}

int saber_iu8_has_kernel(const saber_iu8_ctx *ctx, const char *kernel) {
  return ctx && kernel && ctx->fn.count(kernel) ? 1 : 0;
}

// What a hand-edited descriptor could get wrong for a kernel whose bounds depend on its grid: the
// fused decode linear keeps at most 8 column blocks' weight scales a workgroup and 20 KiB of codes.
static int i32_arg(const saber_iu8_desc *d, const char *name) {
  for (uint32_t i = 0; i < d->n_args; ++i)
    if (d->args[i].kind == SABER_IU8_ARG_I32 && !strcmp(d->args[i].name, name)) return (int)d->args[i].ival;
  return 0;
}

// The decode MLP chain's workgroups meet inside the launch: a grid the card cannot hold all at once
// would wait for workgroups that never start (until the kernel's bounded wait gives up), so it is
// refused here from what the loaded kernel's registers and LDS let reside.
static int chain_guard(const LoadedKernel &lk, const saber_iu8_desc *d) {
  const int64_t m = i32_arg(d, "m"), h = i32_arg(d, "k"), i = i32_arg(d, "n");
  const bool a80 = strstr(d->kernel, "_a80") != nullptr;
  if (m <= 0 || h <= 0 || i <= 0 || !fused_small_holds((uint32_t)m, (uint32_t)h) ||
      !(a80 ? m <= 4 && fused_form_holds(true, (uint32_t)m, (uint32_t)i) : fused_small_holds((uint32_t)m, (uint32_t)i)) || h % 128 || i % 128)
    return fail(SABER_IU8_E_RULE, fmt("%s: %lld rows of %lld / %lld do not fit the fused form", d->kernel, (long long)m, (long long)h,
                                      (long long)i));
  const int64_t nblk = std::max(i / 16, (h + 31) / 32);
  if ((int64_t)d->grid[0] * 8 < nblk || d->grid[0] > MLP_CHAIN_MAX_GRID || d->grid[1] != 1 || d->grid[2] != 1 || i32_arg(d, "spin") <= 0)
    return fail(SABER_IU8_E_RULE, fmt("%s: grid %u x %u x %u: %lld column blocks at most 8 a workgroup, at most %u workgroups, a spin limit",
                                      d->kernel, d->grid[0], d->grid[1], d->grid[2], (long long)nblk, MLP_CHAIN_MAX_GRID));
  if (lk.resident < (int64_t)d->grid[0])
    return fail(SABER_IU8_E_RULE, fmt("%s: %u workgroups must be resident at once; this device holds %lld", d->kernel, d->grid[0],
                                      (long long)lk.resident));
  return 0;
}

static int launch_guard(const LoadedKernel &lk, const saber_iu8_desc *d) {
  if (strncmp(d->kernel, "macaq_iu8f_mlp_", 15) == 0) return chain_guard(lk, d);
  if (strncmp(d->kernel, "macaq_iu8f_gateup_act_", 22) == 0) {
    const int64_t m = i32_arg(d, "m"), n = i32_arg(d, "n"), k = i32_arg(d, "k");
    if (m <= 0 || n <= 0 || k <= 0 || !gate_up_act_holds((uint32_t)m, (uint32_t)k, (uint32_t)n))
      return fail(SABER_IU8_E_RULE, fmt("%s: %lld rows of %lld / %lld do not fit the form", d->kernel, (long long)m, (long long)k, (long long)n));
    if ((int64_t)d->grid[0] * 8 < n / 16 || d->grid[1] != 1 || d->grid[2] != 1)
      return fail(SABER_IU8_E_RULE, fmt("%s: grid %u x %u x %u cannot walk %lld column blocks (at most 8 a workgroup)", d->kernel,
                                        d->grid[0], d->grid[1], d->grid[2], (long long)(n / 16)));
    return 0;
  }
  const size_t klen = strlen(d->kernel);
  const bool s80r = klen > 5 && !strcmp(d->kernel + klen - 5, "_s80r");
  const bool s80 = s80r || (klen > 4 && !strcmp(d->kernel + klen - 4, "_s80"));
  if (strncmp(d->kernel, "macaq_iu8_decq_", 15) != 0 && !s80) return 0;
  int64_t m = 0, n = 0, k = 0;
  for (uint32_t i = 0; i < d->n_args; ++i) {
    if (d->args[i].kind != SABER_IU8_ARG_I32) continue;
    if (!strcmp(d->args[i].name, "m")) m = d->args[i].ival;
    if (!strcmp(d->args[i].name, "n")) n = d->args[i].ival;
    if (!strcmp(d->args[i].name, "k")) k = d->args[i].ival;
  }
  if (s80) {  // the staged tile: 16 rows x K bytes of LDS, the fused forms' block walk
    // the whole-tile kernel indexes 16 rows a K step whatever M is; the rows kernel the live rows rounded up to a power of two
    if (m <= 0 || n <= 0 || k <= 0 || k % 128 || m > 16 || (s80r ? !staged80_holds((uint32_t)m, (uint32_t)k) : (int64_t)k * 16 > 80 * 1024))
      return fail(SABER_IU8_E_RULE, fmt("%s: %lld rows of %lld do not fit one 16-row tile in 80 KiB", d->kernel, (long long)m, (long long)k));
    if ((int64_t)d->grid[0] * 8 < (n + 31) / 32 || d->grid[1] != 1 || d->grid[2] != 1)
      return fail(SABER_IU8_E_RULE, fmt("%s: grid %u x %u x %u cannot walk %lld column blocks (at most 8 a workgroup)", d->kernel,
                                        d->grid[0], d->grid[1], d->grid[2], (long long)((n + 31) / 32)));
    return 0;
  }
  const bool a80 = strstr(d->kernel, "_a80") != nullptr;
  const size_t len = klen;
  if (len > 3 && !strcmp(d->kernel + len - 3, "_r1") && m != 1)
    return fail(SABER_IU8_E_RULE, fmt("%s: the one-row form, got %lld rows", d->kernel, (long long)m));
  if (m <= 0 || n <= 0 || k <= 0 || !fused_form_holds(a80, (uint32_t)m, (uint32_t)k))
    return fail(SABER_IU8_E_RULE, fmt("%s: %lld rows of %lld do not fit the fused form", d->kernel, (long long)m, (long long)k));
  const int64_t nblk = (n + 31) / 32;
  if ((int64_t)d->grid[0] * 8 < nblk || d->grid[1] != 1 || d->grid[2] != 1)
    return fail(SABER_IU8_E_RULE, fmt("%s: grid %u x %u x %u of %u threads cannot walk %lld column blocks (at most 8 a workgroup)",
                                      d->kernel, d->grid[0], d->grid[1], d->grid[2], d->block[0], (long long)nblk));
  return 0;
}

int saber_iu8_launch(saber_iu8_ctx *ctx, const saber_iu8_desc *d, const saber_iu8_binding *bufs, uint32_t n_bufs,
                     void *stream) {
  if (!ctx || !d) return fail(SABER_IU8_E_ARG, "launch: null argument");
  auto it = ctx->fn.find(d->kernel);
  if (it == ctx->fn.end()) return fail(SABER_IU8_E_NOTLOADED, std::string(d->kernel) + ": not in the loaded plugin set");
  if (d->shared_bytes != 0) return fail(SABER_IU8_E_RULE, std::string(d->kernel) + ": dynamic LDS is not part of this ABI");
  if (!d->grid[0] || !d->grid[1] || !d->grid[2] || !d->block[0]) return fail(SABER_IU8_E_RULE, std::string(d->kernel) + ": empty grid");
  // Every kernel of these objects indexes by the workgroup size it was compiled for (its
  // max_flat_workgroup_size): a descriptor from another launch law -- the reference's 256-thread
  // blocks under its own names -- would run and give wrong bytes, so it is refused here by name.
  const uint64_t threads = (uint64_t)d->block[0] * std::max(d->block[1], 1u) * std::max(d->block[2], 1u);
  if (threads != it->second.max_threads)
    return fail(SABER_IU8_E_RULE, fmt("%s: a block of %llu threads; the gfx950 kernel is written for %u (use this object's launch law)",
                                      d->kernel, (unsigned long long)threads, it->second.max_threads));
  if (int rc = launch_guard(it->second, d)) return rc;
  alignas(16) uint8_t image[256];
  uint32_t bytes = 0;
  if (int rc = saber_iu8_pack_kernarg(d, bufs, n_bufs, image, sizeof image, &bytes)) return rc;
  size_t sz = bytes;
  void *extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, image, HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz, HIP_LAUNCH_PARAM_END};
  const hipError_t e = hipModuleLaunchKernel(it->second.fn, d->grid[0], d->grid[1], d->grid[2], d->block[0], d->block[1],
                                             d->block[2], 0, (hipStream_t)stream, nullptr, extra);
  if (e != hipSuccess) return hip_fail(d->kernel, e);
  ctx->counters.launches++;
  return 0;
}

int saber_iu8_quant(saber_iu8_ctx *ctx, const void *x, void *q, float *scale, uint32_t m, uint32_t k, void *stream) {
  saber_iu8_desc d;
  if (int rc = resolve_quant(m, k, &d)) return rc;
  const saber_iu8_binding b[] = {{"x", (void *)x}, {"q", q}, {"scale", scale}};
  return saber_iu8_launch(ctx, &d, b, 3, stream);
}

int saber_iu8_quant_rowmajor(saber_iu8_ctx *ctx, const void *x, void *q, float *scale, uint32_t m, uint32_t k, void *stream) {
  saber_iu8_desc d;
  if (int rc = resolve_quant_rowmajor(m, k, &d)) return rc;
  const saber_iu8_binding b[] = {{"x", (void *)x}, {"q", q}, {"scale", scale}};
  return saber_iu8_launch(ctx, &d, b, 3, stream);
}

int saber_iu8_linear_fused(saber_iu8_ctx *ctx, int wkind, const void *x, const void *w, const float *ws, void *c, void *q,
                           float *scale, uint32_t m, uint32_t n, uint32_t k, void *stream) {
  saber_iu8_desc d;
  if (int rc = resolve_fused(wkind, m, n, k, &d)) return rc;
  // the optional outputs are named-null when absent: the kernel tests the pointers
  if (!q) set_null(&d, "q");
  if (!scale) set_null(&d, "scale");
  const saber_iu8_binding b[] = {{"x", (void *)x}, {"w", (void *)w}, {"ws", (void *)ws}, {"c", c}, {"q", q}, {"scale", scale}};
  return saber_iu8_launch(ctx, &d, b, 6, stream);
}

int saber_iu8_resolve_mlp_chain(uint32_t m, uint32_t hidden, uint32_t inter, uint32_t spin, saber_iu8_desc *out) {
  if (!out) return fail(SABER_IU8_E_ARG, "resolve_mlp_chain: null descriptor");
  return resolve_mlp_chain(m, hidden, inter, spin, out);
}

int saber_iu8_mlp_chain(saber_iu8_ctx *ctx, const void *x, const void *w_gu, const float *ws_gu, const void *w_dn,
                        const float *ws_dn, void *gu, void *p, void *state, void *c, uint32_t m, uint32_t hidden, uint32_t inter,
                        uint32_t spin, void *stream) {
  saber_iu8_desc d;
  if (int rc = resolve_mlp_chain(m, hidden, inter, spin, &d)) return rc;
  if (!gu) set_null(&d, "gu");  // the [gate | up] rows are a tap: the kernel tests the pointer
  const saber_iu8_binding b[] = {{"x", (void *)x},         {"w", (void *)w_gu}, {"ws", (void *)ws_gu}, {"w_b", (void *)w_dn},
                                 {"ws_b", (void *)ws_dn}, {"gu", gu},          {"p", p},              {"state", state},
                                 {"c", c}};
  return saber_iu8_launch(ctx, &d, b, 9, stream);
}

int saber_iu8_gate_up_act_holds(uint32_t m, uint32_t hidden, uint32_t inter) { return gate_up_act_holds(m, hidden, inter) ? 1 : 0; }
int saber_iu8_resolve_gate_up_act(uint32_t m, uint32_t hidden, uint32_t inter, saber_iu8_desc *out) {
  if (!out) return fail(SABER_IU8_E_ARG, "resolve_gate_up_act: null descriptor");
  return resolve_gate_up_act(m, hidden, inter, out);
}
int saber_iu8_gate_up_act(saber_iu8_ctx *ctx, const void *a, const float *as, const void *w_gu, const float *ws_gu, void *gu,
                          void *p, uint32_t m, uint32_t hidden, uint32_t inter, void *stream) {
  saber_iu8_desc d;
  if (int rc = resolve_gate_up_act(m, hidden, inter, &d)) return rc;
  if (!gu) set_null(&d, "gu");  // the [gate | up] rows are a tap: the kernel tests the pointer
  const saber_iu8_binding b[] = {{"a", (void *)a}, {"w", (void *)w_gu}, {"as", (void *)as}, {"ws", (void *)ws_gu}, {"gu", gu}, {"p", p}};
  return saber_iu8_launch(ctx, &d, b, 6, stream);
}

int saber_iu8_rowscale(saber_iu8_ctx *ctx, const void *x, float *scale, uint32_t m, uint32_t k, void *stream) {
  saber_iu8_desc d;
  if (int rc = resolve_rowscale(m, k, &d)) return rc;
  const saber_iu8_binding b[] = {{"x", (void *)x}, {"scale", scale}};
  return saber_iu8_launch(ctx, &d, b, 2, stream);
}

int saber_iu8_resolve_prefill_fused(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out) {
  if (!out) return fail(SABER_IU8_E_ARG, "resolve_prefill_fused: null descriptor");
  return resolve_prefill_fused(wkind, m, n, k, out);
}

int saber_iu8_linear_prefill_fused(saber_iu8_ctx *ctx, int wkind, const void *x, const float *as, const void *w, const float *ws,
                                   void *c, uint32_t m, uint32_t n, uint32_t k, void *stream) {
  saber_iu8_desc d;
  if (int rc = resolve_prefill_fused(wkind, m, n, k, &d)) return rc;
  const saber_iu8_binding b[] = {{"x", (void *)x}, {"w", (void *)w}, {"as", (void *)as}, {"ws", (void *)ws}, {"c", c}};
  return saber_iu8_launch(ctx, &d, b, 5, stream);
}

int saber_iu8_gemm_workspace(int wkind, uint32_t m, uint32_t n, uint32_t k, uint64_t *partial_bytes, uint64_t *counter_bytes) {
  saber_iu8_desc d;
  if (int rc = resolve(wkind, m, n, k, &d)) return rc;
  uint64_t p = 0, c = 0;
  for (uint32_t i = 0; i < d.n_workspaces; ++i) {
    if (!strcmp(d.workspaces[i].name, "decode_partial")) p = d.workspaces[i].bytes;
    if (!strcmp(d.workspaces[i].name, "decode_counter")) c = d.workspaces[i].bytes;
  }
  if (partial_bytes) *partial_bytes = p;
  if (counter_bytes) *counter_bytes = c;
  return 0;
}

static int launch_gemm(saber_iu8_ctx *ctx, const saber_iu8_desc &d, const void *a, const float *as, const void *w,
                       const float *ws, void *c, void *partial, void *counter, void *stream) {
  const saber_iu8_binding b[] = {{"a", (void *)a},   {"w", (void *)w},           {"as", (void *)as},         {"ws", (void *)ws},
                                 {"c", c},           {"decode_partial", partial}, {"decode_counter", counter}};
  return saber_iu8_launch(ctx, &d, b, 7, stream);
}

int saber_iu8_gemm(saber_iu8_ctx *ctx, int wkind, const void *a, const float *as, const void *w, const float *ws,
                   void *c, uint32_t m, uint32_t n, uint32_t k, void *partial, void *counter, void *stream) {
  saber_iu8_desc d;
  if (int rc = resolve(wkind, m, n, k, &d)) return rc;
  return launch_gemm(ctx, d, a, as, w, ws, c, partial, counter, stream);
}

// saber_iu8_gemm with the split-K workspaces in the library's static device array: nothing is
// allocated, cleared or synchronised here (the counters are zero from set-up and left zero by every
// kernel that uses them; the partials are written before they are read).
int saber_iu8_gemm_static(saber_iu8_ctx *ctx, int wkind, const void *a, const float *as, const void *w, const float *ws,
                          void *c, uint32_t m, uint32_t n, uint32_t k, void *stream) {
  if (!ctx) return fail(SABER_IU8_E_ARG, "gemm_static: null context");
  saber_iu8_desc d;
  if (int rc = resolve(wkind, m, n, k, &d)) return rc;
  void *partial = nullptr, *counter = nullptr;
  for (uint32_t i = 0; i < d.n_workspaces; ++i) {
    const saber_iu8_workspace &wsp = d.workspaces[i];
    const bool is_partial = !strcmp(wsp.name, "decode_partial");
    const uint64_t cap = is_partial ? STATIC_WS_PARTIAL_BYTES : STATIC_WS_COUNTER_BYTES;
    if (wsp.bytes > cap)
      return fail(SABER_IU8_E_RULE, fmt("gemm_static: %u x %u x %u needs %llu B of `%s`, the static workspace holds %llu; use saber_iu8_gemm "
                                        "with caller-owned workspaces", m, n, k, (unsigned long long)wsp.bytes, wsp.name, (unsigned long long)cap));
    (is_partial ? partial : counter) = is_partial ? static_ws_partial(ctx->device) : static_ws_counter(ctx->device);
  }
  if (d.n_workspaces && (!partial || !counter))
    return fail(SABER_IU8_E_NOTLOADED, fmt("gemm_static: the static workspace of device %d was not set up%s%s", ctx->device,
                                           ctx->static_ws_error.empty() ? "" : ": ", ctx->static_ws_error.c_str()));
  return launch_gemm(ctx, d, a, as, w, ws, c, partial, counter, stream);
}

int saber_iu8_static_workspace_reset(saber_iu8_ctx *ctx, void *stream) {
  if (!ctx) return fail(SABER_IU8_E_ARG, "static_workspace_reset: null context");
  return static_ws_reset(ctx->device, stream);
}

uint64_t saber_iu8_static_workspace_bytes(void) { return STATIC_WS_BYTES; }

// Two W4 linears on one activation operand in one dispatch (decode band; the launch law's own
// descriptors, which do not split K, so no workspace is bound).
int saber_iu8_gemm_pair(saber_iu8_ctx *ctx, const void *a, const float *as, const void *w, const float *ws, void *c, uint32_t n,
                        const void *w_b, const float *ws_b, void *c_b, uint32_t n_b, uint32_t m, uint32_t k, void *stream) {
  saber_iu8_desc d0, d1, d;
  if (int rc = resolve(SABER_IU8_W4, m, n, k, &d0)) return rc;
  if (int rc = resolve(SABER_IU8_W4, m, n_b, k, &d1)) return rc;
  if (int rc = pair(d0, d1, &d)) return rc;
  if (d.n_workspaces) return fail(SABER_IU8_E_RULE, "gemm_pair: a half splits K; bind its workspaces through saber_iu8_pair + saber_iu8_launch");
  const saber_iu8_binding b[] = {{"a", (void *)a},     {"as", (void *)as},     {"w", (void *)w}, {"ws", (void *)ws}, {"c", c},
                                 {"w_b", (void *)w_b}, {"ws_b", (void *)ws_b}, {"c_b", c_b}};
  return saber_iu8_launch(ctx, &d, b, 8, stream);
}

int saber_iu8_gemm_acc(saber_iu8_ctx *ctx, int wkind, const void *a, const void *w, int32_t *acc, uint32_t m, uint32_t n,
                       uint32_t k, void *stream) {
  if (wkind != SABER_IU8_W4 && wkind != SABER_IU8_W8) return fail(SABER_IU8_E_ARG, "unknown weight kind");
  const char *tag = wkind == SABER_IU8_W8 ? "w8" : "w4";
  saber_iu8_desc d;
  const std::string name = m <= 16 ? fmt("macaq_iu8_dec_%s_tm1_acc", tag) : fmt("macaq_iu8_pf_%s_acc", tag);
  if (int rc = describe(name, m, n, k, 1, &d)) return rc;
  if (ctx && !ctx->fn.count(name))
    return fail(SABER_IU8_E_NOTLOADED, name + ": the accumulator taps live in the test-only object `iu8_taps`; add it with saber_iu8_load_plugin");
  // the taps read no scales; bind the accumulator buffer where a pointer is required
  return launch_gemm(ctx, d, a, (const float *)acc, w, (const float *)acc, acc, nullptr, nullptr, stream);
}

// ---------------------------------------------------------------------------- Hadamard-basis producers

// One workgroup a row, T = 256 threads for rows of up to 10,240 elements (5 groups of 8 a thread),
// 512 up to 20,480 (the reference's t256 / t512 pair, crates/saber-kernels/src/macaq_iu8.rs:864-875).
// Few rows (fewer than CUs) of 4,096 elements and more go 16 waves a row (`<stem>_hadi8_t1024`, no counterpart among the
// reference's symbols) where the workgroup's size does not enter the result -- every producer but add_rms, whose sum
// of squares is a tree over the workgroup and whose 16-wave form keeps the 256-thread order (6.4 -> 4.7 at 16 rows of 5,120): the same bytes, and on this card at 16 rows (graph replay, us) the attention
// gate 6.9 -> 4.8 (table form 7.1 -> 4.4), the GDN norm 7.2 -> 5.7, SiLU * up of 5,120 6.6 -> 4.7 and of 17,408 9.7 -> 9.0
// (table form 7.6 -> 6.2), the plain transform of 5,120 3.6 -> 3.1 (of 17,408 the 512-thread form is as fast: kept);
// from 512 rows on the narrow forms win.
static bool had_t1024(uint32_t rows, uint32_t width) { return rows <= HAD_T1024_ROWS && width >= HAD_T1024_WIDTH; }
static int had_desc(const char *op, const char *stem, uint32_t rows, uint32_t width, saber_iu8_desc *d, bool size_free = false) {
  if (rows == 0 || width == 0) return fail(SABER_IU8_E_RULE, fmt("%s: %u rows of %u has nothing to do", op, rows, width));
  if (width % 64 != 0 || width > 20480)
    return fail(SABER_IU8_E_RULE,
                fmt("%s: row width %u must be a multiple of 64 (whole A fragments, whole 32-blocks), at most 20480", op, width));
  const bool wide = size_free && had_t1024(rows, width);
  const uint32_t t = wide ? 1024 : width <= 10240 ? 256 : 512;
  const std::string name = wide ? fmt("%s_hadi8_t1024", stem) : fmt("%s_hadi8_t%u_tiled1", stem, t);
  const uint32_t grid[3] = {rows, 1, 1};
  if (int rc = saber_iu8_describe_raw(name.c_str(), "mxfp4_hadi8", grid, t, d)) return rc;
  snprintf(d->op, sizeof d->op, "%s", op);
  return 0;
}
static void set_f32(saber_iu8_desc *d, const char *name, float v) {
  for (uint32_t i = 0; i < d->n_args; ++i)
    if (!strcmp(d->args[i].name, name)) {
      d->args[i].kind = SABER_IU8_ARG_F32;
      d->args[i].fval = v;
    }
}

int saber_iu8_quant_had(saber_iu8_ctx *ctx, const void *x, void *q, float *scale, uint32_t m, uint32_t k,
                        const float *had_t, void *stream) {
  saber_iu8_desc d;
  if (int rc = had_desc("quant_had_i8", "quant", m, k, &d, k <= 10240)) return rc;
  set_i32(&d, "k", k);
  const saber_iu8_binding b[] = {{"x", (void *)x}, {"q", q}, {"scale", scale}, {"had_t", (void *)had_t}};
  return saber_iu8_launch(ctx, &d, b, 4, stream);
}

int saber_iu8_silu_mul_quant_had(saber_iu8_ctx *ctx, const void *gu, void *q, float *scale, uint32_t m, uint32_t n,
                                 const float *had_t, void *stream) {
  saber_iu8_desc d;
  if (int rc = had_desc("silu_mul_quant_had_i8", "silu_mul_quant", m, n, &d, true)) return rc;
  set_i32(&d, "n", n);
  const saber_iu8_binding b[] = {{"gu", (void *)gu}, {"q", q}, {"scale", scale}, {"had_t", (void *)had_t}};
  return saber_iu8_launch(ctx, &d, b, 4, stream);
}

int saber_iu8_silu_mul_quant_had_lut(saber_iu8_ctx *ctx, const void *gu, void *q, float *scale, uint32_t m, uint32_t n,
                                     const float *had_t, const uint16_t *silu_lut, void *stream) {
  if (!silu_lut || n < SABER_IU8_SILU_LUT_MIN_WIDTH) return saber_iu8_silu_mul_quant_had(ctx, gu, q, scale, m, n, had_t, stream);
  saber_iu8_desc d;
  if (int rc = had_desc("silu_mul_quant_had_i8", "silu_mul_quant", m, n, &d, true)) return rc;  // the shape checks, grid and block
  const std::string name = fmt("silu_mul_quant_hadi8_lut_t%u", d.block[0]);
  const uint32_t grid[3] = {m, 1, 1};
  if (int rc = saber_iu8_describe_raw(name.c_str(), "mxfp4_hadi8", grid, d.block[0], &d)) return rc;
  snprintf(d.op, sizeof d.op, "silu_mul_quant_had_i8");
  set_i32(&d, "n", n);
  const saber_iu8_binding b[] = {{"gu", (void *)gu}, {"q", q}, {"scale", scale}, {"had_t", (void *)had_t}, {"lut", (void *)silu_lut}};
  return saber_iu8_launch(ctx, &d, b, 5, stream);
}

int saber_iu8_add_rms_quant_had(saber_iu8_ctx *ctx, const void *y, const void *res, const void *w, void *q, float *scale,
                                void *res_out, uint32_t m, uint32_t k, float eps, const float *had_t, void *stream) {
  saber_iu8_desc d;
  // the 16-wave form carries the 256-thread form's sum order (a chain handed through LDS): one group a thread, K <= 8192
  if (int rc = had_desc("add_rms_quant_had_i8", "add_rms_quant", m, k, &d, k <= 8192)) return rc;
  set_i32(&d, "k", k);
  set_f32(&d, "eps", eps);
  const saber_iu8_binding b[] = {{"y", (void *)y}, {"res", (void *)res}, {"w", (void *)w}, {"q", q},
                                 {"scale", scale}, {"res_out", res_out}, {"had_t", (void *)had_t}};
  return saber_iu8_launch(ctx, &d, b, 7, stream);
}

// gdn_norm: rows of whole 128-element heads, one 256-thread workgroup a row (at most 10,240 wide).
int saber_iu8_gdn_norm_quant_had(saber_iu8_ctx *ctx, const void *x, const void *z, int64_t z_stride, const void *w, void *q,
                                 float *scale, uint32_t m, uint32_t n, float eps, const float *had_t, void *stream) {
  if (m == 0 || n == 0) return fail(SABER_IU8_E_RULE, fmt("gdn_norm_quant_had_i8: %u rows of %u has nothing to do", m, n));
  if (n % 128 != 0 || n > 10240)
    return fail(SABER_IU8_E_RULE, fmt("gdn_norm_quant_had_i8: row width %u must be whole 128-element heads, at most 10240", n));
  if (z_stride < (int64_t)n || z_stride % 8 != 0)
    return fail(SABER_IU8_E_RULE, fmt("gdn_norm_quant_had_i8: z stride %lld must cover the row width %u in whole 16-byte pieces", (long long)z_stride, n));
  saber_iu8_desc d;
  const uint32_t grid[3] = {m, 1, 1};
  const bool wide = had_t1024(m, n);  // a head's sum is its 16 lanes' whatever the workgroup's size
  if (int rc = saber_iu8_describe_raw(wide ? "gdn_norm_quant_hadi8_t1024" : "gdn_norm_quant_hadi8_t256_tiled1", "mxfp4_hadi8", grid, wide ? 1024 : 256, &d)) return rc;
  snprintf(d.op, sizeof d.op, "gdn_norm_quant_had_i8");
  set_i32(&d, "n", n);
  set_i32(&d, "zs", z_stride);
  set_f32(&d, "eps", eps);
  const saber_iu8_binding b[] = {{"x", (void *)x}, {"z", (void *)z}, {"w", (void *)w}, {"q", q}, {"scale", scale}, {"had_t", (void *)had_t}};
  return saber_iu8_launch(ctx, &d, b, 6, stream);
}

// attn_gate: the reference's t256 form holds rows of at most 6,144 elements (3 groups of 8 a thread,
// crates/saber-kernels/hip/attn_glue_hadi8.hip:33); heads of `hd` elements, a multiple of 8.
static int attn_gate_launch(saber_iu8_ctx *ctx, const void *core, const void *gate, void *q, float *scale, uint32_t m, uint32_t n,
                            uint32_t head_dim, uint32_t gate_stride, const float *had_t, const uint16_t *lut, void *stream) {
  if (m == 0 || n == 0) return fail(SABER_IU8_E_RULE, fmt("attn_gate_quant_had_i8: %u rows of %u has nothing to do", m, n));
  if (n % 64 != 0 || n > 6144)
    return fail(SABER_IU8_E_RULE, fmt("attn_gate_quant_had_i8: row width %u must be a multiple of 64, at most 6144", n));
  if (head_dim == 0 || head_dim % 8 != 0 || n % head_dim != 0)
    return fail(SABER_IU8_E_RULE, fmt("attn_gate_quant_had_i8: head width %u must be a multiple of 8 dividing %u", head_dim, n));
  if (gate_stride < 2 * n || gate_stride % 8 != 0)
    return fail(SABER_IU8_E_RULE, fmt("attn_gate_quant_had_i8: gate stride %u must cover the [q | gate] block of %u in whole 16-byte pieces", gate_stride, 2 * n));
  saber_iu8_desc d;
  const uint32_t grid[3] = {m, 1, 1};
  const bool wide = had_t1024(m, n);
  const char *name = wide ? (lut ? "attn_gate_quant_hadi8_lut_t1024" : "attn_gate_quant_hadi8_t1024")
                          : (lut ? "attn_gate_quant_hadi8_lut_t256" : "attn_gate_quant_hadi8_t256_tiled1");
  if (int rc = saber_iu8_describe_raw(name, "attn_glue_hadi8", grid, wide ? 1024 : 256, &d)) return rc;
  snprintf(d.op, sizeof d.op, "attn_gate_quant_had_i8");
  set_i32(&d, "n", n);
  set_i32(&d, "hd", head_dim);
  set_i32(&d, "gs", gate_stride);
  const saber_iu8_binding b[] = {{"core", (void *)core}, {"gate", (void *)gate}, {"q", q}, {"scale", scale}, {"had_t", (void *)had_t},
                                 {"lut", (void *)lut}};
  return saber_iu8_launch(ctx, &d, b, lut ? 6 : 5, stream);
}
int saber_iu8_attn_gate_quant_had(saber_iu8_ctx *ctx, const void *core, const void *gate, void *q, float *scale, uint32_t m,
                                  uint32_t n, uint32_t head_dim, uint32_t gate_stride, const float *had_t, void *stream) {
  return attn_gate_launch(ctx, core, gate, q, scale, m, n, head_dim, gate_stride, had_t, nullptr, stream);
}
int saber_iu8_attn_gate_quant_had_lut(saber_iu8_ctx *ctx, const void *core, const void *gate, void *q, float *scale, uint32_t m,
                                      uint32_t n, uint32_t head_dim, uint32_t gate_stride, const float *had_t,
                                      const uint16_t *sigmoid_lut, void *stream) {
  // (the 16-wave form spreads the copy of the table's middle over four times the threads: there it pays at any row count)
  const bool pays = n >= SABER_IU8_SILU_LUT_MIN_WIDTH && (m >= SABER_IU8_SIGMOID_LUT_MIN_ROWS || had_t1024(m, n));
  return attn_gate_launch(ctx, core, gate, q, scale, m, n, head_dim, gate_stride, had_t, pays ? sigmoid_lut : nullptr, stream);
}

// ---------------------------------------------------------------------------- routed experts

uint32_t saber_iu8_moe_rows_cap(uint32_t tokens, uint32_t topk, uint32_t experts) {
  const uint32_t r = tokens * topk;
  return r + 15u * std::min(r, experts);
}
uint32_t saber_iu8_moe_tiles_cap(uint32_t tokens, uint32_t topk, uint32_t experts, uint32_t tile_blocks) {
  const uint32_t r = tokens * topk;
  return std::min(r, experts) + r / (16u * std::max(tile_blocks, 1u)) + 1u;
}
uint32_t saber_iu8_moe_rows_cap_shared(uint32_t tokens, uint32_t topk, uint32_t experts) {
  return saber_iu8_moe_rows_cap(tokens, topk, experts) + (tokens + 15) / 16 * 16;
}
uint32_t saber_iu8_moe_tiles_cap_shared(uint32_t tokens, uint32_t topk, uint32_t experts, uint32_t tile_blocks) {
  const uint32_t g = std::max(tile_blocks, 1u);
  return saber_iu8_moe_tiles_cap(tokens, topk, experts, tile_blocks) + ((tokens + 15) / 16 + g - 1) / g;
}
// Rows a tile (x16). 16-row tiles on the streaming cell while routes are few (up to 7 routes an
// expert on average); above, the MFMA cells, whose sparse forms make a thinly filled tile cost about
// its weight traffic and which stream an expert's weights once instead of once a 16-row tile:
// 128-row tiles while an expert's routes on average do not fill one (the two-cell kernels, which run
// the thin tiles on a small cell), 256-row tiles (one tile an expert more often than not, on the
// dense GEMM's fastest shape) from 128 routes an expert. Speed data of this card, 128 experts, top-8,
// 4096 x 1536, us a layer at tile_blocks 1 / 8 / 16: T=32 255 / 309 / 328, T=64 296 / 335 / 347,
// T=80 318 / 340, T=128 363 / 347 / 362, T=256 730 / 293 / 298, T=512 1282 / 315 / 319,
// T=1024 2349 / 377 / 402, T=1280 - / 425 / 458, T=1536 - / 472 / 528, T=1792 - / 493 / 516,
// T=1920 - / 526 / 532, T=2048 - / 586 / 544, T=4096 - / 960 / 916.
uint32_t saber_iu8_moe_tile_blocks(uint32_t tokens, uint32_t topk, uint32_t experts) {
  const uint64_t routes = (uint64_t)tokens * topk;
  if (routes <= 7ull * experts) return 1u;
  return routes >= 128ull * experts ? 16u : 8u;
}

static int moe_check(const char *what, uint32_t tokens, uint32_t experts, uint32_t topk, const saber_iu8_moe_tables *t) {
  if (!t) return fail(SABER_IU8_E_ARG, std::string(what) + ": null tables");
  if (experts != 128 || topk != 8)
    return fail(SABER_IU8_E_RULE, fmt("%s: %u experts / top-%u; this object ships the 128-expert top-8 router", what, experts, topk));
  if (tokens == 0) return fail(SABER_IU8_E_RULE, std::string(what) + ": no tokens; an empty launch is a caller bug");
  return 0;
}

static int raw_desc(const char *kernel, uint32_t gx, uint32_t gy, uint32_t block, saber_iu8_desc *d) {
  const uint32_t grid[3] = {gx, gy, 1};
  return saber_iu8_describe_raw(kernel, "moe_iu8", grid, block, d);
}

// The router's launches. One routing workgroup (up to 128 tokens) lays out its tables itself. With more, the routing
// launch stops behind the workgroups' counts and ranks and a second launch of as many workgroups lays out the tables,
// every workgroup placing its own routes (moe_iu8_route_place_e128): the one-launch form's last arriver does that
// alone (4,096 tokens: 22 of its 38 us). `x` given: the tokens' quantisation rides in the routing launch.
static int moe_route_launches(saber_iu8_ctx *ctx, const void *logits, const void *x, void *q, float *scale, uint32_t tokens,
                              uint32_t experts, uint32_t k, uint32_t tile_blocks, const saber_iu8_moe_tables *t, void *stream) {
  const uint32_t nblk = (tokens + 127) / 128;
  const bool two = nblk > 1;
  // a row on 256, 512 or 1,024 threads by its length: 4, 2 or 1 rows a quantising workgroup (the kernel's own rule)
  const uint32_t groups = k / 16, rows_wg = groups <= 256 ? 4 : groups <= 512 ? 2 : 1;
  const bool rm = tile_blocks != 1;
  const std::string name = !x ? (two ? "moe_iu8_route_part_topk8_sort_e128" : "moe_iu8_route_topk8_sort_e128")
                              : std::string("moe_iu8_routeq_") + (rm ? "rm_" : "") + (two && rm ? "part_" : "") + "topk8_sort_e128";
  const bool part = name.find("_part_") != std::string::npos;
  auto launch = [&](const std::string &kernel, uint32_t gx, bool with_x, uint32_t block = 1024) {
    saber_iu8_desc d;
    if (int rc = raw_desc(kernel.c_str(), gx, 1, block, &d)) return rc;
    set_i32(&d, "t", tokens);
    set_i32(&d, "e_lo", 0);
    set_i32(&d, "e_loc", experts);
    set_i32(&d, "tile_blocks", tile_blocks);
    set_i32(&d, "with_shared", t->sgate ? 1 : 0);
    if (with_x) set_i32(&d, "k", k);
    const saber_iu8_binding b[] = {{"logits", (void *)logits},      {"topk_ids", t->topk_ids},   {"topk_w", t->topk_w},
                                   {"route_pos", t->route_pos},     {"row_tok", t->row_tok},     {"row_route", t->row_route},
                                   {"tile_expert", t->tile_expert}, {"tile_row0", t->tile_row0}, {"tile_rows", t->tile_rows},
                                   {"expert_cnt", t->expert_cnt},   {"meta", t->meta},           {"blk_cnt", t->blk_cnt},
                                   {"rank", t->rank},               {"arrive", t->arrive},       {"x", (void *)x},
                                   {"q", q},                        {"scale", scale}};
    return saber_iu8_launch(ctx, &d, b, with_x ? 17 : 14, stream);
  };
  if (part) {  // routing workgroups of 32 tokens on 256 threads, a quantising workgroup a token row
    if (int rc = launch(name, (tokens + 31) / 32 + (x ? tokens : 0), x != nullptr, 256)) return rc;
    return launch("moe_iu8_route_place_e128", nblk, false);
  }
  return launch(name, nblk + (x ? (tokens + rows_wg - 1) / rows_wg : 0), x != nullptr);
}

int saber_iu8_moe_route(saber_iu8_ctx *ctx, const void *logits, uint32_t tokens, uint32_t experts, uint32_t topk,
                        uint32_t tile_blocks, const saber_iu8_moe_tables *t, void *stream) {
  if (int rc = moe_check("moe_route", tokens, experts, topk, t)) return rc;
  if (tile_blocks == 0) return fail(SABER_IU8_E_RULE, "moe_route: tile_blocks 0");
  return moe_route_launches(ctx, logits, nullptr, nullptr, nullptr, tokens, experts, 0, tile_blocks, t, stream);
}

int saber_iu8_moe_route_quant(saber_iu8_ctx *ctx, const void *logits, const void *x, void *q, float *scale, uint32_t tokens,
                              uint32_t experts, uint32_t topk, uint32_t k, uint32_t tile_blocks,
                              const saber_iu8_moe_tables *t, void *stream) {
  if (int rc = moe_check("moe_route_quant", tokens, experts, topk, t)) return rc;
  if (tile_blocks == 0) return fail(SABER_IU8_E_RULE, "moe_route_quant: tile_blocks 0");
  if (!x || k == 0 || k % 128 != 0 || k > 16384)
    return fail(SABER_IU8_E_RULE, fmt("moe_route_quant: K=%u must be a multiple of 128 (the slab) up to 16384 (a 16-element group a thread)", k));
  return moe_route_launches(ctx, logits, x, q, scale, tokens, experts, k, tile_blocks, t, stream);
}

int saber_iu8_moe_grouped(saber_iu8_ctx *ctx, const void *a, const float *as, const void *xptr, void *c, uint32_t n,
                          uint32_t k, int gather, uint32_t tokens, uint32_t experts, uint32_t topk, uint32_t tile_blocks,
                          const saber_iu8_moe_tables *t, void *stream) {
  if (int rc = moe_check("moe_grouped", tokens, experts, topk, t)) return rc;
  if (n == 0 || k == 0 || n % 16 != 0 || k % 128 != 0)
    return fail(SABER_IU8_E_RULE, fmt("moe_grouped: N=%u must be a multiple of 16 (whole fragments) and K=%u of 128 (the slab)", n, k));
  if (tile_blocks != 1 && tile_blocks != 8 && tile_blocks != 16)
    return fail(SABER_IU8_E_RULE, fmt("moe_grouped: tile_blocks %u; the cells are 1 (16-row), 8 (128-row) and 16 (256-row)", tile_blocks));
  const bool dec = tile_blocks == 1;
  // the MFMA cells address A with 32-bit byte offsets: token-major codes (gather 1, 2) or rows_cap rows
  if (!dec) {
    const uint64_t a_rows = gather ? (uint64_t)(tokens + 15) / 16 * 16
                                   : t->sgate ? saber_iu8_moe_rows_cap_shared(tokens, topk, experts) : saber_iu8_moe_rows_cap(tokens, topk, experts);
    if (a_rows * k > 0xFFFFFFFFull || (uint64_t)n * k / 2 > 0xFFFFFFFFull)
      return fail(SABER_IU8_E_RULE, fmt("moe_grouped: %llu rows of K=%u (or an expert's %u x %u weights) pass 4 GiB, more than the tile GEMM addresses",
                                        (unsigned long long)a_rows, k, n, k));
  }
  if (gather < 0 || gather > 2 || (gather == 2 && dec))
    return fail(SABER_IU8_E_RULE, fmt("moe_grouped: gather %d; 0 in place, 1 from A fragments, 2 from row-major codes (MFMA cells only)", gather));
  // The streaming cell. Short K (an expert's down projection) takes the two-k-wave form with 64 columns a
  // workgroup (K = 1536: 64 vs 72 us at 48 tokens, 75 vs 86 at 112). Else a tile's rows are staged in LDS
  // while they fit (pow2(rows) * K <= 20 KiB, 4 rows at K = 4096); where a launch's tiles mostly would
  // not (more than two routes an expert on average at that K), the form that streams the rows beside
  // the weights is the faster one.
  const bool short_k = k <= 2048;
  uint32_t cap = 1;
  while ((uint64_t)cap * 2 * k <= 20 * 1024 && cap < 16) cap *= 2;
  const bool stream_rows = !short_k && (uint64_t)tokens * topk * 2 > (uint64_t)cap * experts;
  const std::string name = fmt("moe_iu8_grouped_w4_%s_g%d", dec ? (short_k ? "deck" : stream_rows ? "deca" : "dec") : tile_blocks == 8 ? "pf" : "pf16", gather);
  const uint32_t bn = dec ? (short_k ? 64 : 32) : 256, block = 512;
  saber_iu8_desc d;
  // the streaming cell: a workgroup a (column block, tile), static worst-case grid; the MFMA cell:
  // persistent, one workgroup a CU over the live work items
  const uint32_t tiles_cap = t->sgate ? saber_iu8_moe_tiles_cap_shared(tokens, topk, experts, tile_blocks)
                                      : saber_iu8_moe_tiles_cap(tokens, topk, experts, tile_blocks);
  const uint32_t gx = (n + bn - 1) / bn;
  const uint64_t items = (uint64_t)gx * tiles_cap;
  if (int rc = dec ? raw_desc(name.c_str(), gx, tiles_cap, block, &d)
                   : raw_desc(name.c_str(), (uint32_t)(items < CU_COUNT ? items : CU_COUNT), 1, block, &d))
    return rc;
  set_i32(&d, "n", n);
  set_i32(&d, "k", k);
  set_i32(&d, "pmax", 0);
  set_null(&d, "p");
  set_null(&d, "cnt");
  const saber_iu8_binding b[] = {{"a", (void *)a},           {"xptr", (void *)xptr},         {"tile_expert", t->tile_expert},
                                 {"tile_row0", t->tile_row0}, {"tile_rows", t->tile_rows},   {"row_tok", t->row_tok},
                                 {"meta", t->meta},           {"as", (void *)as},            {"c", c}};
  return saber_iu8_launch(ctx, &d, b, sizeof b / sizeof b[0], stream);
}

// The back half with few tokens: 16 rows of `inter` codes must fit the second launch's 24 KiB of staged rows.
int saber_iu8_moe_back_holds(uint32_t tile_blocks, uint32_t inter) {
  return tile_blocks == 1 && inter != 0 && inter % 128 == 0 && (uint64_t)16 * inter <= 24 * 1024;
}

// ... and pays wherever it holds. Measured on the 128-expert top-8 layer (hidden 4096, inter 1536), layer in us, three
// launches against two: 8 tokens 107.3 / 100.0, 16 tokens 145.2 / 139.4, 32 tokens 190.5 / 183.1, 64 tokens 242.0 / 226.7,
// 112 tokens 296.5 / 271.9 (gate+up with one tile of p a wave up to 1.5 routes an expert, two above).
int saber_iu8_moe_back_pays(uint32_t tokens, uint32_t topk, uint32_t experts, uint32_t tile_blocks, uint32_t inter) {
  (void)tokens, (void)topk, (void)experts;
  return saber_iu8_moe_back_holds(tile_blocks, inter);
}

static int moe_back_launch(saber_iu8_ctx *ctx, const std::string &name, uint32_t gx, const void *a,
                           const float *as, const void *xptr, void *c, uint32_t n, uint32_t k, uint32_t tokens,
                           uint32_t experts, uint32_t topk, const saber_iu8_moe_tables *t, void *stream) {
  const uint32_t tiles_cap = t->sgate ? saber_iu8_moe_tiles_cap_shared(tokens, topk, experts, 1) : saber_iu8_moe_tiles_cap(tokens, topk, experts, 1);
  saber_iu8_desc d;
  if (int rc = raw_desc(name.c_str(), gx, tiles_cap, 512, &d)) return rc;
  set_i32(&d, "n", n);
  set_i32(&d, "k", k);
  set_i32(&d, "pmax", 0);
  set_null(&d, "p");
  set_null(&d, "cnt");
  if (!as) set_null(&d, "as");
  const saber_iu8_binding b[] = {{"a", (void *)a},           {"xptr", (void *)xptr},         {"tile_expert", t->tile_expert},
                                 {"tile_row0", t->tile_row0}, {"tile_rows", t->tile_rows},   {"row_tok", t->row_tok},
                                 {"meta", t->meta},           {"c", c},                      {"as", (void *)as}};
  return saber_iu8_launch(ctx, &d, b, as ? 9 : 8, stream);  // without scales the last binding is left out
}

int saber_iu8_moe_gate_up_act(saber_iu8_ctx *ctx, const void *a, const float *as, const void *xptr, void *p, uint32_t inter,
                              uint32_t k, uint32_t tokens, uint32_t experts, uint32_t topk, uint32_t tile_blocks,
                              const saber_iu8_moe_tables *t, void *stream) {
  if (int rc = moe_check("moe_gate_up_act", tokens, experts, topk, t)) return rc;
  if (!saber_iu8_moe_back_holds(tile_blocks, inter) || k == 0 || k % 128 != 0)
    return fail(SABER_IU8_E_RULE, fmt("moe_gate_up_act: tile_blocks %u, inter %u, K=%u; the fused back half is the 16-row cell's "
                                      "(tile_blocks 1), inter a multiple of 128 up to 1536, K a multiple of 128", tile_blocks, inter, k));
  // one tile of p a wave up to 1.5 routes an expert, two above (the rows streamed beside the weights feed twice the columns)
  const bool wide = (uint64_t)tokens * topk * 2 > (uint64_t)experts * 3;
  return moe_back_launch(ctx, wide ? "moe_iu8_grouped_w4_decpb_g1" : "moe_iu8_grouped_w4_decpa_g1", (inter + (wide ? 31 : 15)) / (wide ? 32 : 16), a,
                         as, xptr, p, 2 * inter, k, tokens, experts, topk, t, stream);
}

int saber_iu8_moe_down_rows(saber_iu8_ctx *ctx, const void *p, const void *xptr, void *y, uint32_t n, uint32_t inter,
                            uint32_t tokens, uint32_t experts, uint32_t topk, uint32_t tile_blocks,
                            const saber_iu8_moe_tables *t, void *stream) {
  if (int rc = moe_check("moe_down_rows", tokens, experts, topk, t)) return rc;
  if (!saber_iu8_moe_back_holds(tile_blocks, inter) || n == 0 || n % 16 != 0)
    return fail(SABER_IU8_E_RULE, fmt("moe_down_rows: tile_blocks %u, inter %u, N=%u; the fused back half is the 16-row cell's "
                                      "(tile_blocks 1), inter a multiple of 128 up to 1536, N a multiple of 16", tile_blocks, inter, n));
  return moe_back_launch(ctx, "moe_iu8_grouped_w4_deckq_g0", (n + 63) / 64, p, nullptr, xptr, y, n, inter, tokens,
                         experts, topk, t, stream);
}

int saber_iu8_moe_quant_rows(saber_iu8_ctx *ctx, const void *x, void *q, float *scale, uint32_t k, uint32_t rows_cap,
                             const saber_iu8_moe_tables *t, void *stream) {
  if (!t) return fail(SABER_IU8_E_ARG, "moe_quant_rows: null tables");
  saber_iu8_desc d;
  if (int rc = resolve_quant_rows(rows_cap, k, &d)) return rc;
  const saber_iu8_binding b[] = {{"x", (void *)x}, {"q", q}, {"scale", scale}, {"row_tok", t->row_tok}, {"meta", t->meta}};
  return saber_iu8_launch(ctx, &d, b, 5, stream);
}

int saber_iu8_moe_silu_mul_quant(saber_iu8_ctx *ctx, const void *gu, void *q, float *scale, uint32_t n, uint32_t rows_cap,
                                 const saber_iu8_moe_tables *t, void *stream) {
  if (!t) return fail(SABER_IU8_E_ARG, "moe_silu_mul_quant: null tables");
  saber_iu8_desc d;
  // From a few thousand rows the table form (memory-bound) overtakes the computed one (bound by the
  // exp and divide of every element); below, copying the table into LDS costs more than it saves.
  if (t->silu_lut && rows_cap >= 4096 && n % 16 == 0 && n <= 4096) {
    const uint32_t tiles = (rows_cap + 15) / 16;
    const uint32_t grid[3] = {tiles < CU_COUNT ? tiles : CU_COUNT, 1, 1};
    if (int rc = saber_iu8_describe_raw("macaq_i8_silu_mul_quant_lut_w64", "macaq_i8q", grid, 1024, &d)) return rc;
    set_i32(&d, "n", n);
    const saber_iu8_binding b[] = {{"gu", (void *)gu}, {"q", q}, {"scale", scale}, {"row_tok", t->row_tok}, {"meta", t->meta},
                                   {"lut", (void *)t->silu_lut}};
    return saber_iu8_launch(ctx, &d, b, 6, stream);
  }
  if (int rc = resolve_silu_mul_quant(rows_cap, n, &d)) return rc;
  set_buffer(&d, "row_tok");
  set_buffer(&d, "meta");
  const saber_iu8_binding b[] = {{"gu", (void *)gu}, {"q", q}, {"scale", scale}, {"row_tok", t->row_tok}, {"meta", t->meta}};
  return saber_iu8_launch(ctx, &d, b, 5, stream);
}

int saber_iu8_moe_combine(saber_iu8_ctx *ctx, const void *y, const saber_iu8_moe_tables *t, void *out, uint32_t tokens,
                          uint32_t topk, uint32_t h, void *stream) {
  if (!t) return fail(SABER_IU8_E_ARG, "moe_combine: null tables");
  if (topk != 8) return fail(SABER_IU8_E_RULE, fmt("moe_combine: top-%u; this object ships top-8", topk));
  if (tokens == 0 || h == 0 || h % 8 != 0) return fail(SABER_IU8_E_RULE, fmt("moe_combine: %u tokens of width %u (a multiple of 8)", tokens, h));
  saber_iu8_desc d;
  if (int rc = raw_desc("moe_iu8_combine_bf16", tokens, 1, 256, &d)) return rc;
  set_i32(&d, "h", h);
  if (!t->sgate) set_null(&d, "sgate");  // no shared expert: the kernel tests the pointer
  const saber_iu8_binding b[] = {{"y", (void *)y},   {"topk_w", t->topk_w}, {"route_pos", t->route_pos},
                                 {"meta", t->meta}, {"out", out},          {"sgate", (void *)t->sgate}};
  return saber_iu8_launch(ctx, &d, b, t->sgate ? 6 : 5, stream);
}

static int table_launch(saber_iu8_ctx *ctx, const char *kernel, const char *plugin, void *out, void *stream) {
  saber_iu8_desc d;
  const uint32_t grid[3] = {256, 1, 1};
  if (int rc = saber_iu8_describe_raw(kernel, plugin, grid, 256, &d)) return rc;
  const saber_iu8_binding b[] = {{"out", out}};
  return saber_iu8_launch(ctx, &d, b, 1, stream);
}
int saber_iu8_sigmoid_table(saber_iu8_ctx *ctx, void *out, void *stream) {
  return table_launch(ctx, "attn_gate_sigmoid_bf16_table", "attn_glue_hadi8", out, stream);
}

int saber_iu8_silu_table(saber_iu8_ctx *ctx, void *out, void *stream) {
  saber_iu8_desc d;
  const uint32_t grid[3] = {256, 1, 1};
  if (int rc = saber_iu8_describe_raw("macaq_silu_bf16_table", "macaq_i8q", grid, 256, &d)) return rc;
  const saber_iu8_binding b[] = {{"out", out}};
  return saber_iu8_launch(ctx, &d, b, 1, stream);
}

}  // extern "C"
