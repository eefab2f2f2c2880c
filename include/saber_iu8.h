/* saber_iu8.h -- C ABI of the MI355X (gfx950) W4A8-iu8 decoder-linear path.
 *
 * The reference (GGZ14/saber-engine) crosses into device code through a data-only plugin
 * boundary: a code object (`.hsaco`) plus a `.manifest.toml`, loaded and launched by its Rust
 * host crates through a dlopen'd libamdhip64 (include/saber_abi.h:24-30 of the reference).
 * This library is the C/C++ counterpart of those host crates for this one path, so that a host
 * without them (or a binding in another language) can resolve, validate, load and launch the
 * gfx950 code objects exactly as `saber-kernels` + `saber-exec` + `saber-hip` would.
 * Each entry point names the reference interface it stands in for (paths relative to the
 * reference tree).
 *
 * Conventions: plain pointers and sizes only. Every function returns 0 on success and a
 * negative SABER_IU8_E_* code on failure; saber_iu8_last_error() returns the message of the
 * calling thread's last failure. Device pointers are raw HIP device addresses owned by the
 * caller; `stream` is a hipStream_t passed as void* (NULL = the null stream). All HIP calls of
 * one context must come from one OS thread (crates/saber-hip/src/lib.rs:11-16).
 */
#ifndef SABER_IU8_H
#define SABER_IU8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SABER_IU8_ABI_VERSION 1

/* error codes */
#define SABER_IU8_OK 0
#define SABER_IU8_E_RULE (-1)      /* a launch rule refused the shape (Error::Rule, macaq_iu8.rs:288-303) */
#define SABER_IU8_E_PARSE (-2)     /* manifest / code object could not be parsed */
#define SABER_IU8_E_VALIDATE (-3)  /* manifest does not describe the code object (manifest.rs:228-324) */
#define SABER_IU8_E_HIP (-4)       /* a HIP call failed (message carries the status) */
#define SABER_IU8_E_ARG (-5)       /* a null / missing / undersized argument */
#define SABER_IU8_E_IO (-6)
#define SABER_IU8_E_NOTLOADED (-7) /* kernel or plugin not in the loaded set */

const char *saber_iu8_last_error(void);
int saber_iu8_abi_version(void);

/* ------------------------------------------------------------------ weight kinds, layouts */

/* WKind (crates/saber-kernels/src/macaq_iu8.rs:64-72). */
#define SABER_IU8_W4 0 /* per-row int4 [-8,7]   -> op "gemm_i4a8" */
#define SABER_IU8_W8 1 /* per-row int8 [-127,127] -> op "gemm_i8a8" */

/* gfx950 device-final layout ids. The reference's pack layouts 17/18 are gfx12 WMMA fragment
 * orders (crates/saber-mem/src/pack/layout.rs:99-104); a new order is a new id
 * (include/saber_abi.h:637-643 of the reference). */
#define SABER_IU8_LAYOUT_I4_ROW_FRAG64 33
#define SABER_IU8_LAYOUT_I8_ROW_FRAG64 34
#define SABER_IU8_LAYOUT_A_TILED_I8_64 35

/* Bytes of the A edge for m rows (padded to 16) of k int8 codes (Layout::ATiledI8,
 * crates/saber-model/src/graph.rs:445-448: same size, gfx950 byte order). */
size_t saber_iu8_a_bytes(uint32_t m, uint32_t k);
/* Byte offset of activation (m,k) in the gfx950 A order / of weight byte (n,k) in the W8 order. */
uint64_t saber_iu8_a_offset(uint32_t m, uint32_t k, uint32_t K);
/* Byte offset of weight (n,k) in the gfx950 W4 order; *high = 1 when it is the high nibble. */
uint64_t saber_iu8_w4_offset(uint32_t n, uint32_t k, uint32_t K, uint32_t *high);

/* Offline repack, host memory to host memory. Canonical forms: W4 row-major [N][K/2], low nibble
 * = even k (the export form, crates/saber-model/src/graph.rs:2591-2592); W8 and A row-major int8.
 * N % 16 == 0 and K % 128 == 0 or SABER_IU8_E_RULE. `a` rows are padded to 16 with zeros. */
int saber_iu8_repack_w4(const uint8_t *canonical, uint32_t n, uint32_t k, uint8_t *frag);
int saber_iu8_repack_w8(const int8_t *rowmajor, uint32_t n, uint32_t k, uint8_t *frag);
int saber_iu8_repack_a(const int8_t *rowmajor, uint32_t m, uint32_t k, uint8_t *frag);
int saber_iu8_unpack_a(const uint8_t *frag, uint32_t m, uint32_t k, int8_t *rowmajor);
/* The reference's gfx12 orders (layouts 17/18 and its A-tiled order) to the gfx950 orders, so a
 * pack written for the reference can be re-ordered without going back to the export. */
int saber_iu8_repack_w4_from_gfx12(const uint8_t *frag12, uint32_t n, uint32_t k, uint8_t *frag);
int saber_iu8_repack_w8_from_gfx12(const uint8_t *frag12, uint32_t n, uint32_t k, uint8_t *frag);

/* ------------------------------------------------------------------ launch descriptors */

/* ArgValue (crates/saber-kernels/src/rules.rs): what the launcher writes into a kernarg slot. */
#define SABER_IU8_ARG_BUFFER 0      /* device pointer of the named buffer */
#define SABER_IU8_ARG_NULL_BUFFER 1 /* a named buffer passed as NULL (workspaces at ks == 1) */
#define SABER_IU8_ARG_I32 2
#define SABER_IU8_ARG_F32 3
#define SABER_IU8_ARG_I64 4 /* an 8-byte by-value integer (a row stride in elements) */

typedef struct {
  char name[24];
  uint32_t offset, size; /* natural alignment (abi.rs:111-130) */
  uint32_t kind;         /* SABER_IU8_ARG_* */
  int64_t ival;
  float fval;
} saber_iu8_slot;

/* WorkspaceKind (crates/saber-kernels/src/rules.rs:473-482; include/saber_abi.h:163-174). */
#define SABER_IU8_WS_SCRATCH 0    /* undefined at entry, written before read, aliasable */
#define SABER_IU8_WS_PERSISTENT 1 /* zeroed once at allocation, left zero by the kernel */

typedef struct {
  char name[24];
  uint32_t kind;
  uint64_t bytes;
  uint32_t zero_once;
} saber_iu8_workspace;

/* LaunchDescriptor (crates/saber-kernels/src/rules.rs:838-853). */
typedef struct {
  char op[24];
  char plugin[24];
  char kernel[64];
  uint32_t grid[3];  /* in workgroups */
  uint32_t block[3];
  uint32_t shared_bytes;  /* always 0: LDS is static */
  uint32_t kernarg_bytes; /* explicit arguments only */
  uint32_t n_args;
  saber_iu8_slot args[24];
  uint32_t n_workspaces;
  saber_iu8_workspace workspaces[4];
  uint32_t n_launches; /* 1: split-K reduce is fused */
  uint32_t ks;         /* grid-level split count (decode), 1 otherwise */
} saber_iu8_desc;

/* macaq_iu8::resolve(WKind, m, n, k) -> LaunchDescriptor (macaq_iu8.rs:425-427) under the gfx950
 * launch law. Refuses (SABER_IU8_E_RULE) an empty launch, N % 16 != 0, K % 128 != 0. */
int saber_iu8_resolve(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out);
/* The same descriptor for an explicitly named kernel of the object and split count (the
 * autotuner's and the parity tests' entry: every variant of one regime gives the same bytes). */
int saber_iu8_describe(const char *kernel, uint32_t m, uint32_t n, uint32_t k, uint32_t ks, saber_iu8_desc *out);
/* A name of the reference's symbol set that these objects do not carry (its gfx1201 tile shapes:
 * macaq_iu8f_dec_*_tm{5..8}, macaq_iu8f_pf_*_bm{128,64}, macaq_iu8f_pf_*_t..., macaq_iu8.rs:520-546)
 * is taken by saber_iu8_describe as a request for the op at that shape and answered with the cell
 * the gfx950 law picks; the all-reduce forms (macaq_iu8f_arnq_*) are refused by name.
 *
 * LAUNCH LAW. The ten names of the reference's `macaq_iu8` object and the pair names are kept, with
 * their kernarg bytes, but NOT the reference's grid/block law or operand byte order: the gfx950
 * kernels are 256-, 512- or 1024-thread workgroups, mostly persistent, over the layouts 33/34/35.
 * A host must take grid and block from saber_iu8_resolve / _describe or from the band table
 * (saber_iu8_band_toml, committed as prebuilt/gfx950/macaq_iu8.band.toml); saber_iu8_launch refuses
 * a descriptor whose block is not the kernel's max_flat_workgroup_size. */

/* The launch law as data (TOML text, NUL-terminated): the cells' geometry, the (op, n, k, rows) ->
 * kernel bands over the 27B-class linears for M = 1..8192, the reference's symbol set and what
 * answers each name, the routed layer's tile thresholds, the pair's block order. The gfx950
 * counterpart of the reference's band tables (macaq_iu8.rs:150-212) for a host that cannot link
 * this library. *need (optional) receives the bytes required; buf may be NULL to ask for it. */
int saber_iu8_band_toml(char *buf, size_t cap, size_t *need);

/* The target as the planner's DeviceProfile (crates/saber-plan/src/device.rs:168-193; the reference's
 * gfx1201 instance: device.rs:208-258) as TOML text in that struct's field names and serde shape:
 * CU count, LDS, wave sizes, capability bits, the matrix shapes, Infinity Cache and VRAM sizes, and
 * the bandwidths with their provenance (DRAM measured on this card; PCIe and xGMI nominal: never
 * valid for sizing, as the reference says of such numbers). Committed as
 * prebuilt/gfx950/device_profile.toml; same calling convention as saber_iu8_band_toml. */
int saber_iu8_device_profile_toml(char *buf, size_t cap, size_t *need);

/* The activation producer's descriptor (i8_twin's role, macaq_iu8.rs:881-916): bf16 [m,k] rows
 * -> int8 A edge + f32 scales. */
int saber_iu8_resolve_quant(uint32_t m, uint32_t k, saber_iu8_desc *out);
/* SiLU(gate) * up + requant over rows of [gate(n) | up(n)] (abi.rs:315-320, 344-351). */
int saber_iu8_resolve_silu_mul_quant(uint32_t rows, uint32_t n, saber_iu8_desc *out);

/* A descriptor for any kernel of the loaded objects with an explicit grid (in workgroups) and
 * block: slots come from the kernel's signature, scalars are then set by name. The replay
 * harness's form (crates/saber-kernels/hip/harness/run_hsaco.cpp:1-15: "launches exactly what the
 * descriptor says"); used for the probe kernels and by sweeps. */
int saber_iu8_describe_raw(const char *kernel, const char *plugin, const uint32_t grid[3], uint32_t block,
                           saber_iu8_desc *out);
int saber_iu8_desc_set_i32(saber_iu8_desc *desc, const char *name, int64_t value);

/* abi::signature_for + abi::pack (abi.rs:111-130, 3495): fills names/offsets/sizes of the
 * explicit arguments of `kernel`; returns the explicit kernarg size in *bytes. */
int saber_iu8_signature(const char *kernel, saber_iu8_slot *slots, uint32_t cap, uint32_t *n_slots, uint32_t *bytes);

/* A buffer binding: name -> device pointer. */
typedef struct {
  const char *name;
  void *ptr;
} saber_iu8_binding;

/* pack_kernarg (crates/saber-exec/src/launch.rs:123): the zero-filled kernarg image of `desc`
 * with 8-byte device pointers / i32 / f32 at their declared offsets. Pure host. */
int saber_iu8_pack_kernarg(const saber_iu8_desc *desc, const saber_iu8_binding *bufs, uint32_t n_bufs, uint8_t *image,
                           uint32_t cap, uint32_t *bytes);

/* ------------------------------------------------------------------ manifests and code objects */

/* saber-kbuild's manifest step (crates/saber-kernels/src/bin/saber-kbuild.rs:234-251,
 * manifest.rs:136-226): reads the code object at `hsaco_path` (clang offload bundle or bare ELF)
 * and writes `<plugin>.manifest.toml` (schema 1) to `out_path`. build_hash = sha256(preprocessed
 * source ++ flags) is computed by the caller's build step and passed in. */
int saber_iu8_manifest_write(const char *hsaco_path, const char *plugin, const char *arch, const char *source,
                             const char *source_sha256, const char *flags, const char *build_hash, const char *out_path);

/* The loader's three validations (crates/saber-exec/src/loader.rs:249-290): kernarg layout against
 * the declared signature, one wave size per plugin, manifest against code object (sha256, target,
 * kernarg size/align, LDS, registers, symbol, per-argument offset/size/value_kind). */
#define SABER_IU8_REFUSED_KERNARG 1
#define SABER_IU8_REFUSED_WAVE 2
#define SABER_IU8_REFUSED_METADATA 3
/* Returns 0 when the pair loads, SABER_IU8_E_VALIDATE when refused (*refusal names the counter
 * that moves), SABER_IU8_E_PARSE / _IO when unreadable. */
int saber_iu8_manifest_validate(const char *manifest_path, const char *arch, int *refusal);

/* sha256 of a file, lowercase hex into out[65]. */
int saber_iu8_sha256_file(const char *path, char *out65);

/* ------------------------------------------------------------------ contexts, loading, launching */

typedef struct saber_iu8_ctx saber_iu8_ctx;

typedef struct {
  uint32_t plugins_loaded, kernels_loaded;
  uint32_t refused_kernarg, refused_wave, refused_metadata; /* loader.rs:249-270 */
  uint32_t launches;
} saber_iu8_counters;

/* PluginSet::load_dir (crates/saber-exec/src/loader.rs:318-396): validates every
 * `*.manifest.toml` under `prebuilt_dir` (the gfx950 directory) and loads the code objects that
 * pass with hipModuleLoadData on `device`. A refused plugin is skipped and counted, as in the
 * reference; no plugin at all is SABER_IU8_E_NOTLOADED. */
int saber_iu8_open(const char *prebuilt_dir, int device, saber_iu8_ctx **out);
/* PluginSet's single-manifest path (crates/saber-exec/src/loader.rs:249-290): validates one
 * `<plugin>.manifest.toml` + code object outside the plugin directory and adds its kernels to the
 * context; a refusal moves the counter it names. The parity suite adds its test-only object
 * (`taps/iu8_taps.manifest.toml`: accumulator and table taps) this way. */
int saber_iu8_load_plugin(saber_iu8_ctx *ctx, const char *manifest_path);
void saber_iu8_close(saber_iu8_ctx *ctx);
int saber_iu8_get_counters(const saber_iu8_ctx *ctx, saber_iu8_counters *out);
/* 1 if `kernel` was loaded. */
int saber_iu8_has_kernel(const saber_iu8_ctx *ctx, const char *kernel);

/* Launcher::launch_op (crates/saber-exec/src/launch.rs:590-660): packs the kernarg image and
 * calls hipModuleLaunchKernel(f, grid, block, 0, stream, NULL, extra) once. Buffers the
 * descriptor names must all be bound (workspaces included when ks > 1). Asynchronous, capture-
 * legal: no allocation, no synchronisation. */
int saber_iu8_launch(saber_iu8_ctx *ctx, const saber_iu8_desc *desc, const saber_iu8_binding *bufs, uint32_t n_bufs,
                     void *stream);

/* ------------------------------------------------------------------ operators (resolve + launch) */

/* Per-token int8 quantisation: x bf16 [m,k] -> q (A edge, saber_iu8_a_bytes) + scale f32 [m]. */
int saber_iu8_quant(saber_iu8_ctx *ctx, const void *x_bf16, void *q, float *scale, uint32_t m, uint32_t k, void *stream);

/* The same law with the codes row-major, q[row * k + col] (m * k bytes): the operand the grouped GEMM
 * of a routed layer gathers whole token rows from (gather 2), as the reference's grouped GEMM does
 * (crates/saber-kernels/hip/moe_grouped.hip:67-74). */
int saber_iu8_quant_rowmajor(saber_iu8_ctx *ctx, const void *x_bf16, void *q, float *scale, uint32_t m, uint32_t k,
                             void *stream);

/* The Hadamard-basis producers in front of a MACaQ-W4A8 GEMM (crates/saber-kernels/hip/mxfp4_hadi8.hip,
 * hip/macaq_had.h): the producer's bf16-rounded values times `had_t` (f32 [width]), a 32-point
 * Hadamard transform per 32-block, times 1/sqrt(32), then the per-token int8 law; codes in the A edge
 * order. Row widths: multiples of 64, at most 20,480.
 *   quant_had           x bf16 [m,k]                                 (the transform + the law alone)
 *   silu_mul_quant_had  gu bf16 [m, 2n] (gate | up) -> bf16(bf16(silu(gate)) * up)
 *   add_rms_quant_had   y, res bf16 [m,k], w bf16 [k]: v = y + res (stored to res_out as bf16),
 *                       bf16(v * inv * (w + 1)) with inv = 1/sqrt(mean(v^2) + eps)
 *   gdn_norm_quant_had  x bf16 [m,n] of 128-element heads, z bf16 rows `z_stride` elements apart,
 *                       w bf16 [128]: bf16(((x * inv_head) * w) * silu(z)), silu in f32, inv_head =
 *                       1/sqrt(mean_head(x^2) + eps); n a multiple of 128, at most 10,240
 *                       (hip/mxfp4_hadi8.hip:148-186, symbol gdn_norm_quant_hadi8_t256_tiled1)
 *   attn_gate_quant_had core bf16 [m,n]; gate = the projection's [q | gate] block, rows `gate_stride`
 *                       elements apart, head h's gate at h*2*head_dim + head_dim:
 *                       bf16(core * bf16(sigmoid(gate))); n at most 6,144
 *                       (hip/attn_glue_hadi8.hip:23-79, symbol attn_gate_quant_hadi8_t256_tiled1)
 * The square-root reciprocal is IEEE here where the reference calls the device's approximate rsqrtf.
 * Up to 256 rows of 4,096 elements and more launch a 1,024-thread form of every producer (kernels
 * `<stem>_hadi8_t1024`, `attn_gate_quant_hadi8[_lut]_t1024`; no counterpart among the reference's symbols): the
 * same bytes -- add_rms, whose sum of squares is a tree over the workgroup, keeps the 256-thread form's order there
 * (rows of up to 8,192) -- and 15-40 % less time while the rows are fewer than the compute units. */
int saber_iu8_quant_had(saber_iu8_ctx *ctx, const void *x_bf16, void *q, float *scale, uint32_t m, uint32_t k,
                        const float *had_t, void *stream);
int saber_iu8_silu_mul_quant_had(saber_iu8_ctx *ctx, const void *gu_bf16, void *q, float *scale, uint32_t m, uint32_t n,
                                 const float *had_t, void *stream);
/* saber_iu8_silu_mul_quant_had with a table of the bf16 silu at hand (`silu_lut`: u16 [65536] on the device
 * as saber_iu8_silu_table wrote it, a 128 KiB persistent workspace of the caller, filled once): for rows of
 * SABER_IU8_SILU_LUT_MIN_WIDTH elements and more the launch reads bf16(silu(gate)) from the table's middle,
 * which every workgroup copies into LDS (kernels silu_mul_quant_hadi8_lut_t{256,512}; the computed form
 * spends more than half of its arithmetic on the exp and the divide and is bound by it); narrower rows, or a
 * null table, are saber_iu8_silu_mul_quant_had. Same bytes either way: the table is the computed form's own
 * output. No counterpart among the reference's operators: its producer computes
 * (crates/saber-kernels/hip/mxfp4_hadi8.hip:117-146). */
#define SABER_IU8_SILU_LUT_MIN_WIDTH 2048u
int saber_iu8_silu_mul_quant_had_lut(saber_iu8_ctx *ctx, const void *gu_bf16, void *q, float *scale, uint32_t m, uint32_t n,
                                     const float *had_t, const uint16_t *silu_lut, void *stream);
/* The attention output gate's producer the same way: saber_iu8_sigmoid_table writes bf16(sigmoid) of every bf16
 * pattern (u16 [65536], 128 KiB, the kernel's own expression: crates/saber-kernels/hip/attn_glue_hadi8.hip:23-79);
 * with it saber_iu8_attn_gate_quant_had_lut launches attn_gate_quant_hadi8_lut_t256 for rows of
 * SABER_IU8_SILU_LUT_MIN_WIDTH elements and more, from SABER_IU8_SIGMOID_LUT_MIN_ROWS rows on (below, the copy of
 * the table's middle costs more than the few rows' exps) and, as attn_gate_quant_hadi8_lut_t1024, wherever the
 * 1,024-thread form is launched (four times the threads share the copy). The GDN norm's f32 gate was tabled too and did not
 * gain: that kernel is not bound by its gate. */
#define SABER_IU8_SIGMOID_LUT_MIN_ROWS 1024u
int saber_iu8_sigmoid_table(saber_iu8_ctx *ctx, void *out_u16, void *stream);
int saber_iu8_attn_gate_quant_had_lut(saber_iu8_ctx *ctx, const void *core_bf16, const void *gate_bf16, void *q, float *scale,
                                      uint32_t m, uint32_t n, uint32_t head_dim, uint32_t gate_stride, const float *had_t,
                                      const uint16_t *sigmoid_lut, void *stream);
int saber_iu8_add_rms_quant_had(saber_iu8_ctx *ctx, const void *y_bf16, const void *res_bf16, const void *w_bf16, void *q,
                                float *scale, void *res_out_bf16, uint32_t m, uint32_t k, float eps, const float *had_t,
                                void *stream);
int saber_iu8_gdn_norm_quant_had(saber_iu8_ctx *ctx, const void *x_bf16, const void *z_bf16, int64_t z_stride,
                                 const void *w_bf16, void *q, float *scale, uint32_t m, uint32_t n, float eps,
                                 const float *had_t, void *stream);
int saber_iu8_attn_gate_quant_had(saber_iu8_ctx *ctx, const void *core_bf16, const void *gate_bf16, void *q, float *scale,
                                  uint32_t m, uint32_t n, uint32_t head_dim, uint32_t gate_stride, const float *had_t,
                                  void *stream);

/* macaq_iu8::pair(first, second) (crates/saber-kernels/src/macaq_iu8.rs:632-704): two W4 decode
 * GEMMs that read one A operand, one dispatch of the fused object's `macaq_iu8f_pair_w4_tm*`
 * (kernarg list abi.rs:3411-3432). Each half is the descriptor saber_iu8_resolve / _describe gave
 * it alone; the grids go end to end, the second half's buffers and workspaces take the suffix `_b`.
 * Refused (SABER_IU8_E_RULE) unless both halves are W4 decode cells of one kernel, M and K. */
int saber_iu8_pair(const saber_iu8_desc *first, const saber_iu8_desc *second, saber_iu8_desc *out);
/* The same with the block order named instead of taken from the law (PAIR_BA_FIRST,
 * macaq_iu8.rs:549-553): second_first = 1 lays the second problem's workgroups first
 * (macaq_iu8f_pairb_w4_tm*), 0 problem 0's (macaq_iu8f_pair_w4_tm*). Same bytes either way. */
int saber_iu8_pair_ordered(const saber_iu8_desc *first, const saber_iu8_desc *second, int second_first,
                           saber_iu8_desc *out);
/* resolve x 2 + pair + launch for the unsplit decode law: c [m,n] and c_b [m,n_b] from one a / a_scale. */
int saber_iu8_gemm_pair(saber_iu8_ctx *ctx, const void *a, const float *a_scale, const void *w, const float *w_scale, void *c,
                        uint32_t n, const void *w_b, const float *w_scale_b, void *c_b, uint32_t n_b, uint32_t m, uint32_t k,
                        void *stream);

/* The whole decode linear in one launch where that is the faster form (saber_iu8_fused_holds: up to
 * 4 rows whose codes, rows rounded up to a power of two, fit 20 KiB of LDS -- kernel `_tm1`, or `_r1` for
 * one row of K >= 8192 -- and 2 rows of K >= 16384 whose codes fit 80 KiB -- kernel `_tm1_a80`,
 * which itself holds up to 16 rows and is reachable by name through saber_iu8_describe_raw; the other
 * row counts measured slower than the two launches): per-token quantisation fused into the
 * GEMV's activation staging. x bf16 [m,k]; q (A edge) and scale f32 [m] are optional outputs (NULL:
 * not stored) with the bytes saber_iu8_quant would write. Other shapes are refused
 * (SABER_IU8_E_RULE): run saber_iu8_quant + saber_iu8_gemm. No counterpart among the reference's
 * iu8 symbols (its fusions put the quantisation behind norm/activation producers,
 * crates/saber-kernels/src/macaq_iu8.rs:864-875); the law and the bytes are the same. */
int saber_iu8_fused_holds(uint32_t m, uint32_t k);
int saber_iu8_resolve_fused(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out);
int saber_iu8_linear_fused(saber_iu8_ctx *ctx, int wkind, const void *x_bf16, const void *w, const float *ws,
                           void *c_bf16, void *q, float *scale, uint32_t m, uint32_t n, uint32_t k, void *stream);

/* The dense decode MLP as ONE persistent launch: gate+up linear -> SiLU(gate) * up with its
 * per-token requantisation -> down linear, for at most 4 rows whose codes fit the fused form at both
 * widths (saber_iu8_mlp_chain_holds: at most 4 rows, 20 KiB of codes at hidden and at inter). The dense twin of the reference's routed
 * back half, which chains gate_up -> silu-quant -> down in one persistent launch with device-counter
 * hand-overs (crates/saber-kernels/hip/moe_grouped.hip:1656-1765, crates/saber-kernels/src/moe.rs:341-345);
 * its dense MLP is three launches (crates/saber-kernels/src/macaq_iu8.rs:864-875), whose bytes this
 * launch reproduces. x bf16 [m, hidden]; w_gu W4 [2*inter, hidden] (gate rows, then up rows) with
 * ws_gu f32 [2*inter]; w_dn W4 [hidden, inter] with ws_dn f32 [hidden]; c bf16 [m, hidden].
 * Workspaces (the descriptor lists them): p bf16 [m, inter], scratch (undefined at entry); state,
 * SABER_IU8_MLP_CHAIN_STATE_BYTES, persistent in the reference's sense (include/saber_abi.h:163-174):
 * zeroed once when allocated and left zero by a launch that completes, except its first 8 KiB (the
 * workgroups' maxima), which every launch rewrites before reading. gu bf16 [m, 2*inter] is an optional
 * tap (NULL: not stored). The workgroups meet through `state` (an arrival word a workgroup), so all
 * of them must be resident at once: the launch is refused (SABER_IU8_E_RULE) on a device that does
 * not hold the grid. A wait lasts at most `spin` polls (0: the default, about a second); a launch
 * that gives up leaves a non-zero word at state + SABER_IU8_MLP_CHAIN_STATUS_OFFSET and every element
 * of c a bf16 NaN (0x7FC0) -- and so does every later launch on that state block while the word is
 * set, e.g. the replays of a captured graph: the failure shows in the output itself. A caller that
 * finds the word set (or NaNs where the inputs had none) zeroes `state` and runs the three launches.
 * Launches that share one `state` must not overlap. Work that other streams run on the device at the
 * same time can hold compute units the grid needs: the launch then waits for it at its meeting (up to
 * `spin`), so keep the stream's neighbours quiet around it or use the three launches.
 * saber_iu8_mlp_chain_pays: where the one launch measured faster than the three on this card (one row
 * of an intermediate width of 12,288 to 20,480, two rows of 13,824 to 20,480: 4-7 % and 2-3 %); elsewhere
 * the three launches are as fast or faster, and a caller takes those.
 * Asynchronous. */
#define SABER_IU8_MLP_CHAIN_STATE_BYTES (13 * 1024)
#define SABER_IU8_MLP_CHAIN_STATUS_OFFSET (12 * 1024)
int saber_iu8_mlp_chain_holds(uint32_t m, uint32_t hidden, uint32_t inter);
int saber_iu8_mlp_chain_pays(uint32_t m, uint32_t hidden, uint32_t inter);
int saber_iu8_resolve_mlp_chain(uint32_t m, uint32_t hidden, uint32_t inter, uint32_t spin, saber_iu8_desc *out);
int saber_iu8_mlp_chain(saber_iu8_ctx *ctx, const void *x_bf16, const void *w_gu, const float *ws_gu, const void *w_dn,
                        const float *ws_dn, void *gu, void *p, void *state, void *c, uint32_t m, uint32_t hidden, uint32_t inter,
                        uint32_t spin, void *stream);

/* The gate+up linear of a dense decode MLP with SiLU(gate) * up in its epilogue, for up to 16 quantised rows whose
 * codes (rows rounded up to a power of two) fit 80 KiB of LDS at the hidden width (saber_iu8_gate_up_act_holds: 16 rows
 * of 5,120): a [m, hidden] int8 codes (A edge) with a_scale f32 [m], w_gu W4 [2*inter, hidden] (gate rows, then up rows)
 * with ws_gu f32 [2*inter] -> p bf16 [m, inter] = bf16(bf16(silu(gate)) * up); gu bf16 [m, 2*inter] is an optional tap
 * of [gate | up] (NULL: not stored). Kernel macaq_iu8f_gateup_act_w4_s80 (plugin macaq_iu8f). The MLP is then
 * quant -> this -> quant(p) -> down in place of quant -> linear -> silu_mul_quant -> down: the same bytes (p is what
 * silu_mul_quant quantises), one pass less over [m, 2*inter] and no exp in a producer. The dense twin of the routed
 * layer's saber_iu8_moe_gate_up_act; the reference's dense MLP keeps the activation in its producer
 * (crates/saber-kernels/hip/mxfp4_hadi8.hip:117-146). Asynchronous. */
int saber_iu8_gate_up_act_holds(uint32_t m, uint32_t hidden, uint32_t inter);
int saber_iu8_resolve_gate_up_act(uint32_t m, uint32_t hidden, uint32_t inter, saber_iu8_desc *out);
int saber_iu8_gate_up_act(saber_iu8_ctx *ctx, const void *a, const float *a_scale, const void *w_gu, const float *ws_gu, void *gu,
                          void *p_bf16, uint32_t m, uint32_t hidden, uint32_t inter, void *stream);

/* The tile GEMM with the per-token quantisation fused into its A-tile load (kernels macaq_iu8_pfq_*):
 * x bf16 [m,k] and the rows' scales a_scale f32 [m] -- from saber_iu8_rowscale (the producer's scale
 * without its codes) or carried from whatever made the rows -- instead of stored codes; c holds the
 * bytes of saber_iu8_quant + saber_iu8_gemm. No counterpart among the reference's symbols: its
 * prefill tile reads codes a producer stored (crates/saber-kernels/hip/macaq_iu8.hip:174-280,
 * producers hip/mxfp4_hadi8.hip:22-58). saber_iu8_resolve_prefill_fused picks the cell; any
 * macaq_iu8_pfq_* kernel is reachable through saber_iu8_describe by name. */
int saber_iu8_rowscale(saber_iu8_ctx *ctx, const void *x_bf16, float *scale, uint32_t m, uint32_t k, void *stream);
int saber_iu8_resolve_prefill_fused(int wkind, uint32_t m, uint32_t n, uint32_t k, saber_iu8_desc *out);
int saber_iu8_linear_prefill_fused(saber_iu8_ctx *ctx, int wkind, const void *x_bf16, const float *a_scale, const void *w,
                                   const float *w_scale, void *c_bf16, uint32_t m, uint32_t n, uint32_t k, void *stream);

/* Workspace bytes the resolved GEMM needs (both 0 when it does not split). Ask before every
 * saber_iu8_gemm of a new shape: the law splits K in one band (K >= 16384, 33..128 rows, few tiles),
 * and such a launch with `partial` / `counter` NULL is refused (SABER_IU8_E_ARG). */
int saber_iu8_gemm_workspace(int wkind, uint32_t m, uint32_t n, uint32_t k, uint64_t *partial_bytes,
                             uint64_t *counter_bytes);

/* C[m,n] bf16 = epilogue(A . W^T): a/as from the producer, w in the gfx950 fragment order, ws f32
 * [n]. `partial` (scratch) and `counter` (zeroed once by the caller, left zero) may be NULL when
 * saber_iu8_gemm_workspace reports 0.
 * Non-finite rows: a row whose scale is infinite (an infinity among its activations) gives infinities
 * where its accumulator is not zero and NaNs where it is (0 * inf), exactly where the contract's two
 * multiplies make them (crates/saber-kernels/hip/macaq_iu8.hip:20-24); that an element of c is a NaN is
 * defined, its sign and payload are not (they are the multiplier's that made it). */
int saber_iu8_gemm(saber_iu8_ctx *ctx, int wkind, const void *a, const float *as, const void *w, const float *ws,
                   void *c_bf16, uint32_t m, uint32_t n, uint32_t k, void *partial, void *counter, void *stream);

/* saber_iu8_gemm for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc between launches. No counterpart in the reference, whose host owns
 * every allocation (include/saber_abi.h:163-174). The split-K workspaces of the launch (`partial`,
 * `counter`) are not arguments: they live in one static device array of the library, 8 MiB of
 * partials + 64 KiB of counters (saber_iu8_static_workspace_bytes), present once on every GPU a context
 * was opened on and held until the process ends. Same kernels, same bytes as saber_iu8_gemm. Allocates,
 * clears and synchronises nothing: the counters are zero from set-up and every kernel leaves them
 * zero. A shape whose split needs more than the array holds is refused (SABER_IU8_E_RULE): use
 * saber_iu8_gemm with caller-owned workspaces. All calls on one GPU share that GPU's array: calls
 * that overlap in time on one GPU (different streams, no event between them) race on it. */
int saber_iu8_gemm_static(saber_iu8_ctx *ctx, int wkind, const void *a, const float *as, const void *w, const float *ws,
                          void *c_bf16, uint32_t m, uint32_t n, uint32_t k, void *stream);
uint64_t saber_iu8_static_workspace_bytes(void);
/* The static array's arrival counters back to zero, by a fill kernel on `stream` (no memset, so it may be
 * captured): recovery for a process in which a split launch was cut short between a tile's first and last
 * arrival (a device error, a destroyed stream), which leaves counters no later launch brings back to zero.
 * Not needed in ordinary use -- every kernel leaves its counters at zero. Belongs to saber_iu8_gemm_static
 * and, like it, has no counterpart in the reference. SABER_IU8_E_NOTLOADED when the device has no array. */
int saber_iu8_static_workspace_reset(saber_iu8_ctx *ctx, void *stream);

/* The raw int32 accumulators of the same GEMM (16 * sum(a*w) for W4, sum(a*w) for W8), int32
 * [m,n]: the parity tap. No counterpart in the reference's shipped object (its tests replay
 * captured bytes, crates/saber-kernels/hip/harness/run_hsaco.cpp:1-15). The tap kernels are not in
 * the plugin directory: SABER_IU8_E_NOTLOADED until the test-only object `iu8_taps` was added with
 * saber_iu8_load_plugin. */
int saber_iu8_gemm_acc(saber_iu8_ctx *ctx, int wkind, const void *a, const void *w, int32_t *acc, uint32_t m,
                       uint32_t n, uint32_t k, void *stream);

/* ------------------------------------------------------------------ routed experts (MoE) */

/* The reference has no iu8 MoE; these entry points compose its routing / tile / combine law
 * (crates/saber-kernels/hip/moe_route.hip, crates/saber-kernels/src/moe.rs) with the iu8 GEMM at
 * 128 experts, top-8 (the one router symbol this build ships: other widths are refused). */

/* Geometry caps (crates/saber-kernels/src/moe.rs:691-708); the `_shared` forms add the shared expert's
 * rows (every token once, padded to 16) and tiles. */
uint32_t saber_iu8_moe_rows_cap(uint32_t tokens, uint32_t topk, uint32_t experts);
uint32_t saber_iu8_moe_tiles_cap(uint32_t tokens, uint32_t topk, uint32_t experts, uint32_t tile_blocks);
uint32_t saber_iu8_moe_rows_cap_shared(uint32_t tokens, uint32_t topk, uint32_t experts);
uint32_t saber_iu8_moe_tiles_cap_shared(uint32_t tokens, uint32_t topk, uint32_t experts, uint32_t tile_blocks);
/* tile_blocks the grouped law picks for `tokens`: 1 (16-row tiles, weight-streaming cells) while an
 * expert averages <= 7 routes, 8 (128-row MFMA tiles) below 128 routes an expert, 16 (256-row) from there. */
uint32_t saber_iu8_moe_tile_blocks(uint32_t tokens, uint32_t topk, uint32_t experts);

/* Device buffers of one routed layer, named as the router kernel's arguments
 * (crates/saber-kernels/src/abi.rs:354-374); all caller-owned. */
typedef struct {
  int32_t *topk_ids;    /* [T * topk] */
  float *topk_w;        /* [T * topk] */
  int32_t *route_pos;   /* [T * topk] */
  int32_t *row_tok;     /* [rows_cap] */
  int32_t *row_route;   /* [rows_cap] */
  int32_t *tile_expert; /* [tiles_cap] */
  int32_t *tile_row0;   /* [tiles_cap] */
  int32_t *tile_rows;   /* [tiles_cap] */
  int32_t *expert_cnt;  /* [experts] */
  int32_t *meta;        /* [8]: [0] tiles, [1] rows, [2] first shared row or -1, [3] routes, [4] experts touched */
  int32_t *blk_cnt;     /* [ceil(T / 32) * experts]  scratch (the one-launch router uses the first ceil(T / 128) * experts) */
  int32_t *rank;        /* [T * topk]                scratch */
  int32_t *arrive;      /* [1]  persistent: zeroed once by the caller, left zero */
  const uint16_t *silu_lut; /* optional (may be NULL): [65536] as saber_iu8_silu_table wrote it; with it
                             * saber_iu8_moe_silu_mul_quant reads the bf16 silu from the table on large row counts */
  const uint16_t *sgate;    /* optional (may be NULL): bf16 [T], the shared expert's gate logits. Given, the layer has a
                             * shared expert (crates/saber-kernels/hip/moe_route.hip:244-272, 299-321): the router appends
                             * every token as a row of expert index `experts` (its weights are entry `experts` of the
                             * grouped GEMMs' pointer table), sized by the `_shared` caps, and the combine adds
                             * sigmoid(sgate[t]) * Y[shared row of t] */
} saber_iu8_moe_tables;

/* Router + expert-major sort + tile table (crates/saber-kernels/hip/moe_route.hip:108-284). logits bf16
 * [T, experts]. One launch up to 128 tokens (one routing workgroup); above, two: routing with the
 * workgroups' counts and ranks (32 tokens a workgroup: blk_cnt is used in full), then the layout with every
 * workgroup placing its own routes. */
int saber_iu8_moe_route(saber_iu8_ctx *ctx, const void *logits_bf16, uint32_t tokens, uint32_t experts, uint32_t topk,
                        uint32_t tile_blocks, const saber_iu8_moe_tables *t, void *stream);

/* The router and the per-token quantisation of the layer's input in one launch (the two are
 * independent; in the reference they are two operators, moe_route.hip:108-284 and the int8 producer
 * mxfp4_hadi8.hip:22-58): what saber_iu8_moe_route and saber_iu8_quant(x, q, scale, tokens, k) would
 * write (tile_blocks 1: q in the A fragment order, [ceil(tokens/16)*16, k] bytes, what the streaming
 * cell gathers from) or saber_iu8_quant_rowmajor (tile_blocks 8 / 16: q row-major [tokens, k], what
 * the MFMA cells gather from). With few tokens a layer's time is its launches; with many, the
 * router's tail -- one workgroup lays out the tables -- runs beside the quantisation instead of in
 * front of it. x bf16 [tokens, k], scale f32 [tokens]; K % 128 == 0, K <= 16384. */
int saber_iu8_moe_route_quant(saber_iu8_ctx *ctx, const void *logits_bf16, const void *x_bf16, void *q, float *scale,
                              uint32_t tokens, uint32_t experts, uint32_t topk, uint32_t k, uint32_t tile_blocks,
                              const saber_iu8_moe_tables *t, void *stream);

/* Grouped W4 GEMM over the tile table: per tile the expert's weights (gfx950 W4 fragments) at
 * xptr[2e] and f32 row scales at xptr[2e + 1] (device array of 2 * experts addresses); A rows
 * gathered through row_tok (gather 1: a is the token-major A edge; gather 2, MFMA cells only: a is
 * token-major row-major codes from saber_iu8_quant_rowmajor; as token-major) or in place (gather 0:
 * a / as are expert-major); C bf16 [rows_cap, n]. tile_blocks as given to the router (1, 8 or 16). */
int saber_iu8_moe_grouped(saber_iu8_ctx *ctx, const void *a, const float *as, const void *xptr, void *c_bf16, uint32_t n,
                          uint32_t k, int gather, uint32_t tokens, uint32_t experts, uint32_t topk, uint32_t tile_blocks,
                          const saber_iu8_moe_tables *t, void *stream);

/* The routed layer's activations gathered and quantised in one pass: output row r (expert-major,
 * rows_cap rows, A edge) = the int8 codes of token row row_tok[r], scale[r] its scale; pad rows and
 * rows past meta[1] are left alone. With it the grouped gate+up GEMM runs on compact rows (gather 0)
 * and reads whole fragments; the reference gathers inside its grouped GEMM from row-major rows
 * (crates/saber-kernels/hip/moe_grouped.hip:67-74), which this object's tiled A order would turn
 * into 16-byte reads. */
int saber_iu8_moe_quant_rows(saber_iu8_ctx *ctx, const void *x_bf16, void *q, float *scale, uint32_t k, uint32_t rows_cap,
                             const saber_iu8_moe_tables *tables, void *stream);

/* SiLU(gate)*up + requant over the live expert-major rows: gu bf16 [rows_cap, 2n] -> q (A edge of
 * rows_cap rows), scale f32 [rows_cap]. Pad rows are skipped. */
int saber_iu8_moe_silu_mul_quant(saber_iu8_ctx *ctx, const void *gu_bf16, void *q, float *scale, uint32_t n,
                                 uint32_t rows_cap, const saber_iu8_moe_tables *t, void *stream);

/* The routed back half with few tokens as two launches instead of three (16-row tiles only,
 * tile_blocks 1, and an intermediate width whose 16 rows fit the second launch's LDS:
 * saber_iu8_moe_back_holds). The reference chains gate_up -> silu-quant -> down inside its persistent
 * back half (crates/saber-kernels/hip/moe_grouped.hip:1656-1765, crates/saber-kernels/src/moe.rs:341-345);
 * here the activation sits in the first GEMM's epilogue and the requantisation in front of the second
 * GEMM's K loop, with the bytes of saber_iu8_moe_grouped -> saber_iu8_moe_silu_mul_quant ->
 * saber_iu8_moe_grouped.
 *   saber_iu8_moe_gate_up_act: a / as the token-major A edge and scales (gathered through row_tok),
 *     xptr the experts' gate+up weights ([2 * inter, k]: gate rows, then up rows) and scales;
 *     p bf16 [rows_cap, inter] = bf16(bf16(silu(gate)) * up).
 *   saber_iu8_moe_down_rows: p as written above, quantised per row in front of the K loop (K = inter);
 *     xptr the experts' down weights ([n, inter]) and scales; y bf16 [rows_cap, n]. */
int saber_iu8_moe_back_holds(uint32_t tile_blocks, uint32_t inter);
/* The launch law's pick: the two-launch form wherever it holds (measured faster at every token count of the 16-row regime). */
int saber_iu8_moe_back_pays(uint32_t tokens, uint32_t topk, uint32_t experts, uint32_t tile_blocks, uint32_t inter);
int saber_iu8_moe_gate_up_act(saber_iu8_ctx *ctx, const void *a, const float *as, const void *xptr, void *p_bf16,
                              uint32_t inter, uint32_t k, uint32_t tokens, uint32_t experts, uint32_t topk,
                              uint32_t tile_blocks, const saber_iu8_moe_tables *t, void *stream);
int saber_iu8_moe_down_rows(saber_iu8_ctx *ctx, const void *p_bf16, const void *xptr, void *y_bf16, uint32_t n,
                            uint32_t inter, uint32_t tokens, uint32_t experts, uint32_t topk, uint32_t tile_blocks,
                            const saber_iu8_moe_tables *t, void *stream);

/* Weighted combine: out[t] = bf16(sum_k w[t,k] * Y[pos(t,k)]) in top-k order; y bf16 [rows_cap, h]. */
int saber_iu8_moe_combine(saber_iu8_ctx *ctx, const void *y_bf16, const saber_iu8_moe_tables *t, void *out_bf16,
                          uint32_t tokens, uint32_t topk, uint32_t h, void *stream);

/* bf16 silu of every bf16 bit pattern as the device computes it: out u16 [65536] (device). The
 * parity suite compares it with the host formula for all 65,536 inputs. */
int saber_iu8_silu_table(saber_iu8_ctx *ctx, void *out_u16, void *stream);

/* ---- tier packs ("SBRPACK1"): reading the iu8 records of a built pack ------------------------------
 * The byte layout of include/saber_abi.h:541-944 and the open-time rules of
 * crates/saber-mem/src/pack/{format,reader}.rs (PackReader::open_with / open_expecting): magic,
 * format version 1..2, 256-byte header, 160-byte records sorted by 4096-aligned data_off, lengths
 * implied by shape and dtype, name prefixes, the chunk-digest blob, the table hash last, and the plan
 * hash when one is expected. Refusals: SABER_IU8_E_PARSE (malformed), SABER_IU8_E_VALIDATE (a hash
 * does not match), SABER_IU8_E_IO. */
typedef struct saber_iu8_pack saber_iu8_pack;
typedef struct {
  uint32_t format_version, record_count, tp_size, rank, chunk_bytes;
  uint64_t data_off, file_bytes, build_unix_seconds;
  uint8_t plan_hash[32], tier_id[32];
} saber_iu8_pack_header;
typedef struct {
  char name[128];       /* the checkpoint's tensor name, NUL-terminated here */
  uint32_t rank, layout_id, flags;
  uint16_t dtype;       /* saber_pack_dtype tag */
  uint8_t ndim, shard_kind;
  uint64_t data_off, length, shape[8];
  uint8_t sha256[32];
} saber_iu8_pack_record;
typedef struct {
  int wkind;            /* SABER_IU8_W4: `<op>.wi4` layout 17; SABER_IU8_W8: `<op>.wi8` layout 18 */
  uint32_t n, k, w_record, s_record;
  uint64_t w_bytes;     /* N*K/2 or N*K */
  uint8_t shard_kind;
} saber_iu8_pack_linear_info;

/* expected_plan_hash: 32 bytes, or NULL to open without the plan check. */
int saber_iu8_pack_open(const char *path, const uint8_t *expected_plan_hash, saber_iu8_pack **out);
void saber_iu8_pack_close(saber_iu8_pack *pack);
int saber_iu8_pack_info(const saber_iu8_pack *pack, saber_iu8_pack_header *out);
int saber_iu8_pack_record_at(const saber_iu8_pack *pack, uint32_t index, saber_iu8_pack_record *out);
/* Index of the record of that name, or -1. */
int saber_iu8_pack_find(const saber_iu8_pack *pack, const char *name);
/* One record's payload (exactly `length` bytes) into dst, verified against its sha256 and its chunk
 * digests where the pack carries them: a bad record is a load error, not a garbage weight. */
int saber_iu8_pack_read(saber_iu8_pack *pack, uint32_t index, void *dst, uint64_t cap);
/* The two records of an iu8 GEMM op (crates/saber-model/src/graph.rs:3848-3914): codes in the gfx12
 * W-fragment order (`<op>.wi4` layout 17 U8 [N/16, K*8] or `<op>.wi8` layout 18 U8 [N/16, K*16]) and
 * the f32 row scale (`<op>.wi4s` / `<op>.wi8s`, layout 19 [N]). */
int saber_iu8_pack_linear(const saber_iu8_pack *pack, const char *op, saber_iu8_pack_linear_info *out);
/* Read + verify + repack offline into the gfx950 fragment order (layout ids 33 / 34): w_gfx950 host
 * memory of w_bytes, w_scale of n floats. */
int saber_iu8_pack_load_linear(saber_iu8_pack *pack, const char *op, uint8_t *w_gfx950, uint64_t w_cap, float *w_scale,
                               uint64_t ws_cap);

#ifdef __cplusplus
}
#endif
#endif /* SABER_IU8_H */
