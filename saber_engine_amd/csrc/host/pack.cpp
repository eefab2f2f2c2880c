// Reader of the tier-pack file format ("SBRPACK1") as far as the W4A8-iu8 linears need it: the
// counterpart of crates/saber-mem/src/pack/{format,reader}.rs against the byte layout of
// include/saber_abi.h:541-944. A pack is a 256-byte header, a table of 160-byte records, a name
// blob, an optional chunk-digest blob (format version 2) and 4096-aligned payloads. Everything the
// reference's reader refuses at open is refused here, in its order: header ranges, record
// structure, names, chunk blob, record placement, and the table hash last (a broken table reports
// its structural fault, not a hash mismatch; reader.rs:39-150). Payloads are hash-verified when read.
//
// The iu8 records of an op (crates/saber-model/src/graph.rs:3848-3914): `<op>.wi4` layout 17 U8
// [N/16, K*8] or `<op>.wi8` layout 18 U8 [N/16, K*16] in the gfx12 W-fragment order, and the row
// scale `<op>.wi4s` / `<op>.wi8s` layout 19 F32 [N]. Loading one repacks the codes offline into the
// gfx950 fragment order (layout.cpp); nothing is transformed on a launch path.
#include <cerrno>
#include <map>
#include <memory>

#include "../../../include/saber_iu8.h"
#include "util.h"

using namespace iu8;

namespace {

constexpr uint64_t ALIGN = 4096, HEADER_BYTES = 256, RECORD_BYTES = 160, CHUNK_ENTRY_HEADER = 40;
constexpr uint32_t VERSION_MIN = 1, VERSION_MAX = 2, FLAGS_KNOWN = 1, MAX_NDIM = 8;
constexpr uint32_t LAYOUT_I4_ROW_FRAG = 17, LAYOUT_I8_ROW_FRAG = 18, LAYOUT_IU8_ROW_SCALE = 19;
constexpr uint16_t DT_U8 = 0, DT_F32 = 10;

uint64_t align_up(uint64_t x) { return (x + ALIGN - 1) / ALIGN * ALIGN; }
uint16_t u16_at(const uint8_t *b, size_t o) { return (uint16_t)(b[o] | b[o + 1] << 8); }
uint32_t u32_at(const uint8_t *b, size_t o) { return (uint32_t)b[o] | (uint32_t)b[o + 1] << 8 | (uint32_t)b[o + 2] << 16 | (uint32_t)b[o + 3] << 24; }
uint64_t u64_at(const uint8_t *b, size_t o) { return (uint64_t)u32_at(b, o) | (uint64_t)u32_at(b, o + 4) << 32; }

// bits per logical element by dtype tag (include/saber_abi.h:600-625); 0 = unknown tag
uint32_t dtype_bits(uint16_t tag) {
  static const uint32_t BITS[17] = {8, 8, 16, 16, 32, 32, 64, 64, 16, 16, 32, 64, 8, 8, 4, 8, 8};
  return tag < 17 ? BITS[tag] : 0;
}

std::string hex32(const uint8_t *h) {
  std::string s;
  for (int i = 0; i < 32; ++i) s += fmt("%02x", h[i]);
  return s;
}

}  // namespace

struct saber_iu8_pack {
  std::string path;
  FILE *fp = nullptr;
  saber_iu8_pack_header header{};
  std::vector<saber_iu8_pack_record> records;
  std::map<std::string, uint32_t> by_name;
  std::map<uint32_t, std::vector<uint8_t>> chunk_digests;  // record index -> n_chunks * 32 bytes
  ~saber_iu8_pack() {
    if (fp) fclose(fp);
  }
};

static bool read_at(FILE *fp, uint64_t off, void *dst, uint64_t n) {
  if (fseeko(fp, (off_t)off, SEEK_SET) != 0) return false;
  return fread(dst, 1, n, fp) == n;
}

extern "C" int saber_iu8_pack_open(const char *path, const uint8_t *expected_plan_hash, saber_iu8_pack **out) {
  if (!path || !out) return fail(SABER_IU8_E_ARG, "pack_open: null argument");
  *out = nullptr;
  std::unique_ptr<saber_iu8_pack> pk(new saber_iu8_pack);
  pk->path = path;
  pk->fp = fopen(path, "rb");
  if (!pk->fp) return fail(SABER_IU8_E_IO, fmt("%s: cannot open (%s)", path, strerror(errno)));
  fseeko(pk->fp, 0, SEEK_END);
  const uint64_t file_len = (uint64_t)ftello(pk->fp);
  auto bad = [&](const std::string &m) { return fail(SABER_IU8_E_PARSE, std::string(path) + ": " + m); };
  if (file_len < ALIGN)
    return bad(fmt("file is %llu bytes; a pack is at least one %llu-byte block", (unsigned long long)file_len, (unsigned long long)ALIGN));

  // ---- header (format.rs:244-408)
  uint8_t hb[HEADER_BYTES];
  if (!read_at(pk->fp, 0, hb, HEADER_BYTES)) return fail(SABER_IU8_E_IO, std::string(path) + ": cannot read the header");
  if (memcmp(hb, "SBRPACK1", 8) != 0) return bad("bad magic: not a pack file");
  saber_iu8_pack_header &h = pk->header;
  h.format_version = u32_at(hb, 8);
  if (h.format_version < VERSION_MIN || h.format_version > VERSION_MAX)
    return bad(fmt("format version %u; this reader reads %u..%u", h.format_version, VERSION_MIN, VERSION_MAX));
  if (u32_at(hb, 12) != HEADER_BYTES) return bad(fmt("header_bytes %u must be %llu", u32_at(hb, 12), (unsigned long long)HEADER_BYTES));
  if (u32_at(hb, 16) != RECORD_BYTES) return bad(fmt("record_bytes %u must be %llu", u32_at(hb, 16), (unsigned long long)RECORD_BYTES));
  for (size_t i = h.format_version >= 2 ? 228 : 176; i < 256; ++i)
    if (hb[i]) return bad("header reserved bytes are not zero");
  h.record_count = u32_at(hb, 20);
  const uint64_t table_off = u64_at(hb, 24), name_blob_off = u64_at(hb, 32), name_blob_bytes = u64_at(hb, 40);
  h.data_off = u64_at(hb, 48);
  h.file_bytes = u64_at(hb, 56);
  h.tp_size = u32_at(hb, 64);
  h.rank = u32_at(hb, 68);
  h.build_unix_seconds = u64_at(hb, 72);
  memcpy(h.plan_hash, hb + 80, 32);
  memcpy(h.tier_id, hb + 112, 32);
  uint8_t table_sha[32], chunk_sha[32] = {0};
  memcpy(table_sha, hb + 144, 32);
  uint64_t chunk_blob_off = 0, chunk_blob_bytes = 0;
  if (h.format_version >= 2) {
    chunk_blob_off = u64_at(hb, 176), chunk_blob_bytes = u64_at(hb, 184);
    memcpy(chunk_sha, hb + 192, 32);
    h.chunk_bytes = u32_at(hb, 224);
  }
  if (table_off != HEADER_BYTES) return bad(fmt("table_off %llu must be %llu", (unsigned long long)table_off, (unsigned long long)HEADER_BYTES));
  const uint64_t want_blob = table_off + (uint64_t)h.record_count * RECORD_BYTES;
  if (name_blob_off != want_blob)
    return bad(fmt("name_blob_off %llu must be %llu (table_off + record_count * 160)", (unsigned long long)name_blob_off, (unsigned long long)want_blob));
  if (h.data_off % ALIGN) return bad(fmt("data_off %llu is not 4096-aligned", (unsigned long long)h.data_off));
  if (name_blob_bytes > file_len) return bad("name blob runs past the file");
  const uint64_t names_end = name_blob_off + name_blob_bytes;
  static const uint8_t ZERO32[32] = {0};
  if (chunk_blob_bytes == 0) {
    if (chunk_blob_off != 0 || h.chunk_bytes != 0 || memcmp(chunk_sha, ZERO32, 32) != 0)
      return bad("a pack with no chunk blob must have all four chunk header fields zero");
  } else {
    if (chunk_blob_off != names_end)
      return bad(fmt("chunk_blob_off %llu must be %llu (immediately after the name blob)", (unsigned long long)chunk_blob_off, (unsigned long long)names_end));
    if (h.chunk_bytes == 0 || h.chunk_bytes % ALIGN) return bad(fmt("chunk_bytes %u must be a non-zero multiple of 4096", h.chunk_bytes));
    if (chunk_blob_bytes > file_len) return bad("chunk blob runs past the file");
  }
  const uint64_t meta_end = chunk_blob_bytes ? chunk_blob_off + chunk_blob_bytes : names_end;
  if (h.data_off < align_up(meta_end))
    return bad(fmt("data_off %llu overlaps the metadata (it ends at %llu after padding)", (unsigned long long)h.data_off, (unsigned long long)align_up(meta_end)));
  if (h.file_bytes % ALIGN) return bad(fmt("file_bytes %llu is not 4096-aligned", (unsigned long long)h.file_bytes));
  if (h.file_bytes < h.data_off) return bad("file_bytes is before data_off");
  if (h.tp_size == 0 || h.rank >= h.tp_size) return bad(fmt("rank %u is not valid for tp_size %u", h.rank, h.tp_size));
  if (h.file_bytes != file_len)
    return bad(fmt("header says file_bytes %llu but the file is %llu bytes", (unsigned long long)h.file_bytes, (unsigned long long)file_len));

  // ---- the metadata region: table, names, chunk blob
  std::vector<uint8_t> meta(meta_end);
  if (!read_at(pk->fp, 0, meta.data(), meta_end)) return fail(SABER_IU8_E_IO, std::string(path) + ": cannot read the metadata");
  pk->records.resize(h.record_count);
  for (uint32_t i = 0; i < h.record_count; ++i) {  // format.rs:487-543
    const uint8_t *b = meta.data() + table_off + (uint64_t)i * RECORD_BYTES;
    saber_iu8_pack_record &r = pk->records[i];
    memset(&r, 0, sizeof r);
    r.flags = u32_at(b, 20);
    if (r.flags & ~FLAGS_KNOWN) return bad(fmt("record %u: flags %#x not understood", i, r.flags));
    for (size_t o = 136; o < 160; ++o)
      if (b[o]) return bad(fmt("record %u: reserved bytes are not zero", i));
    r.ndim = b[18];
    if (r.ndim == 0 || r.ndim > MAX_NDIM) return bad(fmt("record %u: ndim %u outside 1..=8", i, r.ndim));
    for (uint32_t d = 0; d < MAX_NDIM; ++d) {
      const uint64_t v = u64_at(b, 40 + 8 * d);
      if (d < r.ndim && v == 0) return bad(fmt("record %u: shape[%u] is zero but ndim is %u", i, d, r.ndim));
      if (d >= r.ndim && v != 0) return bad(fmt("record %u: shape[%u] is set beyond ndim %u", i, d, r.ndim));
      r.shape[d] = v;
    }
    r.rank = u32_at(b, 8);
    r.layout_id = u32_at(b, 12);
    r.dtype = u16_at(b, 16);
    if (!dtype_bits(r.dtype)) return bad(fmt("record %u: unknown dtype tag %u", i, r.dtype));
    r.shard_kind = b[19];
    if (r.shard_kind > 3) return bad(fmt("record %u: unknown shard kind %u", i, r.shard_kind));
    r.data_off = u64_at(b, 24);
    r.length = u64_at(b, 32);
    memcpy(r.sha256, b + 104, 32);
    // the name: a u16 length prefix sits right before its first byte (reader.rs:385-412)
    const uint32_t name_off = u32_at(b, 0), name_len = u32_at(b, 4);
    if (name_len == 0) return bad(fmt("record %u: empty name", i));
    if (name_off < 2 || (uint64_t)name_off + name_len > name_blob_bytes) return bad(fmt("record %u: name [%u, +%u) is outside the name blob", i, name_off, name_len));
    if (u16_at(meta.data(), name_blob_off + name_off - 2) != name_len) return bad(fmt("record %u: the name's length prefix is not name_len %u", i, name_len));
    if (name_len >= sizeof r.name) return bad(fmt("record %u: a name of %u bytes is longer than this reader holds", i, name_len));
    memcpy(r.name, meta.data() + name_blob_off + name_off, name_len);
  }
  // ---- chunk blob (format.rs:621-680), trusted through its own digest
  if (chunk_blob_bytes) {
    uint8_t dg[32];
    sha256(meta.data() + chunk_blob_off, chunk_blob_bytes, dg);
    if (memcmp(dg, chunk_sha, 32) != 0) return bad("chunk blob hashes to " + hex32(dg) + " but the header says " + hex32(chunk_sha));
    const uint8_t *cb = meta.data() + chunk_blob_off;
    uint64_t off = 0;
    for (uint32_t i = 0; i < h.record_count; ++i) {
      const saber_iu8_pack_record &r = pk->records[i];
      if (!(r.flags & 1)) continue;
      if (off + CHUNK_ENTRY_HEADER > chunk_blob_bytes) return bad(fmt("chunk blob ends inside record %u's entry header", i));
      const uint64_t n = u32_at(cb, off);
      if (u32_at(cb, off + 4) != 0) return bad(fmt("chunk blob entry for record %u: flags not understood", i));
      const uint64_t want = (r.length + h.chunk_bytes - 1) / h.chunk_bytes;
      if (n != want) return bad(fmt("chunk blob entry for record %u: %llu digests, %llu expected", i, (unsigned long long)n, (unsigned long long)want));
      if (memcmp(cb + off + 8, r.sha256, 32) != 0) return bad(fmt("chunk blob entry for record %u names a different record", i));
      const uint64_t end = off + CHUNK_ENTRY_HEADER + 32 * n;
      if (end > chunk_blob_bytes) return bad(fmt("chunk blob ends inside record %u's digest list", i));
      pk->chunk_digests[i].assign(cb + off + CHUNK_ENTRY_HEADER, cb + end);
      off = end;
    }
    if (off != chunk_blob_bytes) return bad(fmt("chunk blob is %llu bytes; its entries account for %llu", (unsigned long long)chunk_blob_bytes, (unsigned long long)off));
  } else {
    for (uint32_t i = 0; i < h.record_count; ++i)
      if (pk->records[i].flags & 1) return bad(fmt("record %u carries the chunk-digest flag but the pack has no chunk blob", i));
  }
  // ---- record placement (reader.rs:172-216): sorted by data_off, no overlap after padding
  uint64_t cursor = h.data_off;
  for (uint32_t i = 0; i < h.record_count; ++i) {
    const saber_iu8_pack_record &r = pk->records[i];
    if (r.rank != h.rank) return bad(fmt("record %u (%s): rank %u but the file is rank %u", i, r.name, r.rank, h.rank));
    if (r.data_off % ALIGN) return bad(fmt("record %u (%s): data_off %llu is not 4096-aligned", i, r.name, (unsigned long long)r.data_off));
    if (r.data_off < cursor)
      return bad(fmt("record %u (%s): data_off %llu is below %llu; the table must be sorted by data_off and records must not overlap after padding",
                     i, r.name, (unsigned long long)r.data_off, (unsigned long long)cursor));
    uint64_t rec_end = 0;  // a data_off near 2^64 must not wrap past the check
    if (r.length > h.file_bytes || __builtin_add_overflow(r.data_off, r.length, &rec_end) || rec_end > h.file_bytes ||
        align_up(rec_end) > h.file_bytes)
      return bad(fmt("record %u (%s): runs past file_bytes", i, r.name));
    unsigned __int128 bits = dtype_bits(r.dtype);
    for (uint32_t d = 0; d < r.ndim; ++d) {
      bits *= r.shape[d];
      if (bits >> 100) return bad(fmt("record %u (%s): shape overflows", i, r.name));
    }
    const uint64_t implied = (uint64_t)((bits + 7) / 8);
    if (implied != r.length) return bad(fmt("record %u (%s): length %llu but its shape and dtype imply %llu", i, r.name, (unsigned long long)r.length, (unsigned long long)implied));
    cursor = align_up(r.data_off + r.length);
  }
  // ---- the table hash, last
  uint8_t dg[32];
  sha256(meta.data() + table_off, names_end - table_off, dg);
  if (memcmp(dg, table_sha, 32) != 0)
    return fail(SABER_IU8_E_VALIDATE, std::string(path) + ": table hash mismatch: header " + hex32(table_sha) + ", table and names hash to " + hex32(dg));
  for (uint32_t i = 0; i < h.record_count; ++i)
    if (!pk->by_name.emplace(pk->records[i].name, i).second) return bad(fmt("duplicate record name \"%s\"", pk->records[i].name));
  // ---- the plan this pack was built for: a mismatch is refused, never re-derived (reader.rs:152-171)
  if (expected_plan_hash && memcmp(expected_plan_hash, h.plan_hash, 32) != 0)
    return fail(SABER_IU8_E_VALIDATE, std::string(path) + ": plan hash " + hex32(h.plan_hash) + " is not the expected " + hex32(expected_plan_hash));
  *out = pk.release();
  return 0;
}

extern "C" void saber_iu8_pack_close(saber_iu8_pack *pk) { delete pk; }

extern "C" int saber_iu8_pack_info(const saber_iu8_pack *pk, saber_iu8_pack_header *out) {
  if (!pk || !out) return fail(SABER_IU8_E_ARG, "pack_info: null argument");
  *out = pk->header;
  return 0;
}

extern "C" int saber_iu8_pack_record_at(const saber_iu8_pack *pk, uint32_t index, saber_iu8_pack_record *out) {
  if (!pk || !out) return fail(SABER_IU8_E_ARG, "pack_record_at: null argument");
  if (index >= pk->records.size()) return fail(SABER_IU8_E_ARG, fmt("%s: record %u of %zu", pk->path.c_str(), index, pk->records.size()));
  *out = pk->records[index];
  return 0;
}

extern "C" int saber_iu8_pack_find(const saber_iu8_pack *pk, const char *name) {
  if (!pk || !name) return -1;
  auto it = pk->by_name.find(name);
  return it == pk->by_name.end() ? -1 : (int)it->second;
}

// The payload of one record into dst (exactly `length` bytes), verified against the record's sha256
// and, where the pack carries them, its chunk digests (the failing chunk is named).
extern "C" int saber_iu8_pack_read(saber_iu8_pack *pk, uint32_t index, void *dst, uint64_t cap) {
  if (!pk || !dst) return fail(SABER_IU8_E_ARG, "pack_read: null argument");
  if (index >= pk->records.size()) return fail(SABER_IU8_E_ARG, fmt("%s: record %u of %zu", pk->path.c_str(), index, pk->records.size()));
  const saber_iu8_pack_record &r = pk->records[index];
  if (cap < r.length) return fail(SABER_IU8_E_ARG, fmt("%s: record %s is %llu bytes, the buffer %llu", pk->path.c_str(), r.name, (unsigned long long)r.length, (unsigned long long)cap));
  if (!read_at(pk->fp, r.data_off, dst, r.length)) return fail(SABER_IU8_E_IO, fmt("%s: cannot read record %s", pk->path.c_str(), r.name));
  const uint8_t *p = (const uint8_t *)dst;
  uint8_t dg[32];
  auto cd = pk->chunk_digests.find(index);
  if (cd != pk->chunk_digests.end()) {
    const uint64_t cbytes = pk->header.chunk_bytes;
    for (uint64_t c = 0, o = 0; o < r.length; ++c, o += cbytes) {
      sha256(p + o, std::min(cbytes, r.length - o), dg);
      if (memcmp(dg, cd->second.data() + 32 * c, 32) != 0)
        return fail(SABER_IU8_E_VALIDATE, fmt("%s: record %s: chunk %llu does not hash to its digest", pk->path.c_str(), r.name, (unsigned long long)c));
    }
  }
  sha256(p, r.length, dg);
  if (memcmp(dg, r.sha256, 32) != 0)
    return fail(SABER_IU8_E_VALIDATE, fmt("%s: record %s hashes to %s, the table says %s", pk->path.c_str(), r.name, hex32(dg).c_str(), hex32(r.sha256).c_str()));
  return 0;
}

// The two records of an iu8 linear, checked against what graph.rs:3848-3914 writes.
extern "C" int saber_iu8_pack_linear(const saber_iu8_pack *pk, const char *op, saber_iu8_pack_linear_info *out) {
  if (!pk || !op || !out) return fail(SABER_IU8_E_ARG, "pack_linear: null argument");
  memset(out, 0, sizeof *out);
  for (int w8 = 0; w8 < 2; ++w8) {
    const std::string wname = std::string(op) + (w8 ? ".wi8" : ".wi4");
    const int wi = saber_iu8_pack_find(pk, wname.c_str());
    if (wi < 0) continue;
    const int si = saber_iu8_pack_find(pk, (wname + "s").c_str());
    if (si < 0) return fail(SABER_IU8_E_RULE, fmt("%s: %s has no row scale record %ss", pk->path.c_str(), wname.c_str(), wname.c_str()));
    const saber_iu8_pack_record &w = pk->records[wi], &s = pk->records[si];
    const uint32_t want_layout = w8 ? LAYOUT_I8_ROW_FRAG : LAYOUT_I4_ROW_FRAG;
    const uint64_t per_k = w8 ? 16 : 8;
    if (w.layout_id != want_layout || w.dtype != DT_U8 || w.ndim != 2 || w.shape[1] % per_k)
      return fail(SABER_IU8_E_RULE, fmt("%s: %s is not a layout-%u U8 [N/16, K*%llu] record", pk->path.c_str(), wname.c_str(), want_layout, (unsigned long long)per_k));
    const uint64_t n = w.shape[0] * 16, k = w.shape[1] / per_k;
    if (n == 0 || k == 0 || k % 128 || n > 0x7fffffffu || k > 0x7fffffffu)
      return fail(SABER_IU8_E_RULE, fmt("%s: %s: N=%llu, K=%llu is not an iu8 shape (K a multiple of 128)", pk->path.c_str(), wname.c_str(), (unsigned long long)n, (unsigned long long)k));
    if (s.layout_id != LAYOUT_IU8_ROW_SCALE || s.dtype != DT_F32 || s.ndim != 1 || s.shape[0] != n)
      return fail(SABER_IU8_E_RULE, fmt("%s: %ss is not a layout-19 F32 [%llu] record", pk->path.c_str(), wname.c_str(), (unsigned long long)n));
    out->wkind = w8 ? SABER_IU8_W8 : SABER_IU8_W4;
    out->n = (uint32_t)n, out->k = (uint32_t)k;
    out->w_record = (uint32_t)wi, out->s_record = (uint32_t)si;
    out->w_bytes = w.length, out->shard_kind = w.shard_kind;
    return 0;
  }
  return fail(SABER_IU8_E_RULE, fmt("%s: no iu8 records (%s.wi4 / %s.wi8)", pk->path.c_str(), op, op));
}

// Read, verify and repack one linear: w_gfx950 receives the codes in the gfx950 fragment order
// (w_bytes of them), ws the N row scales.
extern "C" int saber_iu8_pack_load_linear(saber_iu8_pack *pk, const char *op, uint8_t *w_gfx950, uint64_t w_cap, float *ws, uint64_t ws_cap) {
  saber_iu8_pack_linear_info li;
  if (int rc = saber_iu8_pack_linear(pk, op, &li)) return rc;
  if (!w_gfx950 || !ws || w_cap < li.w_bytes || ws_cap < li.n)
    return fail(SABER_IU8_E_ARG, fmt("pack_load_linear: %s needs %llu code bytes and %u scales", op, (unsigned long long)li.w_bytes, li.n));
  std::vector<uint8_t> frag12(li.w_bytes);
  if (int rc = saber_iu8_pack_read(pk, li.w_record, frag12.data(), li.w_bytes)) return rc;
  if (int rc = saber_iu8_pack_read(pk, li.s_record, ws, (uint64_t)li.n * 4)) return rc;
  return li.wkind == SABER_IU8_W8 ? saber_iu8_repack_w8_from_gfx12(frag12.data(), li.n, li.k, w_gfx950)
                                  : saber_iu8_repack_w4_from_gfx12(frag12.data(), li.n, li.k, w_gfx950);
}
