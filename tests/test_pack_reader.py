"""The tier-pack reader (include/saber_iu8.h `saber_iu8_pack_*`; the reference's
crates/saber-mem/src/pack/reader.rs) against packs written by an independent writer
(tests/pack_writer.py): round trips, the iu8 records of a linear repacked to the gfx950 order, and
one negative control per open-time rule."""
import ctypes
import hashlib
import struct

import numpy as np
import pytest

from oracle import ref
from saber_engine_amd import iu8, synth
from saber_engine_amd.pack import Pack
from tests import pack_writer as pw


def gfx12_w4(codes):
    """int4 codes [N, K] -> the reference's layout-17 bytes, by the oracle's address function."""
    L = ref.lib()
    N, K = codes.shape
    out = np.zeros(N * K // 2, np.uint8)
    for n in range(N):
        for k in range(K):
            nib = ctypes.c_uint32()
            off = L.w4a8_w4_frag_gfx12(n, k, K, ctypes.byref(nib))
            out[off] |= (int(codes[n, k]) & 15) << (4 * nib.value)
    return out


def gfx12_w8(w8):
    L = ref.lib()
    N, K = w8.shape
    out = np.zeros(N * K, np.uint8)
    for n in range(N):
        for k in range(K):
            out[L.w4a8_a_tiled_gfx12(n, k, K)] = w8[n, k].view(np.uint8)
    return out


@pytest.fixture(scope="module")
def case():
    rng = np.random.default_rng(11)
    N, K = 48, 256
    codes = rng.integers(-8, 8, (N, K), dtype=np.int8)
    w8 = rng.integers(-127, 128, (32, 128), dtype=np.int8)
    s4 = (np.abs(rng.standard_normal(N)) * 0.02 + 1e-4).astype(np.float32)
    s8 = (np.abs(rng.standard_normal(32)) * 0.02 + 1e-4).astype(np.float32)
    recs = [
        dict(name="tok.embed", dtype="BF16", shape=[5, 3], data=bytes(range(30))),
        dict(name="L0.down.wi4", dtype="U8", shape=[N // 16, K * 8], layout_id=17, shard_kind=2, data=gfx12_w4(codes).tobytes()),
        dict(name="L0.down.wi4s", dtype="F32", shape=[N], layout_id=19, data=s4.tobytes()),
        dict(name="L0.o.wi8", dtype="U8", shape=[2, 128 * 16], layout_id=18, shard_kind=2, data=gfx12_w8(w8).tobytes()),
        dict(name="L0.o.wi8s", dtype="F32", shape=[32], layout_id=19, data=s8.tobytes()),
        dict(name="fp4", dtype="FP4E2M1X2", shape=[7, 3], data=bytes(11)),            # 21 nibbles -> 11 bytes
    ]
    return dict(recs=recs, codes=codes, w8=w8, s4=s4, s8=s8)


def write(tmp_path, raw, name="rank0.pack"):
    p = tmp_path / name
    p.write_bytes(raw)
    return str(p)


@pytest.mark.parametrize("version", [1, 2])
def test_round_trip_and_linear_load(tmp_path, case, version):
    raw = pw.build(case["recs"], version=version, tp_size=2, rank=1)
    with Pack(write(tmp_path, raw)) as pk:
        h = pk.header
        assert (h.format_version, h.record_count, h.tp_size, h.rank) == (version, 6, 2, 1)
        assert bytes(h.plan_hash) == b"P" * 32 and bytes(h.tier_id) == b"T" * 32 and h.file_bytes == len(raw)
        assert h.chunk_bytes == (4096 if version == 2 else 0)
        for i, r in enumerate(case["recs"]):
            got = pk.record(i)
            assert got.name.decode() == r["name"] and got.length == len(r["data"]) and got.rank == 1
            assert list(got.shape)[:got.ndim] == r["shape"] and got.layout_id == r.get("layout_id", 0)
            assert bytes(got.sha256) == hashlib.sha256(r["data"]).digest()
            assert got.flags == (1 if version == 2 and len(r["data"]) > 4096 else 0)
            assert pk.find(r["name"]) == i
            assert pk.read(i).tobytes() == r["data"]
        assert pk.find("absent") == -1
        li = pk.linear("L0.down")
        assert (li.wkind, li.n, li.k, li.w_bytes, li.shard_kind) == (iu8.W4, 48, 256, 48 * 128, 2)
        wk, n, k, w, ws = pk.load_linear("L0.down")
        np.testing.assert_array_equal(w, iu8.repack_w4(synth.pack_w4(case["codes"])))      # the direct repack
        np.testing.assert_array_equal(ws, case["s4"])
        wk, n, k, w, ws = pk.load_linear("L0.o")
        assert (wk, n, k) == (iu8.W8, 32, 128)
        np.testing.assert_array_equal(w, iu8.repack_w8(case["w8"]))
        np.testing.assert_array_equal(ws, case["s8"])
        with pytest.raises(iu8.IU8Error) as e:
            pk.linear("L0.gate_up")
        assert e.value.code == iu8.E_RULE
    with Pack(write(tmp_path, raw), expected_plan_hash=b"P" * 32):
        pass
    with pytest.raises(iu8.IU8Error) as e:
        Pack(write(tmp_path, raw), expected_plan_hash=b"Q" * 32)          # refused, never re-derived
    assert e.value.code == iu8.E_VALIDATE and "plan hash" in str(e.value)


def put(raw, off, fmt, *vals):
    b = bytearray(raw)
    struct.pack_into(fmt, b, off, *vals)
    return bytes(b)


REC = 256 + 160          # the second record (L0.down.wi4) of the table


def mutations(raw):
    """(name, bytes, code, a word of the message)"""
    nbo = struct.unpack_from("<Q", raw, 32)[0]
    doff = struct.unpack_from("<Q", raw, REC + 24)[0]
    fix = pw.rehash_table
    yield "magic", b"SBRPACK2" + raw[8:], iu8.E_PARSE, "magic"
    yield "version", put(raw, 8, "<I", 3), iu8.E_PARSE, "version"
    yield "header size", put(raw, 12, "<I", 512), iu8.E_PARSE, "header_bytes"
    yield "record size", put(raw, 16, "<I", 168), iu8.E_PARSE, "record_bytes"
    yield "header reserved", put(raw, 250, "<B", 1), iu8.E_PARSE, "reserved"
    yield "table_off", put(raw, 24, "<Q", 512), iu8.E_PARSE, "table_off"
    yield "name_blob_off", put(raw, 32, "<Q", nbo + 8), iu8.E_PARSE, "name_blob_off"
    yield "data_off alignment", put(raw, 48, "<Q", 4100), iu8.E_PARSE, "aligned"
    yield "data_off inside the metadata", put(raw, 48, "<Q", 0), iu8.E_PARSE, "overlaps"
    yield "file_bytes", put(raw, 56, "<Q", len(raw) + 4096), iu8.E_PARSE, "file_bytes"
    yield "truncated", raw[:-4096], iu8.E_PARSE, "file_bytes"
    yield "rank", put(raw, 68, "<I", 9), iu8.E_PARSE, "rank"
    yield "chunk blob offset", put(raw, 176, "<Q", nbo), iu8.E_PARSE, "chunk_blob_off"
    yield "chunk size", put(raw, 224, "<I", 1000), iu8.E_PARSE, "chunk_bytes"
    yield "chunk blob hash", put(raw, 192, "<B", raw[192] ^ 1), iu8.E_PARSE, "chunk blob hashes"
    yield "record flags", fix(put(raw, REC + 20, "<I", 4)), iu8.E_PARSE, "flags"
    yield "record reserved", fix(put(raw, REC + 140, "<B", 1)), iu8.E_PARSE, "reserved"
    yield "ndim", fix(put(raw, REC + 18, "<B", 0)), iu8.E_PARSE, "ndim"
    yield "shape beyond ndim", fix(put(raw, REC + 40 + 16, "<Q", 1)), iu8.E_PARSE, "beyond ndim"
    yield "zero extent", fix(put(raw, REC + 40, "<Q", 0)), iu8.E_PARSE, "zero"
    yield "dtype", fix(put(raw, REC + 16, "<H", 40)), iu8.E_PARSE, "dtype"
    yield "shard kind", fix(put(raw, REC + 19, "<B", 7)), iu8.E_PARSE, "shard"
    yield "name prefix", fix(put(raw, REC + 4, "<I", 10)), iu8.E_PARSE, "prefix"
    yield "record rank", fix(put(raw, REC + 8, "<I", 0)), iu8.E_PARSE, "rank"
    yield "record alignment", fix(put(raw, REC + 24, "<Q", doff + 8)), iu8.E_PARSE, "aligned"
    yield "records out of order", fix(put(raw, REC + 24, "<Q", doff - 4096)), iu8.E_PARSE, "sorted"
    yield "length against shape", fix(put(raw, REC + 32, "<Q", 48 * 128 - 1)), iu8.E_PARSE, "imply"
    yield "past the file", fix(put(raw, REC + 24, "<Q", len(raw))), iu8.E_PARSE, "past"
    yield "data_off + length wraps 64 bits", fix(put(raw, REC + 24, "<Q", 2**64 - 4096)), iu8.E_PARSE, "past"
    yield "table hash", put(raw, REC + 12, "<I", 18), iu8.E_VALIDATE, "table hash"
    names = raw.find(b"L0.down.wi4s")                                           # rename to its neighbour's name + pad
    dup = bytearray(raw)
    dup[names - 2:names + 12] = struct.pack("<H", 12) + b"L0.down.wi4\0"
    yield "names: an edited blob without its hash", bytes(dup), iu8.E_VALIDATE, "table hash"


def test_every_open_rule_refuses(tmp_path, case):
    raw = pw.build(case["recs"], version=2, tp_size=2, rank=1)
    n = 0
    for name, bad, code, word in mutations(raw):
        with pytest.raises(iu8.IU8Error) as e:
            Pack(write(tmp_path, bad, "bad.pack"))
        assert e.value.code == code and word in str(e.value), (name, str(e.value))
        n += 1
    assert n == 31


def test_duplicate_names_and_chunk_entries_refuse(tmp_path, case):
    recs = [dict(r) for r in case["recs"]]
    recs[2]["name"] = "L0.down.wi4"
    with pytest.raises(iu8.IU8Error) as e:
        Pack(write(tmp_path, pw.build(recs)))
    assert e.value.code == iu8.E_PARSE and "duplicate" in str(e.value)
    # a chunk entry that names another record's digest, with the blob's own hash made right again
    raw = bytearray(pw.build(case["recs"]))
    cbo, cbb = struct.unpack_from("<QQ", raw, 176)
    raw[cbo + 8] ^= 1
    raw[192:224] = hashlib.sha256(bytes(raw[cbo:cbo + cbb])).digest()
    with pytest.raises(iu8.IU8Error) as e:
        Pack(write(tmp_path, bytes(raw)))
    assert e.value.code == iu8.E_PARSE and "different record" in str(e.value)
    raw = bytearray(pw.build(case["recs"]))
    struct.pack_into("<I", raw, cbo, 5)                                       # a wrong digest count
    raw[192:224] = hashlib.sha256(bytes(raw[cbo:cbo + cbb])).digest()
    with pytest.raises(iu8.IU8Error) as e:
        Pack(write(tmp_path, bytes(raw)))
    assert "digests" in str(e.value)


def test_a_damaged_payload_is_a_load_error(tmp_path, case):
    raw = bytearray(pw.build(case["recs"]))
    doff = struct.unpack_from("<Q", raw, REC + 24)[0]
    raw[doff + 5000] ^= 0x10                                                   # in the second 4096-byte chunk of the codes
    with Pack(write(tmp_path, bytes(raw))) as pk:                              # opens: payloads are checked when read
        assert pk.read(0).tobytes() == case["recs"][0]["data"]
        with pytest.raises(iu8.IU8Error) as e:
            pk.read(1)
        assert e.value.code == iu8.E_VALIDATE and "chunk 1" in str(e.value)
        with pytest.raises(iu8.IU8Error):
            pk.load_linear("L0.down")
    raw = bytearray(pw.build(case["recs"], version=1))                         # no chunk digests: the record hash catches it
    raw[doff + 5000] ^= 0x10
    with Pack(write(tmp_path, bytes(raw))) as pk:
        with pytest.raises(iu8.IU8Error) as e:
            pk.read(1)
        assert e.value.code == iu8.E_VALIDATE and "hashes to" in str(e.value)


def test_linear_records_must_be_what_the_graph_writes(tmp_path, case):
    for edit, word in [(dict(layout_id=18), "layout-17"), (dict(dtype="I8"), "layout-17"), (dict(shape=[3 * 256 * 8]), "layout-17")]:
        recs = [dict(r) for r in case["recs"]]
        recs[1].update(edit)
        with Pack(write(tmp_path, pw.build(recs))) as pk:
            with pytest.raises(iu8.IU8Error) as e:
                pk.linear("L0.down")
            assert e.value.code == iu8.E_RULE and word in str(e.value)
    recs = [dict(r) for r in case["recs"]]
    recs[2].update(shape=[24, 2])                                              # a scale that is not [N]
    with Pack(write(tmp_path, pw.build(recs))) as pk:
        with pytest.raises(iu8.IU8Error) as e:
            pk.linear("L0.down")
        assert "layout-19" in str(e.value)
    recs = [r for r in case["recs"] if r["name"] != "L0.down.wi4s"]
    with Pack(write(tmp_path, pw.build(recs))) as pk:
        with pytest.raises(iu8.IU8Error) as e:
            pk.linear("L0.down")
        assert "no row scale" in str(e.value)
