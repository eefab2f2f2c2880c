"""A minimal writer of the tier-pack byte layout for the reader's tests, from the format's own
description (include/saber_abi.h:541-944) and the placement the reference's writer test expects
(tools/pack/tests/test_build_pack.py:146-196: the chunk-digest blob right after the name blob, the
chunk flag on records longer than one chunk). Python's hashlib and struct only: nothing of the
library under test is used to build the file."""
import hashlib
import struct

ALIGN = 4096
DT = dict(U8=0, I8=1, U16=2, I16=3, U32=4, I32=5, U64=6, I64=7, F16=8, BF16=9, F32=10, F64=11, F8E4M3=12, F8E5M2=13,
          FP4E2M1X2=14, BOOL=15, E8M0=16)


def align_up(x):
    return (x + ALIGN - 1) // ALIGN * ALIGN


def build(records, version=2, tp_size=1, rank=0, plan_hash=b"P" * 32, tier_id=b"T" * 32, chunk_bytes=4096, seconds=123):
    """records: list of dict(name, dtype (tag name), shape, layout_id, shard_kind, data (bytes)). -> file bytes."""
    n = len(records)
    table_off, name_blob_off = 256, 256 + 160 * n
    names = b""
    name_offs = []
    for r in records:
        nb = r["name"].encode()
        names += struct.pack("<H", len(nb))
        name_offs.append(len(names))
        names += nb
    chunked = [version >= 2 and len(r["data"]) > chunk_bytes for r in records]
    blob = b""
    for r, c in zip(records, chunked):
        if not c:
            continue
        d = r["data"]
        nch = -(-len(d) // chunk_bytes)
        blob += struct.pack("<II", nch, 0) + hashlib.sha256(d).digest()
        for i in range(nch):
            blob += hashlib.sha256(d[i * chunk_bytes:(i + 1) * chunk_bytes]).digest()
    names_end = name_blob_off + len(names)
    meta_end = names_end + len(blob)
    data_off = align_up(meta_end)
    cursor = data_off
    table = b""
    payload = b""
    for r, noff, c in zip(records, name_offs, chunked):
        d = r["data"]
        shape = list(r["shape"]) + [0] * (8 - len(r["shape"]))
        table += struct.pack("<IIIIHBBIQQ8Q", noff, len(r["name"].encode()), rank, r.get("layout_id", 0), DT[r["dtype"]],
                             len(r["shape"]), r.get("shard_kind", 0), 1 if c else 0, cursor, len(d), *shape)
        table += hashlib.sha256(d).digest() + bytes(24)
        payload += d + bytes(align_up(len(d)) - len(d))
        cursor += align_up(len(d))
    file_bytes = cursor
    head = b"SBRPACK1" + struct.pack("<IIII", version, 256, 160, n)
    head += struct.pack("<QQQQQ", table_off, name_blob_off, len(names), data_off, file_bytes)
    head += struct.pack("<IIQ", tp_size, rank, seconds) + plan_hash + tier_id
    head += hashlib.sha256(table + names).digest()
    if version >= 2 and blob:
        head += struct.pack("<QQ", names_end, len(blob)) + hashlib.sha256(blob).digest() + struct.pack("<I", chunk_bytes)
    else:
        head += bytes(16 + 32 + 4)
    head += bytes(28)
    assert len(head) == 256
    meta = head + table + names + blob
    return meta + bytes(data_off - len(meta)) + payload


def rehash_table(raw):
    """Recompute the header's table hash after an edit of the table or the names (for tests that aim at
    a structural rule behind it)."""
    raw = bytearray(raw)
    n = struct.unpack_from("<I", raw, 20)[0]
    nbo, nbb = struct.unpack_from("<QQ", raw, 32)
    raw[144:176] = hashlib.sha256(bytes(raw[256:nbo + nbb])).digest()
    return bytes(raw)
