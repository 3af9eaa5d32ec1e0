"""GGUF reader: the cases the reference's own reader tests hold
(crates/infr-gguf/src/lib.rs:1088-1953; crates/infr-core/src/gguf_split.rs:94-152), rebuilt here as
byte fixtures assembled with ``struct`` so the expected layout is stated independently of the
package's fixture writer, plus the writer checked against those hand-built bytes."""
import os
import struct

import numpy as np
import pytest

import infr_amd.gguf as G
from infr_amd import InfrError, Status

MAGIC = 0x46554747
SPLIT_NO, SPLIT_COUNT, SPLIT_TENSORS = "split.no", "split.count", "split.tensors.count"


def u32(v):
    return struct.pack("<I", v)


def u64(v):
    return struct.pack("<Q", v)


def gstr(s):
    raw = s.encode() if isinstance(s, str) else s
    return u64(len(raw)) + raw


def header(n_tensors, n_kv, version=3):
    return u32(MAGIC) + u32(version) + u64(n_tensors) + u64(n_kv)


def pad32(b):
    return b + bytes(-len(b) % 32)


def fixture():
    """lib.rs:1040-1075: two KVs, one F32[4] tensor at offset 0."""
    b = header(1, 2)
    b += gstr("test.block_count") + u32(4) + u32(30)
    b += gstr("general.architecture") + u32(8) + gstr("diffusion-gemma")
    b += gstr("tensor0") + u32(1) + u64(4) + u32(0) + u64(0)
    return pad32(b) + bytes(16)


def typed_fixture(ggml_type, dim0, data_len):
    """lib.rs:1482-1498."""
    b = header(1, 0) + gstr("tensor0") + u32(1) + u64(dim0) + u32(ggml_type) + u64(0)
    return pad32(b) + bytes(data_len)


def split_shard(split_no, split_count, tensors_total, tensors):
    """lib.rs:1601-1656: F32 tensors, split.* as UINT16/UINT16/INT32, architecture on shard 1 only."""
    first = split_no == 0
    b = header(len(tensors), 4 if first else 3)
    if first:
        b += gstr("general.architecture") + u32(8) + gstr("shardtest")
    b += gstr(SPLIT_NO) + u32(2) + struct.pack("<H", split_no)
    b += gstr(SPLIT_COUNT) + u32(2) + struct.pack("<H", split_count)
    b += gstr(SPLIT_TENSORS) + u32(5) + u32(tensors_total)
    off = 0
    for name, vals in tensors:
        b += gstr(name) + u32(1) + u64(len(vals)) + u32(0) + u64(off)
        off += -(-len(vals) * 4 // 32) * 32
    b = pad32(b)
    for _, vals in tensors:
        b += pad32(struct.pack(f"<{len(vals)}f", *vals))
    return b


def write(tmp_path, data, name="f.gguf"):
    p = tmp_path / name
    p.write_bytes(data)
    return p


def write_shard_set(tmp_path, shards):
    total = len(shards)
    return [write(tmp_path, b, f"m-Q4_K_M-{i + 1:05d}-of-{total:05d}.gguf") for i, b in enumerate(shards)]


def two_shards(tmp_path):
    return write_shard_set(tmp_path, [
        split_shard(0, 2, 3, [("a", [1.0, 2.0, 3.0, 4.0]), ("b", [5.0, 6.0])]),
        split_shard(1, 2, 3, [("c", [7.0, 8.0, 9.0])]),
    ])


def open_err(path, status=Status.Loader):
    with pytest.raises(InfrError) as e:
        G.Gguf.open(path)
    assert e.value.status == status, e.value
    return e.value.msg


def f32s(a):
    return np.frombuffer(bytes(a), "<f4").tolist()


# ── single file ──────────────────────────────────────────────────────────────────────────────

def test_fixture_round_trip(tmp_path):
    data = fixture()
    with G.Gguf.open(write(tmp_path, data)) as g:
        md = g.metadata()
        assert md.u64("test.block_count") == 30
        assert md.str("general.architecture") == "diffusion-gemma"
        assert md.keys() == ["test.block_count", "general.architecture"]
        assert md.u64("general.architecture") is None and md.str("test.block_count") is None
        assert md.get("absent") is None and md.kind("absent") is None
        (t,) = g.tensors()
        assert (t.name, t.dtype, t.shape, t.nbytes) == ("tensor0", 0, (4,), 16)
        assert g.tensor_bytes("tensor0").size == 16
        assert g.chat_template() is None


def test_mapping_reads_the_file_bytes(tmp_path):
    data = bytearray(fixture())
    data[-16:] = bytes(range(1, 17))
    p = write(tmp_path, bytes(data))
    with G.Gguf.open(p) as g:
        assert bytes(g.tensor_bytes("tensor0")) == bytes(range(1, 17))
        off, n = g.tensor_file_range("tensor0")
        assert (off, n) == (len(data) - 16, 16) and off % 32 == 0
        assert g.shards() == [(str(p), len(data))]
        with open(g.shards()[0][0], "rb") as f:
            f.seek(off)
            assert f.read(n) == bytes(g.tensor_bytes("tensor0"))
        with pytest.raises(InfrError):
            g.tensor_file_range("nope")
        with pytest.raises(InfrError, match="tensor not found"):
            g.tensor_bytes("nope")


def test_not_a_gguf_and_bad_version(tmp_path):
    assert "magic" in open_err(write(tmp_path, b"GGUX" + bytes(28)))
    assert "version 1" in open_err(write(tmp_path, u32(MAGIC) + u32(1) + u64(0) + u64(0)))
    open_err(write(tmp_path, b""))                       # empty file: EOF on the magic
    open_err(write(tmp_path, u32(MAGIC) + u32(3)))       # truncated header
    open_err(tmp_path / "missing.gguf", Status.Io)
    with G.Gguf.open(write(tmp_path, u32(MAGIC) + u32(2) + u64(0) + u64(0))) as g:  # version 2 opens
        assert g.tensors() == []


def test_oversized_string_length(tmp_path):
    open_err(write(tmp_path, header(0, 1) + u64(2**64 - 1)))


def test_invalid_utf8_key(tmp_path):
    assert "UTF-8" in open_err(write(tmp_path, header(0, 1) + gstr(b"\xff\xfe") + u32(4) + u32(1)))
    assert "UTF-8" in open_err(write(tmp_path, header(0, 1) + gstr(b"\xed\xa0\x80") + u32(4) + u32(1)))  # surrogate
    assert "UTF-8" in open_err(write(tmp_path, header(0, 1) + gstr(b"\xc0\xaf") + u32(4) + u32(1)))      # overlong
    with G.Gguf.open(write(tmp_path, header(0, 1) + gstr("clé-漢-\U0001f600") + u32(4) + u32(1))) as g:
        assert g.metadata().keys() == ["clé-漢-\U0001f600"]


@pytest.mark.parametrize("vtype,payload,frag", [
    (4, u32(0), "general.alignment 0"),
    (4, u32(33), "general.alignment 33"),
])
def test_bad_alignment(tmp_path, vtype, payload, frag):
    assert frag in open_err(write(tmp_path, header(0, 1) + gstr("general.alignment") + u32(vtype) + payload))


def test_oversized_alignment(tmp_path):
    msg = open_err(write(tmp_path, header(0, 1) + gstr("general.alignment") + u32(10) + u64(1 << 62)))
    assert str(1 << 62) in msg and str(16 << 20) in msg


def test_alignment_moves_the_data_region(tmp_path):
    b = header(1, 1) + gstr("general.alignment") + u32(4) + u32(256)
    b += gstr("t") + u32(1) + u64(2) + u32(0) + u64(0)
    b += bytes(-len(b) % 256) + struct.pack("<2f", 1.5, -2.0)
    with G.Gguf.open(write(tmp_path, b)) as g:
        assert g.tensor_file_range("t") == (256, 8)
        assert f32s(g.tensor_bytes("t")) == [1.5, -2.0]


def test_n_dims(tmp_path):
    b = header(1, 0) + gstr("tensor0") + u32(5) + u64(2) * 5 + u32(0) + u64(0)
    msg = open_err(write(tmp_path, b))
    assert "tensor0" in msg and "5" in msg
    b = header(1, 0) + gstr("tensor0") + u32(4) + u64(4) + u64(1) * 3 + u32(0) + u64(0)
    with G.Gguf.open(write(tmp_path, pad32(b) + bytes(16))) as g:
        assert g.tensors()[0].shape == (4, 1, 1, 1)


def test_duplicate_tensor_name(tmp_path):
    b = header(2, 0)
    for off in (0, 16):
        b += gstr("tensor0") + u32(1) + u64(4) + u32(0) + u64(off)
    msg = open_err(write(tmp_path, pad32(b) + bytes(32)))
    assert "tensor0" in msg and "duplicate" in msg


def test_huge_counts(tmp_path):
    open_err(write(tmp_path, header(2**64 - 1, 0)))
    open_err(write(tmp_path, header(0, 2**64 - 1)))
    # an array that claims 2^60 elements on a 60-byte file fails on the read, not on a reservation
    open_err(write(tmp_path, header(0, 1) + gstr("a") + u32(9) + u32(4) + u64(1 << 60)))


def test_array_nesting(tmp_path):
    b = header(0, 1) + gstr("bomb") + u32(9)
    b += (u32(9) + u64(1)) * 8192 + u32(0) + u64(0)
    assert "nesting" in open_err(write(tmp_path, b))
    b = header(0, 1) + gstr("nested") + u32(9) + u32(9) + u64(2)
    b += (u32(4) + u64(1) + u32(7)) * 2
    with G.Gguf.open(write(tmp_path, b)) as g:
        assert g.metadata().get("nested") == [[7], [7]]
        assert g.metadata().kind("nested") == G.ARR
    # exactly 64 levels parse, 65 do not
    for depth, ok in ((64, True), (65, False)):
        b = header(0, 1) + gstr("deep") + u32(9) + (u32(9) + u64(1)) * (depth - 1) + u32(0) + u64(0)
        p = write(tmp_path, b)
        if ok:
            G.Gguf.open(p).close()
        else:
            assert "nesting" in open_err(p)


def test_every_value_type(tmp_path):
    kv = [
        ("u8", 0, struct.pack("<B", 200), 200), ("i8", 1, struct.pack("<b", -5), -5),
        ("u16", 2, struct.pack("<H", 60000), 60000), ("i16", 3, struct.pack("<h", -300), -300),
        ("u32", 4, u32(4_000_000_000), 4_000_000_000), ("i32", 5, struct.pack("<i", -7), -7),
        ("f32", 6, struct.pack("<f", 0.5), 0.5), ("t", 7, b"\x01", True), ("f", 7, b"\x00", False),
        ("s", 8, gstr("hé"), "hé"), ("u64", 10, u64(2**63 + 1), 2**63 + 1),
        ("i64", 11, struct.pack("<q", -2**62), -2**62), ("f64", 12, struct.pack("<d", 1e-300), 1e-300),
        ("arr", 9, u32(8) + u64(2) + gstr("a") + gstr(""), ["a", ""]),
    ]
    b = header(0, len(kv)) + b"".join(gstr(k) + u32(t) + p for k, t, p, _ in kv)
    with G.Gguf.open(write(tmp_path, b)) as g:
        md = g.metadata()
        for k, _, _, want in kv:
            assert md.get(k) == want, k
        # as_u64 takes a non-negative I64 and refuses a negative one (loader.rs:20-29)
        assert md.u64("i8") is None and md.u64("u8") == 200
        assert md.f64("i32") == -7.0 and md.f64("u16") == 60000.0 and md.f64("s") is None
        assert md.kind("f32") == G.F64 and md.kind("i16") == G.I64 and md.kind("u16") == G.U64
    assert "unknown value type 13" in open_err(write(tmp_path, header(0, 1) + gstr("x") + u32(13) + u32(0)))
    b = header(0, 2) + gstr("k") + u32(4) + u32(1) + gstr("k") + u32(4) + u32(2)  # a repeated key keeps the last
    with G.Gguf.open(write(tmp_path, b)) as g:
        assert g.metadata().u64("k") == 2 and g.metadata().keys() == ["k"]
    b = header(0, 1) + gstr("general.alignment") + u32(5) + struct.pack("<i", 64)  # non-negative I32 counts
    G.Gguf.open(write(tmp_path, b)).close()


def test_chat_template(tmp_path):
    b = header(0, 1) + gstr("tokenizer.chat_template") + u32(8) + gstr("{{ messages }}")
    with G.Gguf.open(write(tmp_path, b)) as g:
        assert g.chat_template() == "{{ messages }}"


# ── block geometry ───────────────────────────────────────────────────────────────────────────

def test_byte_count_overflow(tmp_path):
    open_err(write(tmp_path, typed_fixture(0, 1 << 62, 0)))
    b = header(1, 0) + gstr("t") + u32(2) + u64(1 << 40) + u64(1 << 40) + u32(0) + u64(0)
    assert "overflows" in open_err(write(tmp_path, b))


def test_quant_numel_must_be_whole_blocks(tmp_path):
    msg = open_err(write(tmp_path, typed_fixture(12, 100, 144)))
    assert "tensor0" in msg and "256" in msg
    with G.Gguf.open(write(tmp_path, typed_fixture(12, 256, 144))) as g:
        t = g.tensors()[0]
        assert (t.dtype, t.nbytes) == (12, 144) and g.tensor_bytes("tensor0").size == 144
    msg = open_err(write(tmp_path, typed_fixture(36, 3, 64)))
    assert "tensor0" in msg and "i2_s" in msg
    with G.Gguf.open(write(tmp_path, typed_fixture(36, 64, 32))) as g:  # 64/4 codes + one f32 scale
        assert g.tensors()[0].nbytes == 20
    assert "ggml type 99" in open_err(write(tmp_path, typed_fixture(99, 4, 16)), Status.Unsupported)
    assert "ggml type 4" in open_err(write(tmp_path, typed_fixture(4, 32, 32)), Status.Unsupported)


def test_i32_table_reads_back(tmp_path):
    ids = [0, 1, -1, 255, -2**31, 2**31 - 1]
    b = bytearray(typed_fixture(26, len(ids), 4 * len(ids)))
    b[-4 * len(ids):] = struct.pack("<6i", *ids)
    with G.Gguf.open(write(tmp_path, bytes(b))) as g:
        t = g.tensors()[0]
        assert (t.dtype, t.shape, t.nbytes) == (26, (6,), 24)
        assert np.frombuffer(bytes(g.tensor_bytes("tensor0")), "<i4").tolist() == ids


def test_tensor_past_the_end_of_the_file(tmp_path):
    # open() does not check extents (a directory may be read without the data); the access does
    with G.Gguf.open(write(tmp_path, typed_fixture(12, 512, 144))) as g:
        assert g.tensors()[0].nbytes == 288
        with pytest.raises(InfrError, match="exceeds"):
            g.tensor_bytes("tensor0")
    b = header(1, 0) + gstr("t") + u32(1) + u64(4) + u32(0) + u64(2**62)
    with G.Gguf.open(write(tmp_path, pad32(b) + bytes(16))) as g:
        with pytest.raises(InfrError, match="exceeds"):
            g.tensor_bytes("t")
    # an offset that wraps once the data region's start is added is refused at open (lib.rs:652-656)
    b = header(1, 0) + gstr("t") + u32(1) + u64(4) + u32(0) + u64(2**64 - 8)
    assert "overflows" in open_err(write(tmp_path, pad32(b) + bytes(16)))


# The defining formulas of ggml's type_size for every type id the reader maps
# (crates/infr-core/src/decode_spec.rs:455-490), so a typo in the table cannot pass.
QK = 256
FORMULAS = {
    0: (1, 4), 1: (1, 2), 30: (1, 2), 26: (1, 4),
    2: (32, 2 + 16), 3: (32, 2 + 2 + 16), 6: (32, 2 + 4 + 16), 7: (32, 2 + 2 + 4 + 16), 8: (32, 2 + 32),
    10: (QK, 2 * 2 + QK // 16 + QK // 4), 11: (QK, 2 + QK // 4 + QK // 8 + 12),
    12: (QK, 2 * 2 + 12 + QK // 2), 13: (QK, 2 * 2 + 12 + QK // 8 + QK // 2),
    14: (QK, QK // 2 + QK // 4 + QK // 16 + 2),
    19: (QK, 2 + QK // 8 + QK // 32 * 2), 29: (QK, QK // 8 + QK // 16 + QK // 32),
    16: (QK, 2 + QK // 8 * 2), 17: (QK, 2 + QK // 8 * 2 + QK // 32), 22: (QK, 2 + QK // 4 + QK // 16),
    18: (QK, 2 + 3 * (QK // 8)), 21: (QK, 2 + 13 * (QK // 32) + QK // 64), 20: (32, 2 + 16),
    23: (QK, 2 + 2 + QK // 64 + QK // 2), 34: (QK, 2 + QK // 64 + (QK - 4 * QK // 64) // 5),
    35: (QK, 2 + QK // 4), 42: (64, 2 + 64 // 4), 39: (32, 1 + 16), 40: (64, 4 + 32), 36: (4, 1),
}


def test_block_layout_table():
    for t, want in FORMULAS.items():
        assert G.block_layout(t) == want, t
    for t in set(range(64)) - set(FORMULAS):
        with pytest.raises(InfrError):
            G.block_layout(t)
    assert G.nbytes(12, 0) == 0 and G.nbytes(12, 256) == 144 and G.nbytes(12, 2048) == 8 * 144
    assert G.nbytes(0, 7) == 28
    assert G.nbytes(12, 100) == 144          # rounds UP, never short (lib.rs:373-385)
    assert G.nbytes(36, 64) == 16 + 4
    with pytest.raises(InfrError):
        G.nbytes(0, 2**63)


# ── shard names ──────────────────────────────────────────────────────────────────────────────

def test_parse_shard():
    s = G.parse_shard("model-Q4_K_M-00001-of-00003.gguf")
    assert (s.base, s.index, s.total, s.width) == ("model-Q4_K_M", 1, 3, 5)
    assert G.parse_shard("m-00003-of-00005.gguf").index == 3
    assert G.parse_shard("m-00003-of-00005.GGUF").total == 5
    for bad in ("model-Q4_K_M.gguf", "m-1-of-003.gguf", "m-000ab-of-00003.gguf", "m-00001-of-00002.bin",
                "m-Q4_K_M-0000000001-of-4294967295.gguf", "m-000001-of-999999.gguf", "-of-.gguf", ".gguf", ""):
        assert G.parse_shard(bad) is None, bad
    assert G.parse_shard("m-99999-of-99999.gguf").total == 99999
    assert G.parse_shard("m-01-of-12.gguf").total == 12


def test_shard_set():
    assert G.shard_set("m-Q4_K_M-00001-of-00003.gguf") == [
        "m-Q4_K_M-00001-of-00003.gguf", "m-Q4_K_M-00002-of-00003.gguf", "m-Q4_K_M-00003-of-00003.gguf"]
    assert G.shard_set("m-Q4_K_M-00002-of-00002.gguf")[0] == "m-Q4_K_M-00001-of-00002.gguf"
    assert G.shard_set("plain.gguf") == ["plain.gguf"]
    assert G.shard_set("m-0-of-0.gguf") == ["m-0-of-0.gguf"]
    assert len(G.shard_set("m-01-of-12.gguf")) == 12 and G.shard_set("m-01-of-12.gguf")[11] == "m-12-of-12.gguf"


# ── shard sets ───────────────────────────────────────────────────────────────────────────────

def test_shard_set_reads_each_tensor_from_its_own_file(tmp_path):
    paths = two_shards(tmp_path)
    with G.Gguf.open(paths[0]) as g:
        assert g.metadata().str("general.architecture") == "shardtest"
        assert [t.name for t in g.tensors()] == ["a", "b", "c"]
        assert f32s(g.tensor_bytes("a")) == [1.0, 2.0, 3.0, 4.0]
        assert f32s(g.tensor_bytes("b")) == [5.0, 6.0]
        assert f32s(g.tensor_bytes("c")) == [7.0, 8.0, 9.0]
        len1, len2 = os.path.getsize(paths[0]), os.path.getsize(paths[1])
        assert g.shards() == [(str(paths[0]), len1), (str(paths[1]), len2)]
        off, n = g.tensor_file_range("c")
        assert n == 12 and off >= len1
        # a second reader that lays the files end to end finds the same bytes at the reported ranges
        blob = paths[0].read_bytes() + paths[1].read_bytes()
        for name in "abc":
            off, n = g.tensor_file_range(name)
            assert blob[off:off + n] == bytes(g.tensor_bytes(name))


def test_opening_a_later_shard_loads_the_whole_model(tmp_path):
    paths = two_shards(tmp_path)
    with G.Gguf.open(paths[0]) as a, G.Gguf.open(paths[1]) as b:
        assert b.metadata().str("general.architecture") == "shardtest"
        assert len(b.tensors()) == 3 and b.shards() == a.shards()
        for name in "abc":
            assert bytes(a.tensor_bytes(name)) == bytes(b.tensor_bytes(name))
        assert a.tensors() == b.tensors()


def test_missing_shard(tmp_path):
    paths = two_shards(tmp_path)
    os.remove(paths[1])
    msg = open_err(paths[0])
    assert "m-Q4_K_M-00002-of-00002.gguf" in msg and "shard 2 of 2" in msg


def test_shard_set_disagreements(tmp_path):
    d = tmp_path / "no"
    d.mkdir()
    paths = write_shard_set(d, [split_shard(0, 2, 3, [("a", [1.0]), ("b", [2.0])]),
                                split_shard(2, 2, 3, [("c", [3.0])])])
    msg = open_err(paths[0])
    assert "m-Q4_K_M-00002-of-00002.gguf" in msg and SPLIT_NO in msg and "shard 2 of 2" in msg

    d = tmp_path / "count"
    d.mkdir()
    paths = write_shard_set(d, [split_shard(0, 2, 3, [("a", [1.0]), ("b", [2.0])]),
                                split_shard(1, 5, 3, [("c", [3.0])])])
    msg = open_err(paths[0])
    assert "m-Q4_K_M-00002-of-00002.gguf" in msg and SPLIT_COUNT in msg and "5" in msg

    d = tmp_path / "total"
    d.mkdir()
    paths = write_shard_set(d, [split_shard(0, 7, 3, [("a", [1.0]), ("b", [2.0])]),
                                split_shard(1, 7, 3, [("c", [3.0])])])
    msg = open_err(paths[0])
    assert "m-Q4_K_M-00001-of-00002.gguf" in msg and "7" in msg

    msg = open_err(write(tmp_path, split_shard(0, 2, 3, [("a", [1.0])]), "renamed.gguf"))
    assert "renamed.gguf" in msg and "gguf-split" in msg

    d = tmp_path / "tensors"
    d.mkdir()
    paths = write_shard_set(d, [split_shard(0, 2, 4, [("a", [1.0]), ("b", [2.0])]),
                                split_shard(1, 2, 4, [("c", [3.0])])])
    msg = open_err(paths[0])
    assert SPLIT_TENSORS in msg and "4" in msg and "3" in msg

    d = tmp_path / "dup"
    d.mkdir()
    paths = write_shard_set(d, [split_shard(0, 2, 3, [("a", [1.0]), ("b", [2.0])]),
                                split_shard(1, 2, 3, [("a", [3.0])])])
    assert "duplicate tensor name 'a'" in open_err(paths[0])


def test_split_model_without_a_tensor_total(tmp_path):
    b = header(0, 2) + gstr(SPLIT_NO) + u32(2) + struct.pack("<H", 0) + gstr(SPLIT_COUNT) + u32(2) + \
        struct.pack("<H", 2)
    paths = write_shard_set(tmp_path, [b, split_shard(1, 2, 0, [])])
    assert SPLIT_TENSORS in open_err(paths[0])


def test_shard_index_outside_its_set(tmp_path):
    for name, shown in (("m-00000-of-00002.gguf", "numbered 0 of 2"), ("m-00003-of-00002.gguf", "numbered 3 of 2")):
        msg = open_err(write(tmp_path, split_shard(0, 2, 1, [("a", [1.0])]), name))
        assert name in msg and shown in msg


def test_shard_shaped_name_without_split_metadata_is_one_file(tmp_path):
    with G.Gguf.open(write(tmp_path, fixture(), "m-00001-of-00003.gguf")) as g:
        assert len(g.tensors()) == 1 and len(g.shards()) == 1
    # split.count = 1 names this file and nothing else (lib.rs:479-484)
    b = header(0, 1) + gstr(SPLIT_COUNT) + u32(2) + struct.pack("<H", 1)
    with G.Gguf.open(write(tmp_path, b, "anything.gguf")) as g:
        assert len(g.shards()) == 1


# ── the package's fixture writer against the hand-built bytes ────────────────────────────────

def test_writer_reproduces_the_hand_built_fixture():
    got = G.gguf_bytes({"test.block_count": 30, "general.architecture": "diffusion-gemma"},
                       [("tensor0", (4,), 0, bytes(16))])
    assert got == fixture()
    got = G.gguf_bytes({}, [("tensor0", (256,), 12, bytes(144))])
    assert got == typed_fixture(12, 256, 144)


def test_writer_round_trip_with_quant_tensors(tmp_path):
    from infr_amd import DType, synth_weight
    w4 = synth_weight(DType.Q4K, 3, 8, 512)
    w6 = synth_weight(DType.Q6K, 4, 5, 256)
    w8 = synth_weight(DType.Q8_0, 5, 3, 96)
    p = tmp_path / "w.gguf"
    G.write_gguf(p, {"general.architecture": "qwen3", "qwen3.block_count": 1, "f": 1.5, "flag": True,
                     "names": ["a", "b"], "big": 2**40, "neg": -3},
                 [("blk.0.ffn_up.weight", (512, 8), 12, w4), ("blk.0.ffn_down.weight", (256, 5), 14, w6),
                  ("output.weight", (96, 3), 8, w8)], alignment=64)
    with G.Gguf.open(p) as g:
        md = g.metadata()
        assert md.get("names") == ["a", "b"] and md.u64("big") == 2**40 and md.get("neg") == -3
        assert md.get("f") == 1.5 and md.get("flag") is True and md.u64("general.alignment") == 64
        ts = {t.name: t for t in g.tensors()}
        assert ts["blk.0.ffn_up.weight"].shape == (512, 8) and ts["blk.0.ffn_up.weight"].nbytes == w4.size
        for name, w in (("blk.0.ffn_up.weight", w4), ("blk.0.ffn_down.weight", w6), ("output.weight", w8)):
            assert np.array_equal(g.tensor_bytes(name), w)
            assert g.tensor_file_range(name)[0] % 64 == 0
        assert g.tensor("output.weight").dtype == 8
        with pytest.raises(InfrError):
            g.tensor("nope")
        view = g.tensor_bytes("output.weight")
        with pytest.raises(ValueError):
            view[0] = 1                                   # the mapping is read-only


def test_closed_handle_is_refused(tmp_path):
    g = G.Gguf.open(write(tmp_path, fixture()))
    g.close()
    g.close()
    with pytest.raises(InfrError):
        g.tensors()
