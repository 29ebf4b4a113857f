"""The FlatBuffers layer under the dnx / db files against a third-party implementation, and the dnx bytes against the schema.

`denox_amd/csrc/common/flatbuf.hpp` restates the FlatBuffers binary format by hand (the reference writes dnx.fbs / db.fbs
through flatc-generated code and the FlatBuffers library, neither of which is installed here).  Apache Arrow's IPC
metadata *is* FlatBuffers, and pyarrow reads and writes it with the real library and its verifier, so:

  * what the hand-written Builder emits for Arrow's Message / Schema / RecordBatch tables must load in pyarrow with the
    field values that went in (tables, shared vtables, defaults left out, strings, vectors of tables, unions, vectors of
    structs with 8-byte alignment);
  * what pyarrow emits must decode through the hand-written reader to the values pyarrow reports for the same object.

The helper `tests/flatbuf_probe.cpp` is compiled on the fly (g++, a few seconds).  The last tests walk a compiled model's
bytes with a small independent Python decoder that knows only the wire format and the field order of dnx.fbs.
"""
import ctypes
import struct
import subprocess
from pathlib import Path

import numpy as np
import pyarrow as pa
import pytest

import denox_amd as dx
from denox_amd import networks

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def probe(tmp_path_factory):
    out = tmp_path_factory.mktemp("probe") / "libflatbuf_probe.so"
    subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-Werror", str(ROOT / "tests" / "flatbuf_probe.cpp"), "-o", str(out)],
                   check=True, cwd=ROOT)
    L = ctypes.CDLL(str(out))
    L.probe_error.restype = ctypes.c_char_p
    L.probe_text.restype = ctypes.c_char_p
    L.probe_bytes.restype = ctypes.POINTER(ctypes.c_uint8)
    L.probe_size.restype = ctypes.c_size_t
    L.probe_read_message.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
    return L


def _result(L, rc):
    assert rc == 0, L.probe_error().decode()
    return ctypes.string_at(L.probe_bytes(), L.probe_size())


def _encapsulate(meta: bytes, body: bytes = b"") -> bytes:
    # Arrow IPC framing: continuation marker, metadata size (padded to 8), metadata flatbuffer, body
    meta += b"\0" * (-len(meta) % 8)
    return struct.pack("<Ii", 0xFFFFFFFF, len(meta)) + meta + body


def _strs(items):
    arr = (ctypes.c_char_p * len(items))(*[s.encode() for s in items])
    return arr


def _ints(items, ty=ctypes.c_int):
    return (ty * len(items))(*items)


FIELDS = [("count", 0, 32, 1, 0), ("flags", 0, 8, 0, 1), ("big", 0, 64, 1, 1), ("half", 1, 16, 0, 1), ("x", 1, 64, 0, 0), ("name with spaces and é", 2, 0, 0, 1),
          ("count2", 0, 32, 1, 0)]  # same shape as the first: its vtable must be shared, not written again
PA_TYPES = {(0, 32, 1): pa.int32(), (0, 8, 0): pa.uint8(), (0, 64, 1): pa.int64(), (1, 16, 0): pa.float16(), (1, 64, 0): pa.float64(), (2, 0, 0): pa.utf8()}


def test_schema_written_here_loads_in_pyarrow(probe):
    names = [f[0] for f in FIELDS]
    meta = {"producer": "denox-hip", "": "empty key", "k": ""}
    rc = probe.probe_write_schema(len(FIELDS), _strs(names), _ints([f[1] for f in FIELDS]), _ints([f[2] for f in FIELDS]), _ints([f[3] for f in FIELDS]),
                                  _ints([f[4] for f in FIELDS]), len(meta), _strs(list(meta)), _strs(list(meta.values())))
    fbuf = _result(probe, rc)
    schema = pa.ipc.read_schema(pa.py_buffer(_encapsulate(fbuf)))
    assert schema.names == names
    for f, (name, kind, bits, signed, nullable) in zip(schema, FIELDS):
        assert f.type == PA_TYPES[(kind, bits, signed)] and f.nullable == bool(nullable)
    assert {k.decode(): v.decode() for k, v in schema.metadata.items()} == meta
    # and the bytes re-read here give the same listing as pyarrow's own serialisation of that schema (reader, both ways)
    assert probe.probe_read_message(fbuf, len(fbuf)) == 0
    mine = probe.probe_text().decode()
    theirs = bytes(pa.ipc.read_message(schema.serialize()).metadata)
    assert probe.probe_read_message(theirs, len(theirs)) == 0
    assert probe.probe_text().decode() == mine
    assert mine.count("field ") == len(FIELDS) and "meta producer=denox-hip" in mine


def test_record_batch_written_here_loads_in_pyarrow(probe):
    # int64 column with a null, float64 column without: validity bitmaps and data as Arrow lays them out, 8-byte aligned
    a = np.array([11, -22, 0, 44, 1 << 40], np.int64)
    b = np.array([0.5, -1.25, 3.0, 1e300, -0.0], np.float64)
    validity = bytes([0b11011]) + b"\0" * 7
    body = validity + a.tobytes() + b.tobytes()
    nodes = [5, 1, 5, 0]
    buffers = [0, 8, 8, 40, 48, 0, 48, 40]
    rc = probe.probe_write_batch(5, 2, _ints(nodes, ctypes.c_int64), 4, _ints(buffers, ctypes.c_int64), len(body))
    fbuf = _result(probe, rc)
    schema = pa.schema([("a", pa.int64()), ("b", pa.float64())])
    msg = pa.ipc.read_message(pa.py_buffer(_encapsulate(fbuf, body)))
    batch = pa.ipc.read_record_batch(msg, schema)
    assert batch.num_rows == 5
    assert batch.column(0).to_pylist() == [11, -22, None, 44, 1 << 40]
    assert batch.column(1).to_pylist() == b.tolist()


def test_pyarrow_schema_decodes_here(probe):
    fields = [pa.field("height", pa.int32(), nullable=False), pa.field("u", pa.uint16()), pa.field("w", pa.float32(), metadata={"unit": "ms"}),
              pa.field("s", pa.utf8(), nullable=False), pa.field("i8", pa.int8())]
    schema = pa.schema(fields, metadata={"a": "b", "long key " * 9: "v" * 300})
    fbuf = bytes(pa.ipc.read_message(schema.serialize()).metadata)
    assert probe.probe_read_message(fbuf, len(fbuf)) == 0, probe.probe_error()
    lines = probe.probe_text().decode().splitlines()
    assert lines[:4] == ["version 4", "header 1", "body 0", "endianness 0"]
    got = [l for l in lines if l.startswith("field ")]
    assert got == ["field height nullable=0 type=2 bits=32 signed=1 children=0", "field u nullable=1 type=2 bits=16 signed=0 children=0",
                   "field w nullable=1 type=3 precision=1 children=0", "field s nullable=0 type=5 children=0", "field i8 nullable=1 type=2 bits=8 signed=1 children=0"]
    assert "fieldmeta unit=ms" in lines
    assert sorted(l for l in lines if l.startswith("meta ")) == sorted(["meta a=b", "meta " + "long key " * 9 + "=" + "v" * 300])


def test_pyarrow_record_batch_decodes_here(probe):
    batch = pa.record_batch([pa.array([1, None, 3, None, None, 6, 7], pa.int64()), pa.array([0.5] * 7, pa.float32()), pa.array(list("abcdefg"), pa.utf8())], names=["a", "b", "c"])
    msg = pa.ipc.read_message(batch.serialize())
    fbuf = bytes(msg.metadata)
    assert probe.probe_read_message(fbuf, len(fbuf)) == 0, probe.probe_error()
    lines = probe.probe_text().decode().splitlines()
    assert lines[:4] == ["version 4", "header 3", f"body {msg.body.size}", "length 7"]
    nodes = [tuple(map(int, l.split()[1:])) for l in lines if l.startswith("node ")]
    assert nodes == [(7, 3), (7, 0), (7, 0)]
    bufs = [tuple(map(int, l.split()[1:])) for l in lines if l.startswith("buffer ")]
    assert len(bufs) == 2 + 2 + 3  # validity + data, validity + data, validity + offsets + data
    offs = [o for o, _ in bufs]
    assert offs == sorted(offs) and all(o % 8 == 0 for o in offs) and all(o + n <= msg.body.size for o, n in bufs)
    # the data buffers, cut out of the body at the decoded positions, hold the column values
    body = bytes(msg.body)
    o, n = bufs[1]
    assert n >= 56 and np.frombuffer(body[o:o + 56], np.int64)[[0, 2, 5, 6]].tolist() == [1, 3, 6, 7]
    o, n = bufs[3]
    assert np.frombuffer(body[o:o + 28], np.float32).tolist() == [0.5] * 7
    o, n = bufs[6]
    assert body[o:o + 7] == b"abcdefg"


def test_damaged_arrow_metadata_is_refused_cleanly(probe):
    schema = pa.schema([pa.field(f"f{i}", pa.int32(), metadata={"k": "v" * i}) for i in range(6)], metadata={"x": "y"})
    good = bytes(pa.ipc.read_message(schema.serialize()).metadata)
    rng = np.random.default_rng(1)
    outcomes = set()
    for i in range(2000):
        b = bytearray(good)
        for _ in range(1 + i % 3):
            b[int(rng.integers(0, len(b)))] ^= int(rng.integers(1, 256))
        cut = len(b) if i % 5 else int(rng.integers(0, len(b)))
        rc = probe.probe_read_message(bytes(b[:cut]), cut)
        assert rc in (0, 2), probe.probe_error()
        outcomes.add(rc)
    assert outcomes == {0, 2}


# ------------------------------------------------------------------------------------------------ dnx bytes against dnx.fbs
class _FB:
    """Independent decoder: the FlatBuffers wire format only (positions, vtables, offsets), no knowledge of the C++ code."""

    def __init__(self, buf):
        self.b = buf

    def u(self, fmt, pos):
        return struct.unpack_from("<" + fmt, self.b, pos)[0]

    def root(self):
        return self.u("I", 0)

    def field(self, table, fid):
        vt = table - self.u("i", table)
        if 4 + 2 * fid + 2 > self.u("H", vt):
            return 0
        off = self.u("H", vt + 4 + 2 * fid)
        return table + off if off else 0

    def scalar(self, table, fid, fmt, default=0):
        p = self.field(table, fid)
        return self.u(fmt, p) if p else default

    def indirect(self, table, fid):
        p = self.field(table, fid)
        return p + self.u("I", p) if p else 0

    def string(self, table, fid):
        p = self.indirect(table, fid)
        if not p:
            return None
        n = self.u("I", p)
        assert self.b[p + 4 + n] == 0
        return self.b[p + 4:p + 4 + n].decode()

    def vector(self, table, fid):
        p = self.indirect(table, fid)
        return (p + 4, self.u("I", p)) if p else (0, 0)

    def tables(self, table, fid):
        data, n = self.vector(table, fid)
        return [data + 4 * i + self.u("I", data + 4 * i) for i in range(n)]

    def source(self, table, fid, dp):
        """union ScalarSource (dnx.fbs:16-30) at field ids fid (member index) and fid + 1 (member)."""
        kind = self.scalar(table, fid, "B")
        m = self.indirect(table, fid + 1)
        if kind == 2:
            return dp[self.scalar(m, 0, "I")]
        assert kind == 1
        dtype = self.scalar(m, 0, "B")
        data, n = self.vector(m, 1)
        size, signed = {0: (2, True), 1: (2, False), 2: (4, True), 3: (4, False), 4: (8, True), 5: (8, False)}[dtype]
        assert n == size
        return int.from_bytes(self.b[data:data + n], "little", signed=signed)


def _symir(fb, model, values):
    sym = fb.indirect(model, 10)
    nvar = fb.scalar(sym, 0, "H")
    data, n = fb.vector(sym, 1)
    assert data % 8 == 0  # struct SymIROp holds int64 members
    dp = list(values) + [0] * n
    assert len(values) == nvar
    for i in range(n):
        op, lhs, rhs = struct.unpack_from("<H6xqq", fb.b, data + 24 * i)
        a = lhs if op & 0x8000 else dp[lhs]
        b = rhs if op & 0x4000 else dp[rhs]
        base = op & 0x3FFF
        if base == 1: r = a + b
        elif base == 2: r = a - b
        elif base == 3: r = a * b
        elif base == 4: r = int(a / b) if b else 0
        elif base == 5: r = a % b
        elif base == 6: r = min(a, b)
        else: r = max(a, b)
        dp[nvar + i] = r
    return dp


@pytest.mark.parametrize("net,H,W", [("tiny_unet", 32, 48), ("oidn_unet", 1080, 1920)])
def test_dnx_bytes_follow_the_reference_schema(net, H, W):
    m, _ = networks.build(net)
    blob = dx.compile_model(m)
    d = dx.describe(blob, H=H, W=W)
    fb = _FB(blob)
    assert blob[4:8] == b"dnxx"
    model = fb.root()
    assert model % 4 == 0
    names = {fb.string(t, 0): t for t in fb.tables(model, 11)}  # value_names (field 11): name, value
    assert list(names) == d["value_names"]
    nvar = fb.scalar(fb.indirect(model, 10), 0, "H")
    values = [0] * nvar
    for name, val in (("H", H), ("W", W)):
        t = names[name]
        assert fb.scalar(t, 1, "B") == 2  # symbolic
        values[fb.scalar(fb.indirect(t, 2), 0, "I")] = val
    dp = _symir(fb, model, values)

    feat, nfeat = fb.vector(model, 1)
    assert [fb.u("I", feat + 4 * i) for i in range(nfeat)] == [1]
    info = fb.indirect(model, 2)
    assert fb.string(info, 0) == "denox-hip"

    tensors = fb.tables(model, 3)
    assert len(tensors) == len(d["tensors"])
    for t, ref in zip(tensors, d["tensors"]):
        assert fb.scalar(t, 0, "I") == ref["buffer"]
        assert fb.source(t, 1, dp) == ref["offset"] and fb.source(t, 3, dp) == ref["size"]
        ti = fb.indirect(t, 5)
        assert fb.scalar(ti, 6, "H") == ref["format"] and fb.scalar(ti, 7, "H") == 0 and fb.scalar(ti, 8, "B") == 6  # StorageBuffer, F16
        assert (fb.string(ti, 9) or "") == ref["name"]
        if "width" in ref:
            assert (fb.source(ti, 0, dp), fb.source(ti, 2, dp), fb.source(ti, 4, dp)) == (ref["width"], ref["height"], ref["channels"])
    data, n = fb.vector(model, 5)
    assert [fb.u("I", data + 4 * i) for i in range(n)] == d["inputs"]
    data, n = fb.vector(model, 6)
    assert [fb.u("I", data + 4 * i) for i in range(n)] == d["outputs"]
    buffers = fb.tables(model, 7)
    assert [(fb.source(b, 0, dp), fb.scalar(b, 2, "H")) for b in buffers] == [(x["size"], x["alignment"]) for x in d["buffers"]]

    inits = fb.tables(model, 4)
    params = {i for i, t in enumerate(d["tensors"]) if t["param"]}
    assert {fb.scalar(i, 0, "I") for i in inits} == params
    for i in inits:
        assert fb.vector(i, 1)[1] == d["tensors"][fb.scalar(i, 0, "I")]["size"]

    binaries = fb.tables(model, 9)
    assert len(binaries) == d["binaries"]
    for b in binaries:
        assert fb.vector(b, 0)[1] == 0  # spirv: empty
        data, n = fb.vector(b, 1)
        assert blob[data:data + 4] == b"\x7fELF" and n > 1000  # a code object

    dispatches = fb.tables(model, 8)
    assert len(dispatches) == len(d["dispatches"])
    for t, ref in zip(dispatches, d["dispatches"]):
        assert fb.scalar(t, 0, "I") == ref["binary_id"]
        assert [fb.source(t, 1, dp), fb.source(t, 3, dp), fb.source(t, 5, dp)] == ref["workgroup_count"]
        assert fb.string(t, 7) == ref["entry_point"]
        assert [fb.scalar(t, 11, "I"), fb.scalar(t, 12, "I"), fb.scalar(t, 13, "I")] == ref["workgroup_size"]
        flat = []
        for s in fb.tables(t, 8):
            for b in fb.tables(s, 1):
                flat.append({"set": fb.scalar(s, 0, "H"), "binding": fb.scalar(b, 0, "H"), "access": fb.scalar(b, 1, "B"), "tensor": fb.scalar(b, 2, "I")})
        assert flat == ref["bindings"]
        pc = fb.indirect(t, 9)
        fields = fb.tables(pc, 1)
        assert [fb.source(f, 2, dp) for f in fields] == ref["push_constants"]
        offs = [fb.scalar(f, 1, "H") for f in fields]
        assert offs == sorted(offs) and (not fields or offs[-1] + 4 <= fb.scalar(pc, 0, "H"))
        di = fb.indirect(t, 10)
        assert fb.string(di, 0) == ref["name"] and (fb.string(di, 2) or "") == ref["src_path"]
        if ref["flops"]:
            assert fb.source(di, 7, dp) == ref["flops"]
        if ref["memory_reads"]:
            assert fb.source(di, 3, dp) == ref["memory_reads"] and fb.source(di, 5, dp) == ref["memory_writes"]


def as_written_for_vulkan(blob: bytes) -> bytes:
    """The model with its binaries rewritten the way the reference stores them -- words in `spirv`, no code object
    (serialize.cpp:440-446 of the reference): the spirv field is pointed at the code-object vector, whose count is
    rewritten in words, and field 1 is struck from the (shared) vtables."""
    blob = bytearray(blob)
    fb = _FB(blob)
    binaries = fb.tables(fb.root(), 9)
    fields = [(fb.field(b, 0), fb.field(b, 1), b - fb.u("i", b)) for b in binaries]
    for spirv_field, code_field, _ in fields:
        code = code_field + fb.u("I", code_field)
        struct.pack_into("<I", blob, code, fb.u("I", code) // 4)
        struct.pack_into("<I", blob, spirv_field, code - spirv_field)
    for vt in {vt for _, _, vt in fields}:
        struct.pack_into("<H", blob, vt + 4 + 2, 0)
    return bytes(blob)


def test_model_written_for_vulkan_is_described():
    m, _ = networks.build("tiny_unet")
    blob = dx.compile_model(m)
    foreign = as_written_for_vulkan(blob)
    assert foreign != blob
    d, ref = dx.describe(foreign, H=32, W=48), dx.describe(blob, H=32, W=48)
    assert all(len(x.pop("code_sha256")) == 64 for x in d["dispatches"] + ref["dispatches"])  # (of the code object, which has moved)
    assert d == ref  # the rest of the description does not depend on how the binaries are stored


# ------------------------------------------------------------------------------------------------ timing database against db.fbs
def test_db_bytes_follow_the_reference_schema(tmp_path):
    path = tmp_path / "gpu.db"
    db = dx.Db(str(path))
    m, _ = networks.build("tiny_unet")
    db.populate(m, assume={"H": 64, "W": 64}, conv_config="w4r2k16")
    rng = np.random.default_rng(5)
    samples = rng.normal(80_000, 3_000, 41)
    for s_ in samples:
        db.add_sample(1, s_)
    db.writeback()
    blob = path.read_bytes()
    assert blob[4:8] == b"dbdb"
    fb = _FB(blob)
    root = fb.root()
    assert fb.scalar(root, 0, "I") == 0  # version
    binaries = fb.tables(root, 2)
    shas = []
    for b in binaries:
        data, n = fb.vector(b, 0)
        assert n == 8 and fb.vector(b, 1)[1] == 0  # eight digest words, no SPIR-V
        shas.append(struct.unpack_from("<8I", blob, data))
        assert fb.string(b, 2).endswith(".hip")  # src_path: what the kernel is rebuilt from
    assert len(set(shas)) == len(shas)
    rows = fb.tables(root, 3)
    csv = db.dump_csv().splitlines()[1:]
    assert len(rows) == len(db) == len(csv)
    for i, (t, line) in enumerate(zip(rows, csv)):
        cells = line.split(",")
        assert fb.scalar(t, 0, "I") < len(binaries)
        assert [fb.scalar(t, 1, "I"), fb.scalar(t, 2, "I"), fb.scalar(t, 3, "I")] == [int(c) for c in cells[5:8]]
        info = fb.indirect(t, 8)
        assert f'"{fb.string(info, 0)}"' == cells[0] and f'"{fb.string(info, 1)}"' == cells[1]
        assert fb.scalar(info, 5, "Q") == int(cells[8]) and fb.scalar(info, 3, "Q") == int(cells[9]) and fb.scalar(info, 4, "Q") == int(cells[10])
        nb = len(fb.tables(t, 6))
        ins, outs = fb.vector(info, 7), fb.vector(info, 8)
        assert 0 < ins[1] + outs[1] <= nb
        block = [fb.scalar(t, 10, "I"), fb.scalar(t, 11, "I"), fb.scalar(t, 12, "I")]
        assert 1 <= block[0] * block[1] * block[2] <= 1024 and fb.string(t, 9)
        time = fb.indirect(t, 7)
        if i == 1:
            assert fb.vector(time, 0) == (fb.vector(time, 0)[0], 0)  # samples: present, empty
            assert fb.scalar(time, 3, "Q") == 41
            assert fb.scalar(time, 4, "d") == pytest.approx(samples.mean(), rel=1e-12)
            assert fb.scalar(time, 5, "d") == pytest.approx(samples.var() * 41, rel=1e-9)
            assert fb.scalar(time, 1, "Q") == round(samples.mean()) and fb.scalar(time, 2, "Q") == round(samples.std())
        else:
            assert time == 0
    # flipped bytes and cuts: a clean refusal or a table, never a crash
    for k in range(400):
        b = bytearray(blob)
        b[int(rng.integers(0, len(b)))] ^= int(rng.integers(1, 256))
        cut = len(b) if k % 4 else int(rng.integers(0, len(b)))
        (tmp_path / "damaged.db").write_bytes(bytes(b[:cut]))
        try:
            dx.Db(str(tmp_path / "damaged.db"))
        except dx.DenoxHipError as e:
            assert e.status == 6


def test_db_written_the_reference_way_is_read(probe, tmp_path):
    n = [3, 0, 120]
    mean = [50_000, 0, 1_234_567]
    std = [700, 0, 4_321]
    rc = probe.probe_write_reference_db(3, _ints(n), _ints(mean, ctypes.c_uint64), _ints(std, ctypes.c_uint64))
    path = tmp_path / "vk.db"
    path.write_bytes(_result(probe, rc))
    db = dx.Db(str(path))
    assert len(db) == 3
    for i in range(3):
        cnt, mu, sd = db.row_stats(i)
        assert cnt == n[i]
        if cnt:
            assert mu == mean[i] and sd == pytest.approx(std[i], rel=1e-12)
    rows = db.dump_csv().splitlines()[1:]
    assert [r.split(",")[5] for r in rows] == ["1", "2", "3"] and all(r.startswith('"conv2d","direct_conv_cm","cfg"') for r in rows)
    # and it survives a rewrite in this backend's form
    db.add_sample(1, 10.0)
    db.writeback()
    again = dx.Db(str(path))
    assert [again.row_stats(i)[0] for i in range(3)] == [3, 1, 120] and again.row_stats(2)[1] == mean[2]


def _shared_object_bomb(n: int, name_len: int) -> bytes:
    """A valid dnx buffer, written by hand front to back, whose value_names vector names ONE table `n` times: a few
    hundred KB on disk, n * name_len bytes for a reader that copies every element it visits."""
    out = bytearray(8)
    out[4:8] = b"dnxx"

    def align(k):
        while len(out) % k:
            out.append(0)

    def table(fields, nslots):
        """fields: {slot: (fmt, value)} with 'O' = offset patched later; returns (table position, {slot: field position})."""
        align(4)
        vt = len(out)
        inline = sorted(fields.items(), key=lambda kv: -struct.calcsize("I" if kv[1][0] == "O" else kv[1][0]))
        offs, pos = {}, 4
        for slot, (fmt, _) in inline:
            size = struct.calcsize("I" if fmt == "O" else fmt)
            pos = (pos + size - 1) // size * size
            offs[slot] = pos
            pos += size
        tbl_size = (pos + 3) // 4 * 4
        out.extend(struct.pack("<HH", 4 + 2 * nslots, tbl_size))
        for slot in range(nslots):
            out.extend(struct.pack("<H", offs.get(slot, 0)))
        align(4)
        t = len(out)
        out.extend(struct.pack("<i", t - vt) + bytes(tbl_size - 4))
        where = {}
        for slot, (fmt, value) in fields.items():
            where[slot] = t + offs[slot]
            if fmt != "O":
                struct.pack_into("<" + fmt, out, where[slot], value)
        return t, where

    def point(field_pos, target):
        struct.pack_into("<I", out, field_pos, target - field_pos)

    root, rw = table({11: ("O", None)}, 12)
    struct.pack_into("<I", out, 0, root)
    align(4)
    vec = len(out)
    point(rw[11], vec)
    out.extend(struct.pack("<I", n) + bytes(4 * n))
    vn, vw = table({0: ("O", None), 1: ("B", 1), 2: ("O", None)}, 3)  # ValueName{name, value: literal}
    for i in range(n):
        point(vec + 4 + 4 * i, vn)
    lit, lw = table({0: ("B", 4), 1: ("O", None)}, 2)  # ScalarLiteral{dtype: I64, bytes}
    point(vw[2], lit)
    align(4)
    point(lw[1], len(out))
    out.extend(struct.pack("<Iq", 8, 7))
    align(4)
    point(vw[0], len(out))
    out.extend(struct.pack("<I", name_len) + b"n" * name_len + b"\0")
    align(8)
    return bytes(out)


def test_shared_objects_cannot_make_the_reader_allocate_without_bound():
    small = _shared_object_bomb(3, 10)
    d = dx.describe(small)
    assert d["value_names"] == ["n" * 10] * 3 and d["dispatches"] == []  # the hand-written buffer is a valid (empty) model
    bomb = _shared_object_bomb(100_000, 100_000)  # 0.5 MB on disk, 10 GB if every element were copied
    assert len(bomb) < 1 << 20
    with pytest.raises(dx.DenoxHipError) as e:
        dx.describe(bomb)
    assert e.value.status == 2 and "object graph" in str(e.value)
