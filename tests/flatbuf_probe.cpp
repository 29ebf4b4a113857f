// Test helper (built by tests/test_flatbuf.py with g++, never part of the library): drives the FlatBuffers writer and
// reader of denox_amd/csrc/common/flatbuf.hpp on a schema for which a third-party implementation is installed --
// Apache Arrow's IPC metadata (Message.fbs / Schema.fbs of the Arrow format, read and written by pyarrow through the
// real FlatBuffers library and its verifier).  What pyarrow accepts from the writer, and what the reader extracts from
// pyarrow's bytes, pins the wire-format layer the dnx and db files are built on.
//
// Field ids below are the declaration order in Arrow's published schemas:
//   Message   { version:short, header:MessageHeader (union: Schema = 1, RecordBatch = 3), bodyLength:long, custom_metadata:[KeyValue] }
//   Schema    { endianness:short, fields:[Field], custom_metadata:[KeyValue], features:[long] }
//   Field     { name:string, nullable:bool, type:Type (union), dictionary, children:[Field], custom_metadata:[KeyValue] }
//   Type      union: Int = 2 { bitWidth:int, is_signed:bool }, FloatingPoint = 3 { precision:short }, Utf8 = 5 {}
//   KeyValue  { key:string, value:string }
//   RecordBatch { length:long, nodes:[FieldNode struct {long length, long null_count}], buffers:[Buffer struct {long offset, long length}] }
#include "../denox_amd/csrc/common/flatbuf.hpp"
#include <cstdio>
#include <sstream>

using namespace denox;

namespace {
std::string g_error;
std::vector<uint8_t> g_bytes;
std::string g_text;

fb::Off keyValues(fb::Builder &b, int n, const char *const *keys, const char *const *values) {
  std::vector<fb::Off> kv(static_cast<size_t>(n));
  for (int i = 0; i < n; ++i) {
    const fb::Off k = b.createString(keys[i]), v = b.createString(values[i]);
    b.startTable(2);
    b.addOffset(0, k);
    b.addOffset(1, v);
    kv[static_cast<size_t>(i)] = b.endTable();
  }
  return b.createOffsetVector(kv);
}

fb::Off message(fb::Builder &b, uint8_t headerType, fb::Off header, int64_t bodyLength) {
  b.startTable(5);
  b.addScalar<int16_t>(0, 4, 0); // MetadataVersion V5
  b.addScalar<uint8_t>(1, headerType, 0);
  b.addOffset(2, header);
  b.addScalar<int64_t>(3, bodyLength, 0);
  return b.endTable();
}

template <typename F> int guarded(F &&f) {
  try {
    f();
    return 0;
  } catch (const Error &e) {
    g_error = e.what();
    return static_cast<int>(e.status);
  } catch (const std::exception &e) {
    g_error = e.what();
    return 7;
  }
}
} // namespace

extern "C" {

const char *probe_error() { return g_error.c_str(); }
const uint8_t *probe_bytes() { return g_bytes.data(); }
size_t probe_size() { return g_bytes.size(); }
const char *probe_text() { return g_text.c_str(); }

// kinds: 0 Int(bits, signed), 1 FloatingPoint(bits = 16 / 32 / 64), 2 Utf8
int probe_write_schema(int n, const char *const *names, const int *kinds, const int *bits, const int *isSigned, const int *nullable, int nMeta,
                       const char *const *metaKeys, const char *const *metaValues) {
  return guarded([&] {
    fb::Builder b(64); // small on purpose: the buffer has to grow several times
    std::vector<fb::Off> fields(static_cast<size_t>(n));
    for (int i = 0; i < n; ++i) {
      fb::Off type = 0;
      uint8_t typeType = 0;
      if (kinds[i] == 0) {
        b.startTable(2);
        b.addScalar<int32_t>(0, bits[i], 0);
        b.addScalar<uint8_t>(1, isSigned[i] ? 1 : 0, 0);
        type = b.endTable();
        typeType = 2;
      } else if (kinds[i] == 1) {
        b.startTable(1);
        b.addScalar<int16_t>(0, bits[i] == 16 ? 0 : bits[i] == 32 ? 1 : 2, 0);
        type = b.endTable();
        typeType = 3;
      } else {
        b.startTable(0);
        type = b.endTable();
        typeType = 5;
      }
      const fb::Off name = b.createString(names[i]);
      const fb::Off children = b.createOffsetVector({});
      b.startTable(7);
      b.addOffset(0, name);
      b.addScalar<uint8_t>(1, nullable[i] ? 1 : 0, 0);
      b.addScalar<uint8_t>(2, typeType, 0);
      b.addOffset(3, type);
      b.addOffset(5, children);
      fields[static_cast<size_t>(i)] = b.endTable();
    }
    const fb::Off fieldVec = b.createOffsetVector(fields);
    const fb::Off meta = nMeta ? keyValues(b, nMeta, metaKeys, metaValues) : 0;
    b.startTable(4);
    b.addOffset(1, fieldVec);
    b.addOffset(2, meta);
    const fb::Off schema = b.endTable();
    g_bytes = b.finish(message(b, 1, schema, 0), nullptr);
  });
}

int probe_write_batch(int64_t length, int nNodes, const int64_t *nodes, int nBuffers, const int64_t *buffers, int64_t bodyLength) {
  return guarded([&] {
    fb::Builder b(64);
    const fb::Off bufVec = b.createVector(buffers, 16, 8, static_cast<size_t>(nBuffers));
    const fb::Off nodeVec = b.createVector(nodes, 16, 8, static_cast<size_t>(nNodes));
    b.startTable(3);
    b.addScalar<int64_t>(0, length, 0);
    b.addOffset(1, nodeVec);
    b.addOffset(2, bufVec);
    const fb::Off batch = b.endTable();
    g_bytes = b.finish(message(b, 3, batch, bodyLength), nullptr);
  });
}

// Decodes a Message flatbuffer into a line-oriented text the test compares with what pyarrow says about the same object.
int probe_read_message(const uint8_t *data, size_t size) {
  return guarded([&] {
    const fb::Table msg = fb::Table::root(data, size, nullptr);
    std::ostringstream o;
    const uint8_t headerType = msg.scalar<uint8_t>(1, 0);
    o << "version " << msg.scalar<int16_t>(0, 0) << "\nheader " << static_cast<int>(headerType) << "\nbody " << msg.scalar<int64_t>(3, 0) << "\n";
    const fb::Table h = msg.table(2);
    auto meta = [&](const fb::Table &t, unsigned slot, const char *tag) {
      const fb::Vector kv = t.vector(slot, 4, 4);
      for (uint32_t i = 0; i < kv.size(); ++i) o << tag << " " << kv.table(i).str(0) << "=" << kv.table(i).str(1) << "\n";
    };
    if (headerType == 1) {
      o << "endianness " << h.scalar<int16_t>(0, 0) << "\n";
      const fb::Vector fields = h.vector(1, 4, 4);
      for (uint32_t i = 0; i < fields.size(); ++i) {
        const fb::Table f = fields.table(i);
        const uint8_t tt = f.scalar<uint8_t>(2, 0);
        const fb::Table ty = f.table(3);
        o << "field " << f.str(0) << " nullable=" << static_cast<int>(f.scalar<uint8_t>(1, 0)) << " type=" << static_cast<int>(tt);
        if (tt == 2) o << " bits=" << ty.scalar<int32_t>(0, 0) << " signed=" << static_cast<int>(ty.scalar<uint8_t>(1, 0));
        if (tt == 3) o << " precision=" << ty.scalar<int16_t>(0, 0);
        o << " children=" << f.vector(5, 4, 4).size() << "\n";
        meta(f, 6, "fieldmeta");
      }
      meta(h, 2, "meta");
    } else if (headerType == 3) {
      o << "length " << h.scalar<int64_t>(0, 0) << "\n";
      const fb::Vector nodes = h.vector(1, 16, 8), bufs = h.vector(2, 16, 8);
      for (uint32_t i = 0; i < nodes.size(); ++i) o << "node " << nodes.member<int64_t>(i, 0) << " " << nodes.member<int64_t>(i, 8) << "\n";
      for (uint32_t i = 0; i < bufs.size(); ++i) o << "buffer " << bufs.member<int64_t>(i, 0) << " " << bufs.member<int64_t>(i, 8) << "\n";
    }
    g_text = o.str();
  });
}

// A timing database the way the reference writes one (database/src/denox/db/Db.cpp:270-497): fields of db.fbs only, one
// Sample table per measurement, mean and deviation in whole nanoseconds, SPIR-V words in the binary.  One binary, `n` rows
// that differ in workgroup_count_x (1, 2, ...) with `samplesPerRow[i]` samples each.
int probe_write_reference_db(int n, const int *samplesPerRow, const uint64_t *meanNs, const uint64_t *stdNs) {
  return guarded([&] {
    fb::Builder b(64);
    std::vector<fb::Off> rows(static_cast<size_t>(n));
    for (int r = 0; r < n; ++r) {
      std::vector<fb::Off> samples(static_cast<size_t>(samplesPerRow[r]));
      for (size_t k = 0; k < samples.size(); ++k) {
        b.startTable(3);
        b.addScalar<uint64_t>(0, 1700000000000000000ull + k, 0);
        b.addScalar<uint64_t>(1, meanNs[r] + k, 0);
        samples[k] = b.endTable();
      }
      const fb::Off sampleVec = b.createOffsetVector(samples);
      b.startTable(3);
      b.addOffset(0, sampleVec);
      b.addScalar<uint64_t>(1, meanNs[r], 0);
      b.addScalar<uint64_t>(2, stdNs[r], 0);
      const fb::Off time = b.endTable();
      const fb::Off op = b.createString("conv2d"), shader = b.createString("direct_conv_cm"), config = b.createString("cfg");
      b.startTable(9);
      b.addOffset(0, op);
      b.addOffset(1, shader);
      b.addOffset(2, config);
      b.addScalar<uint64_t>(5, 1000u * static_cast<uint64_t>(r + 1), 0);
      b.addScalar<uint8_t>(6, 1, 0);
      const fb::Off info = b.endTable();
      b.startTable(5);
      b.addScalar<uint32_t>(0, 64, 0);
      const fb::Off binfo = b.endTable();
      b.startTable(8);
      b.addScalar<uint32_t>(1, 0, 0);
      b.addScalar<uint16_t>(3, 1, 0);
      b.addScalar<uint64_t>(5, 4096, 0);
      b.addScalar<uint32_t>(6, 16, 0);
      b.addOffset(7, binfo);
      const fb::Off binding = b.endTable();
      const fb::Off bindings = b.createOffsetVector({binding});
      const uint8_t pcBytes[8] = {1, 2, 3, 4, 5, 6, 7, 8};
      const fb::Off pc = b.createVector(pcBytes, 1, 1, 8);
      b.startTable(9);
      b.addScalar<uint32_t>(1, static_cast<uint32_t>(r + 1), 0);
      b.addScalar<uint32_t>(2, 1, 0);
      b.addScalar<uint32_t>(3, 1, 0);
      b.addOffset(4, pc);
      b.addScalar<uint64_t>(5, 0x1234567890abcdefull + static_cast<uint64_t>(r), 0);
      b.addOffset(6, bindings);
      if (samplesPerRow[r]) b.addOffset(7, time);
      b.addOffset(8, info);
      rows[static_cast<size_t>(r)] = b.endTable();
    }
    const fb::Off dispatches = b.createOffsetVector(rows);
    const uint32_t sha[8] = {0x00010203u, 0x04050607u, 0x08090a0bu, 0x0c0d0e0fu, 0xf0f1f2f3u, 0xf4f5f6f7u, 0xf8f9fafbu, 0xfcfdfeffu};
    const uint32_t spirv[5] = {0x07230203u, 0x00010600u, 0, 1, 0};
    const fb::Off shaVec = b.createVector(sha, 4, 4, 8), spirvVec = b.createVector(spirv, 4, 4, 5);
    b.startTable(2);
    b.addOffset(0, shaVec);
    b.addOffset(1, spirvVec);
    const fb::Off binary = b.endTable();
    const fb::Off binaries = b.createOffsetVector({binary});
    const fb::Off device = b.createString("some Vulkan device"), os = b.createString("Linux"), driver = b.createString("1.2.3"), commit = b.createString("abc"),
                  version = b.createString("0.1");
    b.startTable(10);
    b.addOffset(0, device);
    b.addOffset(1, os);
    b.addOffset(2, driver);
    b.addOffset(3, commit);
    b.addOffset(4, version);
    b.addScalar<uint64_t>(5, 1700000000000000000ull, 0);
    b.addScalar<uint16_t>(6, 2, 0);
    b.addScalar<uint16_t>(9, 100, 0);
    const fb::Off env = b.endTable();
    const fb::Off envs = b.createOffsetVector({env});
    b.startTable(4);
    b.addOffset(1, envs);
    b.addOffset(2, binaries);
    b.addOffset(3, dispatches);
    g_bytes = b.finish(b.endTable(), "dbdb");
  });
}

} // extern "C"
