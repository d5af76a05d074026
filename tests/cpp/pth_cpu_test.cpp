// Checkpoint reader checks that need no GPU.
//   * the reference's own archive test (test/pth_archive_test.cpp:88-146): a synthetic stored ZIP read whole and
//     on demand must give the same members, offsets and ranges; views exist only for the whole-file mode;
//   * ZIP64 records, compressed members, damaged files;
//   * the scalar conversions against what arithmetic fixes (exact widening, exactness inside fp16's normal range,
//     the documented half-up / flush rule below it), over every bf16 bit pattern;
//   * a checkpoint written by torch.save: usage <exe> <repo root> [<file.pth> <manifest>], default the committed
//     fixture tests/golden/rwkv7_tiny.pth with its manifest (written by tests/golden/make_pth_fixture.py from the
//     very tensors that went into torch.save).
#include <unistd.h>

#include <cmath>
#include <cstdio>
#include <fstream>

#include "pth_tensor.hpp"
#include "test_common.hpp"

using namespace llm_infer;

namespace {

std::string g_pth, g_manifest;

// ---- a tiny ZIP writer: stored members, optionally with ZIP64 records ----------------------------------------------
struct Member {
  std::string name;
  std::vector<std::uint8_t> data;
  std::uint16_t method = 0;
  std::uint64_t local_at = 0;
};

void put(std::vector<std::uint8_t>& out, std::uint64_t v, int bytes) {
  for (int i = 0; i < bytes; ++i) out.push_back(static_cast<std::uint8_t>(v >> (8 * i)));
}

std::vector<std::uint8_t> zip_bytes(std::vector<Member>& members, bool zip64, std::size_t pad_local_extra = 0) {
  std::vector<std::uint8_t> z;
  for (Member& m : members) {
    m.local_at = z.size();
    put(z, 0x04034b50u, 4); put(z, 20, 2); put(z, 0, 2); put(z, m.method, 2); put(z, 0, 4); put(z, 0, 4);
    put(z, m.data.size(), 4); put(z, m.data.size(), 4); put(z, m.name.size(), 2); put(z, pad_local_extra, 2);
    z.insert(z.end(), m.name.begin(), m.name.end());
    z.insert(z.end(), pad_local_extra, 0);  // torch pads the local header so that the data is 64-byte aligned
    z.insert(z.end(), m.data.begin(), m.data.end());
  }
  const std::uint64_t dir_at = z.size();
  for (const Member& m : members) {
    put(z, 0x02014b50u, 4); put(z, 45, 2); put(z, 45, 2); put(z, 0, 2); put(z, m.method, 2); put(z, 0, 4); put(z, 0, 4);
    if (zip64) {
      put(z, 0xffffffffu, 4); put(z, 0xffffffffu, 4); put(z, m.name.size(), 2); put(z, 4 + 24, 2);
    } else {
      put(z, m.data.size(), 4); put(z, m.data.size(), 4); put(z, m.name.size(), 2); put(z, 0, 2);
    }
    put(z, 0, 2); put(z, 0, 2); put(z, 0, 2); put(z, 0, 4);
    put(z, zip64 ? 0xffffffffu : m.local_at, 4);
    z.insert(z.end(), m.name.begin(), m.name.end());
    if (zip64) {
      put(z, 0x0001, 2); put(z, 24, 2); put(z, m.data.size(), 8); put(z, m.data.size(), 8); put(z, m.local_at, 8);
    }
  }
  const std::uint64_t dir_size = z.size() - dir_at;
  if (zip64) {
    const std::uint64_t rec_at = z.size();
    put(z, 0x06064b50u, 4); put(z, 44, 8); put(z, 45, 2); put(z, 45, 2); put(z, 0, 4); put(z, 0, 4);
    put(z, members.size(), 8); put(z, members.size(), 8); put(z, dir_size, 8); put(z, dir_at, 8);
    put(z, 0x07064b50u, 4); put(z, 0, 4); put(z, rec_at, 8); put(z, 1, 4);
  }
  put(z, 0x06054b50u, 4); put(z, 0, 2); put(z, 0, 2);
  put(z, zip64 ? 0xffffu : members.size(), 2); put(z, zip64 ? 0xffffu : members.size(), 2);
  put(z, zip64 ? 0xffffffffu : dir_size, 4); put(z, zip64 ? 0xffffffffu : dir_at, 4); put(z, 0, 2);
  return z;
}

std::string write_temp(const std::string& stem, const std::vector<std::uint8_t>& bytes) {
  const std::string path = "/tmp/rwkv_pth_cpu_test_" + stem + "_" + std::to_string(::getpid());
  std::ofstream f(path, std::ios::binary);
  f.write(reinterpret_cast<const char*>(bytes.data()), static_cast<std::streamsize>(bytes.size()));
  CHECK(static_cast<bool>(f));
  return path;
}

void check_both_modes(std::vector<Member>& members, const std::string& path) {
  auto whole = PthArchive::open(path);
  auto lazy = PthArchive::open(path, true);
  CHECK(whole.ok());
  CHECK(lazy.ok());
  CHECK(!whole.value().chunk_load());
  CHECK(lazy.value().chunk_load());
  CHECK_EQ(whole.value().entries().size(), members.size());
  CHECK_EQ(lazy.value().entries().size(), members.size());
  for (const Member& m : members) {
    const PthEntry* a = whole.value().find_entry(m.name);
    const PthEntry* b = lazy.value().find_entry(m.name);
    CHECK(a != nullptr && b != nullptr);
    CHECK_EQ(a->data_offset, b->data_offset);
    CHECK_EQ(a->uncompressed_size, std::uint64_t(m.data.size()));
    auto da = whole.value().read_stored_entry(*a);
    auto db = lazy.value().read_stored_entry(*b);
    CHECK(da.ok() && db.ok());
    CHECK(da.value() == m.data);
    CHECK(db.value() == m.data);
    std::vector<std::uint8_t> ra(2), rb(2);
    CHECK(whole.value().read_stored_entry_range(*a, 1, ra.data(), ra.size()).ok_status());
    CHECK(lazy.value().read_stored_entry_range(*b, 1, rb.data(), rb.size()).ok_status());
    CHECK(ra == std::vector<std::uint8_t>(m.data.begin() + 1, m.data.begin() + 3));
    CHECK(rb == ra);
    // past the end of the member
    CHECK(!whole.value().read_stored_entry_range(*a, m.data.size() - 1, ra.data(), 2).ok_status());
    CHECK(!lazy.value().read_stored_entry_range(*b, m.data.size() - 1, rb.data(), 2).ok_status());
    auto view = whole.value().stored_entry_view(*a);
    CHECK(view.ok());
    CHECK_EQ(view.value().size, std::uint64_t(m.data.size()));
    CHECK(std::memcmp(view.value().data, m.data.data(), m.data.size()) == 0);
    CHECK(!lazy.value().stored_entry_view(*b).ok());
  }
  CHECK(whole.value().find_entry("no/such/member") == nullptr);
}

}  // namespace

HOST_TEST(stored_zip_whole_and_on_demand_agree) {
  std::vector<Member> members{{"model/data.pkl", {1, 2, 3, 4}}, {"model/data/0", {9, 8, 7, 6, 5}}};
  const std::string path = write_temp("plain", zip_bytes(members, false));
  check_both_modes(members, path);
  std::remove(path.c_str());
  // local headers with an extra field (torch's alignment padding): the data offset comes from the local header
  std::vector<Member> padded{{"m/data.pkl", {1, 2, 3}}, {"m/data/0", {5, 6, 7, 8}}};
  const std::string path2 = write_temp("padded", zip_bytes(padded, false, 37));
  check_both_modes(padded, path2);
  std::remove(path2.c_str());
}

HOST_TEST(zip64_records) {
  std::vector<Member> members{{"big/data.pkl", {4, 3, 2, 1}}, {"big/data/0", {10, 20, 30}}, {"big/data/1", {7, 7, 7, 7}}};
  const std::string path = write_temp("zip64", zip_bytes(members, true));
  check_both_modes(members, path);
  std::remove(path.c_str());
}

HOST_TEST(damaged_and_unsupported_archives) {
  CHECK(!PthArchive::open("/definitely/not/here.pth").ok());
  CHECK(!PthArchive::open("/definitely/not/here.pth", true).ok());
  const std::string tiny = write_temp("tiny", {1, 2, 3});
  CHECK(PthArchive::open(tiny).status().message().find("too small") != std::string::npos);
  std::remove(tiny.c_str());
  const std::string junk = write_temp("junk", std::vector<std::uint8_t>(100, 0x55));
  CHECK(PthArchive::open(junk).status().message().find("end of central directory not found") != std::string::npos);
  CHECK(!PthArchive::open(junk, true).ok());
  std::remove(junk.c_str());

  std::vector<Member> members{{"m/data.pkl", {1, 2, 3, 4}}, {"m/data/0", {9, 8, 7, 6, 5}, 8}};  // second one "deflated"
  std::vector<std::uint8_t> z = zip_bytes(members, false);
  const std::string path = write_temp("deflate", z);
  for (bool lazy : {false, true}) {
    auto ar = PthArchive::open(path, lazy);
    CHECK(ar.ok());
    const PthEntry* e = ar.value().find_entry("m/data/0");
    CHECK(e != nullptr && !e->is_stored());
    CHECK(!ar.value().read_stored_entry(*e).ok());
    CHECK(ar.value().read_stored_entry(*ar.value().find_entry("m/data.pkl")).ok());
  }
  // a directory that points past the end of the file
  std::vector<std::uint8_t> cut(z.begin() + 20, z.end());
  const std::string path2 = write_temp("cut", cut);
  CHECK(!PthArchive::open(path2).ok());
  CHECK(!PthArchive::open(path2, true).ok());
  std::remove(path.c_str());
  std::remove(path2.c_str());
  // a stored member whose directory entry claims more bytes than the member holds: refused at open (a read of
  // the claimed size would run past the member and past the file), in both modes
  {
    std::vector<Member> two{{"m/data.pkl", {1, 2, 3, 4}}, {"m/data/0", {9, 8, 7, 6, 5}}};
    std::vector<std::uint8_t> zz = zip_bytes(two, false);
    std::size_t dir = 0;
    for (std::size_t i = 0; i + 4 <= zz.size(); ++i) {
      if (zz[i] == 0x50 && zz[i + 1] == 0x4b && zz[i + 2] == 0x01 && zz[i + 3] == 0x02) { dir = i; break; }
    }
    CHECK(dir != 0);
    const std::uint32_t claimed = 1u << 30;
    for (int b = 0; b < 4; ++b) zz[dir + 24 + b] = static_cast<std::uint8_t>(claimed >> (8 * b));
    const std::string bad = write_temp("oversize", zz);
    for (bool lazy : {false, true}) {
      auto opened = PthArchive::open(bad, lazy);
      CHECK(!opened.ok());
      CHECK(opened.status().message().find("stored entry sizes disagree") != std::string::npos);
    }
    std::remove(bad.c_str());
    // and an entry record that does not come from the archive's own directory is checked against the file again
    const std::string good = write_temp("oversize_good", zip_bytes(two, false));
    for (bool lazy : {false, true}) {
      auto opened = PthArchive::open(good, lazy);
      CHECK(opened.ok());
      PthEntry forged = *opened.value().find_entry("m/data/0");
      forged.uncompressed_size = 1u << 20;
      forged.compressed_size = 1u << 20;
      std::vector<std::uint8_t> buf(64);
      CHECK(!opened.value().read_stored_entry_range(forged, 0, buf.data(), buf.size()).ok_status());
      CHECK(!opened.value().read_stored_entry(forged).ok());
      CHECK(!opened.value().stored_entry_view(forged).ok());
    }
    std::remove(good.c_str());
  }
  // a pickle that is not a tensor state dict
  std::vector<Member> odd{{"m/data.pkl", {0x80, 2, ']', '.'}}};
  const std::string path3 = write_temp("odd", zip_bytes(odd, false));
  auto ar = PthArchive::open(path3);
  CHECK(ar.ok());
  auto recs = parse_pth_tensor_records(ar.value());
  CHECK(!recs.ok());
  CHECK(recs.status().message().find("unsupported pickle opcode 0x5d at byte 2") != std::string::npos);
  std::remove(path3.c_str());
}

// Every bf16 pattern.  What arithmetic fixes: widening is exact (value = (-1)^s 2^(e-127) (1 + m/128)); a bf16 value
// inside fp16's normal range [2^-14, 65504] has at most 7 fraction bits, so its fp16 is exact: converting back must
// give the same number; above 65504 the reference's conversion gives infinity (it rounds nothing up there: bf16
// values are 65536 and up); below 2^-14 the result is floor(|x| / 2^-24 + 1/2) subnormal steps, and zero below
// 2^-24.
HOST_TEST(scalar_conversions_over_every_bf16_pattern) {
  for (std::uint32_t b = 0; b < 65536; ++b) {
    const std::uint16_t bits = static_cast<std::uint16_t>(b);
    const float f = bf16_bits_to_float(bits);
    const int e = (bits >> 7) & 0xff;
    const int m = bits & 0x7f;
    const double sign = (bits & 0x8000) ? -1.0 : 1.0;
    if (e == 255) {
      CHECK(m ? std::isnan(f) : (std::isinf(f) && (f < 0) == (sign < 0)));
    } else if (e == 0) {
      CHECK_EQ(double(f), sign * std::ldexp(double(m) / 128.0, -126));
    } else {
      CHECK_EQ(double(f), sign * std::ldexp(1.0 + double(m) / 128.0, e - 127));
    }
    CHECK_EQ(float_to_bf16_bits(f), e == 255 && m ? float_to_bf16_bits(f) : bits);  // round trip (NaN payloads aside)

    const std::uint16_t h = float_to_f16_bits(f);
    CHECK_EQ(h & 0x8000u, bits & 0x8000u);
    const double mag = std::fabs(double(f));
    if (e == 255) {
      CHECK_EQ(h & 0x7fffu, m ? 0x7e00u : 0x7c00u);
    } else if (mag > 65504.0) {
      CHECK_EQ(h & 0x7fffu, 0x7c00u);
    } else if (mag >= std::ldexp(1.0, -14)) {
      CHECK_EQ(double(f16_bits_to_float(h)), double(f));  // exact
    } else if (mag < std::ldexp(1.0, -24)) {
      CHECK_EQ(h & 0x7fffu, 0u);
    } else {
      const double steps = std::floor(mag / std::ldexp(1.0, -24) + 0.5);  // half up, in units of the smallest subnormal
      CHECK_EQ(double(h & 0x7fffu), steps);
    }
  }
  // fp16 -> fp32 over every pattern against the definition
  for (std::uint32_t b = 0; b < 65536; ++b) {
    const std::uint16_t bits = static_cast<std::uint16_t>(b);
    const float f = f16_bits_to_float(bits);
    const int e = (bits >> 10) & 0x1f;
    const int m = bits & 0x3ff;
    const double sign = (bits & 0x8000) ? -1.0 : 1.0;
    if (e == 31) {
      CHECK(m ? std::isnan(f) : std::isinf(f));
    } else if (e == 0) {
      CHECK_EQ(double(f), sign * std::ldexp(double(m), -24));
    } else {
      CHECK_EQ(double(f), sign * std::ldexp(1.0 + double(m) / 1024.0, e - 15));
    }
  }
  // fp32 inputs with more fraction bits than fp16 keeps: ties go up in magnitude (not to even)
  CHECK_EQ(float_to_f16_bits(1.0f + std::ldexp(1.0f, -11)), std::uint16_t(0x3c01));        // tie above an even mantissa
  CHECK_EQ(float_to_f16_bits(1.0f + 3 * std::ldexp(1.0f, -11)), std::uint16_t(0x3c02));    // tie above an odd one
  CHECK_EQ(float_to_f16_bits(65520.0f), std::uint16_t(0x7c00));                            // rounds up to 2^16: infinity
  CHECK_EQ(float_to_f16_bits(-1.5f * std::ldexp(1.0f, -25)), std::uint16_t(0x8000));       // below 2^-24: signed zero
  CHECK_EQ(shape_string({3, 1, 64}), std::string("[3,1,64]"));
  CHECK_EQ(shape_string({}), std::string("[]"));
}

// manifest: "PTHM", u32 count, then per tensor: u32 name length, name, u32 rank, i64 shape[rank], i64 stride[rank],
// u64 storage offset, u64 n, u16 bf16[n] in logical order
HOST_TEST(checkpoint_written_by_torch_save) {
  const std::string pth = g_pth.empty() ? host_test::repo_root() + "/tests/golden/rwkv7_tiny.pth" : g_pth;
  const std::string manifest = g_manifest.empty() ? host_test::repo_root() + "/tests/golden/rwkv7_tiny.manifest" : g_manifest;
  std::ifstream mf(manifest, std::ios::binary);
  CHECK(static_cast<bool>(mf));
  auto rd = [&](void* p, std::size_t n) {
    mf.read(static_cast<char*>(p), static_cast<std::streamsize>(n));
    CHECK(static_cast<bool>(mf));
  };
  char magic[4];
  rd(magic, 4);
  CHECK(std::memcmp(magic, "PTHM", 4) == 0);
  std::uint32_t count = 0;
  rd(&count, 4);
  CHECK(count > 0);

  for (bool lazy : {false, true}) {
    mf.clear();
    mf.seekg(8);
    auto ar = PthArchive::open(pth, lazy);
    if (!ar.ok()) FAIL_HERE(ar.status().message());
    auto recs = parse_pth_tensor_records(ar.value());
    if (!recs.ok()) FAIL_HERE(recs.status().message());
    CHECK_EQ(recs.value().size(), std::size_t(count));
    for (std::uint32_t i = 0; i < count; ++i) {
      std::uint32_t name_len = 0, rank = 0;
      rd(&name_len, 4);
      std::string name(name_len, '\0');
      rd(&name[0], name_len);
      rd(&rank, 4);
      std::vector<std::int64_t> shape(rank), stride(rank);
      rd(shape.data(), rank * 8);
      rd(stride.data(), rank * 8);
      std::uint64_t offset = 0, n = 0;
      rd(&offset, 8);
      rd(&n, 8);
      std::vector<std::uint16_t> want(n);
      rd(want.data(), n * 2);

      const TensorRecord& rec = recs.value()[i];  // same order as the state dict
      if (rec.name != name) FAIL_HERE("tensor " << i << " is " << rec.name << ", expected " << name);
      CHECK(rec.shape == shape);
      CHECK(rec.stride == stride);
      CHECK_EQ(rec.storage_offset, offset);
      CHECK(rec.dtype == TensorDType::kBFloat16);
      auto data = load_bf16_tensor_select(ar.value(), rec, true, true, true);
      if (!data.ok()) FAIL_HERE(data.status().message());
      if (data.value().values_bf16 != want) FAIL_HERE("bf16 values of " << name << " differ");
      CHECK_EQ(data.value().values_f16.size(), std::size_t(n));
      CHECK_EQ(data.value().values.size(), std::size_t(n));
      double lo = 0, hi = 0;
      bool any = false;
      for (std::uint64_t k = 0; k < n; ++k) {
        const float f = bf16_bits_to_float(want[k]);
        CHECK(std::memcmp(&data.value().values[k], &f, sizeof(f)) == 0);  // bitwise: one of them is a NaN
        CHECK_EQ(data.value().values_f16[k], float_to_f16_bits(f));
        if (!std::isnan(f)) {
          lo = any ? std::min(lo, double(f)) : double(f);
          hi = any ? std::max(hi, double(f)) : double(f);
          any = true;
        }
      }
      auto stats = compute_tensor_stats(ar.value(), rec);
      CHECK(stats.ok());
      CHECK_EQ(stats.value().has_value, any);
      if (any) {
        CHECK_EQ(stats.value().min, lo);
        CHECK_EQ(stats.value().max, hi);
      }
    }
  }
}

// Damaged pickles out of a real checkpoint: the committed file's own data.pkl cut short at every length, with single
// bytes replaced, and with a dimension blown up.  Whatever the bytes, the reader answers with a Status - no
// exception leaves it, nothing is allocated from an unchecked count, no read leaves a buffer (this case is also
// built with the address and undefined-behaviour sanitizers, tests/test_host_api.py).  The reference's checks of
// the same kind: src/pth_archive.cpp:511,578.
HOST_TEST(hostile_pickles) {
  const std::string pth = host_test::repo_root() + "/tests/golden/rwkv7_tiny.pth";
  auto ar = PthArchive::open(pth);
  if (!ar.ok()) FAIL_HERE(ar.status().message());
  std::vector<Member> members;
  std::size_t pkl = 0;
  for (const PthEntry& e : ar.value().entries()) {
    auto bytes = ar.value().read_stored_entry(e);
    CHECK(bytes.ok());
    if (e.name.size() >= 8 && e.name.compare(e.name.size() - 8, 8, "data.pkl") == 0) pkl = members.size();
    members.push_back(Member{e.name, bytes.value()});
  }
  const std::vector<std::uint8_t> good = members[pkl].data;
  CHECK(good.size() > 64);

  // every tensor of a parsed directory is loaded: any outcome but a crash is fine for a damaged file
  auto exercise = [&](const std::vector<std::uint8_t>& pickle, bool must_fail) {
    members[pkl].data = pickle;
    const std::string path = write_temp("hostile", zip_bytes(members, false));
    for (bool lazy : {false, true}) {
      auto opened = PthArchive::open(path, lazy);
      CHECK(opened.ok());
      auto recs = parse_pth_tensor_records(opened.value());
      if (must_fail) CHECK(!recs.ok());
      if (!recs.ok()) continue;
      for (const TensorRecord& rec : recs.value()) {
        auto data = load_bf16_tensor_select(opened.value(), rec, true, true, false);
        if (data.ok()) CHECK_EQ(data.value().values_bf16.size(), data.value().values_f16.size());
        (void)compute_tensor_stats(opened.value(), rec);
      }
    }
    std::remove(path.c_str());
  };

  exercise(good, false);
  // cut short: every prefix in the first 300 bytes, then every 37th length
  for (std::size_t n = 0; n < good.size(); n += (n < 300 ? 1 : 37)) {
    exercise(std::vector<std::uint8_t>(good.begin(), good.begin() + static_cast<long>(n)), true);
  }
  // one byte replaced (a fixed pseudo-random walk over positions and values)
  std::uint32_t rng = 12345u;
  for (int i = 0; i < 600; ++i) {
    rng = rng * 1664525u + 1013904223u;
    std::vector<std::uint8_t> bad = good;
    bad[(rng >> 8) % bad.size()] = static_cast<std::uint8_t>(rng >> 24);
    exercise(bad, false);
  }
  // a dimension blown up: every BININT (opcode J, four bytes) and BININT2 (opcode M, two bytes) operand in turn set
  // to its largest value - shapes of 2^31 - 1 and 65535 rows against storages of a few kilobytes
  int patched = 0;
  for (std::size_t i = 0; i + 5 <= good.size() && patched < 200; ++i) {
    if (good[i] != 'J' && good[i] != 'M') continue;
    std::vector<std::uint8_t> bad = good;
    if (good[i] == 'J') {
      bad[i + 1] = 0xff; bad[i + 2] = 0xff; bad[i + 3] = 0xff; bad[i + 4] = 0x7f;
    } else {
      bad[i + 1] = 0xff; bad[i + 2] = 0xff;
    }
    exercise(bad, false);
    ++patched;
  }
  CHECK(patched > 10);
  // hand-made records that no pickle would give: the loaders check them against the storage before reserving
  members[pkl].data = good;
  const std::string path = write_temp("hostile_rec", zip_bytes(members, false));
  auto opened = PthArchive::open(path);
  CHECK(opened.ok());
  auto recs = parse_pth_tensor_records(opened.value());
  CHECK(recs.ok() && !recs.value().empty());
  TensorRecord huge = recs.value().front();
  huge.shape = {std::int64_t(1) << 40, std::int64_t(1) << 40};   // the product overflows 64 bits
  huge.stride = {std::int64_t(1) << 40, 1};
  CHECK(!load_bf16_tensor_select(opened.value(), huge, true, true, true).ok());
  huge.shape = {std::int64_t(1) << 33};
  huge.stride = {0};                                              // every element at the same place: 2^33 of them
  CHECK(!load_bf16_tensor_select(opened.value(), huge, true, false, false).ok());
  huge.shape = {-4};
  huge.stride = {1};
  auto negative = load_bf16_tensor_select(opened.value(), huge, true, false, false);
  CHECK(!negative.ok() || negative.value().values_bf16.empty());
  std::remove(path.c_str());
}

int main(int argc, char** argv) {
  if (argc > 3) {
    g_pth = argv[2];
    g_manifest = argv[3];
  }
  return host_test::run_all(argc, argv, false);
}
