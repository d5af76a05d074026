// ZIP container reader for PyTorch checkpoints (interface: include/pth_archive.hpp; the reference's
// src/pth_archive.cpp:207-587 is the behaviour restated here: stored members only, whole-file or on-demand
// reads, ZIP64, single-disk archives).  Written against the ZIP application note: the directory is found from the
// end-of-central-directory record at the tail of the file, every member's data offset from its local header.
#include "pth_archive.hpp"

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstring>

namespace llm_infer {
namespace {

constexpr std::uint32_t kSigLocal = 0x04034b50u;
constexpr std::uint32_t kSigCentral = 0x02014b50u;
constexpr std::uint32_t kSigEnd = 0x06054b50u;
constexpr std::uint32_t kSigEnd64 = 0x06064b50u;
constexpr std::uint32_t kSigEnd64Locator = 0x07064b50u;
constexpr std::size_t kEndRecord = 22;        // fixed part of the end-of-central-directory record
constexpr std::size_t kEnd64Locator = 20;
constexpr std::size_t kEnd64Record = 56;
constexpr std::size_t kCentralHeader = 46;
constexpr std::size_t kLocalHeader = 30;
constexpr std::uint16_t kExtraZip64 = 0x0001;

// little-endian field readers over a bounds-checked span
struct Span {
  const std::uint8_t* p = nullptr;
  std::size_t n = 0;
  bool has(std::size_t off, std::size_t len) const { return off <= n && len <= n - off; }
  std::uint16_t u16(std::size_t off) const { return static_cast<std::uint16_t>(p[off] | (p[off + 1] << 8)); }
  std::uint32_t u32(std::size_t off) const {
    return static_cast<std::uint32_t>(p[off]) | (static_cast<std::uint32_t>(p[off + 1]) << 8) |
           (static_cast<std::uint32_t>(p[off + 2]) << 16) | (static_cast<std::uint32_t>(p[off + 3]) << 24);
  }
  std::uint64_t u64(std::size_t off) const { return u32(off) | (static_cast<std::uint64_t>(u32(off + 4)) << 32); }
};

Span span_of(const std::vector<std::uint8_t>& v) { return Span{v.data(), v.size()}; }

std::string describe(const char* what, const std::string& path) { return std::string(what) + ": " + path; }

}  // namespace

// The file of the chunk_load mode.  pread needs no shared file position, so concurrent readers do not serialise;
// pages already consumed are dropped from the page cache (a checkpoint is read once, front to back).
struct PthArchive::StreamReader {
  int fd = -1;
  explicit StreamReader(const std::string& path) {
    fd = ::open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd >= 0) (void)::posix_fadvise(fd, 0, 0, POSIX_FADV_SEQUENTIAL);
  }
  ~StreamReader() {
    if (fd >= 0) ::close(fd);
  }
  StreamReader(const StreamReader&) = delete;
  StreamReader& operator=(const StreamReader&) = delete;

  Status read(std::uint64_t offset, void* destination, std::size_t size) const {
    std::uint8_t* out = static_cast<std::uint8_t*>(destination);
    std::size_t done = 0;
    while (done < size) {
      const ssize_t got = ::pread(fd, out + done, size - done, static_cast<off_t>(offset + done));
      if (got < 0 && errno == EINTR) continue;
      if (got <= 0) return Status::error(got == 0 ? "model file ends inside the requested range" : "failed to read model file range");
      done += static_cast<std::size_t>(got);
    }
    if (size != 0) (void)::posix_fadvise(fd, static_cast<off_t>(offset), static_cast<off_t>(size), POSIX_FADV_DONTNEED);
    return Status::ok();
  }
};

Result<PthArchive> PthArchive::open(const std::string& path, bool chunk_load) {
  PthArchive ar;
  ar.path_ = path;
  ar.chunk_load_ = chunk_load;

  auto reader = std::make_shared<StreamReader>(path);
  if (reader->fd < 0) return Status::error(describe("failed to open file", path));
  struct stat st;
  if (::fstat(reader->fd, &st) != 0 || st.st_size < 0) return Status::error(describe("failed to determine file size", path));
  ar.file_size_ = static_cast<std::uint64_t>(st.st_size);
  if (ar.file_size_ < kEndRecord) return Status::error("file is too small to be a zip archive");

  if (!chunk_load) {
    ar.bytes_.allocate(static_cast<std::size_t>(ar.file_size_));
    Status rd = reader->read(0, ar.bytes_.data(), ar.bytes_.size());
    if (!rd.ok_status()) return Status::error(describe("failed to read file", path));
  } else {
    ar.stream_reader_ = reader;
  }
  // any range of the file, from memory or from the file
  auto fetch = [&](std::uint64_t offset, std::uint64_t size, std::vector<std::uint8_t>* out) -> Status {
    if (offset > ar.file_size_ || size > ar.file_size_ - offset) return Status::error("zip record lies outside the file");
    out->resize(static_cast<std::size_t>(size));
    if (!chunk_load) {
      std::memcpy(out->data(), ar.bytes_.data() + offset, out->size());
      return Status::ok();
    }
    return reader->read(offset, out->data(), out->size());
  };

  // ---- end-of-central-directory record: the last one whose comment length fits the file tail
  const std::uint64_t tail_len = std::min<std::uint64_t>(ar.file_size_, kEndRecord + 65535 + kEnd64Locator);
  const std::uint64_t tail_off = ar.file_size_ - tail_len;
  std::vector<std::uint8_t> tail;
  Status s = fetch(tail_off, tail_len, &tail);
  if (!s.ok_status()) return s;
  const Span t = span_of(tail);
  std::size_t end_pos = tail.size();
  for (std::size_t pos = tail.size() - kEndRecord + 1; pos-- > 0;) {
    if (t.u32(pos) == kSigEnd && pos + kEndRecord + t.u16(pos + 20) <= tail.size()) {
      end_pos = pos;
      break;
    }
  }
  if (end_pos == tail.size()) return Status::error("end of central directory not found");
  if (t.u16(end_pos + 4) != 0 || t.u16(end_pos + 6) != 0) return Status::error("multi-disk zip archives are not supported");
  std::uint64_t n_entries = t.u16(end_pos + 10);
  std::uint64_t dir_size = t.u32(end_pos + 12);
  std::uint64_t dir_offset = t.u32(end_pos + 16);
  if (n_entries == 0xffffu || dir_size == 0xffffffffu || dir_offset == 0xffffffffu) {
    if (end_pos < kEnd64Locator || t.u32(end_pos - kEnd64Locator) != kSigEnd64Locator) {
      return Status::error("zip64 end of central directory locator not found");
    }
    const std::size_t loc = end_pos - kEnd64Locator;
    if (t.u32(loc + 4) != 0 || t.u32(loc + 16) != 1) return Status::error("multi-disk zip64 archives are not supported");
    std::vector<std::uint8_t> rec;
    s = fetch(t.u64(loc + 8), kEnd64Record, &rec);
    if (!s.ok_status()) return Status::error("zip64 end of central directory is out of file bounds");
    const Span r = span_of(rec);
    if (r.u32(0) != kSigEnd64) return Status::error("zip64 end of central directory signature mismatch");
    if (r.u32(16) != 0 || r.u32(20) != 0) return Status::error("multi-disk zip64 archives are not supported");
    n_entries = r.u64(32);
    dir_size = r.u64(40);
    dir_offset = r.u64(48);
  }

  // ---- central directory
  std::vector<std::uint8_t> dir;
  s = fetch(dir_offset, dir_size, &dir);
  if (!s.ok_status()) return Status::error("central directory is out of file bounds");
  const Span d = span_of(dir);
  std::size_t at = 0;
  ar.entries_.reserve(static_cast<std::size_t>(std::min<std::uint64_t>(n_entries, 1u << 20)));
  for (std::uint64_t i = 0; i < n_entries; ++i) {
    if (!d.has(at, kCentralHeader) || d.u32(at) != kSigCentral) {
      return Status::error("central directory entry " + std::to_string(i) + " is malformed");
    }
    PthEntry e;
    e.compression_method = d.u16(at + 10);
    e.crc32 = d.u32(at + 16);
    e.compressed_size = d.u32(at + 20);
    e.uncompressed_size = d.u32(at + 24);
    const std::size_t name_len = d.u16(at + 28);
    const std::size_t extra_len = d.u16(at + 30);
    const std::size_t comment_len = d.u16(at + 32);
    e.local_header_offset = d.u32(at + 42);
    if (!d.has(at + kCentralHeader, name_len + extra_len + comment_len)) {
      return Status::error("central directory entry " + std::to_string(i) + " runs past the directory");
    }
    e.name.assign(reinterpret_cast<const char*>(dir.data() + at + kCentralHeader), name_len);
    // ZIP64 extended information: the 64-bit values follow in this order, each present only if its 32-bit
    // field is saturated
    const bool big_usize = e.uncompressed_size == 0xffffffffu;
    const bool big_csize = e.compressed_size == 0xffffffffu;
    const bool big_offset = e.local_header_offset == 0xffffffffu;
    if (big_usize || big_csize || big_offset) {
      std::size_t x = at + kCentralHeader + name_len;
      const std::size_t x_end = x + extra_len;
      bool found = false;
      while (x + 4 <= x_end) {
        const std::uint16_t id = d.u16(x);
        const std::size_t len = d.u16(x + 2);
        if (x + 4 + len > x_end) break;
        if (id == kExtraZip64) {
          std::size_t v = x + 4;
          const std::size_t v_end = v + len;
          auto take = [&](bool wanted, std::uint64_t* field) {
            if (!wanted) return true;
            if (v + 8 > v_end) return false;
            *field = d.u64(v);
            v += 8;
            return true;
          };
          if (!take(big_usize, &e.uncompressed_size) || !take(big_csize, &e.compressed_size) ||
              !take(big_offset, &e.local_header_offset)) {
            return Status::error("zip64 extra field of " + e.name + " is truncated");
          }
          found = true;
          break;
        }
        x += 4 + len;
      }
      if (!found) return Status::error("zip64 extra field missing for entry: " + e.name);
    }
    ar.entries_.push_back(std::move(e));
    at += kCentralHeader + name_len + extra_len + comment_len;
  }

  // ---- data offsets from the local headers (their name / extra lengths may differ from the directory's)
  std::vector<std::uint8_t> head;
  for (PthEntry& e : ar.entries_) {
    s = fetch(e.local_header_offset, kLocalHeader, &head);
    if (!s.ok_status()) return Status::error("local header is out of file bounds for entry: " + e.name);
    const Span h = span_of(head);
    if (h.u32(0) != kSigLocal) return Status::error("local header signature mismatch for entry: " + e.name);
    e.data_offset = e.local_header_offset + kLocalHeader + h.u16(26) + h.u16(28);
    if (e.data_offset > ar.file_size_ || e.compressed_size > ar.file_size_ - e.data_offset) {
      return Status::error("entry data is out of file bounds: " + e.name);
    }
    // a stored member occupies exactly its uncompressed size: a directory that claims more would let a read
    // run past the member (and past the file)
    if (e.is_stored() && e.uncompressed_size != e.compressed_size) {
      return Status::error("stored entry sizes disagree (compressed " + std::to_string(e.compressed_size) +
                           ", uncompressed " + std::to_string(e.uncompressed_size) + "): " + e.name);
    }
  }
  return ar;
}

const PthEntry* PthArchive::find_entry(const std::string& name) const {
  for (const PthEntry& e : entries_) {
    if (e.name == name) return &e;
  }
  return nullptr;
}

Status PthArchive::read_stored_entry_range(const PthEntry& entry, std::uint64_t entry_offset, void* destination,
                                           std::size_t size) const {
  if (!entry.is_stored()) {
    return Status::error("entry is compressed (method " + std::to_string(entry.compression_method) +
                         "), only stored entries can be read: " + entry.name);
  }
  if (entry_offset > entry.uncompressed_size || size > entry.uncompressed_size - entry_offset) {
    return Status::error("requested range exceeds entry size: " + entry.name);
  }
  if (size == 0) return Status::ok();
  if (destination == nullptr) return Status::error("null destination for entry: " + entry.name);
  // the entry may not come from this archive's own directory: check it against the file again
  // (src/pth_archive.cpp:511 does the same)
  if (entry.data_offset > file_size_ || entry.uncompressed_size > file_size_ - entry.data_offset) {
    return Status::error("entry data is out of file bounds: " + entry.name);
  }
  const std::uint64_t from = entry.data_offset + entry_offset;
  if (!chunk_load_) {
    std::memcpy(destination, bytes_.data() + from, size);
    return Status::ok();
  }
  Status s = stream_reader_->read(from, destination, size);
  if (!s.ok_status()) return Status::error(s.message() + ": " + path_);
  return s;
}

Result<std::vector<std::uint8_t>> PthArchive::read_stored_entry(const PthEntry& entry) const {
  if (entry.is_stored() && (entry.data_offset > file_size_ || entry.uncompressed_size > file_size_ - entry.data_offset)) {
    return Status::error("entry data is out of file bounds: " + entry.name);  // before anything is allocated
  }
  std::vector<std::uint8_t> out(static_cast<std::size_t>(entry.is_stored() ? entry.uncompressed_size : 0));
  Status s = read_stored_entry_range(entry, 0, out.data(), out.size());
  if (!s.ok_status()) return s;
  if (!entry.is_stored()) return Status::error("entry is compressed: " + entry.name);
  return out;
}

Result<PthEntryView> PthArchive::stored_entry_view(const PthEntry& entry) const {
  if (chunk_load_) return Status::error("entry views need the whole file in memory (chunk_load is on): " + entry.name);
  if (!entry.is_stored()) return Status::error("entry is compressed: " + entry.name);
  if (entry.data_offset > file_size_ || entry.uncompressed_size > file_size_ - entry.data_offset) {
    return Status::error("entry data is out of file bounds: " + entry.name);  // src/pth_archive.cpp:578
  }
  PthEntryView view;
  view.data = bytes_.data() + entry.data_offset;
  view.size = entry.uncompressed_size;
  return view;
}

}  // namespace llm_infer
