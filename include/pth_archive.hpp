// Reader for the ZIP container of a PyTorch checkpoint: the reference's `llm_infer::PthArchive`
// (include/pth_archive.hpp:13-66, src/pth_archive.cpp), same types and methods.
//
// torch.save writes every member uncompressed ("stored") and 64-byte aligned, so a tensor's bytes can be read
// straight out of the file.  Two modes, as in the reference: the whole file in memory (entries can be viewed in
// place), or `chunk_load`: only the directory is parsed up front and entry ranges are read from the file on
// demand (a 7.2B checkpoint is 14 GB).  ZIP64 records (members or directory beyond 4 GiB, more than 65534 members)
// are understood; compressed members are listed but cannot be read.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "status.hpp"

namespace llm_infer {

struct PthEntry {
  std::string name;
  std::uint16_t compression_method = 0;
  std::uint32_t crc32 = 0;
  std::uint64_t compressed_size = 0;
  std::uint64_t uncompressed_size = 0;
  std::uint64_t local_header_offset = 0;
  std::uint64_t data_offset = 0;  // first byte of the member's data in the file

  bool is_stored() const { return compression_method == 0; }
};

struct PthEntryView {
  const std::uint8_t* data = nullptr;
  std::uint64_t size = 0;
};

class PthArchive {
public:
  static Result<PthArchive> open(const std::string& path, bool chunk_load = false);

  const std::string& path() const { return path_; }
  const std::vector<PthEntry>& entries() const { return entries_; }
  bool chunk_load() const { return chunk_load_; }
  const PthEntry* find_entry(const std::string& name) const;

  // the whole member / `size` bytes from `entry_offset` on / a pointer into the in-memory file (fails with
  // chunk_load, where there is no such copy)
  Result<std::vector<std::uint8_t>> read_stored_entry(const PthEntry& entry) const;
  Status read_stored_entry_range(const PthEntry& entry, std::uint64_t entry_offset, void* destination,
                                 std::size_t size) const;
  Result<PthEntryView> stored_entry_view(const PthEntry& entry) const;

private:
  struct StreamReader;  // file handle + mutex of the chunk_load mode
  std::string path_;
  std::uint64_t file_size_ = 0;
  bool chunk_load_ = false;
  // the whole file (chunk_load off): allocated without the zero fill a vector would do first, which costs as
  // much as a third of the read on a multi-gigabyte file
  struct FileBytes {
    std::unique_ptr<std::uint8_t[]> p;
    std::size_t n = 0;
    void allocate(std::size_t size) {
      p.reset(new std::uint8_t[size]);
      n = size;
    }
    std::uint8_t* data() { return p.get(); }
    const std::uint8_t* data() const { return p.get(); }
    std::size_t size() const { return n; }
  };
  FileBytes bytes_;
  std::vector<PthEntry> entries_;
  std::shared_ptr<StreamReader> stream_reader_;
};

}  // namespace llm_infer
