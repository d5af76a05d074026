// ModelBackend over the C ABI of librwkv_hip.so.
//
// Mirrors ModelBackend in the reference (src/rwkv7_fast_v4.cu:1349-1592): argument checks and their
// messages, the state layout and zero-initialisation of create_state (:1373-1400), the per-layer strided
// slice copies of copy_state_slice (:1421-1504), copy_logits_slice (:1506-1532) and the capacity formula of
// query_prefill_capacity (:1534-1580), and its load pipeline (:110-701): the checkpoint's bf16 tensors are
// uploaded as they are and converted on the device (fp16, LoRA matrices transposed, embedding through ln0),
// the seven big matrices then quantised on load when a weight format is asked for.  Differences: a model_path
// of the form synthetic:<preset>... builds random-init weights without a file, only the fp32-state mode
// exists, device errors throw instead of exiting, and forward passes run through pooled sessions (stream +
// arena + decode graphs) so concurrent callers do not allocate per call.
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <limits>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <thread>
#include <unordered_map>

#include "pth_tensor.hpp"
#include "rwkv_server_backend.hpp"

namespace rwkv7_server {
namespace {

using rwkv7_fast_v4::check_hip;
using rwkv7_fast_v4::DeviceBuffer;
using rwkv7_fast_v4::ModelDims;

struct Spec {
  ModelDims dims;
  int fmt = RWKV_FMT_F16;
  std::uint64_t seed = 1;
  std::string name;
  std::string checkpoint;  // empty: synthetic weights
};

ModelDims preset(const std::string& name) {
  ModelDims d;
  if (name == "tiny") {
    d.layers = 2; d.channels = 256; d.heads = 4; d.ffn = 1024; d.vocab = 2048;
    d.rank_w = 32; d.rank_a = 32; d.rank_g = 64; d.rank_v = 16;
  } else if (name == "0.1B") {
    d.layers = 12; d.channels = 768; d.heads = 12; d.ffn = 3072; d.vocab = 65536;
    d.rank_w = 64; d.rank_a = 64; d.rank_g = 128; d.rank_v = 32;
  } else if (name == "1.5B") {
    d.layers = 24; d.channels = 2048; d.heads = 32; d.ffn = 8192; d.vocab = 65536;
    d.rank_w = 96; d.rank_a = 96; d.rank_g = 256; d.rank_v = 64;
  } else if (name == "7.2B") {
    d.layers = 32; d.channels = 4096; d.heads = 64; d.ffn = 16384; d.vocab = 65536;
    d.rank_w = 128; d.rank_a = 128; d.rank_g = 480; d.rank_v = 96;
  } else {
    throw std::runtime_error("unknown synthetic model preset: " + name);
  }
  return d;
}

// <file>.pth[:f16|:w8|:w4] - the weight format the big matrices are quantised to on load (default fp16, the
// reference's only one); the model name is the file stem, as in the reference (src/rwkv7_fast_v4.cu:1353-1362).
Spec parse_checkpoint_spec(const std::string& path) {
  Spec spec;
  spec.checkpoint = path;
  const std::size_t colon = path.rfind(':');
  if (colon != std::string::npos) {
    const std::string tail = path.substr(colon + 1);
    const int fmt = tail == "f16" ? RWKV_FMT_F16 : tail == "w8" ? RWKV_FMT_W8 : tail == "w4" ? RWKV_FMT_W4 : -1;
    if (fmt >= 0) {
      spec.fmt = fmt;
      spec.checkpoint = path.substr(0, colon);
    }
  }
  const std::size_t slash = spec.checkpoint.find_last_of('/');
  std::string stem = slash == std::string::npos ? spec.checkpoint : spec.checkpoint.substr(slash + 1);
  const std::size_t dot = stem.rfind('.');
  if (dot != std::string::npos && dot > 0) stem.resize(dot);
  spec.name = stem;
  return spec;
}

Spec parse_spec(const std::string& path) {
  const std::string prefix = "synthetic:";
  if (path.compare(0, prefix.size(), prefix) != 0) return parse_checkpoint_spec(path);
  Spec spec;
  std::stringstream ss(path.substr(prefix.size()));
  std::string part;
  int index = 0;
  while (std::getline(ss, part, ':')) {
    if (index == 0) {
      spec.dims = preset(part);
      spec.name = "synthetic-" + part;
    } else if (part == "f16") {
      spec.fmt = RWKV_FMT_F16;
    } else if (part == "w8") {
      spec.fmt = RWKV_FMT_W8;
    } else if (part == "w4") {
      spec.fmt = RWKV_FMT_W4;
    } else if (part.compare(0, 5, "seed=") == 0) {
      spec.seed = std::stoull(part.substr(5));
    } else {
      throw std::runtime_error("bad synthetic model option: " + part);
    }
    ++index;
  }
  if (index == 0) throw std::runtime_error("empty synthetic model spec");
  return spec;
}

}  // namespace

struct ModelBackend::Impl {
  std::string model_path;
  bool use_wkv32 = false;  // false: the WKV state is fp16 (the reference's default), true: fp32
  std::string model_name;
  Spec spec;
  rwkv_hip_model* model = nullptr;
  std::vector<DeviceBuffer<std::uint8_t>> storage;  // owns every weight tensor
  std::uint64_t fill_counter = 0;
  std::string archive_folder;       // "<folder>/data.pkl" names the checkpoint's top folder

  // Staging of the checkpoint loader (the reference's copy/compute stream pairs with two pinned buffers,
  // src/rwkv7_fast_v4.cu:110-181,212-290).  A tensor travels in pieces of 64 MiB through two pinned host buffers:
  // while one piece is on its way to the device (copy stream) the host reads the next piece from the file into
  // the other buffer.  The pieces land in one of two device buffers for the bf16 patterns, so that the conversion
  // kernel of one tensor (NULL stream, ordered behind the tensor's last copy through an event) runs while the next
  // tensor is being read and copied; a device buffer is reused once the event recorded behind its conversion
  // kernel has happened.
  static constexpr std::size_t kPieceBytes = std::size_t(64) << 20;
  struct PinnedPiece {
    void* host = nullptr;
    void* copied = nullptr;  // event on the copy stream: the piece has left the buffer
    bool in_flight = false;
  };
  struct StageSlot {
    DeviceBuffer<std::uint16_t> dev;
    void* arrived = nullptr;   // event on the copy stream: the device buffer holds the whole tensor
    void* consumed = nullptr;  // event on the NULL stream: the kernel that read the device buffer has run
    bool in_use = false;
  };
  PinnedPiece piece[2];
  int piece_next = 0;
  StageSlot stage[2];
  int stage_next = 0;
  rwkv_stream_t copy_stream = nullptr;
  std::vector<DeviceBuffer<std::uint8_t>> retired;  // fp16 sources of quantised matrices, freed in batches
  std::size_t retired_bytes = 0;
  std::uint64_t loaded_bytes = 0;                   // bf16 bytes that went through the staging
  bool chunk_loading = false;                       // the archive is read on demand (pread) rather than held in memory

  mutable std::mutex pool_mutex;
  mutable std::vector<rwkv_hip_session*> idle_sessions;

  ~Impl() {
    for (auto* s : idle_sessions) rwkv_hip_session_destroy(s);
    release_staging();
    if (model) rwkv_hip_model_destroy(model);
  }

  void* alloc(std::size_t bytes, const char* what) {
    storage.emplace_back();
    storage.back().resize(bytes, what);
    return storage.back().p;
  }

  void* fill(std::size_t elems, float mean, float stdv) {
    void* p = alloc(elems * sizeof(half), "alloc synthetic weight");
    check_hip(rwkv_hip_fill_normal_f16(nullptr, static_cast<int64_t>(elems), spec.seed * 1000003ull + (++fill_counter),
                                       mean, stdv, p),
              "fill synthetic weight");
    return p;
  }

  void set_matrix(int layer, int id, int N, int K) { install_matrix(layer, id, N, K, fill(static_cast<std::size_t>(N) * K, 0.0f, 0.02f)); }

  // w16: fp16 [N,K] in `storage`; kept as the weight for fp16, else quantised on the device and released
  void install_matrix(int layer, int id, int N, int K, void* w16) {
    if (spec.fmt == RWKV_FMT_F16) {
      check_hip(rwkv_hip_model_set_matrix(model, layer, id, RWKV_FMT_F16, w16, nullptr, nullptr), "set matrix");
      return;
    }
    if (spec.fmt == RWKV_FMT_W8) {
      void* q = alloc(static_cast<std::size_t>(N) * K, "alloc int8 codes");
      void* s = alloc(static_cast<std::size_t>(N) * sizeof(half), "alloc scales");
      check_hip(rwkv_hip_quantize_w8(nullptr, N, K, w16, q, s), "quantize_w8");
      check_hip(rwkv_hip_model_set_matrix(model, layer, id, RWKV_FMT_W8, q, s, nullptr), "set matrix");
    } else {
      void* q = alloc(static_cast<std::size_t>(N) * K / 2, "alloc int4 codes");
      void* s = alloc(static_cast<std::size_t>(N) * (K / 128) * sizeof(half), "alloc scales");
      void* z = alloc(static_cast<std::size_t>(N) * (K / 128), "alloc zero points");
      check_hip(rwkv_hip_quantize_w4(nullptr, N, K, w16, q, s, z), "quantize_w4");
      check_hip(rwkv_hip_model_set_matrix(model, layer, id, RWKV_FMT_W4, q, s, z), "set matrix");
    }
    // the fp16 source is no longer needed once the quantisation kernel has run: it is set aside and freed with
    // others of its kind after one device sync per 2 GiB (a sync per matrix would stall the load pipeline)
    for (auto it = storage.rbegin(); it != storage.rend(); ++it) {
      if (it->p == static_cast<std::uint8_t*>(w16)) {
        retired_bytes += it->n;
        retired.push_back(std::move(*it));
        *it = DeviceBuffer<std::uint8_t>();
        break;
      }
    }
    if (retired_bytes > (std::size_t(2) << 30)) free_retired();
  }

  void free_retired() {
    if (retired.empty()) return;
    check_hip(rwkv_hip_device_sync(), "sync before releasing fp16 sources");
    retired.clear();
    retired_bytes = 0;
  }

  void release_staging() {
    for (PinnedPiece& pc : piece) {
      if (pc.host) rwkv_hip_host_free(pc.host);
      if (pc.copied) rwkv_hip_event_destroy(pc.copied);
      pc = PinnedPiece();
    }
    for (StageSlot& slot : stage) {
      if (slot.arrived) rwkv_hip_event_destroy(slot.arrived);
      if (slot.consumed) rwkv_hip_event_destroy(slot.consumed);
      slot = StageSlot();
    }
    if (copy_stream) rwkv_hip_stream_destroy(copy_stream);
    copy_stream = nullptr;
  }

  // ---- checkpoint ------------------------------------------------------------------------------------------
  [[noreturn]] static void load_error(const std::string& what) { throw std::runtime_error("load model: " + what); }

  // File bytes [offset, offset + bytes) of a stored entry into host memory.  From the whole-file copy large ranges
  // are copied by four threads (0.14 -> 0.05 s for 2.7 GB); reads from the file itself stay on one thread - four
  // concurrent preads of one file were slower than one (0.75 s against 0.51 s for the same 2.7 GB out of the page
  // cache).
  static void read_range(const llm_infer::PthArchive& archive, const llm_infer::PthEntry& entry, std::uint64_t offset,
                         void* dst, std::size_t bytes, bool from_memory) {
    constexpr std::size_t kParallelFrom = std::size_t(16) << 20;
    constexpr int kReaders = 4;
    if (bytes < kParallelFrom || !from_memory) {
      llm_infer::Status rd = archive.read_stored_entry_range(entry, offset, dst, bytes);
      if (!rd.ok_status()) load_error(rd.message());
      return;
    }
    std::string errors[kReaders];
    std::vector<std::thread> readers;
    const std::size_t piece = ((bytes / kReaders) + 4095) & ~std::size_t(4095);
    for (int i = 0; i < kReaders; ++i) {
      const std::size_t from = std::min(bytes, piece * i);
      const std::size_t len = std::min(bytes - from, piece);
      if (len == 0) continue;
      readers.emplace_back([&archive, &entry, &errors, i, offset, dst, from, len] {
        llm_infer::Status rd = archive.read_stored_entry_range(entry, offset + from, static_cast<char*>(dst) + from, len);
        if (!rd.ok_status()) errors[i] = rd.message();
      });
    }
    for (auto& t : readers) t.join();
    for (const std::string& e : errors)
      if (!e.empty()) load_error(e);
  }

  // The next device staging buffer, free for reuse and with room for `bytes`.
  StageSlot& take_slot(std::size_t bytes) {
    if (copy_stream == nullptr) {
      check_hip(rwkv_hip_stream_create(&copy_stream), "create copy stream");
      for (PinnedPiece& pc : piece) {
        check_hip(rwkv_hip_host_alloc(&pc.host, kPieceBytes), "alloc pinned staging");
        check_hip(rwkv_hip_event_create(&pc.copied), "create staging event");
      }
      for (StageSlot& slot : stage) {
        check_hip(rwkv_hip_event_create(&slot.arrived), "create staging event");
        check_hip(rwkv_hip_event_create(&slot.consumed), "create staging event");
      }
    }
    StageSlot& slot = stage[stage_next];
    stage_next ^= 1;
    if (slot.in_use) check_hip(rwkv_hip_event_sync(slot.consumed), "wait for staging slot");
    slot.in_use = false;
    if (bytes > slot.dev.n * 2) {
      slot.dev = DeviceBuffer<std::uint16_t>();  // (freeing waits for the device: rare, the largest tensors come first)
      slot.dev.resize((bytes + 1) / 2, "alloc bf16 staging");
    }
    return slot;
  }

  // One piece (at most kPieceBytes) into a pinned buffer by `fill`, then on its way to `dst` on the copy stream.
  template <class Fill>
  void send_piece(void* dst, std::size_t bytes, Fill&& fill) {
    PinnedPiece& pc = piece[piece_next];
    piece_next ^= 1;
    if (pc.in_flight) check_hip(rwkv_hip_event_sync(pc.copied), "wait for pinned buffer");
    fill(pc.host);
    check_hip(rwkv_hip_memcpy_h2d_async(copy_stream, dst, pc.host, bytes), "copy bf16 weight");
    check_hip(rwkv_hip_event_record(pc.copied, copy_stream), "record copy event");
    pc.in_flight = true;
  }

  // The tensor's bf16 patterns in logical order in a staging slot's device buffer: valid until the slot comes
  // round again (two uploads later); the caller enqueues the kernel that reads them on the NULL stream and then
  // calls consumed(slot).  Returns the slot; *count receives the number of elements.
  StageSlot& upload_bf16(const llm_infer::PthArchive& archive, const llm_infer::TensorRecord& rec, std::size_t* count) {
    // Row-major tensors (all of a normal checkpoint): the byte range goes from the file into the pinned buffers and
    // from there to the device, no per-element pass on the host.
    std::uint64_t n = 1;
    std::int64_t expect = 1;
    bool dense = rec.shape.size() == rec.stride.size();
    for (std::size_t i = rec.shape.size(); dense && i-- > 0;) {
      if (rec.shape[i] < 0) dense = false;
      if (rec.shape[i] != 1 && rec.stride[i] != expect) dense = false;
      expect *= rec.shape[i];
      n *= static_cast<std::uint64_t>(rec.shape[i]);
    }
    const llm_infer::PthEntry* entry = dense && n > 0 ? archive.find_entry(archive_folder + "/data/" + rec.storage_key) : nullptr;
    StageSlot* slot = nullptr;
    std::size_t bytes = 0;
    if (entry != nullptr && entry->is_stored() && entry->uncompressed_size == rec.storage_size * 2 &&
        rec.storage_offset + n <= rec.storage_size) {
      bytes = static_cast<std::size_t>(n) * 2;
      slot = &take_slot(bytes);
      for (std::size_t at = 0; at < bytes; at += kPieceBytes) {
        const std::size_t len = std::min(kPieceBytes, bytes - at);
        send_piece(reinterpret_cast<char*>(slot->dev.p) + at, len, [&](void* host) {
          read_range(archive, *entry, rec.storage_offset * 2 + at, host, len, !chunk_loading);
        });
      }
    } else {
      auto data = llm_infer::load_bf16_tensor_select(archive, rec, true, false, false);
      if (!data.ok()) load_error(data.status().message());
      n = data.value().values_bf16.size();
      bytes = static_cast<std::size_t>(n) * 2;
      slot = &take_slot(bytes);
      const char* src = reinterpret_cast<const char*>(data.value().values_bf16.data());
      for (std::size_t at = 0; at < bytes; at += kPieceBytes) {
        const std::size_t len = std::min(kPieceBytes, bytes - at);
        send_piece(reinterpret_cast<char*>(slot->dev.p) + at, len, [&](void* host) { std::memcpy(host, src + at, len); });
      }
    }
    if (bytes) {
      check_hip(rwkv_hip_event_record(slot->arrived, copy_stream), "record copy event");
      check_hip(rwkv_hip_stream_wait_event(nullptr, slot->arrived), "order conversion behind the copy");
    }
    loaded_bytes += bytes;
    *count = static_cast<std::size_t>(n);
    return *slot;
  }

  void consumed(StageSlot& slot) {
    check_hip(rwkv_hip_event_record(slot.consumed, nullptr), "record staging event");
    slot.in_use = true;
  }

  // fp16 copy of a checkpoint tensor in `storage`: elements as they are, or a [rows,cols] matrix into [cols,rows]
  void* convert(const llm_infer::PthArchive& archive, const llm_infer::TensorRecord& rec, std::size_t elems, int t_rows,
                int t_cols) {
    std::size_t n = 1;
    for (std::int64_t d : rec.shape) n *= static_cast<std::size_t>(d);
    if (n != elems) {
      load_error("tensor " + rec.name + " has shape " + llm_infer::shape_string(rec.shape) + ", expected " +
                 std::to_string(elems) + " elements");
    }
    if (t_rows > 0 && (rec.shape.size() != 2 || rec.shape[0] != t_rows || rec.shape[1] != t_cols)) {
      load_error("tensor " + rec.name + " has shape " + llm_infer::shape_string(rec.shape) + ", expected [" +
                 std::to_string(t_rows) + "," + std::to_string(t_cols) + "]");
    }
    void* out = alloc(elems * sizeof(half), "alloc weight tensor");
    std::size_t count = 0;
    StageSlot& raw = upload_bf16(archive, rec, &count);
    if (count != elems) load_error("tensor " + rec.name + " has " + std::to_string(count) + " stored elements");
    if (t_rows > 0) {
      check_hip(rwkv_hip_bf16_to_f16_transpose(nullptr, t_rows, t_cols, raw.dev.p, out), "bf16 -> f16 transpose");
    } else {
      check_hip(rwkv_hip_bf16_to_f16(nullptr, static_cast<int64_t>(elems), raw.dev.p, out), "bf16 -> f16");
    }
    consumed(raw);
    return out;
  }

  void load_checkpoint(bool chunk_load) {
    const auto t_start = std::chrono::steady_clock::now();
    chunk_loading = chunk_load;
    auto opened = llm_infer::PthArchive::open(spec.checkpoint, chunk_load);
    if (!opened.ok()) load_error(opened.status().message());
    const llm_infer::PthArchive& archive = opened.value();
    auto parsed = llm_infer::parse_pth_tensor_records(archive);
    if (!parsed.ok()) load_error(parsed.status().message());
    for (const auto& e : archive.entries()) {
      static const std::string kTail = "/data.pkl";
      if (e.name.size() >= kTail.size() && e.name.compare(e.name.size() - kTail.size(), kTail.size(), kTail) == 0) {
        archive_folder = e.name.substr(0, e.name.size() - kTail.size());
        break;
      }
    }
    std::unordered_map<std::string, const llm_infer::TensorRecord*> by_name;
    for (const auto& rec : parsed.value()) by_name[rec.name] = &rec;
    auto find = [&](const std::string& name) -> const llm_infer::TensorRecord* {
      auto it = by_name.find(name);
      return it == by_name.end() ? nullptr : it->second;
    };
    auto need = [&](const std::string& name) -> const llm_infer::TensorRecord& {
      const llm_infer::TensorRecord* rec = find(name);
      if (rec == nullptr) load_error("missing tensor: " + name);
      return *rec;
    };

    // dimensions from tensor shapes (infer_model_dims, include/rwkv7_fast_v4_common.hpp:262-288; LoRA ranks from
    // the rank-in matrices, src/rwkv7_fast_v4.cu:1168-1172)
    ModelDims d;
    for (const auto& rec : parsed.value()) {
      if (rec.name.compare(0, 7, "blocks.") == 0) {
        char* end = nullptr;
        const long layer = std::strtol(rec.name.c_str() + 7, &end, 10);
        if (end && *end == '.' && layer >= 0) d.layers = std::max(d.layers, static_cast<int>(layer) + 1);
      }
    }
    if (const auto* emb = find("emb.weight"); emb && emb->shape.size() == 2) {
      d.vocab = static_cast<int>(emb->shape[0]);
      d.channels = static_cast<int>(emb->shape[1]);
    }
    if (const auto* rk = find("blocks.0.att.r_k"); rk && rk->shape.size() == 2) {
      d.heads = static_cast<int>(rk->shape[0]);
      d.head_size = static_cast<int>(rk->shape[1]);
    }
    if (const auto* key = find("blocks.0.ffn.key.weight"); key && key->shape.size() == 2) d.ffn = static_cast<int>(key->shape[0]);
    if (!(d.layers > 0 && d.channels > 0 && d.heads > 0 && d.head_size > 0 && d.vocab > 0 && d.ffn > 0)) {
      load_error("could not infer model dimensions");
    }
    if (d.channels != d.heads * d.head_size) load_error("C must equal H*N");
    if (d.head_size != 64) load_error("current kernels require head size 64");
    auto rank_of = [&](const std::string& name) {
      const llm_infer::TensorRecord* rec = find(name);
      if (rec == nullptr || rec->shape.size() != 2 || rec->shape[0] != d.channels) load_error("missing or misshapen tensor: " + name);
      if (rec->shape[1] <= 0 || rec->shape[1] > 512) load_error("LoRA rank of " + name + " must be in 1..512");
      return static_cast<int>(rec->shape[1]);
    };
    d.rank_w = rank_of("blocks.0.att.w1");
    d.rank_a = rank_of("blocks.0.att.a1");
    d.rank_g = rank_of("blocks.0.att.g1");
    d.rank_v = rank_of(d.layers > 1 ? "blocks.1.att.v1" : "blocks.0.att.v1");
    spec.dims = d;

    check_hip(rwkv_hip_model_create(&model, d.layers, d.channels, d.heads, d.ffn, d.vocab, d.rank_w, d.rank_a, d.rank_g,
                                    d.rank_v),
              "create model");
    const std::size_t C = static_cast<std::size_t>(d.channels);
    const int Ci = d.channels;
    auto vector = [&](int layer, int id, const std::string& name) {
      check_hip(rwkv_hip_model_set_tensor(model, layer, id, convert(archive, need(name), C, 0, 0)), "set tensor");
    };
    auto matrix = [&](int layer, int id, const std::string& name, int N, int K) {
      const llm_infer::TensorRecord& rec = need(name);
      if (rec.shape.size() != 2 || rec.shape[0] != N || rec.shape[1] != K) {
        load_error("tensor " + name + " has shape " + llm_infer::shape_string(rec.shape) + ", expected [" + std::to_string(N) +
                   "," + std::to_string(K) + "]");
      }
      install_matrix(layer, id, N, K, convert(archive, rec, static_cast<std::size_t>(N) * K, 0, 0));
    };

    {  // embedding rows through ln0, once (build_cpu_emb_ln0_f16, src/rwkv7_fast_v4.cu:450-572)
      const llm_infer::TensorRecord& emb = need("emb.weight");
      const llm_infer::TensorRecord& w = need("blocks.0.ln0.weight");
      const llm_infer::TensorRecord& b = need("blocks.0.ln0.bias");
      // three tensors at once, two staging slots: the two vectors are copied out of their slots first
      DeviceBuffer<std::uint16_t> wb;
      wb.resize(2 * C, "alloc ln0 vectors");
      std::size_t n_w = 0, n_b = 0, n_emb = 0;
      StageSlot& w_raw = upload_bf16(archive, w, &n_w);
      if (n_w != C) load_error("emb/ln0 shape mismatch for emb+ln0 preprocessing");
      check_hip(rwkv_hip_memcpy_d2d_async(nullptr, wb.p, w_raw.dev.p, C * 2), "copy ln0 weight");
      consumed(w_raw);
      StageSlot& b_raw = upload_bf16(archive, b, &n_b);
      if (n_b != C) load_error("emb/ln0 shape mismatch for emb+ln0 preprocessing");
      check_hip(rwkv_hip_memcpy_d2d_async(nullptr, wb.p + C, b_raw.dev.p, C * 2), "copy ln0 bias");
      consumed(b_raw);
      StageSlot& emb_raw = upload_bf16(archive, emb, &n_emb);
      if (n_emb != static_cast<std::size_t>(d.vocab) * C) load_error("emb/ln0 shape mismatch for emb+ln0 preprocessing");
      void* out = alloc(n_emb * sizeof(half), "alloc emb+ln0");
      check_hip(rwkv_hip_emb_ln0_bf16_to_f16(nullptr, d.vocab, Ci, emb_raw.dev.p, wb.p, wb.p + C, 1e-5f, out), "emb+ln0 preprocess");
      consumed(emb_raw);
      check_hip(rwkv_hip_device_sync(), "sync emb+ln0 preprocess");  // wb is released here
      check_hip(rwkv_hip_model_set_tensor(model, -1, RWKV_T_EMB_LN0, out), "set tensor");
    }
    vector(-1, RWKV_T_LN_OUT_W, "ln_out.weight");
    vector(-1, RWKV_T_LN_OUT_B, "ln_out.bias");
    matrix(-1, RWKV_M_HEAD, "head.weight", d.vocab, Ci);

    struct Named { int id; const char* suffix; };
    static const Named vectors[] = {
        {RWKV_T_LN1_W, "ln1.weight"}, {RWKV_T_LN1_B, "ln1.bias"}, {RWKV_T_LN2_W, "ln2.weight"}, {RWKV_T_LN2_B, "ln2.bias"},
        {RWKV_T_X_R, "att.x_r"}, {RWKV_T_X_W, "att.x_w"}, {RWKV_T_X_K, "att.x_k"}, {RWKV_T_X_V, "att.x_v"},
        {RWKV_T_X_A, "att.x_a"}, {RWKV_T_X_G, "att.x_g"}, {RWKV_T_W0, "att.w0"}, {RWKV_T_A0, "att.a0"},
        {RWKV_T_K_K, "att.k_k"}, {RWKV_T_K_A, "att.k_a"}, {RWKV_T_R_K, "att.r_k"}, {RWKV_T_LNX_W, "att.ln_x.weight"},
        {RWKV_T_LNX_B, "att.ln_x.bias"}, {RWKV_T_FFN_X_K, "ffn.x_k"}};
    // LoRA pairs: the file has the rank-in as [C,R] and the rank-out as [R,C]; the kernels read both transposed
    // ("out,in": [R,C] and [C,R] - the reference's `_t` copies, include/rwkv7_fast_v4_common.hpp:326-338)
    struct Lora { int in_id, out_id; const char* in_name; const char* out_name; int ModelDims::*rank; };
    static const Lora loras[] = {{RWKV_T_W1, RWKV_T_W2, "att.w1", "att.w2", &ModelDims::rank_w},
                                 {RWKV_T_A1, RWKV_T_A2, "att.a1", "att.a2", &ModelDims::rank_a},
                                 {RWKV_T_G1, RWKV_T_G2, "att.g1", "att.g2", &ModelDims::rank_g},
                                 {RWKV_T_V1, RWKV_T_V2, "att.v1", "att.v2", &ModelDims::rank_v}};
    for (int l = 0; l < d.layers; ++l) {
      const std::string p = "blocks." + std::to_string(l) + ".";
      for (const Named& v : vectors) vector(l, v.id, p + v.suffix);
      for (const Lora& lo : loras) {
        const bool value_residual = lo.in_id == RWKV_T_V1;
        if (value_residual && l == 0) continue;  // unused in the first layer (unused_weight_like_v3a, :318-323)
        const int R = d.*(lo.rank);
        check_hip(rwkv_hip_model_set_tensor(model, l, lo.in_id, convert(archive, need(p + lo.in_name), C * R, Ci, R)), "set tensor");
        check_hip(rwkv_hip_model_set_tensor(model, l, lo.out_id, convert(archive, need(p + lo.out_name), C * R, R, Ci)), "set tensor");
        if (value_residual) vector(l, RWKV_T_V0, p + "att.v0");
      }
      matrix(l, RWKV_M_ATT_R, p + "att.receptance.weight", Ci, Ci);
      matrix(l, RWKV_M_ATT_K, p + "att.key.weight", Ci, Ci);
      matrix(l, RWKV_M_ATT_V, p + "att.value.weight", Ci, Ci);
      matrix(l, RWKV_M_ATT_O, p + "att.output.weight", Ci, Ci);
      matrix(l, RWKV_M_FFN_KEY, p + "ffn.key.weight", d.ffn, Ci);
      matrix(l, RWKV_M_FFN_VALUE, p + "ffn.value.weight", Ci, d.ffn);  // the file's own [C,F] layout
    }
    check_hip(rwkv_hip_device_sync(), "sync model build");
    free_retired();
    release_staging();
    const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t_start).count();
    std::printf("[ModelBackend] %s: %.2f GB of bf16 tensors read, converted%s in %.2f s (%.2f GB/s)\n", model_name.c_str(),
                loaded_bytes * 1e-9, spec.fmt == RWKV_FMT_F16 ? "" : " and quantised", seconds,
                seconds > 0 ? loaded_bytes * 1e-9 / seconds : 0.0);
  }

  void build() {
    const ModelDims& d = spec.dims;
    check_hip(rwkv_hip_model_create(&model, d.layers, d.channels, d.heads, d.ffn, d.vocab, d.rank_w, d.rank_a, d.rank_g,
                                    d.rank_v),
              "create model");
    const std::size_t C = static_cast<std::size_t>(d.channels);
    auto tensor = [&](int layer, int id, std::size_t elems, float mean, float stdv) {
      check_hip(rwkv_hip_model_set_tensor(model, layer, id, fill(elems, mean, stdv)), "set tensor");
    };
    tensor(-1, RWKV_T_EMB_LN0, static_cast<std::size_t>(d.vocab) * C, 0.0f, 1.0f);
    tensor(-1, RWKV_T_LN_OUT_W, C, 1.0f, 0.02f);
    tensor(-1, RWKV_T_LN_OUT_B, C, 0.0f, 0.02f);
    set_matrix(-1, RWKV_M_HEAD, d.vocab, d.channels);
    for (int l = 0; l < d.layers; ++l) {
      for (int id : {RWKV_T_LN1_W, RWKV_T_LN2_W, RWKV_T_LNX_W, RWKV_T_K_K, RWKV_T_K_A}) tensor(l, id, C, 1.0f, 0.02f);
      for (int id : {RWKV_T_LN1_B, RWKV_T_LN2_B, RWKV_T_LNX_B, RWKV_T_A0, RWKV_T_V0, RWKV_T_R_K}) tensor(l, id, C, 0.0f, 0.02f);
      for (int id : {RWKV_T_X_R, RWKV_T_X_W, RWKV_T_X_K, RWKV_T_X_V, RWKV_T_X_A, RWKV_T_X_G, RWKV_T_FFN_X_K})
        tensor(l, id, C, 0.5f, 0.15f);
      tensor(l, RWKV_T_W0, C, -2.0f, 1.5f);
      const int ranks[4] = {d.rank_w, d.rank_a, d.rank_g, d.rank_v};
      const int in_ids[4] = {RWKV_T_W1, RWKV_T_A1, RWKV_T_G1, RWKV_T_V1};
      const int out_ids[4] = {RWKV_T_W2, RWKV_T_A2, RWKV_T_G2, RWKV_T_V2};
      for (int i = 0; i < 4; ++i) {
        tensor(l, in_ids[i], static_cast<std::size_t>(ranks[i]) * C, 0.0f, 0.08f);
        tensor(l, out_ids[i], static_cast<std::size_t>(ranks[i]) * C, 0.0f, 0.08f);
      }
      set_matrix(l, RWKV_M_ATT_R, d.channels, d.channels);
      set_matrix(l, RWKV_M_ATT_K, d.channels, d.channels);
      set_matrix(l, RWKV_M_ATT_V, d.channels, d.channels);
      set_matrix(l, RWKV_M_ATT_O, d.channels, d.channels);
      set_matrix(l, RWKV_M_FFN_KEY, d.ffn, d.channels);
      set_matrix(l, RWKV_M_FFN_VALUE, d.channels, d.ffn);
    }
    check_hip(rwkv_hip_device_sync(), "sync model build");
  }

  rwkv_hip_session* acquire() const {
    {
      std::lock_guard<std::mutex> lock(pool_mutex);
      if (!idle_sessions.empty()) {
        rwkv_hip_session* s = idle_sessions.back();
        idle_sessions.pop_back();
        return s;
      }
    }
    rwkv_hip_session* s = nullptr;
    check_hip(rwkv_hip_session_create(&s, model), "create session");
    return s;
  }

  void release(rwkv_hip_session* s) const {
    std::lock_guard<std::mutex> lock(pool_mutex);
    idle_sessions.push_back(s);
  }

  void forward(const std::vector<int64_t>& flat, int B, int T, GenerationState& state, DeviceLogits& out) const {
    const int V = spec.dims.vocab;
    out.values.resize_recycled(static_cast<std::size_t>(B) * V, "alloc backend logits f32");
    rwkv_hip_session* s = acquire();
    int rc = rwkv_hip_session_set_wkv_fp16(s, use_wkv32 ? 0 : 1);
    if (rc == RWKV_OK) {
      void* wkv = use_wkv32 ? static_cast<void*>(state.wkv_state32.p) : static_cast<void*>(state.wkv_state.p);
      rc = rwkv_hip_forward(s, flat.data(), B, T, state.shift.p, wkv, state.elapsed.p, out.values.p, 1);
    }
    const std::string msg = rc == RWKV_OK ? std::string() : std::string(rwkv_hip_last_error());
    release(s);
    if (rc != RWKV_OK) throw std::runtime_error(msg);
    out.rows = B;
    out.vocab_size = V;
  }
};

ModelBackend::ModelBackend(std::string model_path, bool use_wkv32, bool chunk_load) : impl_(std::make_unique<Impl>()) {
  impl_->use_wkv32 = use_wkv32;
  impl_->model_path = std::move(model_path);
  impl_->spec = parse_spec(impl_->model_path);
  impl_->model_name = impl_->spec.name;
  if (impl_->spec.checkpoint.empty()) {
    impl_->build();
  } else {
    impl_->load_checkpoint(chunk_load);
  }
}

ModelBackend::~ModelBackend() = default;
ModelBackend::ModelBackend(ModelBackend&&) noexcept = default;
ModelBackend& ModelBackend::operator=(ModelBackend&&) noexcept = default;

GenerationState ModelBackend::create_state(int batch_size) const {
  if (batch_size <= 0) throw std::runtime_error("batch_size must be positive");
  const ModelDims& d = impl_->spec.dims;
  GenerationState state;
  state.batch_size = batch_size;
  state.wkv32 = impl_->use_wkv32;   // src/rwkv7_fast_v4.cu:1379-1396: one of the two state tensors, by mode
  state.shift.resize_recycled(static_cast<std::size_t>(d.layers) * 2 * batch_size * d.channels, "alloc backend shift state");
  const std::size_t state_elems = static_cast<std::size_t>(d.layers) * batch_size * d.heads * d.head_size * d.head_size;
  if (impl_->use_wkv32) {
    state.wkv_state32.resize_recycled(state_elems, "alloc backend wkv32 state");
  } else {
    state.wkv_state.resize_recycled(state_elems, "alloc backend wkv state");
  }
  state.elapsed.resize_recycled(batch_size, "alloc backend elapsed");
  state.shift.zero("zero backend shift");
  if (impl_->use_wkv32) {
    state.wkv_state32.zero("zero backend wkv32");
  } else {
    state.wkv_state.zero("zero backend wkv");
  }
  state.elapsed.zero("zero backend elapsed");
  check_hip(rwkv_hip_device_sync(), "sync backend state init");
  return state;
}

void ModelBackend::forward_prefill(const std::vector<std::vector<int64_t>>& token_batches, GenerationState& state,
                                   DeviceLogits& logits) const {
  const int B = static_cast<int>(token_batches.size());
  if (B <= 0) throw std::runtime_error("token_batches must not be empty");
  if (state.batch_size != B) throw std::runtime_error("state batch size mismatch");
  if (state.wkv32 != impl_->use_wkv32) throw std::runtime_error("state wkv precision mismatch");  // :1060-1062
  const int T = static_cast<int>(token_batches.front().size());
  if (T <= 0) throw std::runtime_error("token batch length must be positive");
  std::vector<int64_t> flat;
  flat.reserve(static_cast<std::size_t>(B) * T);
  for (const auto& row : token_batches) {
    if (static_cast<int>(row.size()) != T) throw std::runtime_error("all token batches must share the same length");
    flat.insert(flat.end(), row.begin(), row.end());
  }
  impl_->forward(flat, B, T, state, logits);
}

void ModelBackend::forward_decode(const std::vector<int64_t>& token_batch, GenerationState& state,
                                  DeviceLogits& logits) const {
  const int B = static_cast<int>(token_batch.size());
  if (B <= 0) throw std::runtime_error("token_batches must not be empty");
  if (state.batch_size != B) throw std::runtime_error("state batch size mismatch");
  if (state.wkv32 != impl_->use_wkv32) throw std::runtime_error("state wkv precision mismatch");
  impl_->forward(token_batch, B, 1, state, logits);
}

void ModelBackend::copy_state_slice(const GenerationState& src, int src_offset, GenerationState& dst, int dst_offset,
                                    int count) const {
  if (src_offset < 0 || dst_offset < 0 || count <= 0) throw std::runtime_error("invalid backend state slice range");
  if (src.batch_size <= 0 || dst.batch_size <= 0)
    throw std::runtime_error("state slice requires non-empty source and destination");
  if (src.wkv32 != dst.wkv32 || src.wkv32 != impl_->use_wkv32)
    throw std::runtime_error("state slice wkv precision mismatch");  // src/rwkv7_fast_v4.cu:1433-1435
  if (src_offset + count > src.batch_size || dst_offset + count > dst.batch_size)
    throw std::runtime_error("state slice range exceeds batch size");

  const ModelDims& d = impl_->spec.dims;
  const std::size_t C = static_cast<std::size_t>(d.channels);
  const std::size_t lane = static_cast<std::size_t>(d.heads) * d.head_size * d.head_size;
  for (int layer = 0; layer < d.layers; ++layer) {
    for (int which = 0; which < 2; ++which) {
      const half* s = src.shift.p + (static_cast<std::size_t>(layer) * 2 + which) * src.batch_size * C + src_offset * C;
      half* t = dst.shift.p + (static_cast<std::size_t>(layer) * 2 + which) * dst.batch_size * C + dst_offset * C;
      check_hip(rwkv_hip_memcpy_d2d(t, s, count * C * sizeof(half)), "copy backend state slice shift");
    }
    if (impl_->use_wkv32) {
      const float* s = src.wkv_state32.p + (static_cast<std::size_t>(layer) * src.batch_size + src_offset) * lane;
      float* t = dst.wkv_state32.p + (static_cast<std::size_t>(layer) * dst.batch_size + dst_offset) * lane;
      check_hip(rwkv_hip_memcpy_d2d(t, s, count * lane * sizeof(float)), "copy backend state slice wkv32");
    } else {
      const half* s = src.wkv_state.p + (static_cast<std::size_t>(layer) * src.batch_size + src_offset) * lane;
      half* t = dst.wkv_state.p + (static_cast<std::size_t>(layer) * dst.batch_size + dst_offset) * lane;
      check_hip(rwkv_hip_memcpy_d2d(t, s, count * lane * sizeof(half)), "copy backend state slice wkv");
    }
  }
  check_hip(rwkv_hip_memcpy_d2d(dst.elapsed.p + dst_offset, src.elapsed.p + src_offset, count * sizeof(int)),
            "copy backend state slice elapsed");
}

void ModelBackend::copy_logits_slice(const DeviceLogits& src, int src_offset, DeviceLogits& dst, int dst_offset,
                                     int count) const {
  if (src_offset < 0 || dst_offset < 0 || count <= 0) throw std::runtime_error("invalid backend logits slice range");
  if (src.rows <= 0 || src.vocab_size <= 0 || src.values.p == nullptr)
    throw std::runtime_error("logits slice requires non-empty source");
  if (dst.rows <= 0 || dst.vocab_size != src.vocab_size || dst.values.p == nullptr)
    throw std::runtime_error("logits slice destination shape mismatch");
  if (src_offset + count > src.rows || dst_offset + count > dst.rows)
    throw std::runtime_error("logits slice range exceeds row count");
  const std::size_t V = static_cast<std::size_t>(src.vocab_size);
  check_hip(rwkv_hip_memcpy_d2d(dst.values.p + dst_offset * V, src.values.p + src_offset * V, count * V * sizeof(float)),
            "copy backend logits slice");
}

PrefillCapacity ModelBackend::query_prefill_capacity(int prefill_chunk_size) const {
  if (prefill_chunk_size <= 0) throw std::runtime_error("prefill chunk size must be positive");
  PrefillCapacity cap;
  check_hip(rwkv_hip_mem_info(&cap.free_vram_bytes, &cap.total_vram_bytes), "query prefill device memory");
  const ModelDims& d = impl_->spec.dims;
  const std::size_t L = d.layers, C = d.channels, H = d.heads, N = d.head_size, V = d.vocab, F = d.ffn;
  const std::size_t T = static_cast<std::size_t>(prefill_chunk_size);
  const std::size_t rank_max = std::max(std::max(d.rank_w, d.rank_a), std::max(d.rank_g, d.rank_v));
  const std::size_t state_bytes = L * 2 * C * sizeof(half) + L * H * N * N * (impl_->use_wkv32 ? sizeof(float) : sizeof(half)) +
                                  sizeof(int);  // src/rwkv7_fast_v4.cu:1556
  // one batch lane of the session arena for a chunk of T tokens (csrc/model.hip ensure_arena) + fp32 logits
  const std::size_t arena_bytes = T * C * 2 * 28 + T * rank_max * 2 * 4 + T * F * 2 + C * 2 + T * C * 4 * 5;
  cap.bytes_per_batch = state_bytes + arena_bytes + V * sizeof(float);
  constexpr std::size_t kMinimumReserveBytes = static_cast<std::size_t>(512) << 20;
  cap.reserve_vram_bytes = std::max(kMinimumReserveBytes, cap.free_vram_bytes / 10);
  const std::size_t usable = cap.free_vram_bytes > cap.reserve_vram_bytes ? cap.free_vram_bytes - cap.reserve_vram_bytes : 0;
  const std::size_t max_batch = cap.bytes_per_batch ? usable / cap.bytes_per_batch : 0;
  cap.max_batch_size = static_cast<int>(std::min<std::size_t>(max_batch, std::numeric_limits<int>::max()));
  return cap;
}

int ModelBackend::vocab_size() const { return impl_->spec.dims.vocab; }
const std::string& ModelBackend::model_path() const { return impl_->model_path; }
const std::string& ModelBackend::model_name() const { return impl_->model_name; }
const rwkv7_fast_v4::ModelDims& ModelBackend::dims() const { return impl_->spec.dims; }

}  // namespace rwkv7_server
