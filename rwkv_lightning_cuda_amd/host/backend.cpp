// ModelBackend over the C ABI of librwkv_hip.so.
//
// Mirrors ModelBackend in the reference (src/rwkv7_fast_v4.cu:1349-1592): argument checks and their
// messages, the state layout and zero-initialisation of create_state (:1373-1400), the per-layer strided
// slice copies of copy_state_slice (:1421-1504), copy_logits_slice (:1506-1532) and the capacity formula of
// query_prefill_capacity (:1534-1580).  Differences: weights are synthetic random-init (no .pth reader
// here), only the fp32-state mode exists, device errors throw instead of exiting, and forward passes run
// through pooled sessions (stream + arena + decode graphs) so concurrent callers do not allocate per call.
#include <algorithm>
#include <limits>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <unordered_map>

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

Spec parse_spec(const std::string& path) {
  const std::string prefix = "synthetic:";
  if (path.compare(0, prefix.size(), prefix) != 0) {
    throw std::runtime_error(
        "this backend has no checkpoint reader: model_path must be synthetic:<preset>[:f16|w8|w4][:seed=<n>], got " + path);
  }
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
  std::string model_name;
  Spec spec;
  rwkv_hip_model* model = nullptr;
  std::vector<DeviceBuffer<std::uint8_t>> storage;  // owns every weight tensor
  std::uint64_t fill_counter = 0;

  mutable std::mutex pool_mutex;
  mutable std::vector<rwkv_hip_session*> idle_sessions;

  ~Impl() {
    for (auto* s : idle_sessions) rwkv_hip_session_destroy(s);
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

  void set_matrix(int layer, int id, int N, int K) {
    void* w16 = fill(static_cast<std::size_t>(N) * K, 0.0f, 0.02f);
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
    // the fp16 source is no longer needed once quantised: free it (it is the last storage entry but two/three)
    check_hip(rwkv_hip_device_sync(), "sync after quantise");
    for (auto& buf : storage) {
      if (buf.p == static_cast<std::uint8_t*>(w16)) {
        buf = DeviceBuffer<std::uint8_t>();
        break;
      }
    }
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
    out.values.resize(static_cast<std::size_t>(B) * V, "alloc backend logits f32");
    rwkv_hip_session* s = acquire();
    const int rc = rwkv_hip_forward(s, flat.data(), B, T, state.shift.p, state.wkv_state32.p, state.elapsed.p,
                                    out.values.p, 1);
    const std::string msg = rc == RWKV_OK ? std::string() : std::string(rwkv_hip_last_error());
    release(s);
    if (rc != RWKV_OK) throw std::runtime_error(msg);
    out.rows = B;
    out.vocab_size = V;
  }
};

ModelBackend::ModelBackend(std::string model_path, bool use_wkv32, bool /*chunk_load*/) : impl_(std::make_unique<Impl>()) {
  if (!use_wkv32) {
    throw std::runtime_error("this backend provides the fp32 WKV state only: construct it with use_wkv32 = true");
  }
  impl_->model_path = std::move(model_path);
  impl_->spec = parse_spec(impl_->model_path);
  impl_->model_name = impl_->spec.name;
  impl_->build();
}

ModelBackend::~ModelBackend() = default;
ModelBackend::ModelBackend(ModelBackend&&) noexcept = default;
ModelBackend& ModelBackend::operator=(ModelBackend&&) noexcept = default;

GenerationState ModelBackend::create_state(int batch_size) const {
  if (batch_size <= 0) throw std::runtime_error("batch_size must be positive");
  const ModelDims& d = impl_->spec.dims;
  GenerationState state;
  state.batch_size = batch_size;
  state.wkv32 = true;
  state.shift.resize(static_cast<std::size_t>(d.layers) * 2 * batch_size * d.channels, "alloc backend shift state");
  state.wkv_state32.resize(static_cast<std::size_t>(d.layers) * batch_size * d.heads * d.head_size * d.head_size,
                           "alloc backend wkv32 state");
  state.elapsed.resize(batch_size, "alloc backend elapsed");
  state.shift.zero("zero backend shift");
  state.wkv_state32.zero("zero backend wkv32");
  state.elapsed.zero("zero backend elapsed");
  check_hip(rwkv_hip_device_sync(), "sync backend state init");
  return state;
}

void ModelBackend::forward_prefill(const std::vector<std::vector<int64_t>>& token_batches, GenerationState& state,
                                   DeviceLogits& logits) const {
  const int B = static_cast<int>(token_batches.size());
  if (B <= 0) throw std::runtime_error("token_batches must not be empty");
  if (state.batch_size != B) throw std::runtime_error("state batch size mismatch");
  if (!state.wkv32) throw std::runtime_error("state wkv precision mismatch");
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
  if (!state.wkv32) throw std::runtime_error("state wkv precision mismatch");
  impl_->forward(token_batch, B, 1, state, logits);
}

void ModelBackend::copy_state_slice(const GenerationState& src, int src_offset, GenerationState& dst, int dst_offset,
                                    int count) const {
  if (src_offset < 0 || dst_offset < 0 || count <= 0) throw std::runtime_error("invalid backend state slice range");
  if (src.batch_size <= 0 || dst.batch_size <= 0)
    throw std::runtime_error("state slice requires non-empty source and destination");
  if (!src.wkv32 || !dst.wkv32) throw std::runtime_error("state slice wkv precision mismatch");
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
    const float* s = src.wkv_state32.p + (static_cast<std::size_t>(layer) * src.batch_size + src_offset) * lane;
    float* t = dst.wkv_state32.p + (static_cast<std::size_t>(layer) * dst.batch_size + dst_offset) * lane;
    check_hip(rwkv_hip_memcpy_d2d(t, s, count * lane * sizeof(float)), "copy backend state slice wkv32");
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
  const std::size_t state_bytes = L * 2 * C * sizeof(half) + L * H * N * N * sizeof(float) + sizeof(int);
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
