// Tensor directory (data.pkl) and tensor data of a PyTorch checkpoint (interface: include/pth_tensor.hpp; the
// behaviour restated is the reference's src/pth_tensor.cpp: opcode set :160-217, persistent ids :282-306,
// _rebuild_tensor_v2 :321-343, scalar conversions :644-720, tensor loading :757-849).
//
// The pickle machine keeps a value stack and a memo like the real one, but its values are only what a state dict
// of tensors needs: integers, booleans, None, strings, globals, tuples, dicts, storages and tensors.  A tensor
// enters the result the moment it is stored in a dict under a string key, in file order.
#include "pth_tensor.hpp"

#include <algorithm>
#include <cstdint>
#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <utility>

namespace llm_infer {
namespace {

struct Obj;
using ObjPtr = std::shared_ptr<Obj>;

struct Obj {
  enum Tag { kNone, kMark, kInt, kBool, kStr, kGlobal, kTuple, kDict, kStorage, kTensor } tag = kNone;
  std::int64_t num = 0;          // kInt, kBool
  std::string text;              // kStr; kGlobal: "module.name"; kStorage: key
  std::uint64_t count = 0;       // kStorage: elements
  std::vector<ObjPtr> items;     // kTuple
  TensorRecord tensor;           // kTensor
};

ObjPtr make(Obj::Tag tag) {
  auto o = std::make_shared<Obj>();
  o->tag = tag;
  return o;
}

class PickleError : public std::runtime_error {
public:
  using std::runtime_error::runtime_error;
};

class Machine {
public:
  explicit Machine(std::vector<std::uint8_t> bytes) : buf_(std::move(bytes)) {}

  std::vector<TensorRecord> run() {
    for (;;) {
      const std::size_t at = pos_;
      const std::uint8_t op = byte();
      switch (op) {
        case 0x80: (void)byte(); break;                                   // PROTO
        case '}': push(make(Obj::kDict)); break;                          // EMPTY_DICT
        case ')': push(make(Obj::kTuple)); break;                         // EMPTY_TUPLE
        case '(': push(make(Obj::kMark)); break;                          // MARK
        case 'N': push(make(Obj::kNone)); break;                          // NONE
        case 0x88: push(boolean(true)); break;                            // NEWTRUE
        case 0x89: push(boolean(false)); break;                           // NEWFALSE
        case 'K': push(integer(byte())); break;                           // BININT1
        case 'M': push(integer(static_cast<std::int64_t>(little(2)))); break;                       // BININT2
        case 'J': push(integer(static_cast<std::int32_t>(static_cast<std::uint32_t>(little(4))))); break;  // BININT
        case 0x8a: push(integer(signed_long(byte()))); break;             // LONG1
        case 0x8b: push(integer(signed_long(static_cast<std::uint32_t>(little(4))))); break;       // LONG4
        case 'X': {                                                       // BINUNICODE
          const std::size_t n = static_cast<std::size_t>(little(4));
          auto s = make(Obj::kStr);
          s->text = chars(n);
          push(s);
          break;
        }
        case 'c': {                                                       // GLOBAL module\nname\n
          auto g = make(Obj::kGlobal);
          const std::string module = line();
          const std::string name = line();
          if (module.empty() || name.empty()) throw PickleError("malformed GLOBAL opcode");
          g->text = module + "." + name;
          push(g);
          break;
        }
        case 'q': memo_[byte()] = top(); break;                           // BINPUT
        case 'r': memo_[static_cast<std::uint32_t>(little(4))] = top(); break;                     // LONG_BINPUT
        case 'h': push(recall(byte())); break;                            // BINGET
        case 'j': push(recall(static_cast<std::uint32_t>(little(4)))); break;                      // LONG_BINGET
        case 0x85: tuple_of(1); break;                                    // TUPLE1
        case 0x86: tuple_of(2); break;                                    // TUPLE2
        case 0x87: tuple_of(3); break;                                    // TUPLE3
        case 't': {                                                       // TUPLE: everything above the mark
          const std::size_t m = mark();
          auto t = make(Obj::kTuple);
          t->items.assign(stack_.begin() + static_cast<std::ptrdiff_t>(m) + 1, stack_.end());
          stack_.resize(m);
          push(t);
          break;
        }
        case 'Q': persistent_id(); break;                                 // BINPERSID
        case 'R': reduce(); break;                                        // REDUCE
        case 's': {                                                       // SETITEM
          if (stack_.size() < 3) throw PickleError("SETITEM stack underflow");
          ObjPtr value = pop();
          ObjPtr key = pop();
          store(top(), key, value);
          break;
        }
        case 'u': {                                                       // SETITEMS
          const std::size_t m = mark();
          if (m == 0) throw PickleError("SETITEMS without dict / OrderedDict and MARK");
          if ((stack_.size() - m - 1) % 2 != 0) throw PickleError("SETITEMS requires key/value pairs");
          ObjPtr target = stack_[m - 1];
          for (std::size_t i = m + 1; i + 1 < stack_.size(); i += 2) store(target, stack_[i], stack_[i + 1]);
          stack_.resize(m);
          break;
        }
        case 'b': {                                                       // BUILD: the state (e.g. _metadata) is dropped
          if (stack_.size() < 2) throw PickleError("BUILD stack underflow");
          (void)pop();
          break;
        }
        case '.': return std::move(found_);                               // STOP
        default: {
          std::ostringstream msg;
          msg << "unsupported pickle opcode 0x" << std::hex << static_cast<int>(op) << std::dec << " at byte " << at;
          throw PickleError(msg.str());
        }
      }
    }
  }

private:
  // ---- input
  std::uint8_t byte() {
    if (pos_ >= buf_.size()) throw PickleError(pos_ == buf_.size() && !buf_.empty() ? "pickle STOP not found" : "truncated pickle byte");
    return buf_[pos_++];
  }
  std::uint64_t little(std::size_t n) {
    if (n > buf_.size() - pos_) throw PickleError("truncated pickle integer");
    std::uint64_t v = 0;
    for (std::size_t i = 0; i < n; ++i) v |= static_cast<std::uint64_t>(buf_[pos_ + i]) << (8 * i);
    pos_ += n;
    return v;
  }
  std::int64_t signed_long(std::uint32_t n) {  // n little-endian two's-complement bytes
    if (n > 8) throw PickleError("pickle long does not fit int64");
    if (n == 0) return 0;
    std::uint64_t v = little(n);
    if (n < 8 && (v >> (8 * n - 1)) & 1u) v |= ~0ull << (8 * n);
    std::int64_t out;
    std::memcpy(&out, &v, sizeof(out));
    return out;
  }
  std::string chars(std::size_t n) {
    if (n > buf_.size() - pos_) throw PickleError("truncated pickle string");
    std::string s(reinterpret_cast<const char*>(buf_.data() + pos_), n);
    pos_ += n;
    return s;
  }
  std::string line() {
    const std::size_t start = pos_;
    while (pos_ < buf_.size() && buf_[pos_] != '\n') ++pos_;
    if (pos_ >= buf_.size()) return {};
    std::string s(reinterpret_cast<const char*>(buf_.data() + start), pos_ - start);
    ++pos_;
    return s;
  }

  // ---- stack
  void push(ObjPtr o) { stack_.push_back(std::move(o)); }
  ObjPtr pop() {
    if (stack_.empty()) throw PickleError("pickle stack underflow");
    ObjPtr o = std::move(stack_.back());
    stack_.pop_back();
    return o;
  }
  const ObjPtr& top() const {
    if (stack_.empty()) throw PickleError("pickle stack underflow");
    return stack_.back();
  }
  std::size_t mark() const {
    for (std::size_t i = stack_.size(); i-- > 0;) {
      if (stack_[i]->tag == Obj::kMark) return i;
    }
    throw PickleError("TUPLE without MARK");
  }
  ObjPtr recall(std::uint32_t index) const {
    auto it = memo_.find(index);
    if (it == memo_.end()) throw PickleError("BINGET missing memo index " + std::to_string(index));
    return it->second;
  }
  static ObjPtr integer(std::int64_t v) {
    auto o = make(Obj::kInt);
    o->num = v;
    return o;
  }
  static ObjPtr boolean(bool v) {
    auto o = make(Obj::kBool);
    o->num = v ? 1 : 0;
    return o;
  }
  void tuple_of(std::size_t n) {
    if (stack_.size() < n) throw PickleError("tuple opcode underflow");
    auto t = make(Obj::kTuple);
    t->items.assign(stack_.end() - static_cast<std::ptrdiff_t>(n), stack_.end());
    stack_.resize(stack_.size() - n);
    push(t);
  }

  // ---- torch-specific pieces
  // ('storage', <storage class>, key, location, element count)
  void persistent_id() {
    ObjPtr pid = pop();
    if (pid->tag != Obj::kTuple) throw PickleError("BINPERSID expects a tuple persistent id");
    const auto& f = pid->items;
    if (f.size() != 5 || f[0]->tag != Obj::kStr || f[0]->text != "storage" || f[1]->tag != Obj::kGlobal ||
        f[2]->tag != Obj::kStr || f[4]->tag != Obj::kInt) {
      throw PickleError("unsupported persistent id shape");
    }
    if (f[1]->text != "torch.BFloat16Storage") {
      throw PickleError("unsupported storage dtype; this reader only supports torch.BFloat16Storage, got: " + f[1]->text);
    }
    if (f[4]->num < 0) throw PickleError("negative storage element count");
    auto st = make(Obj::kStorage);
    st->text = f[2]->text;
    st->count = static_cast<std::uint64_t>(f[4]->num);
    push(st);
  }

  static bool int_tuple(const ObjPtr& t, std::vector<std::int64_t>* out) {
    if (t->tag != Obj::kTuple) return false;
    out->clear();
    for (const ObjPtr& e : t->items) {
      if (e->tag != Obj::kInt) return false;
      out->push_back(e->num);
    }
    return true;
  }

  void reduce() {
    if (stack_.size() < 2) throw PickleError("REDUCE stack underflow");
    ObjPtr args = pop();
    ObjPtr callee = pop();
    if (callee->tag != Obj::kGlobal || args->tag != Obj::kTuple) throw PickleError("unsupported REDUCE operands");
    if (callee->text == "collections.OrderedDict") {
      push(make(Obj::kDict));
      return;
    }
    if (callee->text == "torch._utils._rebuild_tensor_v2") {
      // (storage, storage_offset, size, stride, requires_grad, backward_hooks[, metadata])
      const auto& a = args->items;
      auto t = make(Obj::kTensor);
      if (a.size() < 4 || a[0]->tag != Obj::kStorage || a[1]->tag != Obj::kInt || !int_tuple(a[2], &t->tensor.shape) ||
          !int_tuple(a[3], &t->tensor.stride)) {
        throw PickleError("unsupported _rebuild_tensor_v2 arguments");
      }
      if (t->tensor.shape.size() != t->tensor.stride.size()) throw PickleError("tensor shape / stride rank mismatch");
      if (a[1]->num < 0) throw PickleError("negative tensor storage offset");
      {
        // dimensions are non-negative and their product fits 63 bits: every later size computation is then exact
        std::uint64_t count = 1;
        for (std::int64_t d : t->tensor.shape) {
          if (d < 0) throw PickleError("negative tensor dimension");
          if (d != 0 && count > (static_cast<std::uint64_t>(1) << 62) / static_cast<std::uint64_t>(d)) {
            throw PickleError("tensor element count overflows");
          }
          count *= static_cast<std::uint64_t>(d);
        }
      }
      t->tensor.dtype = TensorDType::kBFloat16;
      t->tensor.storage_key = a[0]->text;
      t->tensor.storage_size = a[0]->count;
      t->tensor.storage_offset = static_cast<std::uint64_t>(a[1]->num);
      push(t);
      return;
    }
    throw PickleError("unsupported REDUCE callable: " + callee->text);
  }

  void store(const ObjPtr& target, const ObjPtr& key, const ObjPtr& value) {
    if (target->tag != Obj::kDict) throw PickleError("SETITEM target must be dict / OrderedDict");
    if (key->tag == Obj::kStr && value->tag == Obj::kTensor) {
      TensorRecord rec = value->tensor;
      rec.name = key->text;
      found_.push_back(std::move(rec));
    }
  }

  std::vector<std::uint8_t> buf_;
  std::size_t pos_ = 0;
  std::vector<ObjPtr> stack_;
  std::map<std::uint32_t, ObjPtr> memo_;
  std::vector<TensorRecord> found_;
};

// "<prefix>/data.pkl" names the archive's top folder (torch uses the file stem, or "archive")
std::string top_folder(const PthArchive& archive) {
  static const std::string kTail = "/data.pkl";
  for (const PthEntry& e : archive.entries()) {
    if (e.name.size() >= kTail.size() && e.name.compare(e.name.size() - kTail.size(), kTail.size(), kTail) == 0) {
      return e.name.substr(0, e.name.size() - kTail.size());
    }
  }
  return {};
}

// Product of the dimensions; 0 for a negative dimension, saturates instead of wrapping (records from the pickle
// machine are already range-checked, hand-made ones may not be).
std::uint64_t element_count(const std::vector<std::int64_t>& shape) {
  std::uint64_t n = 1;
  for (std::int64_t d : shape) {
    if (d < 0) return 0;
    if (d != 0 && n > UINT64_MAX / static_cast<std::uint64_t>(d)) return UINT64_MAX;
    n *= static_cast<std::uint64_t>(d);
  }
  return n;
}

bool row_major(const std::vector<std::int64_t>& shape, const std::vector<std::int64_t>& stride) {
  if (shape.size() != stride.size()) return false;
  std::int64_t expect = 1;
  for (std::size_t i = shape.size(); i-- > 0;) {
    if (shape[i] == 0) return true;
    if (shape[i] != 1 && stride[i] != expect) return false;
    expect *= shape[i];
  }
  return true;
}

// Calls fn(element index in the storage) for every element in logical order; false if an index leaves the storage.
template <typename Fn>
bool walk(const TensorRecord& rec, Fn&& fn) {
  const std::size_t rank = rec.shape.size();
  const std::uint64_t n = element_count(rec.shape);
  if (n == 0) return true;
  std::vector<std::int64_t> idx(rank, 0);
  std::int64_t at = static_cast<std::int64_t>(rec.storage_offset);
  for (std::uint64_t i = 0; i < n; ++i) {
    if (at < 0 || static_cast<std::uint64_t>(at) >= rec.storage_size) return false;
    fn(static_cast<std::uint64_t>(at));
    for (std::size_t d = rank; d-- > 0;) {  // odometer step
      at += rec.stride[d];
      if (++idx[d] < rec.shape[d]) break;
      at -= rec.stride[d] * rec.shape[d];
      idx[d] = 0;
    }
  }
  return true;
}

// The storage bytes of a tensor, whole (the records of a state dict mostly own their storage).
Status storage_bytes(const PthArchive& archive, const TensorRecord& rec, std::vector<std::uint8_t>* out) {
  const std::string folder = top_folder(archive);
  if (folder.empty()) return Status::error("archive prefix not found");
  const PthEntry* entry = archive.find_entry(folder + "/data/" + rec.storage_key);
  if (entry == nullptr) return Status::error("storage entry not found for tensor: " + rec.name);
  auto bytes = archive.read_stored_entry(*entry);
  if (!bytes.ok()) return bytes.status();
  if (rec.storage_size * dtype_size_bytes(rec.dtype) != bytes.value().size()) {
    return Status::error("storage byte size mismatch for tensor: " + rec.name);
  }
  *out = std::move(bytes.value());
  return Status::ok();
}

std::uint16_t bits_at(const std::vector<std::uint8_t>& storage, std::uint64_t element) {
  std::uint16_t v;
  std::memcpy(&v, storage.data() + element * 2, 2);
  return v;
}

}  // namespace

const char* dtype_name(TensorDType) { return "bfloat16"; }
std::uint64_t dtype_size_bytes(TensorDType) { return 2; }

std::string shape_string(const std::vector<std::int64_t>& dims) {
  std::string s = "[";
  for (std::size_t i = 0; i < dims.size(); ++i) {
    if (i) s += ",";
    s += std::to_string(dims[i]);
  }
  return s + "]";
}

// bf16 is the upper half of an fp32: widening is exact.
float bf16_bits_to_float(std::uint16_t bits) {
  const std::uint32_t wide = static_cast<std::uint32_t>(bits) << 16;
  float f;
  std::memcpy(&f, &wide, sizeof(f));
  return f;
}

float f16_bits_to_float(std::uint16_t bits) {
  const std::uint32_t sign = static_cast<std::uint32_t>(bits & 0x8000u) << 16;
  const std::uint32_t e = (bits >> 10) & 0x1fu;
  std::uint32_t m = bits & 0x3ffu;
  std::uint32_t w;
  if (e == 0x1fu) {
    w = sign | 0x7f800000u | (m << 13);                  // inf / nan
  } else if (e != 0) {
    w = sign | ((e + 112u) << 23) | (m << 13);           // normal: rebias 15 -> 127
  } else if (m == 0) {
    w = sign;                                            // zero
  } else {
    std::uint32_t ex = 113;                              // subnormal: normalise
    while (!(m & 0x400u)) {
      m <<= 1;
      --ex;
    }
    w = sign | (ex << 23) | ((m & 0x3ffu) << 13);
  }
  float f;
  std::memcpy(&f, &w, sizeof(f));
  return f;
}

// round to nearest even on the fp32 bit pattern (src/pth_tensor.cpp:672-678); NaNs are not special-cased there
std::uint16_t float_to_bf16_bits(float value) {
  std::uint32_t w;
  std::memcpy(&w, &value, sizeof(w));
  w += 0x7fffu + ((w >> 16) & 1u);
  return static_cast<std::uint16_t>(w >> 16);
}

// The reference's host-side fp32 -> fp16 (src/pth_tensor.cpp:680-720), bit for bit.  It is NOT IEEE
// round-to-nearest-even: the discarded bits round half UP in magnitude (add half an ulp, truncate), and anything
// below 2^-24 becomes zero, also values above 2^-25 that IEEE would round up to the smallest subnormal.  For bf16
// inputs inside fp16's normal range no bits are discarded, so it is exact there.
std::uint16_t float_to_f16_bits(float value) {
  std::uint32_t w;
  std::memcpy(&w, &value, sizeof(w));
  const std::uint32_t sign = (w >> 16) & 0x8000u;
  const std::int32_t e = static_cast<std::int32_t>((w >> 23) & 0xffu) - 127;
  const std::uint32_t frac = w & 0x7fffffu;
  if (e == 128) return static_cast<std::uint16_t>(sign | (frac ? 0x7e00u : 0x7c00u));
  if (e > 15) return static_cast<std::uint16_t>(sign | 0x7c00u);
  if (e >= -14) {
    std::uint32_t he = static_cast<std::uint32_t>(e + 15);
    std::uint32_t hm = frac + 0x1000u;  // half an fp16 ulp
    if (hm & 0x800000u) {               // the mantissa rounded up to 2.0
      hm = 0;
      if (++he >= 31) return static_cast<std::uint16_t>(sign | 0x7c00u);
    }
    return static_cast<std::uint16_t>(sign | (he << 10) | (hm >> 13));
  }
  if (e < -24) return static_cast<std::uint16_t>(sign);
  const std::uint32_t full = frac | 0x800000u;
  const int drop = (-e - 14) + 13;      // bits that fall off a subnormal result
  return static_cast<std::uint16_t>(sign | ((full >> drop) + ((full >> (drop - 1)) & 1u)));
}

Result<std::vector<TensorRecord>> parse_pth_tensor_records(const PthArchive& archive) {
  const std::string folder = top_folder(archive);
  const PthEntry* pkl = folder.empty() ? nullptr : archive.find_entry(folder + "/data.pkl");
  if (pkl == nullptr) return Status::error("data.pkl entry not found");
  auto bytes = archive.read_stored_entry(*pkl);
  if (!bytes.ok()) return bytes.status();
  try {
    return Machine(std::move(bytes.value())).run();
  } catch (const std::exception& ex) {
    return Status::error(ex.what());
  }
}

Result<TensorStats> compute_tensor_stats(const PthArchive& archive, const TensorRecord& record) {
  std::vector<std::uint8_t> storage;
  Status s = storage_bytes(archive, record, &storage);
  if (!s.ok_status()) return s;
  TensorStats stats;
  const bool inside = walk(record, [&](std::uint64_t at) {
    const double v = bf16_bits_to_float(bits_at(storage, at));
    if (std::isnan(v)) return;
    if (!stats.has_value) {
      stats.min = stats.max = v;
      stats.has_value = true;
    } else {
      stats.min = std::min(stats.min, v);
      stats.max = std::max(stats.max, v);
    }
  });
  if (!inside) return Status::error("tensor data range exceeds storage: " + record.name);
  return stats;
}

Result<TensorData> load_bf16_tensor_select(const PthArchive& archive, const TensorRecord& record, bool need_bf16,
                                           bool need_f16, bool need_float) {
  std::vector<std::uint8_t> storage;
  Status s = storage_bytes(archive, record, &storage);
  if (!s.ok_status()) return s;
  TensorData out;
  out.name = record.name;
  out.shape = record.shape;
  // nothing is reserved before the element count has been checked against the storage: a state dict's tensors are
  // views of their storage without repeated elements, so a count beyond the storage is a damaged record
  const std::uint64_t n64 = element_count(record.shape);
  if (n64 > record.storage_size || record.storage_offset > record.storage_size ||
      (row_major(record.shape, record.stride) && n64 > record.storage_size - record.storage_offset)) {
    return Status::error("tensor data range exceeds storage: " + record.name);
  }
  const std::size_t n = static_cast<std::size_t>(n64);
  if (need_bf16) out.values_bf16.reserve(n);
  if (need_f16) out.values_f16.reserve(n);
  if (need_float) out.values.reserve(n);
  const bool inside = walk(record, [&](std::uint64_t at) {
    const std::uint16_t b = bits_at(storage, at);
    if (need_bf16) out.values_bf16.push_back(b);
    if (need_f16 || need_float) {
      const float f = bf16_bits_to_float(b);
      if (need_f16) out.values_f16.push_back(float_to_f16_bits(f));
      if (need_float) out.values.push_back(f);
    }
  });
  if (!inside) return Status::error("tensor data range exceeds storage: " + record.name);
  return out;
}

Result<TensorData> load_bf16_tensor_as_float(const PthArchive& archive, const TensorRecord& record) {
  return load_bf16_tensor_select(archive, record, true, true, true);
}

}  // namespace llm_infer
