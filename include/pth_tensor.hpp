// Tensor directory and tensor data of a PyTorch checkpoint: the reference's `parse_pth_tensor_records` /
// `load_bf16_tensor_select` and its scalar conversions (include/pth_tensor.hpp:12-59, src/pth_tensor.cpp), same
// names and signatures.
//
// `data.pkl` is interpreted by a pickle machine that knows exactly the opcodes torch.save emits for a state dict
// of tensors (protocol 2: dict / OrderedDict of name -> torch._utils._rebuild_tensor_v2(storage, offset, shape,
// stride, ...)); anything else is an error with the opcode and its position.  As in the reference only
// torch.BFloat16Storage is accepted - RWKV-7 checkpoints are bf16 throughout.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "pth_archive.hpp"
#include "status.hpp"

namespace llm_infer {

enum class TensorDType {
  kBFloat16,
};

struct TensorRecord {
  std::string name;
  TensorDType dtype = TensorDType::kBFloat16;
  std::string storage_key;           // member "<prefix>/data/<storage_key>"
  std::uint64_t storage_size = 0;    // elements in the storage
  std::uint64_t storage_offset = 0;  // first element of the tensor inside it
  std::vector<std::int64_t> shape;
  std::vector<std::int64_t> stride;  // in elements
};

struct TensorStats {
  double min = 0.0;
  double max = 0.0;
  bool has_value = false;
};

struct TensorData {
  std::string name;
  std::vector<std::int64_t> shape;
  std::vector<std::uint16_t> values_bf16;
  std::vector<std::uint16_t> values_bf16_t;
  std::vector<std::uint16_t> values_f16;
  std::vector<std::uint16_t> values_f16_t;
  std::vector<float> values;
  std::vector<float> values_t;
};

const char* dtype_name(TensorDType dtype);
std::uint64_t dtype_size_bytes(TensorDType dtype);
std::string shape_string(const std::vector<std::int64_t>& dims);
float bf16_bits_to_float(std::uint16_t bits);
float f16_bits_to_float(std::uint16_t bits);
std::uint16_t float_to_bf16_bits(float value);
std::uint16_t float_to_f16_bits(float value);

Result<std::vector<TensorRecord>> parse_pth_tensor_records(const PthArchive& archive);
Result<TensorStats> compute_tensor_stats(const PthArchive& archive, const TensorRecord& record);
// Elements in logical (row-major) order whatever the strides; only the requested vectors are filled.
Result<TensorData> load_bf16_tensor_select(const PthArchive& archive, const TensorRecord& record, bool need_bf16,
                                           bool need_f16, bool need_float);
Result<TensorData> load_bf16_tensor_as_float(const PthArchive& archive, const TensorRecord& record);

}  // namespace llm_infer
