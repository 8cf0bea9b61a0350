// Reader of the safetensors container: an 8-byte little-endian header length, a JSON header
// {name: {dtype, shape, data_offsets}}, then the raw little-endian data. The file is mapped into memory and only
// the header is read when it is opened; a tensor's bytes are touched when the caller copies them. The reference
// maps its checkpoints the same way through candle's VarBuilder
// (core/src/model_executor/models/model_factory.rs:133-139).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace lmsf {

struct TensorRecord {
  std::string name;
  std::string dtype;             // as the file says it: F32, BF16, F16, I32, ...
  std::vector<int64_t> shape;
  int64_t begin = 0, end = 0;    // byte offsets inside the data section
};

// Bytes per element of a safetensors dtype, 0 for one this reader does not know.
int safetensors_dtype_size(const std::string& dtype);

// The records of a header (the JSON text alone), in the order of their offsets; every one checked against
// ``data_size`` bytes of data: known dtype, as many bytes as the shape says, inside the data, none overlapping
// another. ``where`` starts the messages (the file's path). Throws lmsf::Error (kValueError).
std::vector<TensorRecord> parse_safetensors_header(const std::string& header, int64_t data_size,
                                                   const std::string& where);

class SafetensorsFile {
 public:
  explicit SafetensorsFile(const std::string& path);   // opens, maps and checks; throws lmsf::Error
  ~SafetensorsFile();
  SafetensorsFile(const SafetensorsFile&) = delete;
  SafetensorsFile& operator=(const SafetensorsFile&) = delete;

  const std::vector<TensorRecord>& tensors() const { return tensors_; }
  const unsigned char* data() const { return map_ + data_start_; }   // the data section (valid until destruction)
  int64_t data_size() const { return size_ - data_start_; }

 private:
  std::vector<TensorRecord> tensors_;
  unsigned char* map_ = nullptr;
  int64_t size_ = 0, data_start_ = 0;
};

}  // namespace lmsf
