#include "safetensors.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstring>

#include "cache_manager.h"   // Error, fail
#include "json.h"

namespace lmsf {

int safetensors_dtype_size(const std::string& dtype) {
  static const struct {
    const char* name;
    int size;
  } kTypes[] = {{"F32", 4}, {"BF16", 2}, {"F16", 2}, {"F64", 8}, {"I64", 8},
                {"I32", 4}, {"I16", 2},  {"I8", 1},  {"U8", 1},  {"BOOL", 1}};
  for (const auto& t : kTypes)
    if (dtype == t.name) return t.size;
  return 0;
}

namespace {

// a non-negative whole number written without sign, fraction or exponent, below 2^62
bool whole_number(const Json& v, int64_t* out) {
  if (v.kind != Json::kNumber || v.text.empty() || v.text.size() > 18) return false;
  int64_t n = 0;
  for (char ch : v.text) {
    if (ch < '0' || ch > '9') return false;
    n = n * 10 + (ch - '0');
  }
  *out = n;
  return true;
}

std::string shape_text(const std::vector<int64_t>& shape) {
  std::string s = "[";
  for (size_t i = 0; i < shape.size(); ++i) s += (i ? ", " : "") + std::to_string(shape[i]);
  return s + "]";
}

}  // namespace

std::vector<TensorRecord> parse_safetensors_header(const std::string& header, int64_t data_size,
                                                   const std::string& where) {
  Json root;
  try {
    root = parse_json(header);
  } catch (const Error& e) {
    fail(kValueError, "%s: header is not valid JSON: %s", where.c_str(), e.message.c_str());
  }
  if (root.kind != Json::kObject) fail(kValueError, "%s: header is not a JSON object", where.c_str());
  std::vector<TensorRecord> out;
  for (const auto& member : root.members) {
    const std::string& name = member.first;
    if (name == "__metadata__") continue;
    const Json& info = member.second;
    const Json* dtype = info.kind == Json::kObject ? info.find("dtype") : nullptr;
    const Json* shape = info.kind == Json::kObject ? info.find("shape") : nullptr;
    const Json* offsets = info.kind == Json::kObject ? info.find("data_offsets") : nullptr;
    TensorRecord r;
    r.name = name;
    bool ok = dtype && dtype->kind == Json::kString && shape && shape->kind == Json::kArray && offsets &&
              offsets->kind == Json::kArray && offsets->items.size() == 2 &&
              whole_number(offsets->items[0], &r.begin) && whole_number(offsets->items[1], &r.end);
    if (ok)
      for (const Json& s : shape->items) {
        int64_t n = 0;
        ok = ok && whole_number(s, &n);
        r.shape.push_back(n);
      }
    if (!ok) fail(kValueError, "%s: malformed header entry for '%s'", where.c_str(), name.c_str());
    r.dtype = dtype->text;
    const int esize = safetensors_dtype_size(r.dtype);
    if (esize == 0)
      fail(kValueError, "%s: tensor '%s' has unsupported dtype %s", where.c_str(), name.c_str(), r.dtype.c_str());
    // elements times element size, refusing what does not fit 62 bits on the way
    int64_t bytes = esize;
    bool fits = true;
    for (int64_t n : r.shape) {
      if (n != 0 && bytes > (INT64_C(1) << 62) / n) fits = false;
      bytes = fits ? bytes * n : 0;
    }
    if (!fits || r.end < r.begin || r.end - r.begin != bytes)
      fail(kValueError, "%s: tensor '%s': %lld bytes for shape %s of %s", where.c_str(), name.c_str(),
           (long long)(r.end - r.begin), shape_text(r.shape).c_str(), r.dtype.c_str());
    if (r.end > data_size)
      fail(kValueError, "%s: tensor '%s' lies outside the file (truncated?)", where.c_str(), name.c_str());
    out.push_back(std::move(r));
  }
  std::stable_sort(out.begin(), out.end(), [](const TensorRecord& a, const TensorRecord& b) { return a.begin < b.begin; });
  for (size_t i = 1; i < out.size(); ++i)
    if (out[i].begin < out[i - 1].end && out[i].end > out[i].begin && out[i - 1].end > out[i - 1].begin)
      fail(kValueError, "%s: tensors '%s' and '%s' overlap", where.c_str(), out[i - 1].name.c_str(),
           out[i].name.c_str());
  std::vector<const std::string*> names;
  for (const TensorRecord& r : out) names.push_back(&r.name);
  std::sort(names.begin(), names.end(), [](const std::string* a, const std::string* b) { return *a < *b; });
  for (size_t i = 1; i < names.size(); ++i)
    if (*names[i] == *names[i - 1])
      fail(kValueError, "%s: tensor '%s' is listed twice", where.c_str(), names[i]->c_str());
  return out;
}

SafetensorsFile::SafetensorsFile(const std::string& path) {
  const int fd = ::open(path.c_str(), O_RDONLY | O_CLOEXEC);
  if (fd < 0) fail(kValueError, "%s: cannot be opened: %s", path.c_str(), std::strerror(errno));
  struct stat st;
  if (::fstat(fd, &st) != 0) {
    const int e = errno;
    ::close(fd);
    fail(kValueError, "%s: cannot be examined: %s", path.c_str(), std::strerror(e));
  }
  size_ = (int64_t)st.st_size;
  if (size_ < 8) {
    ::close(fd);
    fail(kValueError, "%s: too short to be a safetensors file (%lld bytes)", path.c_str(), (long long)size_);
  }
  void* m = ::mmap(nullptr, (size_t)size_, PROT_READ, MAP_PRIVATE, fd, 0);
  const int map_errno = errno;
  ::close(fd);   // (the mapping stays)
  if (m == MAP_FAILED) fail(kValueError, "%s: cannot be mapped: %s", path.c_str(), std::strerror(map_errno));
  map_ = static_cast<unsigned char*>(m);
  try {
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | map_[i];
    if (hlen == 0 || hlen > (uint64_t)(size_ - 8))
      fail(kValueError, "%s: header length %llu does not fit the file of %lld bytes", path.c_str(),
           (unsigned long long)hlen, (long long)size_);
    data_start_ = 8 + (int64_t)hlen;
    tensors_ = parse_safetensors_header(std::string(reinterpret_cast<const char*>(map_ + 8), (size_t)hlen),
                                        size_ - data_start_, path);
  } catch (...) {
    ::munmap(map_, (size_t)size_);
    map_ = nullptr;
    throw;
  }
}

SafetensorsFile::~SafetensorsFile() {
  if (map_ != nullptr) ::munmap(map_, (size_t)size_);
}

}  // namespace lmsf
