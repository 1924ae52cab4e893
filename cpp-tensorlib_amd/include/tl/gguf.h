// GGUF v3 container reader: the model-file side of the decode path.
//
// Same public surface as the reference's reader (include/gguf.h: namespace
// tl::gguf, `model`, `tensor_info`, `metadata_value`, `val_type`, `ggml_type`,
// `ggml_block`), so code written against it compiles against this header. The
// file is mapped read-only and the tensor directory points straight into the
// mapping; nothing is copied and nothing is dequantised here. What differs is
// what happens next: the loader in qwen_decode.h hands the mapped bytes to the
// GPU in their file format (f16 rows) and the conversion to the decode formats
// (bf16 rows, the int4 group format, [K,N] for the seam) runs on the device.
//
// Linux only (mmap). Little-endian on the wire and on the host.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace tl {
namespace gguf {

// Wire codes of metadata values (gguf.h:38-45 of the reference; the numbers are the format's).
enum class val_type : uint32_t {
  u8 = 0, i8 = 1, u16 = 2, i16 = 3, u32 = 4, i32 = 5, f32 = 6, boolean = 7,
  string = 8, array = 9, u64 = 10, i64 = 11, f64 = 12,
};

// Tensor storage codes as ggml numbers them. bf16 (30) is accepted on top of the
// reference's list (gguf.h:48-51): bf16 checkpoints exist and the device converts them.
enum class ggml_type : uint32_t {
  f32 = 0, f16 = 1, q4_0 = 2, q4_1 = 3, q5_0 = 6, q5_1 = 7, q8_0 = 8, q8_1 = 9,
  q2_k = 10, q3_k = 11, q4_k = 12, q5_k = 13, q6_k = 14, q8_k = 15, bf16 = 30,
};

namespace detail {
struct block_geometry { uint32_t code, elems, bytes; };
// elements per block and bytes per block of every storage code
constexpr block_geometry kGeometry[] = {
    {0, 1, 4},      {1, 1, 2},      {2, 32, 18},    {3, 32, 20},    {6, 32, 22},
    {7, 32, 24},    {8, 32, 34},    {9, 32, 36},    {10, 256, 84},  {11, 256, 110},
    {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {15, 256, 292}, {30, 1, 2},
};
[[noreturn]] inline void fail(const std::string& what) { throw std::runtime_error("gguf: " + what); }
}  // namespace detail

// elems = elements one block packs, bytes = its size; a tensor occupies
// n_elements / elems * bytes. Unknown codes throw (gguf.h:56-76).
inline void ggml_block(ggml_type t, uint64_t& elems, uint64_t& bytes) {
  for (const auto& g : detail::kGeometry)
    if (g.code == static_cast<uint32_t>(t)) {
      elems = g.elems;
      bytes = g.bytes;
      return;
    }
  detail::fail("tensor storage code " + std::to_string(static_cast<uint32_t>(t)) + " is not one this reader knows");
}

// One metadata value. Unsigned scalars and bool land in u, signed in i, floats in
// f, strings in s, array elements in arr (gguf.h:80-118).
struct metadata_value {
  val_type type{};
  uint64_t u = 0;
  int64_t i = 0;
  double f = 0;
  std::string s;
  val_type arr_elem_type{};
  std::vector<metadata_value> arr;

  // Typed reads: a wrong key or type fails loudly instead of yielding a garbage hyperparameter.
  uint32_t as_u32() const { return expect(val_type::u32), static_cast<uint32_t>(u); }
  int32_t as_i32() const { return expect(val_type::i32), static_cast<int32_t>(i); }
  float as_f32() const { return expect(val_type::f32), static_cast<float>(f); }
  uint64_t as_u64() const { return expect(val_type::u64), u; }
  const std::string& as_str() const { return expect(val_type::string), s; }
  std::vector<std::string> as_str_array() const {
    if (type != val_type::array || arr_elem_type != val_type::string)
      detail::fail("asked for a list of strings, the value holds something else");
    std::vector<std::string> out;
    out.reserve(arr.size());
    for (const auto& e : arr) out.push_back(e.s);
    return out;
  }
  // Any integer width as a count (hyperparameters are written as u32, u64 or i32 in the wild).
  uint64_t as_count() const {
    switch (type) {
      case val_type::u8: case val_type::u16: case val_type::u32: case val_type::u64: return u;
      case val_type::i8: case val_type::i16: case val_type::i32: case val_type::i64:
        if (i >= 0) return static_cast<uint64_t>(i);
        break;
      default: break;
    }
    detail::fail("asked for a count, the value is not an integer >= 0");
  }

 private:
  void expect(val_type want) const {
    if (type != want)
      detail::fail("the value has code " + std::to_string(static_cast<uint32_t>(type)) + ", asked for as code " +
                   std::to_string(static_cast<uint32_t>(want)));
  }
};

// One entry of the tensor directory. dims are in file order ("ne"): dims[0] is the
// contiguous axis, so a linear layer [out, in] is stored with dims = {in, out}.
struct tensor_info {
  std::string name;
  ggml_type type{};
  std::vector<uint64_t> dims;
  uint64_t rel_offset = 0;     // from the start of the data section
  const void* data = nullptr;  // into the mapping
  uint64_t nbytes = 0;

  uint64_t n_elements() const {
    uint64_t n = 1;
    for (uint64_t d : dims) n *= d;
    return n;
  }
};

class model {
 public:
  // Maps the file and parses header, metadata and tensor directory. Throws
  // std::runtime_error on I/O errors, a wrong magic, a version other than 3, or a
  // directory that points outside the file.
  explicit model(const std::string& path) {
    const int fd = ::open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) detail::fail("open() failed: " + path);
    struct stat st {};
    if (::fstat(fd, &st) != 0 || st.st_size <= 0) {
      ::close(fd);
      detail::fail("fstat() failed: " + path);
    }
    bytes_ = static_cast<size_t>(st.st_size);
    void* m = ::mmap(nullptr, bytes_, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (m == MAP_FAILED) detail::fail("mmap() failed: " + path);
    base_ = static_cast<const uint8_t*>(m);
    // weights are walked once, front to back, by the uploader
    ::posix_madvise(m, bytes_, POSIX_MADV_SEQUENTIAL);
    try {
      parse();
    } catch (...) {
      drop();
      throw;
    }
  }
  ~model() { drop(); }
  model(const model&) = delete;
  model& operator=(const model&) = delete;
  model(model&& o) noexcept { take(std::move(o)); }
  model& operator=(model&& o) noexcept {
    if (this != &o) {
      drop();
      take(std::move(o));
    }
    return *this;
  }

  uint32_t version() const { return version_; }
  uint64_t tensor_count() const { return tensors_.size(); }
  uint64_t alignment() const { return alignment_; }
  uint64_t data_offset() const { return data_start_; }   // file offset of the data section
  size_t file_bytes() const { return bytes_; }

  bool has(const std::string& key) const { return kv_.find(key) != kv_.end(); }
  const metadata_value& kv(const std::string& key) const {
    const auto it = kv_.find(key);
    if (it == kv_.end()) detail::fail("no metadata key " + key);
    return it->second;
  }
  const std::unordered_map<std::string, metadata_value>& metadata() const { return kv_; }
  const tensor_info* tensor(const std::string& name) const {
    const auto it = by_name_.find(name);
    return it == by_name_.end() ? nullptr : &tensors_[it->second];
  }
  const std::vector<tensor_info>& tensors() const { return tensors_; }

 private:
  // Bounds-checked little-endian cursor over the mapping.
  struct cursor {
    const uint8_t* base;
    size_t size, at = 0;
    const uint8_t* need(size_t n) {
      if (n > size || at > size - n) detail::fail("the file ends inside a field");
      const uint8_t* p = base + at;
      at += n;
      return p;
    }
    template <typename T>
    T get() {
      T v;
      std::memcpy(&v, need(sizeof(T)), sizeof(T));
      return v;
    }
    std::string str() {
      const uint64_t len = get<uint64_t>();
      if (len > size) detail::fail("the file ends inside a field");
      const uint8_t* p = need(static_cast<size_t>(len));
      return std::string(reinterpret_cast<const char*>(p), static_cast<size_t>(len));
    }
  };

  static metadata_value value(cursor& c, val_type t) {
    metadata_value v;
    v.type = t;
    switch (t) {
      case val_type::u8: v.u = c.get<uint8_t>(); break;
      case val_type::i8: v.i = c.get<int8_t>(); break;
      case val_type::u16: v.u = c.get<uint16_t>(); break;
      case val_type::i16: v.i = c.get<int16_t>(); break;
      case val_type::u32: v.u = c.get<uint32_t>(); break;
      case val_type::i32: v.i = c.get<int32_t>(); break;
      case val_type::u64: v.u = c.get<uint64_t>(); break;
      case val_type::i64: v.i = c.get<int64_t>(); break;
      case val_type::f32: v.f = c.get<float>(); break;
      case val_type::f64: v.f = c.get<double>(); break;
      case val_type::boolean: v.u = c.get<uint8_t>() ? 1 : 0; break;
      case val_type::string: v.s = c.str(); break;
      case val_type::array: {
        v.arr_elem_type = static_cast<val_type>(c.get<uint32_t>());
        if (v.arr_elem_type == val_type::array) detail::fail("a list of lists in the metadata");
        const uint64_t count = c.get<uint64_t>();
        // every element takes at least one byte: a count beyond the file is a corrupt header
        if (count > c.size) detail::fail("the file ends inside a field");
        v.arr.reserve(static_cast<size_t>(count));
        for (uint64_t k = 0; k < count; k++) v.arr.push_back(value(c, v.arr_elem_type));
        break;
      }
      default:
        detail::fail("metadata value code " + std::to_string(static_cast<uint32_t>(t)) + " is not one this reader knows");
    }
    return v;
  }

  void parse() {
    cursor c{base_, bytes_};
    if (c.get<uint32_t>() != 0x46554747u) detail::fail("the first four bytes are not 'GGUF'");   // "GGUF"
    version_ = c.get<uint32_t>();
    if (version_ != 3) detail::fail("format version " + std::to_string(version_) + " (version 3 is read)");
    const uint64_t n_tensors = c.get<uint64_t>();
    const uint64_t n_kv = c.get<uint64_t>();
    for (uint64_t k = 0; k < n_kv; k++) {
      std::string key = c.str();
      const val_type t = static_cast<val_type>(c.get<uint32_t>());
      kv_.emplace(std::move(key), value(c, t));   // a repeated key keeps its first value
    }
    const auto al = kv_.find("general.alignment");
    if (al != kv_.end()) alignment_ = al->second.type == val_type::u32 ? al->second.as_u32() : al->second.u;
    if (alignment_ == 0) detail::fail("general.alignment is zero");

    if (n_tensors > bytes_) detail::fail("the file ends inside a field");
    tensors_.reserve(static_cast<size_t>(n_tensors));
    for (uint64_t k = 0; k < n_tensors; k++) {
      tensor_info t;
      t.name = c.str();
      const uint32_t n_dims = c.get<uint32_t>();
      for (uint32_t d = 0; d < n_dims; d++) t.dims.push_back(c.get<uint64_t>());
      t.type = static_cast<ggml_type>(c.get<uint32_t>());
      t.rel_offset = c.get<uint64_t>();
      uint64_t per_block = 1, block_bytes = 1;
      ggml_block(t.type, per_block, block_bytes);
      t.nbytes = t.n_elements() / per_block * block_bytes;
      by_name_.emplace(t.name, tensors_.size());
      tensors_.push_back(std::move(t));
    }
    // the data section starts at the end of the directory, rounded up to the alignment
    data_start_ = (c.at + alignment_ - 1) / alignment_ * alignment_;
    for (auto& t : tensors_) {
      if (t.rel_offset > bytes_ || data_start_ > bytes_ - t.rel_offset)
        detail::fail("the file ends inside a field");
      cursor probe{base_, bytes_, static_cast<size_t>(data_start_ + t.rel_offset)};
      t.data = probe.need(static_cast<size_t>(t.nbytes));
    }
  }

  void drop() noexcept {
    if (base_) ::munmap(const_cast<uint8_t*>(base_), bytes_);
    base_ = nullptr;
    bytes_ = 0;
  }
  void take(model&& o) noexcept {
    base_ = o.base_;
    bytes_ = o.bytes_;
    o.base_ = nullptr;
    o.bytes_ = 0;
    version_ = o.version_;
    alignment_ = o.alignment_;
    data_start_ = o.data_start_;
    kv_ = std::move(o.kv_);
    tensors_ = std::move(o.tensors_);
    by_name_ = std::move(o.by_name_);
  }

  const uint8_t* base_ = nullptr;
  size_t bytes_ = 0;
  uint32_t version_ = 0;
  uint64_t alignment_ = 32;   // the format's default; general.alignment overrides
  uint64_t data_start_ = 0;
  std::unordered_map<std::string, metadata_value> kv_;
  std::vector<tensor_info> tensors_;
  std::unordered_map<std::string, size_t> by_name_;
};

}  // namespace gguf
}  // namespace tl
