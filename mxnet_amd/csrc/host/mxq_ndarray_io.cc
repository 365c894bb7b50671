// Reader and writer of the reference's NDArray list files (`.params`, `mx.nd.save`):
//   list container   src/ndarray/ndarray.cc:2126-2146   (magic 0x112, arrays, names)
//   one array        src/ndarray/ndarray.cc:1856-2124   (V2 / V3 records, the two legacy
//                                                        layouts LegacyLoad accepts)
//   shape            include/mxnet/tuple.h:734-765      (int32 ndim, int64 extents)
//   context          include/mxnet/base.h:147-162       (int32 dev_type, int32 dev_id)
// Only dense (default storage) arrays: the quantized models this library serves hold
// nothing else.  Arrays are kept in host memory; the caller moves them to the device.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "../../../include/mxq_ops.h"
#include "mxq_shim.h"

namespace {

const uint64_t kListMagic = 0x112;
const uint32_t kV1Magic = 0xF993fac8;  // int64 shape, no storage type
const uint32_t kV2Magic = 0xF993fac9;  // + storage type
const uint32_t kV3Magic = 0xF993faca;  // V2 written under numpy shape semantics

// mshadow::mshadow_sizeof (3rdparty/mshadow/mshadow/base.h:351-364 for the flags)
size_t TypeSize(int flag) {
  switch (flag) {
    case 0: return 4;   // float32
    case 1: return 8;   // float64
    case 2: return 2;   // float16
    case 3: return 1;   // uint8
    case 4: return 4;   // int32
    case 5: return 1;   // int8
    case 6: return 8;   // int64
    case 7: return 1;   // bool
    case 8: return 2;   // int16
    case 9: return 2;   // uint16
    case 10: return 4;  // uint32
    case 11: return 8;  // uint64
    case 12: return 2;  // bfloat16
    default: LOG_FATAL << "Unknown type flag " << flag;
  }
  return 0;
}

struct Array {
  bool none = true;  // an empty NDArray()
  int dtype = 0;
  std::vector<int64_t> shape;
  std::vector<char> data;
};

struct ArrayList {
  std::vector<Array> arrays;
  std::vector<std::string> names;
};

class Reader {
 public:
  explicit Reader(const std::string& path) : f_(std::fopen(path.c_str(), "rb")) {
    CHECK(f_ != nullptr) << "cannot open " << path;
  }
  ~Reader() {
    if (f_) std::fclose(f_);
  }
  void Read(void* p, size_t n) {
    CHECK(std::fread(p, 1, n, f_) == n) << "Invalid NDArray file format";
  }
  template <typename T>
  T Get() {
    T v;
    Read(&v, sizeof(v));
    return v;
  }

 private:
  FILE* f_;
};

std::vector<int64_t> ReadShape(Reader* r, bool* unknown) {
  const int32_t ndim = r->Get<int32_t>();
  *unknown = ndim < 0;
  CHECK(ndim >= -1 && ndim <= 32) << "Invalid NDArray file format (ndim " << ndim << ")";
  std::vector<int64_t> shape(ndim > 0 ? ndim : 0);
  if (ndim > 0) r->Read(shape.data(), sizeof(int64_t) * ndim);
  return shape;
}

// Product of the extents; a crafted file whose product wraps around is refused rather than
// read into a buffer that no longer matches its shape.
size_t Elements(const std::vector<int64_t>& shape) {
  size_t n = 1;
  for (const int64_t d : shape) {
    CHECK(d >= 0) << "Invalid NDArray file format (negative extent)";
    CHECK(!__builtin_mul_overflow(n, static_cast<size_t>(d), &n))
        << "Invalid NDArray file format (element count overflows)";
  }
  return n;
}

void ReadBody(Reader* r, Array* a) {
  (void)r->Get<int32_t>();  // context: device type
  (void)r->Get<int32_t>();  //          device id
  a->dtype = r->Get<int32_t>();
  size_t bytes = 0;
  CHECK(!__builtin_mul_overflow(static_cast<size_t>(TypeSize(a->dtype)), Elements(a->shape),
                                &bytes))
      << "Invalid NDArray file format (byte count overflows)";
  a->data.resize(bytes);
  if (!a->data.empty()) r->Read(a->data.data(), a->data.size());
  a->none = false;
}

Array ReadArray(Reader* r) {
  Array a;
  const uint32_t magic = r->Get<uint32_t>();
  if (magic == kV2Magic || magic == kV3Magic) {
    const int32_t stype = r->Get<int32_t>();
    CHECK_EQ(stype, 0) << "only dense (default storage) arrays are supported";
    bool unknown = false;
    a.shape = ReadShape(r, &unknown);
    // an empty NDArray(): unknown shape under numpy semantics, zero dimensions otherwise
    if (magic == kV3Magic ? unknown : a.shape.empty()) return a;
    CHECK(!unknown) << "Invalid NDArray file format (unknown shape)";
    ReadBody(r, &a);
    return a;
  }
  // legacy records: V1 carries an int64 shape behind its magic; before that the first word
  // was the number of dimensions itself, followed by uint32 extents
  if (magic == kV1Magic) {
    bool unknown = false;
    a.shape = ReadShape(r, &unknown);
  } else {
    CHECK(magic <= 32) << "Invalid NDArray file format (magic " << magic << ")";
    std::vector<uint32_t> dims(magic);
    if (magic) r->Read(dims.data(), sizeof(uint32_t) * magic);
    a.shape.assign(dims.begin(), dims.end());
  }
  if (a.shape.empty()) return a;
  ReadBody(r, &a);
  return a;
}

class Writer {
 public:
  explicit Writer(const std::string& path) : f_(std::fopen(path.c_str(), "wb")) {
    CHECK(f_ != nullptr) << "cannot open " << path << " for writing";
  }
  ~Writer() {
    if (f_) std::fclose(f_);
  }
  void Write(const void* p, size_t n) {
    CHECK(std::fwrite(p, 1, n, f_) == n) << "write failed";
  }
  // Flushes and closes; a full disk shows up here, not as a silently truncated file.
  void Close() {
    FILE* f = f_;
    f_ = nullptr;
    const int flushed = std::fflush(f);
    const int closed = std::fclose(f);
    CHECK(flushed == 0 && closed == 0) << "write failed (flush / close)";
  }
  template <typename T>
  void Put(T v) {
    Write(&v, sizeof(v));
  }

 private:
  FILE* f_;
};

}  // namespace

extern "C" {

#define IO_API_BEGIN() try {
#define IO_API_END()                 \
  }                                  \
  catch (const std::exception& e) {  \
    mxq_ops_set_error(e.what());     \
    return -1;                       \
  }                                  \
  return 0;

void mxq_ops_set_error(const char* text);

int mxq_ndlist_load(const char* path, void** out_handle, int* out_count, int* out_has_names) {
  IO_API_BEGIN();
  CHECK(path && out_handle && out_count && out_has_names) << "null argument";
  Reader r(path);
  std::unique_ptr<ArrayList> list(new ArrayList());
  CHECK(r.Get<uint64_t>() == kListMagic) << "Invalid NDArray file format";
  (void)r.Get<uint64_t>();  // reserved
  const uint64_t count = r.Get<uint64_t>();
  CHECK(count < (1ull << 32)) << "Invalid NDArray file format";
  for (uint64_t i = 0; i < count; ++i) list->arrays.push_back(ReadArray(&r));
  const uint64_t names = r.Get<uint64_t>();
  CHECK(names == 0 || names == count) << "Invalid NDArray file format";
  for (uint64_t i = 0; i < names; ++i) {
    const uint64_t len = r.Get<uint64_t>();
    CHECK(len < (1ull << 20)) << "Invalid NDArray file format";
    std::string s(len, '\0');
    if (len) r.Read(&s[0], len);
    list->names.push_back(std::move(s));
  }
  *out_count = static_cast<int>(count);
  *out_has_names = names != 0;
  *out_handle = list.release();
  IO_API_END();
}

int mxq_ndlist_get(void* handle, int index, const char** out_name, int* out_is_none,
                   int* out_dtype, int* out_ndim, const int64_t** out_shape,
                   const void** out_data, size_t* out_bytes) {
  IO_API_BEGIN();
  ArrayList* list = static_cast<ArrayList*>(handle);
  CHECK(list && index >= 0 && static_cast<size_t>(index) < list->arrays.size()) << "bad index";
  const Array& a = list->arrays[index];
  *out_name = list->names.empty() ? "" : list->names[index].c_str();
  *out_is_none = a.none;
  *out_dtype = a.dtype;
  *out_ndim = static_cast<int>(a.shape.size());
  *out_shape = a.shape.data();
  *out_data = a.data.data();
  *out_bytes = a.data.size();
  IO_API_END();
}

int mxq_ndlist_free(void* handle) {
  delete static_cast<ArrayList*>(handle);
  return 0;
}

int mxq_ndlist_save(const char* path, int count, const char** names, const mxq_blob* arrays,
                    int np_shape) {
  IO_API_BEGIN();
  CHECK(path && count >= 0 && (count == 0 || arrays)) << "bad argument";
  Writer w(path);
  w.Put<uint64_t>(kListMagic);
  w.Put<uint64_t>(0);
  w.Put<uint64_t>(static_cast<uint64_t>(count));
  for (int i = 0; i < count; ++i) {
    const mxq_blob& b = arrays[i];
    CHECK(b.ndim >= 0 && b.ndim <= MXQ_MAX_NDIM) << "bad ndim";
    CHECK(np_shape || b.ndim > 0)
        << "a zero-dimensional array can only be written under numpy shape semantics";
    w.Put<uint32_t>(np_shape ? kV3Magic : kV2Magic);
    w.Put<int32_t>(0);  // default storage
    w.Put<int32_t>(b.ndim);
    size_t n = 1;
    for (int d = 0; d < b.ndim; ++d) {
      CHECK(b.shape[d] >= 0) << "negative extent";
      w.Put<int64_t>(b.shape[d]);
      n *= static_cast<size_t>(b.shape[d]);
    }
    w.Put<int32_t>(1);  // Context::kCPU
    w.Put<int32_t>(0);
    w.Put<int32_t>(b.dtype);
    const size_t bytes = n * TypeSize(b.dtype);
    CHECK(bytes == 0 || b.data != nullptr) << "null data pointer";
    if (bytes) w.Write(b.data, bytes);
  }
  const uint64_t num_names = names ? static_cast<uint64_t>(count) : 0;
  w.Put<uint64_t>(num_names);
  for (uint64_t i = 0; i < num_names; ++i) {
    const uint64_t len = std::strlen(names[i]);
    w.Put<uint64_t>(len);
    w.Write(names[i], len);
  }
  w.Close();
  IO_API_END();
}

}  // extern "C"
