// NOT TensorFlow.  A declaration-only stand-in for the handful of TensorFlow types that the
// files under tf/ use, written from TensorFlow's public C++ API, so that those files can be
// parsed and type-checked (g++ -fsyntax-only) in an image without TensorFlow.  It checks that
// the calls into include/atex_norms.h and the uses of the framework API are well-formed; it
// links nothing, runs nothing and is no evidence of parity.
#ifndef ATEXN_TF_MOCK_CORE_H_
#define ATEXN_TF_MOCK_CORE_H_

#include <cstdint>
#include <initializer_list>
#include <sstream>
#include <string>
#include <vector>

namespace Eigen {
struct half { uint16_t x; };
struct bfloat16 { uint16_t value; };
struct ThreadPoolDevice {};
struct GpuDevice {
  void* stream() const;  // gpuStream_t = hipStream_t under TensorFlow-ROCm
};
}  // namespace Eigen

namespace tensorflow {

typedef Eigen::bfloat16 bfloat16;
typedef uint8_t uint8;
typedef int64_t int64;

class StringPiece {
 public:
  StringPiece(const char*);
  StringPiece(const std::string&);
  const char* data() const;
  size_t size() const;
};

class Status {
 public:
  Status();
  bool ok() const;
};
Status OkStatus();

namespace errors {
template <typename... Args> Status InvalidArgument(Args... args);
template <typename... Args> Status Internal(Args... args);
}  // namespace errors

#define TF_RETURN_IF_ERROR(...)              \
  do {                                       \
    ::tensorflow::Status s_ = (__VA_ARGS__); \
    if (!s_.ok()) return s_;                 \
  } while (0)

enum DataType { DT_FLOAT = 1, DT_UINT8 = 4, DT_BFLOAT16 = 14, DT_HALF = 19 };

extern const char* const DEVICE_CPU;
extern const char* const DEVICE_GPU;

class TensorShape {
 public:
  TensorShape();
  TensorShape(std::initializer_list<int64_t> dims);
  int dims() const;
  int64_t dim_size(int d) const;
  std::string DebugString() const;
};

template <typename T>
struct FlatView {
  T* data() const;
};

class Tensor {
 public:
  Tensor();
  DataType dtype() const;
  const TensorShape& shape() const;
  int dims() const;
  int64_t dim_size(int d) const;
  int64_t NumElements() const;
  StringPiece tensor_data() const;
  template <typename T> FlatView<T> flat();
  template <typename T> FlatView<const T> flat() const;
};

}  // namespace tensorflow

#endif  // ATEXN_TF_MOCK_CORE_H_
