// Basic vocabulary of the host layer: element types, type metadata, logging
// and CHECK macros. Follows the roles of dragon/core/types.h,
// dragon/core/typeid.h and dragon/utils/logging.h of the reference; this layer
// compiles with a plain C++ compiler and includes no HIP header (the device is
// reached only through include/dragon_hip.h).
#pragma once

#include <cstdint>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace dragon {

using std::string;
using std::vector;
typedef std::vector<int64_t> vec64_t;

// 16-bit storage types: a bare unsigned short, as dragon/core/types.h:36-42.
struct float16 {
  unsigned short x;
};
struct bfloat16 {
  unsigned short x;
};

// Runtime type tag of a tensor. The numeric values are the dtype tags of the
// C ABI (include/dragon_hip.h) for the four floating types.
enum class DType : int {
  kFloat16 = 0,
  kBFloat16 = 1,
  kFloat32 = 2,
  kFloat64 = 3,
  kInt64 = 4,
  kUInt8 = 5,
  kInt32 = 6,
  kUndefined = -1
};

template <typename T>
struct TypeOf;
template <>
struct TypeOf<float16> {
  static constexpr DType value = DType::kFloat16;
};
template <>
struct TypeOf<bfloat16> {
  static constexpr DType value = DType::kBFloat16;
};
template <>
struct TypeOf<float> {
  static constexpr DType value = DType::kFloat32;
};
template <>
struct TypeOf<double> {
  static constexpr DType value = DType::kFloat64;
};
template <>
struct TypeOf<int64_t> {
  static constexpr DType value = DType::kInt64;
};
template <>
struct TypeOf<uint8_t> {
  static constexpr DType value = DType::kUInt8;
};
template <>
struct TypeOf<int> {
  static constexpr DType value = DType::kInt32;
};

inline size_t SizeOf(DType t) {
  switch (t) {
    case DType::kFloat16:
    case DType::kBFloat16: return 2;
    case DType::kFloat32:
    case DType::kInt32: return 4;
    case DType::kFloat64:
    case DType::kInt64: return 8;
    case DType::kUInt8: return 1;
    default: return 0;
  }
}

inline const char* NameOf(DType t) {
  switch (t) {
    case DType::kFloat16: return "float16";
    case DType::kBFloat16: return "bfloat16";
    case DType::kFloat32: return "float32";
    case DType::kFloat64: return "float64";
    case DType::kInt64: return "int64";
    case DType::kUInt8: return "uint8";
    case DType::kInt32: return "int32";
    default: return "unknown";
  }
}

inline DType DTypeFromName(const string& s) {
  if (s == "float16") return DType::kFloat16;
  if (s == "bfloat16") return DType::kBFloat16;
  if (s == "float32") return DType::kFloat32;
  if (s == "float64") return DType::kFloat64;
  if (s == "int64") return DType::kInt64;
  if (s == "uint8") return DType::kUInt8;
  if (s == "int32") return DType::kInt32;
  return DType::kUndefined;
}

namespace math {
// math::Traits<T>::accumulator_type, dragon/utils/math/types.h:69-152.
template <typename T>
struct Traits {
  typedef float accumulator_type;
};
template <>
struct Traits<double> {
  typedef double accumulator_type;
};
} // namespace math

// ---------------------------------------------------------------------------
// Logging. LOG(FATAL) and failed CHECKs print the message and then call the
// fatal handler. The default handler aborts, which is the reference's
// behaviour (dragon/utils/logging.cc:98-102); an embedding that must survive
// (the C API used by the tests) installs a handler that throws FatalError.
// ---------------------------------------------------------------------------
struct FatalError : public std::runtime_error {
  explicit FatalError(const string& what) : std::runtime_error(what) {}
};

typedef void (*FatalHandler)(const string& message);
FatalHandler SetFatalHandler(FatalHandler handler);  // returns the previous one
void ThrowingFatalHandler(const string& message);    // throws FatalError

enum LogSeverity { DEBUG = 0, INFO = 1, WARNING = 2, ERROR = 3, FATAL = 4 };

class MessageLogger {
 public:
  MessageLogger(const char* file, int line, int severity);
  // Terminates through the fatal handler when the severity is FATAL.
  ~MessageLogger() noexcept(false);
  std::stringstream& stream() { return stream_; }

 private:
  int severity_;
  std::stringstream stream_;
};

void SetLogSeverity(int severity);

#define LOG(severity) ::dragon::MessageLogger(__FILE__, __LINE__, ::dragon::severity).stream()
#define CHECK(cond) \
  if (!(cond)) LOG(FATAL) << "Check failed: " #cond " "
#define CHECK_OP(a, b, op) \
  if (!((a)op(b))) LOG(FATAL) << "Check failed: " #a " " #op " " #b " (" << (a) << " vs. " << (b) << ") "
#define CHECK_EQ(a, b) CHECK_OP(a, b, ==)
#define CHECK_NE(a, b) CHECK_OP(a, b, !=)
#define CHECK_LT(a, b) CHECK_OP(a, b, <)
#define CHECK_LE(a, b) CHECK_OP(a, b, <=)
#define CHECK_GT(a, b) CHECK_OP(a, b, >)
#define CHECK_GE(a, b) CHECK_OP(a, b, >=)

inline string DimsToString(const vec64_t& dims) {
  std::stringstream ss;
  ss << "(";
  for (size_t i = 0; i < dims.size(); ++i) ss << (i ? "," : "") << dims[i];
  if (dims.size() == 1) ss << ",";
  ss << ")";
  return ss.str();
}

} // namespace dragon
