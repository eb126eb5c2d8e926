// Element types of table columns.  The integer values are those of the reference's DataType enum
// (include/common/dtypes.h:18-28) so that pickled specs keep their meaning; the Python-visible
// names follow src/common/pybind.cc:54-83 (value 1 is called int8, value 2 uint8).
#pragma once
#include <cstddef>
#include <stdexcept>
#include <string>

namespace gearhost {

enum class DataType : int {
  kBool = 0,
  kInt8 = 1,
  kUint8 = 2,
  kInt16 = 3,
  kInt32 = 4,
  kInt64 = 5,
  kFloat16 = 6,
  kFloat32 = 7,
  kFloat64 = 8,
};

// Bytes per element; float16 is refused like in the reference (include/common/dtypes.h:55-73).
inline size_t sizeof_dtype(DataType t) {
  switch (t) {
    case DataType::kBool:
    case DataType::kInt8:
    case DataType::kUint8: return 1;
    case DataType::kInt16: return 2;
    case DataType::kInt32: return 4;
    case DataType::kInt64: return 8;
    case DataType::kFloat32: return 4;
    case DataType::kFloat64: return 8;
    default: throw std::runtime_error("Unsupported type.");
  }
}

// numpy / torch dtype name for a DataType
inline const char *dtype_name(DataType t) {
  switch (t) {
    case DataType::kBool: return "bool";
    case DataType::kInt8: return "int8";
    case DataType::kUint8: return "uint8";
    case DataType::kInt16: return "int16";
    case DataType::kInt32: return "int32";
    case DataType::kInt64: return "int64";
    case DataType::kFloat16: return "float16";
    case DataType::kFloat32: return "float32";
    case DataType::kFloat64: return "float64";
  }
  return "?";
}

}  // namespace gearhost
