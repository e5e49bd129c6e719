// Data types.  Numeric values equal hetu/core/dtype.h:9-22 of the reference and
// the HK_* dtype codes of the C-ABI, so they pass through unchanged.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <ostream>
#include <string>

#include "hetu/common/except.h"

namespace hetu {

// Host-side 16-bit floats: storage + conversion only.
// fp32 -> bf16 rounds to nearest even and maps NaN to 0x7FC0
// (hetu/core/bfloat16.h:41-53 of the reference).
struct alignas(2) bfloat16 {
  uint16_t val{0};
  bfloat16() = default;
  bfloat16(float f) {
    if (std::isnan(f)) { val = 0x7FC0; return; }
    uint32_t u;
    std::memcpy(&u, &f, 4);
    val = static_cast<uint16_t>((u + (((u >> 16) & 1u) + 0x7FFFu)) >> 16);
  }
  operator float() const {
    uint32_t u = uint32_t(val) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
  }
};

struct alignas(2) float16 {
  uint16_t val{0};
  float16() = default;
  // round to nearest even, subnormals kept, overflow to infinity
  float16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
    u &= 0x7FFFFFFFu;
    if (u >= 0x7F800000u) {   // inf / nan
      val = sign | (u > 0x7F800000u ? 0x7E00u : 0x7C00u);
    } else if (u >= 0x477FF000u) {   // rounds to >= 65520 -> inf
      val = sign | 0x7C00u;
    } else if (u >= 0x38800000u) {   // normal half
      const uint32_t r = u + 0xC8000FFFu + ((u >> 13) & 1u);   // rebias exponent by -112, round
      val = sign | static_cast<uint16_t>(r >> 13);
    } else if (u >= 0x33000000u) {   // subnormal half
      const uint32_t shift = 126u - (u >> 23);                 // 14..24
      const uint32_t mant = (u & 0x7FFFFFu) | 0x800000u;
      const uint32_t q = mant >> shift, rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
      val = sign | static_cast<uint16_t>(q + ((rem > half || (rem == half && (q & 1u))) ? 1u : 0u));
    } else {
      val = sign;
    }
  }
  operator float() const {
    const uint32_t sign = uint32_t(val & 0x8000u) << 16;
    const uint32_t exp = (val >> 10) & 0x1Fu, mant = val & 0x3FFu;
    uint32_t u;
    if (exp == 0x1Fu) {
      u = sign | 0x7F800000u | (mant << 13);
    } else if (exp != 0) {
      u = sign | ((exp + 112u) << 23) | (mant << 13);
    } else if (mant != 0) {
      int e = -1;
      uint32_t m = mant;
      do { m <<= 1; ++e; } while (!(m & 0x400u));
      u = sign | ((112u - uint32_t(e)) << 23) | ((m & 0x3FFu) << 13);
    } else {
      u = sign;
    }
    float f;
    std::memcpy(&f, &u, 4);
    return f;
  }
};

enum class DataType : int8_t {
  UINT8 = 0, INT8, INT16, INT32, INT64, FLOAT16, FLOAT32, FLOAT64, BFLOAT16, BOOL, NUM_DATA_TYPES, UNDETERMINED
};

constexpr DataType kUInt8 = DataType::UINT8;
constexpr DataType kByte = DataType::UINT8;
constexpr DataType kInt8 = DataType::INT8;
constexpr DataType kInt16 = DataType::INT16;
constexpr DataType kInt32 = DataType::INT32;
constexpr DataType kInt = DataType::INT32;
constexpr DataType kInt64 = DataType::INT64;
constexpr DataType kLong = DataType::INT64;
constexpr DataType kFloat16 = DataType::FLOAT16;
constexpr DataType kHalf = DataType::FLOAT16;
constexpr DataType kFloat32 = DataType::FLOAT32;
constexpr DataType kFloat = DataType::FLOAT32;
constexpr DataType kFloat64 = DataType::FLOAT64;
constexpr DataType kDouble = DataType::FLOAT64;
constexpr DataType kBFloat16 = DataType::BFLOAT16;
constexpr DataType kBool = DataType::BOOL;
constexpr DataType kUndeterminedDataType = DataType::UNDETERMINED;

template <DataType D> struct DataType2SpecMeta;
#define HT_DECLARE_SPEC(D, T)                                                   \
  template <> struct DataType2SpecMeta<D> { using spec_type = T; }
HT_DECLARE_SPEC(DataType::UINT8, uint8_t);
HT_DECLARE_SPEC(DataType::INT8, int8_t);
HT_DECLARE_SPEC(DataType::INT16, int16_t);
HT_DECLARE_SPEC(DataType::INT32, int32_t);
HT_DECLARE_SPEC(DataType::INT64, int64_t);
HT_DECLARE_SPEC(DataType::FLOAT16, float16);
HT_DECLARE_SPEC(DataType::FLOAT32, float);
HT_DECLARE_SPEC(DataType::FLOAT64, double);
HT_DECLARE_SPEC(DataType::BFLOAT16, bfloat16);
HT_DECLARE_SPEC(DataType::BOOL, bool);
#undef HT_DECLARE_SPEC

inline size_t DataType2Size(const DataType& t) {
  switch (t) {
    case kUInt8: case kInt8: case kBool: return 1;
    case kInt16: case kFloat16: case kBFloat16: return 2;
    case kInt32: case kFloat32: return 4;
    case kInt64: case kFloat64: return 8;
    default: HT_VALUE_ERROR << "Unknown data type " << int(t); __builtin_unreachable();
  }
}

inline std::string DataType2Str(const DataType& t) {
  switch (t) {
    case kUInt8: return "uint8";
    case kInt8: return "int8";
    case kInt16: return "int16";
    case kInt32: return "int32";
    case kInt64: return "int64";
    case kFloat16: return "float16";
    case kFloat32: return "float32";
    case kFloat64: return "float64";
    case kBFloat16: return "bfloat16";
    case kBool: return "bool";
    default: return "undetermined";
  }
}
inline std::ostream& operator<<(std::ostream& os, const DataType& t) { return os << DataType2Str(t); }

} // namespace hetu
