// hetu/core/reduction_type.h:7-15 of the reference: kSUM = 0, kMEAN = 1 are the
// two this build computes (they equal HK_REDUCE_SUM / HK_REDUCE_MEAN).
#pragma once

#include <cstdint>
#include <ostream>
#include <string>

namespace hetu {

enum class ReductionType : int8_t { SUM = 0, MEAN, MAX, MIN, PROD, NONE, NUM_REDUCTION_TYPES };
constexpr ReductionType kSUM = ReductionType::SUM;
constexpr ReductionType kMEAN = ReductionType::MEAN;
constexpr ReductionType kMAX = ReductionType::MAX;
constexpr ReductionType kMIN = ReductionType::MIN;
constexpr ReductionType kPROD = ReductionType::PROD;
constexpr ReductionType kNONE = ReductionType::NONE;

inline std::string ReductionType2Str(ReductionType r) {
  static const char* const n[] = {"sum", "mean", "max", "min", "prod", "none"};
  int i = static_cast<int>(r);
  return (i >= 0 && i < 6) ? n[i] : "unknown";
}
inline std::ostream& operator<<(std::ostream& os, ReductionType r) { return os << ReductionType2Str(r); }

} // namespace hetu
