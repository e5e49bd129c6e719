// Device descriptor.  kCUDA is the accelerator slot of DeviceType
// (hetu/core/device.h:34-45 of the reference); in this build it is backed by
// HIP on gfx950 and nothing else.
#pragma once

#include <cstdint>
#include <functional>
#include <ostream>
#include <string>

#include "hetu/common/except.h"

namespace hetu {

enum class DeviceType : int8_t { CPU = 0, CUDA, NUM_DEVICE_TYPES, UNDETERMINED };
constexpr DeviceType kCPU = DeviceType::CPU;
constexpr DeviceType kCUDA = DeviceType::CUDA;
constexpr DeviceType kUndeterminedDevice = DeviceType::UNDETERMINED;
constexpr int16_t NUM_DEVICE_TYPES = static_cast<int16_t>(DeviceType::NUM_DEVICE_TYPES);

inline std::string DeviceType2Str(const DeviceType& t) {
  switch (t) {
    case kCPU: return "cpu";
    case kCUDA: return "cuda";
    default: return "undetermined";
  }
}
inline std::ostream& operator<<(std::ostream& os, const DeviceType& t) { return os << DeviceType2Str(t); }

using DeviceIndex = uint8_t;
constexpr int HT_MAX_DEVICE_INDEX = 16;

class Device {
 public:
  Device(DeviceType type = kUndeterminedDevice, DeviceIndex index = 0U) : _type(type), _index(index) {
    HT_ASSERT(index < HT_MAX_DEVICE_INDEX) << "Device index " << int(index) << " out of range";
    if (_type != kCUDA) _index = 0;
  }
  bool operator==(const Device& o) const { return _type == o._type && _index == o._index; }
  bool operator!=(const Device& o) const { return !(*this == o); }
  bool operator<(const Device& o) const { return _type != o._type ? _type < o._type : _index < o._index; }
  DeviceType type() const noexcept { return _type; }
  DeviceIndex index() const noexcept { return _index; }
  bool is_cpu() const noexcept { return _type == kCPU; }
  bool is_cuda() const noexcept { return _type == kCUDA; }
  bool is_undetermined() const noexcept { return _type == kUndeterminedDevice; }
  bool local() const noexcept { return true; }

 private:
  DeviceType _type;
  DeviceIndex _index;
};

inline std::ostream& operator<<(std::ostream& os, const Device& d) {
  os << DeviceType2Str(d.type());
  if (d.is_cuda()) os << ":" << int(d.index());
  return os;
}

} // namespace hetu

namespace std {
template <>
struct hash<hetu::Device> {
  size_t operator()(const hetu::Device& d) const noexcept {
    return (static_cast<size_t>(d.type()) << 8) | d.index();
  }
};
} // namespace std
