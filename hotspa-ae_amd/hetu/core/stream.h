// Stream / Event handles of the host layer (hetu/core/stream.h:7-127 of the
// reference): a Stream is (Device, index 0..15); index 0 is the blocking
// default stream, 1 the computing stream.
#pragma once

#include <cstdint>
#include <functional>
#include <ostream>

#include "hetu/core/device.h"

namespace hetu {

using StreamIndex = int32_t;
constexpr int32_t HT_NUM_STREAMS_PER_DEVICE = 1 << 4;
constexpr StreamIndex kUndeterminedStream = -1;
constexpr StreamIndex kBlockingStream = 0;
constexpr StreamIndex kComputingStream = 1;
constexpr StreamIndex kSwitchComputingStream = 2;
constexpr StreamIndex kH2DStream = 3;
constexpr StreamIndex kD2HStream = 4;
constexpr StreamIndex kP2PStream = 5;
constexpr StreamIndex kCollectiveStream = 6;
constexpr StreamIndex kSwitchCollectiveStream = 7;
constexpr StreamIndex kOptimizerStream = 8;
constexpr StreamIndex kJoinStream = HT_NUM_STREAMS_PER_DEVICE - 1;

using PackedStreamId = uint16_t;

class Stream {
 public:
  Stream(Device device = Device(), StreamIndex id = kBlockingStream) : _device(device), _id(id) {
    HT_ASSERT(_id >= kBlockingStream && _id < HT_NUM_STREAMS_PER_DEVICE) << "Invalid stream index: " << _id;
  }

  void Sync() const;

  // stream id (8 bits) || device type (4 bits) || device index (4 bits)
  PackedStreamId pack() const noexcept {
    return static_cast<PackedStreamId>(((static_cast<uint16_t>(_id) & 0xFF) << 8) |
                                       ((static_cast<uint16_t>(_device.type()) & 0xF) << 4) |
                                       (static_cast<uint16_t>(_device.index()) & 0xF));
  }
  static Stream unpack(PackedStreamId packed) {
    return Stream(Device(static_cast<DeviceType>((packed & 0xF0) >> 4), static_cast<DeviceIndex>(packed & 0xF)),
                  static_cast<StreamIndex>((packed & 0xFF00) >> 8));
  }

  const Device& device() const noexcept { return _device; }
  DeviceType device_type() const noexcept { return _device.type(); }
  DeviceIndex device_index() const noexcept { return _device.index(); }
  StreamIndex stream_index() const noexcept { return _id; }
  bool is_defined() const noexcept { return !_device.is_undetermined(); }
  bool is_blocking() const noexcept { return is_defined() && _id == kBlockingStream; }
  bool operator==(const Stream& s) const { return _device == s._device && _id == s._id; }
  bool operator!=(const Stream& s) const { return !(*this == s); }

 private:
  Device _device;
  StreamIndex _id;
};

void SynchronizeAllStreams(const Device& device = Device());

inline std::ostream& operator<<(std::ostream& os, const Stream& s) {
  return os << "stream(" << s.device() << ", id=" << s.stream_index() << ")";
}

class Event {
 public:
  Event(Device device, bool enable_timing = true) : _device(device), _enable_timing(enable_timing) {}
  virtual ~Event() = default;
  virtual bool IsRecorded() = 0;
  virtual void Record(const Stream& stream) = 0;
  virtual void Sync() = 0;
  virtual void Block(const Stream& stream) = 0;
  virtual int64_t TimeSince(const Event& event) const = 0;   // nanoseconds
  const Device& device() const { return _device; }
  bool enable_timing() const { return _enable_timing; }

 protected:
  const Device _device;
  const bool _enable_timing;
};

} // namespace hetu

namespace std {
template <>
struct hash<hetu::Stream> {
  size_t operator()(const hetu::Stream& s) const noexcept { return s.pack(); }
};
} // namespace std
