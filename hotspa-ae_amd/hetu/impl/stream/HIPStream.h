// HIP streams and events behind hetu::Stream / hetu::Event (what
// hetu/impl/stream/CUDAStream.{h,cc} is to CUDA in the reference): 16 streams
// per device created lazily, index 0 = the default (blocking) stream, the rest
// non-blocking at default priority.
#pragma once

#include <memory>

#include "hetu/core/stream.h"
#include "hetu/impl/utils/hip_utils.h"

namespace hetu {
namespace impl {

class HIPStream {
 public:
  explicit HIPStream(const Stream& stream);
  hkStream_t handle() const { return _handle; }
  operator hkStream_t() const { return _handle; }
  DeviceIndex device_id() const { return _device_id; }
  StreamIndex stream_id() const { return _stream_id; }

 private:
  DeviceIndex _device_id;
  StreamIndex _stream_id;
  hkStream_t _handle;
};

class HIPEvent final : public Event {
 public:
  explicit HIPEvent(Device device, bool enable_timing = true);
  ~HIPEvent() override;
  bool IsRecorded() override { return _recorded; }
  void Record(const Stream& stream) override;
  void Sync() override;
  void Block(const Stream& stream) override;
  bool Query();
  int64_t TimeSince(const Event& event) const override;   // ns from `event` to this one

 private:
  hkEvent_t _event{nullptr};
  bool _recorded{false};
};

// hipStreamSynchronize on one stream / on every stream created for the device
void SyncStream(const Stream& stream);
void SyncAllStreams(const Device& device);

} // namespace impl
} // namespace hetu
