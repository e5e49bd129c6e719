#include "hetu/impl/stream/HIPStream.h"
#include "hetu/impl/stream/CPUStream.h"

#include <mutex>

namespace hetu {
namespace impl {

namespace {
struct StreamTable {
  std::mutex mtx;
  hkStream_t streams[HT_MAX_DEVICE_INDEX][HT_NUM_STREAMS_PER_DEVICE] = {};
  bool created[HT_MAX_DEVICE_INDEX][HT_NUM_STREAMS_PER_DEVICE] = {};
};
StreamTable& table() {
  static StreamTable* t = new StreamTable();
  return *t;
}
} // namespace

HIPStream::HIPStream(const Stream& stream)
: _device_id(stream.device_index()), _stream_id(stream.stream_index()), _handle(nullptr) {
  HT_ASSERT(stream.device().is_cuda()) << "Initializing HIP stream for non-accelerator device: " << stream.device();
  if (_stream_id == kBlockingStream) return;   // the null stream
  auto& t = table();
  std::lock_guard<std::mutex> lock(t.mtx);
  if (!t.created[_device_id][_stream_id]) {
    hip::DeviceGuard guard(_device_id);
    HK_CALL(hk_stream_create(&t.streams[_device_id][_stream_id]));
    t.created[_device_id][_stream_id] = true;
  }
  _handle = t.streams[_device_id][_stream_id];
}

void SyncStream(const Stream& stream) {
  HIPStream hs(stream);
  hip::DeviceGuard guard(hs.device_id());
  HK_CALL(hk_stream_sync(hs.handle()));
}

void SyncAllStreams(const Device& device) {
  hip::DeviceGuard guard(device.index());
  HK_CALL(hk_device_sync());
}

HIPEvent::HIPEvent(Device device, bool enable_timing) : Event(device, enable_timing) {
  HT_ASSERT(device.is_cuda()) << "HIPEvent needs an accelerator device, got " << device;
  hip::DeviceGuard guard(device.index());
  HK_CALL(hk_event_create(&_event, enable_timing ? 1 : 0));
}

HIPEvent::~HIPEvent() {
  if (_event) (void)hk_event_destroy(_event);
}

void HIPEvent::Record(const Stream& stream) {
  HIPStream hs(stream);
  hip::DeviceGuard guard(hs.device_id());
  HK_CALL(hk_event_record(_event, hs.handle()));
  _recorded = true;
}

void HIPEvent::Sync() {
  HT_ASSERT(_recorded) << "Event has not been recorded";
  HK_CALL(hk_event_sync(_event));
}

void HIPEvent::Block(const Stream& stream) {
  HT_ASSERT(_recorded) << "Event has not been recorded";
  HIPStream hs(stream);
  hip::DeviceGuard guard(hs.device_id());
  HK_CALL(hk_stream_wait_event(hs.handle(), _event));
}

bool HIPEvent::Query() {
  if (!_recorded) return true;
  int done = 0;
  HK_CALL(hk_event_query(_event, &done));
  return done != 0;
}

int64_t HIPEvent::TimeSince(const Event& event) const {
  const auto* other = dynamic_cast<const HIPEvent*>(&event);
  HT_VALUE_ERROR_IF(other == nullptr) << "TimeSince needs another HIP event";
  HT_VALUE_ERROR_IF(!enable_timing() || !other->enable_timing()) << "Cannot time events created without timing";
  HT_ASSERT(_recorded && other->_recorded) << "Both events must be recorded";
  int64_t ns = 0;
  HK_CALL(hk_event_elapsed_ns(other->_event, _event, &ns));
  return ns;
}

} // namespace impl

void Stream::Sync() const {
  if (_device.is_cuda()) hetu::impl::SyncStream(*this);
  else if (_device.is_cpu()) hetu::impl::CPUStream(*this).Sync();
}

void SynchronizeAllStreams(const Device& device) {
  if (device.is_cuda()) {
    hetu::impl::SyncAllStreams(device);
  } else if (device.is_cpu()) {
    hetu::impl::SynchronizeAllCPUStreams();
  } else if (device.is_undetermined()) {
    hetu::impl::SynchronizeAllCPUStreams();
    int n = 0;
    if (hk_device_count(&n) != HK_OK) return;
    for (int i = 0; i < n && i < HT_MAX_DEVICE_INDEX; ++i) hetu::impl::SyncAllStreams(Device(kCUDA, DeviceIndex(i)));
  }
}

} // namespace hetu
