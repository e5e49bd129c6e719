// The caching pool over HIP device memory, one per device, registered for every
// accelerator index before main() (the pools themselves are built on first use,
// so no device is touched at load time).
#include "hetu/impl/memory/CachingMemoryPool.h"
#include "hetu/impl/stream/HIPStream.h"
#include "hetu/impl/utils/hip_utils.h"

namespace hetu {
namespace impl {

namespace {

class HIPBackend final : public PoolBackend {
 public:
  explicit HIPBackend(int device) : _device(device) {}
  ~HIPBackend() override {
    for (auto e : _spare_events) (void)hk_event_destroy(e);
  }

  void* RawAlloc(size_t bytes) override {
    hip::DeviceGuard guard(_device);
    void* p = nullptr;
    if (hk_malloc(&p, bytes) != HK_OK) return nullptr;
    return p;
  }
  void RawFree(void* ptr) override {
    hip::DeviceGuard guard(_device);
    HK_CALL(hk_free(ptr));
  }
  void* EventRecord(const Stream& stream) override {
    hip::DeviceGuard guard(_device);
    hkEvent_t e = nullptr;
    if (!_spare_events.empty()) {
      e = _spare_events.back();
      _spare_events.pop_back();
    } else {
      HK_CALL(hk_event_create(&e, /*enable_timing=*/0));
    }
    HK_CALL(hk_event_record(e, HIPStream(stream).handle()));
    return e;
  }
  bool EventDone(void* event) override {
    int done = 0;
    HK_CALL(hk_event_query(static_cast<hkEvent_t>(event), &done));
    return done != 0;
  }
  void EventSync(void* event) override { HK_CALL(hk_event_sync(static_cast<hkEvent_t>(event))); }
  void EventRelease(void* event) override { _spare_events.push_back(static_cast<hkEvent_t>(event)); }
  void StreamWaitEvent(const Stream& stream, void* event) override {
    hip::DeviceGuard guard(_device);
    HK_CALL(hk_stream_wait_event(HIPStream(stream).handle(), static_cast<hkEvent_t>(event)));
  }
  void StreamSync(const Stream& stream) override {
    hip::DeviceGuard guard(_device);
    HK_CALL(hk_stream_sync(HIPStream(stream).handle()));
  }
  void DeviceSync() override {
    hip::DeviceGuard guard(_device);
    HK_CALL(hk_device_sync());
  }

 private:
  int _device;
  std::vector<hkEvent_t> _spare_events;   // used under the pool's lock only
};

struct HIPCachingMemoryPoolRegister {
  HIPCachingMemoryPoolRegister() {
    const size_t max_split = ParsePoolKnobMB("HETU_MAX_SPLIT_SIZE_MB", 200);
    const size_t max_fragment = ParsePoolKnobMB("HETU_MAX_INTERNAL_FRAGMENT_SIZE_MB", 20);
    for (int i = 0; i < HT_MAX_DEVICE_INDEX; ++i) {
      RegisterMemoryPoolCtor(Device(kCUDA, DeviceIndex(i)), [i, max_split, max_fragment]() {
        return std::static_pointer_cast<MemoryPool>(std::make_shared<CachingMemoryPool>(
          Device(kCUDA, DeviceIndex(i)), "HIPCachingMemPool(" + std::to_string(i) + ")",
          std::unique_ptr<PoolBackend>(new HIPBackend(i)), max_split, max_fragment));
      });
    }
  }
};
static HIPCachingMemoryPoolRegister hip_caching_memory_pool_register;

} // namespace
} // namespace impl
} // namespace hetu
