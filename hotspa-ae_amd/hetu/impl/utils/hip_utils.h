// Thin host-side helpers over the C-ABI device layer (hk_rowwise.h): error
// translation into exceptions and the per-call device guard
// (role of hetu/impl/utils/cuda_utils.h:26-29, 103-127 in the reference).
#pragma once

#include "hetu/common/except.h"
#include "hk_rowwise.h"

namespace hetu {
namespace hip {

HT_DECLARE_EXCEPTION(hip_error);

// Translates a C-ABI status into the exception the reference layer would throw:
// unsupported dtype / feature -> not_implemented, the rest -> hip_error.
inline void check(int rc, const char* expr, const char* file, int line) {
  if (rc == HK_OK) return;
  std::string msg = std::string(expr) + " failed (" + std::to_string(rc) + "): " + hk_last_error();
  if (rc == HK_ERR_UNSUPPORTED) throw hetu::not_implemented("Not implemented: " + msg, file, line);
  if (rc == HK_ERR_INVALID) throw hetu::value_error("Value error: " + msg, file, line);
  throw hip_error("HIP error: " + msg, file, line);
}

// Sets the current device for the scope and restores the previous one.
class DeviceGuard {
 public:
  explicit DeviceGuard(int device) : _prev(-1), _changed(false) {
    if (hk_get_device(&_prev) == HK_OK && _prev != device) {
      check(hk_set_device(device), "hk_set_device", __FILE__, __LINE__);
      _changed = true;
    }
  }
  ~DeviceGuard() {
    if (_changed) (void)hk_set_device(_prev);
  }
  DeviceGuard(const DeviceGuard&) = delete;

 private:
  int _prev;
  bool _changed;
};

} // namespace hip
} // namespace hetu

#define HK_CALL(expr) ::hetu::hip::check((expr), #expr, __FILE__, __LINE__)
