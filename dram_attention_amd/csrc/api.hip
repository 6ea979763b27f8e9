// Library-level entry points: version, error text, pinned-host address lookup.
#include "common.hpp"

namespace da {
char *last_error_buffer() {
  static thread_local char buf[256] = {0};
  return buf;
}
}  // namespace da

extern "C" int da_version(void) { return 200; }

extern "C" const char *da_last_error_string(void) { return da::last_error_buffer(); }

extern "C" int da_host_device_pointer(const void *host_ptr, void **device_ptr) {
  using namespace da;
  DA_REQUIRE(host_ptr && device_ptr, "da_host_device_pointer: null pointer");
  void *dev = nullptr;
  hipError_t e = hipHostGetDevicePointer(&dev, const_cast<void *>(host_ptr), 0);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail((int)e, "da_host_device_pointer: %s", hipGetErrorString(e));
  }
  *device_ptr = dev;
  return DA_OK;
}
