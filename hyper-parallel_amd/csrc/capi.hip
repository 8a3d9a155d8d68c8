// Library-level entry points of the C ABI: version, per-thread error text, device check.
#include <string.h>

#include "hpfp8_host.h"

namespace hpfp8 {
char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}
}  // namespace hpfp8

extern "C" {

int hpfp8_version(void) { return 500; }  // 0.5.0

const char* hpfp8_last_error(void) { return hpfp8::error_buffer(); }

int hpfp8_check_device(void) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hpfp8::fail(HPFP8_ERR_DEVICE, "no HIP device: %s", hipGetErrorString(e));
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return hpfp8::fail(HPFP8_ERR_DEVICE, "hipGetDeviceProperties: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return hpfp8::fail(HPFP8_ERR_DEVICE, "device %d is %s; this library is built for gfx950 only", dev,
                       prop.gcnArchName);
  // set-up work for this device: the address of the library's own device memory (used by
  // hpfp8_quantize_per_tensor_noalloc_bf16), so that the first such call needs no set-up of its own
  return hpfp8::prepare_scratch();
}

}  // extern "C"
