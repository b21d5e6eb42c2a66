// Error channel and device queries of the core kernel library.
#include "common.h"
#include "errors.inc"

extern "C" int me_device_info(int* num_cus, int64_t* lds_bytes, char* arch, int arch_len) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  ME_CHECK(e == hipSuccess, "hipGetDevice: %s", hipGetErrorString(e));
  hipDeviceProp_t p;
  e = hipGetDeviceProperties(&p, dev);
  ME_CHECK(e == hipSuccess, "hipGetDeviceProperties: %s", hipGetErrorString(e));
  *num_cus = p.multiProcessorCount;
  *lds_bytes = (int64_t)p.sharedMemPerBlock;
  snprintf(arch, arch_len, "%s", p.gcnArchName);
  return 0;
}
