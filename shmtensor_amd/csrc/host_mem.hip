// Host memory made addressable by kernels.
// Replaces PinMemory / UnpinMemory (src/cache_feature_fetch.cu:6-13 in the
// ShmTensor tree). The reference relies on CUDA unified addressing (host
// pointer == device pointer after cudaHostRegister); here every host pointer
// handed to a kernel is translated explicitly, which also turns "tensor was
// never pinned" into an error instead of a GPU fault.
#include "common.h"

using namespace shmt;

extern "C" {

int shmt_host_register(void *host_ptr, int64_t nbytes) {
  SHMT_REQUIRE(host_ptr != nullptr && nbytes > 0, "shmt_host_register: empty range");
  hipError_t e = hipHostRegister(host_ptr, static_cast<size_t>(nbytes),
                                 hipHostRegisterPortable | hipHostRegisterMapped);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // do not leave the failure for the next HIP call to report
    set_error("shmt_host_register: hipHostRegister(%p, %lld) failed: %s", host_ptr,
              static_cast<long long>(nbytes), hipGetErrorString(e));
    return SHMT_EHIP;
  }
  return SHMT_OK;
}

int shmt_host_unregister(void *host_ptr) {
  SHMT_REQUIRE(host_ptr != nullptr, "shmt_host_unregister: null pointer");
  hipError_t e = hipHostUnregister(host_ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    set_error("shmt_host_unregister: hipHostUnregister(%p) failed: %s", host_ptr,
              hipGetErrorString(e));
    return SHMT_EHIP;
  }
  return SHMT_OK;
}

int shmt_host_devptr(const void *ptr, void **dev_ptr_out) {
  SHMT_REQUIRE(dev_ptr_out != nullptr, "shmt_host_devptr: dev_ptr_out is null");
  *dev_ptr_out = nullptr;
  SHMT_REQUIRE(ptr != nullptr, "shmt_host_devptr: null pointer");
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    set_error("pointer %p is ordinary pageable host memory: pin it first (pin_memory)", ptr);
    return SHMT_ENOTPINNED;
  }
  if (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged) {
    *dev_ptr_out = const_cast<void *>(ptr);
    return SHMT_OK;
  }
  if (attr.type == hipMemoryTypeHost && attr.devicePointer != nullptr) {
    *dev_ptr_out = attr.devicePointer;
    return SHMT_OK;
  }
  void *dev = nullptr;
  e = hipHostGetDevicePointer(&dev, const_cast<void *>(ptr), 0);
  if (e == hipSuccess && dev != nullptr) {
    *dev_ptr_out = dev;
    return SHMT_OK;
  }
  (void)hipGetLastError();
  set_error("pointer %p is ordinary pageable host memory: pin it first (pin_memory)", ptr);
  return SHMT_ENOTPINNED;
}

}  // extern "C"
