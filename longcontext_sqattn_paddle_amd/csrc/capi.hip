// Library-wide pieces of the C ABI: version, thread-local error string, argument checks.
#include <stdarg.h>

#include "common.hpp"

namespace sq {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int check_tensor(const DLTensor* t, const char* name, int ndim, int device_id) {
  SQ_REQUIRE(t != nullptr, SQ_EINVAL, "%s is null", name);
  SQ_REQUIRE(t->data != nullptr || numel_of(t) == 0, SQ_EINVAL, "%s has a null data pointer", name);
  SQ_REQUIRE(on_gpu(t), SQ_EDEVICE, "%s is not on a ROCm device (DLPack device type %d)", name, (int)t->device.device_type);
  SQ_REQUIRE(t->device.device_id == device_id, SQ_EDEVICE, "%s is on device %d, expected %d", name,
             (int)t->device.device_id, device_id);
  SQ_REQUIRE(t->ndim == ndim, SQ_ESHAPE, "%s must have %d dimensions, got %d", name, ndim, (int)t->ndim);
  SQ_REQUIRE(t->shape != nullptr, SQ_EINVAL, "%s has a null shape", name);
  SQ_REQUIRE(stride_of(t, ndim - 1) == 1 || t->shape[ndim - 1] == 1, SQ_ESHAPE, "Last dim of %s must be contiguous.", name);
  SQ_REQUIRE(((uintptr_t)data_of(t) & 15) == 0, SQ_ESHAPE, "%s is not 16-byte aligned", name);
  return SQ_OK;
}

}  // namespace sq

extern "C" int sq_abi_version(void) { return SQ_ABI_VERSION; }

extern "C" const char* sq_last_error(void) { return sq::g_err; }
