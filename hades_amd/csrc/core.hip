// Error state, version and host-memory pinning (reference: src/cuda/pin_memory.cu:9-26).
#include "common.h"

#include <string>

namespace hades {

static thread_local std::string g_last_error;
thread_local ProfileSlot g_profile;

int set_error(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

}  // namespace hades

using namespace hades;

extern "C" {

const char* hades_last_error(void) { return g_last_error.c_str(); }

int hades_version(void) { return 100; }

int hades_profile_kernel(int kernel_id, void* start_event, void* stop_event) {
  HADES_REQUIRE(kernel_id >= 0 && kernel_id <= HADES_KERNEL_LAST, "unknown kernel id %d", kernel_id);
  HADES_REQUIRE(kernel_id == 0 || (start_event && stop_event), "null event");
  g_profile.kernel_id = kernel_id;
  g_profile.start = static_cast<hipEvent_t>(start_event);
  g_profile.stop = static_cast<hipEvent_t>(stop_event);
  return HADES_OK;
}

int hades_pin(void* host_ptr, size_t bytes) {
  HADES_REQUIRE(host_ptr != nullptr, "hades_pin: null pointer");
  if (bytes == 0) return HADES_OK;
  HADES_HIP_TRY(hipHostRegister(host_ptr, bytes, hipHostRegisterMapped | hipHostRegisterPortable));
  return HADES_OK;
}

int hades_unpin(void* host_ptr) {
  HADES_REQUIRE(host_ptr != nullptr, "hades_unpin: null pointer");
  HADES_HIP_TRY(hipHostUnregister(host_ptr));
  return HADES_OK;
}

int hades_host_alloc(void** out_ptr, size_t bytes) {
  HADES_REQUIRE(out_ptr != nullptr, "hades_host_alloc: null out pointer");
  *out_ptr = nullptr;
  if (bytes == 0) return HADES_OK;
  HADES_HIP_TRY(hipHostMalloc(out_ptr, bytes, hipHostMallocMapped | hipHostMallocPortable));
  return HADES_OK;
}

int hades_host_free(void* ptr) {
  if (!ptr) return HADES_OK;
  HADES_HIP_TRY(hipHostFree(ptr));
  return HADES_OK;
}

}  // extern "C"
