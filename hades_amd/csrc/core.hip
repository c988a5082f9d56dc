// Error state, version and host-memory pinning (reference: src/cuda/pin_memory.cu:9-26).
#include "common.h"

#include <stdlib.h>

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

bool is_host_memory(const void* p) {
  if (p == nullptr) return false;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError();   // an ordinary pointer the runtime does not know: not ours to read
    return false;
  }
  return attr.type == hipMemoryTypeHost;
}

// A kernel that reads or writes rows over the host link needs only enough loads in flight to
// cover the link's bandwidth-delay product (a few hundred KB).  Launched as wide as an HBM kernel
// it parks hundreds of thousands of slow requests in the memory pipeline, and every HBM kernel
// that runs beside it on another stream slows down to the link's pace.
// Measured on 76 K rows of 512 bytes: a gather reaches the link's read rate (55 GB/s) from 32 to
// 128 blocks, 53 GB/s with 16; an update that has reads and writes in flight peaks at 128
// (42.6 GB/s each way); an update that only writes (stores are posted: its waves never wait for
// the link) saturates it from 32 blocks, and every further store in flight only queues up in front
// of the HBM traffic of other streams (the segmented sum beside a write-only update of 128 blocks
// took 690 us, beside one of 32 blocks 155 us, the update itself as long either way).
// HADES_HOST_LINK_BLOCKS / _RW / _WO override the three widths for tuning.
int64_t host_link_blocks(HostLinkUse use) {
  static const char* const names[] = {"HADES_HOST_LINK_BLOCKS", "HADES_HOST_LINK_BLOCKS_RW",
                                      "HADES_HOST_LINK_BLOCKS_WO"};
  static const int64_t defaults[] = {16, 128, 32};
  const char* e = getenv(names[use]);
  if (e != nullptr) {
    const long v = atol(e);
    if (v >= 1) return v;
  }
  return defaults[use];
}

}  // namespace hades

using namespace hades;

extern "C" {

const char* hades_last_error(void) { return g_last_error.c_str(); }

int hades_version(void) { return HADES_ABI_VERSION; }

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

int hades_host_alloc_flags(void** out_ptr, size_t bytes, unsigned flags) {
  HADES_REQUIRE(out_ptr != nullptr, "hades_host_alloc: null out pointer");
  HADES_REQUIRE((flags & ~unsigned(HADES_HOST_NONCOHERENT)) == 0, "unknown host allocation flags %u", flags);
  *out_ptr = nullptr;
  if (bytes == 0) return HADES_OK;
  unsigned f = hipHostMallocMapped | hipHostMallocPortable;
  if (flags & HADES_HOST_NONCOHERENT) f |= hipHostMallocNonCoherent;
  HADES_HIP_TRY(hipHostMalloc(out_ptr, bytes, f));
  return HADES_OK;
}

int hades_host_alloc(void** out_ptr, size_t bytes) {
  return hades_host_alloc_flags(out_ptr, bytes, 0);
}

int hades_host_free(void* ptr) {
  if (!ptr) return HADES_OK;
  HADES_HIP_TRY(hipHostFree(ptr));
  return HADES_OK;
}

}  // extern "C"
