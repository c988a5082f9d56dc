// Error state, version and host-memory pinning (reference: src/cuda/pin_memory.cu:9-26).
#include "common.h"

#include <stdlib.h>

#include <atomic>
#include <mutex>
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

// Whether a table lives in host memory decides nothing but the width of the grid that walks it,
// and the answer for a given base pointer does not change while the allocation lives.  The
// runtime query costs a few microseconds and a step asks it for the same handful of tables six
// or more times, so answers are kept in a small table keyed by the pointer.  hades_host_free and
// hades_unpin drop their pointer; an entry that outlives a foreign free can at worst pick the
// other grid width for whatever is allocated there next.
namespace {
constexpr int kPtrCache = 64;
struct PtrCacheEntry {
  const void* ptr = nullptr;
  bool host = false;
};
std::mutex g_ptr_mu;
PtrCacheEntry g_ptr_cache[kPtrCache];
int g_ptr_next = 0;
}  // namespace

void forget_pointer(const void* p) {
  std::lock_guard<std::mutex> lock(g_ptr_mu);
  for (auto& e : g_ptr_cache)
    if (e.ptr == p) e.ptr = nullptr;
}

bool is_host_memory(const void* p) {
  if (p == nullptr) return false;
  {
    std::lock_guard<std::mutex> lock(g_ptr_mu);
    for (const auto& e : g_ptr_cache)
      if (e.ptr == p) return e.host;
  }
  hipPointerAttribute_t attr;
  bool host = false;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError();   // an ordinary pointer the runtime does not know: not ours to read
  } else {
    host = attr.type == hipMemoryTypeHost;
  }
  std::lock_guard<std::mutex> lock(g_ptr_mu);
  g_ptr_cache[g_ptr_next] = PtrCacheEntry{p, host};
  g_ptr_next = (g_ptr_next + 1) % kPtrCache;
  return host;
}

// A kernel that reads or writes rows over the host link needs only enough loads in flight to
// cover the link's bandwidth-delay product (a few hundred KB).  Launched as wide as an HBM kernel
// it parks hundreds of thousands of slow requests in the memory pipeline, and every HBM kernel
// that runs beside it on another stream slows down to the link's pace.
// Measured on 76 K rows of 512 bytes: a gather reaches the link's read rate (55 GB/s) from 32 to
// 128 blocks, 53 GB/s with 16; an update that has reads and writes in flight peaks at 128
// (42.6 GB/s each way); an update that only writes (stores are posted: its waves never wait for
// the link) reaches 40 / 50 / 53 GB/s alone with 16 / 32 / 64 blocks and no more beyond; every
// further store in flight only queues up in front of the HBM traffic of other streams.  Inside a
// step, beside the hot-class sums and update (blocks: cold update / hot sums + hot update, us):
// 24: 951 / 272; 32: 849 / 291; 36: 808 / 305; 40: 787 / 352; 44: 772 / 492; 64: 798 / 662.
// 40 keeps the step within 1 % of its best and the hot class well clear of the cold update.
// HADES_HOST_LINK_BLOCKS / _RW / _WO (read once, at the first use) and
// hades_set_host_link_blocks() override the three widths for tuning.
namespace {
std::atomic<int64_t> g_link_blocks[3] = {{0}, {0}, {0}};   // 0: not set yet
}  // namespace

int64_t host_link_blocks(HostLinkUse use) {
  static const char* const names[] = {"HADES_HOST_LINK_BLOCKS", "HADES_HOST_LINK_BLOCKS_RW",
                                      "HADES_HOST_LINK_BLOCKS_WO"};
  static const int64_t defaults[] = {16, 128, 40};
  int64_t v = g_link_blocks[use].load(std::memory_order_relaxed);
  if (v > 0) return v;
  v = defaults[use];
  const char* e = getenv(names[use]);
  if (e != nullptr) {
    const long ev = atol(e);
    if (ev >= 1) v = ev;
  }
  g_link_blocks[use].store(v, std::memory_order_relaxed);
  return v;
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

int hades_set_host_link_blocks(int use, int64_t blocks) {
  HADES_REQUIRE(use >= 0 && use <= 2, "use must be 0 (copy), 1 (read and write) or 2 (write only)");
  HADES_REQUIRE(blocks >= 0 && blocks <= 65536, "blocks must be in [0, 65536]");
  g_link_blocks[use].store(blocks, std::memory_order_relaxed);   // 0: back to the default
  return HADES_OK;
}

int64_t hades_get_host_link_blocks(int use) {
  if (use < 0 || use > 2) return 0;
  return host_link_blocks(static_cast<HostLinkUse>(use));
}

int hades_unpin(void* host_ptr) {
  HADES_REQUIRE(host_ptr != nullptr, "hades_unpin: null pointer");
  forget_pointer(host_ptr);
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
  forget_pointer(ptr);
  HADES_HIP_TRY(hipHostFree(ptr));
  return HADES_OK;
}

}  // extern "C"
