// POSIX shared-memory segments for host tables and cache buffers that several processes map
// (reference: create_shared_mem / open_shared_mem / release_shared_mem, src/shm/shared_memory.h:
// 14-58).  Host code only.  With pin != 0 the mapping is also registered with the HIP runtime so
// that kernels can address it; where the platform refuses to register existing memory the call
// undoes what it did and returns the runtime's error instead of ending the process (the
// reference's CUDA_CALL exits, src/utils.h:12-24).
#include "common.h"

#include <cerrno>
#include <cstring>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace hades {
namespace {

int map_segment(const char* name, int64_t size, int pin, bool create, void** out_ptr,
                int64_t* out_fd) {
  HADES_REQUIRE(name && name[0], "shared memory: empty name");
  HADES_REQUIRE(size > 0, "shared memory: size must be > 0 (got %lld)", (long long)size);
  HADES_REQUIRE(out_ptr && out_fd, "shared memory: null output pointer");
  *out_ptr = nullptr;
  *out_fd = -1;
  const int fd = shm_open(name, create ? (O_RDWR | O_CREAT) : O_RDWR, S_IRUSR | S_IWUSR);
  if (fd == -1) return set_error(HADES_ERR_ARG, "fail to open %s: %s", name, strerror(errno));
  if (create && ftruncate(fd, static_cast<off_t>(size)) == -1) {
    const int e = errno;
    close(fd);
    shm_unlink(name);
    return set_error(HADES_ERR_ARG, "failed to size %s to %lld bytes: %s", name, (long long)size,
                     strerror(e));
  }
  if (!create) {  // mapping past the end of a segment faults on first touch: refuse it here
    struct stat sb;
    if (fstat(fd, &sb) == -1 || sb.st_size < static_cast<off_t>(size)) {
      close(fd);
      return set_error(HADES_ERR_ARG, "%s holds %lld bytes, fewer than the %lld asked for", name,
                       (long long)sb.st_size, (long long)size);
    }
  }
  void* ptr = mmap(nullptr, static_cast<size_t>(size), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  if (ptr == MAP_FAILED) {
    const int e = errno;
    close(fd);
    if (create) shm_unlink(name);
    return set_error(HADES_ERR_ARG, "failed to map %s: %s", name, strerror(e));
  }
  if (pin) {
    const hipError_t err =
        hipHostRegister(ptr, static_cast<size_t>(size), hipHostRegisterMapped | hipHostRegisterPortable);
    if (err != hipSuccess) {
      (void)hipGetLastError();
      munmap(ptr, static_cast<size_t>(size));
      close(fd);
      if (create) shm_unlink(name);
      return set_error(HADES_ERR_HIP, "cannot register %s with the HIP runtime: %s", name,
                       hipGetErrorString(err));
    }
  }
  *out_ptr = ptr;
  *out_fd = fd;
  return HADES_OK;
}

}  // namespace
}  // namespace hades

using namespace hades;

extern "C" {

int hades_shm_create(const char* name, int64_t size, int pin, void** out_ptr, int64_t* out_fd) {
  return map_segment(name, size, pin, true, out_ptr, out_fd);
}

int hades_shm_open(const char* name, int64_t size, int pin, void** out_ptr, int64_t* out_fd) {
  return map_segment(name, size, pin, false, out_ptr, out_fd);
}

int hades_shm_release(const char* name, int64_t size, void* ptr, int64_t fd, int pin) {
  HADES_REQUIRE(name && ptr && size > 0, "shared memory: bad release arguments");
  int rc = HADES_OK;
  if (pin) {
    const hipError_t err = hipHostUnregister(ptr);
    if (err != hipSuccess) {
      (void)hipGetLastError();
      rc = set_error(HADES_ERR_HIP, "cannot unregister %s: %s", name, hipGetErrorString(err));
    }
  }
  if (munmap(ptr, static_cast<size_t>(size)) == -1 && rc == HADES_OK)
    rc = set_error(HADES_ERR_ARG, "munmap of %s failed: %s", name, strerror(errno));
  close(static_cast<int>(fd));
  shm_unlink(name);  // as the reference: every release unlinks; a name already gone is not an error
  return rc;
}

int hades_shm_exists(const char* name) {
  if (!name || !name[0]) return 0;
  const int fd = shm_open(name, O_RDONLY, S_IRUSR | S_IWUSR);
  if (fd < 0) return 0;
  close(fd);
  return 1;
}

}  // extern "C"
