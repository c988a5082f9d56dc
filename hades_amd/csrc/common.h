// Shared host/device helpers for libhades_hip.so (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/hades_hip.h"

namespace hades {

constexpr int kWave = 64;  // CDNA wavefront width

// ---- error reporting: thread-local message, never exit() -------------------
int set_error(int code, const char* fmt, ...);

#define HADES_HIP_TRY(expr)                                                          \
  do {                                                                               \
    hipError_t _e = (expr);                                                          \
    if (_e != hipSuccess) {                                                          \
      (void)hipGetLastError();                                                       \
      return ::hades::set_error(HADES_ERR_HIP, "%s:%d: %s failed: %s", __FILE__,     \
                                __LINE__, #expr, hipGetErrorString(_e));             \
    }                                                                                \
  } while (0)

#define HADES_REQUIRE(cond, ...)                                                     \
  do {                                                                               \
    if (!(cond)) return ::hades::set_error(HADES_ERR_ARG, __VA_ARGS__);              \
  } while (0)

// Kernel launch with an error check (the reference never checks its launches).  The error state
// is read once before the launch so that a stale error left by an earlier, unrelated HIP call of
// the process is not blamed on this kernel.
#define HADES_LAUNCH(...)                     \
  do {                                        \
    (void)hipGetLastError();                  \
    hipLaunchKernelGGL(__VA_ARGS__);          \
    HADES_HIP_TRY(hipGetLastError());         \
  } while (0)
#define HADES_LAUNCH_CHECK() HADES_HIP_TRY(hipGetLastError())

// Optional timing of one named kernel: hades_profile_kernel() arms a pair of HIP events that the
// next launches of that kernel (on the calling thread) record around themselves, on the stream
// the kernel is launched on.
struct ProfileSlot {
  int kernel_id = 0;
  hipEvent_t start = nullptr, stop = nullptr;
};
extern thread_local ProfileSlot g_profile;

#define HADES_LAUNCH_TIMED(kid, stream_, ...)                                        \
  do {                                                                               \
    const bool _timed = ::hades::g_profile.kernel_id == (kid);                       \
    if (_timed) HADES_HIP_TRY(hipEventRecord(::hades::g_profile.start, (stream_)));  \
    HADES_LAUNCH(__VA_ARGS__);                                                       \
    if (_timed) HADES_HIP_TRY(hipEventRecord(::hades::g_profile.stop, (stream_)));   \
  } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }
inline int ilog2_ceil(uint64_t x) {  // smallest b with 2^b >= x
  int b = 0;
  while (b < 64 && (uint64_t(1) << b) < x) ++b;
  return b;
}
inline uintptr_t align_of_ptr(const void* p) { return reinterpret_cast<uintptr_t>(p); }

// true if `p` is host memory that kernels reach over the host link (hipHostMalloc / registered)
bool is_host_memory(const void* p);
// blocks to launch for a kernel whose table rows cross the host link (see core.hip)
// what a kernel does over the host link: copies rows one way, updates rows in place (reads and
// writes at once), or only writes them (the old rows come from device memory)
enum HostLinkUse { kLinkCopy = 0, kLinkReadWrite = 1, kLinkWriteOnly = 2 };
int64_t host_link_blocks(HostLinkUse use);

// Carve aligned sub-buffers out of a caller-provided workspace.
struct Carver {
  char* base;
  size_t off = 0;
  explicit Carver(void* p) : base(static_cast<char*>(p)) {}
  template <typename T>
  T* take(size_t count) {
    off = (off + 255) & ~size_t(255);
    T* r = base ? reinterpret_cast<T*>(base + off) : nullptr;
    off += count * sizeof(T);
    return r;
  }
  size_t total() const { return (off + 255) & ~size_t(255); }
};

// ---- device helpers ---------------------------------------------------------
#if defined(__HIPCC__)

__device__ __forceinline__ int lane_id() { return __lane_id(); }

// number of entries of ascending a[0..n) that are <= v  (std::upper_bound index)
template <typename T>
__device__ __forceinline__ int64_t upper_bound_dev(const T* __restrict__ a, int64_t n, T v) {
  int64_t lo = 0, len = n;
  while (len > 0) {
    int64_t half = len >> 1;
    T x = a[lo + half];
    if (x <= v) {
      lo += half + 1;
      len -= half + 1;
    } else {
      len = half;
    }
  }
  return lo;
}

// slot of v in the ascending duplicate-free set a[0..n), or -1
__device__ __forceinline__ int64_t lookup_slot_dev(const int64_t* __restrict__ a, int64_t n,
                                                   int64_t v) {
  int64_t pos = upper_bound_dev<int64_t>(a, n, v);
  return (pos > 0 && a[pos - 1] == v) ? pos - 1 : int64_t(-1);
}

// The hot-ID set as the kernels see it: the ascending ids, and optionally a bucket index over
// them.  Index layout (uint32 words): [0] shift, [1] log2(buckets), [2] form, [3] unused, then the
// bucket table; bucket b holds the ids with (id >> shift) == b.
//   form 1: table[b] (one word) = first position whose id >= (b << shift); a lookup reads two
//           adjacent words and then searches the ids of the bucket: two dependent reads.
//   form 2 (built whenever shift <= 24): table[b] (two words) = {first position, (count << 24) |
//           the low `shift` bits of the bucket's first id}, count saturating at 255.  All ids of a
//           bucket share their high bits, so the low bits identify the first id: a query that is
//           the first id of its bucket, or falls into an empty bucket, or below the first id, or
//           into a bucket of one, is answered from the one 8-byte entry - with about one bucket
//           per hot id that is three queries in four - and only the rest go on to search the
//           other ids of the bucket.
//   form 0: no usable index (negative ids, or more than 2^32 - 1 of them): plain binary search.
constexpr int kHotIndexHeader = 4;
struct HotSet {
  const int64_t* sorted;
  int64_t n;
  const uint32_t* index;  // may be null

  __device__ __forceinline__ int64_t search(int64_t lo, int64_t hi, int64_t v) const {
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      const int64_t x = sorted[mid];
      if (x == v) return mid;
      if (x < v) lo = mid + 1; else hi = mid;
    }
    return -1;
  }

  __device__ __forceinline__ int64_t slot(int64_t v) const {
    if (index == nullptr || index[2] == 0u) return lookup_slot_dev(sorted, n, v);
    if (v < 0) return -1;
    const uint32_t shift = index[0];
    const uint64_t b = static_cast<uint64_t>(v) >> shift;
    if (b >> index[1]) return -1;  // beyond the largest hot id
    if (index[2] == 2u) {
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
      const u32x2* table = reinterpret_cast<const u32x2*>(index + kHotIndexHeader);
      const u32x2 e = table[b];
      const uint32_t cnt = e.y >> 24;
      if (cnt == 0u) return -1;
      const uint32_t low = static_cast<uint32_t>(v) & ((1u << shift) - 1u);
      const uint32_t first = e.y & 0xffffffu;
      if (low == first) return e.x;
      if (low < first || cnt == 1u) return -1;
      const int64_t hi = cnt < 255u ? static_cast<int64_t>(e.x) + cnt : static_cast<int64_t>(table[b + 1].x);
      return search(static_cast<int64_t>(e.x) + 1, hi, v);
    }
    return search(index[kHotIndexHeader + b], index[kHotIndexHeader + b + 1], v);
  }
};

// wave64 inclusive prefix sum over the lanes of a wavefront (lane 63 ends up with the wave total)
template <typename T>
__device__ __forceinline__ T wave_inclusive_sum(T v) {
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    T t = __shfl_up(v, d, kWave);
    if (lane_id() >= d) v += t;
  }
  return v;
}

// lanes below mine whose ballot bit is set
__device__ __forceinline__ uint32_t ballot_rank(uint64_t ballot) {
  return __builtin_amdgcn_mbcnt_hi(uint32_t(ballot >> 32),
                                   __builtin_amdgcn_mbcnt_lo(uint32_t(ballot), 0u));
}

#endif  // __HIPCC__

}  // namespace hades

#if defined(__HIPCC__)
namespace hades {

// Exclusive prefix sum of one value per thread over a block of kBlock threads (kBlock a multiple
// of 64, at most 1024).  Returns the exclusive prefix; *total receives the block sum.  `smem`
// must hold kBlock/64 + 1 elements of T.  Contains __syncthreads(): call from all threads.
template <typename T, int kBlock>
__device__ __forceinline__ T block_exclusive_sum(T v, T* smem, T* total) {
  constexpr int kWaves = kBlock / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const T inc = wave_inclusive_sum<T>(v);
  if (lane == kWave - 1) smem[wave] = inc;
  __syncthreads();
  if (threadIdx.x == 0) {
    T run = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      T t = smem[w];
      smem[w] = run;
      run += t;
    }
    smem[kWaves] = run;
  }
  __syncthreads();
  T res = smem[wave] + inc - v;
  *total = smem[kWaves];
  __syncthreads();  // smem may be reused by the caller
  return res;
}

}  // namespace hades
#endif
