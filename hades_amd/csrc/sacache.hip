// Set-associative index cache on the device: the reference's SACacheIndex<int64, int64>
// (src/cache/cache.h:11-259) over 8-entry lines (cache_line, src/cache/cache_line.h:5-103), which
// the reference keeps in host shared memory and walks with OpenMP loops (its device lookup,
// src/cache/lookup.cu:15-45, reads the same structure through pinned memory).
//
// State, in device memory owned by the caller:
//   line_ids int64[lines * 8]   id held by (line, entry), -1 = empty; loc = line * 8 + entry
//   line_age int32[lines * 8]   the access table of the line (LRU ages)
// An id lives in line id % lines.
//
// add and the aging lookup change a line as they go, so their result depends on the order in
// which the ids of one line are handled.  Here that order is the input order, whatever the launch
// geometry: the batch is sorted stably by line (one or two radix passes over the line number) and
// the thread that owns the first id of a line walks all ids of that line in sequence with the
// line in registers.  Different lines are independent.  The reference gets this order with one
// OpenMP thread; with more its result varies from run to run.
#include "internal.h"

namespace hades {
namespace {

constexpr int kThreads = 256;
constexpr int kLine = 8;  // CACHE_LINE_SIZE, src/cache/cache_line.h:5

struct Line {
  int64_t id[kLine];
  int32_t age[kLine];
};

__device__ __forceinline__ void load_line(const int64_t* __restrict__ line_ids,
                                          const int32_t* __restrict__ line_age, int64_t ln,
                                          Line& l) {
#pragma unroll
  for (int e = 0; e < kLine; ++e) {
    l.id[e] = line_ids[ln * kLine + e];
    l.age[e] = line_age[ln * kLine + e];
  }
}

__device__ __forceinline__ void store_line(int64_t* __restrict__ line_ids,
                                           int32_t* __restrict__ line_age, int64_t ln,
                                           const Line& l) {
#pragma unroll
  for (int e = 0; e < kLine; ++e) {
    line_ids[ln * kLine + e] = l.id[e];
    line_age[ln * kLine + e] = l.age[e];
  }
}

// set_id (cache_line.h:20-24) on a register-resident line, entry chosen at run time
__device__ __forceinline__ void set_entry(Line& l, int entry, int64_t v) {
#pragma unroll
  for (int e = 0; e < kLine; ++e)
    if (e == entry) {
      l.id[e] = v;
      l.age[e] = 0;
    }
}

// _add for one id (cache.h:55-86).  Returns the entry, or -1.
__device__ __forceinline__ int add_one(Line& l, int64_t v) {
  // find_or_empty_entry (cache_line.h:66-77): the id's entry, else the last empty one
  int idx = -1;
  bool exist = false;
#pragma unroll
  for (int e = 0; e < kLine; ++e) {
    if (!exist) {
      if (l.id[e] == v) {
        idx = e;
        exist = true;
      } else if (l.id[e] == -1) {
        idx = e;
      }
    }
  }
  if (idx >= 0) {
    if (!exist) set_entry(l, idx, v);
    return idx;
  }
  // find_lru (cache_line.h:91-102): largest age strictly above entry 0's; none if that is 0
  int lru = 0;
  int32_t tmp = l.age[0];
#pragma unroll
  for (int e = 0; e < kLine; ++e)
    if (l.age[e] > tmp && l.age[e] != 0) {
      lru = e;
      tmp = l.age[e];
    }
  if (tmp == 0) return -1;
  set_entry(l, lru, v);
  return lru;
}

// _lookup for one id (cache.h:96-105): find, then access_loc (cache_line.h:79-85)
__device__ __forceinline__ int touch_one(Line& l, int64_t v) {
  int hit = -1;
#pragma unroll
  for (int e = 0; e < kLine; ++e)
    if (hit < 0 && l.id[e] == v) hit = e;
  if (hit >= 0) {
#pragma unroll
    for (int e = 0; e < kLine; ++e) l.age[e] = (e == hit) ? 0 : l.age[e] + 1;
  }
  return hit;
}

__global__ __launch_bounds__(kThreads) void sac_init_kernel(int64_t* __restrict__ line_ids,
                                                           int32_t* __restrict__ line_age,
                                                           int64_t entries) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < entries) {
    line_ids[i] = -1;
    line_age[i] = 0;
  }
}

// negative ids have no line (the reference would index before its array): they are given the
// key `lines`, sort behind every real line, and get loc -1
__global__ __launch_bounds__(kThreads) void sac_line_of_kernel(const int64_t* __restrict__ ids,
                                                              int64_t n, int64_t lines,
                                                              int64_t* __restrict__ key) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) key[i] = ids[i] >= 0 ? ids[i] % lines : lines;
}

template <bool ADD>
__global__ __launch_bounds__(kThreads) void sac_walk_kernel(
    const uint32_t* __restrict__ sorted_line, const uint32_t* __restrict__ perm, int64_t n,
    const int64_t* __restrict__ ids, int64_t lines, int64_t* __restrict__ line_ids,
    int32_t* __restrict__ line_age, int64_t* __restrict__ locs) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (j >= n) return;
  const uint32_t ln = sorted_line[j];
  if (static_cast<int64_t>(ln) >= lines) {       // ids without a line (negative; e.g. the padding
    locs[perm[j]] = -1;                          // of a batch whose length lives on the device):
    return;                                      // every thread answers for its own entry
  }
  if (j > 0 && sorted_line[j - 1] == ln) return;  // not the first id of its line
  Line l;
  load_line(line_ids, line_age, ln, l);
  for (int64_t k = j; k < n && sorted_line[k] == ln; ++k) {
    const uint32_t p = perm[k];
    const int e = ADD ? add_one(l, ids[p]) : touch_one(l, ids[p]);
    locs[p] = e >= 0 ? static_cast<int64_t>(ln) * kLine + e : int64_t(-1);
  }
  store_line(line_ids, line_age, ln, l);
}

// lookupkernel2 (src/cache/lookup.cu:15-45): the search alone, nothing is aged
__global__ __launch_bounds__(kThreads) void sac_lookup_kernel(const int64_t* __restrict__ line_ids,
                                                             int64_t lines,
                                                             const int64_t* __restrict__ ids,
                                                             int64_t n, int64_t* __restrict__ locs) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const int64_t v = ids[i];
  int64_t loc = -1;
  if (v >= 0) {
    const int64_t ln = v % lines;
    typedef int64_t i64x2 __attribute__((ext_vector_type(2)));
    const i64x2* row = reinterpret_cast<const i64x2*>(line_ids + ln * kLine);
#pragma unroll
    for (int h = 0; h < kLine / 2; ++h) {
      const i64x2 two = row[h];
      if (loc < 0 && two.x == v) loc = ln * kLine + 2 * h;
      if (loc < 0 && two.y == v) loc = ln * kLine + 2 * h + 1;
    }
  }
  locs[i] = loc;
}

// _reset (cache.h:109-121).  Ids of one line free different entries, so threads do not collide.
__global__ __launch_bounds__(kThreads) void sac_reset_kernel(int64_t* __restrict__ line_ids,
                                                            int32_t* __restrict__ line_age,
                                                            int64_t lines,
                                                            const int64_t* __restrict__ ids,
                                                            int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const int64_t v = ids[i];
  if (v < 0) return;
  const int64_t ln = v % lines;
  for (int e = 0; e < kLine; ++e)
    if (line_ids[ln * kLine + e] == v) {
      line_ids[ln * kLine + e] = -1;
      line_age[ln * kLine + e] = 0;
      return;
    }
}

__global__ __launch_bounds__(kThreads) void sac_emit_kernel(const int64_t* __restrict__ line_ids,
                                                           const int64_t* __restrict__ pos,
                                                           const int64_t* __restrict__ count,
                                                           int64_t cap,
                                                           int64_t* __restrict__ ids_out,
                                                           int64_t* __restrict__ locs_out,
                                                           int64_t* __restrict__ num_out,
                                                           int64_t* __restrict__ num_valid) {
  const int64_t live = count[0];
  const int64_t m = live < cap ? live : cap;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i == 0) {
    if (num_out) num_out[0] = m;
    if (num_valid) num_valid[0] = live;
  }
  if (i < m) {
    const int64_t p = pos[i];
    ids_out[i] = line_ids[p];
    locs_out[i] = p;
  }
}

inline size_t round256(size_t b) { return (b + 255) & ~size_t(255); }
inline unsigned grid_of(int64_t n) { return static_cast<unsigned>(ceil_div(n > 0 ? n : 1, kThreads)); }

template <bool ADD>
int ordered_pass(int64_t* line_ids, int32_t* line_age, int64_t lines, const int64_t* ids,
                 int64_t n, int64_t* locs, void* workspace, size_t workspace_bytes,
                 hipStream_t st) {
  const size_t sort_bytes = round256(sort_ids_workspace_bytes(n));
  const size_t need = sort_bytes + round256(static_cast<size_t>(n) * 8);
  if (workspace == nullptr || workspace_bytes < need)
    return set_error(HADES_ERR_WORKSPACE, "index cache workspace too small: need %zu bytes, got %zu",
                     need, workspace_bytes);
  int64_t* key = reinterpret_cast<int64_t*>(static_cast<char*>(workspace) + sort_bytes);
  HADES_LAUNCH(sac_line_of_kernel, dim3(grid_of(n)), dim3(kThreads), 0, st, ids, n, lines, key);
  SortResult sr;
  const int rc = sort_ids(key, n, lines + 1, workspace, sort_bytes, st, &sr);
  if (rc != HADES_OK) return rc;
  HADES_REQUIRE(!sr.key64, "internal: line keys must be 32-bit");
  HADES_LAUNCH((sac_walk_kernel<ADD>), dim3(grid_of(n)), dim3(kThreads), 0, st,
               static_cast<const uint32_t*>(sr.sorted_keys), sr.perm, n, ids, lines, line_ids,
               line_age, locs);
  return HADES_OK;
}

int check_state(const void* line_ids, int64_t lines) {
  HADES_REQUIRE(line_ids != nullptr, "line_ids must not be null");
  HADES_REQUIRE(lines >= 1 && lines < (int64_t(1) << 28), "lines must be in [1, 2^28)");
  return HADES_OK;
}

}  // namespace
}  // namespace hades

using namespace hades;

extern "C" {

int hades_sacache_init(int64_t* line_ids, int32_t* line_age, int64_t lines, void* stream) {
  if (int rc = check_state(line_ids, lines)) return rc;
  HADES_REQUIRE(line_age != nullptr, "line_age must not be null");
  HADES_LAUNCH(sac_init_kernel, dim3(grid_of(lines * kLine)), dim3(kThreads), 0,
               static_cast<hipStream_t>(stream), line_ids, line_age, lines * kLine);
  return HADES_OK;
}

size_t hades_sacache_workspace_bytes(int64_t n) {
  if (n < 0) return 0;
  const int64_t nn = n > 0 ? n : 1;
  return round256(sort_ids_workspace_bytes(nn)) + round256(static_cast<size_t>(nn) * 8);
}

int hades_sacache_add(int64_t* line_ids, int32_t* line_age, int64_t lines, const int64_t* ids,
                      int64_t n, int64_t* locs, void* workspace, size_t workspace_bytes,
                      void* stream) {
  if (int rc = check_state(line_ids, lines)) return rc;
  HADES_REQUIRE(n >= 0 && n < (int64_t(1) << 30), "n must be in [0, 2^30)");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(line_age && ids && locs, "null pointer argument");
  return ordered_pass<true>(line_ids, line_age, lines, ids, n, locs, workspace, workspace_bytes,
                            static_cast<hipStream_t>(stream));
}

int hades_sacache_lookup_touch(int64_t* line_ids, int32_t* line_age, int64_t lines,
                               const int64_t* ids, int64_t n, int64_t* locs, void* workspace,
                               size_t workspace_bytes, void* stream) {
  if (int rc = check_state(line_ids, lines)) return rc;
  HADES_REQUIRE(n >= 0 && n < (int64_t(1) << 30), "n must be in [0, 2^30)");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(line_age && ids && locs, "null pointer argument");
  return ordered_pass<false>(line_ids, line_age, lines, ids, n, locs, workspace, workspace_bytes,
                             static_cast<hipStream_t>(stream));
}

int hades_sacache_lookup(const int64_t* line_ids, int64_t lines, const int64_t* ids, int64_t n,
                         int64_t* locs, void* stream) {
  if (int rc = check_state(line_ids, lines)) return rc;
  HADES_REQUIRE(n >= 0 && ceil_div(n, kThreads) < (int64_t(1) << 31), "n out of range");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(ids && locs, "null pointer argument");
  HADES_LAUNCH(sac_lookup_kernel, dim3(grid_of(n)), dim3(kThreads), 0,
               static_cast<hipStream_t>(stream), line_ids, lines, ids, n, locs);
  return HADES_OK;
}

int hades_sacache_reset(int64_t* line_ids, int32_t* line_age, int64_t lines, const int64_t* ids,
                        int64_t n, void* stream) {
  if (int rc = check_state(line_ids, lines)) return rc;
  HADES_REQUIRE(n >= 0 && ceil_div(n, kThreads) < (int64_t(1) << 31), "n out of range");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(line_age && ids, "null pointer argument");
  HADES_LAUNCH(sac_reset_kernel, dim3(grid_of(n)), dim3(kThreads), 0,
               static_cast<hipStream_t>(stream), line_ids, line_age, lines, ids, n);
  return HADES_OK;
}

size_t hades_sacache_getall_workspace_bytes(int64_t lines) {
  if (lines < 1) return 0;
  const int64_t entries = lines * kLine;
  return round256(compact_live_workspace_bytes(entries)) +
         round256(static_cast<size_t>(entries) * 8) + 256;
}

int hades_sacache_getall(const int64_t* line_ids, int64_t lines, int64_t* ids_out,
                         int64_t* locs_out, int64_t* num_out, int64_t* num_valid, int64_t cap,
                         void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_state(line_ids, lines)) return rc;
  HADES_REQUIRE(cap >= 0, "cap must be >= 0");
  HADES_REQUIRE(cap == 0 || (ids_out && locs_out), "null output pointer");
  HADES_REQUIRE(num_out || num_valid, "one of num_out and num_valid must be given");
  const int64_t entries = lines * kLine;
  const size_t cbytes = round256(compact_live_workspace_bytes(entries));
  const size_t need = hades_sacache_getall_workspace_bytes(lines);
  if (workspace == nullptr || workspace_bytes < need)
    return set_error(HADES_ERR_WORKSPACE, "getall workspace too small: need %zu bytes, got %zu",
                     need, workspace_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* base = static_cast<char*>(workspace);
  int64_t* pos = reinterpret_cast<int64_t*>(base + cbytes);
  int64_t* count = reinterpret_cast<int64_t*>(base + cbytes + round256(static_cast<size_t>(entries) * 8));
  const int rc = compact_live_keys(line_ids, entries, pos, count, workspace, cbytes, st);
  if (rc != HADES_OK) return rc;
  const int64_t m = cap < entries ? cap : entries;
  HADES_LAUNCH(sac_emit_kernel, dim3(grid_of(m)), dim3(kThreads), 0, st, line_ids, pos, count, cap,
               ids_out, locs_out, num_out, num_valid);
  return HADES_OK;
}

}  // extern "C"
