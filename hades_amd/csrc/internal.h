// Building blocks shared between translation units of libhades_hip.so (not part of the C ABI).
#pragma once

#include "common.h"

namespace hades {

// index.hip: ascending positions i with keys[i * key_stride] != -1, and their number (device).
// pos_out needs capacity n.
size_t compact_live_workspace_bytes(int64_t n);
int compact_live_keys(const int64_t* keys, int64_t n, int64_t* pos_out, int64_t* count_out,
                      void* workspace, size_t workspace_bytes, hipStream_t st,
                      int64_t key_stride = 1);

// combine.hip: stable radix sort of (id, position) over the bits id_bound leaves significant.
// On return *perm_out[j] is the position in `ids` of the j-th smallest id and *sorted_keys the
// sorted keys in the sort's own key type (*key64 tells which: uint64 with the sign bit flipped,
// or uint32).  Both live in the workspace.
// bad[0..nbad) are flags of the sort's first pass: non-zero where an id was outside [0, id_bound)
// (the result is then not sorted); any_flag_set() folds them inside a consumer kernel.
struct SortResult {
  const void* sorted_keys;
  const uint32_t* perm;
  bool key64;
  const int32_t* bad;
  int64_t nbad;
};

#if defined(__HIPCC__)
// OR of flags[0..n) over the calling block (contains __syncthreads(): call from all threads)
__device__ __forceinline__ int any_flag_set(const int32_t* __restrict__ flags, int64_t n) {
  int v = 0;
  for (int64_t b = threadIdx.x; b < n; b += blockDim.x) v |= flags[b];
  return __syncthreads_or(v);
}
#endif
size_t sort_ids_workspace_bytes(int64_t n);

// combine.hip: where a plan made by hades_combine_plan / _plan_classed with the same (n, dim,
// id_bound) left its sort permutation and its run table inside `workspace`: perm[j] = batch
// position of sorted position j, seg_start[u] = first sorted position of run u (seg_start[U] = n).
int combine_plan_views(void* workspace, size_t workspace_bytes, int64_t n, int64_t dim,
                       int64_t id_bound, const uint32_t** perm, const uint32_t** seg_start);
int sort_ids(const int64_t* ids, int64_t n, int64_t id_bound, void* workspace,
             size_t workspace_bytes, hipStream_t st, SortResult* out);

}  // namespace hades
