// Pre-exchange bucketing: the part of swap_gradients that runs on one GPU before the all-to-all
// (python/EmbCache/sparse_optim.py:33-50):
//   split  = cudaReminder(ids, trainers_per_part)                       (:36)
//          | cudaBinarySearch(ids, partition_range, trainers_per_part)  (:38-39)
//   value, indices = torch.sort(split); ids = ids[indices]; grads = grads[indices]   (:41-45)
//   input_splits = diff(cudaBinarySearch2(arange(num_owners), value))   (:48-52)
// Here it is one call: owner ranks -> stable radix sort of (owner, position) over the few bits
// num_owners needs (one 8-bit pass up to 256 owners) -> per-owner sizes from the sorted owners ->
// gather of ids, counts and gradient rows through the sort permutation.  The sort is stable, so
// rows keep their original order inside each bucket (torch.sort leaves that order unspecified).
#include "internal.h"

namespace hades {
namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void owner_of_kernel(const int64_t* __restrict__ ids,
                                                           int64_t n,
                                                           const int64_t* __restrict__ range,
                                                           int64_t num_part, int64_t m,
                                                           int64_t* __restrict__ owner) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const int64_t v = ids[i];
  int64_t o = v % m;  // C remainder, as ReminderKernel (src/cuda/binary_search.cu:36-43)
  if (range != nullptr)  // BinarySearchKernel (src/cuda/binary_search.cu:11-21)
    o += (upper_bound_dev<int64_t>(range, num_part, v) - 1) * m;
  owner[i] = o;
}

// sizes[g] = number of sorted owners equal to g (difference of two upper bounds, which is what
// the reference takes from cudaBinarySearch2 over arange(num_owners))
// An owner outside [0, num_owners) leaves the owners unsorted: every size is then reported as -1.
__global__ __launch_bounds__(kThreads) void bucket_sizes_kernel(const uint32_t* __restrict__ sorted,
                                                               int64_t n, int64_t num_owners,
                                                               int64_t* __restrict__ sizes,
                                                               const int32_t* __restrict__ bad,
                                                               int64_t nbad) {
  const int violated = any_flag_set(bad, nbad);
  const int64_t g = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (g >= num_owners) return;
  if (violated) {
    sizes[g] = -1;
    return;
  }
  const int64_t hi = upper_bound_dev<uint32_t>(sorted, n, static_cast<uint32_t>(g));
  const int64_t lo = g > 0 ? upper_bound_dev<uint32_t>(sorted, n, static_cast<uint32_t>(g - 1)) : 0;
  sizes[g] = hi - lo;
}

__global__ __launch_bounds__(kThreads) void bucket_gather_kernel(
    const uint32_t* __restrict__ perm, int64_t n, const int64_t* __restrict__ ids,
    const int64_t* __restrict__ cnt, int64_t* __restrict__ ids_out, int64_t* __restrict__ cnt_out,
    int64_t* __restrict__ perm_out) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (j >= n) return;
  const uint32_t p = perm[j];
  ids_out[j] = ids[p];
  if (cnt_out != nullptr) cnt_out[j] = cnt[p];
  if (perm_out != nullptr) perm_out[j] = static_cast<int64_t>(p);
}

__global__ __launch_bounds__(kThreads) void zero_i64_kernel(int64_t* __restrict__ out, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) out[i] = 0;
}

inline size_t round256(size_t b) { return (b + 255) & ~size_t(255); }

}  // namespace
}  // namespace hades

using namespace hades;

extern "C" {

size_t hades_bucket_workspace_bytes(int64_t n) {
  if (n < 0) return 0;
  const int64_t nn = n > 0 ? n : 1;
  return round256(sort_ids_workspace_bytes(nn)) + round256(static_cast<size_t>(nn) * 8);
}

int hades_bucket_by_owner(const int64_t* ids, int64_t n, const int64_t* range_partition,
                          int64_t num_part, int64_t local_num_gpus, int64_t num_owners,
                          const void* grad, int64_t dim, int dtype, const int64_t* cnt,
                          int64_t* ids_out, void* grad_out, int64_t* cnt_out,
                          int64_t* split_sizes, int64_t* perm_out, void* workspace,
                          size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(n >= 0 && n < (int64_t(1) << 30), "bucket: n must be in [0, 2^30) (got %lld)",
                (long long)n);
  HADES_REQUIRE(local_num_gpus >= 1, "local_num_gpus must be >= 1");
  HADES_REQUIRE(num_owners >= 1 && num_owners < (int64_t(1) << 31), "num_owners out of range");
  HADES_REQUIRE(num_part >= 0 && (range_partition == nullptr || num_part >= 1),
                "a partition range needs num_part >= 1");
  HADES_REQUIRE(split_sizes != nullptr, "split_sizes must not be null");
  HADES_REQUIRE((grad == nullptr) == (grad_out == nullptr), "grad and grad_out go together");
  HADES_REQUIRE((cnt == nullptr) == (cnt_out == nullptr), "cnt and cnt_out go together");
  HADES_REQUIRE(grad == nullptr || dim >= 1, "dim must be >= 1");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n == 0) {
    HADES_LAUNCH(zero_i64_kernel, dim3(static_cast<unsigned>(ceil_div(num_owners, kThreads))),
                 dim3(kThreads), 0, st, split_sizes, num_owners);
    return HADES_OK;
  }
  HADES_REQUIRE(ids && ids_out, "null pointer argument");
  const size_t sort_bytes = round256(sort_ids_workspace_bytes(n));
  const size_t need = hades_bucket_workspace_bytes(n);
  if (workspace == nullptr || workspace_bytes < need)
    return set_error(HADES_ERR_WORKSPACE, "bucket workspace too small: need %zu bytes, got %zu",
                     need, workspace_bytes);
  int64_t* owner = reinterpret_cast<int64_t*>(static_cast<char*>(workspace) + sort_bytes);
  const dim3 grid(static_cast<unsigned>(ceil_div(n, kThreads))), block(kThreads);

  HADES_LAUNCH(owner_of_kernel, grid, block, 0, st, ids, n, range_partition, num_part,
               local_num_gpus, owner);
  // owners outside [0, num_owners) (negative ids, ids beyond the last range) are flagged by the
  // sort's first pass, as ids beyond id_bound are in the combine; the sizes kernel reports them
  SortResult sr;
  const int rc = sort_ids(owner, n, num_owners, workspace, sort_bytes, st, &sr);
  if (rc != HADES_OK) return rc;
  HADES_REQUIRE(!sr.key64, "internal: owner keys must be 32-bit");
  HADES_LAUNCH(bucket_sizes_kernel, dim3(static_cast<unsigned>(ceil_div(num_owners, kThreads))),
               block, 0, st, static_cast<const uint32_t*>(sr.sorted_keys), n, num_owners,
               split_sizes, sr.bad, sr.nbad);
  HADES_LAUNCH(bucket_gather_kernel, grid, block, 0, st, sr.perm, n, ids, cnt, ids_out, cnt_out,
               perm_out);
  if (grad != nullptr)  // rows: dst[j, :] = src[perm[j], :] (positions are below 2^30: int32 index)
    return hades_fetch2(grad, sr.perm, grad_out, n, dim, dtype, HADES_I32, stream);
  return HADES_OK;
}

}  // extern "C"
