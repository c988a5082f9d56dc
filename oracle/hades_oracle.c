/*
 * Plain-C restatement of the reference's native (CUDA) operators on the embedding-cache hot
 * path, plus the combine and Adagrad arithmetic.  TEST INFRASTRUCTURE ONLY: built by
 * oracle/Makefile into oracle/libhades_oracle.so and loaded only by tests/ (to cross-check the
 * numpy restatement in hades_oracle.py) and by the cpu_baseline leg of bench.py.  The product
 * never links or loads it.
 *
 * Each function follows the reference kernel it cites, one loop iteration per CUDA thread/warp
 * iteration, with the same index arithmetic.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* cub::UpperBound as used in src/cuda/binary_search.cu:18,30: first index whose entry is > val */
static int64_t upper_bound_i64(const int64_t* a, int64_t n, int64_t val) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    int64_t mid = lo + ((hi - lo) >> 1);
    if (a[mid] <= val) lo = mid + 1; else hi = mid;
  }
  return lo;
}

/* BinarySearchKernel2, src/cuda/binary_search.cu:24-33 */
void o_binary_search2(const int64_t* in, const int64_t* range, int64_t num_part, int64_t* out,
                      int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = upper_bound_i64(range, num_part, in[i]);
}

/* BinarySearchKernel, src/cuda/binary_search.cu:11-21 */
void o_binary_search(const int64_t* in, const int64_t* range_partition, int64_t num_part,
                     int64_t local_num_gpus, int64_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t val = in[i];
    int64_t rank = upper_bound_i64(range_partition, num_part, val);
    out[i] = (rank - 1) * local_num_gpus + val % local_num_gpus;
  }
}

/* ReminderKernel, src/cuda/binary_search.cu:36-43 */
void o_reminder(const int64_t* in, int64_t local_num_gpus, int64_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = in[i] % local_num_gpus;
}

/* membership + slot on top of UpperBound (the EmbCache lookup) */
void o_lookup_sorted(const int64_t* q, int64_t n, const int64_t* sorted_hot, int64_t num_hot,
                     int64_t* loc) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t pos = upper_bound_i64(sorted_hot, num_hot, q[i]);
    loc[i] = (pos > 0 && sorted_hot[pos - 1] == q[i]) ? pos - 1 : -1;
  }
}

/* _split lambda, src/cuda/split.cu:32-44; masks are zero-filled first (:16-24) */
void o_split(const int64_t* ids, const int8_t* mask, int64_t n, uint8_t* local_mask,
             uint8_t* remote_hot_mask, uint8_t* remote_cold_mask) {
  memset(local_mask, 0, (size_t)n);
  memset(remote_hot_mask, 0, (size_t)n);
  memset(remote_cold_mask, 0, (size_t)n);
  for (int64_t i = 0; i < n; ++i) {
    int8_t value = mask[ids[i]];
    if (value == 0) local_mask[i] = 1;
    else if (value == 1) remote_hot_mask[i] = 1;
    else if (value == 2) remote_cold_mask[i] = 1;
  }
}

/* UVAFetchKernel, src/cuda/uva_fetch.cu:11-26 (rows as raw bytes: the copy is type-agnostic) */
void o_fetch(const char* src, const int64_t* src_index, char* dst, const int64_t* dst_index,
             int64_t n, int64_t row_bytes) {
  for (int64_t i = 0; i < n; ++i)
    memcpy(dst + dst_index[i] * row_bytes, src + src_index[i] * row_bytes, (size_t)row_bytes);
}

/* UVAFetchKernel2 / UVAFetch1DKernel2, src/cuda/uva_fetch.cu:48-70 */
void o_fetch2(const char* src, const int64_t* src_index, char* dst, int64_t n, int64_t row_bytes) {
  for (int64_t i = 0; i < n; ++i)
    memcpy(dst + i * row_bytes, src + src_index[i] * row_bytes, (size_t)row_bytes);
}

/* CUDAFetchWithCacheKernel2, src/cuda/uva_fetch.cu:108-130 */
void o_fetch_with_cache2(const char* cpu_src, const char* gpu_src, const int64_t* index,
                         const int64_t* index_map, char* dst, int64_t n, int64_t row_bytes) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t idx = index[i];
    int64_t gpu_idx = index_map[idx];
    const char* s = gpu_idx != -1 ? gpu_src + gpu_idx * row_bytes : cpu_src + idx * row_bytes;
    memcpy(dst + i * row_bytes, s, (size_t)row_bytes);
  }
}

/* UVASetKernel, src/cuda/uva_set.cu:11-24; UVACombineKernel, src/cuda/uva_fetch.cu:195-210 */
void o_set(const char* src, char* dst, const int64_t* dst_index, int64_t n, int64_t row_bytes) {
  for (int64_t i = 0; i < n; ++i)
    memcpy(dst + dst_index[i] * row_bytes, src + i * row_bytes, (size_t)row_bytes);
}

/* CUDASetWithCacheKernel, src/cuda/uva_set.cu:71-93 */
void o_set_with_cache(const char* src, char* cpu_dst, char* gpu_dst, const int64_t* index,
                      const int64_t* index_map, int64_t n, int64_t row_bytes) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t idx = index[i];
    int64_t gpu_idx = index_map[idx];
    char* d = gpu_idx != -1 ? gpu_dst + gpu_idx * row_bytes : cpu_dst + idx * row_bytes;
    memcpy(d, src + i * row_bytes, (size_t)row_bytes);
  }
}

/* combine = only_unique_grads, python/EmbCache/sparse_optim.py:132-139: sorted distinct ids,
 * counts, and per-id float32 sums accumulated from +0.0f in occurrence order (what CPU index_add_
 * does).  Stable merge sort of (id, position).  Returns the number of distinct ids. */
typedef struct { int64_t id; int64_t pos; } pair_t;

static void merge_sort_pairs(pair_t* a, pair_t* tmp, int64_t n) {
  for (int64_t width = 1; width < n; width *= 2) {
    for (int64_t lo = 0; lo < n; lo += 2 * width) {
      int64_t mid = lo + width < n ? lo + width : n;
      int64_t hi = lo + 2 * width < n ? lo + 2 * width : n;
      int64_t i = lo, j = mid, k = lo;
      while (i < mid && j < hi) tmp[k++] = (a[j].id < a[i].id) ? a[j++] : a[i++];
      while (i < mid) tmp[k++] = a[i++];
      while (j < hi) tmp[k++] = a[j++];
    }
    memcpy(a, tmp, (size_t)n * sizeof(pair_t));
  }
}

int64_t o_combine(const int64_t* idx, const float* grad, int64_t n, int64_t dim, int64_t* uids,
                  float* sums, int64_t* cnts) {
  if (n == 0) return 0;
  pair_t* a = (pair_t*)malloc((size_t)n * sizeof(pair_t));
  pair_t* tmp = (pair_t*)malloc((size_t)n * sizeof(pair_t));
  for (int64_t i = 0; i < n; ++i) { a[i].id = idx[i]; a[i].pos = i; }
  merge_sort_pairs(a, tmp, n);
  int64_t u = -1;
  for (int64_t j = 0; j < n; ++j) {
    if (j == 0 || a[j].id != a[j - 1].id) {
      ++u;
      uids[u] = a[j].id;
      cnts[u] = 0;
      for (int64_t c = 0; c < dim; ++c) sums[u * dim + c] = 0.0f;
    }
    cnts[u] += 1;
    const float* g = grad + a[j].pos * dim;
    float* s = sums + u * dim;
    for (int64_t c = 0; c < dim; ++c) s[c] = s[c] + g[c];
  }
  free(a);
  free(tmp);
  return u + 1;
}

/* sparse Adagrad on rows addressed like cached_fetch/cached_set: every operation rounded to
 * float (volatile temporaries keep the compiler from fusing or widening) */
void o_adagrad(const int64_t* uids, const float* g, int64_t num_rows, int64_t dim,
               const int64_t* sorted_hot, int64_t num_hot, float* hot_w, float* hot_s,
               float* cold_w, float* cold_s, float lr, float eps) {
  for (int64_t u = 0; u < num_rows; ++u) {
    int64_t id = uids[u];
    int64_t pos = upper_bound_i64(sorted_hot, num_hot, id);
    int hit = pos > 0 && sorted_hot[pos - 1] == id;
    float* w = hit ? hot_w + (pos - 1) * dim : cold_w + id * dim;
    float* s = hit ? hot_s + (pos - 1) * dim : cold_s + id * dim;
    for (int64_t c = 0; c < dim; ++c) {
      volatile float gg = g[u * dim + c] * g[u * dim + c];
      volatile float s1 = s[c] + gg;
      volatile float sq = sqrtf(s1);
      volatile float sd = sq + eps;
      volatile float lg = lr * g[u * dim + c];
      volatile float q = lg / sd;
      s[c] = s1;
      w[c] = w[c] - q;
    }
  }
}
