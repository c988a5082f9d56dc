// Integer side of the path: routing arithmetic (src/cuda/binary_search.cu), the sorted-hot-set
// lookup, the class split (src/cuda/split.cu) and stable compaction of the split.
#include "internal.h"

namespace hades {
namespace {

constexpr int kThreads = 256;

// ---- routing: one element per thread ---------------------------------------
template <typename T>
__global__ __launch_bounds__(kThreads) void reminder_kernel(const T* __restrict__ in, T m,
                                                           T* __restrict__ out, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) out[i] = in[i] % m;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void owner_rank_kernel(const T* __restrict__ in,
                                                             const T* __restrict__ range,
                                                             int64_t num_part, T m,
                                                             T* __restrict__ out, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    const T v = in[i];
    const int64_t rank = upper_bound_dev<T>(range, num_part, v);
    out[i] = static_cast<T>((rank - 1) * static_cast<int64_t>(m) + static_cast<int64_t>(v % m));
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void upper_bound_kernel(const T* __restrict__ in,
                                                              const T* __restrict__ range,
                                                              int64_t num_part,
                                                              T* __restrict__ out, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) out[i] = static_cast<T>(upper_bound_dev<T>(range, num_part, in[i]));
}

__global__ __launch_bounds__(kThreads) void lookup_sorted_kernel(const int64_t* __restrict__ q,
                                                                int64_t n, HotSet hs,
                                                                int64_t* __restrict__ loc) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) loc[i] = hs.slot(q[i]);
}

// ---- bucket index over the sorted hot set ------------------------------------
// header: shift such that (largest id >> shift) < buckets; valid only for non-negative ids
__global__ void hot_index_header_kernel(const int64_t* __restrict__ sorted, int64_t num_hot,
                                        int buckets_log2, uint32_t* __restrict__ index) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  uint32_t shift = 0, valid = 0;
  if (num_hot > 0 && num_hot < (int64_t(1) << 32) && sorted[0] >= 0) {
    const uint64_t mx = static_cast<uint64_t>(sorted[num_hot - 1]);
    const int bits = mx == 0 ? 1 : 64 - __clzll(static_cast<long long>(mx));
    shift = bits > buckets_log2 ? static_cast<uint32_t>(bits - buckets_log2) : 0u;
    valid = 1;
  }
  index[0] = shift;
  index[1] = static_cast<uint32_t>(buckets_log2);
  index[2] = valid;
  index[3] = 0;
}

__global__ __launch_bounds__(kThreads) void hot_index_table_kernel(const int64_t* __restrict__ sorted,
                                                                  int64_t num_hot,
                                                                  uint32_t* __restrict__ index) {
  const int64_t b = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t buckets = int64_t(1) << index[1];
  if (b > buckets) return;
  if (index[2] == 0u) {
    index[kHotIndexHeader + b] = 0;
    return;
  }
  // first position whose id >= (b << shift): ids are >= 0, so this is upper_bound(key - 1)
  // (the last entry closes the last bucket: every id is below buckets << shift)
  const int64_t key = static_cast<int64_t>(static_cast<uint64_t>(b) << index[0]);
  int64_t pos;
  if (b == buckets) pos = num_hot;
  else if (key <= 0) pos = 0;
  else pos = upper_bound_dev<int64_t>(sorted, num_hot, key - 1);
  index[kHotIndexHeader + b] = static_cast<uint32_t>(pos);
}

int hot_index_buckets_log2(int64_t num_hot) {
  int l = ilog2_ceil(static_cast<uint64_t>(num_hot > 1 ? num_hot : 1));
  return l > 30 ? 30 : l;
}

// ---- split: three masks from the int8 class table --------------------------
template <typename I>
__global__ __launch_bounds__(kThreads) void split_masks_kernel(const I* __restrict__ ids,
                                                              const int8_t* __restrict__ table,
                                                              int64_t n, uint8_t* __restrict__ m0,
                                                              uint8_t* __restrict__ m1,
                                                              uint8_t* __restrict__ m2) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    const int8_t v = table[static_cast<int64_t>(ids[i])];
    m0[i] = v == 0;
    m1[i] = v == 1;
    m2[i] = v == 2;
  }
}

// ---- stable compaction ------------------------------------------------------
// A tile is kTile consecutive elements; thread t of the block owns elements [8t, 8t+8) of the
// tile so that the order of positions inside every class list is ascending.
constexpr int kItems = 8;
constexpr int kTile = kThreads * kItems;
constexpr uint32_t kNone = 3;  // class code of an element that belongs to no list

__device__ __forceinline__ uint64_t pack_counts(uint64_t cls8, int valid) {
  // per-class counts of the (up to 8) class bytes, 21 bits per class
  uint64_t packed = 0;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const uint32_t c = static_cast<uint32_t>(cls8 >> (8 * k)) & 0xffu;
    if (k < valid && c < kNone) packed += uint64_t(1) << (21 * c);
  }
  return packed;
}

// classify + per-block counts.  Classifier returns the class code (0..2, or kNone) of element i.
template <typename Classifier>
__global__ __launch_bounds__(kThreads) void classify_count_kernel(Classifier cf, int64_t n,
                                                                 uint8_t* __restrict__ cls,
                                                                 uint32_t* __restrict__ blk_cnt,
                                                                 int64_t nblocks) {
  __shared__ uint64_t smem[kThreads / kWave + 1];
  const int64_t i0 = static_cast<int64_t>(blockIdx.x) * kTile + threadIdx.x * kItems;
  uint64_t cls8 = 0;
  int valid = 0;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    uint32_t c = kNone;
    if (i0 + k < n) {
      c = cf(i0 + k);
      valid = k + 1;
    }
    cls8 |= static_cast<uint64_t>(c) << (8 * k);
  }
  // cls workspace is padded to a whole number of tiles: the full 8-byte store is always in range
  *reinterpret_cast<uint64_t*>(cls + i0) = cls8;
  uint64_t total;
  (void)block_exclusive_sum<uint64_t, kThreads>(pack_counts(cls8, valid), smem, &total);
  if (threadIdx.x == 0) {
#pragma unroll
    for (int c = 0; c < 3; ++c)
      blk_cnt[c * nblocks + blockIdx.x] = static_cast<uint32_t>(total >> (21 * c)) & 0x1fffffu;
  }
}

// single block: per-class exclusive prefix over the blocks, and the class totals
__global__ __launch_bounds__(kThreads) void block_prefix_kernel(const uint32_t* __restrict__ blk_cnt,
                                                               int64_t* __restrict__ blk_off,
                                                               int64_t nblocks, int num_classes,
                                                               int64_t* __restrict__ totals) {
  __shared__ int64_t smem[kThreads / kWave + 1];
  for (int c = 0; c < num_classes; ++c) {
    int64_t carry = 0;
    for (int64_t base = 0; base < nblocks; base += kThreads) {
      const int64_t b = base + threadIdx.x;
      const int64_t v = b < nblocks ? static_cast<int64_t>(blk_cnt[c * nblocks + b]) : 0;
      int64_t total;
      const int64_t ex = block_exclusive_sum<int64_t, kThreads>(v, smem, &total);
      if (b < nblocks) blk_off[c * nblocks + b] = carry + ex;
      carry += total;
    }
    if (threadIdx.x == 0) totals[c] = carry;
  }
}

struct CompactOut {
  uint8_t* mask[3];
  int64_t* pos[3];
};

__global__ __launch_bounds__(kThreads) void compact_kernel(const uint8_t* __restrict__ cls,
                                                          const int64_t* __restrict__ blk_off,
                                                          int64_t nblocks, int64_t n,
                                                          int num_classes, CompactOut out) {
  __shared__ uint64_t smem[kThreads / kWave + 1];
  const int64_t i0 = static_cast<int64_t>(blockIdx.x) * kTile + threadIdx.x * kItems;
  const uint64_t cls8 = *reinterpret_cast<const uint64_t*>(cls + i0);
  const int64_t left = n - i0;
  const int valid = left >= kItems ? kItems : (left > 0 ? static_cast<int>(left) : 0);
  uint64_t total;
  const uint64_t ex = block_exclusive_sum<uint64_t, kThreads>(pack_counts(cls8, valid), smem, &total);

  int64_t run[3];
#pragma unroll
  for (int c = 0; c < 3; ++c)
    run[c] = c < num_classes
                 ? blk_off[c * nblocks + blockIdx.x] + static_cast<int64_t>((ex >> (21 * c)) & 0x1fffffu)
                 : 0;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    if (k < valid) {
      const uint32_t c = static_cast<uint32_t>(cls8 >> (8 * k)) & 0xffu;
#pragma unroll
      for (int cc = 0; cc < 3; ++cc) {
        if (cc < num_classes && c == cc) {
          if (out.pos[cc]) out.pos[cc][run[cc]] = i0 + k;
          ++run[cc];
        }
      }
    }
  }
#pragma unroll
  for (int cc = 0; cc < 3; ++cc) {
    uint8_t* m = out.mask[cc];
    if (m == nullptr) continue;
    uint64_t bits = 0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
      const uint32_t c = static_cast<uint32_t>(cls8 >> (8 * k)) & 0xffu;
      bits |= static_cast<uint64_t>(c == cc ? 1u : 0u) << (8 * k);
    }
    if (valid == kItems && (reinterpret_cast<uintptr_t>(m + i0) & 7u) == 0) {
      *reinterpret_cast<uint64_t*>(m + i0) = bits;
    } else {
      for (int k = 0; k < valid; ++k) m[i0 + k] = static_cast<uint8_t>(bits >> (8 * k)) & 1u;
    }
  }
}

struct ClassifyLoc {
  const int64_t* loc;
  __device__ __forceinline__ uint32_t operator()(int64_t i) const { return loc[i] >= 0 ? 0u : 1u; }
};
template <typename I>
struct ClassifyTable {
  const I* ids;
  const int8_t* table;
  __device__ __forceinline__ uint32_t operator()(int64_t i) const {
    const int8_t v = table[static_cast<int64_t>(ids[i])];
    return (v >= 0 && v <= 2) ? static_cast<uint32_t>(v) : kNone;
  }
};

struct ClassifyLive {
  const int64_t* keys;
  __device__ __forceinline__ uint32_t operator()(int64_t i) const {
    return keys[i] != int64_t(-1) ? 0u : kNone;
  }
};

struct CompactWs {
  uint8_t* cls;
  uint32_t* blk_cnt;
  int64_t* blk_off;
  size_t bytes;
};
CompactWs carve_compact(void* ws, int64_t n) {
  const int64_t nblocks = ceil_div(n > 0 ? n : 1, kTile);
  Carver c(ws);
  CompactWs w;
  w.cls = c.take<uint8_t>(nblocks * kTile);
  w.blk_cnt = c.take<uint32_t>(3 * nblocks);
  w.blk_off = c.take<int64_t>(3 * nblocks);
  w.bytes = c.total();
  return w;
}

template <typename Classifier>
int run_compact(const Classifier& cf, int64_t n, int num_classes, const CompactOut& out,
                int64_t* counts, void* workspace, size_t workspace_bytes, hipStream_t st) {
  HADES_REQUIRE(n >= 0 && n < (int64_t(1) << 40), "n out of range: %lld", (long long)n);
  HADES_REQUIRE(counts != nullptr, "counts must not be null");
  const CompactWs w = carve_compact(workspace, n);
  if (workspace == nullptr || workspace_bytes < w.bytes)
    return set_error(HADES_ERR_WORKSPACE, "workspace too small: need %zu bytes, got %zu", w.bytes,
                     workspace_bytes);
  HADES_REQUIRE((align_of_ptr(workspace) & 255) == 0, "workspace must be 256-byte aligned");
  const int64_t nblocks = ceil_div(n > 0 ? n : 1, kTile);
  HADES_REQUIRE(nblocks < (int64_t(1) << 31), "n too large");
  HADES_LAUNCH((classify_count_kernel<Classifier>), dim3((unsigned)nblocks), dim3(kThreads), 0,
                     st, cf, n, w.cls, w.blk_cnt, nblocks);
  HADES_LAUNCH_CHECK();
  HADES_LAUNCH(block_prefix_kernel, dim3(1), dim3(kThreads), 0, st, w.blk_cnt, w.blk_off,
                     nblocks, num_classes, counts);
  HADES_LAUNCH_CHECK();
  HADES_LAUNCH(compact_kernel, dim3((unsigned)nblocks), dim3(kThreads), 0, st, w.cls,
                     w.blk_off, nblocks, n, num_classes, out);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

template <typename Fn>
int dispatch_itype(int itype, Fn&& fn) {
  if (itype == HADES_I64) return fn(int64_t{});
  if (itype == HADES_I32) return fn(int32_t{});
  return set_error(HADES_ERR_ARG, "ID can only be int32 or int64 (code %d)", itype);
}

template <typename Fn>
int dispatch_split_id(int id_type, Fn&& fn) {
  switch (id_type) {
    case HADES_I64: return fn(int64_t{});
    case HADES_I32: return fn(int32_t{});
    case HADES_I16: return fn(int16_t{});
    case HADES_I8: return fn(int8_t{});
    case HADES_U8: return fn(uint8_t{});
    default: return set_error(HADES_ERR_ARG, "split: unsupported id type code %d", id_type);
  }
}

inline unsigned grid_1d(int64_t n) { return static_cast<unsigned>(ceil_div(n, kThreads)); }

}  // namespace

size_t compact_live_workspace_bytes(int64_t n) { return carve_compact(nullptr, n < 0 ? 0 : n).bytes; }

int compact_live_keys(const int64_t* keys, int64_t n, int64_t* pos_out, int64_t* count_out,
                      void* workspace, size_t workspace_bytes, hipStream_t st) {
  CompactOut out{{nullptr, nullptr, nullptr}, {pos_out, nullptr, nullptr}};
  return run_compact(ClassifyLive{keys}, n, 1, out, count_out, workspace, workspace_bytes, st);
}

}  // namespace hades

using namespace hades;

extern "C" {

int hades_reminder(const void* in, int64_t local_num_gpus, void* out, int64_t n, int itype,
                   void* stream) {
  HADES_REQUIRE(n >= 0, "n must be >= 0");
  HADES_REQUIRE(local_num_gpus != 0, "local_num_gpus must not be 0");
  if (n == 0) return (itype == HADES_I32 || itype == HADES_I64) ? HADES_OK
                     : set_error(HADES_ERR_ARG, "ID can only be int32 or int64 (code %d)", itype);
  HADES_REQUIRE(in && out, "null pointer argument");
  HADES_REQUIRE(ceil_div(n, kThreads) < (int64_t(1) << 31), "n too large");
  return dispatch_itype(itype, [&](auto tag) {
    using T = decltype(tag);
    HADES_LAUNCH((reminder_kernel<T>), dim3(grid_1d(n)), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), static_cast<const T*>(in),
                       static_cast<T>(local_num_gpus), static_cast<T*>(out), n);
    HADES_LAUNCH_CHECK();
    return HADES_OK;
  });
}

int hades_binary_search(const void* in, const void* range_partition, int64_t num_part,
                        int64_t local_num_gpus, void* out, int64_t n, int itype, void* stream) {
  HADES_REQUIRE(n >= 0 && num_part >= 0, "n and num_part must be >= 0");
  HADES_REQUIRE(local_num_gpus != 0, "local_num_gpus must not be 0");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(in && out && (num_part == 0 || range_partition), "null pointer argument");
  HADES_REQUIRE(ceil_div(n, kThreads) < (int64_t(1) << 31), "n too large");
  return dispatch_itype(itype, [&](auto tag) {
    using T = decltype(tag);
    HADES_LAUNCH((owner_rank_kernel<T>), dim3(grid_1d(n)), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), static_cast<const T*>(in),
                       static_cast<const T*>(range_partition), num_part,
                       static_cast<T>(local_num_gpus), static_cast<T*>(out), n);
    HADES_LAUNCH_CHECK();
    return HADES_OK;
  });
}

int hades_binary_search2(const void* in, const void* range, int64_t num_part, void* out,
                         int64_t n, int itype, void* stream) {
  HADES_REQUIRE(n >= 0 && num_part >= 0, "n and num_part must be >= 0");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(in && out && (num_part == 0 || range), "null pointer argument");
  HADES_REQUIRE(ceil_div(n, kThreads) < (int64_t(1) << 31), "n too large");
  return dispatch_itype(itype, [&](auto tag) {
    using T = decltype(tag);
    HADES_LAUNCH((upper_bound_kernel<T>), dim3(grid_1d(n)), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), static_cast<const T*>(in),
                       static_cast<const T*>(range), num_part, static_cast<T*>(out), n);
    HADES_LAUNCH_CHECK();
    return HADES_OK;
  });
}

int hades_lookup_sorted(const int64_t* q, int64_t n, const int64_t* sorted_hot, int64_t num_hot,
                        const void* hot_index, int64_t* loc, void* stream) {
  HADES_REQUIRE(n >= 0 && num_hot >= 0, "n and num_hot must be >= 0");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(q && loc && (num_hot == 0 || sorted_hot), "null pointer argument");
  HADES_REQUIRE(ceil_div(n, kThreads) < (int64_t(1) << 31), "n too large");
  HADES_LAUNCH(lookup_sorted_kernel, dim3(grid_1d(n)), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), q, n,
                     HotSet{sorted_hot, num_hot, static_cast<const uint32_t*>(hot_index)}, loc);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

size_t hades_hot_index_bytes(int64_t num_hot) {
  if (num_hot < 0) return 0;
  const int64_t buckets = int64_t(1) << hot_index_buckets_log2(num_hot);
  return static_cast<size_t>(kHotIndexHeader + buckets + 1) * sizeof(uint32_t);
}

int hades_hot_index_build(const int64_t* sorted_hot, int64_t num_hot, void* hot_index,
                          size_t hot_index_bytes, void* stream) {
  HADES_REQUIRE(num_hot >= 0 && (num_hot == 0 || sorted_hot), "bad hot set");
  HADES_REQUIRE(hot_index != nullptr && (align_of_ptr(hot_index) % 16) == 0,
                "hot_index must be a 16-byte aligned device buffer");
  if (hot_index_bytes < hades_hot_index_bytes(num_hot))
    return set_error(HADES_ERR_WORKSPACE, "hot index buffer too small: need %zu bytes, got %zu",
                     hades_hot_index_bytes(num_hot), hot_index_bytes);
  const int l2 = hot_index_buckets_log2(num_hot);
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t* index = static_cast<uint32_t*>(hot_index);
  HADES_LAUNCH(hot_index_header_kernel, dim3(1), dim3(64), 0, st, sorted_hot, num_hot, l2,
                     index);
  HADES_LAUNCH_CHECK();
  const int64_t entries = (int64_t(1) << l2) + 1;
  HADES_LAUNCH(hot_index_table_kernel, dim3(grid_1d(entries)), dim3(kThreads), 0, st,
                     sorted_hot, num_hot, index);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

int hades_split(const void* ids, int id_type, const int8_t* class_table, int64_t n,
                uint8_t* local_mask, uint8_t* remote_hot_mask, uint8_t* remote_cold_mask,
                void* stream) {
  HADES_REQUIRE(n >= 0, "n must be >= 0");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(ids && class_table && local_mask && remote_hot_mask && remote_cold_mask,
                "null pointer argument");
  HADES_REQUIRE(ceil_div(n, kThreads) < (int64_t(1) << 31), "n too large");
  return dispatch_split_id(id_type, [&](auto tag) {
    using T = decltype(tag);
    HADES_LAUNCH((split_masks_kernel<T>), dim3(grid_1d(n)), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), static_cast<const T*>(ids), class_table, n,
                       local_mask, remote_hot_mask, remote_cold_mask);
    HADES_LAUNCH_CHECK();
    return HADES_OK;
  });
}

size_t hades_split_compact_workspace_bytes(int64_t n) {
  return carve_compact(nullptr, n < 0 ? 0 : n).bytes;
}

int hades_split_compact(const int64_t* loc, int64_t n, uint8_t* hot_mask, int64_t* hot_pos,
                        int64_t* cold_pos, int64_t* counts, void* workspace,
                        size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(n >= 0, "n must be >= 0");
  HADES_REQUIRE(n == 0 || loc, "null pointer argument");
  CompactOut out{{hot_mask, nullptr, nullptr}, {hot_pos, cold_pos, nullptr}};
  return run_compact(ClassifyLoc{loc}, n, 2, out, counts, workspace, workspace_bytes,
                     static_cast<hipStream_t>(stream));
}

int hades_split3_compact(const void* ids, int id_type, const int8_t* class_table, int64_t n,
                         uint8_t* mask0, uint8_t* mask1, uint8_t* mask2, int64_t* pos0,
                         int64_t* pos1, int64_t* pos2, int64_t* counts, void* workspace,
                         size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(n >= 0, "n must be >= 0");
  HADES_REQUIRE(n == 0 || (ids && class_table), "null pointer argument");
  CompactOut out{{mask0, mask1, mask2}, {pos0, pos1, pos2}};
  return dispatch_split_id(id_type, [&](auto tag) {
    using T = decltype(tag);
    return run_compact(ClassifyTable<T>{static_cast<const T*>(ids), class_table}, n, 3, out, counts,
                       workspace, workspace_bytes, static_cast<hipStream_t>(stream));
  });
}

}  // extern "C"
