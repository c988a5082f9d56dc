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
// header: shift such that (largest id >> shift) < buckets; usable only for non-negative ids.
// form 2 (position + count + low bits of the first id in one entry) when the low bits fit 24 bits.
__global__ void hot_index_header_kernel(const int64_t* __restrict__ sorted, int64_t num_hot,
                                        int buckets_log2, uint32_t* __restrict__ index) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  uint32_t shift = 0, form = 0;
  if (num_hot > 0 && num_hot < (int64_t(1) << 32) && sorted[0] >= 0) {
    const uint64_t mx = static_cast<uint64_t>(sorted[num_hot - 1]);
    const int bits = mx == 0 ? 1 : 64 - __clzll(static_cast<long long>(mx));
    shift = bits > buckets_log2 ? static_cast<uint32_t>(bits - buckets_log2) : 0u;
    form = shift <= 24u ? 2u : 1u;
  }
  index[0] = shift;
  index[1] = static_cast<uint32_t>(buckets_log2);
  index[2] = form;
  index[3] = 0;
}

// first position whose id >= (b << shift), for b in [0, buckets]: ids are >= 0, so this is
// upper_bound(key - 1) (the last entry closes the last bucket: every id is below buckets << shift)
__device__ __forceinline__ int64_t bucket_start(const int64_t* __restrict__ sorted, int64_t num_hot,
                                                int64_t b, int64_t buckets, uint32_t shift) {
  if (b >= buckets) return num_hot;
  const int64_t key = static_cast<int64_t>(static_cast<uint64_t>(b) << shift);
  if (key <= 0) return 0;
  return upper_bound_dev<int64_t>(sorted, num_hot, key - 1);
}

__global__ __launch_bounds__(kThreads) void hot_index_table_kernel(const int64_t* __restrict__ sorted,
                                                                  int64_t num_hot,
                                                                  uint32_t* __restrict__ index) {
  const int64_t b = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t buckets = int64_t(1) << index[1];
  if (b > buckets) return;
  const uint32_t form = index[2], shift = index[0];
  if (form == 0u) {
    index[kHotIndexHeader + b] = 0;
    return;
  }
  const int64_t pos = bucket_start(sorted, num_hot, b, buckets, shift);
  if (form == 1u) {
    index[kHotIndexHeader + b] = static_cast<uint32_t>(pos);
    return;
  }
  const int64_t next = bucket_start(sorted, num_hot, b + 1, buckets, shift);
  const int64_t cnt = next - pos;
  const uint32_t low = cnt > 0 ? static_cast<uint32_t>(sorted[pos]) & ((1u << shift) - 1u) : 0u;
  index[kHotIndexHeader + 2 * b] = static_cast<uint32_t>(pos);
  index[kHotIndexHeader + 2 * b + 1] = (static_cast<uint32_t>(cnt < 255 ? cnt : 255) << 24) | low;
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
// A tile is kTile consecutive elements, taken in kRounds rounds of one element per thread
// (element tile0 + r*kThreads + t in round r: coalesced).  Ranks inside a wave come from a ballot
// of the class predicate and a count of the set bits below the lane (mbcnt); the (round, wave)
// counts of a tile are prefixed in LDS, and the tiles before it are summed from the per-tile
// counts of the first kernel.  Positions inside every class list are ascending.
// Rounds per thread: 8 for classifiers that only read their element; 2 for the fused lookup, whose
// dependent table and id reads per element would otherwise run one after the other in a thread
// while three quarters of the CU's wave slots stay empty (1 M lookups: 43 us with 8 rounds).
constexpr int kRoundsDefault = 8;
constexpr int kRoundsLookup = 2;
constexpr int kWaves = kThreads / kWave;
constexpr uint32_t kNone = 3;           // class code of an element that belongs to no list
constexpr int64_t kSumTilesInKernel = 4096;  // above this many tiles a scan kernel prefixes them

// classify + per-tile counts.  Classifier returns the class code (0..2, or kNone) of element i;
// it is called exactly once per element and may write per-element results of its own.
template <typename Classifier, int kRounds>
__global__ __launch_bounds__(kThreads) void classify_count_kernel(Classifier cf, int64_t n,
                                                                 uint8_t* __restrict__ cls,
                                                                 uint32_t* __restrict__ blk_cnt,
                                                                 int64_t nblocks) {
  __shared__ uint32_t s_cnt[kWaves][3];
  constexpr int kTile = kThreads * kRounds;
  const int64_t tile0 = static_cast<int64_t>(blockIdx.x) * kTile;
  uint32_t cnt[3] = {0, 0, 0};   // wave-uniform
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    const int64_t i = tile0 + r * kThreads + threadIdx.x;
    uint32_t c = kNone;
    if (i < n) {
      c = cf(i);
      cls[i] = static_cast<uint8_t>(c);
    }
#pragma unroll
    for (int k = 0; k < 3; ++k) cnt[k] += __popcll(__ballot(c == static_cast<uint32_t>(k)));
  }
  if (lane_id() == 0) {
#pragma unroll
    for (int k = 0; k < 3; ++k) s_cnt[threadIdx.x / kWave][k] = cnt[k];
  }
  __syncthreads();
  if (threadIdx.x < 3) {
    uint32_t sum = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) sum += s_cnt[w][threadIdx.x];
    blk_cnt[threadIdx.x * nblocks + blockIdx.x] = sum;
  }
}

// single block: per-class exclusive prefix over the tiles (only for inputs of more than
// kSumTilesInKernel tiles; below that every compaction block sums the tiles before it itself)
__global__ __launch_bounds__(kThreads) void block_prefix_kernel(const uint32_t* __restrict__ blk_cnt,
                                                               int64_t* __restrict__ blk_off,
                                                               int64_t nblocks, int num_classes) {
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
  }
}

struct CompactOut {
  uint8_t* mask[3];
  int64_t* pos[3];
};

template <int kRounds>
__global__ __launch_bounds__(kThreads) void compact_kernel(const uint8_t* __restrict__ cls,
                                                          const uint32_t* __restrict__ blk_cnt,
                                                          const int64_t* __restrict__ blk_off,
                                                          int64_t nblocks, int64_t n,
                                                          int num_classes, CompactOut out,
                                                          int64_t* __restrict__ totals) {
  __shared__ int64_t s_wsum[kWaves][3];
  __shared__ int64_t s_base[3];
  __shared__ uint32_t s_cnt[kRounds][kWaves][3];   // counts, then exclusive offsets inside the tile
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  constexpr int kTile = kThreads * kRounds;
  const int64_t tile0 = static_cast<int64_t>(blockIdx.x) * kTile;

  // the tile's class codes first, so that their latency overlaps the sum over earlier tiles
  uint32_t c[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    const int64_t i = tile0 + r * kThreads + threadIdx.x;
    c[r] = i < n ? cls[i] : kNone;
  }

  // elements of each class in the tiles before this one
  if (blk_off != nullptr) {
    if (threadIdx.x < 3)
      s_base[threadIdx.x] = static_cast<int>(threadIdx.x) < num_classes
                                ? blk_off[threadIdx.x * nblocks + blockIdx.x] : 0;
  } else {
    int64_t part[3] = {0, 0, 0};
    for (int64_t b = threadIdx.x; b < static_cast<int64_t>(blockIdx.x); b += kThreads) {
#pragma unroll
      for (int k = 0; k < 3; ++k)
        if (k < num_classes) part[k] += blk_cnt[k * nblocks + b];
    }
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const int64_t w = wave_inclusive_sum<int64_t>(part[k]);
      if (lane == kWave - 1) s_wsum[wave][k] = w;
    }
    __syncthreads();
    if (threadIdx.x < 3) {
      int64_t sum = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) sum += s_wsum[w][threadIdx.x];
      s_base[threadIdx.x] = sum;
    }
  }

#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const uint32_t cnt = __popcll(__ballot(c[r] == static_cast<uint32_t>(k)));
      if (lane == 0) s_cnt[r][wave][k] = cnt;
    }
  }
  __syncthreads();
  if (threadIdx.x < 3) {
    uint32_t run = 0;
    for (int r = 0; r < kRounds; ++r) {
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        const uint32_t t = s_cnt[r][w][threadIdx.x];
        s_cnt[r][w][threadIdx.x] = run;
        run += t;
      }
    }
    if (blockIdx.x == gridDim.x - 1 && static_cast<int>(threadIdx.x) < num_classes)
      totals[threadIdx.x] = s_base[threadIdx.x] + run;
  }
  __syncthreads();

#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    const int64_t i = tile0 + r * kThreads + threadIdx.x;
    const uint32_t cc = c[r];
    uint64_t mine = 0;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const uint64_t bal = __ballot(cc == static_cast<uint32_t>(k));
      if (cc == static_cast<uint32_t>(k)) mine = bal;
    }
    if (i < n) {
      if (static_cast<int>(cc) < num_classes && out.pos[cc] != nullptr)
        out.pos[cc][s_base[cc] + s_cnt[r][wave][cc] + ballot_rank(mine)] = i;
#pragma unroll
      for (int k = 0; k < 3; ++k)
        if (out.mask[k] != nullptr) out.mask[k][i] = cc == static_cast<uint32_t>(k) ? 1 : 0;
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

// lookup fused into the classification: the slot of every query is written on the way
struct ClassifyLookup {
  const int64_t* q;
  HotSet hs;
  int64_t* loc;
  const int64_t* num_live;   // optional: only the first num_live[0] queries count
  int64_t* sort_keys;        // optional: class-ordered sort key of every query (see the header)
  int key_bits;
  __device__ __forceinline__ uint32_t operator()(int64_t i) const {
    if (num_live != nullptr && i >= num_live[0]) return kNone;
    const int64_t id = q[i];
    const int64_t l = hs.slot(id);
    loc[i] = l;
    if (sort_keys != nullptr) sort_keys[i] = l >= 0 ? ((int64_t(1) << key_bits) | l) : id;
    return l >= 0 ? 0u : 1u;
  }
};

struct ClassifyLive {
  const int64_t* keys;
  int64_t stride;
  __device__ __forceinline__ uint32_t operator()(int64_t i) const {
    return keys[i * stride] != int64_t(-1) ? 0u : kNone;
  }
};

struct CompactWs {
  uint8_t* cls;
  uint32_t* blk_cnt;
  int64_t* blk_off;
  size_t bytes;
};
CompactWs carve_compact(void* ws, int64_t n) {
  const int64_t nblocks = ceil_div(n > 0 ? n : 1, kThreads * kRoundsLookup);   // the most tiles any form uses
  Carver c(ws);
  CompactWs w;
  w.cls = c.take<uint8_t>(n > 0 ? n : 1);
  w.blk_cnt = c.take<uint32_t>(3 * nblocks);
  w.blk_off = c.take<int64_t>(nblocks > kSumTilesInKernel ? 3 * nblocks : 1);
  w.bytes = c.total();
  return w;
}

template <typename Classifier, int kRounds = kRoundsDefault>
int run_compact(const Classifier& cf, int64_t n, int num_classes, const CompactOut& out,
                int64_t* counts, void* workspace, size_t workspace_bytes, hipStream_t st) {
  constexpr int kTile = kThreads * kRounds;
  HADES_REQUIRE(n >= 0 && n < (int64_t(1) << 40), "n out of range: %lld", (long long)n);
  HADES_REQUIRE(counts != nullptr, "counts must not be null");
  const CompactWs w = carve_compact(workspace, n);
  if (workspace == nullptr || workspace_bytes < w.bytes)
    return set_error(HADES_ERR_WORKSPACE, "workspace too small: need %zu bytes, got %zu", w.bytes,
                     workspace_bytes);
  HADES_REQUIRE((align_of_ptr(workspace) & 255) == 0, "workspace must be 256-byte aligned");
  const int64_t nblocks = ceil_div(n > 0 ? n : 1, kTile);
  HADES_REQUIRE(nblocks < (int64_t(1) << 31), "n too large");
  HADES_LAUNCH((classify_count_kernel<Classifier, kRounds>), dim3((unsigned)nblocks), dim3(kThreads),
                     0, st, cf, n, w.cls, w.blk_cnt, nblocks);
  const int64_t* blk_off = nullptr;
  if (nblocks > kSumTilesInKernel) {
    HADES_LAUNCH(block_prefix_kernel, dim3(1), dim3(kThreads), 0, st, w.blk_cnt, w.blk_off,
                       nblocks, num_classes);
    blk_off = w.blk_off;
  }
  HADES_LAUNCH((compact_kernel<kRounds>), dim3((unsigned)nblocks), dim3(kThreads), 0, st, w.cls,
                     w.blk_cnt, blk_off, nblocks, n, num_classes, out, counts);
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
                      void* workspace, size_t workspace_bytes, hipStream_t st, int64_t key_stride) {
  CompactOut out{{nullptr, nullptr, nullptr}, {pos_out, nullptr, nullptr}};
  return run_compact(ClassifyLive{keys, key_stride}, n, 1, out, count_out, workspace,
                     workspace_bytes, st);
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
  return static_cast<size_t>(kHotIndexHeader + 2 * (buckets + 1)) * sizeof(uint32_t);   // form 2
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

int hades_lookup_split(const int64_t* q, const int64_t* num_live, int64_t n,
                       const int64_t* sorted_hot, int64_t num_hot,
                       const void* hot_index, int64_t* loc, uint8_t* hot_mask, int64_t* hot_pos,
                       int64_t* cold_pos, int64_t* counts, int64_t* sort_keys, int key_bits,
                       void* workspace, size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(n >= 0 && num_hot >= 0, "n and num_hot must be >= 0");
  HADES_REQUIRE(sort_keys == nullptr || (key_bits >= 1 && key_bits <= 61 &&
                                         num_hot <= (int64_t(1) << key_bits)),
                "key_bits must be in [1, 61] and leave room for every hot slot");
  // entries past num_live[0] get neither a slot nor a key, and the classed combine sorts all n keys
  HADES_REQUIRE(num_live == nullptr || sort_keys == nullptr,
                "num_live and sort_keys cannot be combined: sort keys are written for whole batches only");
  HADES_REQUIRE(n == 0 || (q && loc), "null pointer argument");
  HADES_REQUIRE(num_hot == 0 || sorted_hot, "sorted_hot is null but num_hot > 0");
  CompactOut out{{hot_mask, nullptr, nullptr}, {hot_pos, cold_pos, nullptr}};
  ClassifyLookup cf{q, HotSet{sorted_hot, num_hot, static_cast<const uint32_t*>(hot_index)}, loc,
                    num_live, sort_keys, key_bits};
  return run_compact<ClassifyLookup, kRoundsLookup>(cf, n, 2, out, counts, workspace, workspace_bytes,
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
