// Row gather / scatter kernels: every cudaFetch* / cudaSet* / cudaCombine operator of the
// reference (src/cuda/uva_fetch.cu, src/cuda/uva_set.cu) plus the sorted-hot-set forms.
//
// One kernel template serves all of them.  A block owns ROWS consecutive batch rows:
//   phase 1: one thread per row resolves (source row pointer, destination row pointer): index
//            loads, the index_map probe or the binary search of the hot set, hot/cold select.
//            This is done once per row, not once per lane.
//   phase 2: the block copies its rows as a flat list of 16-byte chunks (8 or 4 bytes when
//            the row size or a base pointer is not 16-byte aligned), UNROLL chunks in flight
//            per thread, adjacent lanes on adjacent chunks.
// Payloads are moved verbatim, so every operator is bit-exact for any element type.
#include "common.h"

namespace hades {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kRowsPerBlock = 64;   // measured: 64 rows 34.7 us, 128 rows 37.1 us, 32 rows 35.6 us
                                    // for 200 K rows of 512 bytes
constexpr int kThreads = 256;
constexpr int kUnroll = 8;

template <typename I>
__device__ __forceinline__ int64_t ld_idx(const void* p, int64_t i) {
  return static_cast<int64_t>(static_cast<const I*>(p)[i]);
}

// ---- address resolvers ------------------------------------------------------
// dst[dst_index[i]] = src[src_index[i]]
template <typename I>
struct AddrFetch {
  const char* src; const void* sidx; char* dst; const void* didx; int64_t row_bytes;
  __device__ __forceinline__ void operator()(int64_t i, const char*& s, char*& d) const {
    s = src + ld_idx<I>(sidx, i) * row_bytes;
    d = dst + ld_idx<I>(didx, i) * row_bytes;
  }
};
// dst[i] = src[src_index[i]]
template <typename I>
struct AddrFetch2 {
  const char* src; const void* sidx; char* dst; int64_t row_bytes;
  __device__ __forceinline__ void operator()(int64_t i, const char*& s, char*& d) const {
    s = src + ld_idx<I>(sidx, i) * row_bytes;
    d = dst + i * row_bytes;
  }
};
// g = map[idx[i]]; dst[i] = g != -1 ? gpu[g] : cpu[idx[i]]
template <typename I>
struct AddrFetchMap {
  const char* cpu; const char* gpu; const void* idx; const void* map; char* dst; int64_t row_bytes;
  __device__ __forceinline__ void operator()(int64_t i, const char*& s, char*& d) const {
    int64_t id = ld_idx<I>(idx, i);
    int64_t g = ld_idx<I>(map, id);
    s = (g != -1) ? gpu + g * row_bytes : cpu + id * row_bytes;
    d = dst + i * row_bytes;
  }
};
// dst[dst_index[i]] = src[i]
template <typename I>
struct AddrSet {
  const char* src; char* dst; const void* didx; int64_t row_bytes;
  __device__ __forceinline__ void operator()(int64_t i, const char*& s, char*& d) const {
    s = src + i * row_bytes;
    d = dst + ld_idx<I>(didx, i) * row_bytes;
  }
};
// g = map[idx[i]]; (g != -1 ? gpu[g] : cpu[idx[i]]) = src[i]
template <typename I>
struct AddrSetMap {
  const char* src; char* cpu; char* gpu; const void* idx; const void* map; int64_t row_bytes;
  __device__ __forceinline__ void operator()(int64_t i, const char*& s, char*& d) const {
    int64_t id = ld_idx<I>(idx, i);
    int64_t g = ld_idx<I>(map, id);
    s = src + i * row_bytes;
    d = (g != -1) ? gpu + g * row_bytes : cpu + id * row_bytes;
  }
};
// loc = lookup(q[i]) in the sorted hot set; dst[i] = loc >= 0 ? hot[loc] : cold[q[i]]
struct AddrFetchSorted {
  const char* cold; const char* hot; const int64_t* q; HotSet hs;
  char* dst; int64_t* loc_out; int64_t row_bytes;
  __device__ __forceinline__ void operator()(int64_t i, const char*& s, char*& d) const {
    int64_t id = q[i];
    int64_t loc = hs.slot(id);
    if (loc_out) loc_out[i] = loc;
    s = (loc >= 0) ? hot + loc * row_bytes : cold + id * row_bytes;
    d = dst + i * row_bytes;
  }
};
// slots already known
struct AddrFetchLoc {
  const char* cold; const char* hot; const int64_t* q; const int64_t* loc; char* dst;
  int64_t row_bytes;
  __device__ __forceinline__ void operator()(int64_t i, const char*& s, char*& d) const {
    int64_t l = loc[i];
    s = (l >= 0) ? hot + l * row_bytes : cold + q[i] * row_bytes;
    d = dst + i * row_bytes;
  }
};
// (loc >= 0 ? hot[loc] : cold[q[i]]) = src[i]
struct AddrSetSorted {
  const char* src; char* cold; char* hot; const int64_t* q; HotSet hs; int64_t row_bytes;
  __device__ __forceinline__ void operator()(int64_t i, const char*& s, char*& d) const {
    int64_t id = q[i];
    int64_t loc = hs.slot(id);
    s = src + i * row_bytes;
    d = (loc >= 0) ? hot + loc * row_bytes : cold + id * row_bytes;
  }
};

// ---- the mover --------------------------------------------------------------
template <typename Vec, typename Addr>
__global__ __launch_bounds__(kThreads) void row_move_kernel(Addr addr, int64_t n,
                                                           int chunks_per_row, int shift) {
  __shared__ const char* s_src[kRowsPerBlock];
  __shared__ char* s_dst[kRowsPerBlock];
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock;
  const int64_t left = n - row0;
  const int rows_here = left < kRowsPerBlock ? static_cast<int>(left) : kRowsPerBlock;

  for (int r = threadIdx.x; r < rows_here; r += kThreads) {
    const char* s;
    char* d;
    addr(row0 + r, s, d);
    s_src[r] = s;
    s_dst[r] = d;
  }
  __syncthreads();

  const int total = rows_here * chunks_per_row;
  for (int base = threadIdx.x; base < total; base += kThreads * kUnroll) {
    Vec v[kUnroll];
    Vec* d[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int c = base + k * kThreads;
      if (c < total) {
        const int r = shift >= 0 ? (c >> shift) : (c / chunks_per_row);
        const int ch = c - r * chunks_per_row;
        v[k] = reinterpret_cast<const Vec*>(s_src[r])[ch];
        d[k] = reinterpret_cast<Vec*>(s_dst[r]) + ch;
      }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int c = base + k * kThreads;
      if (c < total) *d[k] = v[k];
    }
  }
}

// ---- the listed mover ---------------------------------------------------------
// Rows named by a position list whose length lives in device memory (the two halves of a hot/cold
// split): for j < count[0], p = list[j] is a batch position and index[p] a table row.
//   GATHER : batch[p, :] = table[index[p], :]        SCATTER: table[index[p], :] = batch[p, :]
// Blocks stride over the list in steps of kRowsPerBlock rows, so the grid need not match the count.
struct ListedArgs {
  const char* table_ro;        // GATHER source
  char* table_rw;              // SCATTER destination
  int64_t table_stride_bytes;  // bytes between consecutive table rows (>= row bytes)
  const int64_t* index;        // [positions]
  const int64_t* list;         // [max_count]
  const int64_t* count;        // [1]
  int64_t max_count;
  const char* batch_ro;        // SCATTER source
  char* batch_rw;              // GATHER destination
  int64_t row_bytes;
  // FILTER: only the positions whose table row is a member of this ascending set are moved
  const int64_t* only_in;      // [only_in_max]
  const int64_t* only_in_count;  // [1]
  int64_t only_in_max;
};

template <typename Vec, bool GATHER, bool FILTER>
__global__ __launch_bounds__(kThreads) void row_move_listed_kernel(ListedArgs a, int chunks_per_row,
                                                                  int shift) {
  static_assert(kRowsPerBlock <= kWave, "the filter compacts a block's rows inside one wave");
  __shared__ const char* s_src[kRowsPerBlock];
  __shared__ char* s_dst[kRowsPerBlock];
  __shared__ int s_kept;
  int64_t cnt = a.count[0];
  cnt = cnt < a.max_count ? cnt : a.max_count;
  int64_t set_n = 0;
  if (FILTER) {
    set_n = a.only_in_count[0];
    set_n = set_n < a.only_in_max ? set_n : a.only_in_max;
    if (set_n <= 0) return;
  }
  for (int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock; row0 < cnt;
       row0 += static_cast<int64_t>(gridDim.x) * kRowsPerBlock) {
    const int64_t left = cnt - row0;
    int rows_here = left < kRowsPerBlock ? static_cast<int>(left) : kRowsPerBlock;
    if (FILTER) {
      // wave 0: one lane per row; the member rows are packed to the front of the row list
      if (threadIdx.x < kWave) {
        const int r = threadIdx.x;
        int64_t p = 0, row = 0;
        bool member = false;
        if (r < rows_here) {
          p = a.list[row0 + r];
          row = a.index[p];
          const int64_t pos = upper_bound_dev<int64_t>(a.only_in, set_n, row);
          member = pos > 0 && a.only_in[pos - 1] == row;
        }
        const uint64_t mask = __ballot(member);
        if (member) {
          const int slot = __popcll(mask & ((uint64_t(1) << r) - 1));
          const int64_t t = row * a.table_stride_bytes;
          s_src[slot] = GATHER ? a.table_ro + t : a.batch_ro + p * a.row_bytes;
          s_dst[slot] = GATHER ? a.batch_rw + p * a.row_bytes : a.table_rw + t;
        }
        if (r == 0) s_kept = __popcll(mask);
      }
      __syncthreads();
      rows_here = s_kept;
    } else {
      for (int r = threadIdx.x; r < rows_here; r += kThreads) {
        const int64_t p = a.list[row0 + r];
        const int64_t t = a.index[p] * a.table_stride_bytes;
        if (GATHER) {
          s_src[r] = a.table_ro + t;
          s_dst[r] = a.batch_rw + p * a.row_bytes;
        } else {
          s_src[r] = a.batch_ro + p * a.row_bytes;
          s_dst[r] = a.table_rw + t;
        }
      }
      __syncthreads();
    }
    const int total = rows_here * chunks_per_row;
    for (int base = threadIdx.x; base < total; base += kThreads * kUnroll) {
      Vec v[kUnroll];
      Vec* d[kUnroll];
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        const int c = base + k * kThreads;
        if (c < total) {
          const int r = shift >= 0 ? (c >> shift) : (c / chunks_per_row);
          const int ch = c - r * chunks_per_row;
          v[k] = reinterpret_cast<const Vec*>(s_src[r])[ch];
          d[k] = reinterpret_cast<Vec*>(s_dst[r]) + ch;
        }
      }
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        const int c = base + k * kThreads;
        if (c < total) *d[k] = v[k];
      }
    }
    __syncthreads();   // the row pointers are rewritten by the next round
  }
}

constexpr int64_t kMaxListedBlocks = 16384;

template <bool GATHER, bool FILTER = false>
int launch_listed(const ListedArgs& a, int vec, hipStream_t stream) {
  const int64_t cpr64 = a.row_bytes / vec;
  HADES_REQUIRE(cpr64 * kRowsPerBlock < (int64_t(1) << 30), "row of %lld bytes is too large",
                (long long)a.row_bytes);
  const int cpr = static_cast<int>(cpr64);
  const int shift = is_pow2(cpr) ? ilog2_ceil(cpr) : -1;
  int64_t blocks = ceil_div(a.max_count, kRowsPerBlock);
  if (blocks > kMaxListedBlocks) blocks = kMaxListedBlocks;
  // rows that cross the host link: a narrow grid that strides over the list
  const void* table = GATHER ? static_cast<const void*>(a.table_ro) : a.table_rw;
  // (a filtered walk is mostly set look-ups in HBM and moves few rows: it keeps the wide grid)
  if (!FILTER && is_host_memory(table) && blocks > host_link_blocks(kLinkCopy))
    blocks = host_link_blocks(kLinkCopy);
  dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
  if (vec == 16) {
    HADES_LAUNCH((row_move_listed_kernel<u32x4, GATHER, FILTER>), grid, block, 0, stream, a, cpr,
                 shift);
  } else if (vec == 8) {
    HADES_LAUNCH((row_move_listed_kernel<u32x2, GATHER, FILTER>), grid, block, 0, stream, a, cpr,
                 shift);
  } else {
    HADES_LAUNCH((row_move_listed_kernel<uint32_t, GATHER, FILTER>), grid, block, 0, stream, a, cpr,
                 shift);
  }
  return HADES_OK;
}

int pick_vec(int64_t row_bytes, std::initializer_list<const void*> bases) {
  int v = 16;
  while (v > 4) {
    bool ok = (row_bytes % v) == 0;
    for (const void* p : bases) ok = ok && (align_of_ptr(p) % v) == 0;
    if (ok) break;
    v >>= 1;
  }
  return v;
}

template <typename Addr>
int launch_mover(const Addr& addr, int64_t n, int64_t row_bytes, int vec, hipStream_t stream,
                 int kernel_id = -1) {
  if (n == 0) return HADES_OK;
  const int64_t cpr64 = row_bytes / vec;
  HADES_REQUIRE(cpr64 * kRowsPerBlock < (int64_t(1) << 30), "row of %lld bytes is too large",
                (long long)row_bytes);
  const int cpr = static_cast<int>(cpr64);
  const int shift = is_pow2(cpr) ? ilog2_ceil(cpr) : -1;
  const int64_t blocks = ceil_div(n, kRowsPerBlock);
  HADES_REQUIRE(blocks < (int64_t(1) << 31), "too many rows: %lld", (long long)n);
  dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
  if (vec == 16) {
    HADES_LAUNCH_TIMED(kernel_id, stream, (row_move_kernel<u32x4, Addr>), grid, block, 0, stream,
                       addr, n, cpr, shift);
  } else if (vec == 8) {
    HADES_LAUNCH((row_move_kernel<u32x2, Addr>), grid, block, 0, stream, addr, n, cpr, shift);
  } else {
    HADES_LAUNCH((row_move_kernel<uint32_t, Addr>), grid, block, 0, stream, addr, n, cpr, shift);
  }
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

int elem_size(int dtype) { return dtype == HADES_F32 ? 4 : dtype == HADES_F64 ? 8 : 0; }

#define HADES_ROW_ARGS_CHECK()                                                              \
  HADES_REQUIRE(n >= 0 && dim >= 1, "n must be >= 0 and dim >= 1 (n=%lld dim=%lld)",        \
                (long long)n, (long long)dim);                                              \
  HADES_REQUIRE(elem_size(dtype) != 0, "Type can only be float or double (code %d)", dtype);\
  const int64_t row_bytes = dim * elem_size(dtype);

#define HADES_ITYPE_CHECK() \
  HADES_REQUIRE(itype == HADES_I32 || itype == HADES_I64, "ID can only be int32 or int64 (code %d)", itype)

}  // namespace
}  // namespace hades

using namespace hades;

extern "C" {

int hades_fetch(const void* src, const void* src_index, void* dst, const void* dst_index,
                int64_t n, int64_t dim, int dtype, int itype, void* stream) {
  HADES_ROW_ARGS_CHECK();
  HADES_ITYPE_CHECK();
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(src && src_index && dst && dst_index, "null pointer argument");
  const int vec = pick_vec(row_bytes, {src, dst});
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (itype == HADES_I64) {
    AddrFetch<int64_t> a{(const char*)src, src_index, (char*)dst, dst_index, row_bytes};
    return launch_mover(a, n, row_bytes, vec, st);
  }
  AddrFetch<int32_t> a{(const char*)src, src_index, (char*)dst, dst_index, row_bytes};
  return launch_mover(a, n, row_bytes, vec, st);
}

int hades_fetch2(const void* src, const void* src_index, void* dst, int64_t n, int64_t dim,
                 int dtype, int itype, void* stream) {
  HADES_ROW_ARGS_CHECK();
  HADES_ITYPE_CHECK();
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(src && src_index && dst, "null pointer argument");
  const int vec = pick_vec(row_bytes, {src, dst});
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (itype == HADES_I64) {
    AddrFetch2<int64_t> a{(const char*)src, src_index, (char*)dst, row_bytes};
    return launch_mover(a, n, row_bytes, vec, st);
  }
  AddrFetch2<int32_t> a{(const char*)src, src_index, (char*)dst, row_bytes};
  return launch_mover(a, n, row_bytes, vec, st);
}

int hades_fetch_with_cache2(const void* cpu_src, const void* gpu_src, const void* src_index,
                            const void* index_map, void* dst, int64_t n, int64_t dim, int dtype,
                            int itype, void* stream) {
  HADES_ROW_ARGS_CHECK();
  HADES_ITYPE_CHECK();
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(cpu_src && gpu_src && src_index && index_map && dst, "null pointer argument");
  const int vec = pick_vec(row_bytes, {cpu_src, gpu_src, dst});
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (itype == HADES_I64) {
    AddrFetchMap<int64_t> a{(const char*)cpu_src, (const char*)gpu_src, src_index, index_map,
                            (char*)dst, row_bytes};
    return launch_mover(a, n, row_bytes, vec, st);
  }
  AddrFetchMap<int32_t> a{(const char*)cpu_src, (const char*)gpu_src, src_index, index_map,
                          (char*)dst, row_bytes};
  return launch_mover(a, n, row_bytes, vec, st);
}

int hades_set(const void* src, void* dst, const void* dst_index, int64_t n, int64_t dim,
              int dtype, int itype, void* stream) {
  HADES_ROW_ARGS_CHECK();
  HADES_ITYPE_CHECK();
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(src && dst && dst_index, "null pointer argument");
  const int vec = pick_vec(row_bytes, {src, dst});
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (itype == HADES_I64) {
    AddrSet<int64_t> a{(const char*)src, (char*)dst, dst_index, row_bytes};
    return launch_mover(a, n, row_bytes, vec, st);
  }
  AddrSet<int32_t> a{(const char*)src, (char*)dst, dst_index, row_bytes};
  return launch_mover(a, n, row_bytes, vec, st);
}

int hades_combine_scatter(const void* src, void* dst, const void* dst_index, int64_t n,
                          int64_t dim, int dtype, int itype, void* stream) {
  return hades_set(src, dst, dst_index, n, dim, dtype, itype, stream);
}

int hades_set_with_cache(const void* src, void* cpu_dst, void* gpu_dst, const void* dst_index,
                         const void* index_map, int64_t n, int64_t dim, int dtype, int itype,
                         void* stream) {
  HADES_ROW_ARGS_CHECK();
  HADES_ITYPE_CHECK();
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(src && cpu_dst && gpu_dst && dst_index && index_map, "null pointer argument");
  const int vec = pick_vec(row_bytes, {src, cpu_dst, gpu_dst});
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (itype == HADES_I64) {
    AddrSetMap<int64_t> a{(const char*)src, (char*)cpu_dst, (char*)gpu_dst, dst_index, index_map,
                          row_bytes};
    return launch_mover(a, n, row_bytes, vec, st);
  }
  AddrSetMap<int32_t> a{(const char*)src, (char*)cpu_dst, (char*)gpu_dst, dst_index, index_map,
                        row_bytes};
  return launch_mover(a, n, row_bytes, vec, st);
}

int hades_cached_fetch(const void* cold_src, const void* hot_src, const int64_t* q, int64_t n,
                       const int64_t* sorted_hot, int64_t num_hot, const void* hot_index, void* dst,
                       int64_t* loc_out, int64_t dim, int dtype, void* stream) {
  HADES_ROW_ARGS_CHECK();
  HADES_REQUIRE(num_hot >= 0, "num_hot must be >= 0");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(q && dst && (num_hot == 0 || (sorted_hot && hot_src)), "null pointer argument");
  const int vec = pick_vec(row_bytes, {cold_src, hot_src, dst});
  AddrFetchSorted a{(const char*)cold_src, (const char*)hot_src, q,
                    HotSet{sorted_hot, num_hot, static_cast<const uint32_t*>(hot_index)},
                    (char*)dst, loc_out, row_bytes};
  return launch_mover(a, n, row_bytes, vec, static_cast<hipStream_t>(stream),
                      HADES_KERNEL_CACHED_FETCH);
}

int hades_cached_fetch_loc(const void* cold_src, const void* hot_src, const int64_t* q,
                           const int64_t* loc, int64_t n, void* dst, int64_t dim, int dtype,
                           void* stream) {
  HADES_ROW_ARGS_CHECK();
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(q && loc && dst, "null pointer argument");
  const int vec = pick_vec(row_bytes, {cold_src, hot_src, dst});
  AddrFetchLoc a{(const char*)cold_src, (const char*)hot_src, q, loc, (char*)dst, row_bytes};
  return launch_mover(a, n, row_bytes, vec, static_cast<hipStream_t>(stream));
}

int hades_fetch_listed(const void* src, int64_t src_stride, const int64_t* src_index,
                       const int64_t* list, const int64_t* count, int64_t max_count, void* dst,
                       int64_t dim, int dtype, void* stream) {
  HADES_REQUIRE(max_count >= 0 && dim >= 1, "max_count must be >= 0 and dim >= 1");
  HADES_REQUIRE(elem_size(dtype) != 0, "Type can only be float or double (code %d)", dtype);
  HADES_REQUIRE(src_stride == 0 || src_stride >= dim, "src_stride must be 0 or >= dim");
  if (max_count == 0) return HADES_OK;
  HADES_REQUIRE(src && src_index && list && count && dst, "null pointer argument");
  const int64_t row_bytes = dim * elem_size(dtype);
  const int64_t stride_bytes = (src_stride ? src_stride : dim) * elem_size(dtype);
  int vec = pick_vec(row_bytes, {src, dst});
  while (vec > 4 && stride_bytes % vec != 0) vec >>= 1;
  ListedArgs a{(const char*)src, nullptr, stride_bytes, src_index, list, count, max_count,
               nullptr, (char*)dst, row_bytes, nullptr, nullptr, 0};
  return launch_listed<true>(a, vec, static_cast<hipStream_t>(stream));
}

int hades_fetch_listed_in_set(const void* src, int64_t src_stride, const int64_t* src_index,
                              const int64_t* list, const int64_t* count, int64_t max_count,
                              const int64_t* sorted_set, const int64_t* set_count, int64_t set_max,
                              void* dst, int64_t dim, int dtype, void* stream) {
  HADES_REQUIRE(max_count >= 0 && dim >= 1, "max_count must be >= 0 and dim >= 1");
  HADES_REQUIRE(set_max >= 0, "set_max must be >= 0");
  HADES_REQUIRE(elem_size(dtype) != 0, "Type can only be float or double (code %d)", dtype);
  HADES_REQUIRE(src_stride == 0 || src_stride >= dim, "src_stride must be 0 or >= dim");
  if (max_count == 0 || set_max == 0) return HADES_OK;
  HADES_REQUIRE(src && src_index && list && count && sorted_set && set_count && dst,
                "null pointer argument");
  const int64_t row_bytes = dim * elem_size(dtype);
  const int64_t stride_bytes = (src_stride ? src_stride : dim) * elem_size(dtype);
  int vec = pick_vec(row_bytes, {src, dst});
  while (vec > 4 && stride_bytes % vec != 0) vec >>= 1;
  ListedArgs a{(const char*)src, nullptr, stride_bytes, src_index, list, count, max_count,
               nullptr, (char*)dst, row_bytes, sorted_set, set_count, set_max};
  return launch_listed<true, true>(a, vec, static_cast<hipStream_t>(stream));
}

int hades_set_listed(const void* src, void* dst, int64_t dst_stride, const int64_t* dst_index,
                     const int64_t* list, const int64_t* count, int64_t max_count, int64_t dim,
                     int dtype, void* stream) {
  HADES_REQUIRE(max_count >= 0 && dim >= 1, "max_count must be >= 0 and dim >= 1");
  HADES_REQUIRE(elem_size(dtype) != 0, "Type can only be float or double (code %d)", dtype);
  HADES_REQUIRE(dst_stride == 0 || dst_stride >= dim, "dst_stride must be 0 or >= dim");
  if (max_count == 0) return HADES_OK;
  HADES_REQUIRE(src && dst_index && list && count && dst, "null pointer argument");
  const int64_t row_bytes = dim * elem_size(dtype);
  const int64_t stride_bytes = (dst_stride ? dst_stride : dim) * elem_size(dtype);
  int vec = pick_vec(row_bytes, {src, dst});
  while (vec > 4 && stride_bytes % vec != 0) vec >>= 1;
  ListedArgs a{nullptr, (char*)dst, stride_bytes, dst_index, list, count, max_count,
               (const char*)src, nullptr, row_bytes, nullptr, nullptr, 0};
  return launch_listed<false>(a, vec, static_cast<hipStream_t>(stream));
}

int hades_cached_set(const void* src, void* cold_dst, void* hot_dst, const int64_t* q, int64_t n,
                     const int64_t* sorted_hot, int64_t num_hot, const void* hot_index, int64_t dim,
                     int dtype, void* stream) {
  HADES_ROW_ARGS_CHECK();
  HADES_REQUIRE(num_hot >= 0, "num_hot must be >= 0");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(src && q && (num_hot == 0 || (sorted_hot && hot_dst)), "null pointer argument");
  const int vec = pick_vec(row_bytes, {src, cold_dst, hot_dst});
  AddrSetSorted a{(const char*)src, (char*)cold_dst, (char*)hot_dst, q,
                  HotSet{sorted_hot, num_hot, static_cast<const uint32_t*>(hot_index)}, row_bytes};
  return launch_mover(a, n, row_bytes, vec, static_cast<hipStream_t>(stream));
}

}  // extern "C"
