// combine: sort + dedup + segment-sum of duplicate-ID gradient rows
// (only_unique_grads, python/EmbCache/sparse_optim.py:132-139; also the local-aggregation
// reduction at :310 over concatenated trainer batches).
//
// Pipeline, all on one stream, no host synchronisation (the number of distinct ids stays on the
// device):
//   1. stable LSD radix sort of (key = id, value = occurrence position), only over the key bits
//      that id_bound leaves significant.  Stability keeps the positions of equal ids ascending,
//      which is what makes a sequential in-segment sum reproduce CPU index_add_.
//   2. run boundaries -> uids, seg_start, seg_of (index of the run every sorted position is in).
//   3. segmented sum of the gradient rows:
//        EXACT: one lane group per distinct id walks its rows left to right.
//        FAST : the sorted sequence is cut into fixed chunks of R positions, one lane group per
//               chunk; runs inside a chunk are summed left to right and stored directly, runs
//               that cross chunk borders leave partial rows that a second kernel adds in chunk
//               order.  Work per group is uniform whatever the id skew; the shape of the sum
//               depends only on (n, R), so results are reproducible run to run.
#include "internal.h"

namespace hades {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kRadixBits = 8;
constexpr int kBins = 1 << kRadixBits;

// ---- key transforms ---------------------------------------------------------
template <typename KeyT>
__device__ __forceinline__ KeyT key_from_id(int64_t id);
template <>
__device__ __forceinline__ uint32_t key_from_id<uint32_t>(int64_t id) {
  return static_cast<uint32_t>(id);
}
template <>
__device__ __forceinline__ uint64_t key_from_id<uint64_t>(int64_t id) {
  return static_cast<uint64_t>(id) ^ (uint64_t(1) << 63);  // signed order -> unsigned order
}
template <typename KeyT>
__device__ __forceinline__ int64_t id_from_key(KeyT k);
template <>
__device__ __forceinline__ int64_t id_from_key<uint32_t>(uint32_t k) {
  return static_cast<int64_t>(k);
}
template <>
__device__ __forceinline__ int64_t id_from_key<uint64_t>(uint64_t k) {
  return static_cast<int64_t>(k ^ (uint64_t(1) << 63));
}

template <typename KeyT, bool FIRST>
__device__ __forceinline__ KeyT load_key(const void* __restrict__ in, int64_t i) {
  if (FIRST) return key_from_id<KeyT>(static_cast<const int64_t*>(in)[i]);
  return static_cast<const KeyT*>(in)[i];
}

// ---- radix pass, kernel 1: per-tile digit histogram -------------------------
// hist layout: hist[digit * nblocks + block]
template <typename KeyT, bool FIRST, int IPT>
__global__ __launch_bounds__(kThreads) void radix_hist_kernel(const void* __restrict__ keys_in,
                                                             int64_t n, int shift, uint32_t mask,
                                                             uint32_t* __restrict__ hist,
                                                             int64_t nblocks, int64_t id_bound,
                                                             int32_t* __restrict__ status) {
  __shared__ uint32_t s_hist[kBins];
  for (int d = threadIdx.x; d < kBins; d += kThreads) s_hist[d] = 0;
  __syncthreads();
  const int64_t tile0 = static_cast<int64_t>(blockIdx.x) * (kThreads * IPT);
  bool bad = false;
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = tile0 + r * kThreads + threadIdx.x;
    if (i < n) {
      if (FIRST && id_bound > 0) {
        const int64_t id = static_cast<const int64_t*>(keys_in)[i];
        bad = bad || id < 0 || id >= id_bound;
      }
      const KeyT k = load_key<KeyT, FIRST>(keys_in, i);
      atomicAdd(&s_hist[static_cast<uint32_t>(k >> shift) & mask], 1u);
    }
  }
  if (FIRST && bad) atomicOr(status, 1);
  __syncthreads();
  for (int d = threadIdx.x; d < kBins; d += kThreads) hist[d * nblocks + blockIdx.x] = s_hist[d];
}

// ---- single-block exclusive scan of a u32 array (in place) ------------------
constexpr int kScanThreads = 1024;
constexpr int kScanItems = 8;
__global__ __launch_bounds__(kScanThreads) void scan_u32_kernel(uint32_t* __restrict__ data,
                                                               int64_t len,
                                                               uint32_t* __restrict__ total_out) {
  __shared__ uint32_t smem[kScanThreads / kWave + 1];
  uint32_t carry = 0;
  for (int64_t base = 0; base < len; base += kScanThreads * kScanItems) {
    const int64_t i0 = base + static_cast<int64_t>(threadIdx.x) * kScanItems;
    uint32_t v[kScanItems];
    uint32_t sum = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      v[k] = (i0 + k < len) ? data[i0 + k] : 0u;
      sum += v[k];
    }
    uint32_t total;
    uint32_t ex = carry + block_exclusive_sum<uint32_t, kScanThreads>(sum, smem, &total);
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      if (i0 + k < len) data[i0 + k] = ex;
      ex += v[k];
    }
    carry += total;
  }
  if (total_out && threadIdx.x == 0) *total_out = carry;
}

// ---- radix pass, kernel 3: stable scatter -----------------------------------
// Tile order: wave w of the block owns tile positions [w*IPT*64, (w+1)*IPT*64), round r of that
// wave the 64 positions from r*64 on.  Ranks are handed out in exactly that order.
template <typename KeyT, bool FIRST, int IPT>
__global__ __launch_bounds__(kThreads) void radix_scatter_kernel(
    const void* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, int64_t n, int shift,
    uint32_t mask, int bits, const uint32_t* __restrict__ hist_scanned, int64_t nblocks,
    KeyT* __restrict__ keys_out, uint32_t* __restrict__ vals_out) {
  __shared__ uint32_t s_cnt[kWaves][kBins];
  __shared__ uint32_t s_glob[kBins];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  for (int d = threadIdx.x; d < kWaves * kBins; d += kThreads) (&s_cnt[0][0])[d] = 0;
  for (int d = threadIdx.x; d < kBins; d += kThreads)
    s_glob[d] = hist_scanned[d * nblocks + blockIdx.x];
  __syncthreads();

  const int64_t wave0 = static_cast<int64_t>(blockIdx.x) * (kThreads * IPT) + wave * (IPT * kWave);
  KeyT key[IPT];
  uint32_t val[IPT];
  uint32_t rank[IPT];
  const uint64_t lt_mask = (uint64_t(1) << lane) - 1;
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = wave0 + r * kWave + lane;
    const bool valid = i < n;
    key[r] = valid ? load_key<KeyT, FIRST>(keys_in, i) : KeyT(0);
    val[r] = valid ? (FIRST ? static_cast<uint32_t>(i) : vals_in[i]) : 0u;
    const uint32_t d = static_cast<uint32_t>(key[r] >> shift) & mask;
    // lanes of this wave that hold the same digit
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < kRadixBits; ++b) {
      if (b < bits) {
        const uint64_t bal = __ballot((d >> b) & 1u);
        peers &= ((d >> b) & 1u) ? bal : ~bal;
      }
    }
    uint32_t old = 0;
    if (valid) {
      old = s_cnt[wave][d];
    }
    // every peer has read the counter before the leader bumps it: LDS operations of one wave
    // complete in program order
    __builtin_amdgcn_wave_barrier();
    if (valid && (peers & lt_mask) == 0) s_cnt[wave][d] = old + __popcll(peers);
    rank[r] = old + __popcll(peers & lt_mask);
  }
  __syncthreads();
  // exclusive prefix over the waves, per digit
  for (int d = threadIdx.x; d < kBins; d += kThreads) {
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const uint32_t t = s_cnt[w][d];
      s_cnt[w][d] = run;
      run += t;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = wave0 + r * kWave + lane;
    if (i < n) {
      const uint32_t d = static_cast<uint32_t>(key[r] >> shift) & mask;
      const uint32_t pos = s_glob[d] + s_cnt[wave][d] + rank[r];
      keys_out[pos] = key[r];
      vals_out[pos] = val[r];
    }
  }
}

// ---- run boundaries ---------------------------------------------------------
constexpr int kUItems = 8;
constexpr int kUTile = kThreads * kUItems;

template <typename KeyT>
__global__ __launch_bounds__(kThreads) void run_count_kernel(const KeyT* __restrict__ keys,
                                                            int64_t n,
                                                            uint32_t* __restrict__ blk_cnt) {
  __shared__ uint32_t smem[kWaves + 1];
  const int64_t j0 = static_cast<int64_t>(blockIdx.x) * kUTile + threadIdx.x * kUItems;
  uint32_t c = 0;
  if (j0 < n) {
    KeyT prev = j0 > 0 ? keys[j0 - 1] : KeyT(0);
#pragma unroll
    for (int k = 0; k < kUItems; ++k) {
      const int64_t j = j0 + k;
      if (j < n) {
        const KeyT cur = keys[j];
        c += (j == 0 || cur != prev) ? 1u : 0u;
        prev = cur;
      }
    }
  }
  uint32_t total;
  (void)block_exclusive_sum<uint32_t, kThreads>(c, smem, &total);
  if (threadIdx.x == 0) blk_cnt[blockIdx.x] = total;
}

template <typename KeyT>
__global__ __launch_bounds__(kThreads) void run_emit_kernel(
    const KeyT* __restrict__ keys, const uint32_t* __restrict__ perm, int64_t n,
    const uint32_t* __restrict__ blk_off, int64_t* __restrict__ uids,
    uint32_t* __restrict__ seg_start, uint32_t* __restrict__ seg_of,
    int64_t* __restrict__ num_unique, int32_t* __restrict__ inverse) {
  __shared__ uint32_t smem[kWaves + 1];
  const int64_t j0 = static_cast<int64_t>(blockIdx.x) * kUTile + threadIdx.x * kUItems;
  uint32_t flag[kUItems];
  KeyT kk[kUItems];
  uint32_t c = 0;
  if (j0 < n) {
    KeyT prev = j0 > 0 ? keys[j0 - 1] : KeyT(0);
#pragma unroll
    for (int k = 0; k < kUItems; ++k) {
      const int64_t j = j0 + k;
      flag[k] = 0;
      if (j < n) {
        kk[k] = keys[j];
        flag[k] = (j == 0 || kk[k] != prev) ? 1u : 0u;
        prev = kk[k];
        c += flag[k];
      }
    }
  }
  uint32_t total;
  uint32_t u = blk_off[blockIdx.x] + block_exclusive_sum<uint32_t, kThreads>(c, smem, &total);
  // u = number of runs that begin before j0
  if (j0 < n) {
#pragma unroll
    for (int k = 0; k < kUItems; ++k) {
      const int64_t j = j0 + k;
      if (j < n) {
        u += flag[k];
        const uint32_t seg = u - 1;
        seg_of[j] = seg;
        if (inverse) inverse[perm[j]] = static_cast<int32_t>(seg);
        if (flag[k]) {
          uids[seg] = id_from_key<KeyT>(kk[k]);
          seg_start[seg] = static_cast<uint32_t>(j);
        }
        if (j == n - 1) {
          seg_start[u] = static_cast<uint32_t>(n);
          num_unique[0] = static_cast<int64_t>(u);
        }
      }
    }
  }
}

__global__ void set_i64_kernel(int64_t* p, int64_t v) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *p = v;
}

// ---- segmented sums ----------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int VEC>
struct RowVec;
template <>
struct RowVec<4> {
  typedef f32x4 type;
  static __device__ __forceinline__ type zero() { return type{0.f, 0.f, 0.f, 0.f}; }
};
template <>
struct RowVec<1> {
  typedef float type;
  static __device__ __forceinline__ type zero() { return 0.f; }
};

constexpr int kSegUnroll = 8;

struct SegArgs {
  const float* grad;
  const uint32_t* perm;
  const uint32_t* seg_of;
  const uint32_t* seg_start;
  const int64_t* num_unique;
  float* sums;
  int64_t* cnts;
  float* partial;  // [2 * nchunks][dim]
  int64_t n;
  int64_t dim;
  int chunk;       // R: sorted positions per lane group
  int group;       // lanes per group (power of two <= 64)
  int col_tiles;   // ceil(dim / (group * VEC))
};

// FAST, kernel 1: one lane group per chunk of R consecutive sorted positions.
template <int VEC>
__global__ __launch_bounds__(kThreads) void seg_chunk_kernel(SegArgs a) {
  typedef typename RowVec<VEC>::type V;
  const int64_t gtid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t chunk_id = gtid / a.group;
  const int gl = static_cast<int>(gtid & (a.group - 1));
  const int64_t j0 = chunk_id * a.chunk;
  if (j0 >= a.n) return;
  const int64_t j1 = (j0 + a.chunk < a.n) ? j0 + a.chunk : a.n;
  const uint32_t first_run = a.seg_of[j0];

  for (int ct = 0; ct < a.col_tiles; ++ct) {
    const int64_t col = (static_cast<int64_t>(ct) * a.group + gl) * VEC;
    const bool col_ok = col < a.dim;
    V acc = RowVec<VEC>::zero();
    uint32_t cur = first_run;
    for (int64_t jj = j0; jj < j1; jj += kSegUnroll) {
      uint32_t seg[kSegUnroll];
      V row[kSegUnroll];
#pragma unroll
      for (int k = 0; k < kSegUnroll; ++k) {
        const int64_t j = jj + k;
        if (j < j1) {
          seg[k] = a.seg_of[j];
          const int64_t p = a.perm[j];
          row[k] = col_ok ? *reinterpret_cast<const V*>(a.grad + p * a.dim + col)
                          : RowVec<VEC>::zero();
        }
      }
#pragma unroll
      for (int k = 0; k < kSegUnroll; ++k) {
        if (jj + k < j1) {
          if (seg[k] != cur) {
            // run `cur` ends inside this chunk; it is whole unless it began before the chunk
            float* out = (cur != first_run || a.seg_start[cur] >= j0)
                             ? a.sums + static_cast<int64_t>(cur) * a.dim
                             : a.partial + (2 * chunk_id) * a.dim;
            if (col_ok) *reinterpret_cast<V*>(out + col) = acc;
            acc = RowVec<VEC>::zero();
            cur = seg[k];
          }
          acc += row[k];
        }
      }
    }
    // last run of the chunk: whole only if it ends exactly at the chunk end and began inside
    const bool ends_here = a.seg_start[cur + 1] <= j1;
    const bool began_here = a.seg_start[cur] >= j0;
    float* out;
    if (ends_here && began_here) {
      out = a.sums + static_cast<int64_t>(cur) * a.dim;
    } else if (cur == first_run) {
      out = a.partial + (2 * chunk_id) * a.dim;  // head slot
    } else {
      out = a.partial + (2 * chunk_id + 1) * a.dim;  // tail slot
    }
    if (col_ok) *reinterpret_cast<V*>(out + col) = acc;
  }
}

// FAST, kernel 2: block c finishes the run that begins in chunk c and crosses into chunk c+1,
// adding its partial rows in chunk order (lane groups take partials round-robin, then group 0 adds
// the per-group sums in group order).  Also writes the occurrence counts.
template <int VEC>
__global__ __launch_bounds__(kThreads) void seg_fixup_kernel(SegArgs a) {
  typedef typename RowVec<VEC>::type V;
  __shared__ V s_part[kThreads];
  const int64_t U = a.num_unique[0];
  const int64_t gtid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (gtid < U)
    a.cnts[gtid] = static_cast<int64_t>(a.seg_start[gtid + 1]) - static_cast<int64_t>(a.seg_start[gtid]);

  const int64_t c = blockIdx.x;
  const int64_t border = (c + 1) * a.chunk;
  if (border >= a.n) return;
  const uint32_t u = a.seg_of[border - 1];
  if (a.seg_of[border] != u) return;           // no run crosses this border
  const int64_t start = a.seg_start[u];
  if (start < c * a.chunk) return;              // the run began earlier: an earlier block owns it
  const int64_t end = a.seg_start[u + 1];
  const int64_t c_last = (end - 1) / a.chunk;
  const int64_t nparts = c_last - c + 1;
  const int ngroups = kThreads / a.group;
  const int g = threadIdx.x / a.group;
  const int gl = threadIdx.x & (a.group - 1);
  // partial row of chunk c+t: chunk c keeps it in the tail slot unless the run opens the chunk
  const int64_t first_slot = (start == c * a.chunk) ? 2 * c : 2 * c + 1;

  for (int ct = 0; ct < a.col_tiles; ++ct) {
    const int64_t col = (static_cast<int64_t>(ct) * a.group + gl) * VEC;
    const bool col_ok = col < a.dim;
    V acc = RowVec<VEC>::zero();
    for (int64_t t0 = g; t0 < nparts; t0 += static_cast<int64_t>(ngroups) * kSegUnroll) {
      V row[kSegUnroll];
#pragma unroll
      for (int k = 0; k < kSegUnroll; ++k) {
        const int64_t t = t0 + static_cast<int64_t>(k) * ngroups;
        if (t < nparts) {
          const int64_t slot = t == 0 ? first_slot : 2 * (c + t);
          row[k] = col_ok ? *reinterpret_cast<const V*>(a.partial + slot * a.dim + col)
                          : RowVec<VEC>::zero();
        }
      }
#pragma unroll
      for (int k = 0; k < kSegUnroll; ++k) {
        const int64_t t = t0 + static_cast<int64_t>(k) * ngroups;
        if (t < nparts) acc += row[k];
      }
    }
    __syncthreads();
    s_part[threadIdx.x] = acc;
    __syncthreads();
    if (g == 0) {
      V tot = s_part[gl];
      for (int gg = 1; gg < ngroups; ++gg) tot += s_part[gg * a.group + gl];
      if (col_ok) *reinterpret_cast<V*>(a.sums + static_cast<int64_t>(u) * a.dim + col) = tot;
    }
  }
}

// EXACT: one lane group per distinct id, strictly left to right from +0.0f.
template <int VEC>
__global__ __launch_bounds__(kThreads) void seg_exact_kernel(SegArgs a) {
  typedef typename RowVec<VEC>::type V;
  const int64_t U = a.num_unique[0];
  const int64_t gtid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t u = gtid / a.group;
  const int gl = static_cast<int>(gtid & (a.group - 1));
  if (u >= U) return;
  const int64_t j0 = a.seg_start[u];
  const int64_t j1 = a.seg_start[u + 1];
  if (gl == 0) a.cnts[u] = j1 - j0;
  for (int ct = 0; ct < a.col_tiles; ++ct) {
    const int64_t col = (static_cast<int64_t>(ct) * a.group + gl) * VEC;
    if (col >= a.dim) continue;
    V acc = RowVec<VEC>::zero();
    for (int64_t jj = j0; jj < j1; jj += kSegUnroll) {
      V row[kSegUnroll];
#pragma unroll
      for (int k = 0; k < kSegUnroll; ++k) {
        if (jj + k < j1) {
          const int64_t p = a.perm[jj + k];
          row[k] = *reinterpret_cast<const V*>(a.grad + p * a.dim + col);
        }
      }
#pragma unroll
      for (int k = 0; k < kSegUnroll; ++k) {
        if (jj + k < j1) acc += row[k];
      }
    }
    *reinterpret_cast<V*>(a.sums + u * a.dim + col) = acc;
  }
}

__global__ __launch_bounds__(kThreads) void rows_div_kernel(float* __restrict__ sums,
                                                           const int64_t* __restrict__ cnts,
                                                           const int64_t* __restrict__ num_unique,
                                                           int64_t max_rows, int64_t dim,
                                                           int one_plus) {
  const int64_t U = num_unique ? num_unique[0] : max_rows;
  const int64_t total = U * dim;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * kThreads) {
    const int64_t c = cnts[i / dim] + (one_plus ? 1 : 0);
    sums[i] = sums[i] / static_cast<float>(c);
  }
}

// ---- host-side plan ----------------------------------------------------------
constexpr int kIPT = 4;                      // keys per thread in a radix tile
constexpr int kRadixTile = kThreads * kIPT;

struct Plan {
  bool key64;
  int key_bits;
  int passes;
  int chunk;      // R
  int vec;        // 4 or 1
  int group;
  int col_tiles;
  int64_t nblocks_radix;
  int64_t nblocks_runs;
  int64_t nchunks;
};

Plan make_plan(int64_t n, int64_t dim, int64_t id_bound, bool grad_aligned) {
  Plan p;
  if (id_bound > 0 && id_bound <= (int64_t(1) << 32)) {
    p.key64 = false;
    p.key_bits = ilog2_ceil(static_cast<uint64_t>(id_bound));
  } else if (id_bound > 0) {
    p.key64 = true;  // ids are non-negative: the flipped sign bit is constant, skip it
    p.key_bits = ilog2_ceil(static_cast<uint64_t>(id_bound));
  } else {
    p.key64 = true;
    p.key_bits = 64;
  }
  if (p.key_bits < 1) p.key_bits = 1;
  p.passes = (p.key_bits + kRadixBits - 1) / kRadixBits;
  p.vec = (dim % 4 == 0 && grad_aligned) ? 4 : 1;
  const int64_t lanes = (dim + p.vec - 1) / p.vec;
  int g = 1;
  while (g < lanes && g < 64) g <<= 1;
  p.group = g;
  p.col_tiles = static_cast<int>((lanes + g - 1) / g);
  p.chunk = 32;
  p.nblocks_radix = ceil_div(n > 0 ? n : 1, kRadixTile);
  p.nblocks_runs = ceil_div(n > 0 ? n : 1, kUTile);
  p.nchunks = ceil_div(n > 0 ? n : 1, p.chunk);
  return p;
}

// workspace of the sort alone
struct SortWs {
  int32_t* status;
  void* keys[2];
  uint32_t* vals[2];
  uint32_t* hist;
  size_t bytes;
};

void carve_sort(Carver& c, int64_t n, SortWs* w) {
  const int64_t nn = n > 0 ? n : 1;
  w->status = c.take<int32_t>(64);
  for (int i = 0; i < 2; ++i) w->keys[i] = c.take<uint64_t>(nn);  // sized for 64-bit keys
  for (int i = 0; i < 2; ++i) w->vals[i] = c.take<uint32_t>(nn);
  w->hist = c.take<uint32_t>(kBins * ceil_div(nn, kRadixTile));
  w->bytes = c.total();
}

struct Ws {
  SortWs sort;
  uint32_t* run_cnt;
  uint32_t* seg_of;
  uint32_t* seg_start;
  float* partial;
  size_t bytes;
};

Ws carve(void* ws, int64_t n, int64_t dim, const Plan& p) {
  Carver c(ws);
  Ws w;
  const int64_t nn = n > 0 ? n : 1;
  carve_sort(c, n, &w.sort);
  w.run_cnt = c.take<uint32_t>(p.nblocks_runs + 1);
  w.seg_of = c.take<uint32_t>(nn);
  w.seg_start = c.take<uint32_t>(nn + 1);
  w.partial = c.take<float>(2 * p.nchunks * dim);
  w.bytes = c.total();
  return w;
}

template <typename KeyT>
int run_sort(const int64_t* idx, int64_t n, int64_t id_bound, const Plan& p, const SortWs& w,
             hipStream_t st, const void** keys_out, const uint32_t** perm_out) {
  const dim3 grid(static_cast<unsigned>(p.nblocks_radix)), block(kThreads);
  const void* kin = idx;
  const uint32_t* vin = nullptr;
  int cur = 0;
  int shift = 0;
  const int base = p.key_bits / p.passes, extra = p.key_bits % p.passes;
  for (int pass = 0; pass < p.passes; ++pass) {
    const int bits = base + (pass < extra ? 1 : 0);
    const uint32_t mask = (1u << bits) - 1u;
    KeyT* kout = static_cast<KeyT*>(w.keys[cur]);
    uint32_t* vout = w.vals[cur];
    if (pass == 0) {
      hipLaunchKernelGGL((radix_hist_kernel<KeyT, true, kIPT>), grid, block, 0, st, kin, n, shift,
                         mask, w.hist, p.nblocks_radix, id_bound, w.status);
    } else {
      hipLaunchKernelGGL((radix_hist_kernel<KeyT, false, kIPT>), grid, block, 0, st, kin, n, shift,
                         mask, w.hist, p.nblocks_radix, id_bound, w.status);
    }
    HADES_LAUNCH_CHECK();
    hipLaunchKernelGGL(scan_u32_kernel, dim3(1), dim3(kScanThreads), 0, st, w.hist,
                       static_cast<int64_t>(kBins) * p.nblocks_radix,
                       static_cast<uint32_t*>(nullptr));
    HADES_LAUNCH_CHECK();
    if (pass == 0) {
      hipLaunchKernelGGL((radix_scatter_kernel<KeyT, true, kIPT>), grid, block, 0, st, kin, vin, n,
                         shift, mask, bits, w.hist, p.nblocks_radix, kout, vout);
    } else {
      hipLaunchKernelGGL((radix_scatter_kernel<KeyT, false, kIPT>), grid, block, 0, st, kin, vin, n,
                         shift, mask, bits, w.hist, p.nblocks_radix, kout, vout);
    }
    HADES_LAUNCH_CHECK();
    kin = kout;
    vin = vout;
    cur ^= 1;
    shift += bits;
  }
  *keys_out = kin;
  *perm_out = vin;
  return HADES_OK;
}

template <typename KeyT>
int run_runs(const void* sorted_keys, const uint32_t* perm, int64_t n, const Plan& p, const Ws& w,
             int64_t* uids, int64_t* num_unique, int32_t* inverse, hipStream_t st) {
  const KeyT* keys = static_cast<const KeyT*>(sorted_keys);
  const dim3 rgrid(static_cast<unsigned>(p.nblocks_runs)), block(kThreads);
  hipLaunchKernelGGL((run_count_kernel<KeyT>), rgrid, block, 0, st, keys, n, w.run_cnt);
  HADES_LAUNCH_CHECK();
  hipLaunchKernelGGL(scan_u32_kernel, dim3(1), dim3(kScanThreads), 0, st, w.run_cnt,
                     p.nblocks_runs, static_cast<uint32_t*>(nullptr));
  HADES_LAUNCH_CHECK();
  hipLaunchKernelGGL((run_emit_kernel<KeyT>), rgrid, block, 0, st, keys, perm, n, w.run_cnt, uids,
                     w.seg_start, w.seg_of, num_unique, inverse);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

}  // namespace

size_t sort_ids_workspace_bytes(int64_t n) {
  Carver c(nullptr);
  SortWs w;
  carve_sort(c, n, &w);
  return w.bytes;
}

int sort_ids(const int64_t* ids, int64_t n, int64_t id_bound, void* workspace,
             size_t workspace_bytes, hipStream_t st, SortResult* out) {
  HADES_REQUIRE(n >= 1 && n < (int64_t(1) << 30), "sort: n out of range");
  const Plan p = make_plan(n, 1, id_bound, true);
  Carver c(workspace);
  SortWs w;
  carve_sort(c, n, &w);
  if (workspace == nullptr || workspace_bytes < w.bytes)
    return set_error(HADES_ERR_WORKSPACE, "sort workspace too small: need %zu bytes, got %zu",
                     w.bytes, workspace_bytes);
  out->key64 = p.key64;
  return p.key64 ? run_sort<uint64_t>(ids, n, id_bound, p, w, st, &out->sorted_keys, &out->perm)
                 : run_sort<uint32_t>(ids, n, id_bound, p, w, st, &out->sorted_keys, &out->perm);
}

}  // namespace hades

using namespace hades;

extern "C" {

size_t hades_combine_workspace_bytes(int64_t n, int64_t dim) {
  if (n < 0 || dim < 1) return 0;
  const Plan p = make_plan(n, dim, 0, true);
  return carve(nullptr, n, dim, p).bytes;
}

int hades_combine(const int64_t* idx, const float* grad, int64_t n, int64_t dim, int64_t id_bound,
                  int mode, int64_t* uids, float* sums, int64_t* cnts, int64_t* num_unique,
                  int32_t* inverse, void* workspace, size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(n >= 0 && dim >= 1, "n must be >= 0 and dim >= 1");
  HADES_REQUIRE(n < (int64_t(1) << 30), "combine: n must be below 2^30 (got %lld)", (long long)n);
  HADES_REQUIRE(id_bound >= 0, "id_bound must be >= 0");
  HADES_REQUIRE(mode == HADES_COMBINE_FAST || mode == HADES_COMBINE_EXACT, "unknown combine mode %d",
                mode);
  HADES_REQUIRE(num_unique != nullptr, "num_unique must not be null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n == 0) {
    hipLaunchKernelGGL(set_i64_kernel, dim3(1), dim3(64), 0, st, num_unique, int64_t(0));
    HADES_LAUNCH_CHECK();
    return HADES_OK;
  }
  HADES_REQUIRE(idx && grad && uids && sums && cnts, "null pointer argument");
  const bool aligned = (align_of_ptr(grad) % 16) == 0 && (align_of_ptr(sums) % 16) == 0;
  const Plan p = make_plan(n, dim, id_bound, aligned);
  const Ws w = carve(workspace, n, dim, p);
  if (workspace == nullptr || workspace_bytes < w.bytes)
    return set_error(HADES_ERR_WORKSPACE, "combine workspace too small: need %zu bytes, got %zu",
                     w.bytes, workspace_bytes);
  HADES_REQUIRE((align_of_ptr(workspace) & 255) == 0, "workspace must be 256-byte aligned");

  const uint32_t* perm = nullptr;
  const void* sorted_keys = nullptr;
  int rc = p.key64 ? run_sort<uint64_t>(idx, n, id_bound, p, w.sort, st, &sorted_keys, &perm)
                   : run_sort<uint32_t>(idx, n, id_bound, p, w.sort, st, &sorted_keys, &perm);
  if (rc != HADES_OK) return rc;
  rc = p.key64 ? run_runs<uint64_t>(sorted_keys, perm, n, p, w, uids, num_unique, inverse, st)
               : run_runs<uint32_t>(sorted_keys, perm, n, p, w, uids, num_unique, inverse, st);
  if (rc != HADES_OK) return rc;

  SegArgs a;
  a.grad = grad;
  a.perm = perm;
  a.seg_of = w.seg_of;
  a.seg_start = w.seg_start;
  a.num_unique = num_unique;
  a.sums = sums;
  a.cnts = cnts;
  a.partial = w.partial;
  a.n = n;
  a.dim = dim;
  a.chunk = p.chunk;
  a.group = p.group;
  a.col_tiles = p.col_tiles;
  if (mode == HADES_COMBINE_EXACT) {
    const int64_t blocks = ceil_div(n * p.group, kThreads);
    HADES_REQUIRE(blocks < (int64_t(1) << 31), "combine: too many rows");
    if (p.vec == 4)
      hipLaunchKernelGGL((seg_exact_kernel<4>), dim3((unsigned)blocks), dim3(kThreads), 0, st, a);
    else
      hipLaunchKernelGGL((seg_exact_kernel<1>), dim3((unsigned)blocks), dim3(kThreads), 0, st, a);
    HADES_LAUNCH_CHECK();
  } else {
    const int64_t blocks = ceil_div(p.nchunks * p.group, kThreads);
    HADES_REQUIRE(blocks < (int64_t(1) << 31), "combine: too many rows");
    if (p.vec == 4)
      hipLaunchKernelGGL((seg_chunk_kernel<4>), dim3((unsigned)blocks), dim3(kThreads), 0, st, a);
    else
      hipLaunchKernelGGL((seg_chunk_kernel<1>), dim3((unsigned)blocks), dim3(kThreads), 0, st, a);
    HADES_LAUNCH_CHECK();
    // one block per chunk; also covers every u < U <= n with a thread for the counts
    const int64_t fblocks = p.nchunks > ceil_div(n, kThreads) ? p.nchunks : ceil_div(n, kThreads);
    if (p.vec == 4)
      hipLaunchKernelGGL((seg_fixup_kernel<4>), dim3((unsigned)fblocks), dim3(kThreads), 0, st, a);
    else
      hipLaunchKernelGGL((seg_fixup_kernel<1>), dim3((unsigned)fblocks), dim3(kThreads), 0, st, a);
    HADES_LAUNCH_CHECK();
  }
  return HADES_OK;
}

int hades_rows_div_count(float* sums, const int64_t* cnts, const int64_t* num_unique,
                         int64_t max_rows, int64_t dim, int one_plus, void* stream) {
  HADES_REQUIRE(max_rows >= 0 && dim >= 1, "max_rows must be >= 0 and dim >= 1");
  if (max_rows == 0) return HADES_OK;
  HADES_REQUIRE(sums && cnts, "null pointer argument");
  int64_t blocks = ceil_div(max_rows * dim, kThreads);
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(rows_div_kernel, dim3((unsigned)blocks), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), sums, cnts, num_unique, max_rows, dim,
                     one_plus);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

}  // extern "C"
