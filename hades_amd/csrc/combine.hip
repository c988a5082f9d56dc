// combine: sort + dedup + segment-sum of duplicate-ID gradient rows
// (only_unique_grads, python/EmbCache/sparse_optim.py:132-139; also the local-aggregation
// reduction at :310 over concatenated trainer batches).
//
// Pipeline, all on one stream, no host synchronisation (the number of distinct ids stays on the
// device) and no spin-waits between blocks:
//   1. stable LSD radix sort of (key = id, value = occurrence position), 8 bits per pass, only
//      over the key bits that id_bound leaves significant.  Stability keeps the positions of
//      equal ids ascending, which is what makes a sequential in-segment sum reproduce CPU
//      index_add_.  Per pass two kernels: digit counts per tile of 1024 keys and per group of four
//      tiles, then a scatter in which every block derives its own global digit offsets from those
//      counts (column sums over the group rows and the tile rows before it), ranks its keys
//      stably through LDS and writes them out.  From 64 groups on (batches above 256 K ids) a
//      third, tiny kernel turns the group counts into prefixes first, so that a scatter block
//      reads five count rows whatever the batch size.
//   2. run boundaries -> uids, seg_start, seg_of (index of the run every sorted position is in).
//   3. segmented sum of the gradient rows:
//        EXACT: one lane group per distinct id walks its rows left to right.  The rows of a run
//               of 64 rows or more are first copied, by the whole chip, into four-float column
//               slices of a staging area at the end of the workspace; a block per run and slice
//               then streams its slice through LDS and one thread per column adds it in the same
//               order (without the staging area: 1024-thread blocks fetch the rows of their run
//               themselves, one block per 32-float column slice).
//        FAST : the sorted sequence is cut into fixed chunks of 32 positions per lane group; a
//               block stages the sort permutation of its groups in LDS, every group sums its
//               runs left to right with 16 row loads in flight, runs that cross group borders
//               are merged in group order inside the block, and runs that cross block borders
//               leave at most two partial rows per block that a second kernel adds in block
//               order.  Work per group is uniform whatever the id skew; the shape of the sum
//               depends only on (n, dim), so results are reproducible run to run.
#include "internal.h"

#include <stdlib.h>

#include <atomic>
#include <mutex>

// Scratch memory of hades_combine_static: one copy per GPU, held from the moment the code object
// is loaded on that GPU until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress; the address kernels are given is the one that call returns.
static __device__ __align__(256) unsigned char g_static_scratch[HADES_COMBINE_STATIC_SCRATCH_BYTES];

namespace hades {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kRadixBits = 8;
constexpr int kBins = 1 << kRadixBits;
constexpr int kMaxPasses = 8;
constexpr int kGroup = 4;  // tiles counted by one block of the count kernel
constexpr int kIpt = 4;    // keys per thread in a radix tile: tiles of 1024 keys
constexpr int kIptSmall = 2;             // ... tiles of 512 keys for batches of up to kSmallBatch ids:
constexpr int64_t kSmallBatch = 1 << 17; // they would leave three quarters of the chip without a tile
constexpr int kIptLarge = 8;             // ... and tiles of 2 048 keys for batches above kLargeBatch ids
constexpr int64_t kLargeBatch = 1 << 19;
constexpr int kScanFrom = 64;  // groups of tiles from which the group counts get their own scan

// keys per thread of a tile of the three-kernel radix passes
inline int radix_ipt_for(int64_t n) {
  return n <= kSmallBatch ? kIptSmall : (n > kLargeBatch ? kIptLarge : kIpt);
}

// ---- key transforms ---------------------------------------------------------
template <typename KeyT>
__host__ __device__ __forceinline__ KeyT key_from_id(int64_t id);
template <>
__host__ __device__ __forceinline__ uint32_t key_from_id<uint32_t>(int64_t id) {
  return static_cast<uint32_t>(id);
}
template <>
__host__ __device__ __forceinline__ uint64_t key_from_id<uint64_t>(int64_t id) {
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

// lanes of the wave whose `v` equals mine, among the lanes in `among` (nbits significant bits)
__device__ __forceinline__ uint64_t match_any(uint32_t v, int nbits, uint64_t among) {
  uint64_t peers = among;
  for (int b = 0; b < nbits; ++b) {
    const uint64_t bal = __ballot((v >> b) & 1u);
    peers &= ((v >> b) & 1u) ? bal : ~bal;
  }
  return peers;
}

// ---- per-tile digit counts of one pass ------------------------------------------------------
// counts layout: cnt[tile * kBins + digit].  (Counting the next pass's digits with global atomics
// from inside the scatter was measured at twice the cost of this kernel.)
// A block counts kGroup consecutive tiles and also writes their sum, gcnt[group * kBins + digit]:
// the scatter then adds up one row per group plus the few tile rows inside its own group instead
// of one row per tile.
template <typename KeyT, bool FIRST, int IPT>
__global__ __launch_bounds__(kGroup * kThreads) void radix_count_kernel(
    const void* __restrict__ keys_in, int64_t n, int shift, uint32_t mask,
    uint32_t* __restrict__ cnt, uint32_t* __restrict__ gcnt, int64_t ntiles, int64_t id_bound,
    int32_t* __restrict__ bad_blk, int64_t nbad) {
  __shared__ uint32_t s_hist[kGroup][kBins];
  const int g = threadIdx.x / kThreads;  // the tile of the group this thread counts
  const int t = threadIdx.x % kThreads;  // kThreads == kBins: also the digit it writes out
  s_hist[g][t] = 0;
  __syncthreads();
  const int64_t tile = static_cast<int64_t>(blockIdx.x) * kGroup + g;
  const int64_t tile0 = tile * (kThreads * IPT);
  bool bad = false;
  const int lane = t & (kWave - 1);
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = tile0 + r * kThreads + t;
    const bool valid = i < n;
    uint32_t d = 0;
    if (valid) {
      if (FIRST) {
        const int64_t id = static_cast<const int64_t*>(keys_in)[i];
        bad = bad || (id_bound > 0 && (id < 0 || id >= id_bound));
      }
      const KeyT k = load_key<KeyT, FIRST>(keys_in, i);
      d = static_cast<uint32_t>(k >> shift) & mask;
    }
    // After the first pass equal keys sit next to each other, and 64 lanes adding to one LDS
    // counter are served one after the other (the counters showed bank-conflict cycles at 7-9
    // times the useful LDS cycles).  Lanes with the digit of their left neighbour stay silent;
    // the first lane of every stretch adds the length of the stretch.
    const uint32_t left = __shfl_up(d, 1);
    const bool head = valid && (lane == 0 || left != d);
    const uint64_t heads = __ballot(head);
    const uint64_t live = __ballot(valid);          // the valid lanes form a prefix of the wave
    if (head) {
      const uint64_t above = lane == kWave - 1 ? 0 : heads >> (lane + 1);
      const int next = above ? lane + 1 + __builtin_ctzll(above) : __popcll(live);
      atomicAdd(&s_hist[g][d], static_cast<uint32_t>(next - lane));
    }
  }
  // the first pass also checks the promise 0 <= id < id_bound: one flag per block, written by
  // every block on every call, so the flags need no clearing and are never stale
  const int any_bad = __syncthreads_or(FIRST && bad ? 1 : 0);
  if (FIRST && threadIdx.x == 0) bad_blk[blockIdx.x] = any_bad;
  // the flags of the blocks a launch with larger tiles would have had: block 0 clears them
  if (FIRST && blockIdx.x == 0)
    for (int64_t f = gridDim.x + threadIdx.x; f < nbad; f += kGroup * kThreads) bad_blk[f] = 0;
  if (tile < ntiles) cnt[tile * kBins + t] = s_hist[g][t];
  if (g == 0) {
    uint32_t sum = 0;
#pragma unroll
    for (int k = 0; k < kGroup; ++k) sum += s_hist[k][t];  // tiles past the end counted nothing
    gcnt[static_cast<int64_t>(blockIdx.x) * kBins + t] = sum;
  }
}

// ---- prefix of the group counts (large batches only) -------------------------------------------
// gcnt[g][d] becomes the number of keys with digit d in the groups before g, and row `ngroups`
// receives the column totals, so that a scatter block reads two rows of gcnt instead of one per
// group.  One wave per digit column: lanes take 64 consecutive groups, scan them in registers and
// carry the running total to the next 64.
__global__ __launch_bounds__(kThreads) void radix_group_scan_kernel(uint32_t* __restrict__ gcnt,
                                                                   int64_t ngroups) {
  const int lane = threadIdx.x & (kWave - 1);
  const int d = blockIdx.x * kWaves + threadIdx.x / kWave;   // grid = kBins / kWaves blocks
  uint32_t carry = 0;
  for (int64_t g0 = 0; g0 < ngroups; g0 += kWave) {
    const int64_t g = g0 + lane;
    const uint32_t v = g < ngroups ? gcnt[g * kBins + d] : 0u;
    uint32_t incl = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const uint32_t t = __shfl_up(incl, off);
      if (lane >= off) incl += t;
    }
    if (g < ngroups) gcnt[g * kBins + d] = carry + incl - v;
    carry += __shfl(incl, kWave - 1);
  }
  if (lane == 0) gcnt[ngroups * kBins + d] = carry;
}

// ---- one radix pass ---------------------------------------------------------------------
// Tile order: wave w of the block owns tile positions [w*IPT*64, (w+1)*IPT*64), round r of that
// wave the 64 positions from r*64 on.  Ranks are handed out in exactly that order.
template <typename KeyT, bool FIRST, int IPT>
__global__ __launch_bounds__(kThreads) void radix_pass_kernel(
    const void* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, int64_t n, int shift,
    uint32_t mask, int bits, const uint32_t* __restrict__ cnt_cur,
    const uint32_t* __restrict__ gcnt, int64_t ngroups, int scanned, KeyT* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out) {
  __shared__ uint32_t s_cnt[kWaves][kBins];
  __shared__ uint32_t s_glob[kBins];
  __shared__ uint32_t s_scan[kWaves + 1];
  __shared__ uint32_t s_pre[kWaves][kBins];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;

  // the tile's keys are requested first, so that their latency overlaps the column sums
  const int64_t wave0 = static_cast<int64_t>(blockIdx.x) * (kThreads * IPT) + wave * (IPT * kWave);
  KeyT key[IPT];
  uint32_t val[IPT];
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = wave0 + r * kWave + lane;
    const bool valid = i < n;
    key[r] = valid ? load_key<KeyT, FIRST>(keys_in, i) : KeyT(0);
    val[r] = valid ? (FIRST ? static_cast<uint32_t>(i) : vals_in[i]) : 0u;
  }

  // global offset of (digit, this tile): all keys with a smaller digit, plus the keys with this
  // digit in the tiles before this one.  Thread d owns digit d (kThreads == kBins).
  // Rows to add up, unscanned counts: one per group of tiles (all of them for the totals, those
  // before this tile's group for the prefix), then the tile rows of this group before this tile.
  // Scanned counts (large batches, radix_group_scan_kernel has run): the totals row, the prefix
  // row of this tile's group, then the same tile rows - at most five rows whatever the batch.
  // The sums are latency-bound: wave w takes the rows v = w (mod kWaves), lane l the four digits
  // 4l..4l+3 of a row as one 16-byte load, sixteen rows in flight.
  {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    constexpr int kInFlight = 16;
    const int64_t me = blockIdx.x;
    const int64_t my_group = me / kGroup;
    const int64_t nhead = scanned ? 2 : ngroups;   // rows that come from gcnt
    const int64_t nrows = nhead + (me - my_group * kGroup);
    u32x4 tot4 = {0, 0, 0, 0}, pre4 = {0, 0, 0, 0};
    for (int64_t v0 = wave; v0 < nrows; v0 += kWaves * kInFlight) {
      u32x4 h[kInFlight];
#pragma unroll
      for (int k = 0; k < kInFlight; ++k) {
        const int64_t v = v0 + static_cast<int64_t>(k) * kWaves;
        const int64_t head_row = scanned ? (v == 0 ? ngroups : my_group) : v;
        const uint32_t* row = v < nhead ? gcnt + head_row * kBins
                                        : cnt_cur + (my_group * kGroup + (v - nhead)) * kBins;
        h[k] = v < nrows ? reinterpret_cast<const u32x4*>(row)[lane] : u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int k = 0; k < kInFlight; ++k) {
        const int64_t v = v0 + static_cast<int64_t>(k) * kWaves;
        const bool to_tot = scanned ? v == 0 : v < ngroups;
        const bool to_pre = scanned ? v >= 1 : (v < my_group || v >= ngroups);
        if (to_tot) tot4 += h[k];
        if (to_pre) pre4 += h[k];
      }
    }
    // s_cnt doubles as scratch here: rows 0..3 hold the per-wave totals; the per-wave prefixes
    // go to s_pre.  Both are folded over the waves by the thread that owns the digit.
    reinterpret_cast<u32x4*>(&s_cnt[wave][0])[lane] = tot4;
    reinterpret_cast<u32x4*>(&s_pre[wave][0])[lane] = pre4;
    __syncthreads();
    const int d = threadIdx.x;
    uint32_t tot = 0, pre = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      tot += s_cnt[w][d];
      pre += s_pre[w][d];
    }
    uint32_t total;
    const uint32_t base = block_exclusive_sum<uint32_t, kThreads>(tot, s_scan, &total);
    s_glob[d] = base + pre;
    __syncthreads();
    for (int i = threadIdx.x; i < kWaves * kBins; i += kThreads) (&s_cnt[0][0])[i] = 0;
  }
  __syncthreads();

  uint32_t rank[IPT];
  const uint64_t lt_mask = (uint64_t(1) << lane) - 1;
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = wave0 + r * kWave + lane;
    const bool valid = i < n;
    const uint32_t d = static_cast<uint32_t>(key[r] >> shift) & mask;
    const uint64_t peers = match_any(d, bits, __ballot(valid));
    uint32_t old = 0;
    if (valid) old = s_cnt[wave][d];
    // every peer has read the counter before the leader bumps it: LDS operations of one wave
    // complete in program order
    __builtin_amdgcn_wave_barrier();
    if (valid && (peers & lt_mask) == 0) s_cnt[wave][d] = old + __popcll(peers);
    rank[r] = old + __popcll(peers & lt_mask);
  }
  __syncthreads();
  // exclusive prefix over the waves, per digit
  {
    const int d = threadIdx.x;
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

// ---- the one-sweep sort ---------------------------------------------------------------------
// One histogram kernel counts the digits of ALL passes in one read of the ids, one small kernel
// turns the totals into per-pass digit bases, and then every pass is ONE kernel: a tile ranks its
// keys, publishes its digit counts, obtains the counts of the tiles before it by looking back at
// what they published, and scatters.  A pass costs one launch instead of two or three.
//
// A tile's state is one 32-bit word per digit: status in the two top bits (0 nothing yet, 1 the
// tile's own count, 2 the count of this tile and all tiles before it), the count below.  The word
// is read and written whole, so a reader needs no fence: whatever it sees is self-consistent.
//
// Every wait is bounded.  A tile waits only for tiles with a smaller block index, which the
// dispatcher starts earlier; it re-reads their state at most `spin_limit` times and then stops
// waiting and counts the digits of every key before its own tile straight from the pass's input -
// which needs no other block - bumps a counter of such events in the workspace, and carries on
// with the same result.  The sort is correct whatever the order blocks run in; only its speed
// relies on that order.
constexpr uint32_t kStatusShift = 30;
constexpr uint32_t kCountMask = (1u << kStatusShift) - 1u;
constexpr uint32_t kHasOwn = 1u << kStatusShift;
constexpr uint32_t kHasAll = 2u << kStatusShift;
constexpr int kLookback = 8;        // predecessor states a thread requests at a time
constexpr int kHistThreads = 1024;  // the histogram kernel's block
constexpr int kHistItems = 8;       // keys per thread of the histogram kernel: chunks of 8192 keys
constexpr int kHistChunk = kHistThreads * kHistItems;
constexpr int kSweepStatusWords = 64;   // head of the workspace: [0] tiles whose wait ran out

__device__ __forceinline__ uint32_t load_state(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_state(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct SweepDigits {
  int passes;
  int shift[kMaxPasses];
  uint32_t mask[kMaxPasses];
};

// digit counts of every pass over one chunk of the ids; also clears what the pass kernels and the
// run kernel expect cleared (tile states of pass 0, run-tile states, the event counter) and
// writes the id-bound flags
template <typename KeyT>
__global__ __launch_bounds__(kHistThreads) void sweep_hist_kernel(
    const int64_t* __restrict__ ids, int64_t n, SweepDigits dg, uint32_t* __restrict__ hist_part,
    int64_t id_bound, int32_t* __restrict__ bad_blk, int64_t nbad, uint32_t* __restrict__ clear0,
    int64_t clear0_words, uint32_t* __restrict__ clear1, int64_t clear1_words,
    uint32_t* __restrict__ status) {
  __shared__ uint32_t s_hist[kMaxPasses][kBins];
  for (int i = threadIdx.x; i < dg.passes * kBins; i += kHistThreads) (&s_hist[0][0])[i] = 0;
  const int64_t c0 = static_cast<int64_t>(blockIdx.x) * kHistChunk;
  int64_t idv[kHistItems];
#pragma unroll
  for (int r = 0; r < kHistItems; ++r) {
    const int64_t i = c0 + r * kHistThreads + threadIdx.x;
    idv[r] = i < n ? ids[i] : int64_t(0);
  }
  __syncthreads();
  bool bad = false;
#pragma unroll
  for (int r = 0; r < kHistItems; ++r) {
    const int64_t i = c0 + r * kHistThreads + threadIdx.x;
    if (i < n) {
      const int64_t id = idv[r];
      bad = bad || (id_bound > 0 && (id < 0 || id >= id_bound));
      const KeyT k = key_from_id<KeyT>(id);
      for (int p = 0; p < dg.passes; ++p)
        atomicAdd(&s_hist[p][static_cast<uint32_t>(k >> dg.shift[p]) & dg.mask[p]], 1u);
    }
  }
  const int any_bad = __syncthreads_or(bad ? 1 : 0);
  if (threadIdx.x == 0) bad_blk[blockIdx.x] = any_bad;
  // flags past the last chunk belong to nobody: block 0 writes them, so that a reader of all
  // nbad flags never sees a stale one
  if (blockIdx.x == 0)
    for (int64_t b = gridDim.x + threadIdx.x; b < nbad; b += kHistThreads) bad_blk[b] = 0;
  for (int i = threadIdx.x; i < dg.passes * kBins; i += kHistThreads)
    hist_part[static_cast<int64_t>(blockIdx.x) * dg.passes * kBins + i] = (&s_hist[0][0])[i];
  // clearing, spread over the grid
  const int64_t per0 = (clear0_words + gridDim.x - 1) / gridDim.x;
  const int64_t per1 = (clear1_words + gridDim.x - 1) / gridDim.x;
  for (int64_t i = blockIdx.x * per0 + threadIdx.x; i < (blockIdx.x + 1) * per0 && i < clear0_words;
       i += kHistThreads)
    clear0[i] = 0;
  for (int64_t i = blockIdx.x * per1 + threadIdx.x; i < (blockIdx.x + 1) * per1 && i < clear1_words;
       i += kHistThreads)
    clear1[i] = 0;
  if (blockIdx.x == 0 && threadIdx.x < kSweepStatusWords) status[threadIdx.x] = 0;
}

// bases[p][d] = keys of the whole batch whose digit in pass p is below d.  One block per pass;
// thread (g, d) adds up the chunk rows g, g + 4, ... of digit d, eight loads in flight.
__global__ __launch_bounds__(kHistThreads) void sweep_bases_kernel(const uint32_t* __restrict__ hist_part,
                                                                  int64_t nchunks, int passes,
                                                                  uint32_t* __restrict__ bases) {
  constexpr int kParts = kHistThreads / kBins;
  __shared__ uint32_t s_part[kParts][kBins];
  __shared__ uint32_t s_scan[kHistThreads / kWave + 1];
  const int p = blockIdx.x, d = threadIdx.x % kBins, g = threadIdx.x / kBins;
  uint32_t tot = 0;
  for (int64_t c0 = g; c0 < nchunks; c0 += 8 * kParts) {
    uint32_t v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int64_t c = c0 + static_cast<int64_t>(k) * kParts;
      v[k] = c < nchunks ? hist_part[(c * passes + p) * kBins + d] : 0u;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) tot += v[k];
  }
  s_part[g][d] = tot;
  __syncthreads();
  uint32_t sum = 0;
  if (g == 0) {
#pragma unroll
    for (int k = 0; k < kParts; ++k) sum += s_part[k][d];
  }
  uint32_t total;    // threads beyond the first kBins add nothing and come after them in the scan
  const uint32_t ex = block_exclusive_sum<uint32_t, kHistThreads>(sum, s_scan, &total);
  if (g == 0) bases[p * kBins + d] = ex;
}

// one pass of the one-sweep sort; tile order and ranks exactly as in radix_pass_kernel, so both
// sorts give the same permutation
template <typename KeyT, bool FIRST, int IPT>
__global__ __launch_bounds__(kThreads) void sweep_pass_kernel(
    const void* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, int64_t n, int shift,
    uint32_t mask, int bits, const uint32_t* __restrict__ bases, uint32_t* __restrict__ state,
    uint32_t* __restrict__ next_state, int spin_limit, uint32_t* __restrict__ status,
    KeyT* __restrict__ keys_out, uint32_t* __restrict__ vals_out) {
  __shared__ uint32_t s_cnt[kWaves][kBins];
  __shared__ uint32_t s_glob[kBins];
  __shared__ int s_gave_up;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t tile = blockIdx.x;
  const int64_t tile0 = tile * (kThreads * IPT);
  const int64_t wave0 = tile0 + wave * (IPT * kWave);
  KeyT key[IPT];
  uint32_t val[IPT];
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = wave0 + r * kWave + lane;
    const bool valid = i < n;
    key[r] = valid ? load_key<KeyT, FIRST>(keys_in, i) : KeyT(0);
    val[r] = valid ? (FIRST ? static_cast<uint32_t>(i) : vals_in[i]) : 0u;
  }
  const int d = threadIdx.x;                    // the digit this thread owns (kThreads == kBins)
  const uint32_t base = bases[d];
  // the states of the NEXT pass live in the other buffer, last used two passes ago: this tile
  // clears its own row of it (the kernel boundary makes that visible to the next pass)
  if (next_state != nullptr) next_state[tile * kBins + d] = 0;
  for (int i = threadIdx.x; i < kWaves * kBins; i += kThreads) (&s_cnt[0][0])[i] = 0;
  if (threadIdx.x == 0) s_gave_up = 0;
  __syncthreads();

  uint32_t rank[IPT];
  const uint64_t lt_mask = (uint64_t(1) << lane) - 1;
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = wave0 + r * kWave + lane;
    const bool valid = i < n;
    const uint32_t dd = static_cast<uint32_t>(key[r] >> shift) & mask;
    const uint64_t peers = match_any(dd, bits, __ballot(valid));
    uint32_t old = 0;
    if (valid) old = s_cnt[wave][dd];
    __builtin_amdgcn_wave_barrier();   // every peer has read the counter before the leader bumps it
    if (valid && (peers & lt_mask) == 0) s_cnt[wave][dd] = old + __popcll(peers);
    rank[r] = old + __popcll(peers & lt_mask);
  }
  __syncthreads();
  // exclusive prefix over the waves per digit; own = this tile's keys with digit d
  uint32_t own = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const uint32_t t = s_cnt[w][d];
    s_cnt[w][d] = own;
    own += t;
  }
  uint32_t* my_state = state + tile * kBins + d;
  uint32_t before = 0;                          // keys with digit d in the tiles before this one
  if (tile == 0) {
    store_state(my_state, kHasAll | own);
  } else {
    store_state(my_state, kHasOwn | own);
    // look back, kLookback tiles at a time; wave-uniform control, no block barrier inside
    int64_t p = tile - 1;
    bool done = false;
    int spins = 0;
    while (true) {
      bool stuck = false;
      if (!done) {
        uint32_t v[kLookback];
#pragma unroll
        for (int k = 0; k < kLookback; ++k)
          v[k] = p - k >= 0 ? load_state(state + (p - k) * kBins + d) : kHasAll;
#pragma unroll
        for (int k = 0; k < kLookback; ++k) {
          if (!done && !stuck) {
            const uint32_t st = v[k] >> kStatusShift;
            if (st == 0) {
              stuck = true;
            } else {
              before += v[k] & kCountMask;
              --p;
              if (st == 2) done = true;
            }
          }
        }
      }
      if (__ballot(!done) == 0) break;
      if (__ballot(stuck) != 0) {
        if (++spins > spin_limit) {
          if (lane == 0) s_gave_up = 1;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
  }
  __syncthreads();
  if (s_gave_up) {
    // the wait ran out: count the digits of every key before this tile from the input itself
    __shared__ uint32_t s_all[kBins];
    s_all[d] = 0;
    __syncthreads();
    for (int64_t i = threadIdx.x; i < tile0; i += kThreads)
      atomicAdd(&s_all[static_cast<uint32_t>(load_key<KeyT, FIRST>(keys_in, i) >> shift) & mask], 1u);
    __syncthreads();
    before = s_all[d];
    if (threadIdx.x == 0) atomicAdd(status, 1u);
  }
  if (tile != 0) store_state(my_state, kHasAll | (before + own));
  s_glob[d] = base + before;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < IPT; ++r) {
    const int64_t i = wave0 + r * kWave + lane;
    if (i < n) {
      const uint32_t dd = static_cast<uint32_t>(key[r] >> shift) & mask;
      const uint32_t pos = s_glob[dd] + s_cnt[wave][dd] + rank[r];
      keys_out[pos] = key[r];
      vals_out[pos] = val[r];
    }
  }
}

// ---- run boundaries ---------------------------------------------------------
constexpr int kUItems = 8;         // sorted positions per thread of the run kernels ...
constexpr int kUItemsSmall = 2;    // ... and for batches of up to kRunsSmallBatch ids: more and shorter
                                   // blocks (whole step with 8 / 4 / 2 positions per thread: cfg1 71.6 /
                                   // 69.9 / 69.3 us, cfg2 159.8 / 158.3 / 158.0, cfg5 331.7 / 323.5 / 319.3).
                                   // Every block adds up the counts of the tiles before it, which is
                                   // quadratic in the number of tiles: larger batches keep larger tiles.
constexpr int64_t kRunsSmallBatch = 1 << 21;
constexpr int kUTile = kThreads * kUItems;

template <typename KeyT, int ITEMS>
__global__ __launch_bounds__(kThreads) void run_count_kernel(const KeyT* __restrict__ keys,
                                                            int64_t n,
                                                            uint32_t* __restrict__ blk_cnt) {
  __shared__ uint32_t smem[kWaves + 1];
  const int64_t j0 = static_cast<int64_t>(blockIdx.x) * (kThreads * ITEMS) + threadIdx.x * ITEMS;
  uint32_t c = 0;
  if (j0 < n) {
    KeyT prev = j0 > 0 ? keys[j0 - 1] : KeyT(0);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
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

template <typename KeyT, int ITEMS>
__global__ __launch_bounds__(kThreads) void run_emit_kernel(
    const KeyT* __restrict__ keys, const uint32_t* __restrict__ perm, int64_t n,
    const uint32_t* __restrict__ blk_cnt, int64_t* __restrict__ uids,
    uint32_t* __restrict__ seg_start, uint32_t* __restrict__ seg_of,
    int64_t* __restrict__ num_unique, int32_t* __restrict__ inverse,
    const int32_t* __restrict__ bad_blk, int64_t nbad, KeyT thr, int64_t* __restrict__ class_split,
    int32_t* __restrict__ first_pos) {
  __shared__ uint32_t smem[kWaves + 1];
  // the block that writes num_unique first learns whether the first count pass saw an id outside
  // [0, id_bound): it then reports -1 distinct ids, which every consumer treats as "no live rows"
  int violated = 0;
  if (blockIdx.x == gridDim.x - 1) {
    for (int64_t b = threadIdx.x; b < nbad; b += kThreads) violated |= bad_blk[b];
    violated = __syncthreads_or(violated);
  }
  // runs that begin in the tiles before this one
  uint32_t before = 0;
  for (int64_t b = threadIdx.x; b < static_cast<int64_t>(blockIdx.x); b += kThreads)
    before += blk_cnt[b];
  uint32_t blk_base;
  (void)block_exclusive_sum<uint32_t, kThreads>(before, smem, &blk_base);

  const int64_t j0 = static_cast<int64_t>(blockIdx.x) * (kThreads * ITEMS) + threadIdx.x * ITEMS;
  uint32_t flag[ITEMS];
  KeyT kk[ITEMS];
  uint32_t c = 0;
  if (j0 < n) {
    KeyT prev = j0 > 0 ? keys[j0 - 1] : KeyT(0);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
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
  uint32_t u = blk_base + block_exclusive_sum<uint32_t, kThreads>(c, smem, &total);
  // u = number of runs that begin before j0
  if (j0 < n) {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int64_t j = j0 + k;
      if (j < n) {
        u += flag[k];
        const uint32_t seg = u - 1;
        seg_of[j] = seg;
        if (inverse) inverse[perm[j]] = static_cast<int32_t>(seg);
        if (flag[k]) {
          uids[seg] = id_from_key<KeyT>(kk[k]);
          seg_start[seg] = static_cast<uint32_t>(j);
          if (first_pos != nullptr) first_pos[seg] = static_cast<int32_t>(perm[j]);
          // the first key at or above the threshold opens the upper class (keys are ascending)
          if (class_split != nullptr && kk[k] >= thr &&
              (j == 0 || (k > 0 ? kk[k - 1] : keys[j - 1]) < thr)) {
            class_split[0] = j;
            class_split[1] = static_cast<int64_t>(seg);
          }
        }
        if (j == n - 1) {
          seg_start[u] = static_cast<uint32_t>(n);
          num_unique[0] = violated ? int64_t(-1) : static_cast<int64_t>(u);
          if (class_split != nullptr && kk[k] < thr) {   // no key reaches the threshold
            class_split[0] = n;
            class_split[1] = static_cast<int64_t>(u);
          }
        }
      }
    }
  }
}

// run boundaries in one kernel: run_count_kernel's count, the number of runs that begin in earlier
// tiles obtained by looking back at what those tiles published (one state word per tile, the
// protocol and the bounded wait of sweep_pass_kernel), then run_emit_kernel's output
template <typename KeyT>
__global__ __launch_bounds__(kThreads) void run_sweep_kernel(
    const KeyT* __restrict__ keys, const uint32_t* __restrict__ perm, int64_t n,
    uint32_t* __restrict__ tile_state, int spin_limit, uint32_t* __restrict__ status,
    int64_t* __restrict__ uids, uint32_t* __restrict__ seg_start, uint32_t* __restrict__ seg_of,
    int64_t* __restrict__ num_unique, int32_t* __restrict__ inverse,
    const int32_t* __restrict__ bad_blk, int64_t nbad, KeyT thr, int64_t* __restrict__ class_split,
    int32_t* __restrict__ first_pos) {
  __shared__ uint32_t smem[kWaves + 1];
  __shared__ uint32_t s_base;
  __shared__ int s_gave_up;
  const int lane = threadIdx.x & (kWave - 1);
  int violated = 0;
  if (blockIdx.x == gridDim.x - 1) {
    for (int64_t b = threadIdx.x; b < nbad; b += kThreads) violated |= bad_blk[b];
    violated = __syncthreads_or(violated);
  }
  const int64_t tile = blockIdx.x;
  const int64_t j0 = tile * kUTile + threadIdx.x * kUItems;
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
  const uint32_t local = block_exclusive_sum<uint32_t, kThreads>(c, smem, &total);
  if (threadIdx.x == 0) s_gave_up = 0;
  __syncthreads();
  // wave 0: publish, look back 64 tiles at a time, publish again
  if (threadIdx.x < kWave) {
    uint32_t before = 0;
    if (tile == 0) {
      if (lane == 0) store_state(tile_state, kHasAll | total);
    } else {
      if (lane == 0) store_state(tile_state + tile, kHasOwn | total);
      int64_t p = tile - 1;
      int spins = 0;
      bool gave_up = false;
      while (true) {
        const uint32_t v = p - lane >= 0 ? load_state(tile_state + (p - lane)) : kHasAll;
        const uint32_t st = v >> kStatusShift;
        const uint64_t all_m = __ballot(st == 2), none_m = __ballot(st == 0);
        // the nearest tile that knows everything before it, and whether every tile nearer than
        // that has at least published its own count
        const int first_all = all_m ? __builtin_ctzll(all_m) : kWave;
        const int first_none = none_m ? __builtin_ctzll(none_m) : kWave;
        const int upto = first_all < first_none ? first_all + 1 : first_none;   // lanes [0, upto) count
        uint32_t part = lane < upto ? (v & kCountMask) : 0u;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off);
        before += part;
        p -= upto;
        if (first_all < first_none) break;
        if (first_none < kWave) {               // a tile in the window has published nothing yet
          if (++spins > spin_limit) { gave_up = true; break; }
          __builtin_amdgcn_s_sleep(1);
        }
      }
      if (gave_up && lane == 0) s_gave_up = 1;
    }
    if (lane == 0) s_base = before;
  }
  __syncthreads();
  if (s_gave_up) {
    // the wait ran out: count the runs that begin before this tile from the keys themselves
    uint32_t cnt = 0;
    for (int64_t j = threadIdx.x; j < tile * kUTile && j < n; j += kThreads)
      cnt += (j == 0 || keys[j] != keys[j - 1]) ? 1u : 0u;
    uint32_t tot2;
    (void)block_exclusive_sum<uint32_t, kThreads>(cnt, smem, &tot2);
    if (threadIdx.x == 0) {
      s_base = tot2;
      atomicAdd(status, 1u);
    }
    __syncthreads();
  }
  const uint32_t blk_base = s_base;
  if (threadIdx.x == 0 && tile != 0) store_state(tile_state + tile, kHasAll | (blk_base + total));
  uint32_t u = blk_base + local;   // runs that begin before j0
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
          if (first_pos != nullptr) first_pos[seg] = static_cast<int32_t>(perm[j]);
          if (class_split != nullptr && kk[k] >= thr &&
              (j == 0 || (k > 0 ? kk[k - 1] : keys[j - 1]) < thr)) {
            class_split[0] = j;
            class_split[1] = static_cast<int64_t>(seg);
          }
        }
        if (j == n - 1) {
          seg_start[u] = static_cast<uint32_t>(n);
          num_unique[0] = violated ? int64_t(-1) : static_cast<int64_t>(u);
          if (class_split != nullptr && kk[k] < thr) {
            class_split[0] = n;
            class_split[1] = static_cast<int64_t>(u);
          }
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

constexpr int kLongRun = 64;     // EXACT: shortest run that is summed by a block of its own
constexpr int kChunk = 32;       // sorted positions per lane group (large batches; see seg_chunk_for)
constexpr int kMinGroup = 4;     // lanes per group: power of two in [4, 64]
constexpr int kMaxGroups = kThreads / kMinGroup;
constexpr int kSegUnroll = 16;   // row loads in flight per lane
constexpr uint32_t kNoRun = 0xffffffffu;

struct SegArgs {
  const float* grad;
  const uint32_t* perm;
  const uint32_t* seg_of;
  const uint32_t* seg_start;
  const int64_t* num_unique;
  float* sums;
  int64_t* cnts;
  float* partial;  // [2 * nblocks][dim]: head and tail partial row of every block
  int64_t n;
  int64_t dim;
  int group;       // lanes per group
  int col_tiles;   // ceil(dim / (group * VEC))
  // optional restriction to one class of a class-ordered plan: class_split = {first sorted
  // position, first run} of the upper class; which = 0 lower class, 1 upper class, -1 everything
  const int64_t* class_split;
  int which;
  // EXACT with a staging area (else null): see seg_stage_kernel
  float* stage = nullptr;
  uint32_t* long_list = nullptr;
};

// [*pos_lo, *pos_hi) sorted positions and [*run_lo, *run_hi) runs of the class a launch works on
__device__ __forceinline__ void class_range(const SegArgs& a, int64_t U, int64_t* pos_lo,
                                            int64_t* pos_hi, int64_t* run_lo, int64_t* run_hi) {
  *pos_lo = 0; *pos_hi = a.n; *run_lo = 0; *run_hi = U;
  if (a.class_split != nullptr && a.which >= 0) {
    const int64_t sp = a.class_split[0], sr = a.class_split[1];
    if (a.which == 0) { *pos_hi = sp; *run_hi = sr < U ? sr : U; }
    else { *pos_lo = sp; *run_lo = sr; }
  }
}

// FAST, kernel 1.  A block covers (kThreads / group) * CH consecutive sorted positions.
template <int VEC, int CH>
__global__ __launch_bounds__(kThreads) void seg_chunk_kernel(SegArgs a) {
  typedef typename RowVec<VEC>::type V;
  constexpr int kUnroll = CH < kSegUnroll ? CH : kSegUnroll;   // row loads in flight per lane
  __shared__ uint32_t s_perm[kMaxGroups * CH];
  __shared__ uint32_t s_seg[kMaxGroups * CH + 2];   // s_seg[1 + t] = run of position B0 + t
  __shared__ V s_part[kThreads * 2];                    // [group][first|last][lane]
  __shared__ uint32_t s_first[kMaxGroups], s_last[kMaxGroups];
  __shared__ uint8_t s_flags[kMaxGroups];               // 1 head open, 2 tail open, 4 active

  const int G = a.group;
  const int ngroups = kThreads / G;
  const int bp = ngroups * CH;
  const int64_t B0 = static_cast<int64_t>(blockIdx.x) * bp;
  // runs [run_lo, run_hi) are this launch's to write
  uint32_t run_lo = 0, run_hi = kNoRun;
  if (a.class_split != nullptr && a.which >= 0) {
    // a block works if its span touches the class; the block that straddles the class border
    // walks its whole span but writes only the runs of its class (runs never cross that border):
    // the other class may be summed by another kernel at the same time
    const int64_t sp = a.class_split[0];
    if (a.which == 0 ? B0 >= sp : B0 + bp <= sp) return;
    const uint32_t sr = static_cast<uint32_t>(a.class_split[1]);
    if (a.which == 0) run_hi = sr; else run_lo = sr;
  }
  for (int t = threadIdx.x; t < bp + 2; t += kThreads) {
    const int64_t j = B0 - 1 + t;
    s_seg[t] = (j >= 0 && j < a.n) ? a.seg_of[j] : kNoRun;
  }
  for (int t = threadIdx.x; t < bp; t += kThreads) {
    const int64_t j = B0 + t;
    s_perm[t] = j < a.n ? a.perm[j] : 0u;
  }
  __syncthreads();

  const int g = threadIdx.x / G;
  const int gl = threadIdx.x & (G - 1);
  const int t0 = g * CH;                       // block-relative first position of the group
  const int64_t left = a.n - (B0 + t0);
  const int len = left >= CH ? CH : (left > 0 ? static_cast<int>(left) : 0);
  const bool active = len > 0;
  const uint32_t first_run = s_seg[1 + t0];
  const uint32_t last_run = active ? s_seg[t0 + len] : kNoRun;
  const bool head_open = active && s_seg[t0] == first_run;
  const bool tail_open = active && s_seg[1 + t0 + len] == last_run;
  if (gl == 0) {
    s_first[g] = first_run;
    s_last[g] = last_run;
    s_flags[g] = (head_open ? 1 : 0) | (tail_open ? 2 : 0) | (active ? 4 : 0);
  }

  for (int ct = 0; ct < a.col_tiles; ++ct) {
    const int64_t col = (static_cast<int64_t>(ct) * G + gl) * VEC;
    const bool col_ok = col < a.dim;
    V acc = RowVec<VEC>::zero();
    uint32_t cur = first_run;
    for (int tt = 0; tt < len; tt += kUnroll) {
      V row[kUnroll];
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        // clamped, so that every slot loads a valid row and the loads form one straight run of
        // instructions; gradient rows are read exactly once: non-temporal loads keep them from
        // displacing the table rows the neighbouring kernels reuse (measured 41.6 -> 32.0 us)
        const int kk = (tt + k < len) ? tt + k : len - 1;
        const int64_t p = s_perm[t0 + kk];
        row[k] = col_ok ? __builtin_nontemporal_load(
                              reinterpret_cast<const V*>(a.grad + p * a.dim + col))
                        : RowVec<VEC>::zero();
      }
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        if (tt + k < len) {
          const uint32_t seg = s_seg[1 + t0 + tt + k];
          if (seg != cur) {
            // run `cur` ends inside this group: whole unless it is the first run and began earlier
            if (cur == first_run && head_open) {
              s_part[(g * 2 + 0) * G + gl] = acc;
            } else if (col_ok && cur >= run_lo && cur < run_hi) {
              *reinterpret_cast<V*>(a.sums + static_cast<int64_t>(cur) * a.dim + col) = acc;
            }
            acc = RowVec<VEC>::zero();
            cur = seg;
          }
          acc += row[k];
        }
      }
    }
    if (active) {
      // the last run of the group
      const bool mine = col_ok && cur >= run_lo && cur < run_hi;
      if (cur == first_run) {
        if (!head_open && !tail_open) {
          if (mine) *reinterpret_cast<V*>(a.sums + static_cast<int64_t>(cur) * a.dim + col) = acc;
        } else {
          s_part[(g * 2 + 0) * G + gl] = acc;
        }
      } else if (!tail_open) {
        if (mine) *reinterpret_cast<V*>(a.sums + static_cast<int64_t>(cur) * a.dim + col) = acc;
      } else {
        s_part[(g * 2 + 1) * G + gl] = acc;
      }
    }
    __syncthreads();
    // merge, in group order, the runs that cross group borders inside this block (group 0 only)
    if (g == 0) {
      V carry = RowVec<VEC>::zero();
      uint32_t carry_run = kNoRun;
      bool carry_on = false, carry_head = false, carry_outside = false;
      for (int gg = 0; gg < ngroups; ++gg) {
        const uint8_t f = s_flags[gg];
        if (!(f & 4)) break;
        const bool fo = f & 1, to = f & 2;
        const bool single = s_first[gg] == s_last[gg];
        if (fo || (single && to)) {                 // the first run of group gg is not whole
          const V part = s_part[(gg * 2 + 0) * G + gl];
          if (fo && gg > 0) {
            carry += part;                          // continues the run carried in from gg-1
          } else {
            carry = part;
            carry_run = s_first[gg];
            carry_head = gg == 0;
            carry_outside = fo;
            carry_on = true;
          }
          if (!(single && to)) {                    // ... and it ends inside group gg
            const bool to_partial = carry_head && carry_outside;
            float* out = to_partial ? a.partial + (2 * static_cast<int64_t>(blockIdx.x)) * a.dim
                                    : a.sums + static_cast<int64_t>(carry_run) * a.dim;
            if (col_ok && (to_partial || (carry_run >= run_lo && carry_run < run_hi)))
              *reinterpret_cast<V*>(out + col) = carry;
            carry_on = false;
          }
        }
        if (!single && to) {                        // the last run of group gg goes on into gg+1
          carry = s_part[(gg * 2 + 1) * G + gl];
          carry_run = s_last[gg];
          carry_head = false;
          carry_outside = false;
          carry_on = true;
        }
      }
      if (carry_on) {                               // the run goes on into the next block
        float* out = a.partial + (2 * static_cast<int64_t>(blockIdx.x) + (carry_head ? 0 : 1)) * a.dim;
        if (col_ok) *reinterpret_cast<V*>(out + col) = carry;
      }
    }
    __syncthreads();
  }
}

// FAST, kernel 2: block c finishes the run that begins in block c's span and crosses into the
// next one, adding the per-block partial rows in block order (lane groups take partials
// round-robin, then group 0 adds the per-group sums in group order).  Also writes the counts.
template <int VEC, int CH>
__global__ __launch_bounds__(kThreads) void seg_fixup_kernel(SegArgs a) {
  typedef typename RowVec<VEC>::type V;
  __shared__ V s_part[kThreads];
  const int64_t U = a.num_unique[0];
  int64_t pos_lo, pos_hi, run_lo, run_hi;
  class_range(a, U, &pos_lo, &pos_hi, &run_lo, &run_hi);
  const int64_t gtid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (gtid >= run_lo && gtid < run_hi)
    a.cnts[gtid] = static_cast<int64_t>(a.seg_start[gtid + 1]) - static_cast<int64_t>(a.seg_start[gtid]);

  const int G = a.group;
  const int ngroups = kThreads / G;
  const int64_t span = static_cast<int64_t>(ngroups) * CH;
  const int64_t c = blockIdx.x;
  const int64_t border = (c + 1) * span;
  if (border >= a.n) return;
  if (border - 1 < pos_lo || border >= pos_hi) return;   // both sides of the border in the class
  const uint32_t u = a.seg_of[border - 1];
  if (a.seg_of[border] != u) return;           // no run crosses this border
  const int64_t start = a.seg_start[u];
  if (start < c * span) return;                 // the run began earlier: an earlier block owns it
  const int64_t end = a.seg_start[u + 1];
  const int64_t c_last = (end - 1) / span;
  const int64_t nparts = c_last - c + 1;
  const int g = threadIdx.x / G;
  const int gl = threadIdx.x & (G - 1);
  // block c keeps its share in the tail slot unless the run opens the block
  const int64_t first_slot = (start == c * span) ? 2 * c : 2 * c + 1;

  for (int ct = 0; ct < a.col_tiles; ++ct) {
    const int64_t col = (static_cast<int64_t>(ct) * G + gl) * VEC;
    const bool col_ok = col < a.dim;
    V acc = RowVec<VEC>::zero();
    for (int64_t t0 = g; t0 < nparts; t0 += static_cast<int64_t>(ngroups) * 8) {
      V row[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int64_t t = t0 + static_cast<int64_t>(k) * ngroups;
        if (t < nparts) {
          const int64_t slot = t == 0 ? first_slot : 2 * (c + t);
          row[k] = col_ok ? *reinterpret_cast<const V*>(a.partial + slot * a.dim + col)
                          : RowVec<VEC>::zero();
        }
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int64_t t = t0 + static_cast<int64_t>(k) * ngroups;
        if (t < nparts) acc += row[k];
      }
    }
    __syncthreads();
    s_part[threadIdx.x] = acc;
    __syncthreads();
    if (g == 0) {
      V tot = s_part[gl];
      for (int gg = 1; gg < ngroups; ++gg) tot += s_part[gg * G + gl];
      if (col_ok) *reinterpret_cast<V*>(a.sums + static_cast<int64_t>(u) * a.dim + col) = tot;
    }
  }
}

// EXACT: strictly left to right from +0.0f, one accumulator chain per id.
// Runs shorter than kLongRun: one lane group per distinct id.  Longer runs (a heavy-hitter id can
// have tens of thousands of occurrences) are left to seg_exact_long_kernel.
constexpr int kLongThreads = 1024;  // the long-run kernel's block: one CU has to pull a whole run
                                    // through, so it keeps as many row loads in flight as it can
constexpr int kLongRows = 8;    // rows every lane group stages per batch in the long-run kernel
constexpr int kLongSlice = 32;  // floats of a row one block of the long-run kernel sums (128 bytes)

template <int VEC>
__device__ __forceinline__ void exact_short_runs(const SegArgs& a, int64_t block) {
  typedef typename RowVec<VEC>::type V;
  const int64_t U = a.num_unique[0];
  const int64_t gtid = block * kThreads + threadIdx.x;
  const int64_t u = gtid / a.group;
  const int gl = static_cast<int>(gtid & (a.group - 1));
  int64_t pos_lo, pos_hi, run_lo, run_hi;
  class_range(a, U, &pos_lo, &pos_hi, &run_lo, &run_hi);
  if (u < run_lo || u >= run_hi) return;
  const int64_t j0 = a.seg_start[u];
  const int64_t j1 = a.seg_start[u + 1];
  if (gl == 0) a.cnts[u] = j1 - j0;
  if (j1 - j0 >= kLongRun) return;
  for (int ct = 0; ct < a.col_tiles; ++ct) {
    const int64_t col = (static_cast<int64_t>(ct) * a.group + gl) * VEC;
    if (col >= a.dim) continue;
    V acc = RowVec<VEC>::zero();
    for (int64_t jj = j0; jj < j1; jj += 8) {
      V row[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (jj + k < j1) {
          const int64_t p = a.perm[jj + k];
          row[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(a.grad + p * a.dim + col));
        }
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (jj + k < j1) acc += row[k];
      }
    }
    *reinterpret_cast<V*>(a.sums + u * a.dim + col) = acc;
  }
}

template <int VEC>
__global__ __launch_bounds__(kThreads) void seg_exact_kernel(SegArgs a) {
  exact_short_runs<VEC>(a, blockIdx.x);
}

// EXACT, long runs: block c takes the run that begins inside positions [c*kLongRun, (c+1)*kLongRun)
// and is at least kLongRun long (there is at most one: it must cover the last position of that
// span).  All lane groups of the block stage rows into LDS, kLongRows each per batch, with the
// next batch's loads already in flight; one thread per float column adds the staged rows in order,
// so every element's sum is the same single chain ((0 + g1) + g2) + ... as for a short run.
template <int VEC>
__global__ __launch_bounds__(kLongThreads) void seg_exact_long_kernel(SegArgs a) {
  typedef typename RowVec<VEC>::type V;
  extern __shared__ __align__(16) unsigned char s_raw[];
  V* s_rows = reinterpret_cast<V*>(s_raw);   // [rows of a batch][kLongSlice floats]
  const int64_t c = blockIdx.x;
  const int64_t span0 = c * kLongRun;
  if (span0 >= a.n) return;
  const int64_t last = (span0 + kLongRun - 1 < a.n) ? span0 + kLongRun - 1 : a.n - 1;
  const uint32_t u = a.seg_of[last];
  const int64_t start = a.seg_start[u];
  const int64_t end = a.seg_start[u + 1];
  if (start < span0 || end - start < kLongRun) return;
  if (a.class_split != nullptr && a.which >= 0) {
    const int64_t sp = a.class_split[0];
    if (a.which == 0 ? start >= sp : start < sp) return;
  }

  // A block takes a 32-float slice of the columns (blockIdx.y): every element's chain is
  // independent of the other columns, and one CU alone cannot pull whole rows of a long run fast
  // enough, so the slices of a run are summed on different CUs at once.
  constexpr int G = kLongSlice / VEC;          // lanes per row slice
  constexpr int ngroups = kLongThreads / G;
  constexpr int batch = ngroups * kLongRows;
  const int g = threadIdx.x / G;
  const int gl = threadIdx.x & (G - 1);
  const int64_t col = static_cast<int64_t>(blockIdx.y) * kLongSlice + gl * VEC;
  const bool col_ok = col < a.dim;
  // the adders: thread t < kLongSlice owns one float column of the slice and adds the staged
  // rows in order - one dependent add per row and lane
  const float* s_f = reinterpret_cast<const float*>(s_raw);
  float accf = 0.f;
  V row[kLongRows];
  // rows of a batch are dealt to the groups in blocks of kLongRows: group g stages batch rows
  // [g*kLongRows, (g+1)*kLongRows)
  // Two loads deep: while batch b is added, the rows of batch b+1 and the sort positions of
  // batch b+2 are in flight.
  uint32_t pos[kLongRows];
  auto load_pos = [&](int64_t base) {
#pragma unroll
    for (int k = 0; k < kLongRows; ++k) {
      int64_t j = base + g * kLongRows + k;
      if (j >= end) j = end - 1;
      pos[k] = a.perm[j];
    }
  };
  auto issue_rows = [&]() {
#pragma unroll
    for (int k = 0; k < kLongRows; ++k)
      row[k] = col_ok ? __builtin_nontemporal_load(reinterpret_cast<const V*>(
                            a.grad + static_cast<int64_t>(pos[k]) * a.dim + col))
                      : RowVec<VEC>::zero();
  };
  load_pos(start);
  issue_rows();
  load_pos(start + batch);
  for (int64_t base = start; base < end; base += batch) {
#pragma unroll
    for (int k = 0; k < kLongRows; ++k) s_rows[(g * kLongRows + k) * G + gl] = row[k];
    __syncthreads();
    if (base + batch < end) {
      issue_rows();
      load_pos(base + 2 * batch);
    }
    if (threadIdx.x < kLongSlice) {
      const int64_t left = end - base;
      const int rows_here = left < batch ? static_cast<int>(left) : batch;
      int r = 0;
      for (; r + 16 <= rows_here; r += 16) {   // LDS reads issued 16 at a time, adds in order
        float t[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) t[k] = s_f[(r + k) * kLongSlice + threadIdx.x];
#pragma unroll
        for (int k = 0; k < 16; ++k) accf += t[k];
      }
      for (; r < rows_here; ++r) accf += s_f[r * kLongSlice + threadIdx.x];
    }
    __syncthreads();
  }
  if (threadIdx.x < kLongSlice) {
    const int64_t c_out = static_cast<int64_t>(blockIdx.y) * kLongSlice + threadIdx.x;
    if (c_out < a.dim) a.sums[static_cast<int64_t>(u) * a.dim + c_out] = accf;
  }
}

// EXACT, long runs, with a staging area.  One compute unit pulls random rows out of HBM at about a
// hundred cache lines a microsecond, a chain of dependent adds could take five times as many rows:
// a block that fetches the rows of its run itself (seg_exact_long_kernel) is bound by its loads,
// however many it keeps in flight.  So the rows of all long runs are first copied by the whole
// chip, in sorted order, into column slices of four floats: stage[s][j] (16 bytes) = columns
// 4s .. 4s + 3 of the row at sorted position j.  A (run, slice) pair is then one contiguous stream
// in which a cache line carries eight rows, and the block that sums it is bound by its adds.
// The kernel also lists the long runs: long_list[0] runs of kVeryLongRun rows or more from entry 2
// upwards, long_list[1] shorter ones from the last entry downwards, each in no particular order
// (every run is summed on its own).  seg_chain_kernel's blocks take the entries in that order, so
// the runs that decide its length are begun first.
constexpr int64_t kVeryLongRun = 2048;

constexpr int kStagePieces = 4;   // 16-byte pieces per thread: four chains of dependent loads in flight

__global__ __launch_bounds__(kThreads) void seg_stage_kernel(SegArgs a) {
  const int64_t pieces = a.dim / 4;
  int64_t pos_lo, pos_hi, run_lo, run_hi;
  class_range(a, a.num_unique[0], &pos_lo, &pos_hi, &run_lo, &run_hi);
  const int64_t gid0 = static_cast<int64_t>(blockIdx.x) * (kThreads * kStagePieces) + threadIdx.x;
  int64_t j[kStagePieces], sl[kStagePieces];
  uint32_t u[kStagePieces], p[kStagePieces];
  bool live[kStagePieces];
#pragma unroll
  for (int k = 0; k < kStagePieces; ++k) {
    const int64_t gid = gid0 + k * kThreads;
    j[k] = gid / pieces;
    sl[k] = gid - j[k] * pieces;
    live[k] = j[k] >= pos_lo && j[k] < pos_hi;
    u[k] = live[k] ? a.seg_of[j[k]] : 0u;
    p[k] = live[k] ? a.perm[j[k]] : 0u;
  }
  int64_t start[kStagePieces];
#pragma unroll
  for (int k = 0; k < kStagePieces; ++k) {
    start[k] = live[k] ? a.seg_start[u[k]] : 0;
    const int64_t end = live[k] ? a.seg_start[u[k] + 1] : 0;
    live[k] = live[k] && end - start[k] >= kLongRun;
    if (live[k] && sl[k] == 0 && j[k] == start[k]) {
      if (end - start[k] >= kVeryLongRun) {
        a.long_list[2 + atomicAdd(&a.long_list[0], 1u)] = u[k];
      } else {
        const int64_t last_entry = 1 + (a.n + kLongRun - 1) / kLongRun;
        a.long_list[last_entry - atomicAdd(&a.long_list[1], 1u)] = u[k];
      }
    }
  }
  f32x4 v[kStagePieces];
#pragma unroll
  for (int k = 0; k < kStagePieces; ++k)
    if (live[k])
      v[k] = __builtin_nontemporal_load(
          reinterpret_cast<const f32x4*>(a.grad + static_cast<int64_t>(p[k]) * a.dim) + sl[k]);
#pragma unroll
  for (int k = 0; k < kStagePieces; ++k)
    if (live[k]) reinterpret_cast<f32x4*>(a.stage)[sl[k] * a.n + j[k]] = v[k];
}

// Sums the staged slice `sl` of the long runs `first`, `first + stride`, ... of the list, in order of
// occurrence from +0.0f.  All threads copy the stream into LDS, transposed (one array per column),
// 512 rows a batch, two batches of loads in flight and two LDS buffers; threads 0..3 own a column
// each and add it with 16-byte LDS loads (four rows), the loads of the next 32 rows in flight
// while 32 are added.  While they add batch b the others already write batch b + 1.
constexpr int kChainRows = 2;                        // rows per thread and batch
constexpr int kChainBatch = kThreads * kChainRows;   // 512
constexpr int kChainStride = kChainBatch + 4;        // floats between the columns of a buffer

__device__ __forceinline__ void exact_chain_runs(const SegArgs& a, float (&s_buf)[2][4 * kChainStride],
                                                 int64_t sl, uint32_t first, uint32_t stride) {
  const uint32_t very_long = a.long_list[0], count = very_long + a.long_list[1];
  const int64_t last_entry = 1 + (a.n + kLongRun - 1) / kLongRun;
  const f32x4* slice = reinterpret_cast<const f32x4*>(a.stage) + sl * a.n;
  const bool adder = threadIdx.x < 4;
  for (uint32_t li = first; li < count; li += stride) {
    const uint32_t u = li < very_long ? a.long_list[2 + li] : a.long_list[last_entry - (li - very_long)];
    const int64_t start = a.seg_start[u];
    const int64_t len = a.seg_start[u + 1] - start;
    const f32x4* src = slice + start;
    float accf = 0.f;
    f32x4 rows_a[kChainRows], rows_b[kChainRows];
    auto issue_rows = [&](f32x4 (&rows)[kChainRows], int64_t base) {
#pragma unroll
      for (int k = 0; k < kChainRows; ++k) {
        const int64_t r = base + k * kThreads + threadIdx.x;
        rows[k] = r < len ? __builtin_nontemporal_load(src + r) : f32x4{0.f, 0.f, 0.f, 0.f};
      }
    };
    auto stage = [&](const f32x4 (&rows)[kChainRows], float* buf) {
#pragma unroll
      for (int k = 0; k < kChainRows; ++k) {
        const int r = k * kThreads + threadIdx.x;
        buf[0 * kChainStride + r] = rows[k].x;
        buf[1 * kChainStride + r] = rows[k].y;
        buf[2 * kChainStride + r] = rows[k].z;
        buf[3 * kChainStride + r] = rows[k].w;
      }
    };
    auto add_batch = [&](const float* buf, int rows_here) {
      const float* colp = buf + threadIdx.x * kChainStride;
      constexpr int kUnits = 8;                  // 16-byte loads (four rows each) per register set
      f32x4 qa[kUnits], qb[kUnits];
      auto rd = [&](f32x4 (&q)[kUnits], int row0) {
#pragma unroll
        for (int k = 0; k < kUnits; ++k) q[k] = *reinterpret_cast<const f32x4*>(colp + row0 + 4 * k);
      };
      auto ad = [&](const f32x4 (&q)[kUnits]) {
#pragma unroll
        for (int k = 0; k < kUnits; ++k) {
          accf += q[k].x;
          accf += q[k].y;
          accf += q[k].z;
          accf += q[k].w;
        }
      };
      const int nsets = rows_here / (4 * kUnits);   // whole register sets: 32 rows each
      int sidx = 0;
      if (nsets > 0) rd(qa, 0);
      while (sidx < nsets) {
        if (sidx + 1 < nsets) rd(qb, (sidx + 1) * 4 * kUnits);
        ad(qa);
        if (++sidx >= nsets) break;
        if (sidx + 1 < nsets) rd(qa, (sidx + 1) * 4 * kUnits);
        ad(qb);
        ++sidx;
      }
      for (int r = nsets * 4 * kUnits; r < rows_here; ++r) accf += colp[r];
    };
    // step b: batch b (loaded two steps earlier) goes to LDS buffer b & 1, the loads of batch
    // b + 2 are issued, and after the barrier the column threads add batch b - while the others
    // go on to write batch b + 1 into the other buffer, which the column threads left before
    // they reached this barrier
    auto step = [&](f32x4 (&rows)[kChainRows], float* buf, int64_t base) {
      stage(rows, buf);
      if (base + 2 * kChainBatch < len) issue_rows(rows, base + 2 * kChainBatch);
      __syncthreads();
      if (adder) {
        const int64_t left = len - base;
        add_batch(buf, left < kChainBatch ? static_cast<int>(left) : kChainBatch);
      }
    };
    issue_rows(rows_a, 0);
    issue_rows(rows_b, kChainBatch);
    for (int64_t base = 0; base < len; base += 2 * kChainBatch) {
      step(rows_a, s_buf[0], base);
      if (base + kChainBatch < len) step(rows_b, s_buf[1], base + kChainBatch);
    }
    if (adder)
      a.sums[static_cast<int64_t>(u) * a.dim + sl * 4 + threadIdx.x] = accf;
    __syncthreads();   // the buffers are rewritten for the next run of the list
  }
}

// The last kernel of the staged EXACT sum.  Its first pieces * chain_blocks blocks sum the long
// runs: block b takes slice b % pieces of the list entries b / pieces, b / pieces + chain_blocks,
// ... - blocks are handed out in the order of their index, so all slices of the first (longest)
// runs start before anything else.  The blocks after them sum the short runs, one lane group per
// run, on the compute units that the few long chains leave idle.
template <int VEC>
__global__ __launch_bounds__(kThreads) void seg_exact_staged_kernel(SegArgs a, uint32_t pieces,
                                                                   uint32_t chain_blocks) {
  __shared__ __align__(16) float s_buf[2][4 * kChainStride];
  const uint32_t nchain = pieces * chain_blocks;
  if (blockIdx.x < nchain) {
    exact_chain_runs(a, s_buf, blockIdx.x % pieces, blockIdx.x / pieces, chain_blocks);
  } else {
    exact_short_runs<VEC>(a, static_cast<int64_t>(blockIdx.x - nchain));
  }
}

__global__ void clear_u32x2_kernel(uint32_t* p) {
  if (blockIdx.x == 0 && threadIdx.x < 2) p[threadIdx.x] = 0;
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
struct Plan {
  bool key64;
  int key_bits;
  int passes;
  bool scan;      // group counts are prefix-scanned by a kernel of their own
  int vec;        // 4 or 1
  int group;
  int col_tiles;
  int64_t ntiles;        // radix tiles
  int64_t nblocks_runs;
  int chunk;             // sorted positions per lane group of the FAST segmented sum
  int64_t nblocks_seg;   // blocks of the FAST segmented sum
};

// Sorted positions per lane group of the FAST sum.  A small batch gives a chunk of 32 only a
// hundred-odd blocks, each a chain of two rounds of row loads: shorter chunks make more and
// shorter blocks.  The shape of the sum stays a function of (n, dim) alone.
int seg_chunk_for(int64_t n) {
  static const int env = [] { const char* e = getenv("HADES_SEG_CHUNK"); return e ? atoi(e) : 0; }();
  if (env == 8 || env == 16 || env == 32) return env;
  return n <= (int64_t(1) << 17) ? 8 : kChunk;
}

Plan make_plan(int64_t n, int64_t dim, int64_t id_bound, bool grad_aligned) {
  Plan p;
  const int64_t nn = n > 0 ? n : 1;
  if (id_bound > 0) {
    p.key_bits = ilog2_ceil(static_cast<uint64_t>(id_bound));
    p.key64 = p.key_bits > 32;  // ids are non-negative: the flipped sign bit is constant, skip it
  } else {
    p.key64 = true;
    p.key_bits = 64;
  }
  if (p.key_bits < 1) p.key_bits = 1;
  p.passes = (p.key_bits + kRadixBits - 1) / kRadixBits;
  p.ntiles = ceil_div(nn, kThreads * kIpt);
  // past kScanFrom groups of tiles the group counts are turned into prefixes by a kernel of their
  // own (3-4 us), and a scatter block reads five count rows instead of one per group
  p.scan = ceil_div(p.ntiles, kGroup) > kScanFrom;
  p.vec = (dim % 4 == 0 && grad_aligned) ? 4 : 1;
  const int64_t lanes = (dim + p.vec - 1) / p.vec;
  int g = kMinGroup;
  while (g < lanes && g < 64) g <<= 1;
  p.group = g;
  p.col_tiles = static_cast<int>((lanes + g - 1) / g);
  p.nblocks_runs = ceil_div(nn, kUTile);
  p.chunk = seg_chunk_for(nn);
  p.nblocks_seg = ceil_div(nn, static_cast<int64_t>(kThreads / g) * p.chunk);
  return p;
}

// workspace of the sort alone
struct SortWs {
  uint32_t* status;     // [kSweepStatusWords], first thing in the workspace: [0] = tiles of the last
                        // one-sweep sort whose bounded wait ran out (they recounted instead)
  int32_t* bad;         // [nbad]: 1 where a block of the first count pass saw an id outside
                        // [0, id_bound); rewritten in full by every sort
  int64_t nbad;
  void* keys[2];
  uint32_t* vals[2];
  uint32_t* cnt;        // [ntiles][kBins], rewritten by every pass; the one-sweep sort keeps the
                        // tile states of its even passes here
  uint32_t* gcnt;       // [ceil(ntiles / kGroup)][kBins]: sums of kGroup consecutive rows of cnt
  int64_t cnt_len;
  uint32_t* state1;     // [ntiles][kBins]: tile states of the odd passes of the one-sweep sort
  uint32_t* hist_part;  // [nchunks][kMaxPasses][kBins]: per-chunk digit counts of every pass
  uint32_t* bases;      // [kMaxPasses][kBins]
  int64_t nchunks;
  size_t bytes;
};

void carve_sort(Carver& c, int64_t n, SortWs* w) {
  const int64_t nn = n > 0 ? n : 1;
  w->status = c.take<uint32_t>(kSweepStatusWords);
  for (int i = 0; i < 2; ++i) w->keys[i] = c.take<uint64_t>(nn);  // sized for 64-bit keys
  for (int i = 0; i < 2; ++i) w->vals[i] = c.take<uint32_t>(nn);
  // the tile count depends on n only; the one-sweep form keeps its tile states here, kIpt keys per thread
  const int ipt_min = radix_ipt_for(nn) < kIpt ? radix_ipt_for(nn) : kIpt;
  w->cnt_len = ceil_div(nn, kThreads * ipt_min) * kBins;
  w->nchunks = ceil_div(nn, kHistChunk);
  const int64_t ngroups = ceil_div(w->cnt_len / kBins, kGroup);
  w->nbad = ngroups > w->nchunks ? ngroups : w->nchunks;
  w->bad = c.take<int32_t>(w->nbad);
  w->cnt = c.take<uint32_t>(w->cnt_len);
  w->gcnt = c.take<uint32_t>((ngroups + 1) * kBins);  // + totals row
  w->state1 = c.take<uint32_t>(w->cnt_len);
  w->hist_part = c.take<uint32_t>(w->nchunks * kMaxPasses * kBins);
  w->bases = c.take<uint32_t>(kMaxPasses * kBins);
  w->bytes = c.total();
}

struct Ws {
  SortWs sort;
  uint32_t* run_cnt;    // [run tiles + 1]: per-tile run counts, or the tile states of run_sweep_kernel
  uint32_t* seg_of;
  uint32_t* seg_start;
  float* partial;
  uint32_t* long_list;  // [2][2 + ceil(n / kLongRun)]: the long runs of the EXACT sum, see
                        // seg_stage_kernel; the lower class of a classed plan has the second list
  size_t bytes_min;     // what every entry point needs
  float* stage;         // [n * dim]: the rows of the long runs in column slices (EXACT sum); last,
                        // so that a workspace of bytes_min simply lacks it
  size_t bytes;         // with the staging area
};

Ws carve(void* ws, int64_t n, int64_t dim) {
  Carver c(ws);
  Ws w;
  const int64_t nn = n > 0 ? n : 1;
  carve_sort(c, n, &w.sort);
  w.run_cnt = c.take<uint32_t>(ceil_div(nn, kThreads * kUItemsSmall) + 1);
  w.seg_of = c.take<uint32_t>(nn);
  w.seg_start = c.take<uint32_t>(nn + 1);
  // at most two partial rows per block of the FAST sum; the smallest block span is four chunks
  w.partial = c.take<float>(2 * ceil_div(nn, (kThreads / 64) * seg_chunk_for(nn)) * dim);
  w.long_list = c.take<uint32_t>(2 * (2 + ceil_div(nn, kLongRun)));
  w.bytes_min = c.total();
  w.stage = c.take<float>(static_cast<size_t>(nn) * dim);
  w.bytes = c.total();
  return w;
}

// process-wide choice of the sort and the bound of its waits (hades_sort_config).  The default is
// the form without waits: measured on 65 K / 200 K / 1 M keys the one-sweep form was slower by
// 10 / 19 / 30 us per sort - a pass with the look-back inside costs 12 - 14 us at 200 K keys and
// 20 - 26 us at 1 M, as much as the count, scan and scatter kernels it replaces (4.5 + 8.8 us and
// 5 + 3.5 + 14.4 us), and the histogram and base kernels come on top.
std::atomic<int> g_one_sweep{0};
std::atomic<int> g_spin_limit{50000};

template <typename KeyT>
int run_sort_three_kernels(const int64_t* idx, int64_t n, int64_t id_bound, const Plan& p,
                           const SortWs& w, hipStream_t st, const void** keys_out,
                           const uint32_t** perm_out) {
  // 65 536 keys in tiles of 1 024 are 64 blocks a kernel; in tiles of 512 every block's chain of
  // ranking rounds is half as long and twice as many compute units work (whole cfg1 step 76.5 ->
  // 71.3 us; at 200 000 keys the smaller tiles lose: 159.7 -> 163.2 us, tiles of 256: 173.6 us)
  // (one million keys: tiles of 2 048 take 5 us off the sort, 194 -> 189 us for cfg5's combine)
  const int ipt = radix_ipt_for(n);
  const int64_t ntiles = ceil_div(n, static_cast<int64_t>(kThreads) * ipt);
  const int64_t ngroups = ceil_div(ntiles, kGroup);
  HADES_REQUIRE(ntiles * kBins <= w.cnt_len && ngroups <= w.nbad, "internal: radix count buffer too small");
  const dim3 grid(static_cast<unsigned>(ntiles)), cgrid(static_cast<unsigned>(ngroups)),
      block(kThreads), cblock(kGroup * kThreads), sgrid(kBins / kWaves);
  const int scanned = ngroups > kScanFrom ? 1 : 0;
  const int base = p.key_bits / p.passes, extra = p.key_bits % p.passes;
  int bits_of[kMaxPasses], shift_of[kMaxPasses + 1];
  shift_of[0] = 0;
  for (int pass = 0; pass < p.passes; ++pass) {
    bits_of[pass] = base + (pass < extra ? 1 : 0);
    shift_of[pass + 1] = shift_of[pass] + bits_of[pass];
  }
  const void* kin = idx;
  const uint32_t* vin = nullptr;
  int cur = 0;
  for (int pass = 0; pass < p.passes; ++pass) {
    const uint32_t mask = (1u << bits_of[pass]) - 1u;
    KeyT* kout = static_cast<KeyT*>(w.keys[cur]);
    uint32_t* vout = w.vals[cur];
#define HADES_RADIX_PASS(FIRST_, IPT_)                                                              \
  do {                                                                                              \
    HADES_LAUNCH((radix_count_kernel<KeyT, FIRST_, IPT_>), cgrid, cblock, 0, st, kin, n,            \
                 shift_of[pass], mask, w.cnt, w.gcnt, ntiles, id_bound, w.bad, w.nbad);             \
    if (scanned) HADES_LAUNCH(radix_group_scan_kernel, sgrid, block, 0, st, w.gcnt, ngroups);       \
    HADES_LAUNCH_TIMED(HADES_KERNEL_RADIX_PASS, st, (radix_pass_kernel<KeyT, FIRST_, IPT_>), grid,  \
                       block, 0, st, kin, vin, n, shift_of[pass], mask, bits_of[pass], w.cnt,       \
                       w.gcnt, ngroups, scanned, kout, vout);                                       \
  } while (0)
    if (pass == 0) {
      if (ipt == kIptSmall) HADES_RADIX_PASS(true, kIptSmall);
      else if (ipt == kIptLarge) HADES_RADIX_PASS(true, kIptLarge);
      else HADES_RADIX_PASS(true, kIpt);
    } else {
      if (ipt == kIptSmall) HADES_RADIX_PASS(false, kIptSmall);
      else if (ipt == kIptLarge) HADES_RADIX_PASS(false, kIptLarge);
      else HADES_RADIX_PASS(false, kIpt);
    }
#undef HADES_RADIX_PASS
    kin = kout;
    vin = vout;
    cur ^= 1;
  }
  *keys_out = kin;
  *perm_out = vin;
  return HADES_OK;
}

// The one-sweep sort: histogram of all passes, digit bases, then one kernel per pass.
// run_state / run_state_words: further words to clear for the run kernel that follows (or null).
template <typename KeyT>
int run_sort_one_sweep(const int64_t* idx, int64_t n, int64_t id_bound, const Plan& p,
                       const SortWs& w, hipStream_t st, uint32_t* run_state,
                       int64_t run_state_words, const void** keys_out, const uint32_t** perm_out) {
  HADES_REQUIRE(p.ntiles * kBins <= w.cnt_len, "internal: tile state buffer too small");
  constexpr int IPT = kIpt;
  SweepDigits dg;
  dg.passes = p.passes;
  const int base = p.key_bits / p.passes, extra = p.key_bits % p.passes;
  int bits_of[kMaxPasses];
  int shift = 0;
  for (int pass = 0; pass < kMaxPasses; ++pass) {
    bits_of[pass] = pass < p.passes ? base + (pass < extra ? 1 : 0) : 0;
    dg.shift[pass] = shift;
    dg.mask[pass] = bits_of[pass] ? (1u << bits_of[pass]) - 1u : 0u;
    shift += bits_of[pass];
  }
  const dim3 block(kThreads), hblock(kHistThreads), hgrid(static_cast<unsigned>(w.nchunks)),
      grid(static_cast<unsigned>(p.ntiles));
  HADES_LAUNCH((sweep_hist_kernel<KeyT>), hgrid, hblock, 0, st, idx, n, dg, w.hist_part, id_bound,
               w.bad, w.nbad, w.cnt, p.ntiles * kBins, run_state, run_state_words, w.status);
  HADES_LAUNCH(sweep_bases_kernel, dim3(static_cast<unsigned>(p.passes)), hblock, 0, st,
               w.hist_part, w.nchunks, p.passes, w.bases);
  const int spin_limit = g_spin_limit.load(std::memory_order_relaxed);
  // keys per thread of a pass: larger tiles for larger batches, so that a pass has a few hundred
  // tiles whatever the size - the look-back chain and its traffic grow with the number of tiles
  static const int ipt_env = [] { const char* e = getenv("HADES_SWEEP_IPT"); return e ? atoi(e) : 0; }();
  int ipt = n > (int64_t(1) << 19) ? 16 : (n > (int64_t(1) << 18) ? 8 : 4);
  if (ipt_env == 4 || ipt_env == 8 || ipt_env == 16) ipt = ipt_env;
  const dim3 pgrid(static_cast<unsigned>(ceil_div(n, static_cast<int64_t>(kThreads) * ipt)));
  const void* kin = idx;
  const uint32_t* vin = nullptr;
  int cur = 0;
  for (int pass = 0; pass < p.passes; ++pass) {
    KeyT* kout = static_cast<KeyT*>(w.keys[cur]);
    uint32_t* vout = w.vals[cur];
    uint32_t* state = (pass & 1) ? w.state1 : w.cnt;
    uint32_t* next_state = pass + 1 < p.passes ? ((pass & 1) ? w.cnt : w.state1) : nullptr;
#define HADES_SWEEP_PASS(FIRST_, IPT_)                                                             \
  HADES_LAUNCH_TIMED(HADES_KERNEL_RADIX_PASS, st, (sweep_pass_kernel<KeyT, FIRST_, IPT_>), pgrid,  \
                     block, 0, st, kin, vin, n, dg.shift[pass], dg.mask[pass], bits_of[pass],      \
                     w.bases + pass * kBins, state, next_state, spin_limit, w.status, kout, vout)
    if (pass == 0) {
      if (ipt == 16) HADES_SWEEP_PASS(true, 16);
      else if (ipt == 8) HADES_SWEEP_PASS(true, 8);
      else HADES_SWEEP_PASS(true, 4);
    } else {
      if (ipt == 16) HADES_SWEEP_PASS(false, 16);
      else if (ipt == 8) HADES_SWEEP_PASS(false, 8);
      else HADES_SWEEP_PASS(false, 4);
    }
#undef HADES_SWEEP_PASS
    kin = kout;
    vin = vout;
    cur ^= 1;
  }
  *keys_out = kin;
  *perm_out = vin;
  return HADES_OK;
}

template <typename KeyT>
int run_runs(const void* sorted_keys, const uint32_t* perm, int64_t n, const Plan& p, const Ws& w,
             int64_t* uids, int64_t* num_unique, int32_t* inverse, hipStream_t st, bool one_sweep,
             int64_t threshold = 0, int64_t* class_split = nullptr, int32_t* first_pos = nullptr) {
  const KeyT* keys = static_cast<const KeyT*>(sorted_keys);
  const dim3 rgrid(static_cast<unsigned>(p.nblocks_runs)), block(kThreads);
  if (one_sweep) {
    // w.run_cnt holds the tile states, cleared by the sort's histogram kernel
    HADES_LAUNCH((run_sweep_kernel<KeyT>), rgrid, block, 0, st, keys, perm, n, w.run_cnt,
                 g_spin_limit.load(std::memory_order_relaxed), w.sort.status, uids, w.seg_start,
                 w.seg_of, num_unique, inverse, w.sort.bad, w.sort.nbad,
                 key_from_id<KeyT>(threshold), class_split, first_pos);
    return HADES_OK;
  }
  static const int items_env = [] { const char* e = getenv("HADES_RUN_ITEMS"); return e ? atoi(e) : 0; }();
  int items = n <= kRunsSmallBatch ? kUItemsSmall : kUItems;
  if (items_env == 2 || items_env == 4 || items_env == 8) items = items_env;
  const dim3 sgrid(static_cast<unsigned>(ceil_div(n, static_cast<int64_t>(kThreads) * items)));
#define HADES_RUNS(ITEMS_)                                                                          \
  do {                                                                                              \
    HADES_LAUNCH((run_count_kernel<KeyT, ITEMS_>), sgrid, block, 0, st, keys, n, w.run_cnt);        \
    HADES_LAUNCH_CHECK();                                                                           \
    HADES_LAUNCH((run_emit_kernel<KeyT, ITEMS_>), sgrid, block, 0, st, keys, perm, n, w.run_cnt,    \
                 uids, w.seg_start, w.seg_of, num_unique, inverse, w.sort.bad, w.sort.nbad,         \
                 key_from_id<KeyT>(threshold), class_split, first_pos);                             \
    HADES_LAUNCH_CHECK();                                                                           \
  } while (0)
  if (items == 2) HADES_RUNS(2);
  else if (items == 4) HADES_RUNS(4);
  else HADES_RUNS(8);
#undef HADES_RUNS
  return HADES_OK;
}

template <typename KeyT>
int run_sort(const int64_t* idx, int64_t n, int64_t id_bound, const Plan& p, const SortWs& w,
             hipStream_t st, bool one_sweep, uint32_t* run_state, int64_t run_state_words,
             const void** keys_out, const uint32_t** perm_out) {
  if (one_sweep)
    return run_sort_one_sweep<KeyT>(idx, n, id_bound, p, w, st, run_state, run_state_words,
                                    keys_out, perm_out);
  return run_sort_three_kernels<KeyT>(idx, n, id_bound, p, w, st, keys_out, perm_out);
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
  out->bad = w.bad;
  out->nbad = w.nbad;
  const bool sweep = g_one_sweep.load(std::memory_order_relaxed) != 0;
  return p.key64 ? run_sort<uint64_t>(ids, n, id_bound, p, w, st, sweep, nullptr, 0,
                                      &out->sorted_keys, &out->perm)
                 : run_sort<uint32_t>(ids, n, id_bound, p, w, st, sweep, nullptr, 0,
                                      &out->sorted_keys, &out->perm);
}

int combine_plan_views(void* workspace, size_t workspace_bytes, int64_t n, int64_t dim,
                       int64_t id_bound, const uint32_t** perm, const uint32_t** seg_start) {
  HADES_REQUIRE(n >= 1 && n < (int64_t(1) << 30) && dim >= 1 && id_bound >= 0, "bad plan shape");
  const Plan p = make_plan(n, dim, id_bound, true);
  const Ws w = carve(workspace, n, dim);
  if (workspace == nullptr || workspace_bytes < w.bytes_min)
    return set_error(HADES_ERR_WORKSPACE, "combine workspace too small: need %zu bytes, got %zu",
                     w.bytes_min, workspace_bytes);
  HADES_REQUIRE((align_of_ptr(workspace) & 255) == 0, "workspace must be 256-byte aligned");
  *perm = w.sort.vals[(p.passes - 1) & 1];   // where the last pass of the plan left the positions
  *seg_start = w.seg_start;
  return HADES_OK;
}

}  // namespace hades

using namespace hades;

extern "C" {

int hades_sort_config(int one_sweep, int64_t spin_limit) {
  HADES_REQUIRE(one_sweep >= -1 && one_sweep <= 1, "one_sweep must be 0, 1 or -1 (leave as it is)");
  HADES_REQUIRE(spin_limit >= -1 && spin_limit <= (int64_t(1) << 30),
                "spin_limit must be in [0, 2^30] or -1 (leave as it is)");
  if (one_sweep >= 0) g_one_sweep.store(one_sweep, std::memory_order_relaxed);
  if (spin_limit >= 0) g_spin_limit.store(static_cast<int>(spin_limit), std::memory_order_relaxed);
  return HADES_OK;
}

int hades_sort_mode(void) { return g_one_sweep.load(std::memory_order_relaxed); }

size_t hades_combine_workspace_bytes(int64_t n, int64_t dim) {
  if (n < 0 || dim < 1) return 0;
  return carve(nullptr, n, dim).bytes;
}

size_t hades_combine_workspace_bytes_min(int64_t n, int64_t dim) {
  if (n < 0 || dim < 1) return 0;
  return carve(nullptr, n, dim).bytes_min;
}

namespace {

__global__ void set_i64x2_kernel(int64_t* p, int64_t a, int64_t b) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    p[0] = a;
    p[1] = b;
  }
}

int combine_plan_impl(const int64_t* idx, int64_t n, int64_t dim, int64_t id_bound, int64_t* uids,
                      int64_t* num_unique, int32_t* inverse, void* workspace,
                      size_t workspace_bytes, void* stream, int64_t threshold,
                      int64_t* class_split, int32_t* first_pos) {
  HADES_REQUIRE(n >= 0 && dim >= 1, "n must be >= 0 and dim >= 1");
  HADES_REQUIRE(n < (int64_t(1) << 30), "combine: n must be below 2^30 (got %lld)", (long long)n);
  HADES_REQUIRE(id_bound >= 0, "id_bound must be >= 0");
  HADES_REQUIRE(num_unique != nullptr, "num_unique must not be null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n == 0) {
    HADES_LAUNCH(set_i64_kernel, dim3(1), dim3(64), 0, st, num_unique, int64_t(0));
    if (class_split != nullptr)
      HADES_LAUNCH(set_i64x2_kernel, dim3(1), dim3(64), 0, st, class_split, int64_t(0), int64_t(0));
    return HADES_OK;
  }
  HADES_REQUIRE(idx && uids, "null pointer argument");
  const Plan p = make_plan(n, dim, id_bound, true);
  const Ws w = carve(workspace, n, dim);
  if (workspace == nullptr || workspace_bytes < w.bytes_min)
    return set_error(HADES_ERR_WORKSPACE, "combine workspace too small: need %zu bytes, got %zu",
                     w.bytes_min, workspace_bytes);
  HADES_REQUIRE((align_of_ptr(workspace) & 255) == 0, "workspace must be 256-byte aligned");

  const uint32_t* perm = nullptr;
  const void* sorted_keys = nullptr;
  const bool sweep = g_one_sweep.load(std::memory_order_relaxed) != 0;
  int rc = p.key64 ? run_sort<uint64_t>(idx, n, id_bound, p, w.sort, st, sweep, w.run_cnt,
                                        p.nblocks_runs + 1, &sorted_keys, &perm)
                   : run_sort<uint32_t>(idx, n, id_bound, p, w.sort, st, sweep, w.run_cnt,
                                        p.nblocks_runs + 1, &sorted_keys, &perm);
  if (rc != HADES_OK) return rc;
  return p.key64 ? run_runs<uint64_t>(sorted_keys, perm, n, p, w, uids, num_unique, inverse, st,
                                      sweep, threshold, class_split, first_pos)
                 : run_runs<uint32_t>(sorted_keys, perm, n, p, w, uids, num_unique, inverse, st,
                                      sweep, threshold, class_split, first_pos);
}

}  // namespace

int hades_combine_plan(const int64_t* idx, int64_t n, int64_t dim, int64_t id_bound, int64_t* uids,
                       int64_t* num_unique, int32_t* inverse, void* workspace,
                       size_t workspace_bytes, void* stream) {
  return combine_plan_impl(idx, n, dim, id_bound, uids, num_unique, inverse, workspace,
                           workspace_bytes, stream, 0, nullptr, nullptr);
}

int hades_combine_plan_classed(const int64_t* keys, int64_t n, int64_t dim, int64_t key_bound,
                               int64_t threshold, int64_t* ukeys, int64_t* num_unique,
                               int64_t* class_split, int32_t* first_pos, void* workspace,
                               size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(class_split != nullptr, "class_split must not be null");
  HADES_REQUIRE(key_bound > 0 && threshold >= 0 && threshold <= key_bound,
                "key_bound must be > 0 and threshold in [0, key_bound]");
  return combine_plan_impl(keys, n, dim, key_bound, ukeys, num_unique, nullptr, workspace,
                           workspace_bytes, stream, threshold, class_split, first_pos);
}

namespace {

int combine_apply_impl(const float* grad, int64_t n, int64_t dim, int64_t id_bound, int mode,
                       float* sums, int64_t* cnts, const int64_t* num_unique, void* workspace,
                       size_t workspace_bytes, void* stream, const int64_t* class_split, int which) {
  HADES_REQUIRE(n >= 0 && dim >= 1, "n must be >= 0 and dim >= 1");
  HADES_REQUIRE(n < (int64_t(1) << 30), "combine: n must be below 2^30 (got %lld)", (long long)n);
  HADES_REQUIRE(id_bound >= 0, "id_bound must be >= 0");
  HADES_REQUIRE(mode == HADES_COMBINE_FAST || mode == HADES_COMBINE_EXACT, "unknown combine mode %d",
                mode);
  HADES_REQUIRE(num_unique != nullptr, "num_unique must not be null");
  if (n == 0) return HADES_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  HADES_REQUIRE(grad && sums && cnts, "null pointer argument");
  const bool aligned = (align_of_ptr(grad) % 16) == 0 && (align_of_ptr(sums) % 16) == 0;
  const Plan p = make_plan(n, dim, id_bound, aligned);
  const Ws w = carve(workspace, n, dim);
  if (workspace == nullptr || workspace_bytes < w.bytes_min)
    return set_error(HADES_ERR_WORKSPACE, "combine workspace too small: need %zu bytes, got %zu",
                     w.bytes_min, workspace_bytes);
  HADES_REQUIRE((align_of_ptr(workspace) & 255) == 0, "workspace must be 256-byte aligned");

  // a workspace of the full size has the staging area of the EXACT sum behind everything else
  const bool staged = workspace_bytes >= w.bytes;
  SegArgs a;
  a.grad = grad;
  a.perm = w.sort.vals[(p.passes - 1) & 1];  // where the last pass of the plan left the positions
  a.seg_of = w.seg_of;
  a.seg_start = w.seg_start;
  a.num_unique = num_unique;
  a.sums = sums;
  a.cnts = cnts;
  a.partial = w.partial;
  a.n = n;
  a.dim = dim;
  a.group = p.group;
  a.col_tiles = p.col_tiles;
  a.class_split = class_split;
  a.which = class_split != nullptr ? which : -1;
  if (mode == HADES_COMBINE_EXACT) {
    const int64_t blocks = ceil_div(n * p.group, kThreads);
    HADES_REQUIRE(blocks < (int64_t(1) << 31), "combine: too many rows");
    // short runs, then the long ones; the timing hook brackets the pair
    const bool timed = g_profile.kernel_id == HADES_KERNEL_SEG_SUM;
    if (timed) HADES_HIP_TRY(hipEventRecord(g_profile.start, st));
    const dim3 lgrid(static_cast<unsigned>(ceil_div(n, kLongRun)),
                     static_cast<unsigned>(ceil_div(dim, kLongSlice)));
    if (p.vec == 4 && staged) {
      // the rows of the long runs into column slices (and the runs into a list), then one kernel
      // with a chain of adds per long run and slice, and the short runs beside them
      a.stage = w.stage;   // indexed by sorted position: the classes of a classed plan do not meet
      a.long_list = w.long_list + (a.which == 0 ? 2 + ceil_div(n, kLongRun) : 0);
      const int64_t pieces = dim / 4;
      const int64_t sblocks = ceil_div(n * pieces, kThreads * kStagePieces);
      int64_t cblocks = ceil_div(n, kLongRun);   // no more long runs than this
      if (cblocks > 128) cblocks = 128;
      HADES_REQUIRE(sblocks < (int64_t(1) << 31) && blocks + pieces * cblocks < (int64_t(1) << 31),
                    "combine: too many rows");
      HADES_LAUNCH(clear_u32x2_kernel, dim3(1), dim3(64), 0, st, a.long_list);
      HADES_LAUNCH(seg_stage_kernel, dim3((unsigned)sblocks), dim3(kThreads), 0, st, a);
      HADES_LAUNCH((seg_exact_staged_kernel<4>), dim3((unsigned)(blocks + pieces * cblocks)),
                   dim3(kThreads), 0, st, a, static_cast<uint32_t>(pieces),
                   static_cast<uint32_t>(cblocks));
    } else if (p.vec == 4) {
      // 128 KB of dynamic LDS: above the default limit, which has to be raised once per device
      constexpr int kLongLds = kLongThreads * kLongRows * sizeof(f32x4);  // a batch of row slices
      static std::atomic<uint64_t> raised{0};  // bit d: done on device d
      int device = 0;
      HADES_HIP_TRY(hipGetDevice(&device));
      const uint64_t bit = uint64_t(1) << (device & 63);
      if (!(raised.load(std::memory_order_acquire) & bit)) {
        HADES_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&seg_exact_long_kernel<4>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, kLongLds));
        raised.fetch_or(bit, std::memory_order_release);
      }
      HADES_LAUNCH((seg_exact_kernel<4>), dim3((unsigned)blocks), dim3(kThreads), 0, st, a);
      HADES_LAUNCH((seg_exact_long_kernel<4>), lgrid, dim3(kLongThreads), kLongLds, st, a);
    } else {
      HADES_LAUNCH((seg_exact_kernel<1>), dim3((unsigned)blocks), dim3(kThreads), 0, st, a);
      HADES_LAUNCH((seg_exact_long_kernel<1>), lgrid, dim3(kLongThreads),
                   kLongThreads * kLongRows * sizeof(float), st, a);
    }
    if (timed) HADES_HIP_TRY(hipEventRecord(g_profile.stop, st));
  } else {
    HADES_REQUIRE(p.nblocks_seg < (int64_t(1) << 31), "combine: too many rows");
    const dim3 grid(static_cast<unsigned>(p.nblocks_seg));
    // one block of the second kernel per span of the first, and at least one thread per sorted
    // position so that every u < U <= n gets its count written
    const int64_t fblocks = p.nblocks_seg > ceil_div(n, kThreads) ? p.nblocks_seg : ceil_div(n, kThreads);
#define HADES_FAST_SUM(VEC_, CH_)                                                                   \
  do {                                                                                              \
    HADES_LAUNCH_TIMED(HADES_KERNEL_SEG_SUM, st, (seg_chunk_kernel<VEC_, CH_>), grid,               \
                       dim3(kThreads), 0, st, a);                                                   \
    HADES_LAUNCH_CHECK();                                                                           \
    HADES_LAUNCH((seg_fixup_kernel<VEC_, CH_>), dim3((unsigned)fblocks), dim3(kThreads), 0, st, a); \
  } while (0)
    if (p.vec == 4) {
      if (p.chunk == 8) HADES_FAST_SUM(4, 8);
      else if (p.chunk == 16) HADES_FAST_SUM(4, 16);
      else HADES_FAST_SUM(4, 32);
    } else {
      if (p.chunk == 8) HADES_FAST_SUM(1, 8);
      else if (p.chunk == 16) HADES_FAST_SUM(1, 16);
      else HADES_FAST_SUM(1, 32);
    }
#undef HADES_FAST_SUM
    HADES_LAUNCH_CHECK();
  }
  return HADES_OK;
}

}  // namespace

int hades_combine_apply(const float* grad, int64_t n, int64_t dim, int64_t id_bound, int mode,
                        float* sums, int64_t* cnts, const int64_t* num_unique, void* workspace,
                        size_t workspace_bytes, void* stream) {
  return combine_apply_impl(grad, n, dim, id_bound, mode, sums, cnts, num_unique, workspace,
                            workspace_bytes, stream, nullptr, -1);
}

int hades_combine_apply_class(const float* grad, int64_t n, int64_t dim, int64_t key_bound, int mode,
                              int which, float* sums, int64_t* cnts, const int64_t* num_unique,
                              const int64_t* class_split, void* workspace, size_t workspace_bytes,
                              void* stream) {
  HADES_REQUIRE(class_split != nullptr, "class_split must not be null");
  HADES_REQUIRE(which == 0 || which == 1, "which must be 0 (below the threshold) or 1");
  return combine_apply_impl(grad, n, dim, key_bound, mode, sums, cnts, num_unique, workspace,
                            workspace_bytes, stream, class_split, which);
}

int hades_combine(const int64_t* idx, const float* grad, int64_t n, int64_t dim, int64_t id_bound,
                  int mode, int64_t* uids, float* sums, int64_t* cnts, int64_t* num_unique,
                  int32_t* inverse, void* workspace, size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(mode == HADES_COMBINE_FAST || mode == HADES_COMBINE_EXACT, "unknown combine mode %d",
                mode);
  HADES_REQUIRE(n <= 0 || (grad && sums && cnts), "null pointer argument");
  const int rc = hades_combine_plan(idx, n, dim, id_bound, uids, num_unique, inverse, workspace,
                                    workspace_bytes, stream);
  if (rc != HADES_OK) return rc;
  return hades_combine_apply(grad, n, dim, id_bound, mode, sums, cnts, num_unique, workspace,
                             workspace_bytes, stream);
}

int hades_combine_static(const int64_t* idx, const float* grad, int64_t n, int64_t dim,
                         int64_t id_bound, int mode, int64_t* uids, float* sums, int64_t* cnts,
                         int64_t* num_unique, int32_t* inverse, void* stream) {
  HADES_REQUIRE(n >= 0 && dim >= 1, "n must be >= 0 and dim >= 1");
  const size_t need = hades_combine_workspace_bytes_min(n, dim);
  HADES_REQUIRE(need <= size_t(HADES_COMBINE_STATIC_SCRATCH_BYTES),
                "hades_combine_static: n=%lld rows of dim=%lld need %zu bytes of scratch, the "
                "library holds %zu; use hades_combine with a workspace of your own",
                (long long)n, (long long)dim, need, size_t(HADES_COMBINE_STATIC_SCRATCH_BYTES));
  // device address of this GPU's copy of the scratch array, looked up once per device
  static std::mutex mu;
  static void* scratch_of[64] = {};
  int device = 0;
  HADES_HIP_TRY(hipGetDevice(&device));
  HADES_REQUIRE(device >= 0 && device < 64, "device ordinal %d out of range", device);
  void* scratch = nullptr;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (scratch_of[device] == nullptr) {
      void* p = nullptr;
      HADES_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_scratch)));
      HADES_REQUIRE(p != nullptr, "hipGetSymbolAddress returned a null scratch address");
      scratch_of[device] = p;
    }
    scratch = scratch_of[device];
  }
  // Nothing in the scratch has to start at zero: every word a kernel reads was written earlier in
  // the same call (count rows, bound flags, run tables and partial rows are rewritten in full).
  return hades_combine(idx, grad, n, dim, id_bound, mode, uids, sums, cnts, num_unique, inverse,
                       scratch, size_t(HADES_COMBINE_STATIC_SCRATCH_BYTES), stream);
}

int hades_rows_div_count(float* sums, const int64_t* cnts, const int64_t* num_unique,
                         int64_t max_rows, int64_t dim, int one_plus, void* stream) {
  HADES_REQUIRE(max_rows >= 0 && dim >= 1, "max_rows must be >= 0 and dim >= 1");
  if (max_rows == 0) return HADES_OK;
  HADES_REQUIRE(sums && cnts, "null pointer argument");
  int64_t blocks = ceil_div(max_rows * dim, kThreads);
  if (blocks > 65536) blocks = 65536;
  HADES_LAUNCH(rows_div_kernel, dim3((unsigned)blocks), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), sums, cnts, num_unique, max_rows, dim,
                     one_plus);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

}  // extern "C"
