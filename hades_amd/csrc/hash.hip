// Cold-gradient accumulator (delayed synchronisation): an open-addressing hash table in HBM,
// int64 key -> fp32[dim] running sum + int64 count.  It restates on the GPU the arithmetic the
// reference's cache server does on the CPU over shared-memory tensors:
//   accumulate: EmbCacheServer._accumulate_gradients_cold_remote (python/EmbCache/server.py:546-562)
//               buf[slot] += g; cnt[slot] += c; key[slot] = id
//   flush     : _send_staled_gradients (python/EmbCache/server.py:346-497): emit the rows whose
//               count is positive, then reset their key and count (:413-419).  The reference
//               zeroes the gradient rows through a temporary copy (`buf[idx][:] = 0`, :414), so
//               its rows are in fact never zeroed; the evident intent - zero on flush - is what
//               is implemented here.
// The table uses linear probing with a 64-bit compare-and-swap on the key; the reference's index
// is an 8-way set-associative structure on the CPU (src/cache/cache.h:51-118).
#include "internal.h"

namespace hades {
namespace {

constexpr int kThreads = 256;
constexpr int kRows = 64;
constexpr int kUnroll = 4;
constexpr int64_t kEmpty = -1;

typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int VEC> struct Vf;
template <> struct Vf<4> { typedef f32x4 type; static __device__ type zero() { return type{0.f, 0.f, 0.f, 0.f}; } };
template <> struct Vf<1> { typedef float type; static __device__ type zero() { return 0.f; } };

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
  x ^= x >> 30; x *= 0xbf58476d1ce4e5b9ull;
  x ^= x >> 27; x *= 0x94d049bb133111ebull;
  x ^= x >> 31;
  return x;
}

__global__ __launch_bounds__(kThreads) void hash_clear_kernel(int64_t* __restrict__ keys,
                                                             float* __restrict__ accum,
                                                             int64_t* __restrict__ cnt,
                                                             int64_t num_slots, int64_t dim,
                                                             int64_t ss) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  for (int64_t i = t; i < num_slots; i += stride) {
    keys[i * ss] = kEmpty;
    cnt[i * ss] = 0;
  }
  const int64_t total = num_slots * dim;
  for (int64_t i = t; i < total; i += stride) accum[i] = 0.f;
}

struct AccArgs {
  int64_t* keys; float* accum; int64_t* cnt; int64_t num_slots;
  const int64_t* ids; const float* grad; const int64_t* in_cnt; const int64_t* num_rows;
  int64_t max_rows; int64_t dim; int32_t* status;
  int64_t ss;   // int64 words between the keys (and between the counts) of consecutive slots
};

template <int VEC>
__global__ __launch_bounds__(kThreads) void hash_accumulate_kernel(AccArgs a) {
  typedef typename Vf<VEC>::type V;
  __shared__ int64_t s_slot[kRows];
  const int64_t U = a.num_rows ? a.num_rows[0] : a.max_rows;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRows;
  const int64_t left = (U < a.max_rows ? U : a.max_rows) - row0;
  const int rows_here = left >= kRows ? kRows : (left > 0 ? static_cast<int>(left) : 0);
  const uint64_t mask = static_cast<uint64_t>(a.num_slots) - 1;
  for (int r = threadIdx.x; r < rows_here; r += kThreads) {
    const int64_t id = a.ids[row0 + r];
    uint64_t h = mix64(static_cast<uint64_t>(id)) & mask;
    int64_t slot = -1;
    // a negative id is never stored (-1 marks an empty slot): its row is dropped, status bit 3
    // bounded probe: every wave leaves the loop after at most num_slots steps
    for (int64_t probe = 0; id >= 0 && probe < a.num_slots; ++probe) {
      unsigned long long* kp = reinterpret_cast<unsigned long long*>(a.keys + h * a.ss);
      // A plain load is enough to look: a key, once stored, stays until the flush, so a
      // non-empty value is never stale in a harmful way, and a stale "empty" only sends the
      // thread to the compare-and-swap below, which is the arbiter (device-scope atomics are
      // executed beyond the per-XCD L2 and cost a round trip of their own).
      int64_t k = a.keys[h * a.ss];
      if (k == kEmpty) {
        k = static_cast<int64_t>(atomicCAS(kp, static_cast<unsigned long long>(kEmpty),
                                           static_cast<unsigned long long>(id)));
        if (k == kEmpty) k = id;  // claimed
      }
      if (k == id) {
        slot = static_cast<int64_t>(h);
        break;
      }
      h = (h + 1) & mask;
    }
    if (slot < 0) {
      atomicOr(a.status, id < 0 ? 8 : 1);
    } else {
      a.cnt[slot * a.ss] += a.in_cnt ? a.in_cnt[row0 + r] : 1;
    }
    s_slot[r] = slot;
  }
  __syncthreads();
  if (rows_here == 0) return;
  const int cpr = static_cast<int>(a.dim / VEC);
  const int total = rows_here * cpr;
  for (int base = threadIdx.x; base < total; base += kThreads * kUnroll) {
    V g[kUnroll], s[kUnroll];
    V* sp[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int c = base + k * kThreads;
      sp[k] = nullptr;
      if (c < total) {
        const int r = c / cpr;
        const int64_t col = static_cast<int64_t>(c - r * cpr) * VEC;
        if (s_slot[r] >= 0) {
          sp[k] = reinterpret_cast<V*>(a.accum + s_slot[r] * a.dim + col);
          // gradient rows are read exactly once: keep them from displacing table rows in L2
          g[k] = __builtin_nontemporal_load(
              reinterpret_cast<const V*>(a.grad + (row0 + r) * a.dim + col));
          s[k] = *sp[k];
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k)
      if (sp[k]) *sp[k] = s[k] + g[k];
  }
}

// ids of the live slots in slot order, padded with `pad` up to cap (so that the padding sorts last)
__global__ __launch_bounds__(kThreads) void flush_gather_ids_kernel(
    const int64_t* __restrict__ keys, const int64_t* __restrict__ live_pos,
    const int64_t* __restrict__ live_count, int64_t cap, int64_t pad, int64_t* __restrict__ ids_out,
    int64_t* __restrict__ num_out, int32_t* __restrict__ status, int64_t ss) {
  const int64_t L = live_count[0];
  const bool overflow = L > cap;
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (j == 0) {
    num_out[0] = overflow ? 0 : L;
    if (overflow) atomicOr(status, 2);
  }
  if (j < cap) ids_out[j] = (!overflow && j < L) ? keys[live_pos[j] * ss] : pad;
}

struct FlushArgs {
  int64_t* keys; float* accum; int64_t* cnt; int64_t dim;
  const int64_t* live_pos; const uint32_t* perm; const int64_t* num_out;
  int64_t* out_ids; float* out_sums; int64_t* out_cnts; int64_t cap;
  const int32_t* bad; int64_t nbad; int32_t* status;
  int64_t ss;
};

// out row j <- the live slot with the j-th smallest id; the slot is emptied
template <int VEC>
__global__ __launch_bounds__(kThreads) void flush_emit_kernel(FlushArgs a) {
  typedef typename Vf<VEC>::type V;
  __shared__ int64_t s_slot[kRows];
  // a stored id outside [0, id_bound] left the ids unsorted: the rows still leave, status bit 2
  // says that their order is not ascending
  if (blockIdx.x == 0) {
    const int violated = any_flag_set(a.bad, a.nbad);
    if (violated && threadIdx.x == 0) atomicOr(a.status, 4);
  }
  const int64_t L = a.num_out[0];
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRows;
  const int64_t left = (L < a.cap ? L : a.cap) - row0;
  const int rows_here = left >= kRows ? kRows : (left > 0 ? static_cast<int>(left) : 0);
  for (int r = threadIdx.x; r < rows_here; r += kThreads) {
    const int64_t slot = a.live_pos[a.perm[row0 + r]];
    s_slot[r] = slot;
    a.out_ids[row0 + r] = a.keys[slot * a.ss];
    a.out_cnts[row0 + r] = a.cnt[slot * a.ss];
    a.keys[slot * a.ss] = kEmpty;
    a.cnt[slot * a.ss] = 0;
  }
  __syncthreads();
  if (rows_here == 0) return;
  const int cpr = static_cast<int>(a.dim / VEC);
  const int total = rows_here * cpr;
  for (int base = threadIdx.x; base < total; base += kThreads * kUnroll) {
    V s[kUnroll];
    V* sp[kUnroll];
    V* op[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int c = base + k * kThreads;
      sp[k] = nullptr;
      if (c < total) {
        const int r = c / cpr;
        const int64_t col = static_cast<int64_t>(c - r * cpr) * VEC;
        sp[k] = reinterpret_cast<V*>(a.accum + s_slot[r] * a.dim + col);
        op[k] = reinterpret_cast<V*>(a.out_sums + (row0 + r) * a.dim + col);
        s[k] = *sp[k];
      }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      if (sp[k]) {
        *op[k] = s[k];
        *sp[k] = Vf<VEC>::zero();
      }
    }
  }
}

struct FlushWs {
  int64_t* live_pos;
  int64_t* live_count;
  int64_t* ids;
  void* compact_ws;
  size_t compact_bytes;
  void* sort_ws;
  size_t sort_bytes;
  size_t bytes;
};

FlushWs carve_flush(void* ws, int64_t num_slots, int64_t cap) {
  Carver c(ws);
  FlushWs w;
  w.live_pos = c.take<int64_t>(num_slots);
  w.live_count = c.take<int64_t>(4);
  w.ids = c.take<int64_t>(cap > 0 ? cap : 1);
  w.compact_bytes = compact_live_workspace_bytes(num_slots);
  w.compact_ws = c.take<char>(w.compact_bytes);
  w.sort_bytes = sort_ids_workspace_bytes(cap > 0 ? cap : 1);
  w.sort_ws = c.take<char>(w.sort_bytes);
  w.bytes = c.total();
  return w;
}

}  // namespace
}  // namespace hades

using namespace hades;

extern "C" {

int hades_hash_clear(int64_t* keys, float* accum, int64_t* cnt, int64_t num_slots, int64_t dim,
                     int64_t slot_stride, void* stream) {
  HADES_REQUIRE(is_pow2(num_slots), "num_slots must be a power of two (got %lld)",
                (long long)num_slots);
  HADES_REQUIRE(dim >= 1 && keys && accum && cnt, "bad argument");
  HADES_REQUIRE(slot_stride >= 0, "slot_stride must be >= 0");
  const int64_t ss = slot_stride ? slot_stride : 1;
  int64_t blocks = ceil_div(num_slots * dim, kThreads * 8);
  if (blocks > 65536) blocks = 65536;
  HADES_LAUNCH(hash_clear_kernel, dim3((unsigned)blocks), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), keys, accum, cnt, num_slots, dim, ss);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

int hades_hash_accumulate(int64_t* keys, float* accum, int64_t* cnt, int64_t num_slots,
                          const int64_t* ids, const float* grad, const int64_t* in_cnt,
                          const int64_t* num_rows, int64_t max_rows, int64_t dim, int32_t* status,
                          int64_t slot_stride, void* stream) {
  HADES_REQUIRE(is_pow2(num_slots), "num_slots must be a power of two (got %lld)",
                (long long)num_slots);
  HADES_REQUIRE(dim >= 1 && max_rows >= 0, "bad dim or max_rows");
  HADES_REQUIRE(slot_stride >= 0, "slot_stride must be >= 0");
  HADES_REQUIRE(dim * kRows < (int64_t(1) << 30), "dim too large");
  if (max_rows == 0) return HADES_OK;
  HADES_REQUIRE(keys && accum && cnt && ids && grad && status, "null pointer argument");
  AccArgs a{keys, accum, cnt, num_slots, ids, grad, in_cnt, num_rows, max_rows, dim, status,
            slot_stride ? slot_stride : 1};
  const dim3 grid(static_cast<unsigned>(ceil_div(max_rows, kRows))), block(kThreads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec4 = dim % 4 == 0 && (align_of_ptr(accum) % 16) == 0 && (align_of_ptr(grad) % 16) == 0;
  if (vec4)
    HADES_LAUNCH_TIMED(HADES_KERNEL_HASH_ACCUMULATE, st, (hash_accumulate_kernel<4>), grid, block, 0,
                       st, a);
  else
    HADES_LAUNCH_TIMED(HADES_KERNEL_HASH_ACCUMULATE, st, (hash_accumulate_kernel<1>), grid, block, 0,
                       st, a);
  return HADES_OK;
}

size_t hades_hash_flush_workspace_bytes(int64_t num_slots, int64_t cap) {
  if (num_slots < 1 || cap < 0) return 0;
  return carve_flush(nullptr, num_slots, cap).bytes;
}

int hades_hash_flush(int64_t* keys, float* accum, int64_t* cnt, int64_t num_slots, int64_t dim,
                     int64_t id_bound, int64_t* out_ids, float* out_sums, int64_t* out_cnts,
                     int64_t* num_out, int64_t cap, int32_t* status, int64_t slot_stride,
                     void* workspace, size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(is_pow2(num_slots), "num_slots must be a power of two (got %lld)",
                (long long)num_slots);
  HADES_REQUIRE(slot_stride >= 0, "slot_stride must be >= 0");
  const int64_t ss = slot_stride ? slot_stride : 1;
  HADES_REQUIRE(dim >= 1 && cap >= 1 && cap < (int64_t(1) << 30), "bad dim or cap");
  HADES_REQUIRE(id_bound >= 0 && id_bound < INT64_MAX, "bad id_bound");
  HADES_REQUIRE(keys && accum && cnt && out_ids && out_sums && out_cnts && num_out && status,
                "null pointer argument");
  const FlushWs w = carve_flush(workspace, num_slots, cap);
  if (workspace == nullptr || workspace_bytes < w.bytes)
    return set_error(HADES_ERR_WORKSPACE, "flush workspace too small: need %zu bytes, got %zu",
                     w.bytes, workspace_bytes);
  HADES_REQUIRE((align_of_ptr(workspace) & 255) == 0, "workspace must be 256-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc = compact_live_keys(keys, num_slots, w.live_pos, w.live_count, w.compact_ws,
                             w.compact_bytes, st, ss);
  if (rc != HADES_OK) return rc;
  const int64_t pad = id_bound > 0 ? id_bound : INT64_MAX;
  HADES_LAUNCH(flush_gather_ids_kernel, dim3((unsigned)ceil_div(cap, kThreads)),
                     dim3(kThreads), 0, st, keys, w.live_pos, w.live_count, cap, pad, w.ids, num_out,
                     status, ss);
  HADES_LAUNCH_CHECK();
  SortResult sr;
  rc = sort_ids(w.ids, cap, id_bound > 0 ? id_bound + 1 : 0, w.sort_ws, w.sort_bytes, st, &sr);
  if (rc != HADES_OK) return rc;
  FlushArgs a{keys, accum, cnt, dim, w.live_pos, sr.perm, num_out, out_ids, out_sums, out_cnts, cap,
              sr.bad, sr.nbad, status, ss};
  const dim3 grid(static_cast<unsigned>(ceil_div(cap, kRows))), block(kThreads);
  const bool vec4 = dim % 4 == 0 && (align_of_ptr(accum) % 16) == 0 && (align_of_ptr(out_sums) % 16) == 0;
  if (vec4)
    HADES_LAUNCH((flush_emit_kernel<4>), grid, block, 0, st, a);
  else
    HADES_LAUNCH((flush_emit_kernel<1>), grid, block, 0, st, a);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

}  // extern "C"
