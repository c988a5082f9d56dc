// Gradient side of the cold-data cache, with the reference's per-row staleness rule: the
// arithmetic of the cache server (python/EmbCache/server.py) over slot arrays in HBM instead of
// shared-memory tensors walked by torch CPU indexing.
//   insert      _update_cache (:499-544)                 emb[loc] = row; grad[loc] = 0; cnt[loc] = 0; idx[loc] = -1
//   accumulate  _accumulate_gradients_cold_remote (:546-562) and _cold_local (:564-574)
//                                                        idx[loc] = id; thr[loc] = threshold[id]; grad[loc] += g; cnt[loc] += 1
//   flush       _send_staled_gradients (:346-419 remote, :421-497 local)
//                                                        rows with cnt > 0 and (iter >= thr or cnt >= cnt_threshold)
//                                                        leave in slot order; they are zeroed, their ids
//                                                        leave the index cache; iter += 1 for every row
//                                                        with cnt > 0, iter = 0 for the rows that left
// Slots are the locs of the set-associative index cache (sacache.hip) for the remote part, or
// id - id_offset for the dense local part.
// The reference zeroes gradient rows through a temporary (`buf[index][:] = 0`, :414, :489, :537),
// which leaves them as they were; what is implemented is the evident intent, zeroing.
#include "internal.h"

namespace hades {
namespace {

constexpr int kThreads = 256;
constexpr int kLine = 8;

typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int VEC> struct Vf;
template <> struct Vf<4> { typedef f32x4 type; static __device__ type zero() { return type{0.f, 0.f, 0.f, 0.f}; } };
template <> struct Vf<1> { typedef float type; static __device__ type zero() { return 0.f; } };

struct AccArgs {
  const int64_t* locs;       // slot per row, or null: slot = ids[r] - id_offset
  const int64_t* ids;
  const float* grad;
  int64_t n, dim, id_offset, num_slots;
  const int32_t* threshold;  // per id, or null: thr is left alone
  float* grad_buf;
  int32_t* grad_cnt;
  int64_t* grad_idx;         // may be null (dense local part)
  int32_t* iter_threshold;
};

__device__ __forceinline__ int64_t slot_of(const AccArgs& a, int64_t r) {
  const int64_t s = a.locs ? a.locs[r] : a.ids[r] - a.id_offset;
  return (s >= 0 && s < a.num_slots) ? s : int64_t(-1);
}

// one thread per VEC-wide chunk of a row; rows must name distinct slots
template <int VEC>
__global__ __launch_bounds__(kThreads) void cc_accumulate_kernel(AccArgs a) {
  typedef typename Vf<VEC>::type V;
  const int64_t cpr = a.dim / VEC;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (t >= a.n * cpr) return;
  const int64_t r = t / cpr, c = t - r * cpr;
  const int64_t s = slot_of(a, r);
  if (s < 0) return;
  V* dst = reinterpret_cast<V*>(a.grad_buf + s * a.dim + c * VEC);
  const V g = __builtin_nontemporal_load(reinterpret_cast<const V*>(a.grad + r * a.dim + c * VEC));
  *dst = *dst + g;
  if (c == 0) {
    const int64_t id = a.ids[r];
    if (a.grad_idx) a.grad_idx[s] = id;
    if (a.threshold) a.iter_threshold[s] = a.threshold[id];
    a.grad_cnt[s] += 1;
  }
}

struct InsArgs {
  const int64_t* locs;
  const int64_t* ids;
  const int64_t* line_ids;  // the index cache after the add that produced locs
  const float* rows;
  int64_t n, dim, num_slots;
  float* emb_buf;
  float* grad_buf;
  int32_t* grad_cnt;
  int64_t* grad_idx;
};

// Two ids of one batch can be given the same loc: the first was already cached there, the second
// evicted it later in the batch.  The reference's `buf[locs] = rows` (:531) then keeps the row
// written last, the evictor's; here the row is written by whichever id holds the entry after the
// add, which is the same one and needs no ordering between threads.
template <int VEC>
__global__ __launch_bounds__(kThreads) void cc_insert_kernel(InsArgs a) {
  typedef typename Vf<VEC>::type V;
  const int64_t cpr = a.dim / VEC;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (t >= a.n * cpr) return;
  const int64_t r = t / cpr, c = t - r * cpr;
  const int64_t s = a.locs[r];
  if (s < 0 || s >= a.num_slots) return;
  if (a.line_ids[s] != a.ids[r]) return;
  *reinterpret_cast<V*>(a.emb_buf + s * a.dim + c * VEC) =
      *reinterpret_cast<const V*>(a.rows + r * a.dim + c * VEC);
  *reinterpret_cast<V*>(a.grad_buf + s * a.dim + c * VEC) = Vf<VEC>::zero();
  if (c == 0) {
    a.grad_cnt[s] = 0;
    a.grad_idx[s] = -1;
  }
}

// key[s] = s if the row is due, else -1; ages every row that holds gradients
__global__ __launch_bounds__(kThreads) void cc_classify_kernel(
    const int32_t* __restrict__ grad_cnt, int32_t* __restrict__ iter_count,
    const int32_t* __restrict__ iter_threshold, int32_t cnt_threshold, int64_t num_slots,
    int64_t* __restrict__ key) {
  const int64_t s = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (s >= num_slots) return;
  const int32_t c = grad_cnt[s];
  int64_t k = -1;
  if (c > 0) {
    const int32_t it = iter_count[s];
    if (it >= iter_threshold[s] || c >= cnt_threshold) k = s;
    iter_count[s] = it + 1;
  }
  key[s] = k;
}

struct EmitArgs {
  const int64_t* pos;        // due slots, ascending
  const int64_t* count;      // their number
  int64_t out_cap, dim, id_offset;
  float* grad_buf;
  int32_t* grad_cnt;
  const int64_t* grad_idx;   // null: id = slot + id_offset
  int32_t* iter_count;
  int64_t* line_ids;         // index cache to take the ids out of, or null
  int32_t* line_age;
  int64_t lines;
  int64_t* out_ids;
  float* out_grads;
  int64_t* out_cnts;
  int64_t* num_out;
  int32_t* status;
};

template <int VEC>
__global__ __launch_bounds__(kThreads) void cc_emit_kernel(EmitArgs a) {
  typedef typename Vf<VEC>::type V;
  const int64_t due = a.count[0];
  const int64_t m = due < a.out_cap ? due : a.out_cap;
  const int64_t cpr = a.dim / VEC;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (t == 0) {
    a.num_out[0] = m;
    if (due > a.out_cap) atomicOr(a.status, 2);  // the rest stays due and leaves with the next flush
  }
  if (t >= m * cpr) return;
  const int64_t j = t / cpr, c = t - j * cpr;
  const int64_t s = a.pos[j];
  V* src = reinterpret_cast<V*>(a.grad_buf + s * a.dim + c * VEC);
  *reinterpret_cast<V*>(a.out_grads + j * a.dim + c * VEC) = *src;
  *src = Vf<VEC>::zero();
  if (c == 0) {
    const int64_t id = a.grad_idx ? a.grad_idx[s] : s + a.id_offset;
    a.out_ids[j] = id;
    a.out_cnts[j] = a.grad_cnt[s];
    a.grad_cnt[s] = 0;
    a.iter_count[s] = 0;
    if (a.line_ids && id >= 0) {  // IndexCache.reset of the id (src/cache/cache.h:109-121)
      const int64_t ln = id % a.lines;
      for (int e = 0; e < kLine; ++e)
        if (a.line_ids[ln * kLine + e] == id) {
          a.line_ids[ln * kLine + e] = -1;
          a.line_age[ln * kLine + e] = 0;
          break;
        }
    }
  }
}

inline size_t round256(size_t b) { return (b + 255) & ~size_t(255); }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline unsigned grid_of(int64_t n) { return static_cast<unsigned>(ceil_div(n > 0 ? n : 1, kThreads)); }

}  // namespace
}  // namespace hades

using namespace hades;

extern "C" {

int hades_coldcache_insert(const int64_t* locs, const int64_t* ids, const int64_t* line_ids,
                           const float* rows, int64_t n, int64_t dim, int64_t num_slots,
                           float* emb_buf, float* grad_buf, int32_t* grad_cnt, int64_t* grad_idx,
                           void* stream) {
  HADES_REQUIRE(n >= 0 && dim >= 1 && num_slots >= 1, "bad sizes");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(locs && ids && line_ids && rows && emb_buf && grad_buf && grad_cnt && grad_idx,
                "null pointer argument");
  HADES_REQUIRE(ceil_div(n * dim, kThreads) < (int64_t(1) << 31), "n * dim too large");
  const InsArgs a{locs, ids, line_ids, rows, n, dim, num_slots, emb_buf, grad_buf, grad_cnt,
                  grad_idx};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dim % 4 == 0 && aligned16(rows) && aligned16(emb_buf) && aligned16(grad_buf))
    HADES_LAUNCH((cc_insert_kernel<4>), dim3(grid_of(n * (dim / 4))), dim3(kThreads), 0, st, a);
  else
    HADES_LAUNCH((cc_insert_kernel<1>), dim3(grid_of(n * dim)), dim3(kThreads), 0, st, a);
  return HADES_OK;
}

int hades_coldcache_accumulate(const int64_t* locs, const int64_t* ids, const float* grad,
                               int64_t n, int64_t dim, int64_t id_offset, int64_t num_slots,
                               const int32_t* threshold, float* grad_buf, int32_t* grad_cnt,
                               int64_t* grad_idx, int32_t* iter_threshold, void* stream) {
  HADES_REQUIRE(n >= 0 && dim >= 1 && num_slots >= 1, "bad sizes");
  if (n == 0) return HADES_OK;
  HADES_REQUIRE(ids && grad && grad_buf && grad_cnt, "null pointer argument");
  HADES_REQUIRE(threshold == nullptr || iter_threshold != nullptr,
                "threshold needs iter_threshold to write to");
  HADES_REQUIRE(ceil_div(n * dim, kThreads) < (int64_t(1) << 31), "n * dim too large");
  const AccArgs a{locs, ids, grad, n, dim, id_offset, num_slots, threshold,
                  grad_buf, grad_cnt, grad_idx, iter_threshold};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dim % 4 == 0 && aligned16(grad) && aligned16(grad_buf))
    HADES_LAUNCH((cc_accumulate_kernel<4>), dim3(grid_of(n * (dim / 4))), dim3(kThreads), 0, st, a);
  else
    HADES_LAUNCH((cc_accumulate_kernel<1>), dim3(grid_of(n * dim)), dim3(kThreads), 0, st, a);
  return HADES_OK;
}

size_t hades_coldcache_flush_workspace_bytes(int64_t num_slots) {
  if (num_slots < 1) return 0;
  return 256 + round256(compact_live_workspace_bytes(num_slots)) +
         2 * round256(static_cast<size_t>(num_slots) * 8) + 256;
}

int hades_coldcache_flush(int64_t num_slots, int64_t dim, int32_t cnt_threshold,
                          int64_t id_offset, float* grad_buf, int32_t* grad_cnt,
                          const int64_t* grad_idx, int32_t* iter_count,
                          const int32_t* iter_threshold, int64_t* line_ids, int32_t* line_age,
                          int64_t lines, int64_t* out_ids, float* out_grads, int64_t* out_cnts,
                          int64_t* num_out, int64_t out_cap, void* workspace,
                          size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(num_slots >= 1 && num_slots < (int64_t(1) << 31) && dim >= 1, "bad sizes");
  HADES_REQUIRE(out_cap >= 0, "out_cap must be >= 0");
  HADES_REQUIRE(grad_buf && grad_cnt && iter_count && iter_threshold && num_out,
                "null pointer argument");
  HADES_REQUIRE(out_cap == 0 || (out_ids && out_grads && out_cnts), "null output pointer");
  HADES_REQUIRE((line_ids == nullptr) == (line_age == nullptr) && (line_ids == nullptr || lines >= 1),
                "line_ids, line_age and lines go together");
  const size_t need = hades_coldcache_flush_workspace_bytes(num_slots);
  if (workspace == nullptr || workspace_bytes < need)
    return set_error(HADES_ERR_WORKSPACE, "flush workspace too small: need %zu bytes, got %zu",
                     need, workspace_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* base = static_cast<char*>(workspace);
  int32_t* status = reinterpret_cast<int32_t*>(base);  // sticky: bit 1 = out_cap was too small
  const size_t cbytes = round256(compact_live_workspace_bytes(num_slots));
  void* cws = base + 256;
  int64_t* key = reinterpret_cast<int64_t*>(base + 256 + cbytes);
  int64_t* pos = reinterpret_cast<int64_t*>(base + 256 + cbytes + round256(static_cast<size_t>(num_slots) * 8));
  int64_t* count = reinterpret_cast<int64_t*>(base + 256 + cbytes + 2 * round256(static_cast<size_t>(num_slots) * 8));

  HADES_LAUNCH(cc_classify_kernel, dim3(grid_of(num_slots)), dim3(kThreads), 0, st, grad_cnt,
               iter_count, iter_threshold, cnt_threshold, num_slots, key);
  const int rc = compact_live_keys(key, num_slots, pos, count, cws, cbytes, st);
  if (rc != HADES_OK) return rc;
  const EmitArgs a{pos, count, out_cap, dim, id_offset, grad_buf, grad_cnt, grad_idx, iter_count,
                   line_ids, line_age, lines, out_ids, out_grads, out_cnts, num_out, status};
  const int64_t m = out_cap < num_slots ? out_cap : num_slots;
  const bool vec4 = dim % 4 == 0 && aligned16(grad_buf) && (out_grads == nullptr || aligned16(out_grads));
  HADES_REQUIRE(ceil_div(m * dim, kThreads) < (int64_t(1) << 31), "out_cap * dim too large");
  if (vec4)
    HADES_LAUNCH((cc_emit_kernel<4>), dim3(grid_of(m * (dim / 4))), dim3(kThreads), 0, st, a);
  else
    HADES_LAUNCH((cc_emit_kernel<1>), dim3(grid_of(m * dim)), dim3(kThreads), 0, st, a);
  return HADES_OK;
}

}  // extern "C"
