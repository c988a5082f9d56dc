// Sparse row optimizers with the lookup, the state/weight gather and the scatter-back fused into
// one kernel: sparse Adagrad, and the SparseAdam of the reference
// (python/EmbCache/sparse_optim.py:590-685; state gather/scatter python/EmbCache/cache.py:66-131).
//
// A block owns kRows consecutive unique rows.  Phase 1: one thread per row searches the sorted hot
// set and records where the row lives (hot slot in HBM, or the id itself for the cold tables,
// which may be pinned host memory).  Phase 2: the block walks its rows as a flat list of float4
// chunks (scalar when dim is not a multiple of 4): read g, state, w; write state, w.
// This translation unit is compiled with fused multiply-add contraction off: every operation
// rounds to fp32 on its own, like the CPU restatement it is checked against.
#include "internal.h"

namespace hades {
namespace {

constexpr int kThreads = 256;
constexpr int kRows = 64;
constexpr int kUnroll = 4;

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int VEC>
struct Vf;
template <>
struct Vf<4> {
  typedef f32x4 type;
};
template <>
struct Vf<1> {
  typedef float type;
};

// sqrtf and the division operator are correctly rounded (the library is compiled with
// -fhip-fp32-correctly-rounded-divide-sqrt); the __fsqrt_rn intrinsic is the fast native one.
__device__ __forceinline__ float vsqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ f32x4 vsqrt(f32x4 x) {
  return f32x4{sqrtf(x.x), sqrtf(x.y), sqrtf(x.z), sqrtf(x.w)};
}
__device__ __forceinline__ float vdiv(float a, float b) { return a / b; }
__device__ __forceinline__ f32x4 vdiv(f32x4 a, f32x4 b) {
  return f32x4{a.x / b.x, a.y / b.y, a.z / b.z, a.w / b.w};
}

struct RowArgs {
  const int64_t* uids;
  const float* grad;
  const int64_t* num_unique;
  int64_t max_rows;
  int64_t dim;
  HotSet hs;
  // averaging as in ListedRows below: 0 none, 1 divide row u by cnts[u], 2 by cnts[u] + 1
  const int64_t* cnts;
  int average;
};

struct AdagradArgs {
  RowArgs r;
  float* hot_w; float* hot_s; float* cold_w; float* cold_s;
  float lr, eps;
};

struct AdamArgs {
  RowArgs r;
  float* hot_w; float* hot_step; float* hot_m; float* hot_v;
  float* cold_w; float* cold_step; float* cold_m; float* cold_v;
  float lr, beta1, beta2, one_minus_beta1, one_minus_beta2, eps;
};

// phase 1 shared by both optimizers: s_row[r] = element offset of the row in its table,
// s_hot[r] = 1 if that table is the hot one.  Returns the number of live rows of this block.
__device__ __forceinline__ int resolve_rows(const RowArgs& a, int64_t* s_row, uint8_t* s_hot,
                                            float* s_div) {
  const int64_t U = a.num_unique ? a.num_unique[0] : a.max_rows;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRows;
  const int64_t left = (U < a.max_rows ? U : a.max_rows) - row0;
  const int rows_here = left >= kRows ? kRows : (left > 0 ? static_cast<int>(left) : 0);
  for (int r = threadIdx.x; r < rows_here; r += kThreads) {
    const int64_t id = a.uids[row0 + r];
    const int64_t loc = a.hs.slot(id);
    s_row[r] = loc >= 0 ? loc : id;
    s_hot[r] = loc >= 0 ? 1 : 0;
    if (a.average != 0) s_div[r] = static_cast<float>(a.cnts[row0 + r] + (a.average == 2 ? 1 : 0));
  }
  return rows_here;
}

template <int VEC>
__global__ __launch_bounds__(kThreads) void adagrad_kernel(AdagradArgs a) {
  typedef typename Vf<VEC>::type V;
  __shared__ int64_t s_row[kRows];
  __shared__ uint8_t s_hot[kRows];
  __shared__ float s_div[kRows];
  const int rows_here = resolve_rows(a.r, s_row, s_hot, s_div);
  __syncthreads();
  if (rows_here == 0) return;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRows;
  const int cpr = static_cast<int>(a.r.dim / VEC);
  const int total = rows_here * cpr;
  for (int base = threadIdx.x; base < total; base += kThreads * kUnroll) {
    V g[kUnroll], s[kUnroll], w[kUnroll];
    V* sp[kUnroll];
    V* wp[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int c = base + k * kThreads;
      if (c < total) {
        const int r = c / cpr;
        const int64_t col = static_cast<int64_t>(c - r * cpr) * VEC;
        const int64_t off = s_row[r] * a.r.dim + col;
        sp[k] = reinterpret_cast<V*>((s_hot[r] ? a.hot_s : a.cold_s) + off);
        wp[k] = reinterpret_cast<V*>((s_hot[r] ? a.hot_w : a.cold_w) + off);
        // the gradient row is read once; the state and weight rows of hot ids come back next step
        g[k] = __builtin_nontemporal_load(
            reinterpret_cast<const V*>(a.r.grad + (row0 + r) * a.r.dim + col));
        s[k] = *sp[k];
        w[k] = *wp[k];
      }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int c = base + k * kThreads;
      if (c < total) {
        if (a.r.average != 0) g[k] = vdiv(g[k], V(s_div[c / cpr]));
        const V s1 = s[k] + g[k] * g[k];
        const V std_ = vsqrt(s1) + a.eps;
        const V w1 = w[k] - vdiv(a.lr * g[k], std_);
        *sp[k] = s1;
        *wp[k] = w1;
      }
    }
  }
}

// Row updates over the rows named by a position list whose length lives in device memory (one half
// of a hot/cold split), or over one class of the distinct rows of a class-ordered combine.
// Listed form: for j < count[0], p = list[j].  Class form: p runs over [class_split[1],
// num_unique[0]) (which = 1) or [0, class_split[1]) (which = 0).  The gradient is row p of grad;
// the table row is row_index[p] & index_mask, and rows of the weight table and of the per-element
// state tables lie `stride` floats apart (weights and state of a row may sit next to each other
// in one table: s = w + dim, stride = 2 * dim).
struct ListedRows {
  const int64_t* row_index;
  const float* grad;
  const int64_t* list;      // null: class form
  const int64_t* count;     // listed form: number of live list entries
  int64_t max_count;
  const int64_t* num_unique;
  const int64_t* class_split;
  int which;
  int64_t index_mask;
  // optional: the old weight row of position p is row first_pos[p] of w_rows (rows fetched from
  // the same table earlier and still valid) instead of being read from the table again
  const float* w_rows;
  const int32_t* first_pos;
  int64_t dim;
  int64_t stride;
  // Summing class form: `grad` holds one row per QUERY of the batch (not per distinct key) and the
  // gradient of run u is the sum of rows perm[seg_start[u]] .. perm[seg_start[u + 1] - 1], added
  // one after the other from +0.0f in that order - the order of occurrence, since the plan's sort
  // is stable: the arithmetic of the deterministic-order segmented sum, done where it is consumed.
  // sums_out / cnts_out (optional) receive the summed row and the length of every run.
  const uint32_t* perm = nullptr;
  const uint32_t* seg_start = nullptr;
  float* sums_out = nullptr;
  int64_t* cnts_out = nullptr;
  // Averaging (unique_grads, python/EmbCache/sparse_optim.py:142-157): the gradient of a row is
  // divided by its number of occurrences (average = 1) or by one more than that (average = 2:
  // the reference's count starts from ones when counts come with the rows, :145-148) before the
  // update.  The occurrences are the run length (summing form) or run_cnts[p].
  int average = 0;
  const int64_t* run_cnts = nullptr;
};

struct AdagradListedArgs {
  ListedRows r;
  float* w;
  float* s;
  float* w_out;             // optional: the new weight row of position p also goes to row p of w_out
  float lr, eps;
};

struct AdamListedArgs {
  ListedRows r;
  float* w;
  float* step;              // one float per table row
  float* m;
  float* v;
  float lr, beta1, beta2, one_minus_beta1, one_minus_beta2, eps;
};

// the positions [first, end) a launch walks
__device__ __forceinline__ void listed_range(const ListedRows& a, int64_t* first, int64_t* end) {
  if (a.list != nullptr) {
    const int64_t cnt = a.count[0];
    *first = 0;
    *end = cnt < a.max_count ? cnt : a.max_count;
    return;
  }
  int64_t U = a.num_unique[0];
  U = U < a.max_count ? U : a.max_count;
  int64_t sr = a.class_split[1];
  sr = sr < U ? sr : U;
  sr = sr > 0 ? sr : 0;
  *first = a.which ? sr : 0;
  *end = a.which ? U : sr;
}

// Offsets of the rows [row0, row0 + rows_here) of the walk: s_tab[r] = table row, s_grad[r] =
// element offset of the gradient row, s_old[r] = element offset of the old weight row in w_rows.
template <bool SUMMING>
__device__ __forceinline__ void resolve_listed(const ListedRows& a, int64_t row0, int rows_here,
                                               int64_t* s_tab, int64_t* s_grad, int64_t* s_old,
                                               uint32_t* s_j0, uint32_t* s_len, float* s_div) {
  for (int r = threadIdx.x; r < rows_here; r += kThreads) {
    const int64_t p = a.list != nullptr ? a.list[row0 + r] : row0 + r;
    s_tab[r] = a.row_index[p] & a.index_mask;
    int64_t occurrences = 1;
    if (SUMMING) {
      const uint32_t j0 = a.seg_start[p], j1 = a.seg_start[p + 1];
      s_j0[r] = j0;
      s_len[r] = j1 - j0;
      s_grad[r] = static_cast<int64_t>(a.perm[j0]) * a.dim;   // the run's first gradient row
      if (a.cnts_out != nullptr) a.cnts_out[p] = static_cast<int64_t>(j1 - j0);
      occurrences = j1 - j0;
    } else {
      s_grad[r] = p * a.dim;
      if (a.average != 0) occurrences = a.run_cnts[p];
    }
    if (a.average != 0) s_div[r] = static_cast<float>(occurrences + (a.average == 2 ? 1 : 0));
    if (a.w_rows != nullptr) s_old[r] = static_cast<int64_t>(a.first_pos[p]) * a.dim;
  }
}

// acc + rows 2.. of a run, one after the other in sort order (which is occurrence order); four
// rows are requested at a time, the additions stay in order
template <typename V>
__device__ __forceinline__ V add_rest_of_run(const ListedRows& a, uint32_t j0, uint32_t len,
                                             int64_t col, V acc) {
  for (uint32_t j = j0 + 1; j < j0 + len; j += 4) {
    V row[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (j + t < j0 + len) {
        const int64_t q = a.perm[j + t];
        row[t] = __builtin_nontemporal_load(reinterpret_cast<const V*>(a.grad + q * a.dim + col));
      }
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
      if (j + t < j0 + len) acc = acc + row[t];
  }
  return acc;
}

template <int VEC, bool SUMMING>
__global__ __launch_bounds__(kThreads) void adagrad_listed_kernel(AdagradListedArgs a) {
  typedef typename Vf<VEC>::type V;
  __shared__ int64_t s_tab[kRows];
  __shared__ int64_t s_grad[kRows];
  __shared__ int64_t s_old[kRows];
  __shared__ uint32_t s_j0[kRows];
  __shared__ uint32_t s_len[kRows];
  __shared__ float s_div[kRows];
  int64_t first, cnt;
  listed_range(a.r, &first, &cnt);
  const int cpr = static_cast<int>(a.r.dim / VEC);
  for (int64_t row0 = first + static_cast<int64_t>(blockIdx.x) * kRows; row0 < cnt;
       row0 += static_cast<int64_t>(gridDim.x) * kRows) {
    const int64_t left = cnt - row0;
    const int rows_here = left < kRows ? static_cast<int>(left) : kRows;
    resolve_listed<SUMMING>(a.r, row0, rows_here, s_tab, s_grad, s_old, s_j0, s_len, s_div);
    __syncthreads();
    const int total = rows_here * cpr;
    for (int base = threadIdx.x; base < total; base += kThreads * kUnroll) {
      V g[kUnroll], s[kUnroll], w[kUnroll];
      V* sp[kUnroll];
      V* wp[kUnroll];
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        const int c = base + k * kThreads;
        if (c < total) {
          const int r = c / cpr;
          const int64_t col = static_cast<int64_t>(c - r * cpr) * VEC;
          const int64_t off = s_tab[r] * a.r.stride + col;
          sp[k] = reinterpret_cast<V*>(a.s + off);
          wp[k] = reinterpret_cast<V*>(a.w + off);
          g[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(a.r.grad + s_grad[r] + col));
          s[k] = *sp[k];
          w[k] = a.r.w_rows != nullptr ? *reinterpret_cast<const V*>(a.r.w_rows + s_old[r] + col)
                                       : *wp[k];
        }
      }
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        const int c = base + k * kThreads;
        if (c < total) {
          const int r = c / cpr;
          const int64_t col = static_cast<int64_t>(c - r * cpr) * VEC;
          if (SUMMING) {
            V acc = V(0.0f) + g[k];          // from +0.0f, like the segmented sum: -0.0f becomes +0.0f
            if (s_len[r] > 1) acc = add_rest_of_run<V>(a.r, s_j0[r], s_len[r], col, acc);
            g[k] = acc;
            if (a.r.sums_out != nullptr)
              *reinterpret_cast<V*>(a.r.sums_out + (row0 + r) * a.r.dim + col) = acc;
          }
          if (a.r.average != 0) g[k] = vdiv(g[k], V(s_div[r]));
          const V s1 = s[k] + g[k] * g[k];
          const V std_ = vsqrt(s1) + a.eps;
          const V w1 = w[k] - vdiv(a.lr * g[k], std_);
          *sp[k] = s1;
          *wp[k] = w1;
          if (a.w_out != nullptr) *reinterpret_cast<V*>(a.w_out + s_grad[r] + col) = w1;
        }
      }
    }
    __syncthreads();   // the row offsets are rewritten by the next round
  }
}

// SparseAdam over the same walk: the arithmetic of adam_kernel below, one table set per launch.
template <int VEC, bool SUMMING>
__global__ __launch_bounds__(kThreads) void adam_listed_kernel(AdamListedArgs a) {
  typedef typename Vf<VEC>::type V;
  __shared__ int64_t s_tab[kRows];
  __shared__ int64_t s_grad[kRows];
  __shared__ int64_t s_old[kRows];
  __shared__ uint32_t s_j0[kRows];
  __shared__ uint32_t s_len[kRows];
  __shared__ float s_div[kRows];
  __shared__ float s_c1[kRows];
  __shared__ float s_c2[kRows];
  int64_t first, cnt;
  listed_range(a.r, &first, &cnt);
  const int cpr = static_cast<int>(a.r.dim / VEC);
  for (int64_t row0 = first + static_cast<int64_t>(blockIdx.x) * kRows; row0 < cnt;
       row0 += static_cast<int64_t>(gridDim.x) * kRows) {
    const int64_t left = cnt - row0;
    const int rows_here = left < kRows ? static_cast<int>(left) : kRows;
    resolve_listed<SUMMING>(a.r, row0, rows_here, s_tab, s_grad, s_old, s_j0, s_len, s_div);
    // thread r wrote s_tab[r] itself: the step counter and the bias corrections of its row
    for (int r = threadIdx.x; r < rows_here; r += kThreads) {
      float* sp = a.step + s_tab[r];
      const float step = *sp + 1.0f;
      *sp = step;
      s_c1[r] = 1.0f - powf(a.beta1, step);
      s_c2[r] = 1.0f - powf(a.beta2, step);
    }
    __syncthreads();
    const int total = rows_here * cpr;
    for (int base = threadIdx.x; base < total; base += kThreads * kUnroll) {
      V g[kUnroll], m[kUnroll], v[kUnroll], w[kUnroll];
      V* mp[kUnroll];
      V* vp[kUnroll];
      V* wp[kUnroll];
      float c1[kUnroll], c2[kUnroll];
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        const int c = base + k * kThreads;
        if (c < total) {
          const int r = c / cpr;
          const int64_t col = static_cast<int64_t>(c - r * cpr) * VEC;
          const int64_t off = s_tab[r] * a.r.stride + col;
          mp[k] = reinterpret_cast<V*>(a.m + off);
          vp[k] = reinterpret_cast<V*>(a.v + off);
          wp[k] = reinterpret_cast<V*>(a.w + off);
          g[k] = __builtin_nontemporal_load(reinterpret_cast<const V*>(a.r.grad + s_grad[r] + col));
          m[k] = *mp[k];
          v[k] = *vp[k];
          w[k] = a.r.w_rows != nullptr ? *reinterpret_cast<const V*>(a.r.w_rows + s_old[r] + col)
                                       : *wp[k];
          c1[k] = s_c1[r];
          c2[k] = s_c2[r];
        }
      }
#pragma unroll
      for (int k = 0; k < kUnroll; ++k) {
        const int c = base + k * kThreads;
        if (c < total) {
          const int r = c / cpr;
          if (SUMMING) {
            const int64_t col = static_cast<int64_t>(c - r * cpr) * VEC;
            V acc = V(0.0f) + g[k];
            if (s_len[r] > 1) acc = add_rest_of_run<V>(a.r, s_j0[r], s_len[r], col, acc);
            g[k] = acc;
            if (a.r.sums_out != nullptr)
              *reinterpret_cast<V*>(a.r.sums_out + (row0 + r) * a.r.dim + col) = acc;
          }
          if (a.r.average != 0) g[k] = vdiv(g[k], V(s_div[r]));
          const V m1 = a.beta1 * m[k] + a.one_minus_beta1 * g[k];
          const V v1 = a.beta2 * v[k] + a.one_minus_beta2 * (g[k] * g[k]);
          const V mc = vdiv(m1, V(c1[k]));
          const V vc = vdiv(v1, V(c2[k]));
          const V upd = vdiv(a.lr * mc, vsqrt(vc) + a.eps);
          *mp[k] = m1;
          *vp[k] = v1;
          *wp[k] = w[k] - upd;
        }
      }
    }
    __syncthreads();   // the row offsets are rewritten by the next round
  }
}

template <int VEC>
__global__ __launch_bounds__(kThreads) void adam_kernel(AdamArgs a) {
  typedef typename Vf<VEC>::type V;
  __shared__ int64_t s_row[kRows];
  __shared__ uint8_t s_hot[kRows];
  __shared__ float s_c1[kRows];
  __shared__ float s_c2[kRows];
  __shared__ float s_div[kRows];
  const int rows_here = resolve_rows(a.r, s_row, s_hot, s_div);
  // per-row step counter and bias corrections (thread r owns row r in both loops)
  for (int r = threadIdx.x; r < rows_here; r += kThreads) {
    float* sp = (s_hot[r] ? a.hot_step : a.cold_step) + s_row[r];
    const float step = *sp + 1.0f;
    *sp = step;
    s_c1[r] = 1.0f - powf(a.beta1, step);
    s_c2[r] = 1.0f - powf(a.beta2, step);
  }
  __syncthreads();
  if (rows_here == 0) return;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRows;
  const int cpr = static_cast<int>(a.r.dim / VEC);
  const int total = rows_here * cpr;
  for (int base = threadIdx.x; base < total; base += kThreads * kUnroll) {
    V g[kUnroll], m[kUnroll], v[kUnroll], w[kUnroll];
    V* mp[kUnroll];
    V* vp[kUnroll];
    V* wp[kUnroll];
    float c1[kUnroll], c2[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int c = base + k * kThreads;
      if (c < total) {
        const int r = c / cpr;
        const int64_t col = static_cast<int64_t>(c - r * cpr) * VEC;
        const int64_t off = s_row[r] * a.r.dim + col;
        const bool hot = s_hot[r];
        mp[k] = reinterpret_cast<V*>((hot ? a.hot_m : a.cold_m) + off);
        vp[k] = reinterpret_cast<V*>((hot ? a.hot_v : a.cold_v) + off);
        wp[k] = reinterpret_cast<V*>((hot ? a.hot_w : a.cold_w) + off);
        g[k] = *reinterpret_cast<const V*>(a.r.grad + (row0 + r) * a.r.dim + col);
        m[k] = *mp[k];
        v[k] = *vp[k];
        w[k] = *wp[k];
        c1[k] = s_c1[r];
        c2[k] = s_c2[r];
      }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const int c = base + k * kThreads;
      if (c < total) {
        if (a.r.average != 0) g[k] = vdiv(g[k], V(s_div[c / cpr]));
        const V m1 = a.beta1 * m[k] + a.one_minus_beta1 * g[k];
        const V v1 = a.beta2 * v[k] + a.one_minus_beta2 * (g[k] * g[k]);
        const V mc = vdiv(m1, V(c1[k]));
        const V vc = vdiv(v1, V(c2[k]));
        const V upd = vdiv(a.lr * mc, vsqrt(vc) + a.eps);
        *mp[k] = m1;
        *vp[k] = v1;
        *wp[k] = w[k] - upd;
      }
    }
  }
}

bool aligned16(std::initializer_list<const void*> ps) {
  for (const void* p : ps)
    if (p && (align_of_ptr(p) % 16) != 0) return false;
  return true;
}

int check_rows(const int64_t* uids, const float* grad, int64_t max_rows, int64_t dim,
               const int64_t* sorted_hot, int64_t num_hot) {
  HADES_REQUIRE(max_rows >= 0 && dim >= 1, "max_rows must be >= 0 and dim >= 1");
  HADES_REQUIRE(num_hot >= 0, "num_hot must be >= 0");
  HADES_REQUIRE(max_rows == 0 || (uids && grad), "null pointer argument");
  HADES_REQUIRE(num_hot == 0 || sorted_hot, "sorted_hot is null but num_hot > 0");
  HADES_REQUIRE(dim * kRows < (int64_t(1) << 30), "dim too large");
  HADES_REQUIRE(ceil_div(max_rows > 0 ? max_rows : 1, kRows) < (int64_t(1) << 31), "too many rows");
  return HADES_OK;
}

// Grid of a listed walk.  Device tables: one block per kRows rows, capped.  Rows that cross the
// host link: a narrow grid that strides over the list (host_link_blocks: wider when the kernel
// reads and writes over the link than when it only writes there).
dim3 listed_grid(int64_t max_count, bool host_writes, bool host_reads) {
  int64_t blocks = ceil_div(max_count, kRows);
  if (blocks > 16384) blocks = 16384;
  if (host_writes || host_reads) {
    const int64_t cap = host_link_blocks(host_reads ? kLinkReadWrite : kLinkWriteOnly);
    if (blocks > cap) blocks = cap;
  }
  return dim3(static_cast<unsigned>(blocks));
}

int check_listed(const ListedRows& r, bool class_form) {
  HADES_REQUIRE(r.max_count >= 0 && r.dim >= 1, "the row count must be >= 0 and dim >= 1");
  HADES_REQUIRE(r.stride >= r.dim, "stride must be 0 or >= dim");
  HADES_REQUIRE(r.dim * kRows < (int64_t(1) << 30), "dim too large");
  if (r.max_count == 0) return HADES_OK;
  HADES_REQUIRE(r.row_index && r.grad, "null pointer argument");
  HADES_REQUIRE(r.average >= 0 && r.average <= 2, "average must be 0, 1 or 2");
  HADES_REQUIRE(r.average == 0 || r.perm != nullptr || r.run_cnts != nullptr,
                "averaging needs the occurrence counts of the rows (run_cnts)");
  if (class_form) {
    HADES_REQUIRE(r.which == 0 || r.which == 1, "which must be 0 or 1");
    HADES_REQUIRE(r.num_unique && r.class_split, "null pointer argument");
    HADES_REQUIRE((r.w_rows == nullptr) == (r.first_pos == nullptr),
                  "w_rows and first_pos go together");
  } else {
    HADES_REQUIRE(r.list && r.count, "null pointer argument");
  }
  return HADES_OK;
}

int launch_adagrad_listed(const AdagradListedArgs& a, void* stream) {
  const bool w_host = is_host_memory(a.w), s_host = is_host_memory(a.s);
  const dim3 grid = listed_grid(a.r.max_count, w_host || s_host,
                                s_host || (w_host && a.r.w_rows == nullptr)), block(kThreads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec4 = a.r.dim % 4 == 0 && a.r.stride % 4 == 0 &&
                    aligned16({a.r.grad, a.w, a.s, a.r.w_rows, a.w_out, a.r.sums_out});
  if (a.r.perm != nullptr) {
    if (vec4) HADES_LAUNCH((adagrad_listed_kernel<4, true>), grid, block, 0, st, a);
    else HADES_LAUNCH((adagrad_listed_kernel<1, true>), grid, block, 0, st, a);
  } else {
    if (vec4) HADES_LAUNCH((adagrad_listed_kernel<4, false>), grid, block, 0, st, a);
    else HADES_LAUNCH((adagrad_listed_kernel<1, false>), grid, block, 0, st, a);
  }
  return HADES_OK;
}

int launch_adam_listed(const ListedRows& r, float* w, float* step, float* m, float* v, float lr,
                       double beta1, double beta2, float eps, void* stream) {
  // 1 - beta is formed in double and rounded once, as in hades_adam_update
  const AdamListedArgs a{r, w, step, m, v, lr, static_cast<float>(beta1), static_cast<float>(beta2),
                         static_cast<float>(1.0 - beta1), static_cast<float>(1.0 - beta2), eps};
  const bool w_host = is_host_memory(w);
  const bool state_host = is_host_memory(step) || is_host_memory(m) || is_host_memory(v);
  const dim3 grid = listed_grid(r.max_count, w_host || state_host,
                                state_host || (w_host && r.w_rows == nullptr)), block(kThreads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec4 = r.dim % 4 == 0 && r.stride % 4 == 0 &&
                    aligned16({r.grad, w, m, v, r.w_rows, r.sums_out});
  if (r.perm != nullptr) {
    if (vec4) HADES_LAUNCH((adam_listed_kernel<4, true>), grid, block, 0, st, a);
    else HADES_LAUNCH((adam_listed_kernel<1, true>), grid, block, 0, st, a);
  } else {
    if (vec4) HADES_LAUNCH((adam_listed_kernel<4, false>), grid, block, 0, st, a);
    else HADES_LAUNCH((adam_listed_kernel<1, false>), grid, block, 0, st, a);
  }
  return HADES_OK;
}

}  // namespace
}  // namespace hades

using namespace hades;

extern "C" {

int hades_adagrad_update(const int64_t* uids, const float* grad, const int64_t* num_unique,
                         int64_t max_rows, int64_t dim, const int64_t* sorted_hot, int64_t num_hot,
                         const void* hot_index, float* hot_w, float* hot_s, float* cold_w, float* cold_s,
                         const int64_t* cnts, int average, float lr, float eps, void* stream) {
  int rc = check_rows(uids, grad, max_rows, dim, sorted_hot, num_hot);
  if (rc != HADES_OK) return rc;
  HADES_REQUIRE(average >= 0 && average <= 2, "average must be 0, 1 or 2");
  if (max_rows == 0) return HADES_OK;
  HADES_REQUIRE(average == 0 || cnts != nullptr, "averaging needs the occurrence counts of the rows (cnts)");
  HADES_REQUIRE(num_hot == 0 || (hot_w && hot_s), "hot tables are null but num_hot > 0");
  AdagradArgs a{{uids, grad, num_unique, max_rows, dim,
              HotSet{sorted_hot, num_hot, static_cast<const uint32_t*>(hot_index)}, cnts, average},
                hot_w, hot_s, cold_w, cold_s, lr, eps};
  const dim3 grid(static_cast<unsigned>(ceil_div(max_rows, kRows))), block(kThreads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dim % 4 == 0 && aligned16({grad, hot_w, hot_s, cold_w, cold_s}))
    HADES_LAUNCH_TIMED(HADES_KERNEL_ADAGRAD, st, (adagrad_kernel<4>), grid, block, 0, st, a);
  else
    HADES_LAUNCH_TIMED(HADES_KERNEL_ADAGRAD, st, (adagrad_kernel<1>), grid, block, 0, st, a);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

int hades_adagrad_update_listed(const int64_t* row_index, const float* grad, const int64_t* list,
                                const int64_t* count, int64_t max_count, int64_t dim, float* w,
                                float* s, int64_t stride, float* w_out, float lr, float eps,
                                void* stream) {
  HADES_REQUIRE(stride >= 0, "stride must be 0 or >= dim");
  const ListedRows r{row_index, grad, list, count, max_count, nullptr, nullptr, 0, int64_t(-1),
                     nullptr, nullptr, dim, stride == 0 ? dim : stride};
  const int rc = check_listed(r, false);
  if (rc != HADES_OK || max_count == 0) return rc;
  HADES_REQUIRE(w && s, "null pointer argument");
  return launch_adagrad_listed(AdagradListedArgs{r, w, s, w_out, lr, eps}, stream);
}

int hades_adagrad_update_class(const int64_t* ukeys, const float* grad, const int64_t* num_unique,
                               const int64_t* class_split, int which, int64_t key_mask,
                               int64_t max_rows, int64_t dim, float* w, float* s, int64_t stride,
                               const float* w_rows, const int32_t* first_pos,
                               const int64_t* run_cnts, int average, float lr, float eps,
                               void* stream) {
  HADES_REQUIRE(stride >= 0, "stride must be 0 or >= dim");
  ListedRows r{ukeys, grad, nullptr, nullptr, max_rows, num_unique, class_split, which,
               key_mask, w_rows, first_pos, dim, stride == 0 ? dim : stride};
  r.average = average;
  r.run_cnts = run_cnts;
  const int rc = check_listed(r, true);
  if (rc != HADES_OK || max_rows == 0) return rc;
  HADES_REQUIRE(w && s, "null pointer argument");
  return launch_adagrad_listed(AdagradListedArgs{r, w, s, nullptr, lr, eps}, stream);
}

int hades_adagrad_update_class_summing(const int64_t* ukeys, const float* grad_rows, int64_t n,
                                       int64_t key_bound, const int64_t* num_unique,
                                       const int64_t* class_split, int which, int64_t key_mask,
                                       int64_t dim, float* w, float* s, int64_t stride,
                                       const float* w_rows, const int32_t* first_pos,
                                       float* sums_out, int64_t* cnts_out, int average, float lr,
                                       float eps, void* workspace, size_t workspace_bytes,
                                       void* stream) {
  HADES_REQUIRE(stride >= 0, "stride must be 0 or >= dim");
  HADES_REQUIRE(n >= 0, "n must be >= 0");
  if (n == 0) return HADES_OK;
  ListedRows r{ukeys, grad_rows, nullptr, nullptr, n, num_unique, class_split, which,
               key_mask, w_rows, first_pos, dim, stride == 0 ? dim : stride};
  r.average = average;
  const int rv = combine_plan_views(workspace, workspace_bytes, n, dim, key_bound, &r.perm, &r.seg_start);
  if (rv != HADES_OK) return rv;
  const int rc = check_listed(r, true);
  if (rc != HADES_OK) return rc;
  HADES_REQUIRE(w && s, "null pointer argument");
  r.sums_out = sums_out;
  r.cnts_out = cnts_out;
  return launch_adagrad_listed(AdagradListedArgs{r, w, s, nullptr, lr, eps}, stream);
}

int hades_adam_update_class_summing(const int64_t* ukeys, const float* grad_rows, int64_t n,
                                    int64_t key_bound, const int64_t* num_unique,
                                    const int64_t* class_split, int which, int64_t key_mask,
                                    int64_t dim, float* w, float* step, float* m, float* v,
                                    int64_t stride, const float* w_rows, const int32_t* first_pos,
                                    float* sums_out, int64_t* cnts_out, int average, float lr,
                                    double beta1, double beta2, float eps, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  HADES_REQUIRE(stride >= 0, "stride must be 0 or >= dim");
  HADES_REQUIRE(n >= 0, "n must be >= 0");
  if (n == 0) return HADES_OK;
  ListedRows r{ukeys, grad_rows, nullptr, nullptr, n, num_unique, class_split, which,
               key_mask, w_rows, first_pos, dim, stride == 0 ? dim : stride};
  r.average = average;
  const int rv = combine_plan_views(workspace, workspace_bytes, n, dim, key_bound, &r.perm, &r.seg_start);
  if (rv != HADES_OK) return rv;
  const int rc = check_listed(r, true);
  if (rc != HADES_OK) return rc;
  HADES_REQUIRE(w && step && m && v, "null pointer argument");
  r.sums_out = sums_out;
  r.cnts_out = cnts_out;
  return launch_adam_listed(r, w, step, m, v, lr, beta1, beta2, eps, stream);
}

int hades_adam_update_listed(const int64_t* row_index, const float* grad, const int64_t* list,
                             const int64_t* count, int64_t max_count, int64_t dim, float* w,
                             float* step, float* m, float* v, int64_t stride, float lr,
                             double beta1, double beta2, float eps, void* stream) {
  HADES_REQUIRE(stride >= 0, "stride must be 0 or >= dim");
  const ListedRows r{row_index, grad, list, count, max_count, nullptr, nullptr, 0, int64_t(-1),
                     nullptr, nullptr, dim, stride == 0 ? dim : stride};
  const int rc = check_listed(r, false);
  if (rc != HADES_OK || max_count == 0) return rc;
  HADES_REQUIRE(w && step && m && v, "null pointer argument");
  return launch_adam_listed(r, w, step, m, v, lr, beta1, beta2, eps, stream);
}

int hades_adam_update_class(const int64_t* ukeys, const float* grad, const int64_t* num_unique,
                            const int64_t* class_split, int which, int64_t key_mask,
                            int64_t max_rows, int64_t dim, float* w, float* step, float* m,
                            float* v, int64_t stride, const float* w_rows,
                            const int32_t* first_pos, const int64_t* run_cnts, int average,
                            float lr, double beta1, double beta2, float eps, void* stream) {
  HADES_REQUIRE(stride >= 0, "stride must be 0 or >= dim");
  ListedRows r{ukeys, grad, nullptr, nullptr, max_rows, num_unique, class_split, which,
               key_mask, w_rows, first_pos, dim, stride == 0 ? dim : stride};
  r.average = average;
  r.run_cnts = run_cnts;
  const int rc = check_listed(r, true);
  if (rc != HADES_OK || max_rows == 0) return rc;
  HADES_REQUIRE(w && step && m && v, "null pointer argument");
  return launch_adam_listed(r, w, step, m, v, lr, beta1, beta2, eps, stream);
}

int hades_adam_update(const int64_t* uids, const float* grad, const int64_t* num_unique,
                      int64_t max_rows, int64_t dim, const int64_t* sorted_hot, int64_t num_hot,
                      const void* hot_index, float* hot_w, float* hot_step, float* hot_m, float* hot_v, float* cold_w,
                      float* cold_step, float* cold_m, float* cold_v, const int64_t* cnts,
                      int average, float lr, double beta1, double beta2, float eps, void* stream) {
  int rc = check_rows(uids, grad, max_rows, dim, sorted_hot, num_hot);
  if (rc != HADES_OK) return rc;
  HADES_REQUIRE(average >= 0 && average <= 2, "average must be 0, 1 or 2");
  if (max_rows == 0) return HADES_OK;
  HADES_REQUIRE(average == 0 || cnts != nullptr, "averaging needs the occurrence counts of the rows (cnts)");
  HADES_REQUIRE(num_hot == 0 || (hot_w && hot_step && hot_m && hot_v),
                "hot tables are null but num_hot > 0");
  // the betas arrive as doubles because the reference forms 1 - beta in Python double arithmetic
  // before the product with a float32 tensor rounds it (python/EmbCache/sparse_optim.py:641-642):
  // 1 - float(0.999) would be off by 1.3e-5 relative
  const float omb1 = static_cast<float>(1.0 - beta1);
  const float omb2 = static_cast<float>(1.0 - beta2);
  AdamArgs a{{uids, grad, num_unique, max_rows, dim,
              HotSet{sorted_hot, num_hot, static_cast<const uint32_t*>(hot_index)}, cnts, average},
             hot_w, hot_step, hot_m, hot_v, cold_w, cold_step, cold_m, cold_v,
             lr, static_cast<float>(beta1), static_cast<float>(beta2), omb1, omb2, eps};
  const dim3 grid(static_cast<unsigned>(ceil_div(max_rows, kRows))), block(kThreads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dim % 4 == 0 && aligned16({grad, hot_w, hot_m, hot_v, cold_w, cold_m, cold_v}))
    HADES_LAUNCH_TIMED(HADES_KERNEL_ADAM, st, (adam_kernel<4>), grid, block, 0, st, a);
  else
    HADES_LAUNCH_TIMED(HADES_KERNEL_ADAM, st, (adam_kernel<1>), grid, block, 0, st, a);
  HADES_LAUNCH_CHECK();
  return HADES_OK;
}

}  // extern "C"
