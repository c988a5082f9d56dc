// TEST INFRASTRUCTURE ONLY.  Drives the reference's own cache_line class - compiled from
// src/cache/cache_line.h where it lies in the reference tree (the Makefile passes its directory
// with -I; nothing of it is copied here) - through the loops of SACacheIndex in
// src/cache/cache.h:51-135.  cache.h itself needs torch, CUDA and the shared-memory layer and is
// not built; its four loops (_add :51-91, _lookup :93-107, _reset :109-121, _getall :123-137) are
// restated below and run sequentially, i.e. in the order OpenMP would give with one thread
// (with more threads the reference's result depends on which thread reaches a line first).
// The stateless lookup follows lookupkernel2 (src/cache/lookup.cu:15-45), which works on a copy
// of the line and therefore leaves the access table alone.
#include <cstddef>
#include <cstdint>
#include <tuple>

#include "cache_line.h"

namespace {
using Line = distemb::cache_line<int64_t, int64_t, CACHE_LINE_SIZE>;
struct Index {
  Line* lines;
  size_t index_size;
};
}  // namespace

extern "C" {

void* ref_sacache_new(int64_t cache_size) {
  Index* ix = new Index;
  ix->index_size = (cache_size + CACHE_LINE_SIZE - 1) / CACHE_LINE_SIZE;  // cache.h:139
  ix->lines = new Line[ix->index_size];                                   // ctor: ids -1, ages 0
  return ix;
}

void ref_sacache_free(void* h) {
  Index* ix = static_cast<Index*>(h);
  delete[] ix->lines;
  delete ix;
}

int64_t ref_sacache_lines(void* h) { return static_cast<int64_t>(static_cast<Index*>(h)->index_size); }

void ref_sacache_add(void* h, const int64_t* ids, int64_t len, int64_t* locs) {
  Index* ix = static_cast<Index*>(h);
  for (int64_t i = 0; i < len; i++) {
    Line& line = ix->lines[ids[i] % ix->index_size];
    int idx;
    bool is_exist;
    std::tie(idx, is_exist) = line.find_or_empty_entry(ids[i]);
    if (idx >= 0) {
      if (!is_exist) line.set_id(idx, ids[i]);
      locs[i] = line.compute_loc(ids[i] % ix->index_size, idx);
    } else {
      const int lru = line.find_lru();
      if (lru == -1) {
        locs[i] = -1;
      } else {
        line.set_id(lru, ids[i]);
        locs[i] = line.compute_loc(ids[i] % ix->index_size, lru);
      }
    }
  }
}

void ref_sacache_lookup(void* h, const int64_t* ids, int64_t len, int64_t* locs) {
  Index* ix = static_cast<Index*>(h);
  for (int64_t i = 0; i < len; i++) {
    Line& line = ix->lines[ids[i] % ix->index_size];
    const int e = line.find(ids[i]);
    if (e == -1) {
      locs[i] = -1;
    } else {
      locs[i] = line.compute_loc(ids[i] % ix->index_size, e);
      line.access_loc(e);
    }
  }
}

void ref_sacache_lookup_stateless(void* h, const int64_t* ids, int64_t len, int64_t* locs) {
  Index* ix = static_cast<Index*>(h);
  for (int64_t i = 0; i < len; i++) {
    Line line = ix->lines[ids[i] % ix->index_size];  // a copy, as in the kernel
    const int e = line.find(ids[i]);
    locs[i] = e == -1 ? -1 : line.compute_loc(ids[i] % ix->index_size, e);
  }
}

void ref_sacache_reset(void* h, const int64_t* ids, int64_t len) {
  Index* ix = static_cast<Index*>(h);
  for (int64_t i = 0; i < len; i++) {
    Line& line = ix->lines[ids[i] % ix->index_size];
    const int e = line.find(ids[i]);
    if (e != -1) line.set_id(e, -1);
  }
}

int64_t ref_sacache_valid(void* h) {
  Index* ix = static_cast<Index*>(h);
  int64_t v = 0;
  for (size_t i = 0; i < ix->index_size; i++) v += ix->lines[i].get_valid_entries();
  return v;
}

// returns the number of entries written (at most len)
int64_t ref_sacache_getall(void* h, int64_t* ids, int64_t* locs, int64_t len) {
  Index* ix = static_cast<Index*>(h);
  int64_t k = 0;
  for (size_t i = 0; i < ix->index_size && k < len; i++)
    for (int j = 0; j < CACHE_LINE_SIZE && k < len; j++)
      if (ix->lines[i].get_id(j) != -1) {
        ids[k] = ix->lines[i].get_id(j);
        locs[k] = ix->lines[i].compute_loc(static_cast<int>(i), j);
        k++;
      }
  return k;
}

}  // extern "C"
