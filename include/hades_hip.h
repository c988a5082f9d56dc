/*
 * hades_hip.h - C ABI of libhades_hip.so, the MI355X (gfx950) implementation of
 * the HADES per-GPU embedding-cache hot path.
 *
 * Every entry point takes plain pointers, sizes and a HIP stream handle; no
 * torch types cross this boundary.  The caller owns all memory.  Entry points
 * return 0 on success and a non-zero code on failure; the message for the last
 * failure on the calling thread is returned by hades_last_error().  Nothing in
 * this library calls exit() or abort() (the reference's CUDA_CALL does:
 * src/utils.h:12-24).
 *
 * Pointers named "cold"/"cpu" may address pinned host memory (allocated with
 * hades_host_alloc / hipHostMalloc / torch pin_memory=True): kernels read and
 * write it zero-copy over the host link.  All other pointers are device memory.
 * Launches are asynchronous on `stream` (a hipStream_t passed as void*; NULL is
 * the default stream).  Tensors are dense row-major.
 *
 * The first group mirrors, one for one, the functions the reference binds in
 * src/pybind.cc:46-70 (declared in src/cuda/ops.h:9-41).  The second group are
 * the fused operators of the same path (sorted-set lookup, split + compaction,
 * combine, sparse Adagrad, cold-gradient accumulator).
 */
#ifndef HADES_HIP_H_
#define HADES_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of row payloads (reference: FLOAT_TYPE_SWITCH, src/utils.h:26-37) */
#define HADES_F32 0
#define HADES_F64 1
/* index type (reference: INTEGER_TYPE_SWITCH, src/utils.h:39-50) */
#define HADES_I32 0
#define HADES_I64 1
/* extra id types accepted by hades_split only (reference: AT_DISPATCH_ALL_TYPES,
 * src/cuda/split.cu:53-56; the floating-point cases of that dispatch are rejected) */
#define HADES_I16 2
#define HADES_I8 3
#define HADES_U8 4

/* status codes */
#define HADES_OK 0
#define HADES_ERR_ARG 1      /* bad argument (shape, dtype code, alignment, size) */
#define HADES_ERR_HIP 2      /* a HIP runtime call or kernel launch failed */
#define HADES_ERR_WORKSPACE 3 /* workspace too small */

/* combine modes */
#define HADES_COMBINE_FAST 0  /* fixed-shape tree sum: reproducible run to run, <=1e-5 rel. of exact */
#define HADES_COMBINE_EXACT 1 /* strictly sequential sum in occurrence order: bit-equal to CPU index_add_ */

const char* hades_last_error(void);
/* Version of this interface; raised whenever a signature changes, so that a binding can refuse a
 * library built from other sources. */
#define HADES_ABI_VERSION 131
int hades_version(void);

/* Kernel timing hook (no counterpart in the reference, whose scripts time whole calls from the
 * host: test/test_cached_fetch.py:51-56).  Arms a pair of hipEvent_t handles; from then on every
 * launch of the named kernel made by the calling thread records start_event before and
 * stop_event after itself, on the stream it is launched on.  kernel_id 0 disarms. */
#define HADES_KERNEL_NONE 0
#define HADES_KERNEL_CACHED_FETCH 1 /* row mover launched by hades_cached_fetch */
#define HADES_KERNEL_SEG_SUM 2      /* segmented row sum of hades_combine (FAST: chunk kernel; EXACT: exact kernel) */
#define HADES_KERNEL_ADAGRAD 3      /* hades_adagrad_update */
#define HADES_KERNEL_RADIX_PASS 4   /* scatter passes of the sort in hades_combine (the pair keeps the last pass) */
#define HADES_KERNEL_HASH_ACCUMULATE 5 /* hades_hash_accumulate */
#define HADES_KERNEL_ADAM 6         /* hades_adam_update */
#define HADES_KERNEL_LAST 6
int hades_profile_kernel(int kernel_id, void* start_event, void* stop_event);

/* Width, in workgroups, of the kernels whose table rows cross the host link (no counterpart in the
 * reference, whose row kernels are launched one block per 32 rows whatever the memory,
 * src/cuda/uva_fetch.cu:86-95).  use: 0 a row copy one way (gather from / scatter to a host table),
 * 1 an update that reads and writes host rows, 2 an update that only writes them.  blocks = 0
 * restores the default (16 / 128 / 40, or the HADES_HOST_LINK_BLOCKS, _RW, _WO environment
 * variables, which are read once, at first use).  Process-wide; meant for tuning and measurement. */
int hades_set_host_link_blocks(int use, int64_t blocks);
int64_t hades_get_host_link_blocks(int use);

/* ------------------------------------------------------------------------- */
/* Group 1: one entry point per function bound in src/pybind.cc:46-70          */
/* ------------------------------------------------------------------------- */

/* cudaPinPtr / cudaPin: RegisterPtr, PinTensor (src/cuda/pin_memory.cu:9-22).
 * Page-locks and maps an existing host allocation.  Returns HADES_ERR_HIP (and
 * clears the HIP error state) where the platform refuses hipHostRegister. */
int hades_pin(void* host_ptr, size_t bytes);
/* cudaUnpinPtr / cudaUnpin: UnregisterPtr, UnpinTensor (src/cuda/pin_memory.cu:15-26) */
int hades_unpin(void* host_ptr);
/* Pinned, device-mapped host allocation for the cold table where registering
 * existing memory is not possible.  The returned pointer is valid on host and device. */
int hades_host_alloc(void** out_ptr, size_t bytes);
int hades_host_free(void* ptr);
/* The same with flags.  HADES_HOST_NONCOHERENT asks for coarse-grained host memory: the GPU may keep
 * lines of it in its L2 and writes them back at kernel boundaries, so the host sees a kernel's
 * writes only after the stream has been synchronised (which is when the reference's trainers read
 * their tables anyway); in exchange reads and writes cross the host link in whole cache lines. */
#define HADES_HOST_NONCOHERENT 1u
int hades_host_alloc_flags(void** out_ptr, size_t bytes, unsigned flags);

/* create_shared_mem / open_shared_mem / release_shared_mem (src/shm/shared_memory.h:14-58):
 * a POSIX shared-memory segment mapped read-write; pin != 0 also registers the mapping with the
 * HIP runtime (cudaHostRegister in the reference).  create sizes the segment, open refuses a
 * segment smaller than `size`; release unregisters, unmaps, closes and unlinks.  On any failure
 * nothing stays mapped, open or (for create) linked, and an error code comes back where the
 * reference ends the process.  hades_shm_exists: SharedMemory::Exist (:104-112), 1 or 0. */
int hades_shm_create(const char* name, int64_t size, int pin, void** out_ptr, int64_t* out_fd);
int hades_shm_open(const char* name, int64_t size, int pin, void** out_ptr, int64_t* out_fd);
int hades_shm_release(const char* name, int64_t size, void* ptr, int64_t fd, int pin);
int hades_shm_exists(const char* name);

/* cudaFetch: CUDAFetch (src/cuda/uva_fetch.cu:28-45)
 *   dst[dst_index[i], :] = src[src_index[i], :]            for i in [0, n) */
int hades_fetch(const void* src, const void* src_index, void* dst, const void* dst_index,
                int64_t n, int64_t dim, int dtype, int itype, void* stream);

/* cudaFetch2: CUDAFetch2 (src/cuda/uva_fetch.cu:72-105); dim == 1 is the 1-D form (:64-70)
 *   dst[i, :] = src[src_index[i], :] */
int hades_fetch2(const void* src, const void* src_index, void* dst,
                 int64_t n, int64_t dim, int dtype, int itype, void* stream);

/* cudaFetchWithCache2: CUDAFetchWithCache2 (src/cuda/uva_fetch.cu:108-192)
 *   g = index_map[src_index[i]];  dst[i, :] = g != -1 ? gpu_src[g, :] : cpu_src[src_index[i], :] */
int hades_fetch_with_cache2(const void* cpu_src, const void* gpu_src, const void* src_index,
                            const void* index_map, void* dst,
                            int64_t n, int64_t dim, int dtype, int itype, void* stream);

/* cudaSet: CUDASet (src/cuda/uva_set.cu:11-68)
 *   dst[dst_index[i], :] = src[i, :]      (duplicate indices: one writer wins, unspecified which) */
int hades_set(const void* src, void* dst, const void* dst_index,
              int64_t n, int64_t dim, int dtype, int itype, void* stream);

/* cudaSetWithCache: CUDASetWithCache (src/cuda/uva_set.cu:71-153)
 *   g = index_map[dst_index[i]];  (g != -1 ? gpu_dst[g, :] : cpu_dst[dst_index[i], :]) = src[i, :] */
int hades_set_with_cache(const void* src, void* cpu_dst, void* gpu_dst, const void* dst_index,
                         const void* index_map,
                         int64_t n, int64_t dim, int dtype, int itype, void* stream);

/* cudaCombine: CUDACombine (src/cuda/uva_fetch.cu:195-227) - a row scatter despite
 * its name, identical to hades_set */
int hades_combine_scatter(const void* src, void* dst, const void* dst_index,
                          int64_t n, int64_t dim, int dtype, int itype, void* stream);

/* cudaReminder: Reminder / ReminderKernel (src/cuda/binary_search.cu:36-43,76-87)
 *   out[i] = in[i] % local_num_gpus   (C remainder: sign follows the dividend) */
int hades_reminder(const void* in, int64_t local_num_gpus, void* out,
                   int64_t n, int itype, void* stream);

/* cudaBinarySearch: CUDABinarySearch / BinarySearchKernel (src/cuda/binary_search.cu:11-21,45-59)
 *   out[i] = (upper_bound(range_partition, in[i]) - 1) * local_num_gpus + in[i] % local_num_gpus */
int hades_binary_search(const void* in, const void* range_partition, int64_t num_part,
                        int64_t local_num_gpus, void* out,
                        int64_t n, int itype, void* stream);

/* cudaBinarySearch2: CUDABinarySearch2 / BinarySearchKernel2 (src/cuda/binary_search.cu:24-33,61-74)
 *   out[i] = upper_bound(range, in[i]) = number of entries of the ascending `range` that are <= in[i] */
int hades_binary_search2(const void* in, const void* range, int64_t num_part, void* out,
                         int64_t n, int itype, void* stream);

/* cudaSplit: splitCUDA / _split (src/cuda/split.cu:13-56)
 *   v = class_table[ids[i]];  local[i] = v==0; remote_hot[i] = v==1; remote_cold[i] = v==2
 * The three masks are bool (1 byte) arrays of n entries, fully written (no prior zero-fill
 * needed).  class_table (int8) may be device or pinned host memory (test/test_pin.py:24-29). */
int hades_split(const void* ids, int id_type, const int8_t* class_table, int64_t n,
                uint8_t* local_mask, uint8_t* remote_hot_mask, uint8_t* remote_cold_mask,
                void* stream);

/* ------------------------------------------------------------------------- */
/* Group 2: fused operators of the same path                                  */
/* ------------------------------------------------------------------------- */

/* EmbCache lookup: membership + slot of each query in the ascending, duplicate-free hot-ID
 * set.  Closed form over BinarySearchKernel2 (src/cuda/binary_search.cu:24-33):
 *   pos = upper_bound(sorted_hot, q[i]);  loc[i] = (pos > 0 && sorted_hot[pos-1] == q[i]) ? pos-1 : -1
 * Replaces the dense index_map probe (python/EmbCache/cache.py:163-171) and the CPU
 * IndexCache round trip (python/EmbCache/dist_emb.py:184-185).  q, sorted_hot, loc: int64. */
int hades_lookup_sorted(const int64_t* q, int64_t n, const int64_t* sorted_hot, int64_t num_hot,
                        const void* hot_index, int64_t* loc, void* stream);

/* Optional bucket index over the hot set, about one bucket per hot id: an entry holds the first
 * position of its bucket in sorted_hot, the number of ids in it and the low bits of its first id,
 * so that a lookup is ONE 8-byte read for three queries in four (the query is the bucket's first
 * id, or the bucket is empty, or has one id) and one more search over the few ids of the bucket
 * for the rest, instead of log2(num_hot) dependent probes of the sorted array; results are
 * identical.  Build it once per hot set (the reference builds its dense index_map once per cache,
 * python/EmbCache/cache.py:163-171; this takes 8 - 16 bytes per hot id instead of 8 per table row) and
 * pass it as `hot_index` to the operators below; NULL there means plain binary search.  The
 * buffer is device memory, 16-byte aligned, hades_hot_index_bytes(num_hot) bytes. */
size_t hades_hot_index_bytes(int64_t num_hot);
int hades_hot_index_build(const int64_t* sorted_hot, int64_t num_hot, void* hot_index,
                          size_t hot_index_bytes, void* stream);

/* Hot/cold split of a looked-up batch with stable compaction (replaces cudaSplit + torch.nonzero,
 * python/EmbCache/dist_emb.py:174-191):  hot <=> loc[i] >= 0.
 *   hot_mask[i]  = loc[i] >= 0                              (bool[n])
 *   hot_pos      = ascending positions i with loc[i] >= 0   (int64, capacity n)
 *   cold_pos     = ascending positions i with loc[i] <  0   (int64, capacity n)
 *   counts[0..1] = {number hot, number cold}                (int64[2], device)
 * workspace: device scratch of hades_split_compact_workspace_bytes(n) bytes. */
size_t hades_split_compact_workspace_bytes(int64_t n);
int hades_split_compact(const int64_t* loc, int64_t n, uint8_t* hot_mask, int64_t* hot_pos,
                        int64_t* cold_pos, int64_t* counts, void* workspace, size_t workspace_bytes,
                        void* stream);

/* Lookup and hot/cold split in one call: hades_lookup_sorted followed by hades_split_compact, with
 * the slots written on the way (loc int64[n]).  This is the first step of the split schedule of
 * the reference's forward path (python/EmbCache/dist_emb.py:174-211: split first, then a gather
 * per class): the two position lists then drive hades_fetch_listed / hades_adagrad_update_listed
 * over the hot tables in HBM and over the cold tables on the host, on separate streams.
 * num_live (int64[1] on the device, may be NULL) limits the batch to its first num_live[0] entries
 * (the padded output of hades_combine): later entries are in neither list and get no slot (and
 * no sort key: num_live together with sort_keys is refused with HADES_ERR_ARG).
 * sort_keys (int64[n], may be NULL) receives a class-ordered sort key per query, for
 * hades_combine_plan_classed:  cold: the id itself;  hot: (1 << key_bits) | slot.  key_bits must
 * cover the table's ids (ids < 2^key_bits).  Sorted by this key a batch has its cold ids first, in
 * id order, then its hot ids in slot order (which is id order too), and the key of a hot run is
 * its row in the hot tables: one lookup per query serves the gather, the combine and the update.
 * hot_mask may be NULL.  Workspace as hades_split_compact. */
int hades_lookup_split(const int64_t* q, const int64_t* num_live, int64_t n,
                       const int64_t* sorted_hot, int64_t num_hot,
                       const void* hot_index, int64_t* loc, uint8_t* hot_mask, int64_t* hot_pos,
                       int64_t* cold_pos, int64_t* counts, int64_t* sort_keys, int key_bits,
                       void* workspace, size_t workspace_bytes, void* stream);

/* Three-way form of the same thing from the reference's class table (src/cuda/split.cu:11):
 * masks as hades_split, plus pos[k] = ascending positions of class k (each int64 capacity n) and
 * counts[0..2].  Any of the mask pointers may be NULL. */
int hades_split3_compact(const void* ids, int id_type, const int8_t* class_table, int64_t n,
                         uint8_t* mask0, uint8_t* mask1, uint8_t* mask2,
                         int64_t* pos0, int64_t* pos1, int64_t* pos2, int64_t* counts,
                         void* workspace, size_t workspace_bytes, void* stream);

/* cached_fetch keyed by the sorted hot set: lookup fused into the gather
 * (CUDAFetchWithCacheKernel2 semantics, src/cuda/uva_fetch.cu:108-130, with the
 * index_map probe replaced by the binary search above).
 *   loc = lookup(q[i]);  dst[i, :] = loc >= 0 ? hot_src[loc, :] : cold_src[q[i], :]
 * loc_out (int64[n]) may be NULL.  cold_src may be device or pinned host memory. */
int hades_cached_fetch(const void* cold_src, const void* hot_src, const int64_t* q, int64_t n,
                       const int64_t* sorted_hot, int64_t num_hot, const void* hot_index,
                       void* dst, int64_t* loc_out, int64_t dim, int dtype, void* stream);

/* Same gather when the slots are already known (loc from hades_lookup_sorted). */
int hades_cached_fetch_loc(const void* cold_src, const void* hot_src, const int64_t* q,
                           const int64_t* loc, int64_t n, void* dst,
                           int64_t dim, int dtype, void* stream);

/* cached_set keyed by the sorted hot set (CUDASetWithCacheKernel semantics,
 * src/cuda/uva_set.cu:71-93):
 *   loc = lookup(q[i]);  (loc >= 0 ? hot_dst[loc, :] : cold_dst[q[i], :]) = src[i, :] */
int hades_cached_set(const void* src, void* cold_dst, void* hot_dst, const int64_t* q, int64_t n,
                     const int64_t* sorted_hot, int64_t num_hot, const void* hot_index,
                     int64_t dim, int dtype, void* stream);

/* Row gather / scatter over one half of a split (the per-class gathers of
 * python/EmbCache/dist_emb.py:193-211, CUDAFetch2 / CUDASet semantics of src/cuda/uva_fetch.cu:72-105
 * and src/cuda/uva_set.cu:35-68, driven by a position list whose length stays on the device):
 *   fetch: for j < min(count[0], max_count): p = list[j];  dst[p, :] = src[src_index[p], :]
 *   set  : for j < min(count[0], max_count): p = list[j];  dst[dst_index[p], :] = src[p, :]
 * list int64[max_count] holds batch positions, *_index int64[positions] the table row of every
 * position (the slot from hades_lookup_split for the hot table, the id itself for the cold table),
 * count int64[1] on the device.  The table (src of fetch, dst of set) may be pinned host memory and
 * its rows may lie *_stride elements apart (0 = dim).  A negative count is treated as 0. */
int hades_fetch_listed(const void* src, int64_t src_stride, const int64_t* src_index,
                       const int64_t* list, const int64_t* count, int64_t max_count, void* dst,
                       int64_t dim, int dtype, void* stream);
int hades_set_listed(const void* src, void* dst, int64_t dst_stride, const int64_t* dst_index,
                     const int64_t* list, const int64_t* count, int64_t max_count, int64_t dim,
                     int dtype, void* stream);

/* hades_fetch_listed restricted to the positions whose table row src_index[p] is a member of the
 * ascending set sorted_set[0 .. min(set_count[0], set_max)); the other positions of dst are left as
 * they are.  It refreshes rows that were gathered ahead of an update: a trainer that knows the ids
 * of its next batch (the reference's data loader hands them out ahead of the step,
 * python/EmbCache/dist_emb.py:276-288 keeps them in its trace) gathers that batch's cold rows
 * while the current batch's update is still writing the table, and afterwards re-reads exactly
 * the rows that update wrote - sorted_set = the update's distinct cold ids - so that the batch
 * sees what a gather after the update would have seen. */
int hades_fetch_listed_in_set(const void* src, int64_t src_stride, const int64_t* src_index,
                              const int64_t* list, const int64_t* count, int64_t max_count,
                              const int64_t* sorted_set, const int64_t* set_count, int64_t set_max,
                              void* dst, int64_t dim, int dtype, void* stream);

/* combine: sort + dedup + segment-sum of duplicate-ID gradient rows; the arithmetic of
 * only_unique_grads (python/EmbCache/sparse_optim.py:132-139), which is also the
 * local-aggregation reduction (:310) over concatenated trainer batches.
 *   uids  = ascending distinct values of idx                (int64, capacity n)
 *   cnts  = occurrences of each                             (int64, capacity n)
 *   sums  = per-id sum of grad rows, fp32                   (float, capacity n x dim)
 *   num_unique[0] = U                                       (int64[1], device)
 * Entries at and beyond U are left unspecified.  id_bound > 0 promises 0 <= idx[i] < id_bound
 * (fewer sort passes); id_bound == 0 sorts all 64 bits as signed integers.
 * mode: HADES_COMBINE_FAST or HADES_COMBINE_EXACT.  n must be < 2^30.
 * Optional output (may be NULL): inverse[i] = index of idx[i] in uids (int32[n]).
 * If an id violates id_bound, num_unique[0] is set to -1 and the other outputs are unspecified;
 * every operator of this library that takes num_unique treats a negative value as "no live rows",
 * so nothing is read or written out of range downstream.  The workspace needs no initialisation.
 * hades_combine_workspace_bytes is the size to allocate; its tail (n x dim floats) is a staging
 * area in which HADES_COMBINE_EXACT lays out the rows of ids that occur 64 times or more, so that
 * their sums are bound by the chain of adds and not by one compute unit's row loads.  A workspace
 * of hades_combine_workspace_bytes_min (everything but that area) is accepted by every entry point
 * that takes a combine workspace; EXACT then sums such ids about three times more slowly, with
 * the same result. */
size_t hades_combine_workspace_bytes(int64_t n, int64_t dim);
size_t hades_combine_workspace_bytes_min(int64_t n, int64_t dim);
int hades_combine(const int64_t* idx, const float* grad, int64_t n, int64_t dim, int64_t id_bound,
                  int mode, int64_t* uids, float* sums, int64_t* cnts, int64_t* num_unique,
                  int32_t* inverse, void* workspace, size_t workspace_bytes, void* stream);

/* The sort under hades_combine (and under the bucketing, the accumulator's flush and the index
 * cache).  The reference gets its sort from torch.unique (python/EmbCache/sparse_optim.py:133-135);
 * here it is a stable LSD radix sort in one of two forms that give the same permutation:
 *   one_sweep = 1: one histogram kernel for all digits, then ONE kernel per digit in which
 *     every tile learns the digit counts of the tiles before it by looking back at what they have
 *     published.  Each such wait is bounded: after spin_limit fruitless re-reads a tile stops
 *     waiting, counts the keys before it from the pass's input itself and goes on - same result,
 *     and the first 32-bit word of the workspace (cleared by every sort) counts the tiles that did.
 *   one_sweep = 0 (default: the faster one on MI355X at every batch size measured): per digit a
 *     count kernel, for large batches a scan kernel, and a scatter kernel; no kernel ever waits for
 *     another block.
 * -1 leaves a setting as it is.  spin_limit 0 makes every tile that finds a predecessor not ready
 * give up at once (a way to exercise the recount from the host).  Process-wide; hades_sort_mode
 * returns the current form. */
int hades_sort_config(int one_sweep, int64_t spin_limit);
int hades_sort_mode(void);

/* The same in two halves.  The sort and the run boundaries depend on the ids alone, which a
 * trainer knows at forward time (python/EmbCache/dist_emb.py:276-288 saves them for the optimizer),
 * long before the gradients exist: hades_combine_plan can run then, on another stream, and
 * hades_combine_apply (the segmented row sums; also writes cnts) when the gradients arrive.
 * The plan lives in the workspace: apply must get the same n, dim, id_bound and workspace, after the
 * plan has finished, and the workspace must not be reused in between. */
int hades_combine_plan(const int64_t* idx, int64_t n, int64_t dim, int64_t id_bound, int64_t* uids,
                       int64_t* num_unique, int32_t* inverse, void* workspace,
                       size_t workspace_bytes, void* stream);
int hades_combine_apply(const float* grad, int64_t n, int64_t dim, int64_t id_bound, int mode,
                        float* sums, int64_t* cnts, const int64_t* num_unique, void* workspace,
                        size_t workspace_bytes, void* stream);

/* The combine over class-ordered keys (sort_keys of hades_lookup_split), in the same two halves,
 * with the class border kept on the device so that each class can go its own way:
 *   plan : as hades_combine_plan over `keys` (all below key_bound); ukeys = ascending distinct
 *          keys; class_split (int64[2], device) = {first sorted position, first run} whose key is
 *          >= threshold (= {n, num_unique} if there is none); first_pos (int32[n], may be NULL):
 *          the batch position of the first occurrence of every distinct key.
 *   apply: the segmented sums and counts of ONE class: which = 0 the runs below the threshold
 *          (rows [0, class_split[1]) of sums / cnts), which = 1 the runs at or above it.  The two
 *          calls together give exactly what hades_combine_apply gives; made one after the other
 *          they let the update of the first class start while the second class is still summed.
 * The reference has no such split (it combines once, python/EmbCache/sparse_optim.py:614, and
 * splits the distinct ids afterwards, :243-259); the arithmetic per id is the same. */
int hades_combine_plan_classed(const int64_t* keys, int64_t n, int64_t dim, int64_t key_bound,
                               int64_t threshold, int64_t* ukeys, int64_t* num_unique,
                               int64_t* class_split, int32_t* first_pos, void* workspace,
                               size_t workspace_bytes, void* stream);
int hades_combine_apply_class(const float* grad, int64_t n, int64_t dim, int64_t key_bound, int mode,
                              int which, float* sums, int64_t* cnts, const int64_t* num_unique,
                              const int64_t* class_split, void* workspace, size_t workspace_bytes,
                              void* stream);

/* hades_combine with the scratch memory inside the library.  No counterpart in the reference.  It
 * is for callers that cannot allocate device memory or hand over a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The call allocates and frees
 * nothing; its scratch is a fixed array of HADES_COMBINE_STATIC_SCRATCH_BYTES that every GPU the
 * library runs on holds until the process ends.  Same arguments and results as hades_combine
 * without the workspace pair.  A batch whose hades_combine_workspace_bytes_min(n, dim) exceeds the
 * array is refused with HADES_ERR_ARG (the limit admits e.g. 262 144 ids of dim 128).  All calls
 * on one GPU share that GPU's array: two calls that overlap in time on one GPU (different streams
 * or threads) race, and the array must not be relied on between calls.  The first call on a
 * device looks up the array's device address (hipGetSymbolAddress); make that call outside any
 * graph capture. */
#define HADES_COMBINE_STATIC_SCRATCH_BYTES (16u << 20)
int hades_combine_static(const int64_t* idx, const float* grad, int64_t n, int64_t dim,
                         int64_t id_bound, int mode, int64_t* uids, float* sums, int64_t* cnts,
                         int64_t* num_unique, int32_t* inverse, void* stream);

/* unique_grads (python/EmbCache/sparse_optim.py:142-157): in-place division of the first
 * num_unique[0] rows of sums by cnts (plus `one_plus` added to the divisor: the reference starts
 * the count from ones when a cnt vector is supplied, :145-148). */
int hades_rows_div_count(float* sums, const int64_t* cnts, const int64_t* num_unique,
                         int64_t max_rows, int64_t dim, int one_plus, void* stream);

/* Sparse Adagrad row update with the lookup, the state/weight gather and the scatter-back fused
 * (the reference ships SparseAdam only, python/EmbCache/sparse_optim.py:590-685; this is the same
 * gather -> row math -> scatter skeleton, state via cache.py:66-131, for Adagrad):
 *   for u < num_unique[0]:  id = uids[u]; g = grad[u, :]; loc = lookup(id)
 *     (w, s) = loc >= 0 ? (hot_w[loc], hot_s[loc]) : (cold_w[id], cold_s[id])
 *     s += g*g;  w -= lr * g / (sqrt(s) + eps)          (each operation rounded to fp32, no FMA)
 * uids must be duplicate-free.  num_unique may be NULL (then all max_rows rows are live).
 * sorted_hot may be NULL with num_hot == 0 (everything in the cold tables).
 * average: 0 the rows of grad are applied as they are; 1 row u is first divided by cnts[u], its number
 * of occurrences (the mean of unique_grads, python/EmbCache/sparse_optim.py:150-156); 2 by cnts[u] + 1
 * (:145-148).  cnts (int64, the counts hades_combine wrote) may be NULL when average is 0. */
int hades_adagrad_update(const int64_t* uids, const float* grad, const int64_t* num_unique,
                         int64_t max_rows, int64_t dim,
                         const int64_t* sorted_hot, int64_t num_hot, const void* hot_index,
                         float* hot_w, float* hot_s, float* cold_w, float* cold_s,
                         const int64_t* cnts, int average, float lr, float eps, void* stream);

/* The same Adagrad arithmetic over one half of a split, against one table pair:
 *   for j < min(count[0], max_count): p = list[j]; r = row_index[p]; g = grad[p, :]
 *     s[r*stride ..] += g*g;  w[r*stride ..] -= lr * g / (sqrt(s) + eps)
 * row_index is the slot (hot tables) or the id (cold tables) of every position of the combined
 * batch, list/count one of the two lists hades_lookup_split made of its distinct ids.  w and s may
 * be device or pinned host memory; rows lie `stride` floats apart (0 = dim), so the weight and
 * state row of an id may be stored next to each other (s = w + dim, stride = 2*dim): one burst
 * over the host link per cold row and direction instead of two.
 * w_out (optional, float[positions, dim], device): the new weight row of position p is also
 * written to row p of w_out, for a caller that wants the updated rows at hand (the cold-data cache
 * takes in the rows it just applied, python/EmbCache/server.py:499-544) without reading them back
 * over the link. */
int hades_adagrad_update_listed(const int64_t* row_index, const float* grad, const int64_t* list,
                                const int64_t* count, int64_t max_count, int64_t dim, float* w,
                                float* s, int64_t stride, float* w_out, float lr, float eps,
                                void* stream);

/* The same arithmetic over one class of a class-ordered combine: the rows u of (ukeys, grad) in
 * [0, class_split[1]) for which = 0 or [class_split[1], num_unique[0]) for which = 1; the table row
 * is ukeys[u] & key_mask (the id for the cold class, the slot for the hot class, whose keys carry
 * the class bit above key_mask).  No lookup: the keys already name the rows.
 * w_rows / first_pos (both or neither): take the OLD weight row of run u from row first_pos[u] of
 * w_rows - the rows the forward pass fetched for this very batch (hades_fetch_listed output) -
 * instead of reading it from the table again; the new row is still written to the table.  For a
 * cold table in host memory this halves what the update moves over the link.  Only valid while
 * nothing has written those table rows since they were fetched (one batch in flight per table:
 * the reference's trainers are of that kind, python/EmbCache/sparse_optim.py:590-685 runs between
 * a batch's forward and the next one's).
 * average: 0 the rows of grad are applied as they are (sums); 1 row u is divided by run_cnts[u], its
 * number of occurrences, first (the mean of unique_grads, python/EmbCache/sparse_optim.py:150-156);
 * 2 by run_cnts[u] + 1 (the reference's count starts from ones when counts come with the rows,
 * :145-148).  run_cnts (int64, the cnts of hades_combine_apply_class) may be NULL when average is 0. */
int hades_adagrad_update_class(const int64_t* ukeys, const float* grad, const int64_t* num_unique,
                               const int64_t* class_split, int which, int64_t key_mask,
                               int64_t max_rows, int64_t dim, float* w, float* s, int64_t stride,
                               const float* w_rows, const int32_t* first_pos,
                               const int64_t* run_cnts, int average, float lr, float eps,
                               void* stream);

/* hades_adagrad_update_class with the segmented sum of its class folded in: grad_rows holds one
 * gradient row per QUERY of the batch (float[n, dim]) and the gradient of run u is the sum of the
 * rows of its occurrences, added one after the other from +0.0f in occurrence order - for every run
 * exactly what hades_combine_apply_class computes in HADES_COMBINE_EXACT mode (CPU index_add_ order,
 * python/EmbCache/sparse_optim.py:136-138) - taken from the plan that hades_combine_plan_classed left
 * in `workspace` for the same n, dim and key_bound.  Meant for the class whose runs are short (the
 * cold class: nearly every cold id occurs once per batch), where it saves the segmented-sum launches
 * in front of an update that is bound by the host link anyway; a run of thousands of rows is walked
 * by one lane group and takes accordingly long.  sums_out (float[n, dim]) and cnts_out (int64[n]),
 * both optional, receive the summed row and the number of occurrences of every run of the class.
 * average as in hades_adagrad_update_class, with the run length as the number of occurrences (the
 * division happens after sums_out is written: sums_out keeps the sums). */
int hades_adagrad_update_class_summing(const int64_t* ukeys, const float* grad_rows, int64_t n,
                                       int64_t key_bound, const int64_t* num_unique,
                                       const int64_t* class_split, int which, int64_t key_mask,
                                       int64_t dim, float* w, float* s, int64_t stride,
                                       const float* w_rows, const int32_t* first_pos,
                                       float* sums_out, int64_t* cnts_out, int average, float lr,
                                       float eps, void* workspace, size_t workspace_bytes,
                                       void* stream);

/* SparseAdam row update, same fusion (python/EmbCache/sparse_optim.py:632-657,681):
 *   step += 1; m = b1*m + (1-b1)*g; v = b2*v + (1-b2)*g*g
 *   w -= lr * (m / (1 - b1^step)) / (sqrt(v / (1 - b2^step)) + eps)
 * step: float[N] / float[H]; m, v, w: float[., dim].  cnts / average as in hades_adagrad_update
 * (the reference's update always averages: sparse_optim.py:607-614). */
int hades_adam_update(const int64_t* uids, const float* grad, const int64_t* num_unique,
                      int64_t max_rows, int64_t dim,
                      const int64_t* sorted_hot, int64_t num_hot, const void* hot_index,
                      float* hot_w, float* hot_step, float* hot_m, float* hot_v,
                      float* cold_w, float* cold_step, float* cold_m, float* cold_v,
                      const int64_t* cnts, int average,
                      float lr, double beta1, double beta2, float eps, void* stream);

/* The SparseAdam arithmetic of hades_adam_update over one half of a split, against one table
 * set (the per-class form of python/EmbCache/sparse_optim.py:590-685 with the state gathers and
 * scatters of python/EmbCache/cache.py:66-131 fused in): positions, row_index, list and count as
 * in hades_adagrad_update_listed; step is float[rows of the table]; w, m and v have rows `stride`
 * floats apart (0 = dim) and may be device or pinned host memory. */
int hades_adam_update_listed(const int64_t* row_index, const float* grad, const int64_t* list,
                             const int64_t* count, int64_t max_count, int64_t dim, float* w,
                             float* step, float* m, float* v, int64_t stride, float lr,
                             double beta1, double beta2, float eps, void* stream);

/* SparseAdam over one class of a class-ordered combine; arguments as in
 * hades_adagrad_update_class, tables as in hades_adam_update_listed. */
int hades_adam_update_class(const int64_t* ukeys, const float* grad, const int64_t* num_unique,
                            const int64_t* class_split, int which, int64_t key_mask,
                            int64_t max_rows, int64_t dim, float* w, float* step, float* m,
                            float* v, int64_t stride, const float* w_rows,
                            const int32_t* first_pos, const int64_t* run_cnts, int average,
                            float lr, double beta1, double beta2, float eps, void* stream);

/* SparseAdam over one class with the segmented sum folded in; arguments as in
 * hades_adagrad_update_class_summing, tables as in hades_adam_update_listed. */
int hades_adam_update_class_summing(const int64_t* ukeys, const float* grad_rows, int64_t n,
                                    int64_t key_bound, const int64_t* num_unique,
                                    const int64_t* class_split, int which, int64_t key_mask,
                                    int64_t dim, float* w, float* step, float* m, float* v,
                                    int64_t stride, const float* w_rows, const int32_t* first_pos,
                                    float* sums_out, int64_t* cnts_out, int average, float lr,
                                    double beta1, double beta2, float eps, void* workspace,
                                    size_t workspace_bytes, void* stream);

/* Cold-gradient accumulator (delayed synchronisation): an open-addressing hash table in HBM,
 * int64 key -> fp32[dim] running sum and an int64 count.  Restates on the GPU the arithmetic of
 * EmbCacheServer._accumulate_gradients_cold_remote (python/EmbCache/server.py:546-562): per unique
 * incoming id  buf[slot] += g; cnt[slot] += c; key[slot] = id.
 * num_slots must be a power of two.  keys: int64[num_slots] (empty = -1), accum: float[num_slots,dim],
 * cnt: int64[num_slots].  Precondition: the ids of one call are duplicate-free (combine first);
 * duplicates inside a call race on the count and the row.
 * status[0] (int32, device, sticky, cleared by the caller) collects error bits: 1 the table was
 * full and a row was dropped; 2 more live entries than the flush capacity (nothing emitted);
 * 4 a stored id was outside [0, id_bound] at flush time (rows emitted, but not in ascending
 * order); 8 a negative id was offered to accumulate (its row was dropped: -1 marks an empty slot).
 * slot_stride (int64 words; 0 = 1): the key of slot i is keys[i * slot_stride] and its count
 * cnt[i * slot_stride], so that key and count of a slot may share one 16-byte record
 * (cnt = keys + 1, slot_stride = 2): a probe and the count update then touch one memory sector
 * instead of two. */
int hades_hash_clear(int64_t* keys, float* accum, int64_t* cnt, int64_t num_slots, int64_t dim,
                     int64_t slot_stride, void* stream);
int hades_hash_accumulate(int64_t* keys, float* accum, int64_t* cnt, int64_t num_slots,
                          const int64_t* ids, const float* grad, const int64_t* in_cnt,
                          const int64_t* num_rows, int64_t max_rows, int64_t dim,
                          int32_t* status, int64_t slot_stride, void* stream);
/* Flush: emit every live slot as (id, sum row, count) in ascending id order, then clear the table
 * (evident intent of python/EmbCache/server.py:413-419; see the note on :414 in the oracle).
 *   out_ids int64[cap], out_sums float[cap, dim], out_cnts int64[cap], num_out int64[1] (device)
 * cap bounds the number of live slots emitted (status bit 2 and num_out[0] = 0 if exceeded). */
size_t hades_hash_flush_workspace_bytes(int64_t num_slots, int64_t cap);
int hades_hash_flush(int64_t* keys, float* accum, int64_t* cnt, int64_t num_slots, int64_t dim,
                     int64_t id_bound, int64_t* out_ids, float* out_sums, int64_t* out_cnts,
                     int64_t* num_out, int64_t cap, int32_t* status, int64_t slot_stride,
                     void* workspace, size_t workspace_bytes, void* stream);

/* Pre-exchange bucketing: what swap_gradients does on one GPU before the all-to-all
 * (python/EmbCache/sparse_optim.py:33-50), in one call and without a host synchronisation:
 *   owner[i] = ids[i] % local_num_gpus                               when range_partition == NULL (:36)
 *            = (upper_bound(range_partition, ids[i]) - 1) * local_num_gpus
 *              + ids[i] % local_num_gpus                             otherwise (:38-39)
 *   stable sort by owner (:41); ids_out / cnt_out / grad_out = inputs in that order (:42-45);
 *   split_sizes[g] = number of rows owned by g, g in [0, num_owners) (:48-52, int64 on the device)
 *   perm_out[j] (optional) = input position of output row j.
 * grad (dim columns of dtype) and cnt are optional, each together with its output.
 * Rows keep their input order inside a bucket.  If an owner falls outside [0, num_owners) (a
 * negative id, an id beyond the last range), every entry of split_sizes is -1 and the other
 * outputs are unspecified. */
size_t hades_bucket_workspace_bytes(int64_t n);
int hades_bucket_by_owner(const int64_t* ids, int64_t n, const int64_t* range_partition,
                          int64_t num_part, int64_t local_num_gpus, int64_t num_owners,
                          const void* grad, int64_t dim, int dtype, const int64_t* cnt,
                          int64_t* ids_out, void* grad_out, int64_t* cnt_out,
                          int64_t* split_sizes, int64_t* perm_out, void* workspace,
                          size_t workspace_bytes, void* stream);

/* Set-associative index cache on the device: SACacheIndex<int64, int64> of src/cache/cache.h:11-259
 * over the 8-entry lines of src/cache/cache_line.h (bound as EmbCacheLib.IndexCache,
 * src/pybind.cc:17-36).  State is two caller-owned device arrays:
 *   line_ids int64[lines * 8]  (-1 = empty entry),  line_age int32[lines * 8]  (LRU ages);
 * an id lives in line id % lines and its loc is line * 8 + entry.  Negative ids are never cached
 * (loc -1, nothing changes): a batch whose length is only known on the device can be padded with
 * -1 and passed at its capacity.  Batches are handled in input order line by line, which is what the reference's
 * loops give with one OpenMP thread.
 *   init          constructor + _init_cache (cache.h:41-48, cache_line.h:13-18)
 *   add           _add (cache.h:51-91): loc of each id after insertion, -1 if its line has no victim
 *   lookup        lookupkernel2 (src/cache/lookup.cu:15-45): loc or -1, the cache is not changed
 *   lookup_touch  _lookup (cache.h:93-107): loc or -1, a hit ages its line (access_loc)
 *   reset         _reset (cache.h:109-121): ids that are present give their entry back
 *   getall        _getall (cache.h:123-137) + get_valid_entries_ (:180-185): live (id, loc) pairs in
 *                 loc order, at most cap; num_out[0] = pairs written, num_valid[0] = live entries
 *                 (either may be NULL, not both) */
int hades_sacache_init(int64_t* line_ids, int32_t* line_age, int64_t lines, void* stream);
size_t hades_sacache_workspace_bytes(int64_t n); /* add and lookup_touch */
int hades_sacache_add(int64_t* line_ids, int32_t* line_age, int64_t lines, const int64_t* ids,
                      int64_t n, int64_t* locs, void* workspace, size_t workspace_bytes,
                      void* stream);
int hades_sacache_lookup(const int64_t* line_ids, int64_t lines, const int64_t* ids, int64_t n,
                         int64_t* locs, void* stream);
int hades_sacache_lookup_touch(int64_t* line_ids, int32_t* line_age, int64_t lines,
                               const int64_t* ids, int64_t n, int64_t* locs, void* workspace,
                               size_t workspace_bytes, void* stream);
int hades_sacache_reset(int64_t* line_ids, int32_t* line_age, int64_t lines, const int64_t* ids,
                        int64_t n, void* stream);
size_t hades_sacache_getall_workspace_bytes(int64_t lines);
int hades_sacache_getall(const int64_t* line_ids, int64_t lines, int64_t* ids_out,
                         int64_t* locs_out, int64_t* num_out, int64_t* num_valid, int64_t cap,
                         void* workspace, size_t workspace_bytes, void* stream);

/* Gradient side of the cold-data cache with the reference's per-row staleness rule: the
 * arithmetic of the cache server over slot arrays in device memory.  A slot is a loc of the index
 * cache above (remote part) or id - id_offset (dense local part, locs == NULL, grad_idx == NULL).
 * Slot arrays: emb_buf / grad_buf float[num_slots, dim], grad_cnt / iter_count / iter_threshold
 * int32[num_slots], grad_idx int64[num_slots].
 *   insert      _update_cache (python/EmbCache/server.py:499-544): locs = what hades_sacache_add
 *               returned for ids, line_ids = the index cache after that add.  For rows with
 *               locs[r] >= 0 whose id holds that entry (an id evicted later in the same batch does
 *               not): emb_buf[loc] = rows[r]; grad_buf[loc] = 0; grad_cnt[loc] = 0; grad_idx[loc] = -1
 *   accumulate  _accumulate_gradients_cold_remote (:546-562) / _cold_local (:564-574): for rows
 *               with a slot: grad_idx[s] = id; iter_threshold[s] = threshold[id] (if given);
 *               grad_buf[s] += grad[r]; grad_cnt[s] += 1.  Rows must name distinct slots.
 *   flush       _send_staled_gradients (:346-419, :421-497): slots with grad_cnt > 0 and
 *               (iter_count >= iter_threshold or grad_cnt >= cnt_threshold) are written out in slot
 *               order as (id, gradient row, count); they are zeroed, iter_count = 0, and their id is
 *               taken out of the index cache (line_ids / line_age, may be NULL); every other slot
 *               with grad_cnt > 0 ages by one.  num_out[0] = rows written (<= out_cap; if more were
 *               due, bit 1 of the first workspace word is set and the rest leaves with the next
 *               flush).
 * The reference zeroes gradient rows through a temporary copy (:414, :489, :537), which leaves them
 * unchanged; the evident intent, zeroing, is what these entry points do. */
int hades_coldcache_insert(const int64_t* locs, const int64_t* ids, const int64_t* line_ids,
                           const float* rows, int64_t n, int64_t dim, int64_t num_slots,
                           float* emb_buf, float* grad_buf, int32_t* grad_cnt, int64_t* grad_idx,
                           void* stream);
int hades_coldcache_accumulate(const int64_t* locs, const int64_t* ids, const float* grad,
                               int64_t n, int64_t dim, int64_t id_offset, int64_t num_slots,
                               const int32_t* threshold, float* grad_buf, int32_t* grad_cnt,
                               int64_t* grad_idx, int32_t* iter_threshold, void* stream);
size_t hades_coldcache_flush_workspace_bytes(int64_t num_slots);
int hades_coldcache_flush(int64_t num_slots, int64_t dim, int32_t cnt_threshold,
                          int64_t id_offset, float* grad_buf, int32_t* grad_cnt,
                          const int64_t* grad_idx, int32_t* iter_count,
                          const int32_t* iter_threshold, int64_t* line_ids, int32_t* line_age,
                          int64_t lines, int64_t* out_ids, float* out_grads, int64_t* out_cnts,
                          int64_t* num_out, int64_t out_cap, void* workspace,
                          size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HADES_HIP_H_ */
