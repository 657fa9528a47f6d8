/*
 * libzen_hip: MI355X (gfx950) implementation of ZEN's sparse-gradient
 * select / hash-partition / merge path.  Plain C ABI: device pointers, sizes
 * and a HIP stream.  No torch types, no hidden allocation, no host
 * synchronisation: every call only enqueues kernels on `stream`.
 *
 * Conventions
 *   - every pointer is DEVICE memory unless a comment says "host";
 *   - `dtype` is ZEN_F32 or ZEN_BF16 (bf16 as 16-bit patterns);
 *   - `stream` is a hipStream_t (NULL = the null stream);
 *   - the return value is a host-side code (ZEN_OK, ZEN_E...); conditions only
 *     the device can see are OR-ed into `*status` (device int32, written by
 *     kernels with atomic-or; the caller zeroes it and reads it after a sync);
 *   - `workspace` is caller-provided scratch of at least the size the matching
 *     `*_workspace` function returns; contents are undefined on return;
 *   - indices are int32 (N < 2^31) as in the reference (functions_cuda.cpp:25-26
 *     narrows numel() to int).
 *
 * Citations are file:line in the reference (Jabir0/ZEN_repro).
 */
#ifndef ZEN_HIP_H
#define ZEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ZEN_ABI_VERSION 3 /* 2: zen_encode_merge (its argument struct), zen_sample_threshold, zen_round_compact, path code 3; 3: next_n .. next_table */

#define ZEN_F32 0
#define ZEN_BF16 1

/* host return codes */
#define ZEN_OK 0
#define ZEN_EINVAL (-1)     /* bad argument (null, size, dtype, alignment) */
#define ZEN_EHIP (-2)       /* a HIP runtime call failed, see zen_last_error() */
#define ZEN_EWORKSPACE (-3) /* workspace too small */

/* device status bits */
#define ZEN_STAT_SERIAL_OVERFLOW 1 /* a partition had more overflow entries than serial slots */
#define ZEN_STAT_CAPACITY 2        /* more output entries than `capacity`; the excess was dropped */
#define ZEN_STAT_INTERNAL 4        /* a bounded in-kernel wait expired; outputs are invalid */
#define ZEN_STAT_BAD_INDEX 8       /* merge/decode saw an index outside [0, dense_n); it was skipped */
#define ZEN_STAT_RETRY 16          /* the fast path met keys piled on a few values; outputs unspecified:
                                      call again with ZEN_MODE_GENERAL */

/* `mode` argument of the sort-based entry points */
#define ZEN_MODE_FAST 0    /* bucket sort in LDS; flags ZEN_STAT_RETRY on pathological key distributions */
#define ZEN_MODE_GENERAL 1 /* one radix pass per 8 key bits; any input */
/* OR-ed into the `mode` of zen_merge: the caller vouches that the first zen_merge_zero_bytes() bytes of the
   workspace are zero.  The call then skips the kernel that clears them, and leaves them zero again when it
   returns ZEN_OK and raises neither ZEN_STAT_RETRY nor ZEN_STAT_INTERNAL (after those the caller clears
   them).  A workspace allocated zeroed and used for zen_merge only therefore needs no clearing at all. */
#define ZEN_MODE_ZEROED 0x100
/* OR-ed into the `mode` of zen_load_balance: zen_load_balance_prepare has run for this call (see there);
   ZEN_MODE_SECOND names the second of the two sets of sampling memory (without ZEN_MODE_PREPARED: the call takes
   its own sample in that set, e.g. because the first holds the sample of another call that is still to come). */
#define ZEN_MODE_PREPARED 0x200
#define ZEN_MODE_SECOND 0x400
#define ZEN_MODE_DISCARD 0x800 /* zen_load_balance_prepare: drop a sample that no call will pick up */
/* OR-ed into the `mode` of zen_load_balance with k > 0: thr[0] is a key close to the k-th largest magnitude, for
   example what an earlier call on a gradient of the same kind wrote to thr_out.  The call then takes no sample:
   it lists everything from a little below that key (4/128 of its power of two) and picks the exact k-th
   largest among those.  If fewer than k elements qualify, or far too many, ZEN_STAT_RETRY is raised as when a
   sample misleads.  Paths that do not sample ignore the key. */
#define ZEN_MODE_FLOOR 0x1000
/* zen_load_balance, zen_merge, zen_decode_dense: with ZEN_MODE_FAST, stay off the path for up to a few million
   entries (at most 256 wide buckets, one resident workgroup each, whose launches the library keeps from
   overlapping on a device) and take the bucket-slab path wherever that fits.  Results are the same. */
#define ZEN_MODE_SLABS 0x2000

int zen_abi_version(void);

/* host string describing the last ZEN_EHIP / ZEN_EINVAL on this thread */
const char *zen_last_error(void);

/* ------------------------------------------------------------------ hash */

/*
 * out[t] = (h1(t) % n) / (n / partitions) for t in [0, n).
 * Replaces hash_index (extensions/cuda/functions_cuda.cpp:30-36) and
 * hash_index_cuda (functions_cuda_kernel.cu:169-177, 201-205).
 * n % partitions != 0 is allowed and can yield `partitions` as in the
 * reference; n < partitions is ZEN_EINVAL (the reference divides by zero).
 */
int zen_hash_index(int32_t *out, int64_t n, int partitions, void *stream);

/*
 * Ascending list of t in [0,n) per partition, concatenated into out[n]
 * (int64), counts[p] = length of list p.  Replaces calculate_mapping
 * (comm.py:52-56).  Indices whose partition id equals `partitions`
 * (n % partitions != 0) are left out, as in the reference.
 */
size_t zen_mapping_workspace(int64_t n, int partitions);
int zen_mapping(int64_t n, int partitions, int64_t *out, int64_t *counts,
                void *workspace, size_t workspace_bytes, int32_t *status, void *stream);

/* ---------------------------------------------------------------- bitmap */

/*
 * Bitmap form of an index set, the wire format of the second exchange.
 * mapping_p[mapping_n] is one partition's ascending index list (zen_mapping).
 *
 * zen_bitmap_encode replaces encode_bitmap (comm.py:59-85): bit j of the
 * bitmap is set iff some idx[i] has lower-bound position j in mapping_p
 * (torch.searchsorted, left side, comm.py:61-63; an index that is no member
 * marks the next member, as in the reference).  Bits are numbered from the
 * least significant bit of byte 0 (weights 2^0..2^7 per byte, comm.py:79-83).
 * The bitmap is written as zen_bitmap_words(mapping_n) little-endian 32-bit
 * words, i.e. (mapping_n + 7) / 8 meaningful bytes followed by zero padding up
 * to a multiple of four; `bitmap_words` must be 4-byte aligned and that large.
 * idx holds idx_n entries (int32, or int64 if idx64) in any order, of which
 * only the first *idx_n_dev count if that device counter is given.  rank_at is
 * optional: the rank dictionary zen_bitmap_ranks builds for this mapping and
 * `numel` (zen_bitmap_rank_words(numel) words, 16-byte aligned: members below
 * every multiple of 512 and one membership bit per index value; to be kept
 * with the mapping, which the reference caches too, comm.py:132-134).  With it
 * a lookup is two loads instead of a search through the list from an
 * interpolated guess, and indices >= numel count as beyond the last member.
 * For indices in [0, numel) the result is the same with and without.  A position past the end
 * of the list (torch raises an IndexError there) sets ZEN_STAT_BAD_INDEX.
 *
 * zen_bitmap_decode replaces decode_bitmap (comm.py:87-99) for one rank's
 * bitmap: out receives mapping_p[j] for every set bit j < mapping_n in
 * ascending order, *out_count their number (ZEN_STAT_CAPACITY if it exceeds
 * `capacity`; the excess is dropped).  Bits at positions >= mapping_n are
 * ignored (comm.py:97); a bitmap of fewer than (mapping_n + 7) / 8 bytes is
 * ZEN_EINVAL (the reference's mask would not fit the list).  No alignment
 * requirement on `bitmap`.
 */
size_t zen_bitmap_words(int64_t mapping_n);
size_t zen_bitmap_rank_words(int64_t numel);
int zen_bitmap_ranks(const int64_t *mapping_p, int64_t mapping_n, int64_t numel, uint32_t *rank_at, void *stream);
int zen_bitmap_encode(const int64_t *mapping_p, int64_t mapping_n, const void *idx, int idx64, int64_t idx_n,
                      const int64_t *idx_n_dev, const uint32_t *rank_at, int64_t numel, uint32_t *bitmap_words,
                      int32_t *status, void *stream);
size_t zen_bitmap_decode_workspace(int64_t mapping_n);
int zen_bitmap_decode(const int64_t *mapping_p, int64_t mapping_n, const uint8_t *bitmap, int64_t bitmap_bytes,
                      int64_t *out, int64_t capacity, int64_t *out_count, void *workspace, size_t workspace_bytes,
                      int32_t *status, void *stream);

/* ---------------------------------------------------------------- insert */

/*
 * In-place hash-table insert of every nonzero index of `input`.
 * Replaces sparse_balance (functions_cuda.cpp:15-28) and sparse_balance_cuda
 * with its three kernels (functions_cuda_kernel.cu:97-167, 180-199).
 * memory[m] and serial[serial_n] must be zero on entry; offset[partitions]
 * must hold the serial base offsets (extensions/cuda/functions.py:8-11) and
 * ends as base + number of tickets.  The result is the one the reference
 * kernel gives when its threads run in ascending order: a slot belongs to
 * the smallest index that probes it, serial entries are ascending per
 * partition.  Tickets beyond a partition's serial region are dropped and
 * flagged (ZEN_STAT_SERIAL_OVERFLOW) instead of written out of bounds.
 * m % partitions != 0 is ZEN_EINVAL.
 */
int zen_sparse_balance(const void *input, int dtype, int64_t n,
                       int32_t *memory, int64_t m,
                       int32_t *serial, int64_t serial_n,
                       int32_t *offset, int partitions, int rehash,
                       int32_t *status, void *stream);

/* ---------------------------------------------------------------- select */

/*
 * thr[0] = magnitude key (bit pattern with the sign cleared) of the k-th
 * largest |input|, thr[1] = number of elements whose key >= thr[0].
 * Replaces topk(...)[0].min() in compress (train.py:81-82) with the whole
 * tensor (or a caller-gathered sample) as the multiset.  1 <= k <= n.
 */
size_t zen_topk_threshold_workspace(void);
int zen_topk_threshold(const void *input, int dtype, int64_t n, int64_t k,
                       uint32_t *thr, void *workspace, size_t workspace_bytes,
                       void *stream);

/*
 * The threshold compress() applies (train.py:75-84): thr as for
 * zen_topk_threshold over the multiset input[sample_index[j]], j < s, the
 * sample the reference draws with torch.randint and gathers with
 * tensor[sample_index] before its topk.  sample_index: int64 positions on the
 * device, each in [0, n) (one outside sets ZEN_STAT_BAD_INDEX and counts as a
 * zero); 1 <= k <= s.  One gather kernel writes the sample into the workspace,
 * the radix select of zen_topk_threshold runs on it; nothing is allocated and
 * nothing waits for the device.
 */
size_t zen_sample_threshold_workspace(int64_t s, int dtype);
int zen_sample_threshold(const void *input, int dtype, int64_t n,
                         const int64_t *sample_index, int64_t s, int64_t k,
                         uint32_t *thr, void *workspace,
                         size_t workspace_bytes, int32_t *status,
                         void *stream);

/*
 * zen_topk_threshold without a workspace argument and without any allocation.
 * No counterpart in the reference: it is for callers that cannot allocate or
 * carry a workspace (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  The radix select's counters and histogram
 * (8448 bytes) live in a static device array inside the library, one copy per
 * GPU, held until the process ends.  Same arguments otherwise, same result.
 * n > ZEN_TOPK_STATIC_MAX_N is ZEN_EINVAL.  All calls on one GPU share that
 * array: calls that overlap on one GPU (two streams, two host threads) race;
 * calls in stream order do not, each clears the array before it counts.  The
 * first call on a device looks the array's address up
 * (hipGetSymbolAddress); make it outside graph capture.
 */
#define ZEN_TOPK_STATIC_MAX_N 0x7fffffffll
int zen_topk_threshold_static(const void *input, int dtype, int64_t n, int64_t k,
                              uint32_t *thr, void *stream);

/*
 * out[i] = key(input[i]) >= thr[0] ? input[i] : 0.  Replaces
 * torch.where(tensor_abs >= threshold, tensor, 0) (train.py:83).
 */
int zen_compress(const void *input, int dtype, int64_t n, const uint32_t *thr,
                 void *out, void *stream);

/*
 * Ordered compaction: ascending indices i with key(i) >= max(thr[0], 1) and
 * their values.  thr == NULL selects the nonzero elements, which is
 * encode_sparse_tensor (comm.py:47-50).  out_idx is int64 when idx64 != 0,
 * else int32.  *out_count (int64) receives the number found, which may
 * exceed `capacity` (then ZEN_STAT_CAPACITY is set and the excess dropped).
 */
size_t zen_select_workspace(int64_t n, int dtype);
int zen_select(const void *input, int dtype, int64_t n, const uint32_t *thr,
               void *out_idx, int idx64, void *out_val, int64_t capacity,
               int64_t *out_count, void *workspace, size_t workspace_bytes,
               int32_t *status, void *stream);

/* ---------------------------------------------------------- load balance */

/*
 * Fused select + insert + slot-order compaction.  Replaces
 * TensorPartition.load_balance (tensor_load_balance.py:13-51) and, with
 * thr != NULL or k > 0, compress (train.py:75-84) in front of it.
 * Selection: thr == NULL and k == 0: the nonzero elements; thr != NULL: key >=
 * max(thr[0], 1); k > 0: the k largest magnitudes, ties at the k-th kept (thr
 * must be NULL unless ZEN_MODE_FLOOR says what it is; thr_out, if not NULL,
 * receives that key and the number selected).  In ZEN_MODE_FAST the k-th largest is found with one pass over
 * the tensor (sampled floor, exact refinement among the candidates); if the
 * sample misleads, ZEN_STAT_RETRY is raised and nothing valid is produced.
 * Output: out_idx / out_val hold partition 0's entries, then partition 1's,
 * ...; inside a partition, table entries in ascending slot order followed by
 * that partition's serial entries in ascending index order; splits[p] (int64)
 * is partition p's length.  m is the table size of
 * tensor_load_balance.py:15-16; the serial capacity is n / partitions / 10
 * per partition (tensor_load_balance.py:18).
 * `table` is int32[m] scratch that must be all zero on entry and is all zero
 * again on return (so one allocation serves every call, and no call spends a
 * kernel on clearing counters: those live in the table too); after a call that
 * raised ZEN_STAT_RETRY or ZEN_STAT_INTERNAL, or returned an error code, its
 * contents are undefined and the caller clears it.  ZEN_MODE_GENERAL keeps the owner of every probed slot in
 * it, like the reference; ZEN_MODE_FAST sorts the selected entries by their
 * level-1 slot instead and only borrows a corner of the table as a hash map
 * for the few entries that collide (ZEN_STAT_RETRY if there are too many).
 */
size_t zen_load_balance_workspace(int64_t n, int64_t m, int dtype, int64_t capacity, int partitions);
int zen_load_balance(const void *input, int dtype, int64_t n, int64_t m,
                     int partitions, int rehash, const uint32_t *thr, int64_t k,
                     uint32_t *thr_out, int32_t *out_idx, void *out_val,
                     int64_t capacity, int64_t *splits, int32_t *table, int mode,
                     void *workspace, size_t workspace_bytes,
                     int32_t *status, void *stream);

/*
 * The part of a top-k zen_load_balance call (k > 0, ZEN_MODE_FAST) that only needs the tensor: the sample
 * that gives the one-pass selection its floor.  Taken ahead, on another stream, it runs beside whatever the
 * main stream is still busy with (the previous gradient bucket's sort and placement, say) instead of in front
 * of this call's pass over the tensor.  Same input, sizes, k, table and workspace as the zen_load_balance
 * call that follows with mode | ZEN_MODE_PREPARED (that call must be ordered after this one: an event, a
 * stream wait); `mode` is ZEN_MODE_FAST, with ZEN_MODE_SECOND for the second of two sets of sampling memory,
 * which lets a caller prepare call i + 1 while call i (prepared with the other set) is in flight; a set may be
 * prepared again once the call that used it has finished.  A sample that no call will pick up after all is
 * dropped with mode | ZEN_MODE_DISCARD (same arguments; the table is not all zero before that).  On paths with
 * nothing to take ahead the function does nothing and the flag is ignored.  No counterpart in the reference.
 */
int zen_load_balance_prepare(const void *input, int dtype, int64_t n, int64_t m, int partitions, int64_t k,
                             int64_t capacity, int32_t *table, int mode, void *workspace,
                             size_t workspace_bytes, void *stream);

/*
 * Which implementation a zen_load_balance call with these sizes takes: 0 = owner table (the general
 * mode), 1 = sort-based owner resolution, 2 = bucket slabs (large inputs whose expected output is a small
 * fraction of the table: one streaming pass, then per-bucket sorts inside LDS), 3 = wide buckets (the same
 * for an expected output of up to a few million entries: at most 256 buckets, one resident workgroup each,
 * two launches).  No counterpart in the reference; tests and benchmarks use it to know what they measured.
 */
int zen_load_balance_path(int64_t n, int64_t m, int dtype, int64_t capacity, int partitions, int64_t k, int mode);

/* ----------------------------------------------------------------- merge */

/*
 * Merge r received (index, value) entries: sum values of equal indices in
 * fp32, in the order the entries appear, drop sums equal to zero, return the
 * rest in ascending index order.  Replaces decode_sparse_tensors +
 * encode_sparse_tensor of the first exchange (comm.py:32-50, 125-127) without
 * the dense intermediate.  idx is int32 (idx64_in == 0) or int64.  out_idx is
 * int64 when idx64_out != 0.  out_val is fp32.  *out_count is int64.
 * `mode` is ZEN_MODE_FAST or ZEN_MODE_GENERAL (both give identical results),
 * optionally with ZEN_MODE_ZEROED.
 */
size_t zen_merge_workspace(int64_t r, int64_t dense_n);
size_t zen_merge_zero_bytes(void); /* see ZEN_MODE_ZEROED; the same for every r and dense_n */
/* 0 = radix sort (general mode), 1 = one bucket pass + per-range sorts, 2 = bucket slabs, 3 = wide buckets; see
   zen_load_balance_path */
int zen_merge_path(int64_t r, int64_t dense_n, int mode);
int zen_merge(const void *idx, int idx64_in, const void *val, int dtype,
              int64_t r, int64_t dense_n,
              void *out_idx, int idx64_out, float *out_val, int64_t capacity,
              int64_t *out_count, int mode, void *workspace, size_t workspace_bytes,
              int32_t *status, void *stream);

/*
 * The merged entries on their way to the second exchange: comm.py:125-127
 * scatters the sums into a dense tensor of the gradient's type and takes its
 * nonzeros again; here every fp32 sum of zen_merge's output is rounded once to
 * `dtype` and the entries whose sum rounds to zero are dropped, the rest keep
 * their ascending order.  idx / out_idx: int32 or int64 (idx64), *count
 * entries on the device (at most `capacity` are looked at); out_val: `dtype`.
 * out_idx / out_val need room for `capacity` entries and must not be the
 * inputs.  Nothing waits for the device.
 */
size_t zen_round_compact_workspace(int64_t capacity);
int zen_round_compact(const void *idx, int idx64, const float *sums,
                      const int64_t *count, int64_t capacity, int dtype,
                      void *out_idx, void *out_val, int64_t *out_count,
                      void *workspace, size_t workspace_bytes,
                      int32_t *status, void *stream);

/*
 * One step of the path in one call: zen_load_balance of the rank's own gradient and zen_merge of the entries it
 * received, with the arguments of those two calls (the received values have the gradient's type `dtype`).
 * Replaces the two halves of LoadBalanceAllreduce.zen_sparse_comm around the first exchange (comm.py:118-127:
 * load_balance before it, decode_sparse_tensors + encode_sparse_tensor after it) for a caller that holds the
 * received entries of the previous bucket while it encodes the next one.  The encode is enqueued on `stream`,
 * the merge on `merge_stream` (NULL: on `stream`, behind the encode); results and status words are those of
 * the two calls.  No counterpart in the reference: it exists so that a hook crosses the language boundary once
 * per bucket.
 */
typedef struct zen_encode_merge_args {
  /* zen_load_balance */
  const void *input;
  int dtype;
  int64_t n, m;
  int partitions, rehash;
  const uint32_t *thr;
  int64_t k;
  uint32_t *thr_out;
  int32_t *out_idx;
  void *out_val;
  int64_t capacity;
  int64_t *splits;
  int32_t *table;
  int mode;
  void *workspace;
  size_t workspace_bytes;
  int32_t *status;
  /* zen_merge */
  const void *recv_idx;
  int recv_idx64;
  const void *recv_val;
  int64_t r, dense_n;
  void *merged_idx;
  int merged_idx64;
  float *merged_val;
  int64_t merged_capacity;
  int64_t *merged_count;
  int merge_mode;
  void *merge_workspace;
  size_t merge_workspace_bytes;
  int32_t *merge_status;
  void *stream, *merge_stream;
  /* Optional (NULL / 0: none): the gradient of the NEXT call on this workspace, of this one's type and
     partitions, and that call's k.  On the fast paths the pass over `input` then also takes the sample that
     gives the next call's selection its floor (its workgroups do it when they are through with their own
     tensor: no kernel of its own, nothing that waits), in the set of sampling memory this call does not use.
     The next call says so like after zen_load_balance_prepare: ZEN_MODE_PREPARED, with ZEN_MODE_SECOND unless
     THIS call's mode has ZEN_MODE_SECOND.  zen_encode_merge_samples_next tells whether a call with these sizes
     does it (the other paths ignore the fields).  next_input must be readable in the order of `stream`.
       A next call of another size (gradient buckets differ in length) names its own n, m, capacity and table
     in next_n, next_m, next_capacity and next_table (0 / NULL: this call's); its sizes must take path 2 or 3
     (zen_load_balance_path), or the call is refused with ZEN_EINVAL: only those paths keep sampling memory in
     their table.  The workspace must be large enough for either call. */
  const void *next_input;
  int64_t next_k;
  int64_t next_n, next_m, next_capacity;
  int32_t *next_table;
} zen_encode_merge_args;
int zen_encode_merge_samples_next(int64_t n, int64_t m, int dtype, int64_t capacity, int partitions, int64_t k,
                                  int mode);
int zen_encode_merge(const zen_encode_merge_args *args);

/*
 * dense[0..dense_n) = 0, then dense[idx[j]] += val[j] with fp32 accumulation
 * in entry order, rounded once to `dtype`.  Replaces decode_sparse_tensors
 * (comm.py:32-44), whose result is a dense tensor in the value dtype.
 */
size_t zen_decode_dense_workspace(int64_t r, int64_t dense_n);
int zen_decode_dense(const void *idx, int idx64_in, const void *val, int dtype,
                     int64_t r, void *dense, int64_t dense_n, int mode,
                     void *workspace, size_t workspace_bytes,
                     int32_t *status, void *stream);

/*
 * The same for payloads that arrive as `nlists` strictly ascending index lists back to back (list l is
 * idx[list_start[l] .. list_start[l + 1]), list_start a HOST array of nlists + 1 offsets, at most 64 lists):
 * the second exchange of the sparse all-reduce, where every rank receives all ranks' merged shards
 * (comm.py:142-145), and method 1, where it receives all ranks' own selections (comm.py:113-117).  No sort
 * and no cleared dense tensor: one workgroup per tile of the dense tensor gathers its stretch of every list
 * and writes the tile once.  Same result as zen_decode_dense, bit for bit (lists may share indices).  A list
 * that is not strictly ascending or an index outside [0, dense_n) raises ZEN_STAT_RETRY: the dense tensor
 * is then unspecified and the caller repeats with zen_decode_dense.
 */
size_t zen_decode_dense_sorted_workspace(int64_t dense_n, int nlists);
int zen_decode_dense_sorted(const void *idx, int idx64_in, const void *val, int dtype,
                            const int64_t *list_start, int nlists, void *dense, int64_t dense_n,
                            void *workspace, size_t workspace_bytes, int32_t *status, void *stream);

/*
 * The second exchange with bitmaps in one pass: every rank's bitmap (bit j of list p = the j-th index of
 * partition p, comm.py:59-85) and value list straight into the dense gradient.  Replaces decode_bitmap for
 * all ranks followed by decode_sparse_tensors (comm.py:87-99, 136-145) without the indices, the member lists
 * (mapping) or a cleared dense tensor in between.
 *   zen_bitmap_dense_dict builds, once per (numel, partitions), what stands in for the mapping the reference
 * caches (comm.py:132-134): per tile of 8192 indices the places of the tile's indices ordered by partition (16
 * bits each) and the members of every partition below the tile (zen_bitmap_dense_dict_bytes bytes, a little
 * over two per element, 16-byte aligned).  members, if not
 * NULL, is a HOST array that receives the partitions' list lengths (this synchronises on the stream).
 *   zen_bitmap_dense: bitmaps / values hold the lists back to back, list p at byte bitmap_start[p] (of
 * bitmap_start[p + 1] - bitmap_start[p] bytes) and element value_start[p]; both offset arrays are HOST arrays
 * of partitions + 1 entries; at most 64 lists.  dense[t] = 0.0 + value for every index whose bit is set, 0
 * elsewhere: what scatter_add_ into zeros leaves (comm.py:35-39; lists of different partitions never share an
 * index).  Bits beyond a list's length are ignored (comm.py:97).  A bitmap shorter than its list, or more
 * set bits than values, raises ZEN_STAT_BAD_INDEX (the reference raises an index error); the missing ones
 * count as unset / zero.
 */
size_t zen_bitmap_dense_dict_bytes(int64_t numel, int partitions);
int zen_bitmap_dense_dict(int64_t numel, int partitions, void *dict, int64_t *members, void *stream);
size_t zen_bitmap_dense_workspace(int64_t numel, int partitions);
int zen_bitmap_dense(const void *dict, int64_t numel, int partitions, const uint8_t *bitmaps,
                     const int64_t *bitmap_start, const void *values, int dtype, const int64_t *value_start,
                     void *dense, void *workspace, size_t workspace_bytes, int32_t *status, void *stream);

/* --------------------------------------------------------------- utility */

/*
 * Stable ascending sort of (key, value) pairs on the low `bits` bits of the
 * key; count is read from *count_dev if that is not NULL, else `count`.
 * No counterpart in the reference (torch ops sort internally); exposed
 * because both fused paths are built on it and tests exercise it directly.
 * keys/vals are sorted in place.
 */
size_t zen_sort_pairs_workspace(int64_t max_count);
int zen_sort_pairs(uint32_t *keys, uint32_t *vals, int64_t max_count,
                   const uint32_t *count_dev, int bits,
                   void *workspace, size_t workspace_bytes, int32_t *status, void *stream);

/*
 * The same for keys that spread evenly over [0, sentinel), as hash slots and
 * hashed indices do: one scatter pass into 511 key ranges, then every range
 * sorted inside LDS.  Pairs with key >= sentinel come last in no particular
 * order.  A key range too full for LDS sets ZEN_STAT_RETRY in *status (order
 * then unspecified; use zen_sort_pairs).  zen_bucket_sort_fits tells whether
 * (max_count, sentinel) is in the supported range; workspace as zen_sort_pairs.
 * No counterpart in the reference.
 */
int zen_bucket_sort_fits(int64_t max_count, uint32_t sentinel);
int zen_bucket_sort_pairs(uint32_t *keys, uint32_t *vals, int64_t max_count,
                          const uint32_t *count_dev, uint32_t sentinel,
                          void *workspace, size_t workspace_bytes, int32_t *status, void *stream);

/*
 * Reads `bytes` bytes (16-byte aligned) with coalesced non-temporal 16-byte
 * loads and does nothing else: the rate a read-only pass over a tensor can reach
 * on the machine at hand, to set beside the published peak when a streaming
 * kernel is judged.  *sink is a device word the kernel may write.  No counterpart
 * in the reference; benchmarks time it.
 */
int zen_stream_read(const void *input, size_t bytes, uint32_t *sink, void *stream);

/*
 * Per-kernel timing with HIP events recorded on the launch stream, for
 * benchmarks.  The reference's counterpart is its nvtx ranges
 * (tensor_load_balance.py:25-38, comm.py:66-144).  zen_profile_enable(1)
 * clears earlier samples and starts recording; zen_profile_read synchronises
 * on the recorded events of one tag and returns their summed duration and the
 * number of launches.  An event between two kernels costs a few microseconds
 * on the device: zen_profile_only(tag) limits the recording to one tag (a
 * negative tag lifts the limit), and zen_profile_every(n) to every n-th
 * launch of a tag, counted from zen_profile_enable (n = 1: all of them).
 * Process-wide; with recording off a tagged launch site only reads a flag.
 */
int zen_profile_enable(int on);
int zen_profile_only(int tag);
int zen_profile_every(int n);
int zen_profile_tags(void);
const char *zen_profile_name(int tag);
int zen_profile_read(int tag, double *total_ms, int64_t *launches);

#ifdef __cplusplus
}
#endif
#endif
