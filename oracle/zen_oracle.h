/*
 * CPU oracle for ZEN's sparse-gradient encode / hash-partition / merge path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a sequential restatement, in plain C, of
 * the algorithm in the reference (Jabir0/ZEN_repro).  It exists to check the
 * HIP library; nothing in the product path may link, load or call it.
 *
 * Citations are file:line in the reference tree.
 *
 * Parity pinning (the reference ships no tests or golden vectors):
 *   zen_oracle_hash           closed-form known answers, Horner == expanded,
 *                             seed-difference identity, python big-int sweep
 *   zen_oracle_hash_index     part(1..8) known answer, range + histogram
 *                             invariants
 *   zen_oracle_sparse_balance brute-force python model on tiny inputs,
 *                             min-tid-owner fixed point equivalence,
 *                             schedule-independent invariants
 *   zen_oracle_load_balance   numpy flatnonzero restatement over the table
 *   zen_oracle_kth_key/select numpy partition / torch.topk on CPU
 *   zen_oracle_decode*        torch.scatter_add_ on CPU, fp64 sums
 *   zen_oracle_encode         numpy flatnonzero
 *   zen_oracle_mapping        permutation + ascending invariants
 *   zen_oracle_bitmap_*       numpy packbits(bitorder="little")
 * No function here is "parity unpinned".
 */
#ifndef ZEN_ORACLE_H
#define ZEN_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of a gradient tensor */
#define ZEN_ORACLE_F32 0
#define ZEN_ORACLE_BF16 1

/* seeds of the three probe levels: functions_cuda_kernel.cu:101,119,124,144,149,151 */
#define ZEN_ORACLE_SEED1 10001861u
#define ZEN_ORACLE_SEED2 100703u
#define ZEN_ORACLE_SEED3 5002639u

/* status bits returned by the insert / load-balance functions */
#define ZEN_ORACLE_OK 0
#define ZEN_ORACLE_EINVAL (-1)
#define ZEN_ORACLE_SERIAL_OVERFLOW 1 /* a ticket left its partition's serial region */

/* functions_cuda_kernel.cu:80-93: cubic polynomial in uint32 arithmetic. */
uint32_t zen_oracle_hash(int32_t key, uint32_t seed);

/* functions_cuda_kernel.cu:169-177: out[t] = (h1(t) % n) / (n / P), t in [0,n). */
int zen_oracle_hash_index(int32_t *out, int64_t n, int partitions);

/*
 * functions_cuda_kernel.cu:97-167 executed for tid = 0,1,2,... in order (one
 * legal schedule of the racy kernel; the canonical one).  memory[m] and
 * serial[serial_n] must be zeroed by the caller, offset[P] must hold the
 * serial base offsets (extensions/cuda/functions.py:8-11).  rehash outside
 * {2,3} means one probe level (functions_cuda_kernel.cu:192-198).
 * Tickets beyond serial_n are dropped (the reference writes out of bounds).
 */
int zen_oracle_sparse_balance(const void *in, int dtype, int64_t n,
                              int32_t *memory, int64_t m,
                              int32_t *serial, int64_t serial_n,
                              int32_t *offset, int partitions, int rehash);

/*
 * tensor_load_balance.py:13-51.  m is the table size computed by the caller
 * (tensor_load_balance.py:15-16).  Writes partition-contiguous indices (slot
 * order, then the partition's serial region) and the gathered values; splits
 * has P entries.  out_idx / out_val need room for every nonzero of the input.
 * Returns the status of the insert, or ZEN_ORACLE_EINVAL.
 */
int zen_oracle_load_balance(const void *in, int dtype, int64_t n, int64_t m,
                            int partitions, int rehash,
                            int32_t *out_idx, void *out_val, int64_t *splits);

/* magnitude key of element i: the bit pattern with the sign cleared. */
uint32_t zen_oracle_mag_key(const void *in, int dtype, int64_t i);

/*
 * train.py:79-82: threshold = min(topk(|g|, k)) = k-th largest magnitude,
 * returned as a magnitude key.  k in [1, n].
 */
uint32_t zen_oracle_kth_key(const void *in, int dtype, int64_t n, int64_t k);

/*
 * train.py:83: where(|g| >= thr, g, 0) as a dense masked copy.  thr_key == 0
 * keeps every element.  Returns the number of kept elements with nonzero key.
 */
int64_t zen_oracle_mask_dense(const void *in, int dtype, int64_t n,
                              uint32_t thr_key, void *out);

/*
 * The selected set as a list: ascending indices i with key(i) >= thr_key and
 * key(i) != 0, plus their values (bit copies).  Returns the count.
 */
int64_t zen_oracle_select(const void *in, int dtype, int64_t n, uint32_t thr_key,
                          int32_t *out_idx, void *out_val);

/*
 * comm.py:32-44: dense[idx[j]] += val[j] for j = 0..r-1 in order, dense
 * zero-initialised, dense_n elements.
 *   _f32acc : accumulate in fp32, output fp32 (fp32 inputs: this IS the
 *             reference; bf16 inputs: the fp32-accumulation variant)
 *   _native : accumulate in the value dtype as the reference does
 *             (bf16: round to nearest even after every add), output in dtype
 *   _f64    : accumulate in fp64 (ground truth for tolerances)
 * Return ZEN_ORACLE_EINVAL on an index outside [0, dense_n).
 */
int zen_oracle_decode_f32acc(const int32_t *idx, const void *val, int dtype,
                             int64_t r, float *dense, int64_t dense_n);
int zen_oracle_decode_native(const int32_t *idx, const void *val, int dtype,
                             int64_t r, void *dense, int64_t dense_n);
int zen_oracle_decode_f64(const int32_t *idx, const void *val, int dtype,
                          int64_t r, double *dense, int64_t dense_n);

/* comm.py:47-50: ascending indices of nonzero entries + their values. */
int64_t zen_oracle_encode(const void *dense, int dtype, int64_t n,
                          int64_t *out_idx, void *out_val);

/*
 * comm.py:52-56: for each partition p the ascending list of t in [0,n) with
 * hash_index(t) == p, concatenated; counts[p] gets each list's length.
 * Entries with part == P (n % P != 0) belong to no list, as in the reference.
 */
int zen_oracle_mapping(int64_t n, int partitions, int64_t *out, int64_t *counts);

/*
 * comm.py:59-85: bit j of the output is 1 iff mapping_p[j] is in the sorted
 * index list; bit j sits in byte j/8 at weight 2^(j%8).  out has
 * (mapping_n+7)/8 bytes.  Indices absent from mapping_p follow the
 * reference's searchsorted semantics (they set the bit of the insertion
 * point when that is in range).
 */
int zen_oracle_bitmap_encode(const int64_t *mapping_p, int64_t mapping_n,
                             const int64_t *idx, int64_t idx_n, uint8_t *out);

/* comm.py:87-99: mapping_p[j] for every set bit j < mapping_n. Returns count. */
int64_t zen_oracle_bitmap_decode(const int64_t *mapping_p, int64_t mapping_n,
                                 const uint8_t *bitmap, int64_t *out);

#ifdef __cplusplus
}
#endif
#endif
