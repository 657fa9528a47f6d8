/*
 * CPU oracle (test infrastructure only) -- see zen_oracle.h for the contract
 * and for what pins each function.  Sequential, single-threaded, plain C11.
 */
#include "zen_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------- helpers */

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* round-to-nearest-even fp32 -> bf16, NaN kept quiet (torch's conversion) */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float load_as_f32(const void *in, int dtype, int64_t i) {
  if (dtype == ZEN_ORACLE_BF16) return bf16_to_f32(((const uint16_t *)in)[i]);
  return ((const float *)in)[i];
}

static inline int dtype_ok(int dtype) {
  return dtype == ZEN_ORACLE_F32 || dtype == ZEN_ORACLE_BF16;
}

static inline size_t dtype_size(int dtype) { return dtype == ZEN_ORACLE_BF16 ? 2 : 4; }

/* ------------------------------------------------------------------ hash */

/* functions_cuda_kernel.cu:80-88.  The key is an int that meets uint32
 * operands, so every product wraps mod 2^32; written here in the expanded
 * form the reference uses (tests check it equals the Horner form). */
uint32_t zen_oracle_hash(int32_t key, uint32_t seed) {
  const uint32_t k = (uint32_t)key;
  const uint32_t cube = 573729859u * k * k * k;
  const uint32_t square = 0xcc9e2d51u * k * k;
  const uint32_t linear = 0x1b873593u * k;
  return cube + square + linear + seed;
}

/* functions_cuda_kernel.cu:169-177 */
int zen_oracle_hash_index(int32_t *out, int64_t n, int partitions) {
  if (n <= 0 || n > INT32_MAX || partitions <= 0 || n / partitions == 0)
    return ZEN_ORACLE_EINVAL;
  const uint32_t un = (uint32_t)n;
  const int32_t per_part = (int32_t)(n / partitions);
  for (int64_t t = 0; t < n; ++t) {
    const int32_t slot = (int32_t)(zen_oracle_hash((int32_t)t, ZEN_ORACLE_SEED1) % un);
    out[t] = slot / per_part;
  }
  return ZEN_ORACLE_OK;
}

/* ---------------------------------------------------------------- insert */

/* functions_cuda_kernel.cu:97-167, run for tid ascending.  The three kernels
 * differ only in how many probe levels precede the serial ticket, so one loop
 * over `levels` covers them: level 1 probes the whole table (h1 % m), levels
 * 2 and 3 probe inside the partition level 1 landed in. */
int zen_oracle_sparse_balance(const void *in, int dtype, int64_t n,
                              int32_t *memory, int64_t m,
                              int32_t *serial, int64_t serial_n,
                              int32_t *offset, int partitions, int rehash) {
  if (!dtype_ok(dtype) || n < 0 || n > INT32_MAX || m <= 0 || m > INT32_MAX ||
      partitions <= 0 || m % partitions != 0 || serial_n < 0)
    return ZEN_ORACLE_EINVAL;
  const int levels = (rehash == 2 || rehash == 3) ? rehash : 1;
  const uint32_t seeds[3] = {ZEN_ORACLE_SEED1, ZEN_ORACLE_SEED2, ZEN_ORACLE_SEED3};
  const uint32_t um = (uint32_t)m;
  const int32_t per_part = (int32_t)(m / partitions);
  const int64_t serial_per_part = serial_n / partitions;
  int status = ZEN_ORACLE_OK;

  for (int64_t tid = 0; tid < n; ++tid) {
    if (!(load_as_f32(in, dtype, tid) != 0.0f)) continue; /* .cu:100 */
    const int32_t first = (int32_t)(zen_oracle_hash((int32_t)tid, seeds[0]) % um);
    const int32_t part = first / per_part;
    const int32_t base = part * per_part;
    int placed = 0;
    for (int lv = 0; lv < levels && !placed; ++lv) {
      const int32_t slot =
          lv == 0 ? first
                  : base + (int32_t)(zen_oracle_hash((int32_t)tid, seeds[lv]) %
                                     (uint32_t)per_part);
      if (memory[slot] == 0) {
        memory[slot] = (int32_t)tid; /* tid 0 stores the empty marker: a no-op */
        placed = 1;
      }
    }
    if (placed) continue;
    const int64_t ticket = offset[part]++; /* atomicAdd, .cu:107,131,157 */
    if (ticket >= (int64_t)(part + 1) * serial_per_part) status |= ZEN_ORACLE_SERIAL_OVERFLOW;
    if (ticket >= 0 && ticket < serial_n) serial[ticket] = (int32_t)tid;
  }
  return status;
}

/* ---------------------------------------------------------- load balance */

/* tensor_load_balance.py:24-40 for one of the two tables: append the nonzero
 * entries of chunk p (ascending position) and gather their values. */
static int64_t compact_chunk(const int32_t *table, int64_t lo, int64_t hi,
                             const void *in, int dtype, int32_t *out_idx,
                             void *out_val, int64_t at) {
  const size_t es = dtype_size(dtype);
  for (int64_t s = lo; s < hi; ++s) {
    const int32_t t = table[s];
    if (t == 0) continue;
    out_idx[at] = t;
    memcpy((char *)out_val + (size_t)at * es, (const char *)in + (size_t)t * es, es);
    ++at;
  }
  return at;
}

int zen_oracle_load_balance(const void *in, int dtype, int64_t n, int64_t m,
                            int partitions, int rehash,
                            int32_t *out_idx, void *out_val, int64_t *splits) {
  if (!dtype_ok(dtype) || n <= 0 || n > INT32_MAX || partitions <= 0 || m <= 0 ||
      m > INT32_MAX || m % partitions != 0)
    return ZEN_ORACLE_EINVAL;
  /* tensor_load_balance.py:18: serial size = numel // P // 10 * P */
  const int64_t serial_per_part = n / partitions / 10;
  const int64_t serial_n = serial_per_part * partitions;
  int32_t *memory = (int32_t *)calloc((size_t)m, sizeof(int32_t));
  int32_t *serial = (int32_t *)calloc((size_t)(serial_n > 0 ? serial_n : 1), sizeof(int32_t));
  int32_t *offset = (int32_t *)malloc((size_t)partitions * sizeof(int32_t));
  if (!memory || !serial || !offset) {
    free(memory); free(serial); free(offset);
    return ZEN_ORACLE_EINVAL;
  }
  /* extensions/cuda/functions.py:8-10 */
  for (int p = 0; p < partitions; ++p) offset[p] = (int32_t)(p * serial_per_part);
  const int status = zen_oracle_sparse_balance(in, dtype, n, memory, m, serial, serial_n,
                                               offset, partitions, rehash);
  if (status >= 0) {
    /* tensor_load_balance.py:46-50: per partition, table part then serial part.
     * Both tables have a length that is a multiple of P, so torch.chunk(P)
     * yields P equal chunks (P empty ones for a zero-length serial table). */
    const int64_t per_part = m / partitions;
    int64_t at = 0;
    for (int p = 0; p < partitions; ++p) {
      const int64_t begin = at;
      at = compact_chunk(memory, p * per_part, (p + 1) * per_part, in, dtype, out_idx, out_val, at);
      at = compact_chunk(serial, p * serial_per_part, (p + 1) * serial_per_part, in, dtype,
                         out_idx, out_val, at);
      splits[p] = at - begin;
    }
  }
  free(memory); free(serial); free(offset);
  return status;
}

/* ---------------------------------------------------------------- select */

uint32_t zen_oracle_mag_key(const void *in, int dtype, int64_t i) {
  if (dtype == ZEN_ORACLE_BF16) return ((const uint16_t *)in)[i] & 0x7fffu;
  return f32_bits(((const float *)in)[i]) & 0x7fffffffu;
}

static int cmp_u32_desc(const void *a, const void *b) {
  const uint32_t x = *(const uint32_t *)a, y = *(const uint32_t *)b;
  return x < y ? 1 : (x > y ? -1 : 0);
}

/* train.py:81-82: topk(...)[0].min().  For non-NaN values |a| >= |b| iff
 * key(a) >= key(b), so the k-th largest key is the k-th largest magnitude.
 * Done by a full descending sort: slow and obviously right. */
uint32_t zen_oracle_kth_key(const void *in, int dtype, int64_t n, int64_t k) {
  if (!dtype_ok(dtype) || n <= 0 || k < 1 || k > n) return 0xffffffffu;
  uint32_t *keys = (uint32_t *)malloc((size_t)n * sizeof(uint32_t));
  if (!keys) return 0xffffffffu;
  for (int64_t i = 0; i < n; ++i) keys[i] = zen_oracle_mag_key(in, dtype, i);
  qsort(keys, (size_t)n, sizeof(uint32_t), cmp_u32_desc);
  const uint32_t kth = keys[k - 1];
  free(keys);
  return kth;
}

/* train.py:83 */
int64_t zen_oracle_mask_dense(const void *in, int dtype, int64_t n,
                              uint32_t thr_key, void *out) {
  const size_t es = dtype_size(dtype);
  int64_t kept = 0;
  for (int64_t i = 0; i < n; ++i) {
    const uint32_t key = zen_oracle_mag_key(in, dtype, i);
    if (key >= thr_key) {
      memcpy((char *)out + (size_t)i * es, (const char *)in + (size_t)i * es, es);
      kept += key != 0;
    } else {
      memset((char *)out + (size_t)i * es, 0, es);
    }
  }
  return kept;
}

int64_t zen_oracle_select(const void *in, int dtype, int64_t n, uint32_t thr_key,
                          int32_t *out_idx, void *out_val) {
  const size_t es = dtype_size(dtype);
  int64_t at = 0;
  for (int64_t i = 0; i < n; ++i) {
    const uint32_t key = zen_oracle_mag_key(in, dtype, i);
    if (key == 0 || key < thr_key) continue;
    out_idx[at] = (int32_t)i;
    memcpy((char *)out_val + (size_t)at * es, (const char *)in + (size_t)i * es, es);
    ++at;
  }
  return at;
}

/* ----------------------------------------------------------------- merge */

/* comm.py:32-39: zeros + scatter_add_ over the concatenated payloads. */
int zen_oracle_decode_f32acc(const int32_t *idx, const void *val, int dtype,
                             int64_t r, float *dense, int64_t dense_n) {
  if (!dtype_ok(dtype)) return ZEN_ORACLE_EINVAL;
  memset(dense, 0, (size_t)dense_n * sizeof(float));
  for (int64_t j = 0; j < r; ++j) {
    if (idx[j] < 0 || idx[j] >= dense_n) return ZEN_ORACLE_EINVAL;
    dense[idx[j]] += load_as_f32(val, dtype, j);
  }
  return ZEN_ORACLE_OK;
}

int zen_oracle_decode_native(const int32_t *idx, const void *val, int dtype,
                             int64_t r, void *dense, int64_t dense_n) {
  if (!dtype_ok(dtype)) return ZEN_ORACLE_EINVAL;
  if (dtype == ZEN_ORACLE_F32)
    return zen_oracle_decode_f32acc(idx, val, dtype, r, (float *)dense, dense_n);
  uint16_t *d = (uint16_t *)dense;
  memset(d, 0, (size_t)dense_n * sizeof(uint16_t));
  for (int64_t j = 0; j < r; ++j) {
    if (idx[j] < 0 || idx[j] >= dense_n) return ZEN_ORACLE_EINVAL;
    d[idx[j]] = f32_to_bf16(bf16_to_f32(d[idx[j]]) + load_as_f32(val, dtype, j));
  }
  return ZEN_ORACLE_OK;
}

int zen_oracle_decode_f64(const int32_t *idx, const void *val, int dtype,
                          int64_t r, double *dense, int64_t dense_n) {
  if (!dtype_ok(dtype)) return ZEN_ORACLE_EINVAL;
  memset(dense, 0, (size_t)dense_n * sizeof(double));
  for (int64_t j = 0; j < r; ++j) {
    if (idx[j] < 0 || idx[j] >= dense_n) return ZEN_ORACLE_EINVAL;
    dense[idx[j]] += (double)load_as_f32(val, dtype, j);
  }
  return ZEN_ORACLE_OK;
}

/* comm.py:47-50 */
int64_t zen_oracle_encode(const void *dense, int dtype, int64_t n,
                          int64_t *out_idx, void *out_val) {
  const size_t es = dtype_size(dtype);
  int64_t at = 0;
  for (int64_t i = 0; i < n; ++i) {
    if (!(load_as_f32(dense, dtype, i) != 0.0f)) continue; /* torch.nonzero: -0.0 is zero, NaN is not */
    out_idx[at] = i;
    memcpy((char *)out_val + (size_t)at * es, (const char *)dense + (size_t)i * es, es);
    ++at;
  }
  return at;
}

/* --------------------------------------------------------------- mapping */

/* comm.py:52-56 */
int zen_oracle_mapping(int64_t n, int partitions, int64_t *out, int64_t *counts) {
  if (n <= 0 || n > INT32_MAX || partitions <= 0 || n / partitions == 0)
    return ZEN_ORACLE_EINVAL;
  int32_t *part = (int32_t *)malloc((size_t)n * sizeof(int32_t));
  if (!part) return ZEN_ORACLE_EINVAL;
  zen_oracle_hash_index(part, n, partitions);
  int64_t at = 0;
  for (int p = 0; p < partitions; ++p) {
    const int64_t begin = at;
    for (int64_t t = 0; t < n; ++t)
      if (part[t] == p) out[at++] = t;
    counts[p] = at - begin;
  }
  free(part);
  return ZEN_ORACLE_OK;
}

/* ---------------------------------------------------------------- bitmap */

/* comm.py:60-65 (searchsorted, left) + :66-84 (pad to a byte, weights 2^j) */
int zen_oracle_bitmap_encode(const int64_t *mapping_p, int64_t mapping_n,
                             const int64_t *idx, int64_t idx_n, uint8_t *out) {
  memset(out, 0, (size_t)((mapping_n + 7) / 8));
  for (int64_t j = 0; j < idx_n; ++j) {
    int64_t lo = 0, hi = mapping_n;
    while (lo < hi) {
      const int64_t mid = lo + (hi - lo) / 2;
      if (mapping_p[mid] < idx[j]) lo = mid + 1; else hi = mid;
    }
    if (lo >= mapping_n) return ZEN_ORACLE_EINVAL; /* torch raises an index error */
    out[lo >> 3] |= (uint8_t)(1u << (lo & 7));
  }
  return ZEN_ORACLE_OK;
}

/* comm.py:87-99 */
int64_t zen_oracle_bitmap_decode(const int64_t *mapping_p, int64_t mapping_n,
                                 const uint8_t *bitmap, int64_t *out) {
  int64_t at = 0;
  for (int64_t j = 0; j < mapping_n; ++j)
    if (bitmap[j >> 3] & (1u << (j & 7))) out[at++] = mapping_p[j];
  return at;
}
