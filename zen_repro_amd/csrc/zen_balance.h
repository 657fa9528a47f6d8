// Helpers shared by the two load-balance back ends (owner table in
// zen_balance.hip, sort-based resolution in zen_resolve.hip).
#pragma once

#include "zen_select.h"

namespace zen {

constexpr uint32_t kSerialLds = 8192;  // serial tails up to this size are sorted in LDS

// Ascending compare-exchange network (bitonic with mirrored first step), valid
// for any n: positions >= n act as +infinity and never move.
__device__ inline void sort_network(uint32_t *a, uint32_t n) {
  uint32_t n2 = 1;
  while (n2 < n) n2 <<= 1;
  const uint32_t half = n2 >> 1;
  for (uint32_t k = 2; k <= n2; k <<= 1) {
    const uint32_t hk = k >> 1;
    for (uint32_t q = threadIdx.x; q < half; q += blockDim.x) {
      const uint32_t blk = q / hk, r = q % hk;
      const uint32_t i = blk * k + r, l = blk * k + (k - 1 - r);
      if (l < n) {
        const uint32_t x = a[i], y = a[l];
        if (x > y) { a[i] = y; a[l] = x; }
      }
    }
    __syncthreads();
    for (uint32_t j = hk >> 1; j > 0; j >>= 1) {
      for (uint32_t q = threadIdx.x; q < half; q += blockDim.x) {
        const uint32_t i = (q / j) * 2 * j + (q % j), l = i + j;
        if (l < n) {
          const uint32_t x = a[i], y = a[l];
          if (x > y) { a[i] = y; a[l] = x; }
        }
      }
      __syncthreads();
    }
  }
}



__device__ inline uint32_t lower_bound_u32(const uint32_t *a, uint32_t n, uint32_t x) {
  uint32_t lo = 0, hi = n;
  while (lo < hi) {
    const uint32_t mid = lo + ((hi - lo) >> 1);
    if (a[mid] < x) lo = mid + 1; else hi = mid;
  }
  return lo;
}


__device__ inline uint32_t upper_bound_u32(const uint32_t *a, uint32_t n, uint32_t x) {  // entries <= x
  uint32_t lo = 0, hi = n;
  while (lo < hi) {
    const uint32_t mid = lo + ((hi - lo) >> 1);
    if (a[mid] <= x) lo = mid + 1; else hi = mid;
  }
  return lo;
}

// Room for the candidates of a sampled top-k (the selected plus those between
// the sampled floor and the exact threshold).
inline int64_t list_capacity(int64_t capacity) { return capacity + capacity / 2 + 4096; }

// A list entry (candidate index, value) is selected if its index is not 0
// (index 0 is never transmitted) and, when the list still holds candidates of a
// sampled top-k, its magnitude key reaches the exact threshold.
template <typename S>
__device__ inline bool list_selected(const int32_t *cand, const S *vals, const uint32_t *thr, uint32_t j,
                                     uint32_t *t_out) {
  const uint32_t t = (uint32_t)cand[j];
  *t_out = t;
  if (t == 0) return false;
  return !thr || (vals[j] & KeyOf<S>::kMask) >= thr[0];
}

// Canonical order of a partition's serial tail out_idx[ser .. ser+cnt): ascending
// index (the reference hands tickets to ascending indices), values fetched
// again from the dense gradient.  Called by every thread of one block.
template <typename S>
__device__ inline void fix_serial_tail(int32_t *out_idx, S *out_val, const S *dense, uint32_t ser, uint32_t cnt,
                                       uint32_t *lds_buf) {
  if (cnt < 2) return;
  uint32_t *region = reinterpret_cast<uint32_t *>(out_idx + ser);
  if (cnt <= kSerialLds) {
    for (uint32_t i = threadIdx.x; i < cnt; i += blockDim.x) lds_buf[i] = region[i];
    __syncthreads();
    sort_network(lds_buf, cnt);
    for (uint32_t i = threadIdx.x; i < cnt; i += blockDim.x) region[i] = lds_buf[i];
  } else {
    sort_network(region, cnt);
  }
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < cnt; i += blockDim.x) out_val[ser + i] = dense[region[i]];
}

// Sort-based owner resolution (zen_resolve.hip): everything after the selected
// list exists, without touching a table of the reference's size.
struct ResolveArgs {
  const void *dense;          // the gradient (serial tails re-fetch their values)
  int dtype;
  Probe g;
  int partitions;
  int64_t spp;                // serial slots per partition
  const int32_t *list_idx;    // selected / candidate list
  const void *list_val;
  const uint32_t *count;      // its length (device)
  const uint32_t *filter;     // optional exact threshold still to apply
  int64_t list_cap;
  int64_t expected;           // how many entries the caller expects the list to hold
  uint32_t *keys_a, *perm_a, *more_a, *keys_b, *perm_b, *more_b;  // list_cap each
  void *sort_scratch;
  unsigned long long *hash;   // zeroed cells for slot -> smallest index, zero again on return
  uint32_t hash_log2;
  void *scratch;              // resolve_scratch_bytes(list_cap)
  int32_t *out_idx;
  void *out_val;
  int64_t capacity;
  int64_t *splits;
  int32_t *status;
};
// Load balance on bucket slabs (zen_slab_encode.hip): select, sort and place in six launches, for sizes
// slab_balance_fits accepts.
struct SlabBalanceArgs {
  const void *input;          // the dense gradient
  int dtype;
  int64_t n;
  Probe g;
  int partitions;
  int64_t spp;                // serial slots per partition
  const uint32_t *thr;        // optional threshold key (device); with k == 0 and no thr: the nonzeros
  int64_t k;                  // > 0: the k largest magnitudes, ties kept
  uint32_t *thr_out;          // optional, k > 0: receives (threshold key, number selected)
  int32_t *out_idx;
  void *out_val;
  int64_t capacity;
  int64_t *splits;
  unsigned long long *hash;   // zeroed cells for slot -> smallest index, zero again on return
  uint32_t hash_log2;
  void *workspace;            // slab_balance_bytes(...)
  int32_t *status;
  const uint32_t *near_key = nullptr;  // optional, k > 0: a key close to the k-th largest (no sample is taken)
  int prepared = 0;           // 1 / 2: the sampled floor of the first / second set is there already (zen_load_balance_prepare)
  const void *next_input = nullptr;  // the next call's tensor (this one's type): its sample is taken
  int64_t next_k = 0;                // by this call's pass over the tensor, in the other set of sampling memory
  int64_t next_n = 0;                // its length (0: this call's)
  void *next_state = nullptr;        // the zero-between-calls memory in the next call's table (null: this call's)
  bool second = false;        // the call's sample uses the second set of sampling memory (always so with prepared == 2)
  bool only_prepare = false;  // take the sample for that set and nothing else
  bool discard = false;       // with only_prepare: clear the set's sampling memory instead (a sample nobody picks up)
};
bool slab_balance_fits(int64_t n, int64_t m, int partitions, int dtype, int64_t capacity, int64_t k, SlabGeom *geo);
size_t slab_balance_bytes(int64_t m, int partitions, int dtype, int64_t capacity);
int slab_load_balance(const SlabBalanceArgs &a, hipStream_t stream);
int slab_prepare(const SlabBalanceArgs &a, hipStream_t stream);  // only_prepare, whichever of the two paths the call takes
size_t slab_state_offset(uint32_t hash_log2);  // where the zero-between-calls counters start in the caller's table

// Load balance on wide buckets (zen_wide_encode.hip): select and one resident kernel, for selections of a few
// million entries at most on a chip of `cus` compute units.
bool wide_balance_fits(int64_t m, int partitions, int64_t capacity, int64_t k, int cus, SlabGeom *geo);
size_t wide_balance_bytes(int64_t m, int partitions, int dtype, int64_t capacity, int cus);
int wide_load_balance(const SlabBalanceArgs &a, size_t state_offset, hipStream_t stream);
int wide_device_cus();  // compute units of the current device (0: no device)


size_t resolve_scratch_bytes(int64_t list_cap, uint64_t key_limit);  // key_limit = P * (m / P + 1) + 1
int resolve_and_place(const ResolveArgs &a, hipStream_t stream);

}  // namespace zen
