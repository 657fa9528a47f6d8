// Hash partitioning: hash_index, the in-place table insert (sparse_balance) and
// the fused select + insert + slot-order compaction (load_balance).
//
// The reference insert (functions_cuda_kernel.cu:97-167) is a race: plain load,
// plain store.  Run with its threads in ascending order it has one well-defined
// result: a slot belongs to the smallest index that ever probes it, and an
// index probes level l+1 only if a smaller index owns its level-l slot.  That
// fixed point is computed here with atomicMax on the encoding 0 - index (so the
// empty marker 0 stays the smallest value): a thread that takes a slot from a
// larger index carries on with that index's probe sequence, so every lost
// probe is continued exactly once and no rounds or flags are needed.
#include "zen_balance.h"

namespace zen {
namespace {

__device__ inline void insert_chain(uint32_t *table, const Probe &g, uint32_t t) {
  uint32_t cur = t;
  int lv = 0;
  for (;;) {
    uint32_t part;
    const uint32_t slot = probe_slot(g, cur, lv, &part);
    const uint32_t mine = 0u - cur;
    const uint32_t old = atomicMax(&table[slot], mine);
    if (old > mine) {  // a smaller index owns the slot: cur moves on
      if (++lv >= g.levels) return;  // out of levels: found later by its absence
      continue;
    }
    if (old == 0u || old == mine) return;  // took an empty slot
    // took the slot from a larger index w: w held it at its first level that
    // maps here, and now continues from the next one
    const uint32_t w = 0u - old;
    int lw = 0;
    while (lw < g.levels && probe_slot(g, w, lw, &part) != slot) ++lw;
    cur = w;
    lv = lw + 1;
    if (lv >= g.levels) return;
  }
}

// level at which t holds a slot, or -1; *slot_out / *part_out as found
__device__ inline int find_level(const uint32_t *table, const Probe &g, uint32_t t, uint32_t *slot_out,
                                 uint32_t *part_out) {
  const uint32_t mine = 0u - t;
  for (int lv = 0; lv < g.levels; ++lv) {
    const uint32_t slot = probe_slot(g, t, lv, part_out);
    if (table[slot] == mine) {
      *slot_out = slot;
      return lv;
    }
  }
  return -1;
}

// ------------------------------------------------------------- hash_index

__global__ __launch_bounds__(256) void k_hash_index(int32_t *__restrict__ out, uint32_t n, uint32_t per_part) {
  for (uint32_t t = blockIdx.x * 256u + threadIdx.x; t < n; t += gridDim.x * 256u)
    out[t] = (int32_t)(((poly(t) + kSeed1) % n) / per_part);
}

// ------------------------------------------------ in-place insert (dense)

template <typename S, bool ALIGNED>
__global__ __launch_bounds__(256) void k_insert_dense(const S *__restrict__ in, int64_t n, uint32_t *table,
                                                      Probe g) {
  constexpr int V = VecOf<S>::kN;
  const int64_t nvec = (n + V - 1) / V;
  for (int64_t v = blockIdx.x * (int64_t)256 + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * 256) {
    S e[V];
    const int live = load_vec<S, ALIGNED>(in, v * V, n, e);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const uint32_t t = (uint32_t)(v * V + i);
      if (i < live && (e[i] & KeyOf<S>::kMask) != 0 && t != 0) insert_chain(table, g, t);
    }
  }
}

template <typename S, bool ALIGNED>
__global__ __launch_bounds__(256) void k_finalize_dense(const S *__restrict__ in, int64_t n, uint32_t *table,
                                                        Probe g, int32_t *serial, int64_t spp,
                                                        int32_t *offset, int32_t *status) {
  constexpr int V = VecOf<S>::kN;
  const int64_t nvec = (n + V - 1) / V;
  for (int64_t v = blockIdx.x * (int64_t)256 + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * 256) {
    S e[V];
    const int live = load_vec<S, ALIGNED>(in, v * V, n, e);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const uint32_t t = (uint32_t)(v * V + i);
      if (!(i < live && (e[i] & KeyOf<S>::kMask) != 0 && t != 0)) continue;
      uint32_t slot, part;
      if (find_level(table, g, t, &slot, &part) >= 0) {
        table[slot] = t;  // owner only: nobody else compares equal to this slot
      } else {
        const int64_t ticket = atomicAdd(&offset[part], 1);
        if (ticket >= 0 && ticket < (int64_t)(part + 1) * spp)
          serial[ticket] = (int32_t)t;
        else
          atomicOr(status, ZEN_STAT_SERIAL_OVERFLOW);
      }
    }
  }
}

// Tickets are handed out in arrival order; the canonical order is ascending
// index inside each partition's region, so each region is sorted in place.
__global__ __launch_bounds__(256) void k_serial_sort(int32_t *serial, int64_t spp, const int32_t *offset) {
  __shared__ uint32_t buf[kSerialLds];
  const int p = blockIdx.x;
  const int64_t begin = (int64_t)p * spp;
  int64_t end = offset[p];
  if (end > begin + spp) end = begin + spp;
  if (end - begin < 2) return;
  const uint32_t cnt = (uint32_t)(end - begin);
  uint32_t *region = reinterpret_cast<uint32_t *>(serial + begin);
  if (cnt <= kSerialLds) {
    for (uint32_t i = threadIdx.x; i < cnt; i += blockDim.x) buf[i] = region[i];
    __syncthreads();
    sort_network(buf, cnt);
    for (uint32_t i = threadIdx.x; i < cnt; i += blockDim.x) region[i] = buf[i];
  } else {
    sort_network(region, cnt);
  }
}

// ------------------------------------------------- fused path (list based)

template <typename S>
__global__ __launch_bounds__(256) void k_insert_list(const int32_t *__restrict__ cand, const S *__restrict__ vals,
                                                     const uint32_t *count, const uint32_t *__restrict__ thr,
                                                     uint32_t *table, Probe g) {
  const uint32_t j = blockIdx.x * 256u + threadIdx.x;
  if (j >= *count) return;
  uint32_t t;
  if (list_selected<S>(cand, vals, thr, j, &t)) insert_chain(table, g, t);
}

// Sort key = position in the output: partition-major, table slots before the
// partition's serial entries (all serial entries of a partition share one key).
template <typename S>
__global__ __launch_bounds__(256) void k_final_key(const int32_t *__restrict__ cand, const S *__restrict__ vals,
                                                   const uint32_t *count, const uint32_t *__restrict__ thr,
                                                   const uint32_t *__restrict__ table, Probe g, uint32_t drop_key,
                                                   uint32_t *__restrict__ keys, uint32_t *__restrict__ perm) {
  const uint32_t j = blockIdx.x * 256u + threadIdx.x;
  if (j >= *count) return;
  uint32_t t;
  uint32_t key = drop_key;
  if (list_selected<S>(cand, vals, thr, j, &t)) {
    uint32_t slot = 0, part = 0;
    const int lv = find_level(table, g, t, &slot, &part);
    key = part * (g.npp + 1u) + (lv >= 0 ? slot - part * g.npp : g.npp);
  }
  keys[j] = key;
  perm[j] = j;
}

template <typename S>
__global__ __launch_bounds__(256) void k_gather(const uint32_t *__restrict__ keys, const uint32_t *__restrict__ perm,
                                                const uint32_t *count, const int32_t *__restrict__ cand_idx,
                                                const S *__restrict__ cand_val, uint32_t drop_key, Probe g,
                                                int32_t *__restrict__ out_idx, S *__restrict__ out_val,
                                                uint32_t capacity, uint32_t *table) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= *count) return;
  const uint32_t key = keys[i];
  if (key >= drop_key) return;
  const uint32_t j = perm[i];
  if (i < capacity) {
    out_idx[i] = cand_idx[j];
    out_val[i] = cand_val[j];
  }
  const uint32_t part = key / (g.npp + 1u), local = key % (g.npp + 1u);
  if (local < g.npp) table[part * g.npp + local] = 0u;  // leave the table empty again
}

// One block per partition: its length from the sorted keys, and the canonical
// order of its serial tail.  The selected list arrives tile by tile in no
// particular order and all serial entries of a partition share one sort key, so
// the stable sort leaves them in arrival order; the reference order (tickets
// handed out to ascending indices) is restored by sorting the tail by index and
// fetching the values again.
template <typename S>
__global__ __launch_bounds__(256) void k_splits_serial(const uint32_t *__restrict__ keys, const uint32_t *count,
                                                       uint32_t npp, int64_t spp, uint32_t capacity,
                                                       const S *__restrict__ dense, int32_t *__restrict__ out_idx,
                                                       S *__restrict__ out_val, int64_t *__restrict__ splits,
                                                       int32_t *status) {
  __shared__ uint32_t s_bound[3];
  __shared__ uint32_t buf[kSerialLds];
  const uint32_t p = blockIdx.x;
  if (threadIdx.x < 3) {
    const uint32_t first = p * (npp + 1u);
    const uint32_t probe = threadIdx.x == 0 ? first : (threadIdx.x == 1 ? first + npp : first + npp + 1u);
    s_bound[threadIdx.x] = lower_bound_u32(keys, *count, probe);
  }
  __syncthreads();
  const uint32_t lo = s_bound[0], ser = s_bound[1], hi = s_bound[2];
  if (threadIdx.x == 0) {
    splits[p] = (int64_t)(hi - lo);
    if ((int64_t)(hi - ser) > spp) atomicOr(status, ZEN_STAT_SERIAL_OVERFLOW);
    if (hi > capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
  if (hi > capacity) return;
  fix_serial_tail<S>(out_idx, out_val, dense, ser, hi - ser, buf);
}

template <typename S>
int sparse_balance_launch(const S *in, int64_t n, uint32_t *table, Probe g, int32_t *serial, int64_t spp,
                          int32_t *offset, int partitions, int32_t *status, hipStream_t s) {
  constexpr int V = VecOf<S>::kN;
  const int64_t nvec = ceil_div(n, V);
  int64_t blocks = ceil_div(nvec, 256);
  if (blocks > 16384) blocks = 16384;
  const bool aligned = (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
  ProfScope prof(kProfInsertDense, s);
  if (aligned) {
    k_insert_dense<S, true><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(in, n, table, g);
    ZEN_LAUNCH_CHECK("k_insert_dense");
    k_finalize_dense<S, true><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(in, n, table, g, serial, spp, offset, status);
  } else {
    k_insert_dense<S, false><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(in, n, table, g);
    ZEN_LAUNCH_CHECK("k_insert_dense");
    k_finalize_dense<S, false><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(in, n, table, g, serial, spp, offset, status);
  }
  ZEN_LAUNCH_CHECK("k_finalize_dense");
  if (spp > 0) {
    k_serial_sort<<<dim3((unsigned)partitions), dim3(256), 0, s>>>(serial, spp, offset);
    ZEN_LAUNCH_CHECK("k_serial_sort");
  }
  return ZEN_OK;
}

constexpr int64_t kSampleMinElems = 1ll << 24;  // below this the exact full-tensor histogram is cheap anyway

struct BalancePlan {
  int32_t *sel_idx;    // the selected entries or candidates (list_capacity)
  uint32_t *sel_val;   // 4 bytes per value reserved, bf16 uses half
  uint32_t *keys_a, *perm_a, *more_a, *keys_b, *perm_b, *more_b;
  uint32_t *count;     // entries in sel_*
  uint32_t *thr;       // [0..1] exact threshold + count, [2..3] sampled floor
  uint32_t *cand_hist;
  void *topk_scratch;
  void *select_scratch;
  void *sort_scratch;
  void *resolve_scratch;
  size_t bytes;
};

BalancePlan plan_balance(void *workspace, int64_t n, int64_t m, int dtype, int64_t capacity) {
  Carver cv(workspace);
  BalancePlan p;
  const size_t cap = (size_t)list_capacity(capacity > 0 ? capacity : 1);
  p.sel_idx = cv.take<int32_t>(cap);
  p.sel_val = cv.take<uint32_t>(cap);
  p.keys_a = cv.take<uint32_t>(cap);
  p.perm_a = cv.take<uint32_t>(cap);
  p.keys_b = cv.take<uint32_t>(cap);
  p.perm_b = cv.take<uint32_t>(cap);
  p.more_a = cv.take<uint32_t>(cap);
  p.more_b = cv.take<uint32_t>(cap);
  p.count = cv.take<uint32_t>(2);
  p.thr = cv.take<uint32_t>(4);
  p.cand_hist = cv.take<uint32_t>((size_t)kCandHistWords);
  p.topk_scratch = cv.take<char>(topk_scratch_bytes());
  p.select_scratch = cv.take<char>(select_scratch_bytes(n, dtype));
  p.sort_scratch = cv.take<char>(sort_scratch_bytes((int64_t)cap));
  // m + P + 1 <= 2 m + 1 bounds the final-position keys whatever the partition count
  p.resolve_scratch = cv.take<char>(resolve_scratch_bytes((int64_t)cap, 2ull * (uint64_t)m + 1));
  p.bytes = cv.used;
  return p;
}

// Stage 1 of load balance: an (index, value) list in p.sel_* with its length in
// p.count[0], and in *filter the threshold the later stages must still apply to
// it (nullptr: every entry is selected).  k > 0 asks for the k largest
// magnitudes (ties at the threshold kept); the threshold goes to p.thr[0..1].
int select_stage(const BalancePlan &p, const void *input, int dtype, int64_t n, const uint32_t *thr, int64_t k,
                 int64_t capacity, int mode, const uint32_t **filter, int32_t *status, hipStream_t s) {
  SelectArgs sel;
  sel.in = input;
  sel.dtype = dtype;
  sel.n = n;
  sel.thr = thr;
  sel.out_idx = p.sel_idx;
  sel.out_val = p.sel_val;
  sel.capacity = list_capacity(capacity);
  sel.out_count32 = &p.count[0];
  sel.ordered = false;  // the sort below fixes the order
  sel.scratch = p.select_scratch;
  sel.status = status;
  *filter = nullptr;
  if (k <= 0) return select_compact(sel, s);
  int rc;
  if (mode == ZEN_MODE_GENERAL || n < kSampleMinElems) {
    // exact radix select over the whole tensor, then one compaction pass
    if ((rc = topk_exact(input, dtype, n, nullptr, k, p.thr, p.topk_scratch, status, 0, s)) != ZEN_OK) return rc;
    sel.thr = p.thr;
    return select_compact(sel, s);
  }
  // one pass: compact everything at or above a floor estimated from a sample,
  // histogram those candidates on the way, read the exact threshold off the
  // histogram; entries between floor and threshold stay in the list and are
  // filtered by the later stages
  if ((rc = topk_sampled_floor(input, dtype, n, k, p.thr + 2, p.topk_scratch, s)) != ZEN_OK) return rc;
  launch_fill<uint32_t>(p.cand_hist, 0u, (size_t)kCandHistWords, s);
  ZEN_LAUNCH_CHECK("clear candidate histogram");
  sel.thr = p.thr + 2;
  sel.cand_hist = p.cand_hist;
  sel.pick_k = k;
  sel.pick_thr = p.thr;
  if ((rc = select_compact(sel, s)) != ZEN_OK) return rc;
  if (dtype == ZEN_F32) {
    // the histogram resolved 15 key bits; the remaining 16 need the radix select, over the candidates only
    if ((rc = topk_exact(p.sel_val, dtype, sel.capacity, &p.count[0], k, p.thr, p.topk_scratch, status,
                         ZEN_STAT_RETRY, s)) != ZEN_OK)
      return rc;
  }
  *filter = p.thr;
  return ZEN_OK;
}

}  // namespace
}  // namespace zen

extern "C" {

int zen_hash_index(int32_t *out, int64_t n, int partitions, void *stream) {
  using namespace zen;
  if (!out) return fail(ZEN_EINVAL, "zen_hash_index: null pointer");
  if (n <= 0 || n > 0x7fffffffll || partitions <= 0 || n / partitions == 0)
    return fail(ZEN_EINVAL, "zen_hash_index: need 0 < partitions <= n < 2^31");
  int64_t blocks = ceil_div(n, 256 * 4);
  if (blocks > 65536) blocks = 65536;
  k_hash_index<<<dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      out, (uint32_t)n, (uint32_t)(n / partitions));
  ZEN_LAUNCH_CHECK("k_hash_index");
  return ZEN_OK;
}

int zen_sparse_balance(const void *input, int dtype, int64_t n, int32_t *memory, int64_t m, int32_t *serial,
                       int64_t serial_n, int32_t *offset, int partitions, int rehash, int32_t *status,
                       void *stream) {
  using namespace zen;
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_sparse_balance: bad dtype");
  if (n < 0 || n > 0x7fffffffll || m <= 0 || m > 0x7fffffffll || partitions <= 0 || m % partitions != 0 ||
      serial_n < 0 || serial_n > 0x7fffffffll)
    return fail(ZEN_EINVAL, "zen_sparse_balance: need n, m < 2^31 and m a positive multiple of partitions");
  if (n == 0) return ZEN_OK;
  if (!input || !memory || !offset || !status || (serial_n > 0 && !serial))
    return fail(ZEN_EINVAL, "zen_sparse_balance: null pointer");
  Probe g;
  g.m = (uint32_t)m;
  g.npp = (uint32_t)(m / partitions);
  g.levels = (rehash == 2 || rehash == 3) ? rehash : 1;  // functions_cuda_kernel.cu:192-198
  const int64_t spp = serial_n / partitions;
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint32_t *table = reinterpret_cast<uint32_t *>(memory);
  if (dtype == ZEN_BF16)
    return sparse_balance_launch(static_cast<const uint16_t *>(input), n, table, g, serial, spp, offset,
                                 partitions, status, s);
  return sparse_balance_launch(static_cast<const uint32_t *>(input), n, table, g, serial, spp, offset,
                               partitions, status, s);
}

size_t zen_load_balance_workspace(int64_t n, int64_t m, int dtype, int64_t capacity, int partitions) {
  if (n <= 0 || m <= 0 || capacity < 0) return 0;
  const size_t general = zen::plan_balance(nullptr, n, m, dtype, capacity).bytes;
  const size_t slabs = partitions > 0 && m % partitions == 0 ? zen::slab_balance_bytes(m, partitions, dtype, capacity) : 0;
  const size_t wide = partitions > 0 && m % partitions == 0
                          ? zen::wide_balance_bytes(m, partitions, dtype, capacity, zen::wide_device_cus())
                          : 0;
  const size_t fast = slabs > wide ? slabs : wide;
  return general > fast ? general : fast;
}

int zen_load_balance_path(int64_t n, int64_t m, int dtype, int64_t capacity, int partitions, int64_t k, int mode) {
  const bool slabs_only = (mode & ZEN_MODE_SLABS) != 0;
  mode &= 0xff;
  if (mode != ZEN_MODE_FAST || partitions <= 0 || m <= 0 || m % partitions != 0) return 0;
  if (!slabs_only && zen::wide_balance_fits(m, partitions, capacity, k, zen::wide_device_cus(), nullptr)) return 3;
  if (zen::slab_balance_fits(n, m, partitions, dtype, capacity, k, nullptr)) return 2;
  return m >= 4096 ? 1 : 0;
}

namespace {

// the head of the table belongs to the hash map; the megabyte behind it is left to the slab path's counters
uint32_t slab_hash_log2(int64_t m) {
  uint32_t log2 = 0;
  while (log2 < 24 && (16ull << log2) + (1ull << 20) <= (uint64_t)m * sizeof(int32_t)) ++log2;
  return log2;
}

}  // namespace

int zen_load_balance_prepare(const void *input, int dtype, int64_t n, int64_t m, int partitions, int64_t k,
                             int64_t capacity, int32_t *table, int mode, void *workspace, size_t workspace_bytes,
                             void *stream) {
  using namespace zen;
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_load_balance_prepare: bad dtype");
  if (n <= 0 || n > 0x7fffffffll || m <= 0 || m > 0x7fffffffll || partitions <= 0 || partitions > 65535 ||
      m % partitions != 0 || capacity <= 0 || capacity > 0x1fffffffll || k < 0 || k > n)
    return fail(ZEN_EINVAL, "zen_load_balance_prepare: sizes as for zen_load_balance");
  if (!input || !table || !workspace) return fail(ZEN_EINVAL, "zen_load_balance_prepare: null pointer");
  if (workspace_bytes < zen_load_balance_workspace(n, m, dtype, capacity, partitions))
    return fail(ZEN_EWORKSPACE, "zen_load_balance_prepare: workspace too small");
  const int second = (mode & ZEN_MODE_SECOND) != 0;
  if ((mode & 0xff) != ZEN_MODE_FAST || k == 0 || (reinterpret_cast<uintptr_t>(table) & 7u) != 0 ||
      (!slab_balance_fits(n, m, partitions, dtype, capacity, k, nullptr) &&
       !wide_balance_fits(m, partitions, capacity, k, wide_device_cus(), nullptr)))
    return ZEN_OK;  // nothing to take ahead on the other paths
  SlabBalanceArgs sa{};
  sa.input = input;
  sa.dtype = dtype;
  sa.n = n;
  sa.g.m = (uint32_t)m;
  sa.g.npp = (uint32_t)(m / partitions);
  sa.g.levels = 3;
  sa.partitions = partitions;
  sa.k = k;
  sa.capacity = capacity;
  sa.hash = reinterpret_cast<unsigned long long *>(table);
  sa.hash_log2 = slab_hash_log2(m);
  sa.workspace = workspace;
  sa.prepared = second ? 2 : 1;
  sa.second = second != 0;
  sa.only_prepare = true;
  sa.discard = (mode & ZEN_MODE_DISCARD) != 0;
  return slab_prepare(sa, static_cast<hipStream_t>(stream));
}

}  // extern "C"

namespace {

// zen_load_balance, and for zen_encode_merge the same with the next call's tensor handed along.
int load_balance_call(const void *input, int dtype, int64_t n, int64_t m, int partitions, int rehash,
                      const uint32_t *thr, int64_t k, uint32_t *thr_out, int32_t *out_idx, void *out_val,
                      int64_t capacity, int64_t *splits, int32_t *table, int mode, void *workspace,
                      size_t workspace_bytes, int32_t *status, void *stream, const void *next_input, int64_t next_k,
                      int64_t next_n, int64_t next_m, int64_t next_capacity, int32_t *next_table) {
  using namespace zen;
  const int prepared = (mode & ZEN_MODE_PREPARED) ? ((mode & ZEN_MODE_SECOND) ? 2 : 1) : 0;
  const bool second_set = (mode & ZEN_MODE_SECOND) != 0;
  const uint32_t *near_key = nullptr;
  if (mode & ZEN_MODE_FLOOR) {
    if (k <= 0 || !thr) return fail(ZEN_EINVAL, "zen_load_balance: ZEN_MODE_FLOOR needs k > 0 and the key in thr");
    near_key = thr;
    thr = nullptr;  // paths that take no sample have no use for it
  }
  const bool slabs_only = (mode & ZEN_MODE_SLABS) != 0;
  mode &= ~(ZEN_MODE_PREPARED | ZEN_MODE_SECOND | ZEN_MODE_FLOOR | ZEN_MODE_SLABS);
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_load_balance: bad dtype");
  if (mode != ZEN_MODE_FAST && mode != ZEN_MODE_GENERAL) return fail(ZEN_EINVAL, "zen_load_balance: bad mode");
  if (n <= 0 || n > 0x7fffffffll || m <= 0 || m > 0x7fffffffll || partitions <= 0 || partitions > 65535 ||
      m % partitions != 0 || capacity <= 0 || capacity > 0x1fffffffll)
    return fail(ZEN_EINVAL, "zen_load_balance: need 0 < n, m < 2^31, m a multiple of partitions, 0 < capacity < 2^29");
  if (k < 0 || k > n || (k > 0 && thr)) return fail(ZEN_EINVAL, "zen_load_balance: need 0 <= k <= n and no thr with k");
  if (!input || !out_idx || !out_val || !splits || !table || !workspace || !status)
    return fail(ZEN_EINVAL, "zen_load_balance: null pointer");
  if (workspace_bytes < zen_load_balance_workspace(n, m, dtype, capacity, partitions))
    return fail(ZEN_EWORKSPACE, "zen_load_balance: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  Probe g;
  g.m = (uint32_t)m;
  g.npp = (uint32_t)(m / partitions);
  g.levels = (rehash == 2 || rehash == 3) ? rehash : 1;
  const int64_t spp = n / partitions / 10;  // tensor_load_balance.py:18
  const uint32_t drop_key = (uint32_t)partitions * (g.npp + 1u);
  const int bits = ceil_log2_u64(drop_key);
  const bool wide = mode == ZEN_MODE_FAST && !slabs_only && (reinterpret_cast<uintptr_t>(table) & 7u) == 0 &&
                    wide_balance_fits(m, partitions, capacity, k, wide_device_cus(), nullptr);
  if (wide || (mode == ZEN_MODE_FAST && (reinterpret_cast<uintptr_t>(table) & 7u) == 0 &&
               slab_balance_fits(n, m, partitions, dtype, capacity, k, nullptr))) {
    SlabBalanceArgs sa;
    sa.input = input;
    sa.dtype = dtype;
    sa.n = n;
    sa.g = g;
    sa.partitions = partitions;
    sa.spp = spp;
    sa.thr = thr;
    sa.k = k;
    sa.thr_out = thr_out;
    sa.out_idx = out_idx;
    sa.out_val = out_val;
    sa.capacity = capacity;
    sa.splits = splits;
    sa.hash = reinterpret_cast<unsigned long long *>(table);
    sa.hash_log2 = slab_hash_log2(m);
    sa.workspace = workspace;
    sa.status = status;
    sa.prepared = near_key ? 0 : prepared;
    sa.second = second_set;
    sa.near_key = near_key;
    if (next_input && next_k > 0) {
      sa.next_input = next_input;
      sa.next_k = next_k;
      if (next_n > 0 || next_m > 0 || next_capacity > 0 || next_table) {  // a next call of its own size
        const int64_t n2 = next_n > 0 ? next_n : n, m2 = next_m > 0 ? next_m : m;
        const int64_t cap2 = next_capacity > 0 ? next_capacity : capacity;
        int32_t *table2 = next_table ? next_table : table;
        if (n2 > 0x7fffffffll || m2 > 0x7fffffffll || m2 % partitions != 0 || cap2 > 0x1fffffffll || next_k > n2 ||
            (reinterpret_cast<uintptr_t>(table2) & 7u) != 0 ||
            (!(!slabs_only && wide_balance_fits(m2, partitions, cap2, next_k, wide_device_cus(), nullptr)) &&
             !slab_balance_fits(n2, m2, partitions, dtype, cap2, next_k, nullptr)))  // (with this call's ZEN_MODE_SLABS)
          return fail(ZEN_EINVAL, "zen_encode_merge: the next call's sizes do not take a path that keeps a sample");
        if (workspace_bytes < zen_load_balance_workspace(n2, m2, dtype, cap2, partitions))
          return fail(ZEN_EWORKSPACE, "zen_encode_merge: workspace too small for the next call");
        sa.next_n = n2;
        sa.next_state = reinterpret_cast<char *>(table2) + slab_state_offset(slab_hash_log2(m2));
      }
    }
    if (wide) return wide_load_balance(sa, slab_state_offset(sa.hash_log2), s);
    return slab_load_balance(sa, s);
  }
  BalancePlan p = plan_balance(workspace, n, m, dtype, capacity);

  const uint32_t *filter = nullptr;
  int rc = select_stage(p, input, dtype, n, thr, k, capacity, mode, &filter, status, s);
  if (rc != ZEN_OK) return rc;
  if (k > 0 && thr_out) ZEN_HIP_CHECK(hipMemcpyAsync(thr_out, p.thr, 2 * sizeof(uint32_t), hipMemcpyDeviceToDevice, s));
  const int64_t lcap = list_capacity(capacity);
  if (mode == ZEN_MODE_FAST && m >= 4096 && (reinterpret_cast<uintptr_t>(table) & 7u) == 0) {
    // sort-based resolution: the table only lends its (zero) memory to a small hash map
    ResolveArgs ra;
    ra.dense = input;
    ra.dtype = dtype;
    ra.g = g;
    ra.partitions = partitions;
    ra.spp = spp;
    ra.list_idx = p.sel_idx;
    ra.list_val = p.sel_val;
    ra.count = p.count;
    ra.filter = filter;
    ra.list_cap = lcap;
    ra.expected = k > 0 ? k + k / 16 + 1024 : capacity;
    ra.keys_a = p.keys_a;
    ra.perm_a = p.perm_a;
    ra.keys_b = p.keys_b;
    ra.perm_b = p.perm_b;
    ra.more_a = p.more_a;
    ra.more_b = p.more_b;
    ra.sort_scratch = p.sort_scratch;
    ra.hash = reinterpret_cast<unsigned long long *>(table);
    uint32_t log2 = 0;
    while (log2 < 24 && (2ull << log2) <= (uint64_t)m / 2) ++log2;
    ra.hash_log2 = log2;
    ra.scratch = p.resolve_scratch;
    ra.out_idx = out_idx;
    ra.out_val = out_val;
    ra.capacity = capacity;
    ra.splits = splits;
    ra.status = status;
    return resolve_and_place(ra, s);
  }
  const unsigned blocks = (unsigned)ceil_div(lcap, 256);
  uint32_t *tab = reinterpret_cast<uint32_t *>(table);
  const uint16_t *val16 = reinterpret_cast<const uint16_t *>(p.sel_val);
  {
    ProfScope prof(kProfInsertList, s);
    if (dtype == ZEN_BF16)
      k_insert_list<uint16_t><<<dim3(blocks), dim3(256), 0, s>>>(p.sel_idx, val16, p.count, filter, tab, g);
    else
      k_insert_list<uint32_t><<<dim3(blocks), dim3(256), 0, s>>>(p.sel_idx, p.sel_val, p.count, filter, tab, g);
    ZEN_LAUNCH_CHECK("k_insert_list");
  }
  {
    ProfScope prof(kProfFinalKey, s);
    if (dtype == ZEN_BF16)
      k_final_key<uint16_t><<<dim3(blocks), dim3(256), 0, s>>>(p.sel_idx, val16, p.count, filter, tab, g, drop_key,
                                                               p.keys_a, p.perm_a);
    else
      k_final_key<uint32_t><<<dim3(blocks), dim3(256), 0, s>>>(p.sel_idx, p.sel_val, p.count, filter, tab, g, drop_key,
                                                               p.keys_a, p.perm_a);
    ZEN_LAUNCH_CHECK("k_final_key");
  }
  int where;
  {
    ProfScope prof(kProfSort, s);
    where = sort_pairs(p.keys_a, p.perm_a, p.keys_b, p.perm_b, lcap, p.count, bits, p.sort_scratch, status, s);
  }
  if (where < 0) return where;
  const uint32_t *sk = where ? p.keys_b : p.keys_a;
  const uint32_t *sp = where ? p.perm_b : p.perm_a;
  {
    ProfScope prof(kProfGather, s);
    if (dtype == ZEN_BF16)
      k_gather<uint16_t><<<dim3(blocks), dim3(256), 0, s>>>(sk, sp, p.count, p.sel_idx, val16, drop_key, g, out_idx,
                                                            static_cast<uint16_t *>(out_val), (uint32_t)capacity, tab);
    else
      k_gather<uint32_t><<<dim3(blocks), dim3(256), 0, s>>>(sk, sp, p.count, p.sel_idx, p.sel_val, drop_key, g, out_idx,
                                                            static_cast<uint32_t *>(out_val), (uint32_t)capacity, tab);
    ZEN_LAUNCH_CHECK("k_gather");
  }
  if (dtype == ZEN_BF16)
    k_splits_serial<uint16_t><<<dim3((unsigned)partitions), dim3(256), 0, s>>>(
        sk, p.count, g.npp, spp, (uint32_t)capacity, static_cast<const uint16_t *>(input), out_idx,
        static_cast<uint16_t *>(out_val), splits, status);
  else
    k_splits_serial<uint32_t><<<dim3((unsigned)partitions), dim3(256), 0, s>>>(
        sk, p.count, g.npp, spp, (uint32_t)capacity, static_cast<const uint32_t *>(input), out_idx,
        static_cast<uint32_t *>(out_val), splits, status);
  ZEN_LAUNCH_CHECK("k_splits_serial");
  return ZEN_OK;
}

}  // namespace

extern "C" {

int zen_load_balance(const void *input, int dtype, int64_t n, int64_t m, int partitions, int rehash,
                     const uint32_t *thr, int64_t k, uint32_t *thr_out, int32_t *out_idx, void *out_val,
                     int64_t capacity, int64_t *splits, int32_t *table, int mode, void *workspace,
                     size_t workspace_bytes, int32_t *status, void *stream) {
  return load_balance_call(input, dtype, n, m, partitions, rehash, thr, k, thr_out, out_idx, out_val, capacity, splits,
                           table, mode, workspace, workspace_bytes, status, stream, nullptr, 0, 0, 0, 0, nullptr);
}

int zen_encode_merge_samples_next(int64_t n, int64_t m, int dtype, int64_t capacity, int partitions, int64_t k,
                                  int mode) {
  const int path = zen_load_balance_path(n, m, dtype, capacity, partitions, k, mode);
  return path == 2 || path == 3;
}

int zen_encode_merge(const zen_encode_merge_args *a) {
  using namespace zen;
  if (!a) return fail(ZEN_EINVAL, "zen_encode_merge: null pointer");
  const int rc = load_balance_call(a->input, a->dtype, a->n, a->m, a->partitions, a->rehash, a->thr, a->k, a->thr_out,
                                   a->out_idx, a->out_val, a->capacity, a->splits, a->table, a->mode, a->workspace,
                                   a->workspace_bytes, a->status, a->stream, a->next_input, a->next_k, a->next_n,
                                   a->next_m, a->next_capacity, a->next_table);
  if (rc != ZEN_OK) return rc;
  return zen_merge(a->recv_idx, a->recv_idx64, a->recv_val, a->dtype, a->r, a->dense_n, a->merged_idx, a->merged_idx64,
                   a->merged_val, a->merged_capacity, a->merged_count, a->merge_mode, a->merge_workspace,
                   a->merge_workspace_bytes, a->merge_status, a->merge_stream ? a->merge_stream : a->stream);
}

}  // extern "C"
