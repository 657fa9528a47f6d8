// Owner resolution without a table of the reference's size.
//
// The reference insert (functions_cuda_kernel.cu:97-167) decides who owns a slot
// by looking into an int32 table of M entries; at M = 7e8 that is 3 GB of random
// accesses for a few million insertions.  Here the selected entries are sorted
// by their level-1 slot instead.  In the sorted array the smallest index of
// every run of equal slots is that slot's smallest level-1 prober ("head"); all
// other members of a run lost level 1.  Only those losers (well under 1 % of the
// entries at the densities this path sees) and the heads they push out ever
// touch a hash map, which holds per slot the smallest index that probed it at
// level 2 or 3.  The rule is the reference's run in ascending thread order:
//   a slot belongs to the smallest index that ever probes it, and an index
//   probes its next level only if a smaller index owns the slot it tried.
// A thread that takes a slot from a larger index carries on with that index's
// probe sequence, so every lost probe is continued exactly once.
//
// Survivors (heads nobody pushed out) are already in final order; the moved
// entries are sorted by their final position with the two-level bin sort (they
// are few, so its atomics cost nothing) and the two sequences are merged by
// rank: position = own rank + number of entries of the other sequence in front.
#include "zen_balance.h"
#include "zen_binsort.h"
#include "zen_hashmap.h"
#include "zen_slab.h"

namespace zen {
namespace {

// ------------------------------------------------------------ level-1 keys

// Sort records: key = level-1 slot, payloads = the index and the value bits, so
// nothing downstream has to gather from the unsorted list.
template <typename S>
__global__ __launch_bounds__(256) void k_slot_key(const int32_t *__restrict__ list_idx, const S *__restrict__ list_val,
                                                  const uint32_t *count, const uint32_t *__restrict__ filter, Probe g,
                                                  uint32_t *__restrict__ keys, uint32_t *__restrict__ tids,
                                                  uint32_t *__restrict__ vals) {
  const uint32_t j = blockIdx.x * 256u + threadIdx.x;
  if (j >= *count) return;
  uint32_t t;
  keys[j] = list_selected<S>(list_idx, list_val, filter, j, &t) ? first_slot(g, t) : g.m;  // g.m sorts last
  tids[j] = t;
  vals[j] = (uint32_t)list_val[j];
}

// Smallest index among the sorted entries whose slot is s, and where it sits.
__device__ inline uint32_t run_head(const uint32_t *sk, const uint32_t *st, uint32_t n, uint32_t s,
                                    uint32_t *pos_out) {
  uint32_t p = lower_bound_u32(sk, n, s);
  uint32_t best = kNone;
  for (; p < n && sk[p] == s; ++p) {
    const uint32_t t = st[p] & kIndexMask;
    if (t < best) {
      best = t;
      *pos_out = p;
    }
  }
  return best;
}

// Every member of a run except its smallest index lost level 1.  A block looks
// at kHeadItems entries per thread and appends its losers with one atomic add
// (thousands of single adds on one counter would serialise).
constexpr int kHeadBlock = 1024;
constexpr int kHeadItems = 4;

__global__ __launch_bounds__(kHeadBlock) void k_heads(const uint32_t *__restrict__ sk, uint32_t *st,
                                                      const uint32_t *__restrict__ sv, const uint32_t *count,
                                                      uint32_t m, uint32_t log_cap, uint32_t *log_t, uint32_t *log_v,
                                                      Counters *ctr, int32_t *status) {
  __shared__ uint32_t s_count, s_base;
  if (threadIdx.x == 0) s_count = 0;
  __syncthreads();
  const uint32_t n = *count;
  uint32_t lost_t[kHeadItems], lost_v[kHeadItems];
  int mine = 0;
#pragma unroll
  for (int q = 0; q < kHeadItems; ++q) {
    const uint32_t p = (blockIdx.x * kHeadItems + q) * kHeadBlock + threadIdx.x;
    if (p >= n) continue;
    const uint32_t s = sk[p];
    if (s >= m) continue;
    const bool prev_same = p > 0 && sk[p - 1] == s;
    const bool next_same = p + 1 < n && sk[p + 1] == s;
    if (!prev_same && !next_same) continue;
    const uint32_t t = st[p] & kIndexMask;
    bool lost = false;
    for (uint32_t u = p; u > 0 && sk[u - 1] == s && !lost; --u) lost = (st[u - 1] & kIndexMask) < t;
    for (uint32_t u = p + 1; u < n && sk[u] == s && !lost; ++u) lost = (st[u] & kIndexMask) < t;
    if (!lost) continue;
    atomicOr(&st[p], kRemovedBit);
    lost_t[mine] = t;
    lost_v[mine] = sv[p];
    ++mine;
  }
  uint32_t at = mine ? atomicAdd(&s_count, (uint32_t)mine) : 0u;
  __syncthreads();
  if (threadIdx.x == 0 && s_count) s_base = atomicAdd(&ctr->logged, s_count);
  __syncthreads();
  if (!mine) return;
  at += s_base;
  for (int q = 0; q < mine; ++q, ++at) {
    if (at < log_cap) {
      log_t[at] = lost_t[q];
      log_v[at] = lost_v[q];
    } else {
      atomicOr(status, ZEN_STAT_RETRY);
    }
  }
}

__global__ void k_snapshot(Counters *ctr, uint32_t log_cap) {
  ctr->losers = ctr->logged < log_cap ? ctr->logged : log_cap;
}

// Levels 2 and 3 for every loser, with eviction chains.
__global__ __launch_bounds__(256) void k_chains(const uint32_t *__restrict__ sk, uint32_t *st,
                                                const uint32_t *__restrict__ sv, const uint32_t *count, Probe g,
                                                unsigned long long *cells, uint32_t log2, uint32_t log_cap,
                                                uint32_t *log_t, uint32_t *log_v, Counters *ctr, int32_t *status) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= ctr->losers) return;
  const uint32_t n = *count;
  uint32_t cur = log_t[i];
  int lv = 1;
  bool full = false;
  for (uint32_t steps = 0; lv < g.levels; ++steps) {
    if (steps > kChainLimit) {
      atomicOr(status, ZEN_STAT_INTERNAL);
      return;
    }
    uint32_t part;
    const uint32_t slot = probe_slot(g, cur, lv, &part);
    uint32_t head_pos = 0;
    const uint32_t head = run_head(sk, st, n, slot, &head_pos);
    if (head < cur) {  // a smaller index probes this slot at level 1: cur moves on
      ++lv;
      continue;
    }
    const uint32_t old = map_min(cells, log2, slot, cur, ctr, &full);
    if (full) {
      atomicOr(status, ZEN_STAT_RETRY);
      return;
    }
    if (old < cur) {  // a smaller index got here at level 2 or 3
      ++lv;
      continue;
    }
    if (old == kNone) {
      // first level-2/3 prober of this slot: its level-1 head (a larger index, if any) is pushed out
      if (head == kNone) return;
      atomicOr(&st[head_pos], kRemovedBit);
      const uint32_t at = atomicAdd(&ctr->logged, 1u);
      if (at < log_cap) {
        log_t[at] = head;
        log_v[at] = sv[head_pos];
      } else {
        atomicOr(status, ZEN_STAT_RETRY);
      }
      cur = head;
      lv = 1;
      continue;
    }
    if (old == cur) return;
    // took the slot from a larger index that held it at its first level mapping here
    int lw = 1;
    while (lw < g.levels && probe_slot(g, old, lw, &part) != slot) ++lw;
    cur = old;
    lv = lw + 1;
  }
}

// Final position key of every logged index: partition-major, slot inside the
// partition, serial entries behind all slots (they share one key).  Also the
// bin histogram of the sort that follows.
__global__ __launch_bounds__(256) void k_classify(const uint32_t *__restrict__ log_t,
                                                  const Counters *ctr, uint32_t log_cap, Probe g,
                                                  const unsigned long long *__restrict__ cells, uint32_t log2,
                                                  uint32_t *__restrict__ ins_key, uint32_t *__restrict__ ins_j,
                                                  uint32_t *__restrict__ ins_cell, uint32_t *hist, int bshift) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  const uint32_t total = ctr->logged < log_cap ? ctr->logged : log_cap;
  if (i >= total) return;
  const uint32_t t = log_t[i];
  uint32_t part = 0;
  uint32_t key = kNone, cell = kNone;
  for (int lv = 1; lv < g.levels && key == kNone; ++lv) {
    const uint32_t slot = probe_slot(g, t, lv, &part);
    uint32_t at = 0;
    if (map_find(cells, log2, slot, &at) == t) {
      key = part * (g.npp + 1u) + (slot - part * g.npp);
      cell = at;
    }
  }
  ins_cell[i] = cell;
  if (key == kNone) {
    part = first_slot(g, t) / g.npp;
    key = part * (g.npp + 1u) + g.npp;
  }
  ins_key[i] = key;
  ins_j[i] = i;  // the moved entry's place in the log
  atomicAdd(&hist[key >> bshift], 1u);
}

// Every occupied cell ends with the index that finally holds its slot, and that
// index recorded the cell: clearing by cell number leaves the map empty without
// probing through cells that are being cleared.
__global__ __launch_bounds__(256) void k_map_clear(const uint32_t *__restrict__ ins_cell, const Counters *ctr,
                                                   uint32_t log_cap, unsigned long long *cells) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  const uint32_t total = ctr->logged < log_cap ? ctr->logged : log_cap;
  if (i < total && ins_cell[i] != kNone) cells[ins_cell[i]] = 0ull;
}

// Exclusive prefix of "survivor" over the sorted entries, kept per group of 16
// consecutive entries as (survivors before the group, flag bits of the group):
// one coalesced pair of words per thread instead of a word per entry.
constexpr int kSurvBlock = 1024;
constexpr int kSurvItems = 16;
constexpr int kSurvTile = kSurvBlock * kSurvItems;  // few, large tiles: a short prefix chain

__device__ inline uint32_t survivors_before(const uint2 *__restrict__ groups, uint32_t pos) {
  const uint2 gr = groups[pos >> 4];
  return gr.x + (uint32_t)__popc(gr.y & ((1u << (pos & 15u)) - 1u));
}

__global__ __launch_bounds__(kSurvBlock) void k_survivors(const uint32_t *__restrict__ sk, const uint32_t *__restrict__ sp,
                                                          const uint32_t *count, uint32_t m, ScanState st, int ntiles,
                                                          uint2 *__restrict__ groups, int32_t *status) {
  __shared__ uint32_t s_scan[kSurvBlock / 64 + 1];
  __shared__ uint64_t s_bcast;
  __shared__ int s_tile;
  if (threadIdx.x == 0) s_tile = (int)atomicAdd(st.ticket, 1u);
  __syncthreads();
  const int tile = s_tile;
  if (tile >= ntiles) return;
  const uint32_t n = *count;
  const uint32_t first = (uint32_t)tile * kSurvTile + threadIdx.x * kSurvItems;
  uint32_t flags = 0;
  if (first + kSurvItems <= n) {
    const uint4 *k4 = reinterpret_cast<const uint4 *>(sk + first);
    const uint4 *p4 = reinterpret_cast<const uint4 *>(sp + first);
#pragma unroll
    for (int v = 0; v < kSurvItems / 4; ++v) {
      const uint4 kk = k4[v], pp = p4[v];
      const uint32_t ks[4] = {kk.x, kk.y, kk.z, kk.w}, ps[4] = {pp.x, pp.y, pp.z, pp.w};
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (ks[e] < m && !(ps[e] & kRemovedBit)) flags |= 1u << (4 * v + e);
    }
  } else {
#pragma unroll
    for (int q = 0; q < kSurvItems; ++q) {
      const uint32_t p = first + q;
      if (p < n && sk[p] < m && !(sp[p] & kRemovedBit)) flags |= 1u << q;
    }
  }
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kSurvBlock>((uint32_t)__popc(flags), s_scan, &total);
  const uint32_t run = (uint32_t)lookback_exclusive(st, tile, total, status, &s_bcast) + before;
  groups[first >> 4] = make_uint2(run, flags);
}

// Survivors and moved entries to their final places.
template <typename S>
__global__ __launch_bounds__(256) void k_place(const uint32_t *__restrict__ sk, const uint32_t *__restrict__ st,
                                               const uint32_t *__restrict__ sv, const uint32_t *count,
                                               const uint2 *__restrict__ groups, const uint32_t *__restrict__ ik,
                                               const uint32_t *__restrict__ ii, const uint32_t *__restrict__ bin_start,
                                               int bshift, const uint32_t *__restrict__ log_t,
                                               const uint32_t *__restrict__ log_v, const Counters *ctr,
                                               uint32_t log_cap, const uint32_t *retry, Probe g,
                                               int32_t *__restrict__ out_idx, S *__restrict__ out_val,
                                               uint32_t capacity, int32_t *status) {
  const uint32_t x = blockIdx.x * 256u + threadIdx.x;
  const uint32_t n = *count;
  const uint32_t moved = ctr->logged < log_cap ? ctr->logged : log_cap;
  if (*retry) {
    if (x == 0) atomicOr(status, ZEN_STAT_RETRY);
    return;
  }
  if (x < n) {
    const uint32_t s = sk[x];
    const uint32_t t = st[x];
    if (s < g.m && !(t & kRemovedBit)) {
      const uint32_t part = s / g.npp;
      const uint32_t key = part * (g.npp + 1u) + (s - part * g.npp);
      // moved entries in front of it: whole bins below its bin, then a look inside the bin
      const uint32_t b = key >> bshift;
      uint32_t in_front = bin_start[b];
      for (const uint32_t end = bin_start[b + 1]; in_front < end && ik[in_front] < key; ++in_front) {}
      const uint32_t pos = survivors_before(groups, x) + in_front;
      if (pos < capacity) {
        out_idx[pos] = (int32_t)t;
        out_val[pos] = (S)sv[x];
      }
    }
  }
  if (x < moved) {
    const uint32_t key = ik[x];
    const uint32_t part = key / (g.npp + 1u), local = key - part * (g.npp + 1u);
    const uint32_t bound = local < g.npp ? part * g.npp + local : (part + 1u) * g.npp;
    const uint32_t pos = x + survivors_before(groups, lower_bound_u32(sk, n, bound));
    if (pos < capacity) {
      out_idx[pos] = (int32_t)log_t[ii[x]];
      out_val[pos] = (S)log_v[ii[x]];
    }
  }
}

template <typename S>
__global__ __launch_bounds__(256) void k_splits_merged(const uint32_t *__restrict__ sk, const uint32_t *count,
                                                       const uint2 *__restrict__ groups,
                                                       const uint32_t *__restrict__ ik, const Counters *ctr,
                                                       uint32_t log_cap, const uint32_t *retry, Probe g, int64_t spp,
                                                       uint32_t capacity, const S *__restrict__ dense,
                                                       int32_t *__restrict__ out_idx, S *__restrict__ out_val,
                                                       int64_t *__restrict__ splits, int32_t *status) {
  __shared__ uint32_t s_b[5];
  __shared__ uint32_t buf[kSerialLds];
  if (*retry) return;
  const uint32_t p = blockIdx.x;
  const uint32_t n = *count;
  const uint32_t moved = ctr->logged < log_cap ? ctr->logged : log_cap;
  if (threadIdx.x == 0) s_b[0] = survivors_before(groups, lower_bound_u32(sk, n, p * g.npp));
  if (threadIdx.x == 1) s_b[1] = survivors_before(groups, lower_bound_u32(sk, n, (p + 1u) * g.npp));
  if (threadIdx.x == 2) s_b[2] = lower_bound_u32(ik, moved, p * (g.npp + 1u));
  if (threadIdx.x == 3) s_b[3] = lower_bound_u32(ik, moved, p * (g.npp + 1u) + g.npp);
  if (threadIdx.x == 4) s_b[4] = lower_bound_u32(ik, moved, (p + 1u) * (g.npp + 1u));
  __syncthreads();
  const uint32_t lo = s_b[0] + s_b[2], hi = s_b[1] + s_b[4], serial = s_b[4] - s_b[3];
  if (threadIdx.x == 0) {
    splits[p] = (int64_t)(hi - lo);
    if ((int64_t)serial > spp) atomicOr(status, ZEN_STAT_SERIAL_OVERFLOW);
    if (hi > capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
  if (hi > capacity) return;
  fix_serial_tail<S>(out_idx, out_val, dense, hi - serial, serial, buf);
}

struct ResolvePlan {
  Counters *ctr;
  uint32_t *ins_key, *ins_j, *tmp_k, *tmp_v, *srt_k, *srt_v;  // moved entries (log_cap each)
  uint2 *groups;                                              // one per 16 sorted entries
  void *scan;
  BinSort bs;
  uint32_t log_cap;
  int surv_tiles;
  size_t bytes;
};

ResolvePlan plan_resolve(void *scratch, int64_t list_cap, uint64_t key_limit) {
  Carver cv(scratch);
  ResolvePlan r;
  r.log_cap = (uint32_t)(list_cap / 4 + 1024);
  r.surv_tiles = (int)ceil_div(list_cap + 1, kSurvTile);
  r.ins_key = cv.take<uint32_t>(r.log_cap);
  r.ins_j = cv.take<uint32_t>(r.log_cap);
  r.tmp_k = cv.take<uint32_t>(r.log_cap);
  r.tmp_v = cv.take<uint32_t>(r.log_cap);
  r.srt_k = cv.take<uint32_t>(r.log_cap);
  r.srt_v = cv.take<uint32_t>(r.log_cap);
  r.groups = cv.take<uint2>((size_t)r.surv_tiles * (kSurvTile / 16));
  // counters and the survivor scan state sit in the bin sort's cleared area
  const size_t extra = 256 + scan_words(r.surv_tiles) * sizeof(unsigned long long);
  char *base = cv.take<char>(plan_binsort(nullptr, key_limit, r.log_cap, extra).bytes);
  r.bs = plan_binsort(scratch ? base : nullptr, key_limit, r.log_cap, extra);
  r.ctr = static_cast<Counters *>(r.bs.extra);
  r.scan = static_cast<char *>(r.bs.extra) + 256;
  r.bytes = cv.used;
  return r;
}

template <typename S>
int resolve_launch(const ResolveArgs &a, hipStream_t s) {
  const Probe g = a.g;
  const uint32_t drop = (uint32_t)a.partitions * (g.npp + 1u);
  ResolvePlan r = plan_resolve(a.scratch, a.list_cap, (uint64_t)drop + 1);
  const S *list_val = static_cast<const S *>(a.list_val);
  const unsigned blocks = (unsigned)ceil_div(a.list_cap, 256);
  const unsigned log_blocks = (unsigned)ceil_div((int64_t)r.log_cap, 256);
  int rc = binsort_clear(r.bs, s);
  if (rc != ZEN_OK) return rc;
  {
    ProfScope prof(kProfInsertList, s);
    k_slot_key<S><<<dim3(blocks), dim3(256), 0, s>>>(a.list_idx, list_val, a.count, a.filter, g, a.keys_a, a.perm_a,
                                                     a.more_a);
    ZEN_LAUNCH_CHECK("k_slot_key");
  }
  int where;
  {
    ProfScope prof(kProfSort, s);
    // level-1 slots are hash values: they spread evenly over [0, m), filtered entries carry the key m
    if (bucket_sort_fits(a.expected, g.m))
      where = bucket_sort_pairs(a.keys_a, a.perm_a, a.keys_b, a.perm_b, a.list_cap, a.count, g.m, a.sort_scratch,
                                a.status, s, a.more_a, a.more_b);
    else
      where = sort_pairs(a.keys_a, a.perm_a, a.keys_b, a.perm_b, a.list_cap, a.count, ceil_log2_u64(g.m),
                         a.sort_scratch, a.status, s, a.more_a, a.more_b);
  }
  if (where < 0) return where;
  uint32_t *sk = where ? a.keys_b : a.keys_a, *st = where ? a.perm_b : a.perm_a, *sv = where ? a.more_b : a.more_a;
  uint32_t *log_t = where ? a.keys_a : a.keys_b, *log_v = where ? a.more_a : a.more_b;  // the idle buffers
  {
    ProfScope prof(kProfFinalKey, s);
    k_heads<<<dim3((unsigned)ceil_div(a.list_cap, kHeadBlock * kHeadItems)), dim3(kHeadBlock), 0, s>>>(
        sk, st, sv, a.count, g.m, r.log_cap, log_t, log_v, r.ctr, a.status);
    ZEN_LAUNCH_CHECK("k_heads");
    k_snapshot<<<dim3(1), dim3(1), 0, s>>>(r.ctr, r.log_cap);
    ZEN_LAUNCH_CHECK("k_snapshot");
    k_chains<<<dim3(log_blocks), dim3(256), 0, s>>>(sk, st, sv, a.count, g, a.hash, a.hash_log2, r.log_cap, log_t,
                                                    log_v, r.ctr, a.status);
    ZEN_LAUNCH_CHECK("k_chains");
    k_classify<<<dim3(log_blocks), dim3(256), 0, s>>>(log_t, r.ctr, r.log_cap, g, a.hash, a.hash_log2, r.ins_key,
                                                      r.ins_j, r.srt_v, r.bs.hist, r.bs.bshift);
    ZEN_LAUNCH_CHECK("k_classify");
    k_map_clear<<<dim3(log_blocks), dim3(256), 0, s>>>(r.srt_v, r.ctr, r.log_cap, a.hash);
    ZEN_LAUNCH_CHECK("k_map_clear");
    if ((rc = binsort_scan(r.bs, a.status, s)) != ZEN_OK) return rc;
    if ((rc = binsort_scatter(r.bs, r.ins_key, r.ins_j, r.log_cap, &r.ctr->logged, r.tmp_k, r.tmp_v, s)) != ZEN_OK)
      return rc;
    if ((rc = binsort_rank(r.bs, r.tmp_k, r.tmp_v, r.log_cap, &r.ctr->logged, r.srt_k, r.srt_v, s)) != ZEN_OK)
      return rc;
    k_survivors<<<dim3((unsigned)r.surv_tiles), dim3(kSurvBlock), 0, s>>>(sk, st, a.count, g.m,
                                                                           scan_state(r.scan, r.surv_tiles),
                                                                           r.surv_tiles, r.groups, a.status);
    ZEN_LAUNCH_CHECK("k_survivors");
  }
  {
    ProfScope prof(kProfGather, s);
    k_place<S><<<dim3(blocks), dim3(256), 0, s>>>(sk, st, sv, a.count, r.groups, r.srt_k, r.srt_v, r.bs.start,
                                                  r.bs.bshift, log_t, log_v, r.ctr, r.log_cap, r.bs.retry, g,
                                                  a.out_idx, static_cast<S *>(a.out_val), (uint32_t)a.capacity,
                                                  a.status);
    ZEN_LAUNCH_CHECK("k_place");
  }
  k_splits_merged<S><<<dim3((unsigned)a.partitions), dim3(256), 0, s>>>(
      sk, a.count, r.groups, r.srt_k, r.ctr, r.log_cap, r.bs.retry, g, a.spp, (uint32_t)a.capacity,
      static_cast<const S *>(a.dense), a.out_idx, static_cast<S *>(a.out_val), a.splits, a.status);
  ZEN_LAUNCH_CHECK("k_splits_merged");
  return ZEN_OK;
}

}  // namespace

size_t resolve_scratch_bytes(int64_t list_cap, uint64_t key_limit) {
  return plan_resolve(nullptr, list_cap, key_limit).bytes;
}

int resolve_and_place(const ResolveArgs &a, hipStream_t stream) {
  if (a.dtype == ZEN_BF16) return resolve_launch<uint16_t>(a, stream);
  return resolve_launch<uint32_t>(a, stream);
}

}  // namespace zen
