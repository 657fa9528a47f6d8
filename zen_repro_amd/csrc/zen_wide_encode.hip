// Fused load balance on wide buckets (zen_wide.h): the fast path of zen_load_balance for selections of a few
// million entries at most.
//
// The reference inserts every selected index into an int32 table as large as the gradient and then scans that
// table partition by partition (functions_cuda_kernel.cu:97-167, tensor_load_balance.py:13-51).  Here the
// select kernel appends its candidates, as (index, level-1 hash slot, value), straight to at most 256 buckets
// (a bucket = a range of level-1 slots; buckets never straddle a partition), and ONE kernel finishes the job
// with one workgroup per bucket, all of them resident at the same time:
//   sort      the bucket's candidates that reach the exact threshold are ranked by (level-1 slot, index)
//             inside LDS; in a run of equal slots the smallest index is the slot's level-1 owner, the others
//             lost level 1 and are logged, per partition;
//   chains    (behind a barrier between the workgroups of a partition) levels 2 and 3 for the partition's
//             losers through a small hash map, with the reference's rule executed in ascending index order: a
//             slot belongs to the smallest index that ever probes it, and whoever takes a slot from a larger
//             index continues that index's probe sequence;
//   classify  (behind a second barrier) the final slot of every logged entry, handed to the bucket that slot
//             lies in, or to the partition's serial list;
//   place     (behind a third) survivors and moved-in entries merged by rank, straight from LDS to the
//             bucket's place in the partition-major output, which follows from the counts the earlier buckets
//             publish; split sizes.
// Nothing but the sorted indices (for the chains' look-ups) goes through memory between the steps.
#include "zen_balance.h"
#include "zen_hashmap.h"
#include "zen_refine.h"
#include "zen_wide.h"

#include <mutex>

namespace zen {

// ------------------------------------------------- one resident launch at a time

namespace {
constexpr int kLineDevices = 64;
std::mutex g_line_mu;
hipEvent_t g_line_event[kLineDevices];
bool g_line_recorded[kLineDevices];
int g_line_cus[kLineDevices];

bool line_capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st != hipStreamCaptureStatusNone;
}
}  // namespace

int wide_line_enter(hipStream_t stream) {
  if (line_capturing(stream)) return ZEN_OK;
  int dev = 0;
  ZEN_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kLineDevices) return ZEN_OK;
  std::lock_guard<std::mutex> lock(g_line_mu);
  if (g_line_recorded[dev]) ZEN_HIP_CHECK(hipStreamWaitEvent(stream, g_line_event[dev], 0));
  return ZEN_OK;
}

int wide_line_leave(hipStream_t stream) {
  if (line_capturing(stream)) return ZEN_OK;
  int dev = 0;
  ZEN_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kLineDevices) return ZEN_OK;
  std::lock_guard<std::mutex> lock(g_line_mu);
  if (!g_line_event[dev]) ZEN_HIP_CHECK(hipEventCreateWithFlags(&g_line_event[dev], hipEventDisableTiming));
  ZEN_HIP_CHECK(hipEventRecord(g_line_event[dev], stream));
  g_line_recorded[dev] = true;
  return ZEN_OK;
}

int wide_device_cus() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kLineDevices) return 0;
  std::lock_guard<std::mutex> lock(g_line_mu);
  if (g_line_cus[dev] == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      g_line_cus[dev] = v;
    else
      g_line_cus[dev] = -1;
  }
  return g_line_cus[dev] > 0 ? g_line_cus[dev] : 0;
}

namespace {

constexpr int kWideItems = 20;                          // raw records per thread (candidates below the threshold included)
constexpr int kWideRaw = kWideBlock * kWideItems;       // raw records per bucket, at most
constexpr int kWideMove = 1024;                         // entries that may move into one bucket from elsewhere
constexpr int kWideRemoved = 1024;                      // entries of a bucket that may lose their level-1 slot
constexpr int kWideGroupLimit = 512;                    // records in one narrow range: bounds the rank loop
constexpr int kWideIndexStep = 4;                       // every 4th narrow range has its first sorted place written down
constexpr int kWideIndexLen = kWideSubs / kWideIndexStep;
constexpr int kWideCtrPad = 8;                          // words between two per-partition counters
constexpr uint32_t kInvalid = 0xffffffffu;
static_assert(kWideRaw <= (1 << 15) && kWideCap <= kWideRaw, "raw places in 15 bits");
static_assert(kWideMove <= kWideBlock && kWideRemoved <= kWideBlock, "one entry per thread");

struct WideTables {
  // zero between calls (kept in the caller's zero table, behind the hash map)
  uint32_t *cursor;            // [B * kWideSplit * kWidePad] part cursors
  uint32_t *gbar;              // [P * kWidePad] barrier counters of the partitions' workgroups
  uint32_t *log_n;             // [P * kWideCtrPad] entries that lost level 1, per partition
  uint32_t *dlog_n;            // [P * kWideCtrPad] level-1 owners pushed out by a level-2/3 prober, per partition
  uint32_t *serial_n;          // [P * kWideCtrPad] entries that found no slot
  uint32_t *movein_n;          // [B] entries whose final slot lies in the bucket but whose level-1 slot does not own it
  uint32_t *dl_n;              // [B] owners pushed out of the bucket
  unsigned long long *desc;    // [B] what every bucket contributes to the output (flag + count)
  uint32_t *done;              // [1] workgroups that have finished
  Counters *ctr;
  // workspace
  uint32_t *words;             // [3][B * kWideSplit * part_cap] raw candidates: index, level-1 slot, value
  uint32_t *slab_idx;          // [B * kWideCap] sorted indices (| kRemovedBit: lost level 1)
  uint32_t *sub_index;         // [B * kWideIndexLen] first sorted place of narrow range 4 j, and of 4 j + 4 in the high half
  uint32_t *bucket_n;          // [B] sorted records
  uint32_t *bucket_lo;         // [B] smallest level-1 slot
  uint32_t *log_t, *log_cell;  // [P * log_cap] losers; the map cell each ends in (kNone: none)
  uint32_t *dlog_t, *dlog_cell;
  uint32_t *mv_slot, *mv_idx;  // [B * kWideMove]
  uint32_t *dl_pos;            // [B * kWideRemoved] sorted places of the owners pushed out
  uint32_t *ser_idx;           // [P * kSlabSerialCap]
  uint32_t part_cap;
  uint32_t log_cap;            // per partition
  int partitions;
};

template <typename S>
struct WideShared {
  union {
    uint32_t word[kWideCap];  // while ranking: (slot inside its narrow range) << 15 | raw place
    uint32_t idx[kWideCap];   // afterwards: the sorted indices (| kRemovedBit)
  };
  union {
    WideCounters cnt;
    S val[kWideCap];          // the sorted values
  };
  uint32_t mk[kWideMove];     // slots of the moved-in entries
  uint32_t mi[kWideMove];     // their indices
  uint32_t mp[kWideMove];     // sorted place in front of which each slips in, by ascending slot
  uint32_t rm[kWideRemoved];  // losers' indices while they are logged, then the sorted places of the removed entries
  int32_t delta[kWideCap / 64];
  uint32_t scan[kWideBlock / 64 + 1];
  uint64_t scan64[kWideBlock / 64 + 1];
  uint32_t lo, lost_n, nrm, base, flag;
};

__device__ inline unsigned long long cell_fresh(const unsigned long long *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// map_find while other workgroups of the running kernel have been writing the map.
__device__ inline uint32_t map_find_fresh(const unsigned long long *cells, uint32_t log2, uint32_t slot, uint32_t *cell_out) {
  const uint32_t mask = (1u << log2) - 1u;
  uint32_t h = cell_home(slot, log2);
  for (uint32_t probes = 0; probes <= mask; ++probes, h = (h + 1u) & mask) {
    const unsigned long long cur = cell_fresh(&cells[h]);
    if (cur == 0ull) return kNone;
    if ((uint32_t)(cur >> 32) == slot + 1u) {
      *cell_out = h;
      return (uint32_t)cur;
    }
  }
  return kNone;
}

// Smallest index whose level-1 slot is `slot` (kNone if nobody's), which bucket it sits in and at which sorted
// place.  The bucket's index narrows the search to the records of kWideIndexStep narrow ranges (three or
// four); they are fetched four at a time and looked at in sorted order: by ascending slot, and in a run of
// equal slots the smallest index comes first.
__device__ inline uint32_t wide_head(const SlabGeom &geo, const WideTables &tb, uint32_t slot, uint32_t *place_out,
                                     uint32_t *bucket_out) {
  const uint32_t b = geo.bucket_of(slot);
  const uint32_t n = load_agent(&tb.bucket_n[b]);
  const uint32_t lo = load_agent(&tb.bucket_lo[b]);
  const uint32_t j = ((slot - lo) >> geo.sub_shift) / (uint32_t)kWideIndexStep;
  if (j >= (uint32_t)kWideIndexLen) return kNone;
  const uint32_t w = load_agent(&tb.sub_index[(size_t)b * kWideIndexLen + j]);
  uint32_t p = w & 0xffffu, end = w >> 16;
  if (end > n) end = n;
  const uint32_t *idx = tb.slab_idx + (size_t)b * kWideCap;
  for (; p < end; p += 4) {
    uint32_t t[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) t[q] = load_agent(&idx[p + q < end ? p + q : p]) & kIndexMask;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (p + q >= end) return kNone;
      const uint32_t s1 = geo.mod_m(poly(t[q]) + kSeed1);
      if (s1 > slot) return kNone;
      if (s1 == slot) {
        *place_out = p + q;
        *bucket_out = b;
        return t[q];
      }
    }
  }
  return kNone;
}

template <typename S>
__global__ __launch_bounds__(kWideBlock) void k_wide_tail(SlabGeom geo, Probe g, WideTables tb,
                                                          const uint32_t *__restrict__ filter,
                                                          unsigned long long *cells, uint32_t log2, int64_t spp,
                                                          const S *__restrict__ dense, int32_t *__restrict__ out_idx,
                                                          S *__restrict__ out_val, uint32_t capacity,
                                                          int64_t *__restrict__ splits, uint32_t *clear,
                                                          uint32_t clear_words, int32_t *status) {
  __shared__ WideShared<S> sh;
  const uint32_t b = blockIdx.x, B = geo.nbuckets, bpp = geo.bpp;
  const uint32_t part = b / bpp;
  const uint32_t tid = threadIdx.x;
  // counters of the kernels before this one that nobody needs any more: back to zero, a slice per workgroup
  for (uint32_t i = b * kWideBlock + tid; i < clear_words; i += B * kWideBlock) clear[i] = 0;
  if (tid == 0) {
    sh.lo = geo.first_key(b);
    sh.lost_n = 0;
    sh.nrm = 0;
  }
  sh.cnt.clear();
  const WideParts parts = wide_parts(tb.cursor, b, tb.part_cap);
  uint32_t n_raw = parts.total();
  bool declined = false;
  if (n_raw > (uint32_t)kWideRaw) {  // more candidates than the workgroup looks at: another path answers
    declined = true;
    n_raw = 0;
  }
  const uint32_t thr_key = filter ? filter[0] : 0u;
  const size_t plane = (size_t)B * kWideSplit * tb.part_cap;
  const uint32_t *idx_plane = tb.words;
  const uint32_t *slot_plane = tb.words + plane;
  const S *val_plane = reinterpret_cast<const S *>(tb.words + 2 * plane);
  __syncthreads();
  const uint32_t lo = sh.lo;
  const int shift = geo.sub_shift;
  const uint32_t low_mask = (1u << shift) - 1u;

  // ---- the bucket's candidates: slot offsets in registers; loads in no branch, so that all are in flight
  uint32_t off[kWideItems];
#pragma unroll
  for (int i = 0; i < kWideItems; ++i) {
    const uint32_t j = tid + (uint32_t)i * kWideBlock;
    const size_t at = parts.place(j < n_raw ? j : 0u);
    const uint32_t slot = slot_plane[at];
    const S v = val_plane[at];
    const bool keep = j < n_raw && (v & KeyOf<S>::kMask) >= thr_key;
    off[i] = keep ? slot - lo : kInvalid;
  }
#pragma unroll
  for (int i = 0; i < kWideItems; ++i)
    if (off[i] != kInvalid) sh.cnt.count(off[i] >> shift);
  __syncthreads();
  uint32_t n;
  {
    // a narrow range that holds hundreds of records (keys piled on a few values) would keep the rank loop busy
    // for too long: declined as well
    const uint16_t *c16 = sh.cnt.cnt16();
    uint32_t big = 0;
#pragma unroll
    for (int e = 0; e < 16; ++e) big |= c16[tid * 16 + e] > (uint32_t)kWideGroupLimit;
    if (big) sh.lost_n = 1;  // any nonzero value: read back below, then put back to zero
    n = sh.cnt.starts(sh.scan);
  }
  __syncthreads();
  if (n > (uint32_t)kWideCap || sh.lost_n) {
    declined = true;
    __syncthreads();
    sh.cnt.clear();
    if (tid == 0) sh.lost_n = 0;
#pragma unroll
    for (int i = 0; i < kWideItems; ++i) off[i] = kInvalid;
    n = 0;
    __syncthreads();
  }
  if (declined && tid == 0) atomicOr(status, ZEN_STAT_RETRY);
#pragma unroll
  for (int i = 0; i < kWideItems; ++i) {
    if (off[i] != kInvalid) {
      const uint32_t p = sh.cnt.take(off[i] >> shift);
      sh.word[p] = ((off[i] & low_mask) << 15) | (tid + (uint32_t)i * kWideBlock);
    }
  }
  __syncthreads();
  // rank = records of the bucket with a smaller (slot, index): the records of the narrow ranges before it,
  // plus those of its own range with a smaller slot, plus (rare) those with its slot and a smaller index
  uint32_t rk[kWideItems];
  {
    const uint16_t *c16 = sh.cnt.cnt16();
#pragma unroll
    for (int i = 0; i < kWideItems; ++i) {
      rk[i] = kInvalid;
      if (off[i] != kInvalid) {
        const uint32_t sub = off[i] >> shift;
        const uint32_t g1 = c16[sub], g0 = c16[(int)sub - 1];
        const uint32_t j = tid + (uint32_t)i * kWideBlock;
        const uint32_t key = off[i] & low_mask;
        const uint32_t my = (key << 15) | j;
        uint32_t less = 0, twins = 0;
        for (uint32_t u = g0; u < g1; u += 4) {
          const uint32_t last = g1 - 1u;
          uint32_t a[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) a[q] = sh.word[u + q < last ? u + q : last];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (u + q < g1) {
              less += (a[q] >> 15) < key;
              twins += (a[q] >> 15) == key && a[q] != my;
            }
          }
        }
        uint32_t lost = 0;
        if (twins) {  // another candidate with this very slot: the smaller index comes first
          const uint32_t mine = idx_plane[parts.place(j)];
          for (uint32_t u = g0; u < g1; ++u) {
            const uint32_t w = sh.word[u];
            if ((w >> 15) == key && w != my) lost += idx_plane[parts.place(w & 0x7fffu)] < mine;
          }
        }
        rk[i] = (g0 + less + lost) | (lost ? kRemovedBit : 0u);
      }
    }
  }
  __syncthreads();
  // the narrow ranges' first places go to memory for the other workgroups' look-ups before the values take
  // the counters' place
  {
    const uint16_t *c16 = sh.cnt.cnt16();
    for (uint32_t j = tid; j < (uint32_t)kWideIndexLen; j += kWideBlock) {
      const uint32_t s0 = j * kWideIndexStep;
      store_agent(&tb.sub_index[(size_t)b * kWideIndexLen + j],
                  (uint32_t)c16[(int)s0 - 1] | ((uint32_t)c16[s0 + kWideIndexStep - 1] << 16));
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kWideItems; ++i) {
    const uint32_t j = tid + (uint32_t)i * kWideBlock;
    const size_t at = parts.place(rk[i] != kInvalid ? j : 0u);
    const uint32_t t = idx_plane[at];
    const S v = val_plane[at];
    if (rk[i] != kInvalid) {
      const uint32_t r = rk[i] & kIndexMask;
      sh.idx[r] = t | (rk[i] & kRemovedBit);
      sh.val[r] = v;
      if (rk[i] & kRemovedBit) {
        const uint32_t q = atomicAdd(&sh.lost_n, 1u);
        if (q < (uint32_t)kWideRemoved) sh.rm[q] = t;
      }
    }
  }
  __syncthreads();
  uint32_t lost_n = sh.lost_n;
  if (lost_n > (uint32_t)kWideRemoved) {
    if (tid == 0) atomicOr(status, ZEN_STAT_RETRY);
    lost_n = kWideRemoved;
  }
  if (tid == 0) {
    store_agent(&tb.bucket_n[b], n);
    store_agent(&tb.bucket_lo[b], lo);
    sh.base = lost_n ? atomicAdd(&tb.log_n[part * kWideCtrPad], lost_n) : 0u;
  }
  for (uint32_t p = tid; p < n; p += kWideBlock) store_agent(&tb.slab_idx[(size_t)b * kWideCap + p], sh.idx[p]);
  __syncthreads();
  for (uint32_t i = tid; i < lost_n; i += kWideBlock) {
    const uint32_t at = sh.base + i;
    if (at < tb.log_cap)
      store_agent(&tb.log_t[(size_t)part * tb.log_cap + at], sh.rm[i]);
    else
      atomicOr(status, ZEN_STAT_RETRY);
  }
  uint32_t *gbar = &tb.gbar[part * kWidePad];
  group_barrier(gbar, bpp, 1, status);

  // ---- levels 2 and 3 for the partition's losers
  const uint32_t lane_of_group = (b - part * bpp) * kWideBlock + tid, group_threads = bpp * kWideBlock;
  uint32_t losers = load_agent(&tb.log_n[part * kWideCtrPad]);
  if (losers > tb.log_cap) losers = tb.log_cap;
  for (uint32_t i = lane_of_group; i < losers; i += group_threads) {
    uint32_t cur = load_agent(&tb.log_t[(size_t)part * tb.log_cap + i]);
    int lv = 1;
    bool full = false;
    for (uint32_t steps = 0; lv < g.levels; ++steps) {
      if (steps > kChainLimit) {
        atomicOr(status, ZEN_STAT_INTERNAL);
        break;
      }
      uint32_t prt;
      const uint32_t slot = probe_slot(g, cur, lv, &prt);
      uint32_t head_place = 0, head_bucket = 0;
      const uint32_t head = wide_head(geo, tb, slot, &head_place, &head_bucket);
      if (head < cur) {  // a smaller index probes this slot at level 1: cur moves on
        ++lv;
        continue;
      }
      const uint32_t old = map_min(cells, log2, slot, cur, tb.ctr, &full);
      if (full) {
        atomicOr(status, ZEN_STAT_RETRY);
        break;
      }
      if (old < cur) {  // a smaller index got here at level 2 or 3
        ++lv;
        continue;
      }
      if (old == kNone) {
        // first level-2/3 prober of this slot: its level-1 owner (a larger index, if any) is pushed out
        if (head == kNone) break;
        const uint32_t at = atomicAdd(&tb.dl_n[head_bucket], 1u);
        if (at < (uint32_t)kWideRemoved)
          store_agent(&tb.dl_pos[(size_t)head_bucket * kWideRemoved + at], head_place);
        else
          atomicOr(status, ZEN_STAT_RETRY);
        const uint32_t at2 = atomicAdd(&tb.dlog_n[part * kWideCtrPad], 1u);
        if (at2 < tb.log_cap)
          store_agent(&tb.dlog_t[(size_t)part * tb.log_cap + at2], head);
        else
          atomicOr(status, ZEN_STAT_RETRY);
        cur = head;
        lv = 1;
        continue;
      }
      if (old == cur) break;
      // took the slot from a larger index that held it at its first level mapping here
      int lw = 1;
      while (lw < g.levels && probe_slot(g, old, lw, &prt) != slot) ++lw;
      cur = old;
      lv = lw + 1;
    }
  }
  group_barrier(gbar, bpp, 2, status);

  // ---- final place of every logged entry: the level-2/3 slot it holds in the map, or the serial list
  {
    uint32_t pushed = load_agent(&tb.dlog_n[part * kWideCtrPad]);
    if (pushed > tb.log_cap) pushed = tb.log_cap;
    for (uint32_t i = lane_of_group; i < losers + pushed; i += group_threads) {
      const bool first = i < losers;
      const size_t at_log = (size_t)part * tb.log_cap + (first ? i : i - losers);
      const uint32_t t = load_agent(first ? &tb.log_t[at_log] : &tb.dlog_t[at_log]);
      uint32_t prt = 0, cell = kNone, slot = kNone;
      for (int lv = 1; lv < g.levels && slot == kNone; ++lv) {
        const uint32_t s = probe_slot(g, t, lv, &prt);
        uint32_t at = 0;
        if (map_find_fresh(cells, log2, s, &at) == t) {
          slot = s;
          cell = at;
        }
      }
      store_agent(first ? &tb.log_cell[at_log] : &tb.dlog_cell[at_log], cell);
      if (slot != kNone) {
        const uint32_t b2 = geo.bucket_of(slot);
        const uint32_t at = atomicAdd(&tb.movein_n[b2], 1u);
        if (at < (uint32_t)kWideMove) {
          store_agent(&tb.mv_slot[(size_t)b2 * kWideMove + at], slot);
          store_agent(&tb.mv_idx[(size_t)b2 * kWideMove + at], t);
        } else {
          atomicOr(status, ZEN_STAT_RETRY);
        }
      } else {
        const uint32_t at = atomicAdd(&tb.serial_n[part * kWideCtrPad], 1u);
        if (at < (uint32_t)kSlabSerialCap)
          store_agent(&tb.ser_idx[(size_t)part * kSlabSerialCap + at], t);
        else  // more than the partition's serial region holds is an overflow; more than this path carries, a retry
          atomicOr(status, (int64_t)at >= spp ? ZEN_STAT_SERIAL_OVERFLOW : ZEN_STAT_RETRY);
      }
    }
  }
  group_barrier(gbar, bpp, 3, status);

  // ---- place: the sorted bucket is almost its part of the output already
  uint32_t pushed_n = load_agent(&tb.dl_n[b]);
  if (pushed_n > (uint32_t)kWideRemoved) pushed_n = kWideRemoved;
  if (tid < pushed_n) {
    const uint32_t p = load_agent(&tb.dl_pos[(size_t)b * kWideRemoved + tid]);
    if (p < n) sh.idx[p] |= kRemovedBit;  // places are distinct: a slot's owner is pushed out once
  }
  uint32_t mv_n = load_agent(&tb.movein_n[b]);
  if (mv_n > (uint32_t)kWideMove) mv_n = kWideMove;
  if (tid < mv_n) {
    sh.mk[tid] = load_agent(&tb.mv_slot[(size_t)b * kWideMove + tid]);
    sh.mi[tid] = load_agent(&tb.mv_idx[(size_t)b * kWideMove + tid]);
  }
  __syncthreads();
  for (uint32_t p = tid; p < n; p += kWideBlock) {
    if (sh.idx[p] & kRemovedBit) {
      const uint32_t at = atomicAdd(&sh.nrm, 1u);
      if (at < (uint32_t)kWideRemoved) sh.rm[at] = p;
    }
  }
  __syncthreads();
  uint32_t rm_n = sh.nrm;
  if (rm_n > (uint32_t)kWideRemoved) {  // more collisions than this path carries
    if (tid == 0) atomicOr(status, ZEN_STAT_RETRY);
    rm_n = kWideRemoved;
  }
  {
    // the removed places in ascending order; moved-in entry j: its slot's rank among the moved-in slots (they
    // are distinct: a slot has one owner) and the sorted place in front of which it slips in
    uint32_t x = 0, xr = 0;
    if (tid < rm_n) {
      x = sh.rm[tid];
      for (uint32_t u = 0; u < rm_n; ++u) xr += sh.rm[u] < x;
    }
    uint32_t mj = 0, mplace = 0;
    if (tid < mv_n) {
      const uint32_t k = sh.mk[tid];
      for (uint32_t u = 0; u < mv_n; ++u) mj += sh.mk[u] < k;
      const uint32_t j = ((k - lo) >> shift) / (uint32_t)kWideIndexStep;
      const uint32_t w = j < (uint32_t)kWideIndexLen ? load_agent(&tb.sub_index[(size_t)b * kWideIndexLen + j]) : n | (n << 16);
      uint32_t p = w & 0xffffu, end = w >> 16;
      if (end > n) end = n;
      mplace = p;
      for (; p < end; ++p) mplace += geo.mod_m(poly(sh.idx[p] & kIndexMask) + kSeed1) < k;
    }
    __syncthreads();
    if (tid < rm_n) sh.rm[xr] = x;
    if (tid < mv_n) sh.mp[mj] = mplace;
    __syncthreads();
    // what the bucket contributes, and where it starts: the sum of what the earlier buckets publish (every
    // workgroup of the launch is resident; the wait is bounded all the same)
    const bool last_of_part = b % bpp == bpp - 1;
    uint32_t serial = 0, serial_raw = 0;
    if (last_of_part) {
      serial_raw = load_agent(&tb.serial_n[part * kWideCtrPad]);
      serial = serial_raw > (uint32_t)kSlabSerialCap ? (uint32_t)kSlabSerialCap : serial_raw;
    }
    const uint32_t own_n = n - rm_n + mv_n;  // survivors + moved-in
    if (tid == 0) desc_store(&tb.desc[b], kDescAggregate | (uint64_t)(own_n + serial));
    uint64_t before = 0;  // low half: entries of all earlier buckets; high half: of the partition's earlier buckets
    if (tid < b) {
      uint64_t d = desc_load(&tb.desc[tid]);
      uint32_t spins = 0;
      while ((d >> 62) == 0) {
        if (++spins > kSpinLimit) {
          atomicOr(status, ZEN_STAT_INTERNAL);
          break;
        }
        __builtin_amdgcn_s_sleep(2);
        d = desc_load(&tb.desc[tid]);
      }
      const uint64_t v = d & 0xffffffffull;
      before = v | (tid >= part * bpp ? v << 32 : 0ull);
    }
    uint64_t sums;
    block_exclusive_scan<uint64_t, kWideBlock>(before, sh.scan64, &sums);
    const uint32_t out_base = (uint32_t)sums, in_part = (uint32_t)(sums >> 32);
    // Most stretches of 64 consecutive sorted places contain neither a removed entry nor the place where a
    // moved-in entry slips in: all their entries move by the same amount, found once per stretch.
    constexpr int32_t kNoDelta = INT32_MIN;
    for (uint32_t c = tid; c * 64u < n; c += kWideBlock) {
      const uint32_t p0 = c * 64u, p1 = p0 + 63u < n ? p0 + 63u : n - 1u;
      uint32_t mv0 = 0, mv1 = 0, r0 = 0, r1 = 0;
      if (mv_n) {
        mv0 = upper_bound_u32(sh.mp, mv_n, p0);
        mv1 = upper_bound_u32(sh.mp, mv_n, p1);
      }
      if (rm_n) {
        r0 = lower_bound_u32(sh.rm, rm_n, p0);
        r1 = lower_bound_u32(sh.rm, rm_n, p1);
      }
      sh.delta[c] = (mv0 == mv1 && r0 == r1) ? (int32_t)(mv0 - r0) : kNoDelta;
    }
    __syncthreads();
    for (uint32_t p = tid; p < n; p += kWideBlock) {
      const uint32_t t = sh.idx[p];
      if (!(t & kRemovedBit)) {
        int32_t delta = sh.delta[p >> 6];
        if (delta == kNoDelta)
          delta = (int32_t)((mv_n ? upper_bound_u32(sh.mp, mv_n, p) : 0u) - (rm_n ? lower_bound_u32(sh.rm, rm_n, p) : 0u));
        const uint32_t pos = out_base + p + (uint32_t)delta;
        if (pos < capacity) {
          out_idx[pos] = (int32_t)t;
          out_val[pos] = sh.val[p];
        }
      }
    }
    if (tid < mv_n) {
      const uint32_t pos = out_base + mplace + mj - (rm_n ? lower_bound_u32(sh.rm, rm_n, mplace) : 0u);
      if (pos < capacity) {
        const uint32_t t = sh.mi[tid];
        out_idx[pos] = (int32_t)t;
        out_val[pos] = dense[t];  // an entry is a copy of the element it stands for
      }
    }
    if (serial) {
      // the partition's overflow entries in ascending index order (the reference hands its tickets to
      // ascending thread ids, functions_cuda_kernel.cu:107-108), behind everything that found a slot
      __syncthreads();
      for (uint32_t i = tid; i < serial; i += kWideBlock)
        sh.word[i] = load_agent(&tb.ser_idx[(size_t)part * kSlabSerialCap + i]);
      __syncthreads();
      sort_network(sh.word, serial);
      for (uint32_t i = tid; i < serial; i += kWideBlock) {
        const uint32_t pos = out_base + own_n + i;
        if (pos < capacity) {
          out_idx[pos] = (int32_t)sh.word[i];
          out_val[pos] = dense[sh.word[i]];
        }
      }
    }
    if (last_of_part && tid == 0) {
      splits[part] = (int64_t)(in_part + own_n + serial);
      if ((int64_t)serial_raw > spp) atomicOr(status, ZEN_STAT_SERIAL_OVERFLOW);
      if (out_base + own_n + serial > capacity) atomicOr(status, ZEN_STAT_CAPACITY);
    }
  }

  // ---- the workgroup that finishes last leaves the borrowed memory as it was: the map's cells and every
  // counter back at zero
  wait_global_acks();
  __syncthreads();
  if (tid == 0) sh.flag = atomicAdd(tb.done, 1u) == B - 1u;
  __syncthreads();
  if (!sh.flag) return;
  const uint32_t P = (uint32_t)tb.partitions;
  for (uint32_t q = 0; q < P; ++q) {
    uint32_t nl = load_agent(&tb.log_n[q * kWideCtrPad]), nd = load_agent(&tb.dlog_n[q * kWideCtrPad]);
    if (nl > tb.log_cap) nl = tb.log_cap;
    if (nd > tb.log_cap) nd = tb.log_cap;
    // every occupied cell ends with the index that finally holds its slot, and that index recorded the cell
    for (uint32_t i = tid; i < nl + nd; i += kWideBlock) {
      const size_t at = (size_t)q * tb.log_cap + (i < nl ? i : i - nl);
      const uint32_t cell = load_agent(i < nl ? &tb.log_cell[at] : &tb.dlog_cell[at]);
      if (cell != kNone) cells[cell] = 0ull;
    }
  }
  __syncthreads();
  for (uint32_t i = tid; i < B * kWideSplit; i += kWideBlock) tb.cursor[i * kWidePad] = 0;
  for (uint32_t i = tid; i < P; i += kWideBlock) {
    tb.gbar[i * kWidePad] = 0;
    tb.log_n[i * kWideCtrPad] = 0;
    tb.dlog_n[i * kWideCtrPad] = 0;
    tb.serial_n[i * kWideCtrPad] = 0;
  }
  for (uint32_t i = tid; i < B; i += kWideBlock) {
    tb.movein_n[i] = 0;
    tb.dl_n[i] = 0;
    tb.desc[i] = 0ull;
  }
  if (tid == 0) {
    *tb.done = 0;
    tb.ctr->logged = tb.ctr->losers = tb.ctr->claims = tb.ctr->displaced = 0;
  }
}

struct WidePlan {
  WideTables tb;
  uint32_t *sample_hist[2];  // the layout of these four must be the one plan_slab uses: a sample taken ahead
  uint32_t *cand_hist;       // (zen_load_balance_prepare) is found by whichever path the call takes
  uint32_t *ticket;
  uint32_t *refine_hist;
  uint32_t *thr;
  CoarseGeom cg;
  size_t state_bytes, bytes;
};

WidePlan plan_wide(void *workspace, void *state, const SlabGeom &geo, int partitions, int dtype, int64_t list_cap) {
  WidePlan p;
  const size_t B = geo.nbuckets, P = (size_t)partitions;
  {
    Carver cv(state);
    p.sample_hist[0] = cv.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
    p.sample_hist[1] = cv.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
    p.cand_hist = cv.take<uint32_t>((size_t)kCandHistWords);
    p.ticket = cv.take<uint32_t>(select_stage_ticket_words());
    p.tb.cursor = cv.take<uint32_t>(B * kWideSplit * kWidePad);
    p.tb.gbar = cv.take<uint32_t>(P * kWidePad);
    p.tb.log_n = cv.take<uint32_t>(P * kWideCtrPad);
    p.tb.dlog_n = cv.take<uint32_t>(P * kWideCtrPad);
    p.tb.serial_n = cv.take<uint32_t>(P * kWideCtrPad);
    p.tb.movein_n = cv.take<uint32_t>(B);
    p.tb.dl_n = cv.take<uint32_t>(B);
    p.tb.desc = cv.take<unsigned long long>(B);
    p.tb.done = cv.take<uint32_t>(1);
    p.tb.ctr = cv.take<Counters>(1);
    p.refine_hist = cv.take<uint32_t>(dtype == ZEN_BF16 ? 1 : (size_t)kRefineBins + 1);
    p.state_bytes = cv.used;
  }
  Carver cv(workspace);
  p.thr = cv.take<uint32_t>(16);
  p.tb.part_cap = wide_part_cap(geo, list_cap);
  p.cg.groups = geo.nbuckets;
  p.cg.per = 1;
  p.cg.cap = p.tb.part_cap;
  p.cg.inv_per = slab_inverse_below(1);
  p.tb.words = cv.take<uint32_t>((size_t)3 * B * kWideSplit * p.tb.part_cap);
  p.tb.slab_idx = cv.take<uint32_t>(B * kWideCap);
  p.tb.sub_index = cv.take<uint32_t>(B * kWideIndexLen);
  p.tb.bucket_n = cv.take<uint32_t>(B);
  p.tb.bucket_lo = cv.take<uint32_t>(B);
  p.tb.log_cap = (uint32_t)(list_cap / 4 / (int64_t)P + 1024);
  p.tb.log_t = cv.take<uint32_t>(P * p.tb.log_cap);
  p.tb.log_cell = cv.take<uint32_t>(P * p.tb.log_cap);
  p.tb.dlog_t = cv.take<uint32_t>(P * p.tb.log_cap);
  p.tb.dlog_cell = cv.take<uint32_t>(P * p.tb.log_cap);
  p.tb.mv_slot = cv.take<uint32_t>(B * kWideMove);
  p.tb.mv_idx = cv.take<uint32_t>(B * kWideMove);
  p.tb.dl_pos = cv.take<uint32_t>(B * kWideRemoved);
  p.tb.ser_idx = cv.take<uint32_t>(P * kSlabSerialCap);
  p.tb.partitions = partitions;
  p.bytes = cv.used;
  return p;
}

int64_t wide_expected(int64_t capacity, int64_t k) { return k > 0 ? k + k / 32 + 1024 : capacity; }

}  // namespace

bool wide_balance_fits(int64_t m, int partitions, int64_t capacity, int64_t k, int cus, SlabGeom *geo) {
  if (capacity > 0x1fffffffll || cus <= 0) return false;
  SlabGeom g;
  if (!wide_geometry(m, partitions, wide_expected(capacity, k), cus, &g)) return false;
  if (geo) *geo = g;
  return true;
}

// Whatever k a call comes with: the layout only depends on the table and the partitions.
size_t wide_balance_bytes(int64_t m, int partitions, int dtype, int64_t capacity, int cus) {
  SlabGeom geo;
  if (capacity > 0x1fffffffll || cus <= 0 || !wide_geometry(m, partitions, 1, cus, &geo)) return 0;
  return plan_wide(nullptr, nullptr, geo, partitions, dtype, list_capacity(capacity)).bytes;
}

int wide_load_balance(const SlabBalanceArgs &a, size_t state_offset, hipStream_t s) {
  SlabGeom geo;
  if (!wide_balance_fits(a.g.m, a.partitions, a.capacity, a.k, wide_device_cus(), &geo))
    return fail(ZEN_EINVAL, "wide_load_balance: sizes do not suit the wide buckets");
  char *state = reinterpret_cast<char *>(a.hash) + state_offset;
  WidePlan p = plan_wide(a.workspace, state, geo, a.partitions, a.dtype, list_capacity(a.capacity));
  if (state_offset + p.state_bytes > (size_t)a.g.m * sizeof(int32_t))
    return fail(ZEN_EINVAL, "wide_load_balance: table too small for the counters");
  const bool refine = a.k > 0 && a.dtype == ZEN_F32;
  StageArgs sc;
  sc.in = a.input;
  sc.dtype = a.dtype;
  sc.n = a.n;
  sc.thr = a.thr;
  sc.geo = geo;
  sc.cg = p.cg;
  sc.wide = true;
  sc.coarse_cursor = p.tb.cursor;
  sc.coarse_words = p.tb.words;
  sc.ticket = p.ticket;
  sc.status = a.status;
  int rc;
  const int set = a.prepared == 2 ? 1 : 0;
  uint32_t *floor = p.thr + 2 + 4 * set;
  if (a.k > 0) {
    if (a.near_key) {
      sc.thr = a.near_key;
      sc.floor_margin = a.dtype == ZEN_BF16 ? 4u : 4u << 16;
    } else {
      if (!a.prepared &&
          (rc = topk_sampled_floor(a.input, a.dtype, a.n, a.k, floor, p.sample_hist[set], s, true)) != ZEN_OK)
        return rc;
      sc.thr = floor;
    }
    sc.cand_hist = p.cand_hist;
    sc.pick_k = a.k;
    sc.pick_thr = p.thr;
    sc.pick_above = p.thr + 4;
    sc.thr_copy = refine ? nullptr : a.thr_out;
    sc.clear = p.sample_hist[set];
    sc.clear_words = (uint32_t)(sampled_floor_zero_bytes() / sizeof(uint32_t));
  }
  if ((rc = select_stage_slabs(sc, s)) != ZEN_OK) return rc;
  uint32_t *clear = p.cand_hist;  // the candidates' histogram and the select kernel's tickets lie side by side
  uint32_t clear_words = (uint32_t)(reinterpret_cast<char *>(p.tb.cursor) - reinterpret_cast<char *>(p.cand_hist)) / 4u;
  if (refine) {
    const uint32_t refine_parts = p.cg.groups * (uint32_t)kCoarseSplit;
    k_refine_threshold<<<dim3(refine_parts < 128u ? refine_parts : 128u), dim3(kRefineBlock), 0, s>>>(
        p.cg, 2, p.tb.cursor, p.tb.words, static_cast<const uint32_t *>(a.input), p.thr, p.thr + 4, (uint32_t)a.k,
        p.refine_hist, a.thr_out, a.status);
    ZEN_LAUNCH_CHECK("k_refine_threshold");
  }
  const uint32_t *filter = a.k > 0 ? p.thr : nullptr;
  if ((rc = wide_line_enter(s)) != ZEN_OK) return rc;
  {
    ProfScope prof(kProfWideTail, s);
    if (a.dtype == ZEN_BF16)
      k_wide_tail<uint16_t><<<dim3(geo.nbuckets), dim3(kWideBlock), 0, s>>>(
          geo, a.g, p.tb, filter, a.hash, a.hash_log2, a.spp, static_cast<const uint16_t *>(a.input), a.out_idx,
          static_cast<uint16_t *>(a.out_val), (uint32_t)a.capacity, a.splits, clear, clear_words, a.status);
    else
      k_wide_tail<uint32_t><<<dim3(geo.nbuckets), dim3(kWideBlock), 0, s>>>(
          geo, a.g, p.tb, filter, a.hash, a.hash_log2, a.spp, static_cast<const uint32_t *>(a.input), a.out_idx,
          static_cast<uint32_t *>(a.out_val), (uint32_t)a.capacity, a.splits, clear, clear_words, a.status);
    ZEN_LAUNCH_CHECK("k_wide_tail");
  }
  if (refine) {
    // the refinement histogram is the tail kernel's to clear on the other path; here a fill does it
    launch_fill<uint32_t>(p.refine_hist, 0u, (size_t)kRefineBins + 1, s);
    ZEN_LAUNCH_CHECK("wide: clear the refinement histogram");
  }
  return wide_line_leave(s);
}

}  // namespace zen
