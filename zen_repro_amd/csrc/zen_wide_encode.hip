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

constexpr int kWideRounds = 3;                          // a part of a bucket's slab is read in rounds of kWideBlock records
constexpr int kWideItems = kWideSplit * kWideRounds;    // raw records per thread (candidates below the threshold included)
constexpr int kWidePartMax = kWideBlock * kWideRounds;  // raw records of one part, at most
constexpr int kWideMove = 1024;                         // entries that may move into one bucket from elsewhere
constexpr int kWideRemoved = 1024;                      // entries of a bucket that may lose their level-1 slot
constexpr int kWideQueue = (2 * kWideMove + kWideMove + kWideRemoved) / 2;  // records set aside while ranking
constexpr int kWideLanes = 4;                           // records a thread handles per step of the ranking loops
constexpr int kWideGroupLimit = 512;                    // records in one narrow range: bounds the rank loop
constexpr int kWideIndexStep = 4;                       // every 4th narrow range has its first sorted place written down
constexpr int kWideIndexLen = kWideSubs / kWideIndexStep;
constexpr int kWideCtrPad = 8;                          // words between two per-partition counters
constexpr int kWideSteps = kWideSplit * kWideRounds / 4;  // = kWideItems / kWideLanes
constexpr int kWideProbeLimit = 512;                    // probes in the map before it counts as full
constexpr uint32_t kInvalid = 0xffffffffu;
// a record's raw place: part * 4096 + place inside the part
static_assert(kWidePartMax <= 4096 && kWideSplit * 4096 <= (1 << 15), "raw places in 15 bits");
static_assert(kWideMove <= kWideBlock && kWideRemoved <= kWideBlock, "one entry per thread");
static_assert(kWideSplit % 4 == 0, "steps of four records");
static_assert(kWideMove < (1 << 12) && kWideRemoved < (1 << 12), "two counts in one word");

struct WideTables {
  // zero between calls (kept in the caller's zero table, behind the hash map)
  uint32_t *cursor;            // [B * kWideSplit * kWidePad] part cursors
  uint32_t *gbar;              // [P * kWidePad] barrier counters of the partitions' workgroups
  uint32_t *pdone;             // [P * kWidePad] workgroups of the partition that have finished
  uint32_t *log_n;             // [P * kWideCtrPad] entries that lost level 1, per partition
  uint32_t *dlog_n;            // [P * kWideCtrPad] level-1 owners pushed out by a level-2/3 prober, per partition
  unsigned long long *desc;    // [B] what every bucket contributes to the output (flag + count)
  uint32_t *done;              // [1] workgroups that have finished
  Counters *ctr;               // [P] (the claims of the partition's map)
  // workspace
  uint32_t *words;             // [B * kWideSplit * part_cap] raw candidates, two words each: index, value bits
  uint32_t *slab_idx;          // [B * kWideCap] sorted indices (| kRemovedBit: lost level 1)
  uint32_t *sub_index;         // [B * kWideIndexLen] first sorted place of narrow range 4 j, and of 4 j + 4 in the high half
  uint32_t *log_t, *log_cell;  // [P * log_cap] losers; the map cell each ends in (kNone: none)
  uint32_t *dlog_t, *dlog_cell, *dlog_at;  // the same for the owners pushed out, and bucket << 16 | sorted place of each
  uint32_t *ser_idx;           // [P * kSlabSerialCap]
  uint32_t part_cap;
  uint32_t log_cap;            // per partition
  uint32_t map_log2;           // cells of one partition's map
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
  union {
    struct {
      uint32_t mk[kWideMove];     // slots of the moved-in entries
      uint32_t mi[kWideMove];     // their indices
      uint32_t mp[kWideMove];     // sorted place in front of which each slips in, by ascending slot
      uint32_t rm[kWideRemoved];  // losers' indices while they are logged, then the sorted places of the removed entries
    };
    struct {                      // while ranking: the records set aside
      uint32_t q_word[kWideQueue];   // the record's word, then its rank (| kRemovedBit)
      uint32_t q_range[kWideQueue];  // where its narrow range starts | where it ends << 16
    };
  };
  int32_t delta[kWideCap / 64];
  uint32_t scan[kWideBlock / 64 + 1];
  uint64_t scan64[kWideBlock / 64 + 1];
  uint32_t lo, lost_n, nrm, mv_n, ser_n, base, flag, big;
};

__device__ inline unsigned long long cell_fresh(const unsigned long long *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// map_min (zen_hashmap.h) with one trip to memory where the slot is met for the first time: the cell is
// claimed with a compare-and-swap straight away, and the count of claims is raised without waiting for it (a
// map that fills up shows in the length of the probe sequences instead).
__device__ inline uint32_t map_min_claim(unsigned long long *cells, uint32_t log2, uint32_t slot, uint32_t t,
                                         Counters *ctr, bool *full) {
  const uint32_t mask = (1u << log2) - 1u;
  const unsigned long long mine = ((unsigned long long)(slot + 1u) << 32) | t;
  uint32_t h = cell_home(slot, log2);
  for (uint32_t probes = 0; probes <= mask && probes < (uint32_t)kWideProbeLimit; ++probes, h = (h + 1u) & mask) {
    const unsigned long long cur = atomicCAS(&cells[h], 0ull, mine);
    if (cur == 0ull) {
      atomicAdd(&ctr->claims, 1u);
      return kNone;
    }
    if ((uint32_t)(cur >> 32) == slot + 1u) return (uint32_t)atomicMin(&cells[h], mine);
  }
  *full = true;
  return 0u;  // pretend a smaller index owns it: the chain moves on and the call is retried anyway
}

// map_find while other workgroups of the running kernel have been writing the map.
__device__ inline uint32_t map_find_fresh(const unsigned long long *cells, uint32_t log2, uint32_t slot, uint32_t *cell_out) {
  const uint32_t mask = (1u << log2) - 1u;
  uint32_t h = cell_home(slot, log2);
  for (uint32_t probes = 0; probes <= mask && probes < (uint32_t)kWideProbeLimit; ++probes, h = (h + 1u) & mask) {
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
  const uint32_t j = ((slot - geo.first_key(b)) >> geo.sub_shift) / (uint32_t)kWideIndexStep;
  if (j >= (uint32_t)kWideIndexLen) return kNone;
  const uint32_t w = load_agent(&tb.sub_index[(size_t)b * kWideIndexLen + j]);
  uint32_t p = w & 0xffffu;
  const uint32_t end = w >> 16;
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

#ifdef ZEN_WIDE_TIMING
__device__ unsigned long long g_wide_dbg[256 * 32];
#define WIDE_MARK(k) do { if (threadIdx.x == 0) g_wide_dbg[blockIdx.x * 32 + (k)] = wall_clock64(); } while (0)
#else
#define WIDE_MARK(k) do { } while (0)
#endif

template <typename S>
__global__ __launch_bounds__(kWideBlock) void k_wide_tail(SlabGeom geo, Probe g, WideTables tb,
                                                          const uint32_t *__restrict__ filter,
                                                          unsigned long long *cells, int64_t spp,
                                                          const S *__restrict__ dense, int32_t *__restrict__ out_idx,
                                                          S *__restrict__ out_val, uint32_t capacity,
                                                          int64_t *__restrict__ splits, uint32_t *clear,
                                                          uint32_t clear_words, uint32_t *clear_too,
                                                          uint32_t clear_too_words, int32_t *status) {
  __shared__ WideShared<S> sh;
  const uint32_t b = blockIdx.x, B = geo.nbuckets, bpp = geo.bpp;
  const uint32_t part = b / bpp;
  const uint32_t tid = threadIdx.x;
  WIDE_MARK(0);
  // counters of the kernels before this one that nobody needs any more: back to zero, a slice per workgroup
  for (uint32_t i = b * kWideBlock + tid; i < clear_words; i += B * kWideBlock) clear[i] = 0;
  for (uint32_t i = b * kWideBlock + tid; i < clear_too_words; i += B * kWideBlock) clear_too[i] = 0;  // fp32: the refinement's histogram
  if (tid == 0) {
    sh.lo = geo.first_key(b);
    sh.lost_n = sh.nrm = sh.mv_n = sh.ser_n = sh.big = 0;
  }
  sh.cnt.clear();
  // the bucket's candidates sit in kWideSplit parts; item r * kWideSplit + q of a thread is the record at
  // place tid + r * kWideBlock of part q
  uint32_t pcount[kWideSplit];
  uint32_t longest = 0;
#pragma unroll
  for (int q = 0; q < kWideSplit; ++q) {
    pcount[q] = tb.cursor[(b * kWideSplit + q) * kWidePad];
    if (pcount[q] > tb.part_cap) pcount[q] = tb.part_cap;  // the producer flagged the overflow
    longest = pcount[q] > longest ? pcount[q] : longest;
  }
  bool declined = false;
  if (longest > (uint32_t)kWidePartMax) {  // more candidates than the workgroup looks at: another path answers
    declined = true;
#pragma unroll
    for (int q = 0; q < kWideSplit; ++q) pcount[q] = 0;
    longest = 0;
  }
  const uint32_t thr_key = filter ? filter[0] : 0u;
  // the bucket's records: (index, value bits), kWideSplit parts of part_cap records
  const uint2 *records = reinterpret_cast<const uint2 *>(tb.words) + (size_t)b * kWideSplit * tb.part_cap;
  __syncthreads();
  const uint32_t lo = sh.lo;
  const int shift = geo.sub_shift;
  const uint32_t low_mask = (1u << shift) - 1u;

  // ---- slot offsets in registers; loads in no branch (places past a part's end are pulled back onto its
  // first record), so that all are in flight together
  uint32_t off[kWideItems];
#pragma unroll
  for (int r = 0; r < kWideRounds; ++r) {
#pragma unroll
    for (int q = 0; q < kWideSplit; ++q) off[r * kWideSplit + q] = kInvalid;
    if ((uint32_t)r * kWideBlock < longest) {
#pragma unroll
      for (int q = 0; q < kWideSplit; ++q) {
        const uint32_t e = tid + (uint32_t)r * kWideBlock;
        const size_t at = (size_t)q * tb.part_cap + (e < pcount[q] ? e : 0u);
        const uint2 rec = records[at];
        const uint32_t slot = geo.mod_m(poly(rec.x) + kSeed1);  // the level-1 slot: a dozen instructions, not a plane of its own
        const bool keep = e < pcount[q] && (rec.y & KeyOf<S>::kMask) >= thr_key;
        off[r * kWideSplit + q] = keep ? slot - lo : kInvalid;
      }
    }
  }
  WIDE_MARK(1);
#pragma unroll
  for (int i = 0; i < kWideItems; ++i)
    if (off[i] != kInvalid) sh.cnt.count(off[i] >> shift);
  __syncthreads();
  // a narrow range that holds hundreds of records (keys piled on a few values) would keep the rank loop busy
  // for too long: declined as well
  uint32_t n = sh.cnt.starts(sh.scan, (uint32_t)kWideGroupLimit, &sh.big);
  __syncthreads();
  if (n > (uint32_t)kWideCap || sh.big) {
    declined = true;
    __syncthreads();
    sh.cnt.clear();
#pragma unroll
    for (int i = 0; i < kWideItems; ++i) off[i] = kInvalid;
    n = 0;
    __syncthreads();
  }
  if (declined && tid == 0) atomicOr(status, ZEN_STAT_RETRY);
  // From here on a thread's records are worked through in kWideSteps steps of kWideLanes records, by a loop
  // whose body always handles the first kWideLanes registers of the set and then rotates the set: with the
  // body written out for all records the kernel's code no longer fits the instruction cache, and every
  // workgroup runs it just once.
  auto rotate = [](uint32_t (&a)[kWideItems]) {
    uint32_t head[kWideLanes];
#pragma unroll
    for (int k = 0; k < kWideLanes; ++k) head[k] = a[k];
#pragma unroll
    for (int i = 0; i + kWideLanes < kWideItems; ++i) a[i] = a[i + kWideLanes];
#pragma unroll
    for (int k = 0; k < kWideLanes; ++k) a[kWideItems - kWideLanes + k] = head[k];
  };
  // raw place of the record in lane k of step s: part * 4096 + place inside the part
  auto raw_place = [&](int s, int k) {
    constexpr int kPer = kWideSplit / kWideLanes;  // steps per round
    return (uint32_t)((s % kPer) * kWideLanes + k) * 4096u + tid + (uint32_t)(s / kPer) * kWideBlock;
  };
  // steps of rounds that no part of the slab reaches hold nothing: the loops stop short of them
  const int steps = longest == 0 ? 0 : (int)((longest + kWideBlock - 1) / kWideBlock) * (kWideSplit / kWideLanes);
#pragma unroll 1
  for (int s = 0; s < kWideSteps; ++s) {
    if (s < steps) {
#pragma unroll
      for (int k = 0; k < kWideLanes; ++k) {
        if (off[k] != kInvalid) {
          const uint32_t p = sh.cnt.take(off[k] >> shift);
          sh.word[p] = ((off[k] & low_mask) << 15) | raw_place(s, k);
        }
      }
    }
    rotate(off);
  }
  __syncthreads();
  WIDE_MARK(2);
  // rank = records of the bucket with a smaller (slot, index): the records of the narrow ranges before it,
  // plus those of its own range with a smaller slot, plus (rare) those with its slot and a smaller index.
  // A round's eight records at a time: first where every record's range starts and ends, then the range's
  // first three words of each (most ranges hold no more), all in flight together.
  uint32_t rk[kWideItems];
  auto raw_at = [&](uint32_t j) { return (size_t)(j >> 12) * tb.part_cap + (j & 4095u); };
#pragma unroll
  for (int i = 0; i < kWideItems; ++i) rk[i] = kInvalid;
#pragma unroll 1
  for (int s = 0; s < kWideSteps; ++s) {
    constexpr int kAhead = 4;
    uint32_t out[kWideLanes];
#pragma unroll
    for (int k = 0; k < kWideLanes; ++k) out[k] = kInvalid;
    if (s < steps) {
    uint32_t g0[kWideLanes], g1[kWideLanes], a[kWideLanes][kAhead];
#pragma unroll
    for (int k = 0; k < kWideLanes; ++k) {
      const uint32_t sub = off[k] != kInvalid ? off[k] >> shift : 0u;
      g0[k] = sh.cnt.start_of(sub);
      g1[k] = sh.cnt.end_of(sub);
    }
#pragma unroll
    for (int k = 0; k < kWideLanes; ++k) {
      const uint32_t last = g1[k] > g0[k] ? g1[k] - 1u : g0[k];
#pragma unroll
      for (int e = 0; e < kAhead; ++e) a[k][e] = sh.word[g0[k] + e < last ? g0[k] + e : last];
    }
#pragma unroll
    for (int k = 0; k < kWideLanes; ++k) {
      if (off[k] != kInvalid) {
        const uint32_t key = off[k] & low_mask;
        const uint32_t my = (key << 15) | raw_place(s, k);
        uint32_t less = 0, twins = 0;
#pragma unroll
        for (int e = 0; e < kAhead; ++e) {
          if (g0[k] + e < g1[k]) {
            less += (a[k][e] >> 15) < key;
            twins += (a[k][e] >> 15) == key && a[k][e] != my;
          }
        }
        uint32_t x = g0[k] + less;
        if (twins || g1[k] - g0[k] > (uint32_t)kAhead) {
          // A range of more than kAhead records, or another candidate with this very slot (the smaller
          // index then comes first, and comparing indices takes trips to memory): a wave would wait for
          // every lane that has one of these, at every record.  They are set aside and settled afterwards,
          // one per thread.
          const uint32_t at = atomicAdd(&sh.lost_n, 1u);
          if (at < (uint32_t)kWideQueue) {
            sh.q_word[at] = my;
            sh.q_range[at] = g0[k] | (g1[k] << 16);
            x = kRemovedBit | at;  // pending: place in the queue
          }
        }
        out[k] = x;
      }
    }
    }
    rotate(off);
    rotate(rk);  // the step's ranks enter at the end: after the last step rank i belongs to record i
#pragma unroll
    for (int k = 0; k < kWideLanes; ++k) rk[kWideItems - kWideLanes + k] = out[k];
    WIDE_MARK(16 + s);
  }
  WIDE_MARK(22);
  __syncthreads();
  {
    WIDE_MARK(23);
    uint32_t pending = sh.lost_n;
    if (pending > (uint32_t)kWideQueue) {
      if (tid == 0) atomicOr(status, ZEN_STAT_RETRY);
      pending = kWideQueue;
    }
    for (uint32_t e = tid; e < pending; e += kWideBlock) {
      const uint32_t my = sh.q_word[e], key = my >> 15;
      const uint32_t g0 = sh.q_range[e] & 0xffffu, g1 = sh.q_range[e] >> 16;
      uint32_t less = 0, twins = 0;
      for (uint32_t u = g0; u < g1; ++u) {
        const uint32_t w = sh.word[u];
        less += (w >> 15) < key;
        twins += (w >> 15) == key && w != my;
      }
      uint32_t lost = 0;
      if (twins) {
        const uint32_t mine = records[raw_at(my & 0x7fffu)].x;
        for (uint32_t u = g0; u < g1; ++u) {
          const uint32_t w = sh.word[u];
          if ((w >> 15) == key && w != my) lost += records[raw_at(w & 0x7fffu)].x < mine;
        }
      }
      sh.q_word[e] = (g0 + less + lost) | (lost ? kRemovedBit : 0u);  // the entry's thread is its only reader
    }
    WIDE_MARK(24);
    __syncthreads();
    WIDE_MARK(25);
#pragma unroll
    for (int i = 0; i < kWideItems; ++i)
      if (rk[i] != kInvalid && (rk[i] & kRemovedBit)) rk[i] = sh.q_word[rk[i] & kIndexMask];
    __syncthreads();  // the queue's memory serves other lists from here on
    if (tid == 0) sh.lost_n = 0;
  }
  __syncthreads();
  WIDE_MARK(3);
  // the narrow ranges' first places go to memory for the other workgroups' look-ups before the values take
  // the counters' place
  for (uint32_t j = tid; j < (uint32_t)kWideIndexLen; j += kWideBlock) {
    const uint32_t s0 = j * kWideIndexStep;
    store_agent(&tb.sub_index[(size_t)b * kWideIndexLen + j],
                sh.cnt.start_of(s0) | (sh.cnt.end_of(s0 + kWideIndexStep - 1) << 16));
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kWideRounds; ++r) {
    if ((uint32_t)r * kWideBlock < longest) {
      uint32_t t[kWideSplit];
      S v[kWideSplit];
#pragma unroll
      for (int q = 0; q < kWideSplit; ++q) {
        const uint32_t e = tid + (uint32_t)r * kWideBlock;
        const size_t at = (size_t)q * tb.part_cap + (rk[r * kWideSplit + q] != kInvalid ? e : 0u);
        const uint2 rec = records[at];
        t[q] = rec.x;
        v[q] = (S)rec.y;
      }
#pragma unroll
      for (int q = 0; q < kWideSplit; ++q) {
        const uint32_t x = rk[r * kWideSplit + q];
        if (x != kInvalid) {
          const uint32_t p = x & kIndexMask;
          sh.idx[p] = t[q] | (x & kRemovedBit);
          sh.val[p] = v[q];
          if (x & kRemovedBit) {
            const uint32_t at = atomicAdd(&sh.lost_n, 1u);
            if (at < (uint32_t)kWideRemoved) sh.rm[at] = t[q];
          }
        }
      }
    }
  }
  __syncthreads();
  WIDE_MARK(4);
  uint32_t lost_n = sh.lost_n;
  if (lost_n > (uint32_t)kWideRemoved) {
    if (tid == 0) atomicOr(status, ZEN_STAT_RETRY);
    lost_n = kWideRemoved;
  }
  if (tid == 0) sh.base = lost_n ? atomicAdd(&tb.log_n[part * kWideCtrPad], lost_n) : 0u;
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
  WIDE_MARK(5);
  group_barrier(gbar, bpp, 1, status);
  WIDE_MARK(6);

  // ---- levels 2 and 3 for the partition's losers: loser i is the business of workgroup i % bpp, thread
  // i / bpp (more than bpp * 1024 of them: in rounds)
  unsigned long long *pcells = cells + ((size_t)part << tb.map_log2);
  Counters *pctr = &tb.ctr[part];
  const uint32_t local = b - part * bpp;
  uint32_t losers = load_agent(&tb.log_n[part * kWideCtrPad]);
  if (losers > tb.log_cap) losers = tb.log_cap;
  for (uint32_t i = tid * bpp + local; i < losers; i += bpp * kWideBlock) {
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
      const uint32_t old = map_min_claim(pcells, tb.map_log2, slot, cur, pctr, &full);
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
        const uint32_t at = atomicAdd(&tb.dlog_n[part * kWideCtrPad], 1u);
        if (at < tb.log_cap) {
          store_agent(&tb.dlog_t[(size_t)part * tb.log_cap + at], head);
          store_agent(&tb.dlog_at[(size_t)part * tb.log_cap + at], (head_bucket << 16) | head_place);
        } else {
          atomicOr(status, ZEN_STAT_RETRY);
        }
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
  WIDE_MARK(7);
  group_barrier(gbar, bpp, 2, status);
  WIDE_MARK(8);

  // ---- every workgroup of the partition looks at every logged entry: where it finally sits (the level-2/3
  // slot it holds in the map, or nowhere), and keeps what concerns its bucket: entries whose final slot lies
  // in it move in, its own owners that were pushed out drop out; the partition's last bucket also gathers the
  // entries that found no slot
  const bool last_of_part = local == bpp - 1;
  uint32_t pushed = load_agent(&tb.dlog_n[part * kWideCtrPad]);
  if (pushed > tb.log_cap) pushed = tb.log_cap;
  for (uint32_t i = tid; i < losers + pushed; i += kWideBlock) {
    const bool first = i < losers;
    const size_t at_log = (size_t)part * tb.log_cap + (first ? i : i - losers);
    const uint32_t t = load_agent(first ? &tb.log_t[at_log] : &tb.dlog_t[at_log]);
    const uint32_t from = first ? 0u : load_agent(&tb.dlog_at[at_log]);
    if (!first && (from >> 16) == b && (from & 0xffffu) < n) sh.idx[from & 0xffffu] |= kRemovedBit;  // pushed out once
    uint32_t prt = 0, cell = kNone, slot = kNone;
    for (int lv = 1; lv < g.levels && slot == kNone; ++lv) {
      const uint32_t s = probe_slot(g, t, lv, &prt);
      uint32_t at = 0;
      if (map_find_fresh(pcells, tb.map_log2, s, &at) == t) {
        slot = s;
        cell = at;
      }
    }
    if (i % bpp == local) store_agent(first ? &tb.log_cell[at_log] : &tb.dlog_cell[at_log], cell);
    if (slot != kNone) {
      if (geo.bucket_of(slot) == b) {
        const uint32_t at = atomicAdd(&sh.mv_n, 1u);
        if (at < (uint32_t)kWideMove) {
          sh.mk[at] = slot;
          sh.mi[at] = t;
        }
      }
    } else if (last_of_part) {
      const uint32_t at = atomicAdd(&sh.ser_n, 1u);
      if (at < (uint32_t)kSlabSerialCap) store_agent(&tb.ser_idx[(size_t)part * kSlabSerialCap + at], t);
    }
  }
  __syncthreads();
  WIDE_MARK(9);
  uint32_t mv_n = sh.mv_n;
  if (mv_n > (uint32_t)kWideMove) {
    if (tid == 0) atomicOr(status, ZEN_STAT_RETRY);
    mv_n = kWideMove;
  }
  const uint32_t serial_raw = sh.ser_n;
  uint32_t serial = serial_raw;
  if (serial > (uint32_t)kSlabSerialCap) {
    // more than the partition's serial region holds is an overflow; more than this path carries, a retry
    if (tid == 0) atomicOr(status, (int64_t)kSlabSerialCap >= spp ? ZEN_STAT_SERIAL_OVERFLOW : ZEN_STAT_RETRY);
    serial = kSlabSerialCap;
  }
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
  // what the bucket contributes is known: published at once, so that the later buckets find it while this
  // one still works out its places
  const uint32_t own_n = n - rm_n + mv_n;  // survivors + moved-in
  if (tid == 0) desc_store(&tb.desc[b], kDescAggregate | (uint64_t)(own_n + serial));
  {
    // the removed places in ascending order; moved-in entry j: its slot's rank among the moved-in slots (they
    // are distinct: a slot has one owner) and the sorted place in front of which it slips in (a bisection of
    // the bucket, whose slots are hashed again)
    uint32_t x = 0, xr = 0;
    if (tid < rm_n) {
      x = sh.rm[tid];
      for (uint32_t u = 0; u < rm_n; ++u) xr += sh.rm[u] < x;
    }
    uint32_t mj = 0, mplace = 0;
    if (tid < mv_n) {
      const uint32_t k = sh.mk[tid];
      for (uint32_t u = 0; u < mv_n; ++u) mj += sh.mk[u] < k;
      uint32_t p0 = 0, p1 = n;
      while (p0 < p1) {
        const uint32_t mid = p0 + ((p1 - p0) >> 1);
        if (geo.mod_m(poly(sh.idx[mid] & kIndexMask) + kSeed1) < k) p0 = mid + 1; else p1 = mid;
      }
      mplace = p0;
    }
    __syncthreads();
    if (tid < rm_n) sh.rm[xr] = x;
    if (tid < mv_n) sh.mp[mj] = mplace;
    __syncthreads();
    // where the bucket starts: the sum of what the earlier buckets publish (every workgroup of the launch is
    // resident; the wait is bounded all the same)
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
    WIDE_MARK(10);
    uint64_t sums;
    block_exclusive_scan<uint64_t, kWideBlock>(before, sh.scan64, &sums);
    const uint32_t out_base = (uint32_t)sums, in_part = (uint32_t)(sums >> 32);
    // Most stretches of 64 consecutive sorted places contain neither a removed entry nor the place where a
    // moved-in entry slips in: all their entries move by the same amount, found once per stretch.
    // Per stretch of 64 consecutive sorted places: how many moved-in entries slip in at or before its first
    // place and how many removed entries lie before it (12 bits each), and whether that holds for the whole
    // stretch (most contain neither a removed entry nor a place where an entry slips in).
    constexpr uint32_t kSame = 1u << 31;
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
      sh.delta[c] = (int32_t)(mv0 | (r0 << 12) | ((mv0 == mv1 && r0 == r1) ? kSame : 0u));
    }
    __syncthreads();
    WIDE_MARK(11);
#pragma unroll 4
    for (uint32_t p = tid; p < n; p += kWideBlock) {
      const uint32_t t = sh.idx[p];
      const S v = sh.val[p];
      const uint32_t d = (uint32_t)sh.delta[p >> 6];
      if (!(t & kRemovedBit)) {
        uint32_t mv = d & 0xfffu, r = (d >> 12) & 0xfffu;
        if (!(d & kSame)) {  // a few steps from the stretch's first place
          while (mv < mv_n && sh.mp[mv] <= p) ++mv;
          while (r < rm_n && sh.rm[r] < p) ++r;
        }
        const uint32_t pos = out_base + p + mv - r;
        if (pos < capacity) {
          out_idx[pos] = (int32_t)t;
          out_val[pos] = v;
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
  WIDE_MARK(12);

  // ---- the borrowed memory goes back as it was.  This workgroup was the only reader of its part cursors;
  // the partition's workgroup that finishes last (all of them are through with the map and the logs then)
  // empties the cells the partition holds and clears its counters; the launch's last workgroup clears what
  // the buckets published.
  if (tid < (uint32_t)kWideSplit) tb.cursor[(b * kWideSplit + tid) * kWidePad] = 0;
  wait_global_acks();
  __syncthreads();
  if (tid == 0) {
    const uint32_t here = atomicAdd(&tb.pdone[part * kWidePad], 1u), all = atomicAdd(tb.done, 1u);
    sh.flag = (here == bpp - 1u ? 1u : 0u) | (all == B - 1u ? 2u : 0u);
  }
  __syncthreads();
  WIDE_MARK(13);
  if (sh.flag & 1u) {
    // every occupied cell ends with the index that finally holds its slot, and that index's cell was recorded
    for (uint32_t i = tid; i < losers + pushed; i += kWideBlock) {
      const size_t at = (size_t)part * tb.log_cap + (i < losers ? i : i - losers);
      const uint32_t cell = load_agent(i < losers ? &tb.log_cell[at] : &tb.dlog_cell[at]);
      if (cell != kNone) pcells[cell] = 0ull;
    }
    if (tid == 0) {
      tb.gbar[part * kWidePad] = 0;
      tb.pdone[part * kWidePad] = 0;
      tb.log_n[part * kWideCtrPad] = 0;
      tb.dlog_n[part * kWideCtrPad] = 0;
      pctr->logged = pctr->losers = pctr->claims = pctr->displaced = 0;
    }
  }
  if (sh.flag & 2u) {
    for (uint32_t i = tid; i < B; i += kWideBlock) tb.desc[i] = 0ull;
    if (tid == 0) *tb.done = 0;
  }
  WIDE_MARK(14);
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
    p.tb.pdone = cv.take<uint32_t>(P * kWidePad);
    p.tb.log_n = cv.take<uint32_t>(P * kWideCtrPad);
    p.tb.dlog_n = cv.take<uint32_t>(P * kWideCtrPad);
    p.tb.desc = cv.take<unsigned long long>(B);
    p.tb.done = cv.take<uint32_t>(1);
    p.tb.ctr = cv.take<Counters>(P);
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
  p.tb.words = cv.take<uint32_t>((size_t)2 * B * kWideSplit * p.tb.part_cap);
  p.tb.slab_idx = cv.take<uint32_t>(B * kWideCap);
  p.tb.sub_index = cv.take<uint32_t>(B * kWideIndexLen);
  p.tb.log_cap = (uint32_t)(list_cap / 4 / (int64_t)P + 1024);
  p.tb.log_t = cv.take<uint32_t>(P * p.tb.log_cap);
  p.tb.log_cell = cv.take<uint32_t>(P * p.tb.log_cap);
  p.tb.dlog_t = cv.take<uint32_t>(P * p.tb.log_cap);
  p.tb.dlog_cell = cv.take<uint32_t>(P * p.tb.log_cap);
  p.tb.dlog_at = cv.take<uint32_t>(P * p.tb.log_cap);
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
  // with few expected records the buckets take half the chip, else all of it: room for either
  SlabGeom half, full;
  if (capacity > 0x1fffffffll || cus <= 0 || !wide_geometry(m, partitions, 1, cus, &half)) return 0;
  size_t bytes = plan_wide(nullptr, nullptr, half, partitions, dtype, list_capacity(capacity)).bytes;
  const int64_t most = cus < kWideMaxBuckets ? cus : kWideMaxBuckets;
  if (wide_geometry(m, partitions, most * (int64_t)kWideTarget, cus, &full)) {
    const size_t other = plan_wide(nullptr, nullptr, full, partitions, dtype, list_capacity(capacity)).bytes;
    if (other > bytes) bytes = other;
  }
  return bytes;
}

int wide_load_balance(const SlabBalanceArgs &a, size_t state_offset, hipStream_t s) {
  SlabGeom geo;
  if (!wide_balance_fits(a.g.m, a.partitions, a.capacity, a.k, wide_device_cus(), &geo))
    return fail(ZEN_EINVAL, "wide_load_balance: sizes do not suit the wide buckets");
  char *state = reinterpret_cast<char *>(a.hash) + state_offset;
  WidePlan p = plan_wide(a.workspace, state, geo, a.partitions, a.dtype, list_capacity(a.capacity));
  if (state_offset + p.state_bytes > (size_t)a.g.m * sizeof(int32_t))
    return fail(ZEN_EINVAL, "wide_load_balance: table too small for the counters");
  // the map is cut into one part per partition (a partition's chains never leave its slots), so that a
  // partition's workgroups can empty their part as soon as they are through with it
  const int part_bits = ceil_log2_u64((uint64_t)a.partitions - 1u);
  if ((int)a.hash_log2 < part_bits + 8) return fail(ZEN_EINVAL, "wide_load_balance: table too small for the map");
  p.tb.map_log2 = a.hash_log2 - (uint32_t)part_bits;
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
  const int set = (a.prepared == 2 || a.second) ? 1 : 0;
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
  if (a.next_input && a.next_k > 0) {
    sc.next_in = a.next_input;
    sc.next_k = a.next_k;
    sc.next_n = a.next_n;
    sc.next_hist = p.sample_hist[1 - set];
    if (a.next_state) {  // the sampling memory sits at the head of that table's zero-between-calls memory
      Carver cn(a.next_state);
      uint32_t *first = cn.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
      uint32_t *second = cn.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
      sc.next_hist = set ? first : second;
    }
    sc.next_floor = p.thr + 2 + 4 * (1 - set);
  }
  if ((rc = select_stage_slabs(sc, s)) != ZEN_OK) return rc;
  uint32_t *clear = p.cand_hist;  // the candidates' histogram and the select kernel's tickets lie side by side
  uint32_t clear_words = (uint32_t)(reinterpret_cast<char *>(p.tb.cursor) - reinterpret_cast<char *>(p.cand_hist)) / 4u;
  if (refine) {
    const uint32_t refine_parts = p.cg.groups * (uint32_t)kCoarseSplit;
    k_refine_threshold<<<dim3(refine_parts < 128u ? refine_parts : 128u), dim3(kRefineBlock), 0, s>>>(
        p.cg, -1, p.tb.cursor, p.tb.words, static_cast<const uint32_t *>(a.input), p.thr, p.thr + 4, (uint32_t)a.k,
        p.refine_hist, a.thr_out, a.status);
    ZEN_LAUNCH_CHECK("k_refine_threshold");
  }
  const uint32_t *filter = a.k > 0 ? p.thr : nullptr;
  uint32_t *clear_too = refine ? p.refine_hist : nullptr;
  const uint32_t clear_too_words = refine ? (uint32_t)kRefineBins + 1u : 0u;
  if ((rc = wide_line_enter(s)) != ZEN_OK) return rc;
  {
    ProfScope prof(kProfWideTail, s);
    if (a.dtype == ZEN_BF16)
      k_wide_tail<uint16_t><<<dim3(geo.nbuckets), dim3(kWideBlock), 0, s>>>(
          geo, a.g, p.tb, filter, a.hash, a.spp, static_cast<const uint16_t *>(a.input), a.out_idx,
          static_cast<uint16_t *>(a.out_val), (uint32_t)a.capacity, a.splits, clear, clear_words, clear_too,
          clear_too_words, a.status);
    else
      k_wide_tail<uint32_t><<<dim3(geo.nbuckets), dim3(kWideBlock), 0, s>>>(
          geo, a.g, p.tb, filter, a.hash, a.spp, static_cast<const uint32_t *>(a.input), a.out_idx,
          static_cast<uint32_t *>(a.out_val), (uint32_t)a.capacity, a.splits, clear, clear_words, clear_too,
          clear_too_words, a.status);
    ZEN_LAUNCH_CHECK("k_wide_tail");
  }
  return wide_line_leave(s);
}

}  // namespace zen

#ifdef ZEN_WIDE_TIMING
extern "C" int zen_wide_debug_read(unsigned long long *host) {
  return hipMemcpyFromSymbol(host, HIP_SYMBOL(zen::g_wide_dbg), sizeof(unsigned long long) * 256 * 32) == hipSuccess ? 0 : -1;
}
#endif
