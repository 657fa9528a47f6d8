// Receive side on wide buckets (zen_wide.h): the fast path of zen_merge for a few million received entries at
// most.
//
// The reference builds a dense zero tensor of the full gradient length, scatter-adds every payload into it
// and extracts the nonzeros again (comm.py:32-50).  The indices a destination receives were assigned to it by
// a hash, so they spread evenly over [0, dense_n): the entries go to at most 256 buckets by index range, as
// (index, arrival number, value) records (k_wide_scatter: a workgroup orders its 4096 entries by bucket in
// LDS and writes one run per bucket), and one workgroup per bucket sorts its bucket by (index, arrival number)
// inside LDS, sums every run of equal indices in arrival order from +0 (bit-identical to a sequential
// scatter_add_), drops zero sums and writes what is left at the place the buckets before it leave off
// (k_wide_merge).  Two launches; zen_merge.hip needs three, and a thousand buckets, for the same input.
#include "zen_wide.h"

namespace zen {
namespace {

constexpr uint32_t kWmCursorWords = kWideMaxBuckets * kWideSplit * kWmPad;
static_assert(kWmCursorWords <= kCoarseCursorWords, "the cursors fit the zero region of the slab path's coarse cursors");
constexpr int kWmRounds = 3;                               // a part of a bucket's slab is read in rounds of kWideBlock records
constexpr int kWmItems = kWideSplit * kWmRounds;           // records per thread
constexpr int kWmPartMax = kWideBlock * kWmRounds;         // records of one part, at most
constexpr int kWmLanes = 4;                                // records a thread handles per step of the ranking loops
constexpr int kWmSteps = kWmItems / kWmLanes;
constexpr int kWmQueue = 6144;                             // records of large groups set aside while ranking
constexpr int kWmGroupLimit = 2048;                        // records in one narrow range: bounds the rank loop
constexpr int kWmSumItems = 17;                            // sorted records per thread while summing (odd: no LDS bank conflicts)
constexpr uint32_t kInvalid = 0xffffffffu;
static_assert(kWideBlock * kWmSumItems >= kWideCap, "every sorted place needs an owner");
static_assert(kWmQueue <= (1 << 14) && kWideCap <= (1 << 14) && kWideSubs <= (1 << 14), "queue entries in one word");

// ------------------------------------------------------------ list -> buckets

constexpr int kWsBlock = 512;
constexpr int kWsItems = 8;
constexpr int kWsBatch = kWsBlock * kWsItems;  // list entries per workgroup

template <typename S>
__global__ __launch_bounds__(kWsBlock) void k_wide_scatter(WideList list) {
  // 32 KB of LDS: five workgroups share a compute unit and the whole grid is resident in one round (the values
  // do not pass through LDS for that reason: they are fetched again when the record is written)
  __shared__ WideScatterShared<kWsBlock, kWsItems> sh;
  wide_scatter_prepare(list, sh);
  wide_scatter_batch<S>(list, blockIdx.x, blockIdx.x % kWideSplit, sh);
}

// ------------------------------------------------------------ a bucket

struct WideMergeShared {
  union {
    uint32_t word[kWideCap];  // while ranking: (index inside its narrow range) << tie_bits | arrival number
    uint32_t key[kWideCap];   // afterwards: the sorted indices (minus the bucket's first), then the kept ones
  };
  union {
    WideCounters cnt;
    float val[kWideCap];      // the sorted values, then the kept sums
  };
  uint32_t queue[kWmQueue];   // records set aside: place in `word` | narrow range << 14, then the rank
  uint32_t scan[kWideBlock / 64 + 1];
  uint64_t scan64[kWideBlock / 64 + 1];
  uint32_t qn, big;
  int tile;
};

template <typename I, typename S>
__global__ __launch_bounds__(kWideBlock) void k_wide_merge(SlabGeom geo, WideSlabs in, I *__restrict__ out_idx,
                                                           float *__restrict__ out_val, int64_t capacity,
                                                           ScanState st, int tie_bits, int64_t *out_count,
                                                           int32_t *status) {
  __shared__ WideMergeShared sh;
  const uint32_t tid = threadIdx.x;
  if (tid == 0) {
    sh.tile = (int)atomicAdd(st.ticket, 1u);
    sh.qn = sh.big = 0;
  }
  sh.cnt.clear();
  __syncthreads();
  const uint32_t b = (uint32_t)sh.tile;  // buckets are taken in order, so every earlier bucket already runs
  const uint32_t nb = geo.nbuckets;
  if (b >= nb) return;
  const uint32_t lo = geo.first_key(b);
  uint32_t pcount[kWideSplit];
  uint32_t longest = 0;
#pragma unroll
  for (int q = 0; q < kWideSplit; ++q) {
    pcount[q] = in.cursor[(b * kWideSplit + q) * kWmPad];
    if (pcount[q] > in.part_cap) pcount[q] = in.part_cap;  // the scatter flagged the overflow
    longest = pcount[q] > longest ? pcount[q] : longest;
  }
  bool declined = false;
  if (longest > (uint32_t)kWmPartMax) {
    declined = true;
#pragma unroll
    for (int q = 0; q < kWideSplit; ++q) pcount[q] = 0;
    longest = 0;
  }
  const uint2 *rec_plane = in.rec + (size_t)b * kWideSplit * in.part_cap;
  const uint32_t *val_plane = in.val32 + (size_t)b * kWideSplit * in.part_cap;
  const int shift = geo.sub_shift;
  const uint32_t low_mask = (1u << shift) - 1u;

  // item r * kWideSplit + q of a thread is the record at place tid + r * kWideBlock of part q; loads in no
  // branch, so that all are in flight together
  uint32_t w[kWmItems], ps[kWmItems];  // the record's word; then its place in `word` | narrow range << 14
#pragma unroll
  for (int r = 0; r < kWmRounds; ++r) {
#pragma unroll
    for (int q = 0; q < kWideSplit; ++q) w[r * kWideSplit + q] = ps[r * kWideSplit + q] = kInvalid;
    if ((uint32_t)r * kWideBlock < longest) {
#pragma unroll
      for (int q = 0; q < kWideSplit; ++q) {
        const uint32_t e = tid + (uint32_t)r * kWideBlock;
        const size_t at = (size_t)q * in.part_cap + (e < pcount[q] ? e : 0u);
        const uint2 rec = rec_plane[at];
        const uint32_t off = wm_off(rec), arr = wm_arr(rec);
        if (e < pcount[q]) {
          w[r * kWideSplit + q] = ((off & low_mask) << tie_bits) | arr;
          ps[r * kWideSplit + q] = off >> shift;  // the narrow range, for now
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kWmItems; ++i)
    if (ps[i] != kInvalid) sh.cnt.count(ps[i]);
  __syncthreads();
  uint32_t n = sh.cnt.starts(sh.scan, (uint32_t)kWmGroupLimit, &sh.big);
  __syncthreads();
  if (n > (uint32_t)kWideCap || sh.big) {  // more than fits, or keys piled on a few values: another path answers
    declined = true;
    __syncthreads();
    sh.cnt.clear();
#pragma unroll
    for (int i = 0; i < kWmItems; ++i) w[i] = ps[i] = kInvalid;
    n = 0;
    longest = 0;
    __syncthreads();
  }
  if (declined && tid == 0) atomicOr(status, ZEN_STAT_RETRY);
  // this workgroup was the only reader of its part cursors: back to zero for the next call
  if (tid < (uint32_t)kWideSplit) in.cursor[(b * kWideSplit + tid) * kWmPad] = 0;

  // The thread's records are worked through in steps of kWmLanes, by loops whose body handles the first
  // kWmLanes registers of a set and then rotates the set (the body written out for all records would not fit
  // the instruction cache, and every workgroup runs it once).
  auto rotate = [](uint32_t (&a)[kWmItems]) {
    uint32_t head[kWmLanes];
#pragma unroll
    for (int k = 0; k < kWmLanes; ++k) head[k] = a[k];
#pragma unroll
    for (int i = 0; i + kWmLanes < kWmItems; ++i) a[i] = a[i + kWmLanes];
#pragma unroll
    for (int k = 0; k < kWmLanes; ++k) a[kWmItems - kWmLanes + k] = head[k];
  };
  const int steps = longest == 0 ? 0 : (int)((longest + kWideBlock - 1) / kWideBlock) * (kWideSplit / kWmLanes);
#pragma unroll 1
  for (int s = 0; s < kWmSteps; ++s) {
    if (s < steps) {
#pragma unroll
      for (int k = 0; k < kWmLanes; ++k) {
        if (ps[k] != kInvalid) {
          const uint32_t p = sh.cnt.take(ps[k]);
          sh.word[p] = w[k];
          ps[k] = p | (ps[k] << 14);
        }
      }
    }
    rotate(w);
    rotate(ps);
  }
  __syncthreads();
  // rank = records of the bucket with a smaller (index, arrival number): those of the narrow ranges before,
  // plus those of the record's own range with a smaller word.  The range's first four words are fetched in one
  // go, which settles ranges up to that size; where many records share an index (payloads that overlap) a few
  // lanes of every wave would walk through dozens of words while the others wait: records of larger ranges
  // are set aside and handed out again afterwards, one per thread.
  uint32_t rk[kWmItems];
#pragma unroll
  for (int i = 0; i < kWmItems; ++i) rk[i] = kInvalid;
#pragma unroll 1
  for (int s = 0; s < kWmSteps; ++s) {
    constexpr int kAhead = 4;
    uint32_t out[kWmLanes];
#pragma unroll
    for (int k = 0; k < kWmLanes; ++k) out[k] = kInvalid;
    if (s < steps) {
      uint32_t g0[kWmLanes], g1[kWmLanes], a[kWmLanes][kAhead];
#pragma unroll
      for (int k = 0; k < kWmLanes; ++k) {
        const uint32_t sub = ps[k] != kInvalid ? ps[k] >> 14 : 0u;
        g0[k] = sh.cnt.start_of(sub);
        g1[k] = sh.cnt.end_of(sub);
      }
#pragma unroll
      for (int k = 0; k < kWmLanes; ++k) {
        const uint32_t last = g1[k] > g0[k] ? g1[k] - 1u : g0[k];
#pragma unroll
        for (int e = 0; e < kAhead; ++e) a[k][e] = sh.word[g0[k] + e < last ? g0[k] + e : last];
      }
#pragma unroll
      for (int k = 0; k < kWmLanes; ++k) {
        if (ps[k] != kInvalid) {
          uint32_t less = 0;
#pragma unroll
          for (int e = 0; e < kAhead; ++e) less += g0[k] + e < g1[k] && a[k][e] < w[k];
          uint32_t x = g0[k] + less;
          if (g1[k] - g0[k] > (uint32_t)kAhead) {
            const uint32_t at = atomicAdd(&sh.qn, 1u);
            if (at < (uint32_t)kWmQueue) {
              sh.queue[at] = ps[k];
              x = 0x80000000u | at;  // pending: place in the queue
            }
          }
          out[k] = x;
        }
      }
    }
    rotate(w);
    rotate(ps);
    rotate(rk);  // the step's ranks enter at the end: after the last step rank i belongs to record i
#pragma unroll
    for (int k = 0; k < kWmLanes; ++k) rk[kWmItems - kWmLanes + k] = out[k];
  }
  __syncthreads();
  {
    uint32_t pending = sh.qn;
    if (pending > (uint32_t)kWmQueue) {
      if (tid == 0) atomicOr(status, ZEN_STAT_RETRY);
      pending = kWmQueue;
    }
    for (uint32_t e = tid; e < pending; e += kWideBlock) {
      const uint32_t p = sh.queue[e] & 0x3fffu, sub = sh.queue[e] >> 14;
      const uint32_t g0 = sh.cnt.start_of(sub), g1 = sh.cnt.end_of(sub);
      const uint32_t my = sh.word[p];
      uint32_t less = 0;
      for (uint32_t u = g0; u < g1; u += 4) {
        const uint32_t last = g1 - 1u;
        const uint32_t a0 = sh.word[u], a1 = sh.word[u + 1 < last ? u + 1 : last];
        const uint32_t a2 = sh.word[u + 2 < last ? u + 2 : last], a3 = sh.word[u + 3 < last ? u + 3 : last];
        less += (a0 < my) + (u + 1 < g1 && a1 < my) + (u + 2 < g1 && a2 < my) + (u + 3 < g1 && a3 < my);
      }
      sh.queue[e] = g0 + less;  // the entry's thread is its only reader
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kWmItems; ++i)
      if (rk[i] != kInvalid && (rk[i] & 0x80000000u)) rk[i] = sh.queue[rk[i] & 0x7fffffffu];
  }
  __syncthreads();  // everybody is through with the words and the counters: the sorted records take their place
#pragma unroll
  for (int r = 0; r < kWmRounds; ++r) {
    if ((uint32_t)r * kWideBlock < longest) {
      uint32_t v[kWideSplit];
#pragma unroll
      for (int q = 0; q < kWideSplit; ++q) {
        const uint32_t e = tid + (uint32_t)r * kWideBlock;
        const size_t at = (size_t)q * in.part_cap + (rk[r * kWideSplit + q] != kInvalid ? e : 0u);
        v[q] = sizeof(S) == 2 ? rec_plane[at].y >> 16 : val_plane[at];
      }
#pragma unroll
      for (int q = 0; q < kWideSplit; ++q) {
        const int i = r * kWideSplit + q;
        if (rk[i] != kInvalid) {
          sh.key[rk[i]] = ((ps[i] >> 14) << shift) | (w[i] >> tie_bits);
          sh.val[rk[i]] = KeyOf<S>::to_f32((S)v[q]);
        }
      }
    }
  }
  __syncthreads();
  // Thread t owns the sorted places [t * per, (t + 1) * per): as few per thread as cover the bucket (and an odd
  // number, which keeps the lanes of a wave on different LDS banks).  It fetches them all at once and walks
  // through them in registers.  A run of equal indices is summed in arrival order from +0 (like the dense
  // tensor of comm.py:35) and belongs to the thread that holds its last record; where that run began before
  // the thread's first place (rare: runs are short next to `per`, long ones come from payloads that overlap),
  // the part in front is summed first, from the run's head on.
  const uint32_t per = ((n + kWideBlock - 1) / kWideBlock) | 1u;  // <= kWmSumItems
  const uint32_t first = tid * per;
  uint32_t k[kWmSumItems];
  float sum[kWmSumItems];
  uint32_t keep = 0;
  {
    constexpr uint32_t kNoKey = 0xffffffffu;  // offsets are below the bucket width
    float v[kWmSumItems];
#pragma unroll
    for (int q = 0; q < kWmSumItems; ++q) {
      const uint32_t p = first + q;
      const bool have = (uint32_t)q < per && p < n;
      const uint32_t from = have ? p : 0u;
      k[q] = sh.key[from];
      v[q] = sh.val[from];
      if (!have) k[q] = kNoKey;
    }
    const uint32_t before_k = first > 0 && first < n ? sh.key[first - 1] : kNoKey;
    const uint32_t after_k = first + per < n ? sh.key[first + per] : kNoKey;
    float acc = 0.0f;
    if (first < n && before_k == k[0]) {
      // the run began before this thread's places: find its head, sum up to the place in front of `first`
      uint32_t head = first - 1;
      while (head > 0 && sh.key[head - 1] == before_k) --head;
      for (uint32_t u = head; u < first; ++u) acc += sh.val[u];
    }
    uint32_t prev = before_k;
#pragma unroll
    for (int q = 0; q < kWmSumItems; ++q) {
      const uint32_t next = q + 1 < kWmSumItems ? ((uint32_t)(q + 1) < per ? k[q + 1] : after_k) : after_k;
      if (k[q] != kNoKey) {
        if (k[q] != prev) acc = 0.0f;
        acc += v[q];
        prev = k[q];
        sum[q] = acc;
        if (k[q] != next && acc != 0.0f) keep |= 1u << q;  // torch.nonzero keeps NaN, drops +-0
      } else {
        sum[q] = 0.0f;
      }
    }
  }
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kWideBlock>((uint32_t)__popc(keep), sh.scan, &total);
  // where this bucket's output starts: the sum of what all earlier buckets keep.  Every thread asks for one of
  // them (bounded wait), nobody waits for a chain of prefixes; while the answers are on their way the kept
  // entries are gathered in LDS (everybody is past reading the sorted bucket: the scan synchronised).
  if (tid == 0) desc_store(&st.desc[b], kDescAggregate | total);
  uint64_t d = tid < b ? desc_load(&st.desc[tid]) : kDescAggregate;
  uint32_t li = before;
#pragma unroll
  for (int q = 0; q < kWmSumItems; ++q) {
    if (keep & (1u << q)) {
      sh.key[li] = k[q] + lo;
      sh.val[li] = sum[q];
      ++li;
    }
  }
  {
    uint32_t spins = 0;
    while ((d >> 62) == 0) {
      if (++spins > kSpinLimit) {
        atomicOr(status, ZEN_STAT_INTERNAL);
        break;
      }
      __builtin_amdgcn_s_sleep(2);
      d = desc_load(&st.desc[tid]);
    }
  }
  uint64_t all_before;
  block_exclusive_scan<uint64_t, kWideBlock>(d & kDescValue, sh.scan64, &all_before);  // its barriers also publish the gathered entries
  if (b == nb - 1 && tid == 0) {
    const uint64_t all = all_before + total;
    *out_count = (int64_t)all;
    if (all > (uint64_t)capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
  for (uint32_t i = tid; i < total; i += kWideBlock) {
    const uint64_t pos = all_before + i;
    if (pos < (uint64_t)capacity) {
      out_idx[pos] = (I)sh.key[i];
      out_val[pos] = sh.val[i];
    }
  }
  // every workgroup has read the descriptors it needs before it gets here: the last one to finish clears the
  // prefix state
  uint32_t *finished = reinterpret_cast<uint32_t *>(st.desc + nb + 1);
  __syncthreads();
  if (tid == 0) sh.tile = atomicAdd(finished, 1u) == nb - 1u;
  __syncthreads();
  if (sh.tile) {
    for (uint32_t i = tid; i < nb; i += kWideBlock) st.desc[i] = 0ull;
    if (tid == 0) {
      *st.ticket = 0;
      *finished = 0;
    }
  }
}

}  // namespace

bool wide_merge_fits(int64_t r, int64_t dense_n, int cus, SlabGeom *geo) {
  SlabGeom g;
  if (r < (1 << 12) || r > 0x7ffffffell || cus <= 0 || !wide_geometry(dense_n, 1, r, cus, &g)) return false;
  if (g.sub_shift + ceil_log2_u64((uint64_t)r) > 32) return false;  // (index inside a narrow range, arrival number) must fit a word
  // a slab record carries the index's offset inside its bucket and the arrival number in fixed fields
  if ((uint64_t)g.sub_shift + 14 > kWmOffBits || (uint64_t)r >= (1ull << kWmArrBits)) return false;
  if (geo) *geo = g;
  return true;
}

static uint32_t wide_merge_part_cap(const SlabGeom &geo, int64_t r) { return wide_part_cap(geo, r + r / 4); }

// Workspace of the wide path behind the zero region at the head of zen_merge's workspace.
size_t wide_merge_bytes(int64_t r, int64_t dense_n, int cus) {
  SlabGeom geo;
  if (!wide_merge_fits(r, dense_n, cus, &geo)) return 0;
  const size_t entries = (size_t)geo.nbuckets * kWideSplit * wide_merge_part_cap(geo, r);
  return align_up(entries * sizeof(uint2), 256) + align_up(entries * sizeof(uint32_t), 256);
}

// The received entries as the scatter wants them: cursor: kCoarseCursorWords zeroed words (zero again when
// k_wide_merge has run); rest: wide_merge_bytes(...) bytes.  False if the sizes do not suit the wide buckets.
bool wide_merge_list(const void *idx, int idx64_in, const void *val, int64_t r, int64_t dense_n, uint32_t *cursor,
                     void *rest, int cus, int32_t *status, WideList *list) {
  SlabGeom geo;
  if (!wide_merge_fits(r, dense_n, cus, &geo)) return false;
  WideSlabs slabs;
  slabs.part_cap = wide_merge_part_cap(geo, r);
  const size_t entries = (size_t)geo.nbuckets * kWideSplit * slabs.part_cap;
  Carver cv(rest);
  slabs.cursor = cursor;
  slabs.rec = cv.take<uint2>(entries);
  slabs.val32 = cv.take<uint32_t>(entries);
  list->geo = geo;
  list->idx = idx;
  list->val = val;
  list->r = (uint32_t)r;
  list->dense_n = (uint32_t)dense_n;
  list->idx64 = idx64_in;
  list->out = slabs;
  list->status = status;
  return true;
}

uint32_t wide_scatter_batches(const WideList &list, int batch) { return (uint32_t)ceil_div((int64_t)list.r, batch); }

// The two launches (one if the entries are in the buckets' slabs already: `scattered`).  scan: zeroed prefix
// state for 256 buckets (descriptors, ticket, finished count), zero again when the launch ends.
int wide_merge(const WideList &list, int dtype, bool scattered, void *out_idx, int idx64_out, float *out_val,
               int64_t capacity, int64_t *out_count, unsigned long long *scan, hipStream_t s) {
  if (!scattered) {
    ProfScope prof(kProfWideScatter, s);
    if (dtype == ZEN_BF16)
      k_wide_scatter<uint16_t><<<dim3(wide_scatter_batches(list, kWsBatch)), dim3(kWsBlock), 0, s>>>(list);
    else
      k_wide_scatter<uint32_t><<<dim3(wide_scatter_batches(list, kWsBatch)), dim3(kWsBlock), 0, s>>>(list);
    ZEN_LAUNCH_CHECK("k_wide_scatter");
  }
  const ScanState st = scan_state(scan, (int64_t)list.geo.nbuckets);
  const int tie_bits = ceil_log2_u64((uint64_t)list.r);  // arrival numbers are < r
  ProfScope prof(kProfWideMerge, s);
  const dim3 grid(list.geo.nbuckets), block(kWideBlock);
  if (dtype == ZEN_BF16) {
    if (idx64_out)
      k_wide_merge<int64_t, uint16_t><<<grid, block, 0, s>>>(list.geo, list.out, static_cast<int64_t *>(out_idx), out_val,
                                                             capacity, st, tie_bits, out_count, list.status);
    else
      k_wide_merge<int32_t, uint16_t><<<grid, block, 0, s>>>(list.geo, list.out, static_cast<int32_t *>(out_idx), out_val,
                                                             capacity, st, tie_bits, out_count, list.status);
  } else {
    if (idx64_out)
      k_wide_merge<int64_t, uint32_t><<<grid, block, 0, s>>>(list.geo, list.out, static_cast<int64_t *>(out_idx), out_val,
                                                             capacity, st, tie_bits, out_count, list.status);
    else
      k_wide_merge<int32_t, uint32_t><<<grid, block, 0, s>>>(list.geo, list.out, static_cast<int32_t *>(out_idx), out_val,
                                                             capacity, st, tie_bits, out_count, list.status);
  }
  ZEN_LAUNCH_CHECK("k_wide_merge");
  return ZEN_OK;
}

}  // namespace zen
