// Stable LSD radix sort of (uint32 key, uint32 value[, uint32 value]) records.
// Four kernels per digit: per-tile histogram, digit totals, offsets, stable
// scatter.  The scatter ranks its tile in LDS (wave ballots + per-wave digit
// counters), reorders the tile in LDS and writes every digit's run with
// consecutive lanes, so global stores are contiguous runs instead of 4-byte
// scatters.  The element count may live on the device, so grids are sized by
// the capacity and surplus tiles retire immediately.
#include "zen_common.h"

namespace zen {

thread_local char g_last_error[256] = "";

namespace {

constexpr int kSortBlock = 256;
constexpr int kSortItems = 16;                       // keys per thread
constexpr int kSortTile = kSortBlock * kSortItems;   // 4096 keys per tile
constexpr int kWaveSpan = 64 * kSortItems;           // contiguous keys owned by one wave
constexpr int kMaxRadix = 1024;

// Digit of a key: a bit field (LSD passes), or a monotone map of [0, sentinel) onto `last` equal ranges
// with every key >= sentinel in a range of its own (bucket pass).
struct DigitField {
  int shift;
  uint32_t mask;
  __device__ uint32_t operator()(uint32_t k) const { return (k >> shift) & mask; }
};
struct DigitRange {
  uint32_t mult;      // floor(last * 2^32 / sentinel)
  uint32_t sentinel;
  uint32_t last;      // number of real ranges = index of the sentinel's own
  __device__ uint32_t operator()(uint32_t k) const {
    return k >= sentinel ? last : (uint32_t)(((uint64_t)k * mult) >> 32);
  }
  __device__ uint32_t first_key(uint32_t b) const {  // smallest key of range b
    return (uint32_t)((((uint64_t)b << 32) + mult - 1) / mult);
  }
};

__device__ inline uint32_t live_count(const uint32_t *count_dev, uint32_t count_imm) {
  if (!count_dev) return count_imm;
  const uint32_t c = *count_dev;
  return c < count_imm ? c : count_imm;
}

// hist[d * nblk + tile] = number of keys of this tile whose digit is d
template <int RB, typename Digit>
__global__ __launch_bounds__(kSortBlock) void k_sort_hist(const uint32_t *__restrict__ keys,
                                                          const uint32_t *count_dev, uint32_t count_imm,
                                                          Digit digit, int nblk,
                                                          uint32_t *__restrict__ hist) {
  constexpr int R = 1 << RB;
  __shared__ uint32_t bins[R];
  const uint32_t count = live_count(count_dev, count_imm);
  const uint32_t base = blockIdx.x * (uint32_t)kSortTile;
  for (int d = threadIdx.x; d < R; d += kSortBlock) bins[d] = 0;
  __syncthreads();
  if (base < count) {
    const uint32_t wave_base = base + (threadIdx.x >> 6) * kWaveSpan + (threadIdx.x & 63);
    uint32_t k[kSortItems];
#pragma unroll
    for (int i = 0; i < kSortItems; ++i) {
      const uint32_t at = wave_base + i * 64;
      k[i] = at < count ? keys[at] : 0u;
    }
#pragma unroll
    for (int i = 0; i < kSortItems; ++i)
      if (wave_base + i * 64 < count) atomicAdd(&bins[digit(k[i])], 1u);
  }
  __syncthreads();
  for (int d = threadIdx.x; d < R; d += kSortBlock) hist[(size_t)d * nblk + blockIdx.x] = bins[d];
}

// Block d: totals[d] = sum of row d.
__global__ __launch_bounds__(kSortBlock) void k_sort_totals(const uint32_t *__restrict__ hist, int nblk,
                                                            uint32_t *__restrict__ totals) {
  __shared__ uint32_t smem[kSortBlock / 64 + 1];
  const uint32_t *row = hist + (size_t)blockIdx.x * nblk;
  uint32_t mine = 0;
  for (int b = threadIdx.x; b < nblk; b += kSortBlock) mine += row[b];
  uint32_t total;
  block_exclusive_scan<uint32_t, kSortBlock>(mine, smem, &total);
  if (threadIdx.x == 0) totals[blockIdx.x] = total;
}

// Block d: the row of per-tile counts becomes per-tile global start offsets
// (keys of all lower digits first, then this digit's keys of earlier tiles).
__global__ __launch_bounds__(kSortBlock) void k_sort_offsets(uint32_t *__restrict__ hist, int nblk,
                                                             const uint32_t *__restrict__ totals) {
  __shared__ uint32_t smem[kSortBlock / 64 + 1];
  const int d = blockIdx.x;
  uint32_t below = 0;
  for (int e = threadIdx.x; e < d; e += kSortBlock) below += totals[e];
  uint32_t running;
  block_exclusive_scan<uint32_t, kSortBlock>(below, smem, &running);
  uint32_t *row = hist + (size_t)d * nblk;
  for (int b0 = 0; b0 < nblk; b0 += kSortBlock) {
    const int b = b0 + threadIdx.x;
    const uint32_t v = b < nblk ? row[b] : 0u;
    uint32_t chunk;
    const uint32_t ex = block_exclusive_scan<uint32_t, kSortBlock>(v, smem, &chunk);
    if (b < nblk) row[b] = running + ex;
    running += chunk;
  }
}

template <int RB, typename Digit>
__global__ __launch_bounds__(kSortBlock) void k_sort_scatter(
    const uint32_t *__restrict__ keys_in, const uint32_t *__restrict__ vals_in,
    const uint32_t *__restrict__ more_in, uint32_t *__restrict__ keys_out, uint32_t *__restrict__ vals_out,
    uint32_t *__restrict__ more_out, const uint32_t *count_dev,
    uint32_t count_imm, Digit digit, int nblk, const uint32_t *__restrict__ offsets) {
  constexpr int R = 1 << RB;
  constexpr int kPer = R / kSortBlock;  // digits per thread in the prefix step
  __shared__ uint32_t wcnt[kSortBlock / 64][R];  // per wave: count, then start inside the tile
  __shared__ uint32_t gshift[R];                 // global position = gshift[digit] + position in the tile
  __shared__ uint32_t smem[kSortBlock / 64 + 1];
  __shared__ uint32_t skey[kSortTile];
  __shared__ uint32_t sval[kSortTile];
  const uint32_t count = live_count(count_dev, count_imm);
  const uint32_t base = blockIdx.x * (uint32_t)kSortTile;
  if (base >= count) return;
  const uint32_t tile_count = count - base < (uint32_t)kSortTile ? count - base : (uint32_t)kSortTile;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  for (int w = 0; w < kSortBlock / 64; ++w)
    for (int d = threadIdx.x; d < R; d += kSortBlock) wcnt[w][d] = 0;
  __syncthreads();

  const uint32_t wave_base = base + wave * kWaveSpan + lane;
  uint32_t key[kSortItems];
  uint32_t rank[kSortItems];
  const uint64_t below = lanes_below();
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    const uint32_t at = wave_base + i * 64;
    key[i] = at < count ? keys_in[at] : 0u;
  }
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    const bool valid = wave_base + i * 64 < count;
    const uint32_t d = digit(key[i]);
    // lanes of this wave holding the same digit
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const bool bit = (d >> b) & 1u;
      const uint64_t vote = __ballot(valid && bit);
      peers &= bit ? vote : ~vote;
    }
    uint32_t old = 0;
    const int leader = valid ? __ffsll((unsigned long long)peers) - 1 : lane;
    if (valid && lane == leader) {
      old = wcnt[wave][d];
      wcnt[wave][d] = old + (uint32_t)__popcll(peers);
    }
    old = __shfl(old, leader, 64);
    rank[i] = old + (uint32_t)__popcll(peers & below);
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();
  {
    // thread owns kPer consecutive digits: start of each digit inside the tile, then one start per wave
    uint32_t c[kPer][kSortBlock / 64];
    uint32_t mine = 0;
#pragma unroll
    for (int e = 0; e < kPer; ++e)
#pragma unroll
      for (int w = 0; w < kSortBlock / 64; ++w) {
        c[e][w] = wcnt[w][threadIdx.x * kPer + e];
        mine += c[e][w];
      }
    uint32_t unused;
    uint32_t running = block_exclusive_scan<uint32_t, kSortBlock>(mine, smem, &unused);
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      const int d = threadIdx.x * kPer + e;
      gshift[d] = offsets[(size_t)d * nblk + blockIdx.x] - running;
#pragma unroll
      for (int w = 0; w < kSortBlock / 64; ++w) {
        wcnt[w][d] = running;
        running += c[e][w];
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    const uint32_t at = wave_base + i * 64;
    if (at < count) {
      const uint32_t pos = wcnt[wave][digit(key[i])] + rank[i];
      skey[pos] = key[i];
      sval[pos] = vals_in[at];
    }
  }
  __syncthreads();
  for (uint32_t j = threadIdx.x; j < tile_count; j += kSortBlock) {
    const uint32_t k = skey[j];
    const uint32_t g = gshift[digit(k)] + j;
    keys_out[g] = k;
    vals_out[g] = sval[j];
  }
  if (!more_in) return;
  // a second payload travels through the same LDS buffer in a second round
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    const uint32_t at = wave_base + i * 64;
    if (at < count) sval[wcnt[wave][digit(key[i])] + rank[i]] = more_in[at];
  }
  __syncthreads();
  for (uint32_t j = threadIdx.x; j < tile_count; j += kSortBlock)
    more_out[gshift[digit(skey[j])] + j] = sval[j];
}

__global__ void k_copy_pairs(const uint32_t *__restrict__ ka, const uint32_t *__restrict__ va,
                             uint32_t *__restrict__ kb, uint32_t *__restrict__ vb,
                             const uint32_t *count_dev, uint32_t count_imm) {
  const uint32_t count = live_count(count_dev, count_imm);
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) {
    kb[i] = ka[i];
    vb[i] = va[i];
  }
}

inline int num_tiles(int64_t max_count) {
  const int64_t t = ceil_div(max_count, kSortTile);
  return (int)(t < 1 ? 1 : t);
}

}  // namespace

size_t sort_scratch_bytes(int64_t max_count) {
  const size_t nblk = (size_t)num_tiles(max_count);
  return align_up(nblk * kMaxRadix * sizeof(uint32_t), 256) + align_up(kMaxRadix * sizeof(uint32_t), 256);
}

template <int RB, typename Digit>
static int sort_pass(uint32_t *ks, uint32_t *vs, uint32_t *ms, uint32_t *kd, uint32_t *vd, uint32_t *md,
                     int64_t max_count, const uint32_t *count_dev, Digit digit, int nblk,
                     uint32_t *hist, uint32_t *totals, hipStream_t stream) {
  constexpr int R = 1 << RB;
  k_sort_hist<RB, Digit><<<dim3(nblk), dim3(kSortBlock), 0, stream>>>(ks, count_dev, (uint32_t)max_count, digit,
                                                                      nblk, hist);
  ZEN_LAUNCH_CHECK("k_sort_hist");
  k_sort_totals<<<dim3(R), dim3(kSortBlock), 0, stream>>>(hist, nblk, totals);
  ZEN_LAUNCH_CHECK("k_sort_totals");
  k_sort_offsets<<<dim3(R), dim3(kSortBlock), 0, stream>>>(hist, nblk, totals);
  ZEN_LAUNCH_CHECK("k_sort_offsets");
  k_sort_scatter<RB, Digit><<<dim3(nblk), dim3(kSortBlock), 0, stream>>>(ks, vs, ms, kd, vd, md, count_dev,
                                                                         (uint32_t)max_count, digit, nblk, hist);
  ZEN_LAUNCH_CHECK("k_sort_scatter");
  return ZEN_OK;
}

int sort_pairs(uint32_t *keys_a, uint32_t *vals_a, uint32_t *keys_b, uint32_t *vals_b,
               int64_t max_count, const uint32_t *count_dev, int bits, void *scratch, int32_t *status,
               hipStream_t stream, uint32_t *more_a, uint32_t *more_b) {
  (void)status;
  if (max_count < 0 || max_count > 0x7fffffffll || bits < 0 || bits > 32)
    return fail(ZEN_EINVAL, "sort_pairs: bad count or bits");
  if (max_count == 0 || bits == 0) return 0;
  const int nblk = num_tiles(max_count);
  Carver cv(scratch);
  uint32_t *hist = cv.take<uint32_t>((size_t)nblk * kMaxRadix);
  uint32_t *totals = cv.take<uint32_t>(kMaxRadix);
  // 8-bit digits: 10-bit ones would save a pass on 25..30-bit keys, but with 4096-key tiles a digit's run
  // shrinks to 4 keys and the scatter loses more than the pass gains (measured on MI355X)
  constexpr int rb = 8;
  const int passes = (bits + rb - 1) / rb;
  uint32_t *ks = keys_a, *vs = vals_a, *kd = keys_b, *vd = vals_b, *ms = more_a, *md = more_b;
  for (int p = 0; p < passes; ++p) {
    const int shift = p * rb;
    const int width = bits - shift < rb ? bits - shift : rb;
    const uint32_t mask = (1u << width) - 1u;
    const int rc = sort_pass<8>(ks, vs, ms, kd, vd, md, max_count, count_dev, DigitField{shift, mask}, nblk, hist,
                                totals, stream);
    if (rc != ZEN_OK) return rc;
    uint32_t *t = ks; ks = kd; kd = t;
    t = vs; vs = vd; vd = t;
    t = ms; ms = md; md = t;
  }
  return passes & 1;
}

namespace {

// ---------------------------------------------------------------------------
// Bucket sort for keys that spread evenly over [0, sentinel): one scatter pass
// by DigitRange puts every key range into a contiguous bucket, then one
// workgroup per bucket sorts its records inside LDS and writes them back in
// place.  Inside a bucket the keys spread evenly as well, so the workgroup
// distributes them over up to kBktSubs narrow key ranges with one LDS atomic
// each (about one record per range), and every record finds its place inside
// its range by counting the range's records that precede it in (key, arrival)
// order, which one packed word per record decides: equal keys keep their
// arrival order.  Records with key >= sentinel end up behind all buckets,
// unsorted.  A bucket beyond kBktCap records, or a narrow range beyond
// kBktGroupLimit, raises ZEN_STAT_RETRY and the bucket stays unsorted.

constexpr int kBktBlock = 1024;
constexpr int kBktItems = 10;
constexpr int kBktCap = kBktBlock * kBktItems;  // 10240 records
constexpr int kBktSubs = 8192;
constexpr int kBktSubsPer = kBktSubs / kBktBlock;
constexpr int kBktGroupLimit = 2048;            // bounds the counting loop on piled-up keys
constexpr int kBktDigitBits = 9;                // 511 buckets + the sentinel's

template <bool MORE>
__global__ __launch_bounds__(kBktBlock) void k_bucket_sort(uint32_t *__restrict__ keys, uint32_t *__restrict__ vals,
                                                           uint32_t *__restrict__ more,
                                                           const uint32_t *__restrict__ totals, DigitRange digit,
                                                           int sub_shift, int32_t *status) {
  // first the records grouped by narrow range, as (key bits below the range << 14 | arrival position); in
  // the end the sorted keys
  __shared__ uint32_t s_a[kBktCap];
  __shared__ uint32_t s_b[kBktCap];
  __shared__ uint32_t s_c[MORE ? kBktCap : 1];
  __shared__ uint32_t s_cnt[kBktSubs + 1];
  __shared__ uint32_t smem[kBktBlock / 64 + 1];
  __shared__ uint32_t s_bad;
  const uint32_t b = blockIdx.x;
  uint32_t before = 0;
  for (uint32_t e = threadIdx.x; e < b; e += kBktBlock) before += totals[e];
  uint32_t start;
  block_exclusive_scan<uint32_t, kBktBlock>(before, smem, &start);
  const uint32_t n = totals[b];
  if (n > (uint32_t)kBktCap) {
    if (threadIdx.x == 0) atomicOr(status, ZEN_STAT_RETRY);
    return;
  }
  if (n < 2) return;
  const uint32_t lo = digit.first_key(b);
  for (int d = threadIdx.x; d <= kBktSubs; d += kBktBlock) s_cnt[d] = 0;
  if (threadIdx.x == 0) s_bad = 0;
  __syncthreads();
  uint32_t k[kBktItems], v[kBktItems], m[kBktItems], sub[kBktItems], at[kBktItems];
#pragma unroll
  for (int i = 0; i < kBktItems; ++i) {
    const uint32_t j = threadIdx.x + i * kBktBlock;
    k[i] = v[i] = m[i] = sub[i] = at[i] = 0;
    if (j < n) {
      k[i] = keys[start + j] - lo;
      v[i] = vals[start + j];
      if (MORE) m[i] = more[start + j];
    }
  }
#pragma unroll
  for (int i = 0; i < kBktItems; ++i) {
    if (threadIdx.x + i * kBktBlock < n) {
      sub[i] = k[i] >> sub_shift;
      at[i] = atomicAdd(&s_cnt[sub[i]], 1u);
    }
  }
  __syncthreads();
  {
    // counts become range starts; s_cnt[kBktSubs] = n
    uint32_t c[kBktSubsPer];
    uint32_t sum = 0, big = 0;
#pragma unroll
    for (int e = 0; e < kBktSubsPer; ++e) {
      c[e] = s_cnt[threadIdx.x * kBktSubsPer + e];
      sum += c[e];
      big |= c[e] > (uint32_t)kBktGroupLimit;
    }
    if (big) s_bad = 1;
    uint32_t unused;
    uint32_t running = block_exclusive_scan<uint32_t, kBktBlock>(sum, smem, &unused);
#pragma unroll
    for (int e = 0; e < kBktSubsPer; ++e) {
      s_cnt[threadIdx.x * kBktSubsPer + e] = running;
      running += c[e];
    }
    if (threadIdx.x == kBktBlock - 1) s_cnt[kBktSubs] = running;
  }
  __syncthreads();
  if (s_bad) {
    if (threadIdx.x == 0) atomicOr(status, ZEN_STAT_RETRY);
    return;
  }
  const uint32_t low_mask = (1u << sub_shift) - 1u;
#pragma unroll
  for (int i = 0; i < kBktItems; ++i) {
    const uint32_t j = threadIdx.x + i * kBktBlock;
    if (j < n) s_a[s_cnt[sub[i]] + at[i]] = ((k[i] & low_mask) << 14) | j;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kBktItems; ++i) {
    const uint32_t j = threadIdx.x + i * kBktBlock;
    if (j < n) {
      const uint32_t g0 = s_cnt[sub[i]], g1 = s_cnt[sub[i] + 1];
      const uint32_t mine = ((k[i] & low_mask) << 14) | j;
      uint32_t less = 0;
      for (uint32_t u = g0; u < g1; ++u) less += s_a[u] < mine;
      at[i] = g0 + less;
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kBktItems; ++i) {
    if (threadIdx.x + i * kBktBlock < n) {
      s_a[at[i]] = k[i];
      s_b[at[i]] = v[i];
      if (MORE) s_c[at[i]] = m[i];
    }
  }
  __syncthreads();
  for (uint32_t j = threadIdx.x; j < n; j += kBktBlock) {
    keys[start + j] = s_a[j] + lo;
    vals[start + j] = s_b[j];
    if (MORE) more[start + j] = s_c[j];
  }
}

}  // namespace

bool bucket_sort_fits(int64_t expected, uint32_t sentinel) {
  // an even spread must leave the buckets a fifth of their capacity to spare
  return expected >= (1 << 16) && expected <= (int64_t)((1 << kBktDigitBits) - 1) * (kBktCap * 4 / 5) &&
         sentinel >= (1u << 20);
}

int bucket_sort_pairs(uint32_t *keys_a, uint32_t *vals_a, uint32_t *keys_b, uint32_t *vals_b, int64_t max_count,
                      const uint32_t *count_dev, uint32_t sentinel, void *scratch, int32_t *status,
                      hipStream_t stream, uint32_t *more_a, uint32_t *more_b) {
  if (max_count < 1 || max_count > 0x7fffffffll || sentinel < (1u << 20))
    return fail(ZEN_EINVAL, "bucket_sort_pairs: size out of range");
  const int nblk = num_tiles(max_count);
  Carver cv(scratch);
  uint32_t *hist = cv.take<uint32_t>((size_t)nblk * kMaxRadix);
  uint32_t *totals = cv.take<uint32_t>(kMaxRadix);
  DigitRange digit;
  digit.last = (1u << kBktDigitBits) - 1u;
  digit.sentinel = sentinel;
  digit.mult = (uint32_t)((((uint64_t)digit.last) << 32) / sentinel);
  const uint64_t width = ((1ull << 32) + digit.mult - 1) / digit.mult + 1;  // keys per bucket, at most
  static_assert(kBktCap <= (1 << 14), "arrival positions are packed into 14 bits");
  const int width_bits = ceil_log2_u64(width);  // at most 24 (mult >= 511), so sub_shift + 14 fits a word
  const int sub_shift = width_bits > 13 ? width_bits - 13 : 0;
  const int rc = sort_pass<kBktDigitBits>(keys_a, vals_a, more_a, keys_b, vals_b, more_b, max_count, count_dev, digit,
                                          nblk, hist, totals, stream);
  if (rc != ZEN_OK) return rc;
  if (more_a)
    k_bucket_sort<true><<<dim3(digit.last), dim3(kBktBlock), 0, stream>>>(keys_b, vals_b, more_b, totals, digit,
                                                                          sub_shift, status);
  else
    k_bucket_sort<false><<<dim3(digit.last), dim3(kBktBlock), 0, stream>>>(keys_b, vals_b, nullptr, totals, digit,
                                                                           sub_shift, status);
  ZEN_LAUNCH_CHECK("k_bucket_sort");
  return 1;
}


}  // namespace zen

extern "C" {

int zen_abi_version(void) { return ZEN_ABI_VERSION; }

const char *zen_last_error(void) { return zen::g_last_error; }

size_t zen_sort_pairs_workspace(int64_t max_count) {
  if (max_count < 0) return 0;
  return 2 * zen::align_up((size_t)max_count * sizeof(uint32_t), 256) + zen::sort_scratch_bytes(max_count);
}

int zen_sort_pairs(uint32_t *keys, uint32_t *vals, int64_t max_count, const uint32_t *count_dev,
                   int bits, void *workspace, size_t workspace_bytes, int32_t *status, void *stream) {
  using namespace zen;
  if (max_count == 0) return ZEN_OK;
  if (!keys || !vals || !workspace || !status) return fail(ZEN_EINVAL, "zen_sort_pairs: null pointer");
  if (workspace_bytes < zen_sort_pairs_workspace(max_count))
    return fail(ZEN_EWORKSPACE, "zen_sort_pairs: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  Carver cv(workspace);
  uint32_t *kb = cv.take<uint32_t>((size_t)max_count);
  uint32_t *vb = cv.take<uint32_t>((size_t)max_count);
  void *scratch = cv.take<char>(sort_scratch_bytes(max_count));
  const int where = sort_pairs(keys, vals, kb, vb, max_count, count_dev, bits, scratch, status, s);
  if (where < 0) return where;
  if (where == 1) {
    const int64_t blocks = ceil_div(max_count, 1024);
    k_copy_pairs<<<dim3((unsigned)(blocks < 2048 ? blocks : 2048)), dim3(256), 0, s>>>(
        kb, vb, keys, vals, count_dev, (uint32_t)max_count);
    ZEN_LAUNCH_CHECK("k_copy_pairs");
  }
  return ZEN_OK;
}

int zen_bucket_sort_fits(int64_t max_count, uint32_t sentinel) { return zen::bucket_sort_fits(max_count, sentinel); }

int zen_bucket_sort_pairs(uint32_t *keys, uint32_t *vals, int64_t max_count, const uint32_t *count_dev,
                          uint32_t sentinel, void *workspace, size_t workspace_bytes, int32_t *status,
                          void *stream) {
  using namespace zen;
  if (!keys || !vals || !workspace || !status) return fail(ZEN_EINVAL, "zen_bucket_sort_pairs: null pointer");
  if (!bucket_sort_fits(max_count, sentinel)) return fail(ZEN_EINVAL, "zen_bucket_sort_pairs: size out of range");
  if (workspace_bytes < zen_sort_pairs_workspace(max_count))
    return fail(ZEN_EWORKSPACE, "zen_bucket_sort_pairs: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  Carver cv(workspace);
  uint32_t *kb = cv.take<uint32_t>((size_t)max_count);
  uint32_t *vb = cv.take<uint32_t>((size_t)max_count);
  void *scratch = cv.take<char>(sort_scratch_bytes(max_count));
  const int where = bucket_sort_pairs(keys, vals, kb, vb, max_count, count_dev, sentinel, scratch, status, s);
  if (where < 0) return where;
  const int64_t blocks = ceil_div(max_count, 1024);
  k_copy_pairs<<<dim3((unsigned)(blocks < 2048 ? blocks : 2048)), dim3(256), 0, s>>>(kb, vb, keys, vals, count_dev,
                                                                                     (uint32_t)max_count);
  ZEN_LAUNCH_CHECK("k_copy_pairs");
  return ZEN_OK;
}

}  // extern "C"
