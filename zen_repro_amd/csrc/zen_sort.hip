// Stable LSD radix sort of (uint32 key, uint32 value) pairs, 8-bit digits.
// Three kernels per digit: per-tile histogram, scan, stable scatter.  The
// scatter ranks its tile in LDS (wave ballots + per-wave digit counters),
// reorders the tile in LDS and writes every digit's run with consecutive lanes,
// so global stores are contiguous runs instead of 4-byte scatters.  The element
// count may live on the device, so grids are sized by the capacity and surplus
// tiles retire immediately.
#include "zen_common.h"

namespace zen {

thread_local char g_last_error[256] = "";

namespace {

constexpr int kSortBlock = 256;
constexpr int kSortItems = 16;                       // keys per thread
constexpr int kSortTile = kSortBlock * kSortItems;   // 4096 keys per tile
constexpr int kWaveSpan = 64 * kSortItems;           // contiguous keys owned by one wave
constexpr int kRadix = 256;
constexpr int kMaxPasses = 4;

__device__ inline uint32_t live_count(const uint32_t *count_dev, uint32_t count_imm) {
  return count_dev ? *count_dev : count_imm;
}

// hist[d * nblk + tile] = number of keys of this tile whose digit is d
__global__ __launch_bounds__(kSortBlock) void k_sort_hist(const uint32_t *__restrict__ keys,
                                                          const uint32_t *count_dev, uint32_t count_imm,
                                                          int shift, uint32_t mask, int nblk,
                                                          uint32_t *__restrict__ hist) {
  __shared__ uint32_t bins[kRadix];
  const uint32_t count = live_count(count_dev, count_imm);
  const uint32_t base = blockIdx.x * (uint32_t)kSortTile;
  bins[threadIdx.x] = 0;
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
      if (wave_base + i * 64 < count) atomicAdd(&bins[(k[i] >> shift) & mask], 1u);
  }
  __syncthreads();
  hist[(size_t)threadIdx.x * nblk + blockIdx.x] = bins[threadIdx.x];
}

// One block per digit (taken in ticket order): the digit's total goes through
// the tile-prefix protocol to give the sum of all lower digits, then the row of
// per-tile counts becomes per-tile global start offsets.
__global__ __launch_bounds__(kSortBlock) void k_sort_scan(uint32_t *__restrict__ hist, int nblk, ScanState st,
                                                          int32_t *status) {
  __shared__ uint32_t smem[kSortBlock / 64 + 1];
  __shared__ uint64_t s_bcast;
  __shared__ int s_digit;
  if (threadIdx.x == 0) s_digit = (int)atomicAdd(st.ticket, 1u);
  __syncthreads();
  const int d = s_digit;
  uint32_t *row = hist + (size_t)d * nblk;
  uint32_t mine = 0;
  for (int b = threadIdx.x; b < nblk; b += kSortBlock) mine += row[b];
  uint32_t row_total;
  block_exclusive_scan<uint32_t, kSortBlock>(mine, smem, &row_total);
  uint32_t running = (uint32_t)lookback_exclusive(st, d, row_total, status, &s_bcast);
  for (int b0 = 0; b0 < nblk; b0 += kSortBlock) {
    const int b = b0 + threadIdx.x;
    const uint32_t v = b < nblk ? row[b] : 0u;
    uint32_t chunk;
    const uint32_t ex = block_exclusive_scan<uint32_t, kSortBlock>(v, smem, &chunk);
    if (b < nblk) row[b] = running + ex;
    running += chunk;
  }
}

__global__ __launch_bounds__(kSortBlock) void k_sort_scatter(
    const uint32_t *__restrict__ keys_in, const uint32_t *__restrict__ vals_in,
    const uint32_t *__restrict__ more_in, uint32_t *__restrict__ keys_out, uint32_t *__restrict__ vals_out,
    uint32_t *__restrict__ more_out, const uint32_t *count_dev,
    uint32_t count_imm, int shift, uint32_t mask, int nblk, const uint32_t *__restrict__ offsets) {
  __shared__ uint32_t wcnt[kSortBlock / 64][kRadix];  // per wave: count, then start inside the tile
  __shared__ uint32_t gshift[kRadix];                 // global position = gshift[digit] + position in the tile
  __shared__ uint32_t smem[kSortBlock / 64 + 1];
  __shared__ uint32_t skey[kSortTile];
  __shared__ uint32_t sval[kSortTile];
  const uint32_t count = live_count(count_dev, count_imm);
  const uint32_t base = blockIdx.x * (uint32_t)kSortTile;
  if (base >= count) return;
  const uint32_t tile_count = count - base < (uint32_t)kSortTile ? count - base : (uint32_t)kSortTile;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int w = 0; w < kSortBlock / 64; ++w) wcnt[w][threadIdx.x] = 0;
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
    const uint32_t d = (key[i] >> shift) & mask;
    // lanes of this wave holding the same digit
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
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
    // thread = digit: start of the digit inside the tile, then one start per wave
    uint32_t c[kSortBlock / 64];
    uint32_t total = 0;
#pragma unroll
    for (int w = 0; w < kSortBlock / 64; ++w) {
      c[w] = wcnt[w][threadIdx.x];
      total += c[w];
    }
    uint32_t unused;
    uint32_t running = block_exclusive_scan<uint32_t, kSortBlock>(total, smem, &unused);
    gshift[threadIdx.x] = offsets[(size_t)threadIdx.x * nblk + blockIdx.x] - running;
#pragma unroll
    for (int w = 0; w < kSortBlock / 64; ++w) {
      wcnt[w][threadIdx.x] = running;
      running += c[w];
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    const uint32_t at = wave_base + i * 64;
    if (at < count) {
      const uint32_t pos = wcnt[wave][(key[i] >> shift) & mask] + rank[i];
      skey[pos] = key[i];
      sval[pos] = vals_in[at];
    }
  }
  __syncthreads();
  for (uint32_t j = threadIdx.x; j < tile_count; j += kSortBlock) {
    const uint32_t k = skey[j];
    const uint32_t g = gshift[(k >> shift) & mask] + j;
    keys_out[g] = k;
    vals_out[g] = sval[j];
  }
  if (!more_in) return;
  // a second payload travels through the same LDS buffer in a second round
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    const uint32_t at = wave_base + i * 64;
    if (at < count) sval[wcnt[wave][(key[i] >> shift) & mask] + rank[i]] = more_in[at];
  }
  __syncthreads();
  for (uint32_t j = threadIdx.x; j < tile_count; j += kSortBlock)
    more_out[gshift[(skey[j] >> shift) & mask] + j] = sval[j];
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
  return align_up(nblk * kRadix * sizeof(uint32_t), 256) +
         align_up(kMaxPasses * scan_words(kRadix) * sizeof(unsigned long long), 256);
}

int sort_pairs(uint32_t *keys_a, uint32_t *vals_a, uint32_t *keys_b, uint32_t *vals_b,
               int64_t max_count, const uint32_t *count_dev, int bits, void *scratch, int32_t *status,
               hipStream_t stream, uint32_t *more_a, uint32_t *more_b) {
  if (max_count < 0 || max_count > 0x7fffffffll || bits < 0 || bits > 32)
    return fail(ZEN_EINVAL, "sort_pairs: bad count or bits");
  if (max_count == 0 || bits == 0) return 0;
  const int nblk = num_tiles(max_count);
  Carver cv(scratch);
  uint32_t *hist = cv.take<uint32_t>((size_t)nblk * kRadix);
  unsigned long long *scan = cv.take<unsigned long long>(kMaxPasses * scan_words(kRadix));
  launch_fill<unsigned long long>(scan, 0ull, kMaxPasses * scan_words(kRadix), stream);
  ZEN_LAUNCH_CHECK("sort: clear scan state");
  const int passes = (bits + 7) / 8;
  uint32_t *ks = keys_a, *vs = vals_a, *kd = keys_b, *vd = vals_b, *ms = more_a, *md = more_b;
  for (int p = 0; p < passes; ++p) {
    const int shift = p * 8;
    const int width = bits - shift < 8 ? bits - shift : 8;
    const uint32_t mask = (1u << width) - 1u;
    k_sort_hist<<<dim3(nblk), dim3(kSortBlock), 0, stream>>>(ks, count_dev, (uint32_t)max_count, shift, mask, nblk,
                                                             hist);
    ZEN_LAUNCH_CHECK("k_sort_hist");
    k_sort_scan<<<dim3(kRadix), dim3(kSortBlock), 0, stream>>>(
        hist, nblk, scan_state(scan + (size_t)p * scan_words(kRadix), kRadix), status);
    ZEN_LAUNCH_CHECK("k_sort_scan");
    k_sort_scatter<<<dim3(nblk), dim3(kSortBlock), 0, stream>>>(ks, vs, ms, kd, vd, md, count_dev,
                                                                (uint32_t)max_count, shift, mask, nblk, hist);
    ZEN_LAUNCH_CHECK("k_sort_scatter");
    uint32_t *t = ks; ks = kd; kd = t;
    t = vs; vs = vd; vd = t;
    t = ms; ms = md; md = t;
  }
  return passes & 1;
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

}  // extern "C"
