#include "zen_binsort.h"

namespace zen {
namespace {

__device__ inline uint32_t live_count(const uint32_t *count_dev, uint32_t count_imm) {
  if (!count_dev) return count_imm;
  const uint32_t c = *count_dev;
  return c < count_imm ? c : count_imm;
}

// Exclusive prefix of the bin histogram in one pass (look-back over tiles).
__global__ __launch_bounds__(kBsScanBlock) void k_bs_scan(const uint32_t *__restrict__ hist, uint32_t nbins,
                                                          uint32_t *__restrict__ start, uint32_t *__restrict__ cursor,
                                                          ScanState st, int ntiles,
                                                          uint32_t *retry, int32_t *status) {
  __shared__ uint32_t s_scan[kBsScanBlock / 64 + 1];
  __shared__ uint64_t s_bcast;
  __shared__ int s_tile;
  if (threadIdx.x == 0) s_tile = (int)atomicAdd(st.ticket, 1u);
  __syncthreads();
  const int tile = s_tile;
  if (tile >= ntiles) return;
  const uint32_t first = (uint32_t)tile * kBsScanTile + threadIdx.x * kBsScanItems;
  uint32_t c[kBsScanItems];
  uint32_t mine = 0, biggest = 0;
#pragma unroll
  for (int i = 0; i < kBsScanItems; ++i) {
    c[i] = first + i < nbins ? hist[first + i] : 0u;
    mine += c[i];
    biggest = c[i] > biggest ? c[i] : biggest;
  }
  if (biggest > kBinLimit) *retry = 1u;
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kBsScanBlock>(mine, s_scan, &total);
  const uint64_t tile_start = lookback_exclusive(st, tile, total, status, &s_bcast);
  uint32_t run = (uint32_t)tile_start + before;
#pragma unroll
  for (int i = 0; i < kBsScanItems; ++i) {
    if (first + i < nbins) {
      start[first + i] = run;
      cursor[first + i] = run;
    }
    run += c[i];
  }
  if (tile == ntiles - 1 && threadIdx.x == kBsScanBlock - 1) start[nbins] = run;
}

__global__ __launch_bounds__(256) void k_bs_scatter(const uint32_t *__restrict__ keys, const uint32_t *__restrict__ vals,
                                                    const uint32_t *count_dev, uint32_t count_imm, int bshift,
                                                    uint32_t *cursor, const uint32_t *retry,
                                                    uint32_t *__restrict__ tmp_keys, uint32_t *__restrict__ tmp_vals) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= live_count(count_dev, count_imm) || *retry) return;
  const uint32_t k = keys[i];
  const uint32_t pos = atomicAdd(&cursor[k >> bshift], 1u);
  tmp_keys[pos] = k;
  tmp_vals[pos] = vals ? vals[i] : i;
}

__global__ __launch_bounds__(256) void k_bs_rank(const uint32_t *__restrict__ tmp_keys, const uint32_t *__restrict__ tmp_vals,
                                                 const uint32_t *count_dev, uint32_t count_imm, int bshift,
                                                 const uint32_t *__restrict__ start, const uint32_t *retry,
                                                 uint32_t *__restrict__ out_keys, uint32_t *__restrict__ out_vals) {
  const uint32_t p = blockIdx.x * 256u + threadIdx.x;
  if (p >= live_count(count_dev, count_imm) || *retry) return;
  const uint32_t k = tmp_keys[p], v = tmp_vals[p];
  const uint32_t b = k >> bshift;
  const uint32_t lo = start[b], hi = start[b + 1];
  uint32_t rank = 0;
  for (uint32_t q = lo; q < hi; ++q) {
    const uint32_t kq = tmp_keys[q];
    rank += (kq < k) || (kq == k && tmp_vals[q] < v);
  }
  out_keys[lo + rank] = k;
  out_vals[lo + rank] = v;
}

}  // namespace

BinSort plan_binsort(void *scratch, uint64_t key_limit, int64_t expected, size_t extra_zero_bytes) {
  BinSort bs;
  // aim at ~8 entries per bin, never more than 2^21 bins
  int bshift = 0;
  const uint64_t want_bins = (uint64_t)(expected > 8 ? expected / 8 : 1);
  while (bshift < 31 && ((key_limit >> bshift) > want_bins || (key_limit >> bshift) > (1ull << 21))) ++bshift;
  bs.bshift = bshift;
  bs.nbins = (uint32_t)(((key_limit - 1) >> bshift) + 1);
  bs.scan_tiles = (int)ceil_div((int64_t)bs.nbins, kBsScanTile);
  Carver cv(scratch);
  bs.hist = cv.take<uint32_t>(bs.nbins);
  bs.desc = cv.take<unsigned long long>(scan_words(bs.scan_tiles));
  bs.retry = cv.take<uint32_t>(1);
  bs.extra = cv.take<char>(extra_zero_bytes);
  bs.zero_begin = bs.hist;
  bs.zero_bytes = cv.used;
  bs.start = cv.take<uint32_t>((size_t)bs.nbins + 1);
  bs.cursor = cv.take<uint32_t>(bs.nbins);
  bs.bytes = cv.used;
  return bs;
}

int binsort_clear(const BinSort &bs, hipStream_t stream) {
  launch_fill<uint32_t>(static_cast<uint32_t *>(bs.zero_begin), 0u, bs.zero_bytes / sizeof(uint32_t), stream);
  ZEN_LAUNCH_CHECK("binsort: clear");
  return ZEN_OK;
}

int binsort_scan(const BinSort &bs, int32_t *status, hipStream_t stream) {
  k_bs_scan<<<dim3((unsigned)bs.scan_tiles), dim3(kBsScanBlock), 0, stream>>>(bs.hist, bs.nbins, bs.start, bs.cursor,
                                                                            scan_state(bs.desc, bs.scan_tiles), bs.scan_tiles, bs.retry,
                                                                            status);
  ZEN_LAUNCH_CHECK("k_bs_scan");
  return ZEN_OK;
}

int binsort_scatter(const BinSort &bs, const uint32_t *keys, const uint32_t *vals, int64_t max_count,
                    const uint32_t *count_dev, uint32_t *tmp_keys, uint32_t *tmp_vals, hipStream_t stream) {
  k_bs_scatter<<<dim3((unsigned)ceil_div(max_count, 256)), dim3(256), 0, stream>>>(
      keys, vals, count_dev, (uint32_t)max_count, bs.bshift, bs.cursor, bs.retry, tmp_keys, tmp_vals);
  ZEN_LAUNCH_CHECK("k_bs_scatter");
  return ZEN_OK;
}

int binsort_rank(const BinSort &bs, const uint32_t *tmp_keys, const uint32_t *tmp_vals, int64_t max_count,
                 const uint32_t *count_dev, uint32_t *out_keys, uint32_t *out_vals, hipStream_t stream) {
  k_bs_rank<<<dim3((unsigned)ceil_div(max_count, 256)), dim3(256), 0, stream>>>(
      tmp_keys, tmp_vals, count_dev, (uint32_t)max_count, bs.bshift, bs.start, bs.retry, out_keys, out_vals);
  ZEN_LAUNCH_CHECK("k_bs_rank");
  return ZEN_OK;
}

}  // namespace zen
