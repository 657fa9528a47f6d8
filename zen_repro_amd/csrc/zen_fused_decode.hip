// Second half of the sparse all-reduce with bitmaps, in one pass: every rank's bitmap over its partition's
// member list and its value list go straight into the dense gradient.  The reference turns each bitmap back
// into int64 indices by masking the cached member list (comm.py:87-99, 136-141) and scatter-adds all
// (index, value) lists into a zeroed dense tensor (comm.py:142-145, 32-44).  Neither the indices nor the
// member lists are needed for that: which partition an index belongs to is a hash away, and bit j of
// partition p's bitmap stands for the j-th index of that partition.  So the dense tensor is cut into tiles of
// 8192 indices; a dictionary built once per (numel, partitions) holds the partition id of every index (one
// byte) and, per partition and tile, how many members lie below the tile; a call first counts, per tile and
// partition, the set bits of the tile's bit range (which gives where the tile's values start in every value
// list), and then one workgroup per tile ranks its indices inside their partitions, looks their bits up and
// writes the tile once, zeros included: the dense tensor is never cleared and nothing is scattered.
#include "zen_common.h"

namespace zen {
namespace {

constexpr int kFdTile = 8192;
constexpr int kFdBlock = 512;
constexpr int kFdPer = kFdTile / kFdBlock;   // consecutive indices per thread (16)
constexpr int kFdMaxLists = 64;
constexpr int kFdChunk = 16;                  // thread columns whose counts one thread adds up
constexpr int kFdChunks = kFdBlock / kFdChunk;
constexpr int kFdMaxBytes = kFdTile / 8 + 2 * kFdMaxLists;  // bitmap bytes a tile's bit ranges can span
static_assert(kFdChunks == 32, "a wave's lower half scans the chunk sums");

struct ListStarts {
  int64_t at[kFdMaxLists + 1];
};

__device__ inline uint32_t part_of(uint32_t t, uint32_t n, uint32_t npp) {
  return ((poly(t) + kSeed1) % n) / npp;  // functions_cuda_kernel.cu:172-175
}

// Dictionary, step 1: partition id of every index, and per tile the number of indices of every partition.
__global__ __launch_bounds__(kFdBlock) void k_fd_parts(uint32_t n, uint32_t npp, int P, uint8_t *__restrict__ part,
                                                      uint32_t *__restrict__ below) {
  __shared__ uint32_t s_cnt[kFdMaxLists];
  if (threadIdx.x < kFdMaxLists) s_cnt[threadIdx.x] = 0;
  __syncthreads();
  const uint32_t base = blockIdx.x * (uint32_t)kFdTile + threadIdx.x * (uint32_t)kFdPer;
  uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
  for (int e = 0; e < kFdPer; ++e) {
    uint32_t p = 0xffu;
    if (base + e < n) {
      p = part_of(base + e, n, npp);
      if (p < (uint32_t)P) atomicAdd(&s_cnt[p], 1u);
    }
    w[e >> 2] |= p << (8 * (e & 3));
  }
  if (base + kFdPer <= n) {
    *reinterpret_cast<uint4 *>(part + base) = make_uint4(w[0], w[1], w[2], w[3]);
  } else {
    for (int e = 0; e < kFdPer && base + e < n; ++e) part[base + e] = (uint8_t)(w[e >> 2] >> (8 * (e & 3)));
  }
  __syncthreads();
  if (threadIdx.x < P) below[(size_t)threadIdx.x * (gridDim.x + 1) + blockIdx.x] = s_cnt[threadIdx.x];
}

// Per list (blockIdx.x): exclusive prefix over the tiles of a [P][tiles + 1] table of counts, in place; the last
// entry of a row receives the total.  A thread takes eight consecutive entries per round (two 16-byte loads),
// a round covers 8192 of them.
constexpr int kFdScanBlock = 1024;
constexpr int kFdScanPer = 8;
__global__ __launch_bounds__(kFdScanBlock) void k_fd_scan(uint32_t *__restrict__ table, uint32_t tiles) {
  __shared__ uint32_t s_scan[kFdScanBlock / 64 + 1];
  uint32_t *row = table + (size_t)blockIdx.x * (tiles + 1);
  uint32_t carry = 0;
  for (uint32_t base = 0; base < tiles; base += kFdScanBlock * kFdScanPer) {
    const uint32_t first = base + threadIdx.x * kFdScanPer;
    uint32_t c[kFdScanPer], sum = 0;
#pragma unroll
    for (int j = 0; j < kFdScanPer; ++j) {
      c[j] = first + j < tiles ? row[first + j] : 0u;
      sum += c[j];
    }
    uint32_t total;
    uint32_t running = carry + block_exclusive_scan<uint32_t, kFdScanBlock>(sum, s_scan, &total);
#pragma unroll
    for (int j = 0; j < kFdScanPer; ++j) {
      if (first + j < tiles) row[first + j] = running;
      running += c[j];
    }
    carry += total;
  }
  if (threadIdx.x == 0) row[tiles] = carry;
}

// Set bits of bitmap `bm` in the bit range [b0, b1); bytes at or beyond `bytes` count as zero.
__device__ inline uint32_t popcount_range(const uint8_t *__restrict__ bm, int64_t bytes, uint32_t b0, uint32_t b1) {
  if (b1 <= b0) return 0;
  uint32_t first = b0 >> 3, last = (b1 - 1) >> 3;  // bytes first..last
  if ((int64_t)first >= bytes) return 0;
  if ((int64_t)last >= bytes) {
    last = (uint32_t)(bytes - 1);
    b1 = (last + 1u) << 3;
  }
  const uint32_t head_mask = 0xffu << (b0 & 7u);
  const uint32_t tail_mask = 0xffu >> (7u - ((b1 - 1u) & 7u));
  if (first == last) return (uint32_t)__popc(bm[first] & head_mask & tail_mask);
  uint32_t c = (uint32_t)__popc(bm[first] & head_mask) + (uint32_t)__popc(bm[last] & tail_mask);
  uint32_t i = first + 1;
  while (i < last && ((reinterpret_cast<uintptr_t>(bm) + i) & 7u)) c += (uint32_t)__popc(bm[i++]);
  for (; i + 8 <= last; i += 8) c += (uint32_t)__popcll(*reinterpret_cast<const unsigned long long *>(bm + i));
  for (; i < last; ++i) c += (uint32_t)__popc(bm[i]);
  return c;
}

// Per (tile, list): set bits in the tile's bit range of the list's bitmap.  A bitmap shorter than its list
// (the reference's mask would not fit the member list, comm.py:97-98) raises ZEN_STAT_BAD_INDEX.
__global__ __launch_bounds__(256) void k_fd_count(const uint32_t *__restrict__ below, uint32_t tiles, int P,
                                                  const uint8_t *__restrict__ bitmaps, ListStarts bm,
                                                  uint32_t *__restrict__ vstart, int32_t *status) {
  const uint32_t tile = blockIdx.x * 256u + threadIdx.x;
  const int p = blockIdx.y;
  if (tile >= tiles) return;
  const size_t i = (size_t)p * (tiles + 1) + tile;
  const uint32_t b0 = below[i], b1 = below[i + 1];
  const int64_t bytes = bm.at[p + 1] - bm.at[p];
  if (tile == tiles - 1 && ((int64_t)b1 + 7) / 8 > bytes) atomicOr(status, ZEN_STAT_BAD_INDEX);
  vstart[i] = popcount_range(bitmaps + bm.at[p], bytes, b0, b1);
}

template <typename S>
__device__ inline S fd_value(S v);  // what a zeroed element holds after one scatter_add_ of v (comm.py:35-39)
template <>
__device__ inline uint16_t fd_value<uint16_t>(uint16_t v) {
  return f32_to_bf16_rne(0.0f + KeyOf<uint16_t>::to_f32(v));
}
template <>
__device__ inline uint32_t fd_value<uint32_t>(uint32_t v) {
  return __float_as_uint(0.0f + __uint_as_float(v));
}

// One workgroup per tile.  Dynamic LDS: P * kFdBlock 16-bit counters.
template <typename S>
__global__ __launch_bounds__(kFdBlock) void k_fd_tiles(const uint8_t *__restrict__ part, const uint32_t *__restrict__ below,
                                                      const uint32_t *__restrict__ vstart, int P, uint32_t n,
                                                      const uint8_t *__restrict__ bitmaps, ListStarts bm,
                                                      const S *__restrict__ values, ListStarts vs,
                                                      S *__restrict__ dense, int32_t *status) {
  extern __shared__ uint16_t s_cnt[];                 // [P][kFdBlock]: indices of list p in lower threads' stretches
  __shared__ uint16_t s_chunk[kFdMaxLists][kFdChunks + 1];  // per list: the same over chunks of 16 threads; [32] = the tile's total
  __shared__ uint2 s_meta[kFdMaxLists];               // per list: first bit of the tile's range; where its bytes start in s_byte
  __shared__ uint32_t s_vbase[kFdMaxLists];           // per list: value number of the range's first bit, minus the
                                                      // set bits in front of it inside s_byte
  __shared__ uint8_t s_byte[kFdMaxBytes + 8];
  __shared__ uint16_t s_bpre[kFdMaxBytes + 8];        // set bits in the bytes before, over all of s_byte
  __shared__ uint32_t s_scan[kFdBlock / 64 + 1];
  __shared__ uint32_t s_nbytes;
  // the lists' offsets, looked up by list number further down: in LDS, because a kernel argument indexed with a
  // number that differs from lane to lane is fetched from memory, one round trip per look
  __shared__ int64_t s_bm[kFdMaxLists + 1], s_vs[kFdMaxLists + 1];
  if (threadIdx.x <= (uint32_t)P) {
    s_bm[threadIdx.x] = bm.at[threadIdx.x];
    s_vs[threadIdx.x] = vs.at[threadIdx.x];
  }
  const uint32_t tile = blockIdx.x;
  const uint32_t base = tile * (uint32_t)kFdTile + threadIdx.x * (uint32_t)kFdPer;
  // the thread's 16 partition ids (0xff: past the end of the tensor)
  uint32_t w[4];
  if (base + kFdPer <= n) {
    const uint4 q = *reinterpret_cast<const uint4 *>(part + base);
    w[0] = q.x; w[1] = q.y; w[2] = q.z; w[3] = q.w;
  } else {
    w[0] = w[1] = w[2] = w[3] = 0xffffffffu;
    for (int e = 0; e < kFdPer && base + e < n; ++e)
      w[e >> 2] = (w[e >> 2] & ~(0xffu << (8 * (e & 3)))) | ((uint32_t)part[base + e] << (8 * (e & 3)));
  }
  {
    uint32_t *z = reinterpret_cast<uint32_t *>(s_cnt);
    for (int i = threadIdx.x; i < P * kFdBlock / 2; i += kFdBlock) z[i] = 0;
  }
  __syncthreads();
  // rank of each index among the thread's own indices of the same list (its column of counters is private)
  uint64_t ranks = 0;  // 4 bits each
#pragma unroll
  for (int e = 0; e < kFdPer; ++e) {
    const uint32_t p = (w[e >> 2] >> (8 * (e & 3))) & 0xffu;
    if (p < (uint32_t)P) {
      const uint32_t c = s_cnt[p * kFdBlock + threadIdx.x];
      s_cnt[p * kFdBlock + threadIdx.x] = (uint16_t)(c + 1u);
      ranks |= (uint64_t)c << (4 * e);
    }
  }
  __syncthreads();
  // per list: exclusive prefix over the thread columns, in two levels (chunks of 16 columns, then the 32 chunks)
  for (int q = threadIdx.x; q < P * kFdChunks; q += kFdBlock) {
    const int p = q / kFdChunks, c = q % kFdChunks;
    uint16_t *col = s_cnt + p * kFdBlock + c * kFdChunk;
    uint32_t run = 0;
#pragma unroll
    for (int i = 0; i < kFdChunk; ++i) {
      const uint32_t x = col[i];
      col[i] = (uint16_t)run;
      run += x;
    }
    s_chunk[p][c] = (uint16_t)run;
  }
  __syncthreads();
  for (int p = threadIdx.x >> 6; p < P; p += kFdBlock / 64) {
    const int lane = lane_id();
    const uint32_t x = lane < kFdChunks ? s_chunk[p][lane] : 0u;
    const uint32_t incl = wave_inclusive_scan(x);
    if (lane < kFdChunks) s_chunk[p][lane] = (uint16_t)(incl - x);
    if (lane == kFdChunks - 1) s_chunk[p][kFdChunks] = (uint16_t)incl;
  }
  __syncthreads();
  // the bytes of every list's bit range, side by side in s_byte
  if (threadIdx.x < 64) {
    const int p = threadIdx.x;
    uint32_t b0 = 0, nb = 0;
    if (p < P) {
      b0 = below[(size_t)p * (gridDim.x + 1) + tile];
      const uint32_t cnt = s_chunk[p][kFdChunks];
      nb = cnt ? ((b0 + cnt - 1u) >> 3) - (b0 >> 3) + 1u : 0u;
    }
    const uint32_t incl = wave_inclusive_scan(nb);
    if (p < P) s_meta[p] = make_uint2(b0, incl - nb);
    if (p == 63) s_nbytes = incl;
  }
  __syncthreads();
  {
    // byte i of s_byte belongs to the list whose stretch it falls into (the stretches' starts ascend): found by
    // bisection, so that every thread fetches its bytes in one go instead of list after list
    const uint32_t total_bytes = s_nbytes;
    for (uint32_t i = threadIdx.x; i < total_bytes; i += kFdBlock) {
      int lo = 0, hi = P - 1;  // the last list whose stretch starts at or before i
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (s_meta[mid].y <= i) lo = mid; else hi = mid - 1;
      }
      const uint2 m = s_meta[lo];
      const int64_t g = (int64_t)(m.x >> 3) + (i - m.y);
      const int64_t bytes = s_bm[lo + 1] - s_bm[lo];
      s_byte[i] = g < bytes ? bitmaps[s_bm[lo] + g] : (uint8_t)0;  // a short bitmap was flagged by the count kernel
    }
  }
  __syncthreads();
  {
    constexpr int kPer = (kFdMaxBytes + kFdBlock - 1) / kFdBlock;  // 3
    const uint32_t total_bytes = s_nbytes;
    uint32_t c[kPer], sum = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const uint32_t i = threadIdx.x * kPer + j;
      c[j] = i < total_bytes ? (uint32_t)__popc(s_byte[i]) : 0u;
      sum += c[j];
    }
    uint32_t total;
    uint32_t run = block_exclusive_scan<uint32_t, kFdBlock>(sum, s_scan, &total);
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const uint32_t i = threadIdx.x * kPer + j;
      if (i < kFdMaxBytes + 8) s_bpre[i] = (uint16_t)run;
      run += c[j];
    }
  }
  __syncthreads();
  if (threadIdx.x < P) {
    const int p = threadIdx.x;
    const uint2 m = s_meta[p];
    const uint32_t front = s_bpre[m.y] + (uint32_t)__popc(s_byte[m.y] & ((1u << (m.x & 7u)) - 1u));
    s_vbase[p] = vstart[(size_t)p * (gridDim.x + 1) + tile] - front;  // unsigned wrap-around undone when a position is added
  }
  __syncthreads();
  // every index: its place among its list's members, its bit, and if that is set where its value is.  The
  // values are then fetched all at once, outside any branch (an unset index fetches the first value of all):
  // one round trip to memory instead of one per index.
  const int64_t first_value = s_vs[0], all_values = s_vs[P] - first_value;
  int64_t from[kFdPer];
  uint32_t set = 0;
  bool bad = false;
#pragma unroll
  for (int e = 0; e < kFdPer; ++e) {
    from[e] = first_value;
    const uint32_t p = (w[e >> 2] >> (8 * (e & 3))) & 0xffu;
    if (p < (uint32_t)P) {
      const uint32_t j = (uint32_t)s_chunk[p][threadIdx.x / kFdChunk] + s_cnt[p * kFdBlock + threadIdx.x] +
                         (uint32_t)((ranks >> (4 * e)) & 15u);
      const uint2 m = s_meta[p];
      const uint32_t bit = m.x + j;
      const uint32_t at = m.y + (bit >> 3) - (m.x >> 3);
      const uint32_t byte = s_byte[at];
      if ((byte >> (bit & 7u)) & 1u) {
        const uint32_t v = s_vbase[p] + s_bpre[at] + (uint32_t)__popc(byte & ((1u << (bit & 7u)) - 1u));
        const int64_t v0 = s_vs[p];
        if ((int64_t)v < s_vs[p + 1] - v0) {
          from[e] = v0 + v;
          set |= 1u << e;
        } else {
          bad = true;  // more set bits than values
        }
      }
    }
  }
  S got[kFdPer];
#pragma unroll
  for (int e = 0; e < kFdPer; ++e) got[e] = all_values > 0 ? values[from[e]] : (S)0;
  uint32_t out[kFdPer * sizeof(S) / 4];
#pragma unroll
  for (int i = 0; i < (int)(kFdPer * sizeof(S) / 4); ++i) out[i] = 0;
#pragma unroll
  for (int e = 0; e < kFdPer; ++e) {
    const S val = (set >> e) & 1u ? fd_value<S>(got[e]) : (S)0;
    if (sizeof(S) == 2)
      out[e >> 1] |= (uint32_t)val << (16 * (e & 1));
    else
      out[e] = (uint32_t)val;
  }
  if (bad) atomicOr(status, ZEN_STAT_BAD_INDEX);
  if (base + kFdPer <= n && (reinterpret_cast<uintptr_t>(dense) & 15u) == 0) {
    uint4 *dst = reinterpret_cast<uint4 *>(dense + base);
#pragma unroll
    for (int i = 0; i < (int)(kFdPer * sizeof(S) / 16); ++i) dst[i] = make_uint4(out[4 * i], out[4 * i + 1], out[4 * i + 2], out[4 * i + 3]);
  } else {
    for (int e = 0; e < kFdPer && base + e < n; ++e)
      dense[base + e] = sizeof(S) == 2 ? (S)(out[e >> 1] >> (16 * (e & 1))) : (S)out[e];
  }
}

inline uint32_t fd_tiles(int64_t numel) { return (uint32_t)ceil_div(numel, kFdTile); }
inline size_t fd_part_bytes(int64_t numel) { return align_up((size_t)numel, 256); }
inline size_t fd_table_bytes(int64_t numel, int P) { return align_up(((size_t)fd_tiles(numel) + 1) * P * sizeof(uint32_t), 256); }

int fd_check(int64_t numel, int partitions) {
  if (numel <= 0 || numel > 0x7fffffffll || partitions < 1 || partitions > kFdMaxLists || numel / partitions == 0)
    return fail(ZEN_EINVAL, "zen_bitmap_dense: need 0 < partitions <= 64 and partitions <= numel < 2^31");
  return ZEN_OK;
}

}  // namespace
}  // namespace zen

extern "C" {

size_t zen_bitmap_dense_dict_bytes(int64_t numel, int partitions) {
  if (zen::fd_check(numel, partitions) != ZEN_OK) return 0;
  return zen::fd_part_bytes(numel) + zen::fd_table_bytes(numel, partitions);
}

int zen_bitmap_dense_dict(int64_t numel, int partitions, void *dict, int64_t *members, void *stream) {
  using namespace zen;
  const int rc = fd_check(numel, partitions);
  if (rc != ZEN_OK) return rc;
  if (!dict || (reinterpret_cast<uintptr_t>(dict) & 15u)) return fail(ZEN_EINVAL, "zen_bitmap_dense_dict: null or unaligned dictionary");
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint8_t *part = static_cast<uint8_t *>(dict);
  uint32_t *below = reinterpret_cast<uint32_t *>(part + fd_part_bytes(numel));
  const uint32_t tiles = fd_tiles(numel);
  k_fd_parts<<<dim3(tiles), dim3(kFdBlock), 0, s>>>((uint32_t)numel, (uint32_t)(numel / partitions), partitions, part, below);
  ZEN_LAUNCH_CHECK("k_fd_parts");
  k_fd_scan<<<dim3((unsigned)partitions), dim3(kFdScanBlock), 0, s>>>(below, tiles);
  ZEN_LAUNCH_CHECK("k_fd_scan");
  if (members) {  // the list lengths, for a caller that sizes bitmaps without a mapping
    for (int p = 0; p < partitions; ++p) members[p] = 0;
    ZEN_HIP_CHECK(hipStreamSynchronize(s));
    uint32_t host[kFdMaxLists];
    for (int p = 0; p < partitions; ++p) {
      ZEN_HIP_CHECK(hipMemcpy(&host[p], below + (size_t)p * (tiles + 1) + tiles, sizeof(uint32_t), hipMemcpyDeviceToHost));
      members[p] = host[p];
    }
  }
  return ZEN_OK;
}

size_t zen_bitmap_dense_workspace(int64_t numel, int partitions) {
  if (zen::fd_check(numel, partitions) != ZEN_OK) return 0;
  return zen::fd_table_bytes(numel, partitions);
}

int zen_bitmap_dense(const void *dict, int64_t numel, int partitions, const uint8_t *bitmaps,
                     const int64_t *bitmap_start, const void *values, int dtype, const int64_t *value_start,
                     void *dense, void *workspace, size_t workspace_bytes, int32_t *status, void *stream) {
  using namespace zen;
  const int rc = fd_check(numel, partitions);
  if (rc != ZEN_OK) return rc;
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_bitmap_dense: bad dtype");
  if (!dict || !bitmap_start || !value_start || !dense || !workspace || !status)
    return fail(ZEN_EINVAL, "zen_bitmap_dense: null pointer");
  if (workspace_bytes < zen_bitmap_dense_workspace(numel, partitions))
    return fail(ZEN_EWORKSPACE, "zen_bitmap_dense: workspace too small");
  ListStarts bm, vs;
  for (int p = 0; p <= partitions; ++p) {
    bm.at[p] = bitmap_start[p];
    vs.at[p] = value_start[p];
    if (p && (bm.at[p] < bm.at[p - 1] || vs.at[p] < vs.at[p - 1]))
      return fail(ZEN_EINVAL, "zen_bitmap_dense: list offsets must not decrease");
  }
  if ((bm.at[partitions] > bm.at[0] && !bitmaps) || (vs.at[partitions] > vs.at[0] && !values))
    return fail(ZEN_EINVAL, "zen_bitmap_dense: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint8_t *part = static_cast<const uint8_t *>(dict);
  const uint32_t *below = reinterpret_cast<const uint32_t *>(part + fd_part_bytes(numel));
  uint32_t *vstart = static_cast<uint32_t *>(workspace);
  const uint32_t tiles = fd_tiles(numel);
  ProfScope prof(kProfDecodeFused, s);
  k_fd_count<<<dim3((tiles + 255) / 256, (unsigned)partitions), dim3(256), 0, s>>>(below, tiles, partitions, bitmaps, bm,
                                                                                vstart, status);
  ZEN_LAUNCH_CHECK("k_fd_count");
  k_fd_scan<<<dim3((unsigned)partitions), dim3(kFdScanBlock), 0, s>>>(vstart, tiles);
  ZEN_LAUNCH_CHECK("k_fd_scan");
  const size_t lds = (size_t)partitions * kFdBlock * sizeof(uint16_t);
  if (lds > 32768) {  // beyond what a launch may ask for without saying so first
    const void *fn = dtype == ZEN_BF16 ? reinterpret_cast<const void *>(&k_fd_tiles<uint16_t>)
                                       : reinterpret_cast<const void *>(&k_fd_tiles<uint32_t>);
    ZEN_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  }
  if (dtype == ZEN_BF16)
    k_fd_tiles<uint16_t><<<dim3(tiles), dim3(kFdBlock), lds, s>>>(part, below, vstart, partitions, (uint32_t)numel, bitmaps, bm,
                                                                 static_cast<const uint16_t *>(values), vs,
                                                                 static_cast<uint16_t *>(dense), status);
  else
    k_fd_tiles<uint32_t><<<dim3(tiles), dim3(kFdBlock), lds, s>>>(part, below, vstart, partitions, (uint32_t)numel, bitmaps, bm,
                                                                 static_cast<const uint32_t *>(values), vs,
                                                                 static_cast<uint32_t *>(dense), status);
  ZEN_LAUNCH_CHECK("k_fd_tiles");
  return ZEN_OK;
}

}  // extern "C"
