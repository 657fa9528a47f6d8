// Second half of the sparse all-reduce with bitmaps, in one pass: every rank's bitmap over its partition's
// member list and its value list go straight into the dense gradient.  The reference turns each bitmap back
// into int64 indices by masking the cached member list (comm.py:87-99, 136-141) and scatter-adds all
// (index, value) lists into a zeroed dense tensor (comm.py:142-145, 32-44).  Neither the indices nor the
// member lists are needed for that: which partition an index belongs to is a hash away, and bit j of
// partition p's bitmap stands for the j-th index of that partition.  So the dense tensor is cut into tiles of
// 8192 indices; a dictionary built once per (numel, partitions) holds, per tile, the places of the tile's
// indices ordered by partition (16 bits each: partition 0's members in ascending order, then partition 1's,
// ...) and, per partition and tile, how many members lie below the tile.  A call first counts, per tile and
// partition, the set bits of the tile's bit range (which gives where the tile's values start in every value
// list); then a workgroup per tile brings the tile's bit ranges and values into LDS, looks up the place of
// every SET bit's member in the dictionary, and writes the tile once, zeros included: the dense tensor is
// never cleared, nothing is scattered in memory, and of the dictionary only the set bits' entries are read.
#include <mutex>

#include "zen_common.h"

namespace zen {
namespace {

#ifndef ZEN_FD_TILE
#define ZEN_FD_TILE 8192
#endif
constexpr int kFdTile = ZEN_FD_TILE;
constexpr int kFdBlock = 512;
constexpr int kFdPer = kFdTile / kFdBlock;   // consecutive indices per thread (16)
constexpr int kFdMaxLists = 64;
constexpr int kFdChunk = 16;                  // thread columns whose counts one thread adds up
constexpr int kFdChunks = kFdBlock / kFdChunk;
constexpr int kFdChunkRow = kFdChunks + 8;   // 16-bit words per list in the chunk table (rows stay 16-byte aligned)
constexpr int kFdMaxBytes = kFdTile / 8 + 2 * kFdMaxLists;  // bitmap bytes a tile's bit ranges can span
static_assert(kFdChunks == 32, "a wave's lower half scans the chunk sums");

struct ListStarts {
  int64_t at[kFdMaxLists + 1];
};

__device__ inline uint32_t part_of(uint32_t t, uint32_t n, uint32_t npp) {
  return ((poly(t) + kSeed1) % n) / npp;  // functions_cuda_kernel.cu:172-175
}

// Dictionary, step 1: per tile the places of its indices ordered by partition, and the number of indices of
// every partition.  Dynamic LDS: P * (kFdBlock + kFdChunkRow) 16-bit counters.  Every thread counts, for its 16
// consecutive indices, how many belong to each list; prefix sums over the threads, in two levels (chunks of
// 16 threads, then the 32 chunks), give every index its rank inside its list.
__global__ __launch_bounds__(kFdBlock) void k_fd_order(uint32_t n, uint32_t npp, int P, uint16_t *__restrict__ order,
                                                      uint32_t *__restrict__ below) {
  extern __shared__ __attribute__((aligned(16))) uint16_t s_cnt[];  // [P][kFdBlock]
  uint16_t (*s_chunk)[kFdChunkRow] = reinterpret_cast<uint16_t (*)[kFdChunkRow]>(s_cnt + P * kFdBlock);  // [32]: the tile's total
  __shared__ uint32_t s_base[kFdMaxLists];  // members of lower lists in the tile
  const uint32_t tile_base = blockIdx.x * (uint32_t)kFdTile;
  const uint32_t base = tile_base + threadIdx.x * (uint32_t)kFdPer;
  uint32_t part[kFdPer];
#pragma unroll
  for (int e = 0; e < kFdPer; ++e) part[e] = base + e < n ? part_of(base + e, n, npp) : 0xffu;
  for (int p = 0; p < P; ++p) {
    uint32_t c = 0;
#pragma unroll
    for (int e = 0; e < kFdPer; ++e) c += part[e] == (uint32_t)p;
    s_cnt[p * kFdBlock + threadIdx.x] = (uint16_t)c;
  }
  __syncthreads();
  for (int q = threadIdx.x; q < P * kFdChunks; q += kFdBlock) {
    const int p = q / kFdChunks, c = q % kFdChunks;
    uint16_t *col = s_cnt + p * kFdBlock + c * kFdChunk;
    uint32_t run = 0;
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
  if (threadIdx.x < 64) {
    const uint32_t total = threadIdx.x < (uint32_t)P ? s_chunk[threadIdx.x][kFdChunks] : 0u;
    const uint32_t incl = wave_inclusive_scan(total);
    if (threadIdx.x < (uint32_t)P) {
      s_base[threadIdx.x] = incl - total;
      below[(size_t)threadIdx.x * (gridDim.x + 1) + blockIdx.x] = total;
    }
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < kFdPer; ++e) {
    const uint32_t p = part[e];
    if (p >= (uint32_t)P) continue;  // past the end of the tensor
    uint32_t rank = s_base[p] + s_chunk[p][threadIdx.x / kFdChunk] + s_cnt[p * kFdBlock + threadIdx.x];
#pragma unroll
    for (int f = 0; f < e; ++f) rank += part[f] == p;
    order[tile_base + rank] = (uint16_t)(threadIdx.x * kFdPer + e);
  }
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

// Set bits of bitmap `bm` in the bit range [b0, b1); bytes at or beyond `bytes` count as zero.  Read as
// aligned 64-bit words: a word that holds one byte of the bitmap lies in that byte's page, and what it holds
// beside the bitmap is masked away.
__device__ inline uint32_t popcount_range(const uint8_t *__restrict__ bm, int64_t bytes, uint32_t b0, uint32_t b1) {
  const uint64_t limit = (uint64_t)bytes * 8u;
  if (b1 > limit) b1 = (uint32_t)limit;
  if (b1 <= b0) return 0;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(bm);
  const uint64_t *words = reinterpret_cast<const uint64_t *>(addr & ~(uintptr_t)7);
  const uint64_t lo = (uint64_t)b0 + (addr & 7u) * 8u, hi = (uint64_t)b1 + (addr & 7u) * 8u;  // bit numbers from words[0] on
  const uint64_t first = lo >> 6, last = (hi - 1u) >> 6;
  uint32_t c = 0;
  for (uint64_t w = first; w <= last; ++w) {
    unsigned long long x = words[w];
    if (w == first) x &= ~0ull << (lo & 63u);
    if (w == last) x &= ~0ull >> (63u - ((hi - 1u) & 63u));
    c += (uint32_t)__popcll(x);
  }
  return c;
}

// Where the values of a tile start in every list, in two levels: the tiles are taken in groups of 256; a row of
// 257 words per (list, group) holds the set bits of the group's tiles in front of each tile (entry 256: of the
// whole group), a second table the set bits in front of each group.
constexpr int kFdGroup = 256;
constexpr int kFdGroupRow = kFdGroup + 1;
inline uint32_t fd_groups(uint32_t tiles) { return (tiles + kFdGroup - 1) / kFdGroup; }

// Per (group of tiles, list): set bits in each tile's bit range of the list's bitmap, summed up inside the
// group.  A bitmap shorter than its list (the reference's mask would not fit the member list, comm.py:97-98)
// raises ZEN_STAT_BAD_INDEX.
__global__ __launch_bounds__(kFdGroup) void k_fd_count(const uint32_t *__restrict__ below, uint32_t tiles, int P,
                                                       const uint8_t *__restrict__ bitmaps, ListStarts bm,
                                                       uint32_t *__restrict__ vstart, uint32_t *__restrict__ gsum,
                                                       int32_t *status) {
  __shared__ uint32_t s_scan[kFdGroup / 64 + 1];
  const uint32_t tile = blockIdx.x * (uint32_t)kFdGroup + threadIdx.x;
  const int p = blockIdx.y;
  uint32_t cnt = 0;
  if (tile < tiles) {
    const size_t i = (size_t)p * (tiles + 1) + tile;
    const uint32_t b0 = below[i], b1 = below[i + 1];
    const int64_t bytes = bm.at[p + 1] - bm.at[p];
    if (tile == tiles - 1 && ((int64_t)b1 + 7) / 8 > bytes) atomicOr(status, ZEN_STAT_BAD_INDEX);
    cnt = popcount_range(bitmaps + bm.at[p], bytes, b0, b1);
  }
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kFdGroup>(cnt, s_scan, &total);
  const size_t g = (size_t)p * gridDim.x + blockIdx.x;
  vstart[g * kFdGroupRow + threadIdx.x] = before;
  if (threadIdx.x == 0) {
    vstart[g * kFdGroupRow + kFdGroup] = total;
    gsum[g] = total;
  }
}

// Per list (blockIdx.x): exclusive prefix over the groups' sums, in place (a tensor of 2^31 elements has 1024 groups).
constexpr int kFdGroupsMax = 1024;
__global__ __launch_bounds__(kFdGroupsMax) void k_fd_groups(uint32_t *__restrict__ gsum, uint32_t groups) {
  __shared__ uint32_t s_scan[kFdGroupsMax / 64 + 1];
  uint32_t *row = gsum + (size_t)blockIdx.x * groups;
  const uint32_t v = threadIdx.x < groups ? row[threadIdx.x] : 0u;
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kFdGroupsMax>(v, s_scan, &total);
  if (threadIdx.x < groups) row[threadIdx.x] = before;
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

// A workgroup takes one tile after the other (tile = blockIdx.x, + gridDim.x, ...): the tile's bit ranges and
// its values (contiguous stretches of the lists) come into LDS, the set bits are written out as a list, and the
// threads take one SET bit each: its member's place in the tile is one entry of the dictionary, the value goes
// there, into a copy of the tile in LDS that is written out once.  The next tile's table entries are asked for
// while this tile is worked on.
constexpr int kFdValStage = kFdTile / 8;  // values of a tile kept in LDS (tiles with more set bits fetch the rest one by one)
constexpr int kFdHitStage = kFdTile / 8;  // set bits of a tile listed at a time
constexpr int kFdBytesPer = (kFdMaxBytes + kFdBlock - 1) / kFdBlock;  // 3
constexpr int kFdValsPer = kFdValStage / kFdBlock;                    // 2
#ifndef ZEN_FD_MIN_WAVES
#define ZEN_FD_MIN_WAVES 6  // waves per SIMD the tile kernel is compiled for: three workgroups to a compute unit
#endif

// Thread p < P: list p's members below the tile and below the next, the set bits below the tile's group, below
// the tile inside the group, below the next tile inside the group.
__device__ __forceinline__ void fd_fetch_dict(const uint32_t *__restrict__ below, const uint32_t *__restrict__ vstart,
                                              const uint32_t *__restrict__ gpre, uint32_t tiles, uint32_t groups, int P,
                                              uint32_t tile, uint32_t (&d)[5]) {
  d[0] = d[1] = d[2] = d[3] = d[4] = 0;
  if (threadIdx.x < (uint32_t)P) {
    const size_t at = (size_t)threadIdx.x * (tiles + 1) + tile;
    const size_t g = (size_t)threadIdx.x * groups + tile / kFdGroup;
    const size_t va = g * kFdGroupRow + tile % kFdGroup;
    d[0] = below[at];
    d[1] = below[at + 1];
    d[2] = gpre[g];
    d[3] = vstart[va];
    d[4] = vstart[va + 1];
  }
}

constexpr int kFdByteBlocks = (kFdMaxBytes + 15) / 16;
constexpr int kFdValBlocks = kFdValStage / 16;

// Wave 0: the table of a tile's lists from the entries fetched for it.
__device__ __forceinline__ void fd_list_table(const uint32_t (&d)[5], int P, uint4 *meta, uint4 *len, uint8_t *byte_lut,
                                              uint8_t *val_lut) {
  const int p = threadIdx.x;
  uint32_t b0 = 0, cnt = 0, nb = 0, v0 = 0, nv = 0;
  if (p < P) {
    b0 = d[0];
    cnt = d[1] - d[0];
    if (cnt > (uint32_t)kFdTile) cnt = kFdTile;  // cannot be with a table this library built
    nb = cnt ? ((b0 + cnt - 1u) >> 3) - (b0 >> 3) + 1u : 0u;
    v0 = d[2] + d[3];
    nv = d[4] - d[3];
    if (nv > cnt) nv = cnt;  // cannot be (the count kernel counted the same bits)
  }
  const uint32_t bincl = wave_inclusive_scan(nb), vincl = wave_inclusive_scan(nv), cincl = wave_inclusive_scan(cnt);
  if (p < P) {
    meta[p] = make_uint4(b0, bincl - nb, v0, vincl - nv);
    len[p] = make_uint4(cnt, nv, cincl - cnt, 0);
  }
  if (p == 63) meta[P] = make_uint4(0, bincl, cincl, vincl);
  // the list that holds the first entry of every block of 16 entries of the side-by-side arrays
  for (uint32_t blk = (bincl - nb + 15u) >> 4; (blk << 4) < bincl && blk < (uint32_t)kFdByteBlocks; ++blk) byte_lut[blk] = (uint8_t)p;
  for (uint32_t blk = (vincl - nv + 15u) >> 4; (blk << 4) < vincl && blk < (uint32_t)kFdValBlocks; ++blk) val_lut[blk] = (uint8_t)p;
}

// A tile's bitmap bytes and values as they will lie side by side in LDS, asked for one tile ahead and kept in
// registers meanwhile.  Entry i of such an array belongs to the last list whose stretch starts at or before i
// (the stretches' starts ascend): the list of the block's first entry is looked up, the few lists that may start
// inside the block are stepped over, so that every thread fetches its entries in one go instead of list after list.
template <typename S>
__device__ __forceinline__ void fd_fetch_lists(const uint4 *meta, int P, const uint8_t *byte_lut, const uint8_t *val_lut,
                                               const int64_t *s_bm, const int64_t *s_vs,
                                               const uint8_t *__restrict__ bitmaps, const S *__restrict__ values,
                                               uint32_t (&byte_in)[kFdBytesPer], uint32_t (&byte_list)[kFdBytesPer],
                                               S (&val_in)[kFdValsPer]) {
  uint32_t total_bytes = meta[P].y;
  if (total_bytes > (uint32_t)kFdMaxBytes || meta[P].z > (uint32_t)kFdTile) total_bytes = 0;
  const uint32_t total_vals = min(meta[P].w, (uint32_t)kFdValStage);
#pragma unroll
  for (int k = 0; k < kFdBytesPer; ++k) {
    const uint32_t i = threadIdx.x + (uint32_t)k * kFdBlock;
    byte_in[k] = 0;
    byte_list[k] = 0;
    if (i < total_bytes) {
      int lo = byte_lut[i >> 4];
      while (lo + 1 < P && meta[lo + 1].y <= i) ++lo;
      const int64_t g = (int64_t)(meta[lo].x >> 3) + (i - meta[lo].y);
      byte_list[k] = (uint32_t)lo;
      if (g < s_bm[lo + 1] - s_bm[lo]) byte_in[k] = bitmaps[s_bm[lo] + g];  // a short bitmap was flagged by the count kernel
    }
  }
#pragma unroll
  for (int k = 0; k < kFdValsPer; ++k) {
    const uint32_t i = threadIdx.x + (uint32_t)k * kFdBlock;
    val_in[k] = 0;
    if (i < total_vals) {
      int lo = val_lut[i >> 4];
      while (lo + 1 < P && meta[lo + 1].w <= i) ++lo;
      const int64_t g = (int64_t)meta[lo].z + (i - meta[lo].w);
      if (g < s_vs[lo + 1] - s_vs[lo]) val_in[k] = values[s_vs[lo] + g];
    }
  }
}

template <typename S>
__global__ __launch_bounds__(kFdBlock, ZEN_FD_MIN_WAVES) void k_fd_tiles(const uint16_t *__restrict__ order,
                                                                        const uint32_t *__restrict__ below,
                                                                        const uint32_t *__restrict__ vstart,
                                                                        const uint32_t *__restrict__ gpre, uint32_t tiles,
                                                                        int P, uint32_t n,
                                                                        const uint8_t *__restrict__ bitmaps, ListStarts bm,
                                                                        const S *__restrict__ values, ListStarts vs,
                                                                        S *__restrict__ dense, int32_t *status) {
  // per list: first bit of the tile's range; where its bytes start in s_bl; number of the tile's first value in
  // the list; where its values start in s_val (entry P: the totals)
  __shared__ uint4 s_meta[2][kFdMaxLists + 1];        // two sets: this tile's and the next one's
  __shared__ uint4 s_len[2][kFdMaxLists];             // per list: members in the tile; set bits among them; members of lower lists in the tile
  __shared__ uint8_t s_blut[2][kFdByteBlocks + 3], s_vlut[2][kFdValBlocks];  // list of every 16th byte and value
  __shared__ uint32_t s_front[kFdMaxLists];           // per list: set bits of the tile in the lists before it
  __shared__ uint16_t s_bl[kFdMaxBytes + 8];          // the bitmap bytes of the tile's ranges (low half) and their list (high half)
  __shared__ S s_val[kFdValStage];
  __shared__ __attribute__((aligned(16))) S s_tile[kFdTile];  // the tile of the dense tensor
  __shared__ uint32_t s_hit[kFdHitStage];             // set bits: list << 16 | place in s_bl << 3 | bit
  __shared__ uint32_t s_scan[kFdBlock / 64 + 1];
  // the lists' offsets, looked up by list number further down: in LDS, because a kernel argument indexed with a
  // number that differs from lane to lane is fetched from memory, one round trip per look
  __shared__ int64_t s_bm[kFdMaxLists + 1], s_vs[kFdMaxLists + 1];
  if (threadIdx.x <= (uint32_t)P) {
    s_bm[threadIdx.x] = bm.at[threadIdx.x];
    s_vs[threadIdx.x] = vs.at[threadIdx.x];
  }
  const uint32_t groups = (tiles + kFdGroup - 1) / kFdGroup;
  const bool aligned = (reinterpret_cast<uintptr_t>(dense) & 15u) == 0;
  uint32_t byte_in[kFdBytesPer], byte_list[kFdBytesPer];
  S val_in[kFdValsPer];
  uint32_t dn[5];
  if (blockIdx.x >= tiles) return;
  if (threadIdx.x < 64) {
    fd_fetch_dict(below, vstart, gpre, tiles, groups, P, blockIdx.x, dn);
    fd_list_table(dn, P, s_meta[0], s_len[0], s_blut[0], s_vlut[0]);
    if (blockIdx.x + gridDim.x < tiles) fd_fetch_dict(below, vstart, gpre, tiles, groups, P, blockIdx.x + gridDim.x, dn);
  }
  __syncthreads();
  fd_fetch_lists<S>(s_meta[0], P, s_blut[0], s_vlut[0], s_bm, s_vs, bitmaps, values, byte_in, byte_list, val_in);
  bool bad = false;
  int set = 0;
  for (uint32_t tile = blockIdx.x; tile < tiles; tile += gridDim.x, set ^= 1) {
    const uint32_t tile_base = tile * (uint32_t)kFdTile;
    const uint32_t next = tile + gridDim.x;
    if (threadIdx.x < 64 && next < tiles) {
      fd_list_table(dn, P, s_meta[set ^ 1], s_len[set ^ 1], s_blut[set ^ 1], s_vlut[set ^ 1]);
      if (next + gridDim.x < tiles) fd_fetch_dict(below, vstart, gpre, tiles, groups, P, next + gridDim.x, dn);
    }
    {
      // the tile is put together in LDS and written once at the end, with full-width stores: scattered two-byte
      // stores to memory cost one request each
      uint4 *z = reinterpret_cast<uint4 *>(s_tile);
#pragma unroll
      for (int i = 0; i < (int)(kFdTile * sizeof(S) / 16) / kFdBlock; ++i) z[i * kFdBlock + threadIdx.x] = make_uint4(0, 0, 0, 0);
    }
    uint32_t total_bytes = s_meta[set][P].y;
    // cannot be: the lists' members in a tile add up to its size at most
    if (total_bytes > (uint32_t)kFdMaxBytes || s_meta[set][P].z > (uint32_t)kFdTile) {
      total_bytes = 0;
      bad = true;
    }
    const uint32_t total_vals = min(s_meta[set][P].w, (uint32_t)kFdValStage);
#pragma unroll
    for (int k = 0; k < kFdBytesPer; ++k) {
      const uint32_t i = threadIdx.x + (uint32_t)k * kFdBlock;
      if (i < total_bytes) {
        // bits outside the list's range of this tile belong to other tiles (or to nobody)
        const uint32_t lo = byte_list[k];
        const uint4 m = s_meta[set][lo];
        const uint32_t cnt = s_len[set][lo].x;
        const uint32_t first_bit = ((m.x >> 3) + (i - m.y)) << 3;
        uint32_t byte = byte_in[k];
        if (first_bit < m.x) byte &= 0xffu << (m.x - first_bit);
        if (first_bit + 8u > m.x + cnt) byte &= 0xffu >> (first_bit + 8u - (m.x + cnt));
        s_bl[i] = (uint16_t)(byte | (lo << 8));
      }
    }
#pragma unroll
    for (int k = 0; k < kFdValsPer; ++k) {
      const uint32_t i = threadIdx.x + (uint32_t)k * kFdBlock;
      if (i < total_vals) s_val[i] = val_in[k];
    }
    __syncthreads();
    if (next < tiles) fd_fetch_lists<S>(s_meta[set ^ 1], P, s_blut[set ^ 1], s_vlut[set ^ 1], s_bm, s_vs, bitmaps, values, byte_in, byte_list, val_in);
    // every thread takes three consecutive bytes; the set bits in front of them by a prefix sum over the threads
    uint32_t mine[kFdBytesPer], sum = 0;
#pragma unroll
    for (int k = 0; k < kFdBytesPer; ++k) {
      const uint32_t i = threadIdx.x * kFdBytesPer + k;
      mine[k] = i < total_bytes ? (uint32_t)s_bl[i] : 0u;
      sum += (uint32_t)__popc(mine[k] & 0xffu);
    }
    uint32_t before_list = 0xffffu;  // the list of the byte in front of the thread's first
    if (threadIdx.x > 0 && threadIdx.x * kFdBytesPer <= total_bytes) before_list = s_bl[threadIdx.x * kFdBytesPer - 1] >> 8;
    uint32_t total_hits;
    const uint32_t first_hit = block_exclusive_scan<uint32_t, kFdBlock>(sum, s_scan, &total_hits);
    // The set bits, listed (kFdHitStage at a time) and then taken one per thread and turn: a thread that went
    // through the bits of its own bytes to the end would keep a whole wave busy for as long as its fullest
    // byte takes.
    for (uint32_t hbase = 0; hbase < total_hits; hbase += kFdHitStage) {
      {
        uint32_t h = first_hit, prev = before_list;
#pragma unroll
        for (int k = 0; k < kFdBytesPer; ++k) {
          const uint32_t i = threadIdx.x * kFdBytesPer + k;
          if (i < total_bytes) {
            const uint32_t p = mine[k] >> 8;
            if (hbase == 0 && p != prev) s_front[p] = h;  // the bytes are masked: nothing set in front of the range inside its first byte
            prev = p;
            for (uint32_t bits = mine[k] & 0xffu; bits; bits &= bits - 1u, ++h)
              if (h - hbase < (uint32_t)kFdHitStage) s_hit[h - hbase] = (p << 16) | (i << 3) | ((uint32_t)__ffs((int)bits) - 1u);
          }
        }
      }
      __syncthreads();
      const uint32_t hend = min(total_hits, hbase + (uint32_t)kFdHitStage);
      for (uint32_t h = hbase + threadIdx.x; h < hend; h += kFdBlock) {
        const uint32_t ent = s_hit[h - hbase];
        const uint32_t p = ent >> 16, i = (ent >> 3) & 0x1fffu, bit = ent & 7u;
        const uint4 m = s_meta[set][p];
        const uint4 ln = s_len[set][p];
        const int64_t list_vals = s_vs[p + 1] - s_vs[p];
        const uint32_t j = (((m.x >> 3) + (i - m.y)) << 3) + bit - m.x;  // member number inside the tile (below ln.x: the bytes are masked)
        const uint32_t nth = h - s_front[p];                            // value number inside the tile's stretch
        const uint32_t at = order[(size_t)tile_base + ln.z + j] & (uint32_t)(kFdTile - 1);
        const uint32_t vl = m.w + nth;
        if (nth < ln.y && (int64_t)m.z + nth < list_vals) {
          const S v = vl < (uint32_t)kFdValStage ? s_val[vl] : values[s_vs[p] + m.z + nth];
          s_tile[at] = fd_value<S>(v);
        } else {
          bad = true;  // more set bits than values
        }
      }
      __syncthreads();
    }
    // written out in 16-byte pieces, consecutive threads consecutive pieces: every store instruction fills whole lines
    if (aligned && tile_base + (uint32_t)kFdTile <= n) {
      constexpr int kPieces = (int)(kFdTile * sizeof(S) / 16);
      const uint4 *src = reinterpret_cast<const uint4 *>(s_tile);
      uint4 *dst = reinterpret_cast<uint4 *>(dense + tile_base);
#pragma unroll
      for (int i = 0; i < kPieces / kFdBlock; ++i) dst[i * kFdBlock + threadIdx.x] = src[i * kFdBlock + threadIdx.x];
    } else {
      for (uint32_t e = threadIdx.x; e < (uint32_t)kFdTile && tile_base + e < n; e += kFdBlock) dense[tile_base + e] = s_tile[e];
      __syncthreads();  // here the tile is cleared again by other threads than those that have just read it
    }
  }
  if (bad) atomicOr(status, ZEN_STAT_BAD_INDEX);
}

inline uint32_t fd_tiles(int64_t numel) { return (uint32_t)ceil_div(numel, kFdTile); }
inline size_t fd_order_bytes(int64_t numel) { return (size_t)fd_tiles(numel) * kFdTile * sizeof(uint16_t); }
inline size_t fd_table_bytes(int64_t numel, int P) { return align_up(((size_t)fd_tiles(numel) + 1) * P * sizeof(uint32_t), 256); }
inline size_t fd_vstart_bytes(int64_t numel, int P) {
  return align_up((size_t)fd_groups(fd_tiles(numel)) * kFdGroupRow * P * sizeof(uint32_t), 256);
}
inline size_t fd_gsum_bytes(int64_t numel, int P) { return align_up((size_t)fd_groups(fd_tiles(numel)) * P * sizeof(uint32_t), 256); }

// Workgroups of the tile kernel that fit the device at once (it walks over the tiles with that many).
int fd_resident_blocks(const void *fn, size_t lds) {
  struct Known { const void *fn; size_t lds; int dev; int blocks; };
  static std::mutex mu;
  static Known known[8];
  static int n_known = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < n_known; ++i)
    if (known[i].fn == fn && known[i].lds == lds && known[i].dev == dev) return known[i].blocks;
  int per_cu = 0, cus = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, kFdBlock, lds) != hipSuccess || per_cu < 1) return 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) return 0;
  const int blocks = per_cu * cus;
  known[n_known < 8 ? n_known++ : 7] = Known{fn, lds, dev, blocks};
  return blocks;
}

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
  return zen::fd_order_bytes(numel) + zen::fd_table_bytes(numel, partitions);
}

int zen_bitmap_dense_dict(int64_t numel, int partitions, void *dict, int64_t *members, void *stream) {
  using namespace zen;
  const int rc = fd_check(numel, partitions);
  if (rc != ZEN_OK) return rc;
  if (!dict || (reinterpret_cast<uintptr_t>(dict) & 15u)) return fail(ZEN_EINVAL, "zen_bitmap_dense_dict: null or unaligned dictionary");
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint16_t *order = static_cast<uint16_t *>(dict);
  uint32_t *below = reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(dict) + fd_order_bytes(numel));
  const uint32_t tiles = fd_tiles(numel);
  const size_t lds = (size_t)partitions * (kFdBlock + kFdChunkRow) * sizeof(uint16_t);
  if (lds > 32768)  // beyond what a launch may ask for without saying so first
    ZEN_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_fd_order), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  k_fd_order<<<dim3(tiles), dim3(kFdBlock), lds, s>>>((uint32_t)numel, (uint32_t)(numel / partitions), partitions, order, below);
  ZEN_LAUNCH_CHECK("k_fd_order");
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
  return zen::fd_vstart_bytes(numel, partitions) + zen::fd_gsum_bytes(numel, partitions);
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
  const uint16_t *order = static_cast<const uint16_t *>(dict);
  const uint32_t *below = reinterpret_cast<const uint32_t *>(static_cast<const uint8_t *>(dict) + fd_order_bytes(numel));
  uint32_t *vstart = static_cast<uint32_t *>(workspace);
  uint32_t *gsum = reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(workspace) + fd_vstart_bytes(numel, partitions));
  const uint32_t tiles = fd_tiles(numel);
  const uint32_t groups = fd_groups(tiles);
  const size_t lds = 0;
  const void *fn = dtype == ZEN_BF16 ? reinterpret_cast<const void *>(&k_fd_tiles<uint16_t>)
                                     : reinterpret_cast<const void *>(&k_fd_tiles<uint32_t>);
  const int resident = fd_resident_blocks(fn, lds);
  if (resident < 1) return fail(ZEN_EHIP, "zen_bitmap_dense: the tile kernel does not fit the device");
  const uint32_t grid = tiles < (uint32_t)resident ? tiles : (uint32_t)resident;
  ProfScope prof(kProfDecodeFused, s);
  k_fd_count<<<dim3(groups, (unsigned)partitions), dim3(kFdGroup), 0, s>>>(below, tiles, partitions, bitmaps, bm, vstart, gsum,
                                                                       status);
  ZEN_LAUNCH_CHECK("k_fd_count");
  k_fd_groups<<<dim3((unsigned)partitions), dim3(kFdGroupsMax), 0, s>>>(gsum, groups);
  ZEN_LAUNCH_CHECK("k_fd_groups");
  if (dtype == ZEN_BF16)
    k_fd_tiles<uint16_t><<<dim3(grid), dim3(kFdBlock), 0, s>>>(order, below, vstart, gsum, tiles, partitions, (uint32_t)numel,
                                                                bitmaps, bm, static_cast<const uint16_t *>(values), vs,
                                                                static_cast<uint16_t *>(dense), status);
  else
    k_fd_tiles<uint32_t><<<dim3(grid), dim3(kFdBlock), 0, s>>>(order, below, vstart, gsum, tiles, partitions, (uint32_t)numel,
                                                                bitmaps, bm, static_cast<const uint32_t *>(values), vs,
                                                                static_cast<uint32_t *>(dense), status);
  ZEN_LAUNCH_CHECK("k_fd_tiles");
  return ZEN_OK;
}

}  // extern "C"
