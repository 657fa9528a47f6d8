// Bitmap index codec of the second exchange (comm.py:59-99): a rank describes
// which members of its partition's ascending index list are present by one bit
// per member, least significant bit first inside each byte.
//
// Encode is a lookup per index.  A rank dictionary kept next to the mapping
// (members below every multiple of 512, plus one membership bit per index
// value) answers it with two loads; without the dictionary the position is
// estimated by interpolation (the members are spread evenly, that is what the
// hash is for), bracketed by doubling steps and found by bisection.  Decode is a compaction of the set bits: count per
// block, scan the block counts, write mapping[position] for every set bit.
#include "zen_common.h"

namespace zen {
namespace {

constexpr int kBmBlock = 256;
constexpr int kBmBytes = 16;                       // bitmap bytes per thread in decode
constexpr int kBmSpan = kBmBlock * kBmBytes * 8;   // positions per workgroup (32768)

// First position whose member is >= v (torch.searchsorted, left; comm.py:61), looked for around position g:
// doubling steps away from g until v is bracketed, then bisection inside the bracket.
__device__ inline int64_t member_lower_bound_near(const int64_t *__restrict__ map, int64_t count, int64_t g,
                                                  int64_t step, int64_t v) {
  int64_t lo, hi;  // map[lo] < v (lo = -1: nothing below), map[hi] >= v (hi = count: nothing at or above)
  if (map[g] < v) {
    lo = g;
    hi = g + step;
    while (hi < count && map[hi] < v) {
      lo = hi;
      step <<= 1;
      hi += step;
    }
    if (hi > count) hi = count;
  } else {
    hi = g;
    lo = g - step;
    while (lo >= 0 && map[lo] >= v) {
      hi = lo;
      step <<= 1;
      lo -= step;
    }
    if (lo < -1) lo = -1;
  }
  while (hi - lo > 1) {
    const int64_t mid = lo + ((hi - lo) >> 1);
    if (map[mid] < v)
      lo = mid;
    else
      hi = mid;
  }
  return hi;
}

// Rank dictionary of one partition's member list, kept next to the list: the index range is cut into blocks
// of 512 values; rank[b] = number of members below block b (one more entry at the end = the member count),
// followed by 512 membership bits per block.  The position of any index is then rank[b] + the number of
// membership bits below it in its block: two loads that neighbouring indices share, 1/8 byte per index value
// instead of a search through eight-byte members.
constexpr int kBmShift = 9;
constexpr int kBmBlockWords = (1 << kBmShift) / 32;  // 16 words = one 64-byte line per block

__global__ __launch_bounds__(kBmBlock) void k_bitmap_ranks(const int64_t *__restrict__ map, int64_t count,
                                                           int64_t blocks, uint32_t *__restrict__ rank_at) {
  const int64_t b = (int64_t)blockIdx.x * kBmBlock + threadIdx.x;
  if (b > blocks) return;
  if (b == blocks) {
    rank_at[b] = (uint32_t)count;
    return;
  }
  const int64_t v = b << kBmShift;
  int64_t lo = -1, hi = count;
  while (hi - lo > 1) {
    const int64_t mid = lo + ((hi - lo) >> 1);
    if (map[mid] < v)
      lo = mid;
    else
      hi = mid;
  }
  rank_at[b] = (uint32_t)hi;
}

// One thread per block: the block's members (consecutive in the list) become its 512 membership bits.
__global__ __launch_bounds__(kBmBlock) void k_bitmap_members(const int64_t *__restrict__ map, int64_t blocks,
                                                             const uint32_t *__restrict__ rank_at,
                                                             uint32_t *__restrict__ bits) {
  const int64_t b = (int64_t)blockIdx.x * kBmBlock + threadIdx.x;
  if (b >= blocks) return;
  uint32_t w[kBmBlockWords];
#pragma unroll
  for (int q = 0; q < kBmBlockWords; ++q) w[q] = 0;
  for (int64_t j = rank_at[b]; j < (int64_t)rank_at[b + 1]; ++j) {
    const uint32_t off = (uint32_t)(map[j] & ((1 << kBmShift) - 1));
#pragma unroll
    for (int q = 0; q < kBmBlockWords; ++q) w[q] |= (off >> 5) == (uint32_t)q ? 1u << (off & 31) : 0u;
  }
  uint4 *out = reinterpret_cast<uint4 *>(bits + b * kBmBlockWords);
#pragma unroll
  for (int q = 0; q < kBmBlockWords / 4; ++q) out[q] = make_uint4(w[4 * q], w[4 * q + 1], w[4 * q + 2], w[4 * q + 3]);
}

// One index per thread, neighbouring threads neighbouring indices; the indices may come in any order.
// Without the dictionary the position is estimated by interpolation over the whole list (the members are
// spread evenly, that is what the hash is for; float arithmetic lands within a few thousand places) and
// corrected by a search around the estimate.
template <typename I>
__global__ __launch_bounds__(kBmBlock) void k_bitmap_mark(const int64_t *__restrict__ map, int64_t count,
                                                          const I *__restrict__ idx, int64_t idx_n,
                                                          const int64_t *__restrict__ idx_n_dev,
                                                          const uint32_t *__restrict__ rank_at, int64_t rank_blocks,
                                                          uint32_t *__restrict__ words, int32_t *status) {
  int64_t n = idx_n;
  if (idx_n_dev) {
    const int64_t d = *idx_n_dev;
    n = d < n ? (d < 0 ? 0 : d) : n;
  }
  if (count <= 0) {
    if (n > 0 && blockIdx.x == 0 && threadIdx.x == 0) atomicOr(status, ZEN_STAT_BAD_INDEX);
    return;
  }
  const int64_t j = (int64_t)blockIdx.x * kBmBlock + threadIdx.x;
  const bool live = j < n;
  const int64_t v = live ? (int64_t)idx[j] : 0;
  int64_t pos;
  if (!live) {
    pos = count;
  } else if (rank_at) {
    if (v < 0) {
      pos = 0;
    } else if ((v >> kBmShift) >= rank_blocks) {
      pos = count;  // beyond the index range: beyond every member
    } else {
      const int64_t b = v >> kBmShift;
      const uint4 *line = reinterpret_cast<const uint4 *>(rank_at + (rank_blocks + 1 + 3) / 4 * 4 + b * kBmBlockWords);
      const uint32_t off = (uint32_t)(v & ((1 << kBmShift) - 1));
      uint32_t below = rank_at[b];
#pragma unroll
      for (int q = 0; q < kBmBlockWords / 4; ++q) {
        const uint4 m = line[q];
        const uint32_t ws[4] = {m.x, m.y, m.z, m.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t first_bit = (uint32_t)(q * 4 + e) * 32u;
          uint32_t x = ws[e];
          if (off <= first_bit)
            x = 0;
          else if (off - first_bit < 32u)
            x &= (1u << (off - first_bit)) - 1u;
          below += (uint32_t)__popc(x);
        }
      }
      pos = below;
    }
  } else {
    const int64_t first = map[0], last = map[count - 1];
    if (v <= first) {
      pos = 0;
    } else if (v > last) {
      pos = count;
    } else {
      const float slope = (float)(count - 1) / (float)(last - first);
      int64_t g = (int64_t)((float)(v - first) * slope);
      g = g > count - 1 ? count - 1 : (g < 0 ? 0 : g);
      pos = member_lower_bound_near(map, count, g, 64, v);
    }
  }
  // Neighbouring lanes often mark the same word (ascending indices: positions a few places apart).  Each lane
  // gathers the bits of the lanes before it that name the same word; only the last lane of such a stretch
  // goes to memory.  (A lane may also pick up bits of the same word from further away: harmless for an OR.)
  const bool bad = !live || pos >= count;
  if (live && bad) atomicOr(status, ZEN_STAT_BAD_INDEX);  // torch raises an index error here (comm.py:63)
  const uint32_t word = bad ? 0xffffffffu : (uint32_t)(pos >> 5);
  uint32_t bits = bad ? 0u : 1u << (pos & 31);
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t w2 = (uint32_t)__shfl_up((int)word, off);
    const uint32_t b2 = (uint32_t)__shfl_up((int)bits, off);
    if (lane >= off && w2 == word) bits |= b2;
  }
  const uint32_t next = (uint32_t)__shfl_down((int)word, 1);
  if (!bad && (lane == 63 || next != word)) atomicOr(&words[word], bits);
}

// Bits of the 16 bitmap bytes of thread t of block b that lie below `count` positions, as four words.
__device__ inline void load_bits(const uint8_t *__restrict__ bitmap, int64_t bytes, int64_t count, int64_t byte0,
                                 uint32_t (&w)[4]) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uint32_t x = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int64_t at = byte0 + q * 4 + e;
      if (at < bytes) x |= (uint32_t)bitmap[at] << (8 * e);
    }
    const int64_t pos0 = (byte0 + q * 4) * 8;  // position of bit 0 of this word
    if (pos0 >= count)
      x = 0;
    else if (count - pos0 < 32)
      x &= (1u << (count - pos0)) - 1u;
    w[q] = x;
  }
}

__global__ __launch_bounds__(kBmBlock) void k_bitmap_count(const uint8_t *__restrict__ bitmap, int64_t bytes,
                                                           int64_t count, uint32_t *__restrict__ partial) {
  __shared__ uint32_t s_scan[kBmBlock / 64];
  uint32_t w[4];
  load_bits(bitmap, bytes, count, ((int64_t)blockIdx.x * kBmBlock + threadIdx.x) * kBmBytes, w);
  const uint32_t c = (uint32_t)(__popc(w[0]) + __popc(w[1]) + __popc(w[2]) + __popc(w[3]));
  uint32_t total;
  block_exclusive_scan<uint32_t, kBmBlock>(c, s_scan, &total);
  if (threadIdx.x == 0) partial[blockIdx.x] = total;
}

// One workgroup: partial[b] becomes the number of set bits before block b; the total goes to *out_count.
__global__ __launch_bounds__(1024) void k_bitmap_scan(uint32_t *__restrict__ partial, uint32_t blocks,
                                                      int64_t capacity, int64_t *__restrict__ out_count,
                                                      int32_t *status) {
  __shared__ uint64_t s_scan[1024 / 64];
  __shared__ uint64_t s_carry;
  if (threadIdx.x == 0) s_carry = 0;
  __syncthreads();
  for (uint32_t base = 0; base < blocks; base += 1024) {
    const uint32_t b = base + threadIdx.x;
    const uint64_t c = b < blocks ? partial[b] : 0;
    uint64_t total;
    const uint64_t before = block_exclusive_scan<uint64_t, 1024>(c, s_scan, &total);
    const uint64_t carry = s_carry;
    // the offsets stay below 2^32: a bitmap describes fewer than 2^31 positions
    if (b < blocks) partial[b] = (uint32_t)(carry + before);
    __syncthreads();
    if (threadIdx.x == 0) s_carry = carry + total;
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    *out_count = (int64_t)s_carry;
    if ((int64_t)s_carry > capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
}

constexpr int kBmList = 4096;  // set bits a workgroup hands on per round

// The positions of the set bits go through a list in LDS, in order: consecutive threads then fetch
// consecutive entries (loads that do not wait for each other) and write consecutive outputs.
__global__ __launch_bounds__(kBmBlock) void k_bitmap_emit(const int64_t *__restrict__ map,
                                                          const uint8_t *__restrict__ bitmap, int64_t bytes,
                                                          int64_t count, const uint32_t *__restrict__ partial,
                                                          int64_t *__restrict__ out, int64_t capacity) {
  __shared__ uint32_t s_scan[kBmBlock / 64];
  __shared__ uint32_t s_pos[kBmList];
  uint32_t w[4];
  const int64_t byte0 = ((int64_t)blockIdx.x * kBmBlock + threadIdx.x) * kBmBytes;
  load_bits(bitmap, bytes, count, byte0, w);
  const uint32_t c = (uint32_t)(__popc(w[0]) + __popc(w[1]) + __popc(w[2]) + __popc(w[3]));
  uint32_t total;
  const uint32_t mine = block_exclusive_scan<uint32_t, kBmBlock>(c, s_scan, &total);
  const int64_t base = (int64_t)partial[blockIdx.x];
  const int64_t pos0 = (int64_t)blockIdx.x * kBmSpan;  // first position of this workgroup
  for (uint32_t round = 0; round < total; round += kBmList) {
    uint32_t at = mine;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t x = w[q];
      while (x) {
        const int bit = __ffs((int)x) - 1;
        x &= x - 1;
        if (at - round < (uint32_t)kBmList) s_pos[at - round] = threadIdx.x * (kBmBytes * 8) + q * 32 + bit;
        ++at;
      }
    }
    __syncthreads();
    const uint32_t here = total - round < (uint32_t)kBmList ? total - round : (uint32_t)kBmList;
    for (uint32_t e = threadIdx.x; e < here; e += kBmBlock) {
      const int64_t o = base + round + e;
      if (o < capacity) out[o] = map[pos0 + s_pos[e]];
    }
    __syncthreads();
  }
}

inline int64_t decode_blocks(int64_t count) { return ceil_div(count > 0 ? count : 1, kBmSpan); }

}  // namespace
}  // namespace zen

extern "C" {

size_t zen_bitmap_words(int64_t mapping_n) { return mapping_n > 0 ? (size_t)((mapping_n + 31) / 32) : 0; }

size_t zen_bitmap_rank_words(int64_t numel) {
  if (numel <= 0) return 0;
  const size_t blocks = (size_t)(((numel - 1) >> zen::kBmShift) + 1);
  // the membership lines start on a 16-byte boundary: blocks + 1 rank words are padded to a multiple of four
  return (blocks + 1 + 3) / 4 * 4 + blocks * zen::kBmBlockWords;
}

int zen_bitmap_ranks(const int64_t *mapping_p, int64_t mapping_n, int64_t numel, uint32_t *rank_at, void *stream) {
  using namespace zen;
  if (mapping_n < 0 || mapping_n > 0x7fffffffll || numel <= 0 || numel > 0x7fffffffll)
    return fail(ZEN_EINVAL, "zen_bitmap_ranks: need 0 < numel < 2^31");
  if (!rank_at || (mapping_n > 0 && !mapping_p)) return fail(ZEN_EINVAL, "zen_bitmap_ranks: null pointer");
  if (reinterpret_cast<uintptr_t>(rank_at) & 15u) return fail(ZEN_EINVAL, "zen_bitmap_ranks: table not 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t blocks = ((numel - 1) >> kBmShift) + 1;
  k_bitmap_ranks<<<dim3((unsigned)ceil_div(blocks + 1, kBmBlock)), dim3(kBmBlock), 0, s>>>(mapping_p, mapping_n, blocks,
                                                                                         rank_at);
  ZEN_LAUNCH_CHECK("k_bitmap_ranks");
  k_bitmap_members<<<dim3((unsigned)ceil_div(blocks, kBmBlock)), dim3(kBmBlock), 0, s>>>(
      mapping_p, blocks, rank_at, rank_at + (blocks + 1 + 3) / 4 * 4);
  ZEN_LAUNCH_CHECK("k_bitmap_members");
  return ZEN_OK;
}

int zen_bitmap_encode(const int64_t *mapping_p, int64_t mapping_n, const void *idx, int idx64, int64_t idx_n,
                      const int64_t *idx_n_dev, const uint32_t *rank_at, int64_t numel, uint32_t *bitmap_words,
                      int32_t *status, void *stream) {
  using namespace zen;
  if (mapping_n < 0 || mapping_n > 0x7fffffffll || idx_n < 0) return fail(ZEN_EINVAL, "zen_bitmap_encode: bad size");
  if (!status || (mapping_n > 0 && (!mapping_p || !bitmap_words)) || (idx_n > 0 && !idx))
    return fail(ZEN_EINVAL, "zen_bitmap_encode: null pointer");
  if (rank_at && (numel <= 0 || numel > 0x7fffffffll || (reinterpret_cast<uintptr_t>(rank_at) & 15u)))
    return fail(ZEN_EINVAL, "zen_bitmap_encode: a rank dictionary needs its numel (below 2^31) and 16-byte alignment");
  if (reinterpret_cast<uintptr_t>(bitmap_words) & 3u) return fail(ZEN_EINVAL, "zen_bitmap_encode: bitmap not 4-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  launch_fill<uint32_t>(bitmap_words, 0u, zen_bitmap_words(mapping_n), s);
  ZEN_LAUNCH_CHECK("zen_bitmap_encode: clear");
  if (idx_n == 0) return ZEN_OK;
  const int64_t blocks = ceil_div(idx_n, kBmBlock);
  if (blocks > 0x7fffffffll) return fail(ZEN_EINVAL, "zen_bitmap_encode: too many indices");
  const int64_t rank_blocks = rank_at ? ((numel - 1) >> kBmShift) + 1 : 0;
  if (idx64)
    k_bitmap_mark<int64_t><<<dim3((unsigned)blocks), dim3(kBmBlock), 0, s>>>(
        mapping_p, mapping_n, static_cast<const int64_t *>(idx), idx_n, idx_n_dev, rank_at, rank_blocks,
        bitmap_words, status);
  else
    k_bitmap_mark<int32_t><<<dim3((unsigned)blocks), dim3(kBmBlock), 0, s>>>(
        mapping_p, mapping_n, static_cast<const int32_t *>(idx), idx_n, idx_n_dev, rank_at, rank_blocks,
        bitmap_words, status);
  ZEN_LAUNCH_CHECK("k_bitmap_mark");
  return ZEN_OK;
}

size_t zen_bitmap_decode_workspace(int64_t mapping_n) {
  return zen::align_up((size_t)zen::decode_blocks(mapping_n) * sizeof(uint32_t), 256);
}

int zen_bitmap_decode(const int64_t *mapping_p, int64_t mapping_n, const uint8_t *bitmap, int64_t bitmap_bytes,
                      int64_t *out, int64_t capacity, int64_t *out_count, void *workspace, size_t workspace_bytes,
                      int32_t *status, void *stream) {
  using namespace zen;
  if (mapping_n < 0 || mapping_n > 0x7fffffffll || capacity < 0 || bitmap_bytes < 0)
    return fail(ZEN_EINVAL, "zen_bitmap_decode: bad size");
  if (bitmap_bytes < (mapping_n + 7) / 8)  // the reference's mask would be shorter than the list it indexes
    return fail(ZEN_EINVAL, "zen_bitmap_decode: bitmap shorter than the mapping");
  if (!out_count || !status || !workspace || (mapping_n > 0 && (!mapping_p || !bitmap)) || (capacity > 0 && !out))
    return fail(ZEN_EINVAL, "zen_bitmap_decode: null pointer");
  if (workspace_bytes < zen_bitmap_decode_workspace(mapping_n))
    return fail(ZEN_EWORKSPACE, "zen_bitmap_decode: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint32_t *partial = static_cast<uint32_t *>(workspace);
  const int64_t blocks = decode_blocks(mapping_n);
  k_bitmap_count<<<dim3((unsigned)blocks), dim3(kBmBlock), 0, s>>>(bitmap, bitmap_bytes, mapping_n, partial);
  ZEN_LAUNCH_CHECK("k_bitmap_count");
  k_bitmap_scan<<<dim3(1), dim3(1024), 0, s>>>(partial, (uint32_t)blocks, capacity, out_count, status);
  ZEN_LAUNCH_CHECK("k_bitmap_scan");
  k_bitmap_emit<<<dim3((unsigned)blocks), dim3(kBmBlock), 0, s>>>(mapping_p, bitmap, bitmap_bytes, mapping_n, partial,
                                                                 out, capacity);
  ZEN_LAUNCH_CHECK("k_bitmap_emit");
  return ZEN_OK;
}

}  // extern "C"
