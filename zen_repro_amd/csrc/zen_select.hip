// Magnitude selection: exact k-th largest |g| by radix select over the
// magnitude bit pattern (train.py:81-82), the masked dense copy
// (train.py:83), and the ordered single-pass compaction that turns a dense
// tensor into ascending (index, value) lists (comm.py:47-50).
#include <math.h>

#include <mutex>

#include "zen_select.h"

namespace zen {
namespace {

// ------------------------------------------------------------ radix select

constexpr int kHistBins = 2048;
constexpr int kHistBlock = 256;
constexpr int kSampleLog2Min = 6, kSampleLog2Max = 10;  // the sample is one 16-byte vector in 64 ... 1024
constexpr int64_t kSampleHits = 7000;  // sample elements wanted at or above the threshold

// How thin the sample is (one vector of V elements in 2^log2) and the rank looked for in it.
struct SamplePlan {
  int log2;
  int64_t nblocks;
  uint32_t rank;
};
inline SamplePlan sample_plan(int64_t n, int64_t k, int V) {
  SamplePlan sp;
  const int64_t nvec = ceil_div(n, V);
  // The sample is as thin as leaves about kSampleHits of its elements above the threshold (their count then
  // scatters by 1.2 %, and the six deviations allowed for below cost 7 % more candidates): a thicker one
  // lengthens the load and histogram phases and buys nothing.
  sp.log2 = kSampleLog2Max;
  while (sp.log2 > kSampleLog2Min && (k >> sp.log2) < kSampleHits) --sp.log2;
  sp.nblocks = ceil_div(nvec, 1ll << sp.log2);
  // rank to look for in the sample: the expected one plus six standard
  // deviations of a binomial count, so that the full tensor almost surely holds
  // at least k elements at or above the bin found (callers verify and retry)
  const double expect = (double)k * ((double)sp.nblocks * V) / (double)n;
  const double want = expect + 6.0 * sqrt(expect) + 16.0;
  sp.rank = want > 4.0e9 ? 0xffffffffu : (uint32_t)want;
  return sp;
}

struct TopkState {
  uint32_t prefix;    // key bits fixed so far (right aligned)
  uint32_t k_rem;     // rank still to find among elements matching the prefix
  uint32_t count_gt;  // elements known to be strictly larger than any match
  uint32_t pad;
};

__global__ void k_topk_init(TopkState *st, uint32_t *hist, uint32_t k) {
  for (int i = threadIdx.x; i < kHistBins; i += blockDim.x) hist[i] = 0;
  if (threadIdx.x == 0) {
    st->prefix = 0;
    st->k_rem = k;
    st->count_gt = 0;
    st->pad = 0;
  }
}

// Histogram of the digit (key >> shift) & (2^width - 1) over elements whose
// higher bits equal the prefix found so far.
template <typename S, bool ALIGNED>
__global__ __launch_bounds__(kHistBlock) void k_topk_hist(const S *__restrict__ in, int64_t n_max,
                                                          const uint32_t *__restrict__ n_dev,
                                                          const TopkState *__restrict__ st, int shift,
                                                          int width, int pass,
                                                          uint32_t *__restrict__ hist) {
  constexpr int V = VecOf<S>::kN;
  __shared__ uint32_t bins[kHistBins];
  int64_t n = n_max;
  if (n_dev && (int64_t)*n_dev < n) n = (int64_t)*n_dev;
  for (int i = threadIdx.x; i < kHistBins; i += kHistBlock) bins[i] = 0;
  __syncthreads();
  const uint32_t prefix = st->prefix;
  const uint32_t digit_mask = (1u << width) - 1u;
  const int upper = shift + width;
  const int64_t nvec = (n + V - 1) / V;
  for (int64_t v = blockIdx.x * (int64_t)kHistBlock + threadIdx.x; v < nvec;
       v += (int64_t)gridDim.x * kHistBlock) {
    S e[V];
    const int live = load_vec<S, ALIGNED>(in, v * V, n, e);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const uint32_t key = e[i] & KeyOf<S>::kMask;
      const bool take = i < live && (pass == 0 || (key >> upper) == prefix);
      if (take) atomicAdd(&bins[(key >> shift) & digit_mask], 1u);
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kHistBins; i += kHistBlock) {
    const uint32_t c = bins[i];
    if (c) atomicAdd(&hist[i], c);
  }
}

// One block: find the digit that holds the k_rem-th largest match, extend the
// prefix, clear the histogram for the next pass.  On the last pass the result
// goes to thr_out as (prefix << final_shift, number of elements >= it).  Fewer
// than k_rem matches: thr_out = (0, matches) and `short_bit` is raised.
__global__ __launch_bounds__(kHistBlock) void k_topk_pick(TopkState *st, uint32_t *hist, int width, int last,
                                                          int final_shift, uint32_t *thr_out, int32_t *status,
                                                          int short_bit) {
  constexpr int kPer = kHistBins / kHistBlock;
  __shared__ uint32_t smem[kHistBlock / 64 + 1];
  const uint32_t prefix = st->prefix, k_rem = st->k_rem, count_gt = st->count_gt;
  // thread t owns the bins kHistBins-1-(t*kPer+j): walking from the top bin down
  uint32_t c[kPer];
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    c[j] = hist[kHistBins - 1 - (threadIdx.x * kPer + j)];
    mine += c[j];
  }
  uint32_t total;
  uint32_t above = block_exclusive_scan<uint32_t, kHistBlock>(mine, smem, &total);
  __syncthreads();
  if (total < k_rem) {
    if (threadIdx.x == 0) {
      st->prefix = 0;
      if (last) {
        thr_out[0] = 0;
        thr_out[1] = count_gt + total;
      }
      if (short_bit) atomicOr(status, short_bit);
    }
  } else {
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      if (above < k_rem && k_rem <= above + c[j]) {
        const uint32_t bin = kHistBins - 1 - (threadIdx.x * kPer + j);
        const uint32_t np = (prefix << width) | bin;
        st->prefix = np;
        st->k_rem = k_rem - above;
        st->count_gt = count_gt + above;
        if (last) {
          thr_out[0] = np << final_shift;
          thr_out[1] = count_gt + above + c[j];
        }
      }
      above += c[j];
    }
  }
#pragma unroll
  for (int j = 0; j < kPer; ++j) hist[kHistBins - 1 - (threadIdx.x * kPer + j)] = 0;
}

// Histogram of the top 15 key bits (for bf16: the whole key) over a sample: one
// 16-byte vector out of every 2^block_log2 consecutive vectors, at a
// pseudo-random place inside its block so that regular layouts (rows, columns)
// are not sampled in lockstep.  The block's histogram lives in LDS as 32768
// 16-bit counters packed two per word; a block never sees more than 65535
// sample elements, so they cannot overflow into each other.
constexpr int kFineBins = 32768;
constexpr int kSampleBlock = 1024;

// Device-wide atomics on one 128-byte line are carried out one after the other (about 10 ns each), and the
// populated part of a magnitude histogram is a few hundred neighbouring bins.  So neighbouring bins are kept
// 2 KiB apart in the global histogram.
__device__ inline uint32_t fine_place(uint32_t bin) { return ((bin & 63u) << 9) | (bin >> 6); }

// Run by one whole block once the histogram is complete: the lowest fine bin b
// such that `rank` sample elements lie in bins >= b; floor_out[0] = lowest key
// of that bin (0 if the sample is too small).

// Walks down from the highest populated bin (hist[kFineBins + 1]) in windows of one bin per thread, with
// consecutive lanes on consecutive words (one workgroup fetching 32768 scattered words past the caches would
// take tens of microseconds), until `rank` sample elements lie at or above a bin.
template <int BLOCK>
__device__ inline void sample_pick_block(const uint32_t *hist, uint32_t rank, int key_shift, uint32_t *floor_out,
                                         uint32_t *smem) {
  int base = (int)load_fresh(&hist[kFineBins + 1]);
  if (base > kFineBins - 1) base = kFineBins - 1;
  uint32_t cum = 0;
  for (;; base -= BLOCK) {
    const int bin = base - (int)threadIdx.x;
    const uint32_t c = bin >= 0 ? load_fresh(&hist[fine_place((uint32_t)bin)]) : 0u;
    uint32_t total;
    const uint32_t above = cum + block_exclusive_scan<uint32_t, BLOCK>(c, smem, &total);
    if (above < rank && rank <= above + c) floor_out[0] = (uint32_t)bin << key_shift;
    cum += total;
    if (cum >= rank) return;
    if (base < BLOCK) break;
  }
  if (threadIdx.x == 0) floor_out[0] = 0;  // the sample is too small
}

// The sample: vector number sample_vec(b) for b = 0 .. nblocks - 1, one out of every 2^block_log2.
__device__ inline int64_t sample_vec(int64_t b, int block_log2) {
  return (b << block_log2) + (poly((uint32_t)b) >> 7 & ((1u << block_log2) - 1u));
}

template <typename S, bool ALIGNED>
__global__ __launch_bounds__(kSampleBlock) void k_sample_hist(const S *__restrict__ in, int64_t n, int block_log2,
                                                              uint32_t *__restrict__ hist, uint32_t rank,
                                                              uint32_t *floor_out) {
  constexpr int V = VecOf<S>::kN;
  constexpr int kShift = KeyOf<S>::kBits - 15;
  // one pad word per 32: the flush below reads 16 consecutive words per thread, which would otherwise put
  // all lanes of a wave on two LDS banks
  __shared__ uint32_t bins[kFineBins / 2 + kFineBins / 64];
  __shared__ uint32_t smem[kSampleBlock / 64 + 1];
  __shared__ bool s_last;
  for (int i = threadIdx.x; i < kFineBins / 2 + kFineBins / 64; i += kSampleBlock) bins[i] = 0;
  __syncthreads();
  const int64_t nvec = (n + V - 1) / V;
  const int64_t nblocks = (nvec + (1ll << block_log2) - 1) >> block_log2;
  for (int64_t b = blockIdx.x * (int64_t)kSampleBlock + threadIdx.x; b < nblocks;
       b += (int64_t)gridDim.x * kSampleBlock) {
    const int64_t v = sample_vec(b, block_log2);
    if (v >= nvec) continue;
    S e[V];
    const int live = load_vec<S, ALIGNED>(in, v * V, n, e);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      if (i < live) {
        const uint32_t bin = (e[i] & KeyOf<S>::kMask) >> kShift;
        atomicAdd(&bins[(bin >> 1) + (bin >> 6)], 1u << (16 * (bin & 1u)));
      }
    }
  }
  __syncthreads();
  // Only the top of the histogram matters (the rank looked for is a small fraction of the sample), and a
  // global atomic per populated bin and block is what this kernel would spend its time on.  So a block adds
  // its bins from the top down only until it has added 16 times its share of the rank: counts further down
  // stay too low, which can only make the floor lower (more candidates), never higher.
  {
    constexpr int kWords = kFineBins / 2 / kSampleBlock;
    const uint64_t lim64 = 16ull * rank / gridDim.x + 1024ull;
    const uint32_t limit = lim64 > 0xffffffffull ? 0xffffffffu : (uint32_t)lim64;
    uint32_t c[kWords];
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kWords; ++j) {
      const int w = kFineBins / 2 - 1 - (threadIdx.x * kWords + j);
      c[j] = bins[w + (w >> 5)];
      mine += (c[j] & 0xffffu) + (c[j] >> 16);
    }
    uint32_t total;
    uint32_t above = block_exclusive_scan<uint32_t, kSampleBlock>(mine, smem, &total);
    // the highest populated bin of the block belongs to the first thread that has anything
    if (mine && above == 0) {
      int top = 0;
#pragma unroll
      for (int j = kWords - 1; j >= 0; --j) {
        const int w = kFineBins / 2 - 1 - (threadIdx.x * kWords + j);
        if (c[j] & 0xffffu) top = 2 * w;
        if (c[j] >> 16) top = 2 * w + 1;
      }
      atomicMax(&hist[kFineBins + 1], (uint32_t)top);
    }
#pragma unroll
    for (int j = 0; j < kWords; ++j) {
      const int w = kFineBins / 2 - 1 - (threadIdx.x * kWords + j);
      const uint32_t hi = c[j] >> 16, lo = c[j] & 0xffffu;
      if (hi && above < limit) atomicAdd(&hist[fine_place(2 * w + 1)], hi);
      above += hi;
      if (lo && above < limit) atomicAdd(&hist[fine_place(2 * w)], lo);
      above += lo;
    }
  }
  // The block that finishes last reads the threshold off the complete histogram (hist[kFineBins] counts
  // finished blocks).  The adds above return nothing, so they are all in flight together.  They are carried
  // out where device-wide atomics are carried out; every wave waits until its own have been acknowledged
  // (a device-scope fence would also write the whole L2 back, once per wave) before this block's count goes
  // up, and the reader loads from that same place (load_fresh).
  wait_global_acks();
  __syncthreads();
  if (threadIdx.x == 0) s_last = atomicAdd(&hist[kFineBins], 1u) == gridDim.x - 1;
  __syncthreads();
  if (!s_last) return;
  sample_pick_block<kSampleBlock>(hist, rank, kShift, floor_out, smem);
}

// Run by one whole block (BLOCK threads) over the complete candidate
// histogram (bin = min((key - floor) >> shift, kCandBins-1), kCandRows partial
// rows): the exact k-th largest key when the bins are single keys (shift 0),
// else the lowest key of its bin.  thr_out = (key, number of candidates >=
// key).  Too few candidates, or the k-th lies in the clipped last bin:
// ZEN_STAT_RETRY.
// Place of a candidate bin inside its row of the global histogram: neighbours 256 bytes apart (see fine_place).
constexpr uint32_t kCandCols = kCandBins / 32;
static_assert(kCandBins % 32 == 0, "bins are laid out in 32 groups");
__device__ inline uint32_t cand_place(uint32_t bin) { return (bin & 31u) * kCandCols + (bin >> 5); }
__device__ inline uint32_t cand_bin_at(uint32_t place) { return ((place % kCandCols) << 5) | (place / kCandCols); }

template <int BLOCK>
__device__ inline void cand_pick_block(const uint32_t *hist, uint32_t base, uint32_t k, int shift,
                                       uint32_t *thr_out, int32_t *status, uint32_t *smem, uint32_t *s_sum,
                                       uint32_t *above_out = nullptr) {
  constexpr int kPer = kCandBins / BLOCK;
  // the rows are summed into s_sum (kCandBins words of LDS) with consecutive lanes on consecutive words
  __syncthreads();
  for (int i = threadIdx.x; i < kCandBins; i += BLOCK) {
    uint32_t sum = 0;
#pragma unroll
    for (int row = 0; row < kCandRows; ++row) sum += load_fresh(&hist[row * kCandBins + i]);
    s_sum[cand_bin_at((uint32_t)i)] = sum;
  }
  __syncthreads();
  uint32_t c[kPer];
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    c[j] = s_sum[kCandBins - 1 - (threadIdx.x * kPer + j)];
    mine += c[j];
  }
  uint32_t total;
  uint32_t above = block_exclusive_scan<uint32_t, BLOCK>(mine, smem, &total);
  if (total < k) {
    if (threadIdx.x == 0) {
      thr_out[0] = 0;
      thr_out[1] = total;
      atomicOr(status, ZEN_STAT_RETRY);
    }
  } else {
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      if (above < k && k <= above + c[j]) {
        const uint32_t bin = kCandBins - 1 - (threadIdx.x * kPer + j);
        thr_out[0] = base + (bin << shift);
        thr_out[1] = above + c[j];
        if (above_out) *above_out = above;  // candidates in the bins above the k-th's
        if (bin == kCandBins - 1) atomicOr(status, ZEN_STAT_RETRY);
      }
      above += c[j];
    }
  }
}

// ------------------------------------------------------------- masked copy

template <typename S, bool ALIGNED>
__global__ __launch_bounds__(256) void k_compress(const S *__restrict__ in, int64_t n,
                                                  const uint32_t *__restrict__ thr, S *__restrict__ out) {
  constexpr int V = VecOf<S>::kN;
  const uint32_t t = thr[0];
  const int64_t nvec = (n + V - 1) / V;
  for (int64_t v = blockIdx.x * (int64_t)256 + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * 256) {
    S e[V];
    const int live = load_vec<S, ALIGNED>(in, v * V, n, e);
#pragma unroll
    for (int i = 0; i < V; ++i)
      if ((e[i] & KeyOf<S>::kMask) < t) e[i] = 0;
    if (ALIGNED && live == V) {
      uint4 q;
      __builtin_memcpy(&q, e, 16);
      *reinterpret_cast<uint4 *>(out + v * V) = q;
    } else {
      for (int i = 0; i < live; ++i) out[v * V + i] = e[i];
    }
  }
}

}  // namespace

// ------------------------------------------------------ stream compaction
//
// A tile is `subs` consecutive sub-tiles; in a sub-tile every thread owns
// kSelVecs consecutive 16-byte vectors (64 contiguous bytes), so element order
// is thread order and one block scan of per-thread counts places everything.
// A block walks its tile once, staging the selected (index, value) pairs in
// LDS in ascending order; only then does it need its place in the output.
// Ordered mode gets it from the tile-prefix protocol (the output is ascending
// in the index); unordered mode reserves a range with one atomic add (tiles
// land in arrival order, each tile's entries stay ascending), which callers
// that sort afterwards prefer because no tile ever waits.  The LDS stage makes
// the write-out coalesced.  A tile with more selected elements than the stage
// holds is walked a second time and written directly.
//
// A CDNA compute unit retires 64 lane-operations per clock while HBM delivers
// about 8 bytes per clock and unit, so a bf16 stream has ~16 operations per
// element before the vector ALU, not memory, sets the pace.  The predicate is
// therefore evaluated two bf16 at a time on packed words (3 operations per
// pair), the flags of a thread's 32 elements end in one register, and only the
// few selected elements take the longer extraction path.
// The input is a dense tensor (an element's index is its position) or a list
// (src_idx gives the index carried by each element).

constexpr int kSelStage = 3072;    // staged pairs per tile
constexpr int kReserveShift = 40;  // unordered mode: tiles done above, entries reserved below

// Inclusive prefix sum across the 64 lanes with DPP row shifts and broadcasts.
__device__ inline uint32_t wave_inclusive_scan_dpp(uint32_t x) {
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, false);  // row_shr:1
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, false);  // row_shr:2
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xf, 0xf, false);  // row_shr:4
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xf, 0xf, false);  // row_shr:8
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xa, 0xf, false);  // row_bcast:15 -> rows 1,3
  x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xc, 0xf, false);  // row_bcast:31 -> rows 2,3
  return x;
}

// Flags of the elements a thread owns in one sub-tile, one bit per element,
// plus the translation between bit positions and element offsets.
template <typename S>
struct Flags;

// bf16: element (vector j, word w, half h) sits at bit 4j + w + 16h, i.e. the
// even elements fill the low half-word and the odd ones the high half-word.
template <>
struct Flags<uint16_t> {
  static constexpr int kElems = kSelVecs * 8;
  static __device__ inline uint32_t build(const uint4 (&q)[kSelVecs], uint32_t floor_key) {
    // per 16-bit lane: key + (0x8000 - floor) carries into bit 15 iff key >= floor
    const uint32_t c = (0x8000u - floor_key) * 0x00010001u;
    uint32_t x = 0;
#pragma unroll
    for (int j = 0; j < kSelVecs; ++j) {
      const uint32_t m0 = ((q[j].x & 0x7fff7fffu) + c) & 0x80008000u;
      const uint32_t m1 = ((q[j].y & 0x7fff7fffu) + c) & 0x80008000u;
      const uint32_t m2 = ((q[j].z & 0x7fff7fffu) + c) & 0x80008000u;
      const uint32_t m3 = ((q[j].w & 0x7fff7fffu) + c) & 0x80008000u;
      const uint32_t v = (m0 >> 15) | (m1 >> 14) | (m2 >> 13) | (m3 >> 12);  // bits 0-3 and 16-19
      x |= v << (4 * j);
    }
    return x;
  }
  // flags of the elements whose offset is below `count`
  static __device__ inline uint32_t below(int count) {
    const int a = (count >> 3) * 4 + ((count & 7) >> 1), h = count & 1;
    return (uint32_t)((1ull << (a + h)) - 1ull) | ((uint32_t)((1ull << a) - 1ull) << 16);
  }
  static __device__ inline int offset_of(int bit) {  // element offset of a flag bit
    const int a = bit & 15;
    return ((a >> 2) << 3) + ((a & 3) << 1) + (bit >> 4);
  }
  static __device__ inline uint32_t vec_mask(int j) { return (0xfu << (4 * j)) * 0x00010001u; }  // flags of vector j
  // where the element of flag `bit` sits relative to the thread's first element of the sub-tile, when vector j
  // of thread t starts at element (j * kSelBlock + t) * 8: bit = 4j + w + 16h is element 2w + h of vector j
  static __device__ inline uint32_t elem_step(uint32_t bit) {
    const uint32_t a = bit & 15u;
    return (a >> 2) * (uint32_t)(kSelBlock * 8) + ((a & 3u) << 1) + (bit >> 4);
  }
  static __device__ inline uint16_t pick(const uint4 (&q)[kSelVecs], uint32_t bit);
};

// fp32: element e sits at bit e.
template <>
struct Flags<uint32_t> {
  static constexpr int kElems = kSelVecs * 4;
  static __device__ inline uint32_t build(const uint4 (&q)[kSelVecs], uint32_t floor_key) {
    uint32_t x = 0;
#pragma unroll
    for (int j = 0; j < kSelVecs; ++j) {
      x |= (uint32_t)((q[j].x & 0x7fffffffu) >= floor_key) << (4 * j);
      x |= (uint32_t)((q[j].y & 0x7fffffffu) >= floor_key) << (4 * j + 1);
      x |= (uint32_t)((q[j].z & 0x7fffffffu) >= floor_key) << (4 * j + 2);
      x |= (uint32_t)((q[j].w & 0x7fffffffu) >= floor_key) << (4 * j + 3);
    }
    return x;
  }
  static __device__ inline uint32_t below(int count) { return (uint32_t)((1ull << count) - 1ull); }
  static __device__ inline int offset_of(int bit) { return bit; }
  static __device__ inline uint32_t vec_mask(int j) { return 0xfu << (4 * j); }  // flags of vector j
  static __device__ inline uint32_t elem_step(uint32_t bit) {  // bit = 4j + w is element w of vector j
    return (bit >> 2) * (uint32_t)(kSelBlock * 4) + (bit & 3u);
  }
  static __device__ inline uint32_t pick(const uint4 (&q)[kSelVecs], uint32_t bit);
};

template <typename S, typename I, bool ALIGNED, bool STAGED>
__device__ inline uint32_t select_walk_tile(const S *__restrict__ in, int64_t n, uint32_t floor_key,
                                            int64_t tile_base, int subs, const int32_t *__restrict__ src_idx,
                                            uint32_t *s_wave, int32_t *st_idx, S *st_val, uint32_t *s_hist,
                                            I *__restrict__ out_idx, S *__restrict__ out_val, uint64_t out_base,
                                            int64_t capacity) {
  constexpr int V = VecOf<S>::kN;
  constexpr int kChunk = Flags<S>::kElems;  // elements per thread and sub-tile
  constexpr int kSub = kSelBlock * kChunk;
  const int wave = threadIdx.x >> 6;
  uint32_t running = 0;
  for (int sub = 0; sub < subs; ++sub) {
    const int64_t sub_base = tile_base + (int64_t)sub * kSub;
    if (sub_base >= n) break;
    const int64_t first = sub_base + (int64_t)threadIdx.x * kChunk;
    uint4 q[kSelVecs];
    if (ALIGNED && first + kChunk <= n) {
      const uint4 *src = reinterpret_cast<const uint4 *>(in + first);
#pragma unroll
      for (int j = 0; j < kSelVecs; ++j) q[j] = src[j];
    } else {
#pragma unroll
      for (int j = 0; j < kSelVecs; ++j) {
        S e[V];
        load_vec<S, false>(in, first + j * V, n, e);
        __builtin_memcpy(&q[j], e, 16);
      }
    }
    uint32_t x = Flags<S>::build(q, floor_key);
    if (first + kChunk > n) x &= first < n ? Flags<S>::below((int)(n - first)) : 0u;
    const uint32_t cnt = (uint32_t)__popc(x);
    // block-wide exclusive prefix of cnt
    const uint32_t incl = wave_inclusive_scan_dpp(cnt);
    if ((threadIdx.x & 63) == 63) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = running + incl - cnt, total = 0;
#pragma unroll
    for (int w = 0; w < kSelBlock / 64; ++w) {
      const uint32_t t = s_wave[w];
      if (w < wave) before += t;
      total += t;
    }
    __syncthreads();
    const uint32_t all = x;
    while (x) {
      const int bit = __ffs((int)x) - 1;
      x &= x - 1;
      const int off = Flags<S>::offset_of(bit);
      const uint32_t pos = before + (uint32_t)__popc(all & Flags<S>::below(off));
      const S v = in[first + off];  // just streamed through the cache; selected elements are few
      if (STAGED) {
        if (s_hist) {
          const uint32_t bin = ((v & KeyOf<S>::kMask) - floor_key) >> (sizeof(S) == 2 ? 0 : 16);
          atomicAdd(&s_hist[bin < (uint32_t)kCandBins - 1u ? bin : (uint32_t)kCandBins - 1u], 1u);
        }
        if (pos < (uint32_t)kSelStage) {
          st_idx[pos] = (int32_t)(first + off);
          st_val[pos] = v;
        }
      } else if (out_base + pos < (uint64_t)capacity) {
        out_idx[out_base + pos] = (I)(src_idx ? src_idx[first + off] : first + off);
        out_val[out_base + pos] = v;
      }
    }
    running += total;
  }
  return running;
}

template <typename S, typename I, bool ALIGNED, bool ORDERED>
__global__ __launch_bounds__(kSelBlock) void k_select_compact(
    const S *__restrict__ in, int64_t n_max, const uint32_t *__restrict__ n_dev, const uint32_t *__restrict__ thr,
    const int32_t *__restrict__ src_idx, I *__restrict__ out_idx, S *__restrict__ out_val, int64_t capacity,
    ScanState st, int ntiles, int subs, uint32_t *cand_hist, uint32_t pick_k, uint32_t *pick_thr,
    int64_t *out_count, uint32_t *out_count32, int32_t *status) {
  constexpr int kSub = kSelBlock * Flags<S>::kElems;
  __shared__ uint32_t s_wave[kSelBlock / 64];
  __shared__ uint64_t s_bcast;
  __shared__ int s_tile;
  __shared__ int32_t st_idx[kSelStage];
  __shared__ S st_val[kSelStage];
  __shared__ uint32_t s_hist[ORDERED ? 1 : kCandBins];
  uint32_t *hist = (!ORDERED && cand_hist) ? s_hist : nullptr;
  if (hist) {
    for (int i = threadIdx.x; i < kCandBins; i += kSelBlock) s_hist[i] = 0;
    __syncthreads();
  }
  int64_t n = n_max;
  if (n_dev && (int64_t)*n_dev < n) n = (int64_t)*n_dev;
  uint32_t floor_key = thr ? thr[0] : 1u;
  if (floor_key == 0) floor_key = 1u;  // zeros are never selected
  if (floor_key > KeyOf<S>::kMask) floor_key = KeyOf<S>::kMask + 1u;  // nothing qualifies

  // ordered: tiles are taken by ticket, so that every earlier tile already runs
  {
    int tile = (int)blockIdx.x;
    if (ORDERED) {
      if (threadIdx.x == 0) s_tile = (int)atomicAdd(st.ticket, 1u);
      __syncthreads();
      tile = s_tile;
    }
    if (tile >= ntiles) return;
    const int64_t tile_base = (int64_t)tile * subs * kSub;
    const uint32_t found = select_walk_tile<S, I, ALIGNED, true>(in, n, floor_key, tile_base, subs, src_idx, s_wave,
                                                                 st_idx, st_val, hist, out_idx, out_val, 0, capacity);
    uint64_t tile_start, all = 0;
    bool last;
    if (ORDERED) {
      tile_start = lookback_exclusive(st, tile, found, status, &s_bcast);
      last = tile == ntiles - 1;
      all = tile_start + found;
    } else {
      if (threadIdx.x == 0)
        s_bcast = __hip_atomic_fetch_add(st.desc, (1ull << kReserveShift) | found, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      const uint64_t old = s_bcast;
      tile_start = old & ((1ull << kReserveShift) - 1);
      last = (int)(old >> kReserveShift) == ntiles - 1;  // every other tile has reserved already
      all = tile_start + found;
    }
    if (last && threadIdx.x == 0) {
      if (out_count) *out_count = (int64_t)all;
      if (out_count32) *out_count32 = (uint32_t)(all < (uint64_t)capacity ? all : (uint64_t)capacity);
      if (all > (uint64_t)capacity) atomicOr(status, ZEN_STAT_CAPACITY);
    }
    if (found <= (uint32_t)kSelStage) {
      for (uint32_t i = threadIdx.x; i < found; i += kSelBlock) {
        const uint64_t pos = tile_start + i;
        if (pos < (uint64_t)capacity) {
          const int32_t at = st_idx[i];
          out_idx[pos] = (I)(src_idx ? src_idx[at] : at);
          out_val[pos] = st_val[i];
        }
      }
    } else {
      select_walk_tile<S, I, ALIGNED, false>(in, n, floor_key, tile_base, subs, src_idx, s_wave, st_idx, st_val,
                                             nullptr, out_idx, out_val, tile_start, capacity);
    }
  }
  if (hist) {
    // spread over kCandRows partial histograms: fewer blocks meet on one counter
    __syncthreads();
    uint32_t *row = cand_hist + (size_t)(blockIdx.x % kCandRows) * kCandBins;
    for (int i = threadIdx.x; i < kCandBins; i += kSelBlock) {
      const uint32_t c = s_hist[i];
      if (c) atomicAdd(&row[cand_place((uint32_t)i)], c);  // nothing returned: the adds are in flight together
    }
    if (pick_thr) {
      // The block that finishes last reads the exact threshold off the complete histogram
      // (cand_hist[kCandRows * kCandBins] counts finished blocks).
      __shared__ bool s_last;
      // the adds are carried out (where device-wide atomics are) before the count goes up; no device-scope
      // fence: that would write the L2 back once per wave
      wait_global_acks();
      __syncthreads();
      if (threadIdx.x == 0) s_last = atomicAdd(&cand_hist[kCandRows * kCandBins], 1u) == (uint32_t)ntiles - 1u;
      __syncthreads();
      if (s_last) {
        cand_pick_block<kSelBlock>(cand_hist, floor_key, pick_k, KeyOf<S>::kBits == 15 ? 0 : 16, pick_thr, status,
                                   reinterpret_cast<uint32_t *>(st_idx), s_hist);
      }
    }
  }
}

// Sub-tiles per tile: large tiles for large inputs (few descriptors, few
// atomics), but never so large that the grid falls below a few workgroups per
// compute unit.
static int select_subs(int64_t n, int dtype) {
  const int v = dtype == ZEN_BF16 ? 8 : 4;
  const int64_t sub = (int64_t)kSelBlock * kSelVecs * v;
  int subs = 16;
  while (subs > 1 && ceil_div(n, sub * subs) < 2048) subs >>= 1;
  return subs;
}

size_t select_scratch_bytes(int64_t n, int dtype) {
  const int v = dtype == ZEN_BF16 ? 8 : 4;
  const int64_t tile = (int64_t)kSelBlock * kSelVecs * v * select_subs(n > 0 ? n : 1, dtype);
  const int64_t ntiles = ceil_div(n > 0 ? n : 1, tile);
  return align_up(scan_words(ntiles) * sizeof(unsigned long long), 256);
}

template <typename S, typename I>
static int select_launch(const SelectArgs &a, hipStream_t stream) {
  constexpr int V = VecOf<S>::kN;
  const int subs = select_subs(a.n, a.dtype);
  const int64_t tile = (int64_t)kSelBlock * kSelVecs * V * subs;
  const int64_t ntiles = ceil_div(a.n, tile);
  if (ntiles > 0xffffff) return fail(ZEN_EINVAL, "select: too many tiles");
  const ScanState st = scan_state(a.scratch, ntiles);
  launch_fill<unsigned long long>(st.desc, 0ull, a.ordered ? scan_words(ntiles) : 1, stream);
  ZEN_LAUNCH_CHECK("select: clear scan state");
  const S *in = static_cast<const S *>(a.in);
  I *out_idx = static_cast<I *>(a.out_idx);
  S *out_val = static_cast<S *>(a.out_val);
  const bool aligned = (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
  const dim3 grid((unsigned)ntiles), block(kSelBlock);
  ProfScope prof(kProfSelectCompact, stream);
#define ZEN_SELECT_GO(AL, ORD)                                                                                 \
  k_select_compact<S, I, AL, ORD><<<grid, block, 0, stream>>>(in, a.n, a.n_dev, a.thr, a.src_idx, out_idx,   \
                                                              out_val, a.capacity, st, (int)ntiles, subs,    \
                                                              a.cand_hist, (uint32_t)a.pick_k, a.pick_thr,   \
                                                              a.out_count, a.out_count32, a.status)
  if (aligned && a.ordered) ZEN_SELECT_GO(true, true);
  else if (aligned) ZEN_SELECT_GO(true, false);
  else if (a.ordered) ZEN_SELECT_GO(false, true);
  else ZEN_SELECT_GO(false, false);
#undef ZEN_SELECT_GO
  ZEN_LAUNCH_CHECK("k_select_compact");
  return ZEN_OK;
}

int select_compact(const SelectArgs &a, hipStream_t stream) {
  if (a.dtype == ZEN_BF16)
    return a.idx64 ? select_launch<uint16_t, int64_t>(a, stream) : select_launch<uint16_t, int32_t>(a, stream);
  return a.idx64 ? select_launch<uint32_t, int64_t>(a, stream) : select_launch<uint32_t, int32_t>(a, stream);
}

// ------------------------------------------- compaction in no particular order
//
// The fused encode does not need its candidates in any order: they are sorted
// by hash slot afterwards.  So this kernel runs as a few persistent workgroups
// per compute unit, reads the tensor with fully coalesced non-temporal loads
// (the next sub-tile is already in flight while the current one is examined),
// needs one barrier per sub-tile (the wave totals are double buffered), and
// stages candidates in LDS until kScatStage of them are there.  A full stage
// is flushed to the coarse slabs (zen_slab_feed.h): ordered by coarse slab
// inside LDS, one reservation per slab, consecutive lanes writing consecutive
// places of a run; the candidate histogram is taken at flush time.

constexpr int kScatStage = 2048;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename S, bool ALIGNED>
__device__ inline void stage_load(const S *__restrict__ in, int64_t n, int64_t sub_base, uint4 (&q)[kSelVecs]) {
  constexpr int V = VecOf<S>::kN;
#pragma unroll
  for (int j = 0; j < kSelVecs; ++j) {
    const int64_t first = sub_base + ((int64_t)j * kSelBlock + threadIdx.x) * V;
    if (ALIGNED && first + V <= n) {
      const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in + first));
      q[j] = make_uint4(v.x, v.y, v.z, v.w);
    } else if (first < n) {
      S e[V];
      load_vec<S, false>(in, first, n, e);  // elements past the end read as zero: never selected
      __builtin_memcpy(&q[j], e, 16);
    } else {
      q[j] = make_uint4(0u, 0u, 0u, 0u);
    }
  }
}

// The same for a 16-byte aligned tensor, without a branch: vector numbers past the last complete vector are
// pulled back onto it (their flags are cleared by the caller).  Loads that sit in branches make the compiler
// wait for every load in flight wherever one of them is needed, and the point of the exercise is to have the
// next two sub-tiles in flight while the current one is examined.
template <typename S>
__device__ inline void stage_load_fast(const S *__restrict__ in, uint32_t last_vec, uint32_t vec0,
                                       uint4 (&q)[kSelVecs]) {
  constexpr int V = VecOf<S>::kN;
#pragma unroll
  for (int j = 0; j < kSelVecs; ++j) {
    uint32_t v = vec0 + (uint32_t)j * kSelBlock + threadIdx.x;
    v = v < last_vec ? v : last_vec;
    const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in + (size_t)v * V));
    q[j] = make_uint4(t.x, t.y, t.z, t.w);
  }
}

// Word w (0..15) of the 64 bytes a thread holds, without indexing registers dynamically.
__device__ inline uint32_t pick_word(const uint4 (&q)[kSelVecs], int w) {
  uint32_t r = 0;
#pragma unroll
  for (int j = 0; j < kSelVecs; ++j) {
    r = w == 4 * j ? q[j].x : r;
    r = w == 4 * j + 1 ? q[j].y : r;
    r = w == 4 * j + 2 ? q[j].z : r;
    r = w == 4 * j + 3 ? q[j].w : r;
  }
  return r;
}
// The element a flag bit stands for, straight from the flag's number (word 4j + w, half h for bf16).
__device__ inline uint16_t Flags<uint16_t>::pick(const uint4 (&q)[kSelVecs], uint32_t bit) {
  const uint32_t w = pick_word(q, (int)(bit & 15u));
  return (uint16_t)((bit >> 4) ? (w >> 16) : (w & 0xffffu));
}
__device__ inline uint32_t Flags<uint32_t>::pick(const uint4 (&q)[kSelVecs], uint32_t bit) {
  return pick_word(q, (int)bit);
}

template <typename S>
__device__ inline S pick_elem(const uint4 (&q)[kSelVecs], int off);
template <>
__device__ inline uint16_t pick_elem<uint16_t>(const uint4 (&q)[kSelVecs], int off) {
  const uint32_t w = pick_word(q, off >> 1);
  return (uint16_t)((off & 1) ? (w >> 16) : (w & 0xffffu));
}
template <>
__device__ inline uint32_t pick_elem<uint32_t>(const uint4 (&q)[kSelVecs], int off) {
  return pick_word(q, off);
}

// Where the candidates go: the coarse slabs of zen_slab_feed.h (two word planes: index, value), or straight to
// wide buckets (zen_wide.h; records of two words: index, value bits).  Either way a destination is kept in
// kCoarseSplit parts with a cursor each.
struct StageSlabs {
  SlabGeom geo;
  CoarseGeom cg;     // wide: groups = buckets, per = 1, cap = entries per part
  uint32_t *cursor;  // part cursors
  uint32_t *words;   // word planes
  uint32_t wide;
};

constexpr int kStageDstMax = 256;  // destinations of a flush, at most (one counter per thread)
static_assert(kStageDstMax == kSelBlock && kCoarseMax <= kStageDstMax, "a thread per destination");

struct StageFlushShared {
  uint32_t cnt[kStageDstMax], pref[kStageDstMax + 1], gbase[kStageDstMax];
  uint32_t scan[kSelBlock / 64 + 1];
  uint16_t dst[kScatStage];
};

// Called by the whole block after a barrier made the staged entries visible.  What k_coarse_scatter does for
// a list, done for the staged candidates: every entry finds its destination (from the level-1 hash slot of
// its index), the stage is put in destination order in place, every destination's run is reserved with one
// atomic and consecutive lanes write consecutive places.  Element 0 is not handed on (index 0 is never
// transmitted: 0 is the table's empty marker, tensor_load_balance.py:31), but counts in the histogram.
template <typename S>
__device__ inline void stage_flush(uint32_t count, int32_t *st_idx, S *st_val, StageFlushShared &fl,
                                   uint32_t *s_hist, uint32_t floor_key, const StageSlabs &out, int32_t *status) {
  constexpr int kPer = kScatStage / kSelBlock;
  constexpr uint32_t kNoDst = 0xffffu;
  static_assert(kScatStage % kSelBlock == 0, "flush layout");
  const uint32_t ndst = out.cg.groups;
  fl.cnt[threadIdx.x] = 0;
  __syncthreads();
  const uint32_t part = blockIdx.x % kCoarseSplit;
  uint32_t t[kPer], d[kPer], r[kPer];
  S v[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const uint32_t e = threadIdx.x + i * kSelBlock;
    d[i] = kNoDst;
    t[i] = r[i] = 0;
    v[i] = 0;
    if (e < count) {
      t[i] = (uint32_t)st_idx[e];
      v[i] = st_val[e];
      if (s_hist) {
        const uint32_t bin = ((v[i] & KeyOf<S>::kMask) - floor_key) >> (sizeof(S) == 2 ? 0 : 16);
        atomicAdd(&s_hist[bin < (uint32_t)kCandBins - 1u ? bin : (uint32_t)kCandBins - 1u], 1u);
      }
      if (t[i] != 0) {
        uint32_t rem;
        const uint32_t bucket = out.geo.bucket_of(out.geo.mod_m(poly(t[i]) + kSeed1));
        d[i] = out.wide ? bucket : SlabGeom::div_small(bucket, out.cg.per, out.cg.inv_per, &rem);
        r[i] = atomicAdd(&fl.cnt[d[i]], 1u);
      }
    }
  }
  __syncthreads();
  {
    const uint32_t c = threadIdx.x < ndst ? fl.cnt[threadIdx.x] : 0u;
    uint32_t total;
    const uint32_t before = block_exclusive_scan<uint32_t, kSelBlock>(c, fl.scan, &total);
    if (threadIdx.x < ndst) {
      fl.pref[threadIdx.x] = before;
      fl.gbase[threadIdx.x] = c ? atomicAdd(&out.cursor[(threadIdx.x * kCoarseSplit + part) * kCoarsePad], c) : 0u;
    }
    if (threadIdx.x == 0) fl.pref[ndst] = total;
  }
  __syncthreads();  // every thread holds its entries in registers: the stage is reordered in place
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    if (d[i] != kNoDst) {
      const uint32_t p = fl.pref[d[i]] + r[i];
      st_idx[p] = (int32_t)t[i];
      st_val[p] = v[i];
      fl.dst[p] = (uint16_t)d[i];
    }
  }
  __syncthreads();
  const uint32_t total = fl.pref[ndst];
  const size_t plane = (size_t)ndst * kCoarseSplit * out.cg.cap;
  S *val_plane = reinterpret_cast<S *>(out.words + plane);
  uint2 *records = reinterpret_cast<uint2 *>(out.words);
  for (uint32_t p = threadIdx.x; p < total; p += kSelBlock) {
    const uint32_t g = fl.dst[p];
    const uint32_t at = fl.gbase[g] + (p - fl.pref[g]);
    if (at < out.cg.cap) {
      const size_t o = (size_t)(g * kCoarseSplit + part) * out.cg.cap + at;
      const uint32_t idx = (uint32_t)st_idx[p];
      if (out.wide) {
        // one 8-byte record per candidate: a run of eight fills two 32-byte sectors (three planes of their
        // own cost three partly filled ones per run, and the scattered stores are what a flush spends its
        // time on)
        records[o] = make_uint2(idx, (uint32_t)st_val[p]);
      } else {
        out.words[o] = idx;
        val_plane[o] = st_val[p];
      }
    } else {
      atomicOr(status, ZEN_STAT_RETRY);  // a slab is full: another path answers
    }
  }
  __syncthreads();
}

// How the sub-tiles (kSelBlock * kSelVecs vectors each) are handed out.  Every workgroup first takes
// `fixed` tiles of kStageBig sub-tiles, tile i of workgroup b being number i * workgroups + b: no counter, and
// the workgroups move through memory side by side (short tiles measured a little faster than long ones).
// The rest of the tensor goes out in short tiles through ticket counters, so that workgroups that ran ahead take more and all finish within one short tile of each
// other.  A device-wide counter serves about 90 tickets per microsecond, and 768 workgroups asking one
// counter every few microseconds would queue up for it: the workgroups form kStageGroups groups (by number
// modulo kStageGroups) with a counter each, and ticket t of group g is short tile number g + t * kStageGroups.
constexpr int kStageBig = 2;    // both tile lengths must be at least 2: the loads run two sub-tiles ahead
constexpr int kStageSmall = 2;
constexpr int kStageGroups = 8;
constexpr int kStageTicketPad = 32;  // words between two ticket counters: a 128-byte line each
struct StageSched {
  uint32_t fixed;        // counter-free tiles per workgroup
  uint32_t fixed_subs;   // sub-tiles they cover together
  uint32_t ticket_tiles; // tiles of kStageSmall sub-tiles after that
};

// LDS of a selecting workgroup that changes hands: the stage with what a flush needs, and after the last
// flush the window of the next call's sample (16-bit counters, two to a word, a pad word per 32).
constexpr int kSampleWindow = 8192;  // bins below a workgroup's largest sample element that it counts
template <typename S>
struct StageRun {
  union {
    struct {
      int32_t idx[kScatStage];
      S val[kScatStage];
      StageFlushShared flush;
    } run;
    uint32_t window[kSampleWindow / 2 + kSampleWindow / 64];
  };
};
static_assert(sizeof(StageRun<uint16_t>) == sizeof(int32_t) * kScatStage + 2 * kScatStage + sizeof(StageFlushShared),
              "the window fits where the stage is");

// The sample of the NEXT call's tensor, taken by the workgroups of this call's selecting kernel when they are
// through with their own tensor: no launch of its own, and nothing that waits.  Every workgroup histograms its
// share of the sample (the vectors k_sample_hist would read) in a window of kSampleWindow exact bins below
// its own largest element (a factor 2^64 in magnitude; what lies further down cannot matter unless the
// workgroup's largest element towers that far above the threshold, and leaving it out only lowers the floor)
// and adds the top of it to the device-wide histogram; the workgroup that finishes last reads the floor off
// the complete histogram, as k_sample_hist's last workgroup does.  The histogram is left as k_sample_hist
// leaves it: the call that picks the sample up clears it.
template <typename S>
__device__ inline void stage_sample_next(const StageSample &smp, uint32_t *window, uint32_t *smem) {
  constexpr int V = VecOf<S>::kN;
  constexpr int kShift = KeyOf<S>::kBits - 15;
  constexpr int kWords = kSampleWindow / 2 / kSelBlock;  // window words per thread (16)
  __shared__ uint32_t s_top;
  __shared__ bool s_last;
  const S *in = static_cast<const S *>(smp.in);
  const int64_t n = smp.n;
  const int64_t nvec = (n + V - 1) / V;
  const int64_t first = (int64_t)blockIdx.x * kSelBlock + threadIdx.x, step = (int64_t)gridDim.x * kSelBlock;
  if (threadIdx.x == 0) s_top = 0;
  for (int i = threadIdx.x; i < kSampleWindow / 2 + kSampleWindow / 64; i += kSelBlock) window[i] = 0;
  __syncthreads();
  uint32_t top = 0;
  for (int64_t b = first; b < smp.nblocks; b += step) {
    const int64_t v = sample_vec(b, smp.block_log2);
    if (v >= nvec) continue;
    S e[V];
    const int live = load_vec<S, false>(in, v * V, n, e);
#pragma unroll
    for (int i = 0; i < V; ++i)
      if (i < live) {
        const uint32_t bin = (e[i] & KeyOf<S>::kMask) >> kShift;
        top = bin > top ? bin : top;
      }
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    const uint32_t o = __shfl_xor(top, d, 64);
    top = o > top ? o : top;
  }
  if ((threadIdx.x & 63) == 0 && top) atomicMax(&s_top, top);
  __syncthreads();
  const uint32_t hi_bin = s_top;
  const uint32_t lo_bin = hi_bin >= (uint32_t)kSampleWindow - 1u ? hi_bin - ((uint32_t)kSampleWindow - 1u) : 0u;
  for (int64_t b = first; b < smp.nblocks; b += step) {  // the same vectors again (they are in the caches now)
    const int64_t v = sample_vec(b, smp.block_log2);
    if (v >= nvec) continue;
    S e[V];
    const int live = load_vec<S, false>(in, v * V, n, e);
#pragma unroll
    for (int i = 0; i < V; ++i)
      if (i < live) {
        const uint32_t bin = (e[i] & KeyOf<S>::kMask) >> kShift;
        if (bin >= lo_bin) {
          const uint32_t w = bin - lo_bin;
          atomicAdd(&window[(w >> 1) + (w >> 6)], 1u << (16 * (w & 1u)));
        }
      }
  }
  __syncthreads();
  {
    // from the top down, until the workgroup has added a few times its share of the rank (see k_sample_hist)
    const uint64_t lim64 = 4ull * smp.rank / gridDim.x + 256ull;
    const uint32_t limit = lim64 > 0xffffffffull ? 0xffffffffu : (uint32_t)lim64;
    uint32_t c[kWords];
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kWords; ++j) {
      const int w = kSampleWindow / 2 - 1 - (threadIdx.x * kWords + j);
      c[j] = window[w + (w >> 5)];
      mine += (c[j] & 0xffffu) + (c[j] >> 16);
    }
    uint32_t total;
    uint32_t above = block_exclusive_scan<uint32_t, kSelBlock>(mine, smem, &total);
    if (threadIdx.x == 0 && total) atomicMax(&smp.hist[kFineBins + 1], hi_bin);
#pragma unroll
    for (int j = 0; j < kWords; ++j) {
      const int w = kSampleWindow / 2 - 1 - (threadIdx.x * kWords + j);
      const uint32_t hi = c[j] >> 16, lo = c[j] & 0xffffu;
      if (hi && above < limit) atomicAdd(&smp.hist[fine_place(lo_bin + 2 * w + 1)], hi);
      above += hi;
      if (lo && above < limit) atomicAdd(&smp.hist[fine_place(lo_bin + 2 * w)], lo);
      above += lo;
    }
  }
  // the adds are carried out before the workgroup counts itself as finished (see k_sample_hist)
  wait_global_acks();
  __syncthreads();
  if (threadIdx.x == 0) s_last = atomicAdd(&smp.hist[kFineBins], 1u) == gridDim.x - 1;
  __syncthreads();
  if (s_last) sample_pick_block<kSelBlock>(smp.hist, smp.rank, kShift, smp.floor_out, smem);
}

template <typename S, bool ALIGNED>
__global__ __launch_bounds__(kSelBlock, 3) void k_select_stage(
    const S *__restrict__ in, int64_t n, const uint32_t *__restrict__ thr, StageSlabs out, uint32_t *ticket,
    StageSched sch, uint32_t *cand_hist, uint32_t pick_k, uint32_t *pick_thr, uint32_t *pick_above,
    uint32_t *thr_copy, uint32_t *clear, uint32_t clear_words, uint32_t floor_margin, StageSample next,
    int32_t *status) {
  constexpr int V = VecOf<S>::kN;
  constexpr int kSub = kSelBlock * kSelVecs * V;
  constexpr int kWaves = kSelBlock / 64;
  // what the kernel before this one needed at zero and nobody needs any more (the sample's histogram): back
  // to zero, a slice per workgroup
  for (uint32_t i = blockIdx.x * kSelBlock + threadIdx.x; i < clear_words; i += gridDim.x * kSelBlock) clear[i] = 0;
  __shared__ uint32_t s_wave[2][kWaves];
  __shared__ uint32_t s_next[2];
  // the stage and what a flush needs; after the last flush, the window of the next call's sample
  __shared__ StageRun<S> s_run;
  int32_t (&st_idx)[kScatStage] = s_run.run.idx;
  S (&st_val)[kScatStage] = s_run.run.val;
  StageFlushShared &s_flush = s_run.run.flush;
  __shared__ uint32_t s_tail;
  __shared__ uint32_t s_pick[kSelBlock / 64 + 1];
  __shared__ uint32_t s_hist[kCandBins];
  uint32_t *hist = cand_hist ? s_hist : nullptr;
  if (hist)
    for (int i = threadIdx.x; i < kCandBins; i += kSelBlock) s_hist[i] = 0;
  uint32_t floor_key = thr ? thr[0] : 1u;
  floor_key = floor_key > floor_margin ? floor_key - floor_margin : 1u;
  if (floor_key == 0) floor_key = 1u;  // zeros are never selected
  if (floor_key > KeyOf<S>::kMask) floor_key = KeyOf<S>::kMask + 1u;  // nothing qualifies
  const int wave = threadIdx.x >> 6;

  // A tile is (first sub-tile, number of sub-tiles); length 0 means there is none.  The current tile and the
  // one after it are always known (the loads run two sub-tiles ahead); the ticket of the tile after those is
  // drawn when the current tile starts and handed to the other threads at its last sub-tile, so the counter
  // has a whole tile's time to answer.  Three register sets take turns: while one sub-tile is examined the loads
  // of the next two are in flight.
  uint32_t cur_first = 0, cur_len = 0, nxt_first = 0, nxt_len = 0;
  auto fixed_tile = [&](uint32_t i, uint32_t &first, uint32_t &len) {
    first = (i * gridDim.x + blockIdx.x) * (uint32_t)kStageBig;
    len = (uint32_t)kStageBig;
  };
  auto ticket_tile = [&](uint32_t j, uint32_t &first, uint32_t &len) {
    first = sch.fixed_subs + j * (uint32_t)kStageSmall;
    len = j < sch.ticket_tiles ? (uint32_t)kStageSmall : 0u;
  };
  const uint32_t group = blockIdx.x % kStageGroups;
  // workgroups of this group: its first tickets are theirs without asking (number blockIdx.x / kStageGroups)
  const uint32_t group_size = (gridDim.x - group + kStageGroups - 1) / kStageGroups;
  uint32_t turn = 0;   // tiles this block has started
  uint32_t par = 0;    // sub-tiles this block has processed
  uint32_t count = 0;  // staged entries
  bool ticket_pending = false;
  uint32_t drawn = 0;  // thread 0: the ticket on its way
  uint32_t far_first = 0, far_len = 0;  // the tile after the next one
  // what the counter returns is kept as it is until it is handed over: any arithmetic on it here would make
  // the wave wait for the answer, and for all its loads in flight with it
  auto draw = [&]() { return atomicAdd(&ticket[group * kStageTicketPad], 1u); };
  auto drawn_tile = [&](uint32_t raw) { return group + (group_size + raw) * kStageGroups; };
  // tile number tn of this block if no ticket is needed for it: counter-free tiles first, then the block's
  // own first short tile
  auto known_tile = [&](uint32_t tn, uint32_t &first, uint32_t &len) {
    if (tn < sch.fixed) {
      fixed_tile(tn, first, len);
      return true;
    }
    if (tn == sch.fixed) {
      ticket_tile(blockIdx.x, first, len);  // = group + (blockIdx.x / kStageGroups) * kStageGroups
      return true;
    }
    return false;
  };
  int64_t sub_base = 0;
  uint32_t sub = 0;
  uint4 qa[kSelVecs], qb[kSelVecs], qc[kSelVecs];

  // complete vectors of the tensor (an aligned tensor's last n % V elements are looked at separately, below)
  constexpr uint32_t kSubVecs = kSelBlock * kSelVecs;
  const uint32_t full_vecs = (uint32_t)(n / V);
  // loads the sub-tile `ahead` places after the current one in the block's sequence; if there is none, an
  // aligned tensor still gets its loads (of the last vector: every wave always has the same number of loads
  // in flight, which lets the compiler wait for exactly the ones it needs)
  auto load_ahead = [&](uint32_t ahead, uint4 (&q)[kSelVecs]) {
    const uint32_t p = sub + ahead;
    const bool here = p < cur_len, there = !here && p - cur_len < nxt_len;
    const uint32_t unit = here ? cur_first + p : nxt_first + p - cur_len;
    if (ALIGNED)
      stage_load_fast<S>(in, full_vecs - 1u, here || there ? unit * kSubVecs : 0xffffffffu - kSubVecs, q);
    else if (here || there)
      stage_load<S, false>(in, n, (int64_t)unit * kSub, q);
  };

  // one sub-tile: cur holds its data, far receives the data of the sub-tile two places on
  auto body = [&](uint4 (&cur)[kSelVecs], uint4 (&far)[kSelVecs]) {
    uint32_t x = Flags<S>::build(cur, floor_key);
    if (ALIGNED) {
      const uint32_t vec0 = (cur_first + sub) * kSubVecs;
      if (vec0 + kSubVecs > full_vecs) {  // the tensor ends inside this sub-tile (or before it)
#pragma unroll
        for (int j = 0; j < kSelVecs; ++j)
          if (vec0 + (uint32_t)j * kSelBlock + threadIdx.x >= full_vecs) x &= ~Flags<S>::vec_mask(j);
      }
    }
    const uint32_t cnt = (uint32_t)__popc(x);
    const uint32_t incl = wave_inclusive_scan_dpp(cnt);
    if ((threadIdx.x & 63) == 63) s_wave[par & 1][wave] = incl;
    const bool hand_over = ticket_pending && sub + 1 == cur_len;
    if (hand_over && threadIdx.x == 0) s_next[turn & 1] = drawn;
    __syncthreads();
    if (hand_over) {
      ticket_tile(drawn_tile(s_next[turn & 1]), far_first, far_len);
      ticket_pending = false;
    }
    load_ahead(2, far);
    uint32_t before = incl - cnt, total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const uint32_t t = s_wave[par & 1][w];
      if (w < wave) before += t;
      total += t;
    }
    const uint32_t all = x;
    const uint32_t first_elem = (uint32_t)sub_base + threadIdx.x * (uint32_t)V;  // indices are below 2^31
    uint32_t done = 0;
    for (;;) {
      const uint32_t room = (uint32_t)kScatStage - count;
      const uint32_t hi = done + room;
      uint32_t y = x;
      while (y) {
        const uint32_t bit = (uint32_t)__ffs((int)y) - 1u;
        y &= y - 1;
        // the thread's candidates take their places in the order of their flag bits (the stage has no order
        // to keep, and a place counted off the flag word costs two instructions)
        const uint32_t pos = before + (uint32_t)__popc(all & ((1u << bit) - 1u));
        if (pos < hi) {
          x &= ~(1u << bit);
          const uint32_t at = count + pos - done;
          st_idx[at] = (int32_t)(first_elem + Flags<S>::elem_step(bit));
          st_val[at] = Flags<S>::pick(cur, bit);
        }
      }
      const uint32_t take = total - done < room ? total - done : room;
      count += take;
      done += take;
      if (count < (uint32_t)kScatStage) break;
      __syncthreads();
      stage_flush<S>(count, st_idx, st_val, s_flush, hist, floor_key, out, status);
      count = 0;
      if (done == total) break;
    }
  };

  known_tile(0, cur_first, cur_len);
  if (!known_tile(1, nxt_first, nxt_len)) {  // short inputs: the second tile already needs a ticket
    if (threadIdx.x == 0) s_next[1] = draw();
    __syncthreads();
    ticket_tile(drawn_tile(s_next[1]), nxt_first, nxt_len);
  }
  if (cur_len) {
    sub = 0;
    if (ALIGNED)
      stage_load_fast<S>(in, full_vecs - 1u, cur_first * kSubVecs, qa);
    else
      stage_load<S, false>(in, n, (int64_t)cur_first * kSub, qa);
    load_ahead(1, qb);  // tiles have at least two sub-tiles
  }
  // Starts a tile: the ticket of the tile after the next one is asked for.
  auto open_tile = [&]() {
    far_len = 0;
    if (!known_tile(turn + 2, far_first, far_len)) {
      ticket_pending = true;
      if (threadIdx.x == 0) drawn = draw();
    }
  };
  // One sub-tile of the block's sequence, then on to the next place in it.  False when the sequence has ended.
  auto step = [&](uint4 (&cur)[kSelVecs], uint4 (&far)[kSelVecs]) {
    if (cur_len == 0) return false;
    if (sub == 0) open_tile();
    sub_base = (int64_t)(cur_first + sub) * kSub;
    body(cur, far);
    ++par;
    if (++sub == cur_len) {
      cur_first = nxt_first;
      cur_len = nxt_len;
      nxt_first = far_first;
      nxt_len = far_len;
      ++turn;
      sub = 0;
    }
    return true;
  };
  // The three register sets keep their roles in straight-line code (a set chosen by a run-time number would be
  // copied from tile to tile, and the copy waits for every load in flight).
  for (;;) {
    if (!step(qa, qc)) break;
    if (!step(qb, qa)) break;
    if (!step(qc, qb)) break;
  }
  __syncthreads();
  if (count) stage_flush<S>(count, st_idx, st_val, s_flush, hist, floor_key, out, status);
  if (ALIGNED && blockIdx.x == 0 && (int64_t)full_vecs * V < n) {
    // the elements behind the last complete vector (fewer than V): a small stage of their own
    if (threadIdx.x == 0) {
      uint32_t c = 0;
      for (int64_t e = (int64_t)full_vecs * V; e < n; ++e) {
        const S v = in[e];
        if ((v & KeyOf<S>::kMask) >= floor_key) {
          st_idx[c] = (int32_t)e;
          st_val[c] = v;
          ++c;
        }
      }
      s_tail = c;
    }
    __syncthreads();
    const uint32_t c = s_tail;
    if (c) stage_flush<S>(c, st_idx, st_val, s_flush, hist, floor_key, out, status);
  }
  if (next.hist) {
    __syncthreads();  // the stage is no longer needed
    stage_sample_next<S>(next, s_run.window, s_pick);
  }
  if (hist) {
    __syncthreads();
    uint32_t *row = cand_hist + (size_t)(blockIdx.x % kCandRows) * kCandBins;
    for (int i = threadIdx.x; i < kCandBins; i += kSelBlock) {
      const uint32_t c = s_hist[i];
      if (c) atomicAdd(&row[cand_place((uint32_t)i)], c);  // nothing returned: the adds are in flight together
    }
    if (pick_thr) {
      // the block that finishes last reads the exact threshold off the complete histogram
      __shared__ bool s_last;
      // the adds are carried out (where device-wide atomics are) before the count goes up; no device-scope
      // fence: that would write the L2 back once per wave
      wait_global_acks();
      __syncthreads();
      if (threadIdx.x == 0) s_last = atomicAdd(&cand_hist[kCandRows * kCandBins], 1u) == gridDim.x - 1u;
      __syncthreads();
      if (s_last) {
        cand_pick_block<kSelBlock>(cand_hist, floor_key, pick_k, KeyOf<S>::kBits == 15 ? 0 : 16, pick_thr, status,
                                   s_pick, s_hist, pick_above);
        __syncthreads();
        if (thr_copy && threadIdx.x < 2)
          thr_copy[threadIdx.x] = __hip_atomic_load(&pick_thr[threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

static int device_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      cus = v;
    else
      cus = 256;
  }
  return cus;
}

template <typename S>
static int stage_launch(const StageArgs &a, hipStream_t stream) {
  constexpr int V = VecOf<S>::kN;
  const int64_t sub = (int64_t)kSelBlock * kSelVecs * V;
  const int64_t subs = ceil_div(a.n > 0 ? a.n : 1, sub);
  if (subs > 0x3fffffff) return fail(ZEN_EINVAL, "select_stage: tensor too large");
  // three workgroups per compute unit (measured: two are 10 % slower, four no faster); their LDS, 60 KB per
  // unit, leaves room for another stream's kernels next to this long one
#ifndef ZEN_STAGE_WGS
#define ZEN_STAGE_WGS 3
#endif
  int64_t blocks = (int64_t)device_cus() * ZEN_STAGE_WGS;
  const int64_t least = ceil_div(subs, kStageSmall);
  if (blocks > least) blocks = least;
  // seven eighths of the tensor in counter-free tiles, the rest through tickets (measured on 1.5 GB: all
  // tickets 280 us, two thirds fixed 252, seven eighths 247, everything fixed 258)
  StageSched sch;
  sch.fixed = (uint32_t)(subs * 7 / 8 / ((int64_t)kStageBig * blocks));
  sch.fixed_subs = sch.fixed * (uint32_t)kStageBig * (uint32_t)blocks;
  sch.ticket_tiles = (uint32_t)ceil_div(subs - (int64_t)sch.fixed_subs, kStageSmall);
  const S *in = static_cast<const S *>(a.in);
  const bool aligned = (reinterpret_cast<uintptr_t>(in) & 15u) == 0 && a.n >= V;
  const StageSlabs out{a.geo, a.cg, a.coarse_cursor, a.coarse_words, a.wide ? 1u : 0u};
  StageSample next;
  if (a.next_in && a.next_hist && a.next_k > 0) {
    const int64_t next_n = a.next_n > 0 ? a.next_n : a.n;  // the next tensor has this one's type
    const SamplePlan sp = sample_plan(next_n, a.next_k, V);
    next.in = a.next_in;
    next.n = next_n;
    next.hist = a.next_hist;
    next.rank = sp.rank;
    next.block_log2 = sp.log2;
    next.nblocks = sp.nblocks;
    next.floor_out = a.next_floor;
  }
  ProfScope prof(kProfSelectStage, stream);
  if (aligned)
    k_select_stage<S, true><<<dim3((unsigned)blocks), dim3(kSelBlock), 0, stream>>>(
        in, a.n, a.thr, out, a.ticket, sch, a.cand_hist, (uint32_t)a.pick_k, a.pick_thr, a.pick_above, a.thr_copy,
        a.clear, a.clear_words, a.floor_margin, next, a.status);
  else
    k_select_stage<S, false><<<dim3((unsigned)blocks), dim3(kSelBlock), 0, stream>>>(
        in, a.n, a.thr, out, a.ticket, sch, a.cand_hist, (uint32_t)a.pick_k, a.pick_thr, a.pick_above, a.thr_copy,
        a.clear, a.clear_words, a.floor_margin, next, a.status);
  ZEN_LAUNCH_CHECK("k_select_stage");
  return ZEN_OK;
}

size_t select_stage_ticket_words() { return (size_t)kStageGroups * kStageTicketPad; }

int select_stage_slabs(const StageArgs &a, hipStream_t stream) {
  if (a.dtype == ZEN_BF16) return stage_launch<uint16_t>(a, stream);
  return stage_launch<uint32_t>(a, stream);
}

namespace {

template <typename S>
int topk_launch(const S *in, int64_t n, const uint32_t *n_dev, int64_t k, uint32_t *thr, void *workspace,
                int32_t *status, int short_bit, hipStream_t stream) {
  Carver cv(workspace);
  TopkState *st = cv.take<TopkState>(1);
  uint32_t *hist = cv.take<uint32_t>(kHistBins);
  k_topk_init<<<dim3(1), dim3(256), 0, stream>>>(st, hist, (uint32_t)k);
  ZEN_LAUNCH_CHECK("k_topk_init");
  // digit widths from the top of the key: bf16 15 = 11+4, fp32 31 = 11+10+10
  const int widths16[2] = {11, 4};
  const int widths32[3] = {11, 10, 10};
  const int npass = sizeof(S) == 2 ? 2 : 3;
  const int *widths = sizeof(S) == 2 ? widths16 : widths32;
  constexpr int V = VecOf<S>::kN;
  const int64_t nvec = ceil_div(n, V);
  int64_t blocks = ceil_div(nvec, kHistBlock);
  if (blocks > 2048) blocks = 2048;
  const bool aligned = (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
  int shift = KeyOf<S>::kBits;
  for (int p = 0; p < npass; ++p) {
    shift -= widths[p];
    {
      ProfScope prof(kProfTopkHist, stream);
      if (aligned)
        k_topk_hist<S, true><<<dim3((unsigned)blocks), dim3(kHistBlock), 0, stream>>>(in, n, n_dev, st, shift,
                                                                                      widths[p], p, hist);
      else
        k_topk_hist<S, false><<<dim3((unsigned)blocks), dim3(kHistBlock), 0, stream>>>(in, n, n_dev, st, shift,
                                                                                       widths[p], p, hist);
      ZEN_LAUNCH_CHECK("k_topk_hist");
    }
    k_topk_pick<<<dim3(1), dim3(kHistBlock), 0, stream>>>(st, hist, widths[p], p == npass - 1, 0, thr, status,
                                                          short_bit);
    ZEN_LAUNCH_CHECK("k_topk_pick");
  }
  return ZEN_OK;
}

template <typename S>
int sample_launch(const S *in, int64_t n, int64_t k, uint32_t *thr_lo, void *workspace, hipStream_t stream,
                  bool is_zero) {
  constexpr int V = VecOf<S>::kN;
  uint32_t *hist = static_cast<uint32_t *>(workspace);
  const SamplePlan sp = sample_plan(n, k, V);
  const int sample_log2 = sp.log2;
  const int64_t nblocks = sp.nblocks;
  const uint32_t rank = sp.rank;
  if (!is_zero) {
    launch_fill<uint32_t>(hist, 0u, kFineBins + 2, stream);
    ZEN_LAUNCH_CHECK("sample: clear histogram");
  }
  // every block must see fewer than 65536 sample elements (16-bit LDS counters)
  int64_t blocks = ceil_div(nblocks * V, 32768);
  if (blocks < 128) blocks = 128;
  const bool aligned = (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
  {
    ProfScope prof(kProfSampleHist, stream);
    if (aligned)
      k_sample_hist<S, true><<<dim3((unsigned)blocks), dim3(kSampleBlock), 0, stream>>>(in, n, sample_log2, hist, rank,
                                                                                        thr_lo);
    else
      k_sample_hist<S, false><<<dim3((unsigned)blocks), dim3(kSampleBlock), 0, stream>>>(in, n, sample_log2, hist,
                                                                                         rank, thr_lo);
    ZEN_LAUNCH_CHECK("k_sample_hist");
  }
  return ZEN_OK;
}

template <typename S>
int compress_launch(const S *in, int64_t n, const uint32_t *thr, S *out, hipStream_t stream) {
  constexpr int V = VecOf<S>::kN;
  const int64_t nvec = ceil_div(n, V);
  int64_t blocks = ceil_div(nvec, 256);
  if (blocks > 8192) blocks = 8192;
  const bool aligned =
      ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  ProfScope prof(kProfCompress, stream);
  if (aligned)
    k_compress<S, true><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(in, n, thr, out);
  else
    k_compress<S, false><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(in, n, thr, out);
  ZEN_LAUNCH_CHECK("k_compress");
  return ZEN_OK;
}

}  // namespace

size_t topk_scratch_bytes() {
  const size_t exact = align_up(sizeof(TopkState), 256) + align_up(kHistBins * sizeof(uint32_t), 256);
  const size_t sampled = align_up((kFineBins + 2) * sizeof(uint32_t), 256);
  return exact > sampled ? exact : sampled;
}

int topk_exact(const void *in, int dtype, int64_t n, const uint32_t *n_dev, int64_t k, uint32_t *thr,
               void *scratch, int32_t *status, int short_bit, hipStream_t stream) {
  if (dtype == ZEN_BF16)
    return topk_launch(static_cast<const uint16_t *>(in), n, n_dev, k, thr, scratch, status, short_bit, stream);
  return topk_launch(static_cast<const uint32_t *>(in), n, n_dev, k, thr, scratch, status, short_bit, stream);
}

int topk_sampled_floor(const void *in, int dtype, int64_t n, int64_t k, uint32_t *thr_lo, void *scratch,
                       hipStream_t stream, bool scratch_is_zero) {
  if (dtype == ZEN_BF16)
    return sample_launch(static_cast<const uint16_t *>(in), n, k, thr_lo, scratch, stream, scratch_is_zero);
  return sample_launch(static_cast<const uint32_t *>(in), n, k, thr_lo, scratch, stream, scratch_is_zero);
}

size_t sampled_floor_zero_bytes() { return (kFineBins + 2) * sizeof(uint32_t); }

}  // namespace zen

// The radix select's counters and histogram for callers that cannot bring a workspace along: one array per
// GPU, part of the loaded code object, which that GPU holds until the process ends.  Host code never passes
// the array's name to a kernel (on the host it is a stand-in, not a device address): it asks for the address
// once per device and keeps it.
namespace {

constexpr size_t kTopkStaticBytes = 256 /* TopkState */ + zen::kHistBins * sizeof(uint32_t);
static_assert(sizeof(zen::TopkState) <= 256, "TopkState outgrew its slot");
static __device__ __align__(256) unsigned char g_topk_static[kTopkStaticBytes];

constexpr int kMaxDevices = 64;
std::mutex g_topk_static_mu;
void *g_topk_static_at[kMaxDevices];  // device address of g_topk_static, per device; null = not asked yet

// Address of the current device's copy of g_topk_static.
int topk_static_scratch(void **out) {
  int dev = -1;
  ZEN_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return zen::fail(ZEN_EINVAL, "zen_topk_threshold_static: device number out of range");
  std::lock_guard<std::mutex> lock(g_topk_static_mu);
  if (!g_topk_static_at[dev]) {
    void *p = nullptr;
    ZEN_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(g_topk_static)));
    if (!p) return zen::fail(ZEN_EHIP, "zen_topk_threshold_static: no address for the static scratch array");
    g_topk_static_at[dev] = p;
  }
  *out = g_topk_static_at[dev];
  return ZEN_OK;
}

}  // namespace

namespace zen {
namespace {

// Reads `vecs` 16-byte vectors with coalesced non-temporal loads and does nothing else: what a read-only pass
// over a tensor can reach on the machine at hand.  A workgroup reads kReadChunks consecutive chunks of 256
// vectors (32 KB in a row; many short-lived workgroups, the arrangement that measured fastest for a bare
// read).  sink receives a word only if the data XOR to a given value, which keeps the loads alive without a
// store per thread.
constexpr int kReadChunks = 8;
__global__ __launch_bounds__(256) void k_stream_read(const u32x4 *__restrict__ in, size_t vecs, uint32_t *sink) {
  uint32_t acc = 0;
  const size_t base = (size_t)blockIdx.x * kReadChunks * 256 + threadIdx.x;
  const size_t last = vecs - 1;
  u32x4 q[kReadChunks];
#pragma unroll
  for (int i = 0; i < kReadChunks; ++i) {
    const size_t at = base + (size_t)i * 256;
    q[i] = __builtin_nontemporal_load(in + (at < last ? at : last));  // no branch around the loads
  }
#pragma unroll
  for (int i = 0; i < kReadChunks; ++i) acc ^= q[i].x ^ q[i].y ^ q[i].z ^ q[i].w;
  if (acc == 0x9e3779b9u) *sink = acc;
}

}  // namespace
}  // namespace zen

namespace zen {
namespace {

// out[j] = in[sample_index[j]] for j < s: the sample compress() draws (train.py:78-80), gathered for the
// radix select that follows.  Four positions per thread; a position outside [0, n) is flagged and reads as zero.
constexpr int kGatherBlock = 256, kGatherItems = 4;
template <typename S>
__global__ __launch_bounds__(kGatherBlock) void k_sample_gather(const S *__restrict__ in, int64_t n,
                                                                const int64_t *__restrict__ at, int64_t s,
                                                                S *__restrict__ out, int32_t *status) {
  const int64_t base = (int64_t)blockIdx.x * (kGatherBlock * kGatherItems) + threadIdx.x;
  int64_t pos[kGatherItems];
  S v[kGatherItems];
  bool bad = false;
#pragma unroll
  for (int i = 0; i < kGatherItems; ++i) {
    const int64_t j = base + (int64_t)i * kGatherBlock;
    pos[i] = j < s ? __builtin_nontemporal_load(at + j) : 0;
    if (pos[i] < 0 || pos[i] >= n) {
      bad = true;
      pos[i] = -1;
    }
  }
#pragma unroll
  for (int i = 0; i < kGatherItems; ++i) v[i] = pos[i] >= 0 ? in[pos[i]] : S(0);
#pragma unroll
  for (int i = 0; i < kGatherItems; ++i) {
    const int64_t j = base + (int64_t)i * kGatherBlock;
    if (j < s) out[j] = v[i];
  }
  if (bad) atomicOr(status, ZEN_STAT_BAD_INDEX);
}

size_t sample_gather_bytes(int64_t s, int dtype) { return align_up((size_t)s * (dtype == ZEN_BF16 ? 2 : 4), 256); }

template <typename S>
int sample_threshold_launch(const S *in, int64_t n, const int64_t *at, int64_t s, int64_t k, uint32_t *thr,
                            void *workspace, int32_t *status, hipStream_t stream) {
  S *sample = static_cast<S *>(workspace);
  void *topk = static_cast<unsigned char *>(workspace) + sample_gather_bytes(s, sizeof(S) == 2 ? ZEN_BF16 : ZEN_F32);
  const int64_t blocks = ceil_div(s, (int64_t)kGatherBlock * kGatherItems);
  k_sample_gather<S><<<dim3((unsigned)blocks), dim3(kGatherBlock), 0, stream>>>(in, n, at, s, sample, status);
  ZEN_LAUNCH_CHECK("k_sample_gather");
  return topk_launch(sample, s, nullptr, k, thr, topk, nullptr, 0, stream);
}

}  // namespace
}  // namespace zen

extern "C" {

int zen_stream_read(const void *input, size_t bytes, uint32_t *sink, void *stream) {
  using namespace zen;
  if (!input || !sink || (reinterpret_cast<uintptr_t>(input) & 15u)) return fail(ZEN_EINVAL, "zen_stream_read: null or unaligned pointer");
  const size_t vecs = bytes / 16;
  if (vecs == 0) return ZEN_OK;
  const size_t blocks = (vecs + (size_t)kReadChunks * 256 - 1) / ((size_t)kReadChunks * 256);
  if (blocks > 0x7fffffffull) return fail(ZEN_EINVAL, "zen_stream_read: too large");
  k_stream_read<<<dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const u32x4 *>(input), vecs, sink);
  ZEN_LAUNCH_CHECK("k_stream_read");
  return ZEN_OK;
}

size_t zen_topk_threshold_workspace(void) { return zen::topk_scratch_bytes(); }

int zen_topk_threshold_static(const void *input, int dtype, int64_t n, int64_t k, uint32_t *thr, void *stream) {
  using namespace zen;
  if (!input || !thr) return fail(ZEN_EINVAL, "zen_topk_threshold_static: null pointer");
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_topk_threshold_static: bad dtype");
  if (n <= 0 || n > ZEN_TOPK_STATIC_MAX_N)
    return fail(ZEN_EINVAL, "zen_topk_threshold_static: n exceeds ZEN_TOPK_STATIC_MAX_N (2^31 - 1 elements)");
  if (k < 1 || k > n) return fail(ZEN_EINVAL, "zen_topk_threshold_static: need 1 <= k <= n");
  void *scratch_at = nullptr;
  const int rc = topk_static_scratch(&scratch_at);
  if (rc != ZEN_OK) return rc;
  // k_topk_init clears the counters and the histogram at the head of every call, so what the previous call
  // left in the array does not matter.
  return topk_exact(input, dtype, n, nullptr, k, thr, scratch_at, nullptr, 0, static_cast<hipStream_t>(stream));
}

int zen_topk_threshold(const void *input, int dtype, int64_t n, int64_t k, uint32_t *thr, void *workspace,
                       size_t workspace_bytes, void *stream) {
  using namespace zen;
  if (!input || !thr || !workspace) return fail(ZEN_EINVAL, "zen_topk_threshold: null pointer");
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_topk_threshold: bad dtype");
  if (n <= 0 || n > 0x7fffffffll || k < 1 || k > n) return fail(ZEN_EINVAL, "zen_topk_threshold: need 1 <= k <= n < 2^31");
  if (workspace_bytes < zen_topk_threshold_workspace()) return fail(ZEN_EWORKSPACE, "zen_topk_threshold: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  return topk_exact(input, dtype, n, nullptr, k, thr, workspace, nullptr, 0, s);
}

size_t zen_sample_threshold_workspace(int64_t s, int dtype) {
  if (s < 0) return 0;
  return zen::sample_gather_bytes(s, dtype) + zen::topk_scratch_bytes();
}

int zen_sample_threshold(const void *input, int dtype, int64_t n, const int64_t *sample_index, int64_t s, int64_t k,
                         uint32_t *thr, void *workspace, size_t workspace_bytes, int32_t *status, void *stream) {
  using namespace zen;
  if (!input || !sample_index || !thr || !workspace || !status) return fail(ZEN_EINVAL, "zen_sample_threshold: null pointer");
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_sample_threshold: bad dtype");
  if (n <= 0 || s <= 0 || s > 0x7fffffffll || k < 1 || k > s)
    return fail(ZEN_EINVAL, "zen_sample_threshold: need n > 0 and 1 <= k <= s < 2^31");
  if (workspace_bytes < zen_sample_threshold_workspace(s, dtype))
    return fail(ZEN_EWORKSPACE, "zen_sample_threshold: workspace too small");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t *at = sample_index;
  if (dtype == ZEN_BF16)
    return sample_threshold_launch(static_cast<const uint16_t *>(input), n, at, s, k, thr, workspace, status, st);
  return sample_threshold_launch(static_cast<const uint32_t *>(input), n, at, s, k, thr, workspace, status, st);
}

int zen_compress(const void *input, int dtype, int64_t n, const uint32_t *thr, void *out, void *stream) {
  using namespace zen;
  if (n == 0) return ZEN_OK;
  if (!input || !thr || !out) return fail(ZEN_EINVAL, "zen_compress: null pointer");
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_compress: bad dtype");
  if (n < 0 || n > 0x7fffffffll) return fail(ZEN_EINVAL, "zen_compress: need 0 <= n < 2^31");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == ZEN_BF16)
    return compress_launch(static_cast<const uint16_t *>(input), n, thr, static_cast<uint16_t *>(out), s);
  return compress_launch(static_cast<const uint32_t *>(input), n, thr, static_cast<uint32_t *>(out), s);
}

size_t zen_select_workspace(int64_t n, int dtype) { return zen::select_scratch_bytes(n, dtype); }

int zen_select(const void *input, int dtype, int64_t n, const uint32_t *thr, void *out_idx, int idx64,
               void *out_val, int64_t capacity, int64_t *out_count, void *workspace, size_t workspace_bytes,
               int32_t *status, void *stream) {
  using namespace zen;
  if (!out_count || !status) return fail(ZEN_EINVAL, "zen_select: null pointer");
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_select: bad dtype");
  if (n < 0 || n > 0x7fffffffll || capacity < 0) return fail(ZEN_EINVAL, "zen_select: need 0 <= n < 2^31");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (n == 0) {
    launch_fill<int64_t>(out_count, 0, 1, s);
    ZEN_LAUNCH_CHECK("zen_select: zero count");
    return ZEN_OK;
  }
  if (!input || !workspace || (capacity > 0 && (!out_idx || !out_val)))
    return fail(ZEN_EINVAL, "zen_select: null pointer");
  if (workspace_bytes < zen_select_workspace(n, dtype)) return fail(ZEN_EWORKSPACE, "zen_select: workspace too small");
  SelectArgs a;
  a.in = input;
  a.dtype = dtype;
  a.n = n;
  a.thr = thr;
  a.out_idx = out_idx;
  a.idx64 = idx64;
  a.out_val = out_val;
  a.capacity = capacity;
  a.out_count = out_count;
  a.ordered = true;
  a.scratch = workspace;
  a.status = status;
  return select_compact(a, s);
}

}  // extern "C"
