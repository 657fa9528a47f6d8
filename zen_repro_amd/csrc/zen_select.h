// Vector loads and the ordered-compaction entry shared by the select and
// load-balance translation units.
#pragma once

#include "zen_common.h"
#include "zen_slab.h"
#include "zen_slab_feed.h"

namespace zen {

template <typename S>
struct VecOf {
  static constexpr int kN = 16 / sizeof(S);  // elements per 16-byte load
};

// Loads the VecOf<S>::kN elements starting at `first` (a multiple of kN).
// Returns how many of them lie inside [0, n); the rest read as 0.
template <typename S, bool ALIGNED>
__device__ inline int load_vec(const S *__restrict__ in, int64_t first, int64_t n, S (&e)[VecOf<S>::kN]) {
  constexpr int V = VecOf<S>::kN;
  if (ALIGNED && first + V <= n) {
    const uint4 q = *reinterpret_cast<const uint4 *>(in + first);
    __builtin_memcpy(e, &q, 16);
    return V;
  }
  int live = 0;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const bool ok = first + i < n;
    e[i] = ok ? in[first + i] : S(0);
    live += ok;
  }
  return live;
}

constexpr int kSelBlock = 256;
constexpr int kSelVecs = 4;  // 16-byte vectors per thread and tile

// Compaction of the elements with key >= max(thr[0], 1) (thr == nullptr: the
// nonzero ones) into (index, value) lists.
struct SelectArgs {
  const void *in = nullptr;           // dense tensor, or the values of a list
  int dtype = ZEN_F32;
  int64_t n = 0;                      // elements (capacity of the list when n_dev is set)
  const uint32_t *n_dev = nullptr;    // optional device-side element count (<= n)
  const uint32_t *thr = nullptr;      // optional device threshold key
  const int32_t *src_idx = nullptr;   // list input: the index each element carries
  void *out_idx = nullptr;
  int idx64 = 0;                      // out_idx is int64 instead of int32
  void *out_val = nullptr;
  int64_t capacity = 0;
  int64_t *out_count = nullptr;       // optional: number found (may exceed capacity)
  uint32_t *out_count32 = nullptr;    // optional: the same clamped to capacity
  bool ordered = true;                // ascending output (false: tiles in arrival order)
  uint32_t *cand_hist = nullptr;      // optional (unordered mode): kCandHistWords counters, zero on entry: kCandRows
                                      // partial histograms of min((key - floor) >> (bf16: 0, fp32: 16), kCandBins-1)
                                      // over the selected, then a count of finished blocks
  int64_t pick_k = 0;                 // with cand_hist and pick_thr: the block that finishes last writes
  uint32_t *pick_thr = nullptr;       // pick_thr[0] = k-th largest key as far as the histogram resolves it (bf16:
                                      // exactly; fp32: its top 15 bits), pick_thr[1] = candidates at or above it;
                                      // ZEN_STAT_RETRY if the candidates are fewer than k
  void *scratch = nullptr;            // select_scratch_bytes(n, dtype)
  int32_t *status = nullptr;
};

size_t select_scratch_bytes(int64_t n, int dtype);
int select_compact(const SelectArgs &args, hipStream_t stream);

// Exact k-th largest magnitude key by radix select: thr[0] = key, thr[1] = number
// of elements with key >= it.  `in` is a dense tensor or any array of values;
// n_dev optionally holds the live element count.  Fewer than k elements:
// thr = (0, count) and `short_bit` (if nonzero) is OR-ed into *status.
size_t topk_scratch_bytes();
int topk_exact(const void *in, int dtype, int64_t n, const uint32_t *n_dev, int64_t k, uint32_t *thr,
               void *scratch, int32_t *status, int short_bit, hipStream_t stream);

// Lower bound for that key from a 1/256 sample: thr_lo[0] is the lowest key of
// the 15-bit magnitude bin (for bf16: the key itself) in which the sample
// reaches the expected rank plus a safety margin.  Almost surely at least k
// elements of the tensor lie at or above it; compacting them with a candidate
// histogram (SelectArgs::cand_hist, pick_k, pick_thr) gives the exact
// threshold with one pass over the tensor, or ZEN_STAT_RETRY if the
// candidates are fewer than k after all.  For fp32 the histogram resolves the
// top 15 key bits only; topk_exact over the candidates finishes the job.
int topk_sampled_floor(const void *in, int dtype, int64_t n, int64_t k, uint32_t *thr_lo, void *scratch,
                       hipStream_t stream, bool scratch_is_zero = false);
size_t sampled_floor_zero_bytes();  // leading part of the scratch that must be zero (scratch_is_zero: the caller did it)
constexpr int kCandBins = 512;   // four octaves of 15-bit magnitudes above the floor; the rest shares the last bin
constexpr int kCandRows = 8;   // partial candidate histograms (blocks spread over them)
constexpr int kCandHistWords = kCandRows * kCandBins + 1;

// One pass over a dense tensor, by persistent workgroups, that hands every element with key >= max(thr[0], 1)
// (thr == nullptr: the nonzero ones) except element 0 to the coarse slabs of zen_slab_feed.h, as (index,
// value) and keyed by the level-1 hash slot of its index: whenever a workgroup has gathered a couple of
// thousand candidates it orders them by coarse slab in LDS and appends one run per slab.  coarse_cursor,
// *ticket and cand_hist must be zero on entry; a coarse slab that overflows raises ZEN_STAT_RETRY.  With
// cand_hist / pick_k / pick_thr the k-th largest key is read off the candidates' histogram (element 0
// included) as in SelectArgs (and copied to thr_copy if that is not null): exactly for bf16, for fp32 the
// lowest key of its bin of 65536 keys.
// What the selecting kernel needs to take the next call's sample (see StageArgs::next_in).
struct StageSample {
  const void *in = nullptr;
  int64_t n = 0;
  uint32_t *hist = nullptr;
  uint32_t rank = 0;
  int block_log2 = 0;
  int64_t nblocks = 0;
  uint32_t *floor_out = nullptr;
};

struct StageArgs {
  const void *in = nullptr;
  int dtype = ZEN_F32;
  int64_t n = 0;
  const uint32_t *thr = nullptr;
  uint32_t floor_margin = 0;        // what is taken off thr[0] (a key near the threshold, not a floor below it)
  SlabGeom geo;                     // buckets of the level-1 hash slots
  CoarseGeom cg;
  uint32_t *coarse_cursor = nullptr;
  uint32_t *coarse_words = nullptr;  // plane 0: indices; plane 1: values in the tensor's type
  bool wide = false;                // the destinations are wide buckets (zen_wide.h): cg.groups of them (at most
                                    // 256), cg.per = 1, cg.cap entries per part; coarse_words holds records of two
                                    // words (index, value bits) instead of planes
  uint32_t *ticket = nullptr;       // select_stage_ticket_words() words
  uint32_t *cand_hist = nullptr;
  int64_t pick_k = 0;
  uint32_t *pick_thr = nullptr;
  uint32_t *pick_above = nullptr;   // optional: number of candidates in the histogram bins above the k-th's
  uint32_t *thr_copy = nullptr;
  uint32_t *clear = nullptr;        // optional: clear_words words the kernel sets to zero (memory of an earlier
  uint32_t clear_words = 0;         // kernel that nobody needs any more)
  // The sample of the NEXT call on the same workspace (a tensor of this one's type and of next_n elements, 0:
  // this one's length; next_k its k) is taken by this kernel's workgroups when they are through with their own
  // tensor: next_hist = that call's sampling memory (zero, left as k_sample_hist leaves it), next_floor
  // receives its floor key.
  const void *next_in = nullptr;
  int64_t next_k = 0;
  int64_t next_n = 0;
  uint32_t *next_hist = nullptr;
  uint32_t *next_floor = nullptr;
  int32_t *status = nullptr;
};
int select_stage_slabs(const StageArgs &a, hipStream_t stream);
size_t select_stage_ticket_words();

}  // namespace zen
