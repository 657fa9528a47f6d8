// Two-level sort of (key, value) pairs whose (key, value) combinations are
// distinct: a counting sort into coarse key bins (global histogram, one scan,
// atomic cursors) followed by an exact rank inside each bin.  Bins are sized so
// that they hold a handful of entries, which makes the in-bin rank a short
// linear scan; the result is ascending in (key, value) and does not depend on
// the order in which the atomics happened.  Two passes over the entries instead
// of one per radix digit.
//
// A bin with more than kBinLimit entries (keys piled on a few values) makes the
// rank quadratic; then the scan raises `retry`, every later stage returns at
// once and the caller reports ZEN_STAT_RETRY so the general radix path can run.
#pragma once

#include "zen_common.h"

namespace zen {

constexpr uint32_t kBinLimit = 4096;
constexpr int kBsScanBlock = 256;
constexpr int kBsScanItems = 8;
constexpr int kBsScanTile = kBsScanBlock * kBsScanItems;

struct BinSort {
  int bshift;           // bin = key >> bshift
  uint32_t nbins;       // bins 0 .. nbins-1
  uint32_t *hist;       // [nbins]      zeroed by the caller before counting
  uint32_t *start;      // [nbins + 1]  exclusive prefix of hist
  uint32_t *cursor;     // [nbins]      scatter cursors
  unsigned long long *desc;  // prefix state of the scan kernel (scan_words(scan_tiles))
  uint32_t *retry;      // [1] set when a bin exceeds kBinLimit
  void *extra;          // caller's own to-be-zeroed area (extra_zero_bytes), cleared with the rest
  int scan_tiles;
  void *zero_begin;     // region the caller clears before every use
  size_t zero_bytes;
  size_t bytes;
};

// key_limit: keys are < key_limit.  expected: typical number of entries.
BinSort plan_binsort(void *scratch, uint64_t key_limit, int64_t expected, size_t extra_zero_bytes);

// Clears hist, descriptors, retry and the caller's extra area.
int binsort_clear(const BinSort &bs, hipStream_t stream);

// After the histogram is filled: start/cursor/retry.
int binsort_scan(const BinSort &bs, int32_t *status, hipStream_t stream);

// Generic scatter (value = given array, or the entry's position when vals is
// null) and the in-bin rank.
int binsort_scatter(const BinSort &bs, const uint32_t *keys, const uint32_t *vals, int64_t max_count,
                    const uint32_t *count_dev, uint32_t *tmp_keys, uint32_t *tmp_vals, hipStream_t stream);
int binsort_rank(const BinSort &bs, const uint32_t *tmp_keys, const uint32_t *tmp_vals, int64_t max_count,
                 const uint32_t *count_dev, uint32_t *out_keys, uint32_t *out_vals, hipStream_t stream);

}  // namespace zen
