// The last step of an fp32 top-k threshold on the slab paths (zen_slab_encode.hip, zen_wide_encode.hip).
#pragma once

#include "zen_select.h"
#include "zen_slab_feed.h"

namespace zen {
namespace {

// --------------------------------------------- fp32: the threshold's last 16 bits

constexpr int kRefineBins = 65536;
constexpr int kRefineBlock = 512;

// The candidates' histogram resolves the 15 leading bits of an fp32 key: after the select kernel thr[0] is
// the lowest key of the bin the k-th largest lies in, thr[1] the number of candidates at or above it and
// *above the number in the bins above.  This kernel histograms the low 16 key bits of the candidates of that
// bin (they sit in word plane `val_plane` of the coarse slabs, or with val_plane < 0 in the second word of the
// wide buckets' two-word records; element 0, which is never handed on, is looked at in the tensor), and the
// workgroup that finishes last replaces thr[0..1] by the exact key and the number of elements at or above it.
// Grid: any number of workgroups, which take the parts of the coarse slabs in turn.  hist: kRefineBins + 1 zeroed words.
__global__ __launch_bounds__(kRefineBlock) void k_refine_threshold(CoarseGeom cg, int val_plane,
                                                                   const uint32_t *__restrict__ coarse_cursor,
                                                                   const uint32_t *__restrict__ coarse_words,
                                                                   const uint32_t *__restrict__ dense,
                                                                   uint32_t *thr, const uint32_t *above, uint32_t k,
                                                                   uint32_t *hist, uint32_t *thr_copy, int32_t *status) {
  __shared__ uint32_t s_scan[kRefineBlock / 64 + 1];
  __shared__ bool s_last;
  const uint32_t base = thr[0];
  const size_t plane = (size_t)cg.groups * kCoarseSplit * cg.cap;
  const uint32_t parts = cg.groups * (uint32_t)kCoarseSplit;
  // a workgroup takes several parts: every workgroup ends with an atomic on one counter, and a thousand of
  // those stand in line for 11 us
  for (uint32_t part = blockIdx.x; part < parts; part += gridDim.x) {
    uint32_t count = coarse_cursor[part * kCoarsePad];
    if (count > cg.cap) count = cg.cap;
    const uint32_t *vals = val_plane < 0 ? coarse_words + (size_t)part * cg.cap * 2 + 1
                                         : coarse_words + (size_t)val_plane * plane + (size_t)part * cg.cap;
    const uint32_t stride = val_plane < 0 ? 2u : 1u;
    for (uint32_t e = threadIdx.x; e < count; e += kRefineBlock) {
      const uint32_t d = (vals[e * stride] & KeyOf<uint32_t>::kMask) - base;
      if (d < (uint32_t)kRefineBins) atomicAdd(&hist[d], 1u);
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    const uint32_t key0 = dense[0] & KeyOf<uint32_t>::kMask;  // counted by the select kernel if it was a candidate
    if (key0 - base < (uint32_t)kRefineBins) atomicAdd(&hist[key0 - base], 1u);  // base is at or above the floor
  }
  wait_global_acks();
  __syncthreads();
  if (threadIdx.x == 0) s_last = atomicAdd(&hist[kRefineBins], 1u) == gridDim.x - 1u;
  __syncthreads();
  if (!s_last) return;
  // from the top down: thread t owns the kPer bins below kRefineBins - t * kPer.  The counts were raised
  // by atomics in memory and this workgroup has not looked at them before: once the cache lines it may
  // hold are dropped, plain 16-byte loads see them all, and many of them are in flight together (one
  // uncached load after the other took 50 us here)
  constexpr int kPer = kRefineBins / kRefineBlock;
  static_assert(kPer % 4 == 0, "a thread's bins are read four at a time");
  const uint32_t hi = (uint32_t)kRefineBins - threadIdx.x * (uint32_t)kPer;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  uint32_t mine = 0;
  {
    const uint4 *own = reinterpret_cast<const uint4 *>(hist + (hi - (uint32_t)kPer));
#pragma unroll 8
    for (int j = 0; j < kPer / 4; ++j) {
      const uint4 q = own[j];
      mine += q.x + q.y + q.z + q.w;
    }
  }
  uint32_t total;
  uint32_t before = block_exclusive_scan<uint32_t, kRefineBlock>(mine, s_scan, &total);
  const uint32_t over = above[0];
  const uint32_t need = k > over ? k - over : 1u;  // rank inside the bin, from the top
  if (total < need) {
    if (threadIdx.x == 0) atomicOr(status, ZEN_STAT_RETRY);  // the two histograms disagree: let the general mode answer
    return;
  }
  // the thread whose bins hold the rank hands them to the first wave: a lane takes two bins, from the top down
  __shared__ uint32_t s_hi, s_before;
  if (before < need && need <= before + mine) {
    s_hi = hi;
    s_before = before;
  }
  __syncthreads();
  if (threadIdx.x >= 64) return;
  static_assert(kPer == 128, "two bins per lane of one wave");
  const uint32_t top = s_hi;  // the bins top - 1, top - 2, ... top - kPer
  const uint2 two = *reinterpret_cast<const uint2 *>(hist + (top - 2u * (threadIdx.x + 1u)));  // .y is the upper bin
  const uint32_t pair = two.x + two.y;
  const uint32_t incl = wave_inclusive_scan(pair);
  const uint32_t ahead = s_before + incl - pair;  // elements above the lane's two bins
  if (ahead < need && need <= ahead + pair) {
    const bool upper = need <= ahead + two.y;
    const uint32_t bin = top - 2u * threadIdx.x - (upper ? 1u : 2u);
    const uint32_t at_or_above = over + ahead + two.y + (upper ? 0u : two.x);
    thr[0] = base + bin;
    thr[1] = at_or_above;
    if (thr_copy) {
      thr_copy[0] = base + bin;
      thr_copy[1] = at_or_above;
    }
  }
}

}  // namespace
}  // namespace zen
