// Small open-addressing map in borrowed zeroed memory: per table slot the
// smallest index that probed it at rehash level 2 or 3.  Shared by the two
// sort-based owner resolutions.
#pragma once

#include "zen_common.h"

namespace zen {

constexpr uint32_t kNone = 0xffffffffu;
constexpr uint32_t kChainLimit = 1u << 22;    // bounded chain: flag instead of spinning forever

struct Counters {
  uint32_t logged;      // entries in the log (losers, then displaced heads)
  uint32_t losers;      // snapshot of `logged` after the head pass
  uint32_t claims;      // occupied hash cells
  uint32_t displaced;   // slab path: level-1 owners pushed out by a level-2/3 prober (logged behind the losers)
};

__device__ inline uint32_t first_slot(const Probe &g, uint32_t t) { return (poly(t) + kSeed1) % g.m; }

// ---------------------------------------------------------------- hash map
// cell = (slot + 1) << 32 | index; 0 = empty.  Same-slot cells order by index,
// so atomicMin keeps the smallest prober.

__device__ inline uint32_t cell_home(uint32_t slot, uint32_t log2) { return (slot * 0x9E3779B1u) >> (32 - log2); }

// Returns the previous smallest index for `slot` (kNone if there was none) after
// entering t; *full is set if the map has no room.
__device__ inline uint32_t map_min(unsigned long long *cells, uint32_t log2, uint32_t slot, uint32_t t,
                                   Counters *ctr, bool *full) {
  const uint32_t mask = (1u << log2) - 1u;
  const unsigned long long mine = ((unsigned long long)(slot + 1u) << 32) | t;
  uint32_t h = cell_home(slot, log2);
  for (uint32_t probes = 0; probes <= mask; ++probes, h = (h + 1u) & mask) {
    unsigned long long cur = __hip_atomic_load(&cells[h], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (cur == 0ull) {
      const unsigned long long seen = atomicCAS(&cells[h], 0ull, mine);
      if (seen == 0ull) {
        if (atomicAdd(&ctr->claims, 1u) > (mask >> 1)) *full = true;
        return kNone;
      }
      cur = seen;
    }
    if ((uint32_t)(cur >> 32) == slot + 1u) {
      const unsigned long long old = atomicMin(&cells[h], mine);
      return (uint32_t)old;
    }
  }
  *full = true;
  return 0u;  // pretend a smaller index owns it: the chain moves on and the call is retried anyway
}

__device__ inline uint32_t map_find(const unsigned long long *cells, uint32_t log2, uint32_t slot, uint32_t *cell_out) {
  const uint32_t mask = (1u << log2) - 1u;
  uint32_t h = cell_home(slot, log2);
  for (uint32_t probes = 0; probes <= mask; ++probes, h = (h + 1u) & mask) {
    const unsigned long long cur = cells[h];
    if (cur == 0ull) return kNone;
    if ((uint32_t)(cur >> 32) == slot + 1u) {
      if (cell_out) *cell_out = h;
      return (uint32_t)cur;
    }
  }
  return kNone;
}

}  // namespace zen
