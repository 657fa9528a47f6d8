// Vector loads and the ordered-compaction entry shared by the select and
// load-balance translation units.
#pragma once

#include "zen_common.h"

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

// Ascending (index, value) list of the elements with key >= max(thr[0], 1);
// thr == nullptr means "nonzero".  out_count (int64) and out_count32 (clamped
// to capacity) are optional.  scratch: select_scratch_bytes(n, dtype).
size_t select_scratch_bytes(int64_t n, int dtype);
int select_compact(const void *in, int dtype, int64_t n, const uint32_t *thr, void *out_idx, int idx64,
                   void *out_val, int64_t capacity, int64_t *out_count, uint32_t *out_count32,
                   void *scratch, int32_t *status, hipStream_t stream);

}  // namespace zen
