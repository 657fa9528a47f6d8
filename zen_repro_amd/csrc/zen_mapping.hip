// calculate_mapping (comm.py:52-56): for every partition the ascending list of
// indices that hash to it.  Built as one stable sort of (partition id, index)
// instead of the reference's P full scans of an int32[n] tensor.
#include "zen_common.h"

namespace zen {
namespace {

__global__ __launch_bounds__(256) void k_map_prep(uint32_t n, uint32_t per_part, uint32_t *__restrict__ keys,
                                                  uint32_t *__restrict__ vals) {
  for (uint32_t t = blockIdx.x * 256u + threadIdx.x; t < n; t += gridDim.x * 256u) {
    keys[t] = ((poly(t) + kSeed1) % n) / per_part;
    vals[t] = t;
  }
}

__global__ __launch_bounds__(256) void k_map_out(const uint32_t *__restrict__ keys, const uint32_t *__restrict__ vals,
                                                 uint32_t n, uint32_t partitions, int64_t *__restrict__ out) {
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += gridDim.x * 256u)
    if (keys[i] < partitions) out[i] = (int64_t)vals[i];
}

__global__ void k_map_counts(const uint32_t *__restrict__ keys, uint32_t n, int partitions,
                             int64_t *__restrict__ counts) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= partitions) return;
  uint32_t bound[2];
  for (int s = 0; s < 2; ++s) {
    uint32_t lo = 0, hi = n;
    const uint32_t x = (uint32_t)p + s;
    while (lo < hi) {
      const uint32_t mid = lo + ((hi - lo) >> 1);
      if (keys[mid] < x) lo = mid + 1; else hi = mid;
    }
    bound[s] = lo;
  }
  counts[p] = (int64_t)(bound[1] - bound[0]);
}

}  // namespace
}  // namespace zen

extern "C" {

size_t zen_mapping_workspace(int64_t n, int partitions) {
  (void)partitions;
  if (n <= 0) return 0;
  return 4 * zen::align_up((size_t)n * sizeof(uint32_t), 256) + zen::sort_scratch_bytes(n);
}

int zen_mapping(int64_t n, int partitions, int64_t *out, int64_t *counts, void *workspace, size_t workspace_bytes,
                int32_t *status, void *stream) {
  using namespace zen;
  if (!out || !counts || !workspace || !status) return fail(ZEN_EINVAL, "zen_mapping: null pointer");
  if (n <= 0 || n > 0x7fffffffll || partitions <= 0 || n / partitions == 0)
    return fail(ZEN_EINVAL, "zen_mapping: need 0 < partitions <= n < 2^31");
  if (workspace_bytes < zen_mapping_workspace(n, partitions)) return fail(ZEN_EWORKSPACE, "zen_mapping: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  Carver cv(workspace);
  uint32_t *ka = cv.take<uint32_t>((size_t)n), *va = cv.take<uint32_t>((size_t)n);
  uint32_t *kb = cv.take<uint32_t>((size_t)n), *vb = cv.take<uint32_t>((size_t)n);
  void *scratch = cv.take<char>(sort_scratch_bytes(n));
  int64_t blocks = ceil_div(n, 1024);
  if (blocks > 65536) blocks = 65536;
  k_map_prep<<<dim3((unsigned)blocks), dim3(256), 0, s>>>((uint32_t)n, (uint32_t)(n / partitions), ka, va);
  ZEN_LAUNCH_CHECK("k_map_prep");
  const int where = sort_pairs(ka, va, kb, vb, n, nullptr, ceil_log2_u64((uint64_t)partitions), scratch, status, s);
  if (where < 0) return where;
  const uint32_t *sk = where ? kb : ka, *sv = where ? vb : va;
  k_map_out<<<dim3((unsigned)blocks), dim3(256), 0, s>>>(sk, sv, (uint32_t)n, (uint32_t)partitions, out);
  ZEN_LAUNCH_CHECK("k_map_out");
  k_map_counts<<<dim3((unsigned)ceil_div(partitions, 64)), dim3(64), 0, s>>>(sk, (uint32_t)n, partitions, counts);
  ZEN_LAUNCH_CHECK("k_map_counts");
  return ZEN_OK;
}

}  // extern "C"
