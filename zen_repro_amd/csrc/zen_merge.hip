// Receive side: merge many (index, value) payloads.  The reference builds a
// dense zero tensor of the full gradient length, scatter-adds every payload
// into it and extracts the nonzeros again (comm.py:32-50).  Here the entries
// are stably sorted by index, equal indices are summed in fp32 in arrival order
// (the order a sequential scatter_add_ uses, so the result is reproducible),
// zero sums are dropped and the survivors leave in ascending index order.
#include "zen_common.h"

namespace zen {
namespace {

constexpr int kMrgBlock = 256;
constexpr int kMrgItems = 4;  // consecutive sorted entries per thread
constexpr int kMrgTile = kMrgBlock * kMrgItems;

template <typename I>
__global__ __launch_bounds__(256) void k_merge_prep(const I *__restrict__ idx, uint32_t r, uint32_t dense_n,
                                                    uint32_t *__restrict__ keys, uint32_t *__restrict__ perm,
                                                    int32_t *status) {
  const uint32_t j = blockIdx.x * 256u + threadIdx.x;
  if (j >= r) return;
  const I k = idx[j];
  const bool ok = k >= 0 && (uint64_t)k < (uint64_t)dense_n;
  if (!ok) atomicOr(status, ZEN_STAT_BAD_INDEX);
  keys[j] = ok ? (uint32_t)k : dense_n;  // bad indices sort behind every good one
  perm[j] = j;
}

template <typename S, typename I>
__global__ __launch_bounds__(kMrgBlock) void k_merge_reduce(
    const uint32_t *__restrict__ keys, const uint32_t *__restrict__ perm, const S *__restrict__ val, uint32_t r,
    uint32_t dense_n, I *__restrict__ out_idx, float *__restrict__ out_val, int64_t capacity,
    unsigned long long *desc, uint32_t *ticket, int ntiles, int64_t *out_count, int32_t *status) {
  __shared__ uint32_t s_scan[kMrgBlock / 64 + 1];
  __shared__ uint64_t s_bcast;
  __shared__ int s_tile;
  if (threadIdx.x == 0) s_tile = (int)atomicAdd(ticket, 1u);
  __syncthreads();
  const int tile = s_tile;
  if (tile >= ntiles) return;
  const uint32_t first = (uint32_t)tile * kMrgTile + threadIdx.x * kMrgItems;
  uint32_t k[kMrgItems];
  float sum[kMrgItems];
  uint32_t keep = 0;
  uint32_t prev = first > 0 && first - 1 < r ? keys[first - 1] : 0xffffffffu;
#pragma unroll
  for (int q = 0; q < kMrgItems; ++q) {
    const uint32_t i = first + q;
    k[q] = i < r ? keys[i] : 0xffffffffu;
    const bool head = i < r && k[q] < dense_n && (i == 0 || k[q] != prev);
    prev = k[q];
    sum[q] = 0.0f;
    if (head) {
      float acc = 0.0f;  // the dense tensor starts at +0 (comm.py:35)
      for (uint32_t u = i; u < r && keys[u] == k[q]; ++u) acc += KeyOf<S>::to_f32(val[perm[u]]);
      sum[q] = acc;
      if (acc != 0.0f) keep |= 1u << q;  // torch.nonzero keeps NaN, drops +-0
    }
  }
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kMrgBlock>((uint32_t)__popc(keep), s_scan, &total);
  const uint64_t tile_start = lookback_exclusive(desc, tile, total, status, &s_bcast);
  if (tile == ntiles - 1 && threadIdx.x == 0) {
    const uint64_t all = tile_start + total;
    *out_count = (int64_t)all;
    if (all > (uint64_t)capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
  uint64_t pos = tile_start + before;
#pragma unroll
  for (int q = 0; q < kMrgItems; ++q) {
    if (keep & (1u << q)) {
      if (pos < (uint64_t)capacity) {
        out_idx[pos] = (I)k[q];
        out_val[pos] = sum[q];
      }
      ++pos;
    }
  }
}

template <typename S>
__global__ __launch_bounds__(256) void k_scatter_dense(const int32_t *__restrict__ idx, const float *__restrict__ sum,
                                                       const int64_t *count, S *__restrict__ dense);
template <>
__global__ __launch_bounds__(256) void k_scatter_dense<uint32_t>(const int32_t *__restrict__ idx,
                                                                 const float *__restrict__ sum,
                                                                 const int64_t *count, uint32_t *__restrict__ dense) {
  const int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x;
  if (i < *count) dense[idx[i]] = __float_as_uint(sum[i]);
}
template <>
__global__ __launch_bounds__(256) void k_scatter_dense<uint16_t>(const int32_t *__restrict__ idx,
                                                                 const float *__restrict__ sum,
                                                                 const int64_t *count, uint16_t *__restrict__ dense) {
  const int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x;
  if (i < *count) dense[idx[i]] = f32_to_bf16_rne(sum[i]);
}

struct MergePlan {
  uint32_t *keys_a, *perm_a, *keys_b, *perm_b;
  unsigned long long *desc;  // ntiles descriptors + ticket
  void *sort_scratch;
  size_t bytes;
  int ntiles;
};

MergePlan plan_merge(void *workspace, int64_t r) {
  Carver cv(workspace);
  MergePlan p;
  const size_t cap = (size_t)(r > 0 ? r : 1);
  p.keys_a = cv.take<uint32_t>(cap);
  p.perm_a = cv.take<uint32_t>(cap);
  p.keys_b = cv.take<uint32_t>(cap);
  p.perm_b = cv.take<uint32_t>(cap);
  p.ntiles = (int)ceil_div((int64_t)cap, kMrgTile);
  p.desc = cv.take<unsigned long long>((size_t)p.ntiles + 2);
  p.sort_scratch = cv.take<char>(sort_scratch_bytes((int64_t)cap));
  p.bytes = cv.used;
  return p;
}

template <typename S>
int merge_launch(const void *idx, int idx64_in, const S *val, int64_t r, int64_t dense_n, void *out_idx,
                 int idx64_out, float *out_val, int64_t capacity, int64_t *out_count, void *workspace,
                 int32_t *status, hipStream_t s) {
  MergePlan p = plan_merge(workspace, r);
  const unsigned blocks = (unsigned)ceil_div(r, 256);
  {
    ProfScope prof(kProfMergePrep, s);
    if (idx64_in)
      k_merge_prep<int64_t><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const int64_t *>(idx), (uint32_t)r,
                                                               (uint32_t)dense_n, p.keys_a, p.perm_a, status);
    else
      k_merge_prep<int32_t><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const int32_t *>(idx), (uint32_t)r,
                                                               (uint32_t)dense_n, p.keys_a, p.perm_a, status);
    ZEN_LAUNCH_CHECK("k_merge_prep");
  }
  const int bits = ceil_log2_u64((uint64_t)dense_n);
  int where;
  {
    ProfScope prof(kProfSort, s);
    where = sort_pairs(p.keys_a, p.perm_a, p.keys_b, p.perm_b, r, nullptr, bits, p.sort_scratch, s);
  }
  if (where < 0) return where;
  const uint32_t *sk = where ? p.keys_b : p.keys_a;
  const uint32_t *sp = where ? p.perm_b : p.perm_a;
  launch_fill<unsigned long long>(p.desc, 0ull, (size_t)p.ntiles + 1, s);
  ZEN_LAUNCH_CHECK("merge: clear descriptors");
  uint32_t *ticket = reinterpret_cast<uint32_t *>(p.desc + p.ntiles);
  ProfScope prof(kProfMergeReduce, s);
  if (idx64_out)
    k_merge_reduce<S, int64_t><<<dim3((unsigned)p.ntiles), dim3(kMrgBlock), 0, s>>>(
        sk, sp, val, (uint32_t)r, (uint32_t)dense_n, static_cast<int64_t *>(out_idx), out_val, capacity, p.desc,
        ticket, p.ntiles, out_count, status);
  else
    k_merge_reduce<S, int32_t><<<dim3((unsigned)p.ntiles), dim3(kMrgBlock), 0, s>>>(
        sk, sp, val, (uint32_t)r, (uint32_t)dense_n, static_cast<int32_t *>(out_idx), out_val, capacity, p.desc,
        ticket, p.ntiles, out_count, status);
  ZEN_LAUNCH_CHECK("k_merge_reduce");
  return ZEN_OK;
}

int merge_check(const void *idx, const void *val, int dtype, int64_t r, int64_t dense_n, const char **why) {
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) { *why = "bad dtype"; return ZEN_EINVAL; }
  if (r < 0 || r > 0x7ffffffell || dense_n <= 0 || dense_n > 0x7fffffffll) {
    *why = "need 0 <= r < 2^31 - 1 and 0 < dense_n < 2^31";
    return ZEN_EINVAL;
  }
  if (r > 0 && (!idx || !val)) { *why = "null pointer"; return ZEN_EINVAL; }
  return ZEN_OK;
}

}  // namespace
}  // namespace zen

extern "C" {

size_t zen_merge_workspace(int64_t r) {
  if (r < 0) return 0;
  return zen::plan_merge(nullptr, r).bytes;
}

int zen_merge(const void *idx, int idx64_in, const void *val, int dtype, int64_t r, int64_t dense_n, void *out_idx,
              int idx64_out, float *out_val, int64_t capacity, int64_t *out_count, void *workspace,
              size_t workspace_bytes, int32_t *status, void *stream) {
  using namespace zen;
  const char *why = "";
  if (merge_check(idx, val, dtype, r, dense_n, &why) != ZEN_OK) return fail(ZEN_EINVAL, why);
  if (!out_count || !status || capacity < 0) return fail(ZEN_EINVAL, "zen_merge: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (r == 0) {
    launch_fill<int64_t>(out_count, 0, 1, s);
    ZEN_LAUNCH_CHECK("zen_merge: zero count");
    return ZEN_OK;
  }
  if (!workspace || (capacity > 0 && (!out_idx || !out_val))) return fail(ZEN_EINVAL, "zen_merge: null pointer");
  if (workspace_bytes < zen_merge_workspace(r)) return fail(ZEN_EWORKSPACE, "zen_merge: workspace too small");
  if (dtype == ZEN_BF16)
    return merge_launch(idx, idx64_in, static_cast<const uint16_t *>(val), r, dense_n, out_idx, idx64_out, out_val,
                        capacity, out_count, workspace, status, s);
  return merge_launch(idx, idx64_in, static_cast<const uint32_t *>(val), r, dense_n, out_idx, idx64_out, out_val,
                      capacity, out_count, workspace, status, s);
}

size_t zen_decode_dense_workspace(int64_t r) {
  if (r < 0) return 0;
  const size_t cap = (size_t)(r > 0 ? r : 1);
  return zen::align_up(cap * sizeof(int32_t), 256) + zen::align_up(cap * sizeof(float), 256) + 256 +
         zen_merge_workspace(r);
}

int zen_decode_dense(const void *idx, int idx64_in, const void *val, int dtype, int64_t r, void *dense,
                     int64_t dense_n, void *workspace, size_t workspace_bytes, int32_t *status, void *stream) {
  using namespace zen;
  const char *why = "";
  if (merge_check(idx, val, dtype, r, dense_n, &why) != ZEN_OK) return fail(ZEN_EINVAL, why);
  if (!dense || !status) return fail(ZEN_EINVAL, "zen_decode_dense: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == ZEN_BF16)
    launch_fill<uint16_t>(static_cast<uint16_t *>(dense), (uint16_t)0, (size_t)dense_n, s);
  else
    launch_fill<uint32_t>(static_cast<uint32_t *>(dense), 0u, (size_t)dense_n, s);
  ZEN_LAUNCH_CHECK("zen_decode_dense: clear");
  if (r == 0) return ZEN_OK;
  if (!workspace) return fail(ZEN_EINVAL, "zen_decode_dense: null pointer");
  if (workspace_bytes < zen_decode_dense_workspace(r)) return fail(ZEN_EWORKSPACE, "zen_decode_dense: workspace too small");
  Carver cv(workspace);
  int32_t *m_idx = cv.take<int32_t>((size_t)r);
  float *m_val = cv.take<float>((size_t)r);
  int64_t *m_count = cv.take<int64_t>(1);
  void *inner = cv.take<char>(zen_merge_workspace(r));
  int rc;
  if (dtype == ZEN_BF16)
    rc = merge_launch(idx, idx64_in, static_cast<const uint16_t *>(val), r, dense_n, m_idx, 0, m_val, r, m_count,
                      inner, status, s);
  else
    rc = merge_launch(idx, idx64_in, static_cast<const uint32_t *>(val), r, dense_n, m_idx, 0, m_val, r, m_count,
                      inner, status, s);
  if (rc != ZEN_OK) return rc;
  const unsigned blocks = (unsigned)ceil_div(r, 256);
  if (dtype == ZEN_BF16)
    k_scatter_dense<uint16_t><<<dim3(blocks), dim3(256), 0, s>>>(m_idx, m_val, m_count, static_cast<uint16_t *>(dense));
  else
    k_scatter_dense<uint32_t><<<dim3(blocks), dim3(256), 0, s>>>(m_idx, m_val, m_count, static_cast<uint32_t *>(dense));
  ZEN_LAUNCH_CHECK("k_scatter_dense");
  return ZEN_OK;
}

}  // extern "C"
