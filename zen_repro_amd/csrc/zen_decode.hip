// Dense decode of payloads that arrive as ascending lists (zen_decode_dense_sorted).
//
// The second exchange of the sparse all-reduce hands every rank all ranks'
// merged shards, each an ascending index list, and the reference scatter-adds
// them into a zeroed dense tensor (comm.py:142-145 with :32-44); method 1 does
// the same with every rank's own ascending selection (comm.py:113-117).  A
// dense result needs no sort: the dense tensor is cut into tiles of kDecTile
// elements, a first kernel finds where every tile starts in every list, and one
// workgroup per tile gathers its entries (a contiguous stretch of every list)
// into a copy of the tile in LDS and writes the tile out with full-width
// stores.  The dense tensor is written exactly once and never cleared first.
//
// Sums are taken in fp32 from +0 in payload order and rounded once, like
// zen_decode_dense: inside a list every index occurs once (the lists are
// strictly ascending; that is checked), so a tile whose entries are all
// distinct takes them in any order, and a tile in which two lists meet on an
// index goes through the lists one after the other.
#include "zen_common.h"

namespace zen {
namespace {

constexpr int kDecTile = 8192;   // dense elements per workgroup (its LDS copy: 16 KB for bf16, 32 KB for fp32)
constexpr int kDecBlock = 256;
constexpr int kDecMaxLists = 64;

struct DecLists {
  int64_t start[kDecMaxLists + 1];  // where every list starts in idx / val; start[n] = number of entries
  int n;
};

// starts[l * (ntiles + 1) + t] = number of entries of list l with index < t * kDecTile (by bisection, which
// assumes the list ascending; the tile kernel checks that it is).
template <typename I>
__global__ __launch_bounds__(256) void k_decode_starts(const I *__restrict__ idx, DecLists lists, int64_t ntiles,
                                                       uint32_t *__restrict__ starts) {
  const int64_t per_list = ntiles + 1;
  const int64_t g = blockIdx.x * (int64_t)256 + threadIdx.x;
  if (g >= per_list * lists.n) return;
  const int l = (int)(g / per_list);
  const int64_t t = g - (int64_t)l * per_list;
  const I *list = idx + lists.start[l];
  const uint32_t len = (uint32_t)(lists.start[l + 1] - lists.start[l]);
  uint32_t lo = 0, hi = len;
  if (t == 0) {
    hi = 0;
  } else if (t == ntiles) {
    lo = len;
  } else {
    const int64_t key = t * (int64_t)kDecTile;
    while (lo < hi) {
      const uint32_t mid = lo + ((hi - lo) >> 1);
      if ((int64_t)list[mid] < key)
        lo = mid + 1;
      else
        hi = mid;
    }
  }
  starts[g] = lo;
}

// The value a dense element gets from one entry: +0 + v in fp32, rounded to the tensor's type (-0 becomes +0,
// like in a scatter_add_ into zeros).
__device__ inline uint16_t single_value(uint16_t v) { return f32_to_bf16_rne(0.0f + KeyOf<uint16_t>::to_f32(v)); }
__device__ inline uint32_t single_value(uint32_t v) { return __float_as_uint(0.0f + __uint_as_float(v)); }
__device__ inline uint16_t rounded(float f, uint16_t) { return f32_to_bf16_rne(f); }
__device__ inline uint32_t rounded(float f, uint32_t) { return __float_as_uint(f); }

// n elements (a multiple of 16 bytes' worth, from a 16-byte aligned LDS array) to dense[first ..), as wide as
// the tensor's end and alignment allow.
template <typename S>
__device__ inline void store_run(const S *src, int n, S *__restrict__ dense, int64_t first, int64_t dense_n) {
  constexpr int V = 16 / sizeof(S);
  const bool wide = (reinterpret_cast<uintptr_t>(dense + first) & 15u) == 0;
  for (int j = threadIdx.x * V; j < n; j += kDecBlock * V) {
    if (wide && first + j + V <= dense_n) {
      *reinterpret_cast<uint4 *>(dense + first + j) = *reinterpret_cast<const uint4 *>(src + j);
    } else {
      for (int q = 0; q < V; ++q)
        if (first + j + q < dense_n) dense[first + j + q] = src[j + q];
    }
  }
}

constexpr int kDecStage = 2048;  // entries of a tile kept in LDS for the case that lists meet

// One workgroup per tile.  Anything that contradicts "every list strictly ascending, every index inside
// [0, dense_n)" raises ZEN_STAT_RETRY (the caller repeats with zen_decode_dense, which takes any input).
// The stretches of all lists are numbered through (list after list) and dealt to the threads in that order,
// so that the loads of a tile's few hundred entries are in flight together whatever list they belong to.
template <typename I, typename S>
__global__ __launch_bounds__(kDecBlock) void k_decode_tiles(const I *__restrict__ idx, const S *__restrict__ val,
                                                            DecLists lists, int64_t ntiles,
                                                            const uint32_t *__restrict__ starts, S *__restrict__ dense,
                                                            int64_t dense_n, int32_t *status) {
  // The tile in the tensor's own type; where lists meet the same memory holds fp32 sums for a part of the tile
  // at a time (LDS decides how many tiles a compute unit has in flight, and the kernel lives on that).
  __shared__ __attribute__((aligned(16))) S tile[kDecTile];
  __shared__ uint32_t occ[kDecTile / 32];
  __shared__ int64_t s_base[kDecMaxLists];      // where the list's stretch starts in idx / val
  __shared__ uint32_t s_first[kDecMaxLists];    // entry number inside the list of the stretch's first entry
  __shared__ uint32_t s_pref[kDecMaxLists + 1];  // entries of the lists before, in this tile
  __shared__ uint16_t st_off[kDecStage];
  __shared__ S st_val[kDecStage];
  __shared__ uint32_t s_meet, s_wrong;
  static_assert(kDecMaxLists == 64 && kDecTile <= 65536, "one wave scans the lists; offsets are 16 bits");
  const int64_t t = blockIdx.x;
  const int64_t first = t * (int64_t)kDecTile;
  const int64_t per_list = ntiles + 1;
  uint32_t a = 0, b = 0;  // asked for first: the answer is on its way while the tile is cleared
  if ((int)threadIdx.x < lists.n) {
    a = starts[threadIdx.x * per_list + t];
    b = starts[threadIdx.x * per_list + t + 1];
  }
  for (int j = threadIdx.x; j < kDecTile; j += kDecBlock) tile[j] = 0;
  for (int j = threadIdx.x; j < kDecTile / 32; j += kDecBlock) occ[j] = 0;
  if (threadIdx.x == 0) s_meet = s_wrong = 0;
  if (threadIdx.x < 64) {
    uint32_t len = 0;
    bool back = false;
    if ((int)threadIdx.x < lists.n) {
      back = b < a;  // the bisection went astray: the list is not ascending
      len = back ? 0u : b - a;
      s_first[threadIdx.x] = a;
      s_base[threadIdx.x] = lists.start[threadIdx.x] + a;
    }
    const uint32_t incl = wave_inclusive_scan(len);
    if ((int)threadIdx.x < lists.n) s_pref[threadIdx.x] = incl - len;
    if ((int)threadIdx.x == lists.n - 1) s_pref[lists.n] = incl;
    if (back) atomicOr(&s_wrong, 1u);
  }
  __syncthreads();
  const uint32_t total = s_pref[lists.n];
  bool wrong = false, meet = false;
  for (uint32_t f = threadIdx.x; f < total; f += kDecBlock) {
    int lo = 0, hi = lists.n;  // the list f belongs to: the last one with s_pref <= f
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_pref[mid] <= f)
        lo = mid;
      else
        hi = mid;
    }
    const uint32_t within = f - s_pref[lo];
    const int64_t at = s_base[lo] + within;
    const int64_t k = (int64_t)idx[at];
    const uint64_t off = (uint64_t)(k - first);
    // the entry before it in its list (if there is one) must be smaller
    const bool has_prev = s_first[lo] + within > 0;
    if (off >= (uint64_t)kDecTile || k >= dense_n || (has_prev && (int64_t)idx[at - 1] >= k)) {
      wrong = true;
      continue;
    }
    const S v = val[at];
    const uint32_t bit = 1u << (off & 31u);
    if (atomicOr(&occ[off >> 5], bit) & bit) meet = true;
    tile[off] = single_value(v);
    if (f < (uint32_t)kDecStage) {
      st_off[f] = (uint16_t)off;
      st_val[f] = v;
    }
  }
  if (wrong) s_wrong = 1;
  if (meet) s_meet = 1;
  __syncthreads();
  if (s_wrong) {
    if (threadIdx.x == 0) atomicOr(status, ZEN_STAT_RETRY);
    return;  // the caller repeats the whole call: what this tile holds does not matter
  }
  if (!s_meet) {
    store_run<S>(tile, kDecTile, dense, first, dense_n);
    return;
  }
  // Two lists share an index here: fp32 sums, the lists one after the other (inside a list every index occurs
  // once), from the staged copy, or from memory again if the tile holds more entries than the stage.  The
  // tile's memory holds the sums of kPart elements at a time; each part is rounded in place and written out.
  constexpr int kPart = kDecTile * (int)sizeof(S) / (int)sizeof(float);
  float *acc = reinterpret_cast<float *>(tile);
  for (int part = 0; part < kDecTile; part += kPart) {
    for (int j = threadIdx.x; j < kPart; j += kDecBlock) acc[j] = 0.0f;
    __syncthreads();
    for (int l = 0; l < lists.n; ++l) {
      const uint32_t f0 = s_pref[l], f1 = s_pref[l + 1];
      for (uint32_t f = f0 + threadIdx.x; f < f1; f += kDecBlock) {
        uint32_t off;
        S v;
        if (f < (uint32_t)kDecStage) {
          off = st_off[f];
          v = st_val[f];
        } else {
          const int64_t at = s_base[l] + (f - f0);
          off = (uint32_t)((int64_t)idx[at] - first);
          v = val[at];
        }
        if (off - (uint32_t)part < (uint32_t)kPart) acc[off - (uint32_t)part] += KeyOf<S>::to_f32(v);
      }
      __syncthreads();
    }
    // rounded where it stands: a thread reads the sums of its own 16 bytes of output before it writes them
    // (the narrower type's array overlays the first part of the sums' memory, ahead of what is still unread
    // only for other threads' elements, hence the barrier between reading and writing)
    constexpr int V = 16 / (int)sizeof(S);
    S out[kPart / kDecBlock];
#pragma unroll
    for (int i = 0; i < kPart / kDecBlock / V; ++i)
#pragma unroll
      for (int q = 0; q < V; ++q) out[i * V + q] = rounded(acc[(threadIdx.x + i * kDecBlock) * V + q], S(0));
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kPart / kDecBlock / V; ++i)
#pragma unroll
      for (int q = 0; q < V; ++q) tile[(threadIdx.x + i * kDecBlock) * V + q] = out[i * V + q];
    __syncthreads();
    store_run<S>(tile, kPart, dense, first + part, dense_n);
    __syncthreads();
  }
}

template <typename I, typename S>
int decode_sorted_launch(const I *idx, const S *val, const DecLists &lists, S *dense, int64_t dense_n, uint32_t *starts,
                         int32_t *status, hipStream_t s) {
  const int64_t ntiles = ceil_div(dense_n, (int64_t)kDecTile);
  const int64_t searches = (ntiles + 1) * lists.n;
  k_decode_starts<I><<<dim3((unsigned)ceil_div(searches, (int64_t)256)), dim3(256), 0, s>>>(idx, lists, ntiles, starts);
  ZEN_LAUNCH_CHECK("k_decode_starts");
  k_decode_tiles<I, S><<<dim3((unsigned)ntiles), dim3(kDecBlock), 0, s>>>(idx, val, lists, ntiles, starts, dense,
                                                                          dense_n, status);
  ZEN_LAUNCH_CHECK("k_decode_tiles");
  return ZEN_OK;
}

}  // namespace
}  // namespace zen

extern "C" {

size_t zen_decode_dense_sorted_workspace(int64_t dense_n, int nlists) {
  if (dense_n <= 0 || nlists <= 0) return 256;
  const int64_t ntiles = zen::ceil_div(dense_n, (int64_t)zen::kDecTile);
  return (size_t)((ntiles + 1) * nlists) * sizeof(uint32_t) + 256;
}

int zen_decode_dense_sorted(const void *idx, int idx64_in, const void *val, int dtype, const int64_t *list_start,
                            int nlists, void *dense, int64_t dense_n, void *workspace, size_t workspace_bytes,
                            int32_t *status, void *stream) {
  using namespace zen;
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_decode_dense_sorted: bad dtype");
  if (!dense || !status || !list_start || !workspace) return fail(ZEN_EINVAL, "zen_decode_dense_sorted: null pointer");
  if (nlists < 1 || nlists > kDecMaxLists) return fail(ZEN_EINVAL, "zen_decode_dense_sorted: 1 to 64 lists");
  if (dense_n <= 0 || dense_n > 0x7fffffff00ll) return fail(ZEN_EINVAL, "zen_decode_dense_sorted: bad dense size");
  DecLists lists;
  lists.n = nlists;
  for (int l = 0; l <= nlists; ++l) {
    lists.start[l] = list_start[l];
    if (list_start[l] < 0 || (l > 0 && (list_start[l] < list_start[l - 1] || list_start[l] - list_start[l - 1] > 0xfffffffell)))
      return fail(ZEN_EINVAL, "zen_decode_dense_sorted: list offsets must ascend (lists below 2^32 entries)");
  }
  if (lists.start[0] != 0) return fail(ZEN_EINVAL, "zen_decode_dense_sorted: the first list starts at 0");
  if (lists.start[nlists] > 0 && (!idx || !val)) return fail(ZEN_EINVAL, "zen_decode_dense_sorted: null pointer");
  if (workspace_bytes < zen_decode_dense_sorted_workspace(dense_n, nlists))
    return fail(ZEN_EWORKSPACE, "zen_decode_dense_sorted: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint32_t *starts = static_cast<uint32_t *>(workspace);
  if (dtype == ZEN_BF16) {
    if (idx64_in)
      return decode_sorted_launch(static_cast<const int64_t *>(idx), static_cast<const uint16_t *>(val), lists,
                                  static_cast<uint16_t *>(dense), dense_n, starts, status, s);
    return decode_sorted_launch(static_cast<const int32_t *>(idx), static_cast<const uint16_t *>(val), lists,
                                static_cast<uint16_t *>(dense), dense_n, starts, status, s);
  }
  if (idx64_in)
    return decode_sorted_launch(static_cast<const int64_t *>(idx), static_cast<const uint32_t *>(val), lists,
                                static_cast<uint32_t *>(dense), dense_n, starts, status, s);
  return decode_sorted_launch(static_cast<const int32_t *>(idx), static_cast<const uint32_t *>(val), lists,
                              static_cast<uint32_t *>(dense), dense_n, starts, status, s);
}

}  // extern "C"
