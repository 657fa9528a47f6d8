// Magnitude selection: exact k-th largest |g| by radix select over the
// magnitude bit pattern (train.py:81-82), the masked dense copy
// (train.py:83), and the ordered single-pass compaction that turns a dense
// tensor into ascending (index, value) lists (comm.py:47-50).
#include "zen_select.h"

namespace zen {
namespace {

// ------------------------------------------------------------ radix select

constexpr int kHistBins = 2048;
constexpr int kHistBlock = 256;

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
__global__ __launch_bounds__(kHistBlock) void k_topk_hist(const S *__restrict__ in, int64_t n,
                                                          const TopkState *__restrict__ st, int shift,
                                                          int width, int pass,
                                                          uint32_t *__restrict__ hist) {
  constexpr int V = VecOf<S>::kN;
  __shared__ uint32_t bins[kHistBins];
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
// prefix, clear the histogram for the next pass.
__global__ __launch_bounds__(kHistBlock) void k_topk_pick(TopkState *st, uint32_t *hist, int width,
                                                          int last, uint32_t *thr_out) {
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
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    if (above < k_rem && k_rem <= above + c[j]) {
      const uint32_t bin = kHistBins - 1 - (threadIdx.x * kPer + j);
      const uint32_t np = (prefix << width) | bin;
      st->prefix = np;
      st->k_rem = k_rem - above;
      st->count_gt = count_gt + above;
      if (last) {
        thr_out[0] = np;
        thr_out[1] = count_gt + above + c[j];
      }
    }
    above += c[j];
  }
#pragma unroll
  for (int j = 0; j < kPer; ++j) hist[kHistBins - 1 - (threadIdx.x * kPer + j)] = 0;
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

// ------------------------------------------------------ ordered compaction
//
// A tile is `subs` consecutive sub-tiles of kSelBlock * kSelVecs 16-byte
// vectors.  A block walks its tile once, staging the selected (index, value)
// pairs in LDS in ascending order; only then does it need the number of
// selected elements in all earlier tiles, which it gets by look-back over one
// descriptor per tile.  Large tiles keep the descriptor chain short (the
// look-back frontier advances 64 tiles per memory round trip), the LDS stage
// makes the write-out coalesced.  A tile with more selected elements than the
// stage holds is walked a second time and written directly.

constexpr int kSelStage = 4096;  // staged pairs per tile

template <typename S, typename I, bool ALIGNED, bool STAGED>
__device__ inline uint32_t select_walk_tile(const S *__restrict__ in, int64_t n, uint32_t floor_key,
                                            int64_t tile_base, int subs, uint64_t *s_scan, int32_t *st_idx,
                                            S *st_val, I *__restrict__ out_idx, S *__restrict__ out_val,
                                            uint64_t out_base, int64_t capacity) {
  constexpr int V = VecOf<S>::kN;
  constexpr int kSub = kSelBlock * kSelVecs * V;
  uint32_t running = 0;
  for (int sub = 0; sub < subs; ++sub) {
    const int64_t sub_base = tile_base + (int64_t)sub * kSub;
    if (sub_base >= n) break;
    S e[kSelVecs][V];
    uint32_t bits[kSelVecs];
    uint64_t packed = 0;  // four 16-bit counters, one per vector of this thread
#pragma unroll
    for (int j = 0; j < kSelVecs; ++j) {
      const int64_t first = sub_base + ((int64_t)j * kSelBlock + threadIdx.x) * V;
      const int live = first < n ? load_vec<S, ALIGNED>(in, first, n, e[j]) : 0;
      uint32_t b = 0;
#pragma unroll
      for (int i = 0; i < V; ++i)
        if (i < live && (e[j][i] & KeyOf<S>::kMask) >= floor_key) b |= 1u << i;
      bits[j] = b;
      packed |= (uint64_t)__popc(b) << (16 * j);
    }
    uint64_t totals;
    const uint64_t before = block_exclusive_scan<uint64_t, kSelBlock>(packed, s_scan, &totals);
    uint32_t vec_start = running;
#pragma unroll
    for (int j = 0; j < kSelVecs; ++j) {
      uint32_t pos = vec_start + (uint32_t)((before >> (16 * j)) & 0xffffu);
      const int64_t first = sub_base + ((int64_t)j * kSelBlock + threadIdx.x) * V;
      const uint32_t b = bits[j];
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if (b & (1u << i)) {
          if (STAGED) {
            if (pos < (uint32_t)kSelStage) {
              st_idx[pos] = (int32_t)(first + i);
              st_val[pos] = e[j][i];
            }
          } else if (out_base + pos < (uint64_t)capacity) {
            out_idx[out_base + pos] = (I)(first + i);
            out_val[out_base + pos] = e[j][i];
          }
          ++pos;
        }
      }
      vec_start += (uint32_t)((totals >> (16 * j)) & 0xffffu);
    }
    running = vec_start;
  }
  return running;
}

template <typename S, typename I, bool ALIGNED>
__global__ __launch_bounds__(kSelBlock) void k_select_compact(
    const S *__restrict__ in, int64_t n, const uint32_t *__restrict__ thr, I *__restrict__ out_idx,
    S *__restrict__ out_val, int64_t capacity, unsigned long long *desc, uint32_t *ticket, int ntiles, int subs,
    int64_t *out_count, uint32_t *out_count32, int32_t *status) {
  constexpr int V = VecOf<S>::kN;
  constexpr int kSub = kSelBlock * kSelVecs * V;
  __shared__ uint64_t s_scan[kSelBlock / 64 + 1];
  __shared__ uint64_t s_bcast;
  __shared__ int s_tile;
  __shared__ int32_t st_idx[kSelStage];
  __shared__ S st_val[kSelStage];
  if (threadIdx.x == 0) s_tile = (int)atomicAdd(ticket, 1u);
  __syncthreads();
  const int tile = s_tile;
  if (tile >= ntiles) return;
  uint32_t floor_key = thr ? thr[0] : 1u;
  if (floor_key == 0) floor_key = 1u;  // zeros are never selected
  const int64_t tile_base = (int64_t)tile * subs * kSub;

  const uint32_t found = select_walk_tile<S, I, ALIGNED, true>(in, n, floor_key, tile_base, subs, s_scan, st_idx,
                                                               st_val, out_idx, out_val, 0, capacity);
  const uint64_t tile_start = lookback_exclusive(desc, tile, found, status, &s_bcast);
  if (tile == ntiles - 1 && threadIdx.x == 0) {
    const uint64_t all = tile_start + found;
    if (out_count) *out_count = (int64_t)all;
    if (out_count32) *out_count32 = (uint32_t)(all < (uint64_t)capacity ? all : (uint64_t)capacity);
    if (all > (uint64_t)capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
  if (found <= (uint32_t)kSelStage) {
    for (uint32_t i = threadIdx.x; i < found; i += kSelBlock) {
      const uint64_t pos = tile_start + i;
      if (pos < (uint64_t)capacity) {
        out_idx[pos] = (I)st_idx[i];
        out_val[pos] = st_val[i];
      }
    }
  } else {
    select_walk_tile<S, I, ALIGNED, false>(in, n, floor_key, tile_base, subs, s_scan, st_idx, st_val, out_idx,
                                           out_val, tile_start, capacity);
  }
}

// Sub-tiles per tile: large tiles for large inputs, but never so large that
// the grid falls below a few workgroups per compute unit.
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
  return align_up((size_t)(ntiles + 2) * sizeof(unsigned long long), 256);
}

template <typename S, typename I>
static int select_launch(const S *in, int64_t n, const uint32_t *thr, I *out_idx, S *out_val,
                         int64_t capacity, int64_t *out_count, uint32_t *out_count32, void *scratch,
                         int32_t *status, hipStream_t stream) {
  constexpr int V = VecOf<S>::kN;
  const int subs = select_subs(n, sizeof(S) == 2 ? ZEN_BF16 : ZEN_F32);
  const int64_t tile = (int64_t)kSelBlock * kSelVecs * V * subs;
  const int64_t ntiles = ceil_div(n, tile);
  if (ntiles > 0x7fffffff) return fail(ZEN_EINVAL, "select: too many tiles");
  // descriptors followed by the ticket counter, cleared together
  unsigned long long *desc = static_cast<unsigned long long *>(scratch);
  uint32_t *ticket = reinterpret_cast<uint32_t *>(desc + ntiles);
  launch_fill<unsigned long long>(desc, 0ull, (size_t)ntiles + 1, stream);
  ZEN_LAUNCH_CHECK("select: clear descriptors");
  const bool aligned = (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
  ProfScope prof(kProfSelectCompact, stream);
  if (aligned)
    k_select_compact<S, I, true><<<dim3((unsigned)ntiles), dim3(kSelBlock), 0, stream>>>(
        in, n, thr, out_idx, out_val, capacity, desc, ticket, (int)ntiles, subs, out_count, out_count32, status);
  else
    k_select_compact<S, I, false><<<dim3((unsigned)ntiles), dim3(kSelBlock), 0, stream>>>(
        in, n, thr, out_idx, out_val, capacity, desc, ticket, (int)ntiles, subs, out_count, out_count32, status);
  ZEN_LAUNCH_CHECK("k_select_compact");
  return ZEN_OK;
}

int select_compact(const void *in, int dtype, int64_t n, const uint32_t *thr, void *out_idx, int idx64,
                   void *out_val, int64_t capacity, int64_t *out_count, uint32_t *out_count32,
                   void *scratch, int32_t *status, hipStream_t stream) {
  if (dtype == ZEN_BF16) {
    auto *p = static_cast<const uint16_t *>(in);
    auto *v = static_cast<uint16_t *>(out_val);
    return idx64 ? select_launch<uint16_t, int64_t>(p, n, thr, static_cast<int64_t *>(out_idx), v, capacity,
                                                    out_count, out_count32, scratch, status, stream)
                 : select_launch<uint16_t, int32_t>(p, n, thr, static_cast<int32_t *>(out_idx), v, capacity,
                                                    out_count, out_count32, scratch, status, stream);
  }
  auto *p = static_cast<const uint32_t *>(in);
  auto *v = static_cast<uint32_t *>(out_val);
  return idx64 ? select_launch<uint32_t, int64_t>(p, n, thr, static_cast<int64_t *>(out_idx), v, capacity,
                                                  out_count, out_count32, scratch, status, stream)
               : select_launch<uint32_t, int32_t>(p, n, thr, static_cast<int32_t *>(out_idx), v, capacity,
                                                  out_count, out_count32, scratch, status, stream);
}

namespace {

template <typename S>
int topk_launch(const S *in, int64_t n, int64_t k, uint32_t *thr, void *workspace, hipStream_t stream) {
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
        k_topk_hist<S, true><<<dim3((unsigned)blocks), dim3(kHistBlock), 0, stream>>>(in, n, st, shift,
                                                                                      widths[p], p, hist);
      else
        k_topk_hist<S, false><<<dim3((unsigned)blocks), dim3(kHistBlock), 0, stream>>>(in, n, st, shift,
                                                                                       widths[p], p, hist);
      ZEN_LAUNCH_CHECK("k_topk_hist");
    }
    k_topk_pick<<<dim3(1), dim3(kHistBlock), 0, stream>>>(st, hist, widths[p], p == npass - 1, thr);
    ZEN_LAUNCH_CHECK("k_topk_pick");
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
}  // namespace zen

extern "C" {

size_t zen_topk_threshold_workspace(void) {
  return zen::align_up(sizeof(zen::TopkState), 256) + zen::align_up(zen::kHistBins * sizeof(uint32_t), 256);
}

int zen_topk_threshold(const void *input, int dtype, int64_t n, int64_t k, uint32_t *thr, void *workspace,
                       size_t workspace_bytes, void *stream) {
  using namespace zen;
  if (!input || !thr || !workspace) return fail(ZEN_EINVAL, "zen_topk_threshold: null pointer");
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_topk_threshold: bad dtype");
  if (n <= 0 || n > 0x7fffffffll || k < 1 || k > n) return fail(ZEN_EINVAL, "zen_topk_threshold: need 1 <= k <= n < 2^31");
  if (workspace_bytes < zen_topk_threshold_workspace()) return fail(ZEN_EWORKSPACE, "zen_topk_threshold: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == ZEN_BF16) return topk_launch(static_cast<const uint16_t *>(input), n, k, thr, workspace, s);
  return topk_launch(static_cast<const uint32_t *>(input), n, k, thr, workspace, s);
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
  return select_compact(input, dtype, n, thr, out_idx, idx64, out_val, capacity, out_count, nullptr,
                        workspace, status, s);
}

}  // extern "C"
