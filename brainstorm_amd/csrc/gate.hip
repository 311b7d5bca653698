// Gate front-end: scores -> int32 hot mask with ones at the k largest scores of every row.
//
// Replaces the three torch launches of the reference's TopKProtocol
// (python/brt/router/protocol/topk.py:26-31: torch.topk, zeros_like, scatter_) with one pass
// that reads the scores once and writes the mask once.  Order of torch.topk: NaN above every
// number; among equal scores (which torch leaves unspecified) the lowest column wins.
//
// Lanes are columns.  Up to 64 columns: a wavefront takes 64/ep rows per step (ep = columns
// rounded up to a power of two) and every selection is a butterfly max inside the row's lane
// segment plus a ballot that picks the lowest lane holding the maximum.  More than 64 columns:
// one row per step, every lane keeps the columns lane, lane+64, ... in registers.
//
// The compact form of the same pass writes, instead of (or beside) the dense mask, the k chosen
// columns of every row in the order of selection and their weights: the scores themselves, or
// their softmax over the row (fp32: exp(x - max) / sum, the front end of the Switch router,
// benchmark/switch_moe/switch_transformer.py:240-253, and of the Swin-MoE gate,
// python/brt/router/protocol/swin_moe.py:100-107).  k words per row instead of E.
#include <algorithm>

#include "common.hpp"

namespace brt {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxPerLane = 16;  // columns per lane in the wide path: up to 1024 columns

struct GateArgs {
  const void* scores;
  int* mask;       // [T, E] or null
  int* ids;        // [T, k] chosen columns in the order of selection (compact form only)
  float* weights;  // [T, k] or null
  int softmax;     // weights are the softmax of the row instead of the scores
  int T, E, k;
  int ep_shift;  // log2 of the lane segment of a row (E <= 64)
  int rows_pw;   // rows per wavefront
};

// Scores as unsigned keys whose order is torch.topk's: larger key = ranked higher, NaN on top.
// 0 is below every real key and marks a column that is taken (or does not exist).
__device__ __forceinline__ uint32_t score_key(float f) {
  if (f != f) return 0xffffffffu;
  const uint32_t u = f == 0.0f ? 0u : __float_as_uint(f);  // -0 and +0 are one score
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);       // never 0: ~u of a number is >= 0x007fffff
}

template <int DT>
__device__ __forceinline__ float load_score(const void* p, size_t i) {
  if (DT == BRT_F32) return static_cast<const float*>(p)[i];
  return half_bits_to_float<DT>(static_cast<const uint16_t*>(p)[i]);
}

__device__ __forceinline__ float segment_sum(float v, int width) {
  return segment_all_reduce(v, width, [](float x, float y) { return x + y; });
}
__device__ __forceinline__ float segment_max(float v, int width) {
  return segment_all_reduce(v, width, [](float x, float y) { return fmaxf(x, y); });
}
__device__ __forceinline__ uint32_t segment_max(uint32_t v, int width) {
  return static_cast<uint32_t>(segment_all_reduce(static_cast<int>(v), width, [](int x, int y) {
    return static_cast<int>(max(static_cast<uint32_t>(x), static_cast<uint32_t>(y)));
  }));
}
__device__ __forceinline__ int segment_min(int v, int width) {
  return segment_all_reduce(v, width, [](int x, int y) { return min(x, y); });
}

template <int DT, bool COMPACT>
__global__ __launch_bounds__(kBlock) void topk_mask_kernel(GateArgs a) {
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int ep = 1 << a.ep_shift, rps = kWave >> a.ep_shift;
  const int e = lane & (ep - 1), sub = lane >> a.ep_shift;
  const unsigned long long seg = (ep == kWave ? ~0ull : ((1ull << ep) - 1ull)) << (sub * ep);
  const long t0 = wave * a.rows_pw;
  const int nt = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - t0)));
  for (int r0 = 0; r0 < nt; r0 += rps) {
    const int row = r0 + sub;
    const bool live = row < nt && e < a.E;
    const float x = live ? load_score<DT>(a.scores, static_cast<size_t>(t0 + row) * a.E + e) : 0.0f;
    uint32_t key = live ? score_key(x) : 0u;
    float weight = x;
    if (COMPACT && a.softmax) {
      const float top = segment_max(live ? x : -INFINITY, ep);
      const float ex = live ? expf(x - top) : 0.0f;
      weight = ex / segment_sum(ex, ep);
    }
    int taken = 0;
    for (int pass = 0; pass < a.k; ++pass) {
      const uint32_t best = segment_max(key, ep);
      const unsigned long long tied = __ballot(key == best && key != 0) & seg;
      if (tied != 0 && lane == __builtin_ctzll(tied)) {
        taken = 1;
        key = 0;
        if (COMPACT) {
          const size_t slot = static_cast<size_t>(t0 + row) * a.k + pass;
          a.ids[slot] = e;
          if (a.weights) a.weights[slot] = weight;
        }
      }
    }
    if (live && (!COMPACT || a.mask)) a.mask[static_cast<size_t>(t0 + row) * a.E + e] = taken;
  }
}

template <int DT, bool COMPACT>
__global__ __launch_bounds__(kBlock) void topk_mask_wide_kernel(GateArgs a) {
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const long t0 = wave * a.rows_pw;
  const int nt = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - t0)));
  const int per_lane = (a.E + kWave - 1) / kWave;
  for (int row = 0; row < nt; ++row) {
    const size_t base = static_cast<size_t>(t0 + row) * a.E;
    uint32_t key[kMaxPerLane];
    float weight[kMaxPerLane];
    unsigned taken = 0;
#pragma unroll
    for (int c = 0; c < kMaxPerLane; ++c) {
      const int col = c * kWave + lane;
      const bool live = c < per_lane && col < a.E;
      weight[c] = live ? load_score<DT>(a.scores, base + col) : -INFINITY;
      key[c] = live ? score_key(weight[c]) : 0u;
    }
    if (COMPACT && a.softmax) {
      float top = -INFINITY;
#pragma unroll
      for (int c = 0; c < kMaxPerLane; ++c) top = fmaxf(top, weight[c]);
      top = segment_max(top, kWave);
      float sum = 0.0f;
#pragma unroll
      for (int c = 0; c < kMaxPerLane; ++c) {
        weight[c] = weight[c] == -INFINITY ? 0.0f : expf(weight[c] - top);
        sum += weight[c];
      }
      sum = segment_sum(sum, kWave);
#pragma unroll
      for (int c = 0; c < kMaxPerLane; ++c) weight[c] = weight[c] / sum;
    }
    for (int pass = 0; pass < a.k; ++pass) {
      uint32_t mine = 0;
#pragma unroll
      for (int c = 0; c < kMaxPerLane; ++c) mine = max(mine, key[c]);
      const uint32_t best = segment_max(mine, kWave);
      // lowest column holding the maximum: lowest c first, then lowest lane
      int my_c = kMaxPerLane;
#pragma unroll
      for (int c = kMaxPerLane - 1; c >= 0; --c)
        if (key[c] == best && best != 0) my_c = c;
      const int low_c = segment_min(my_c, kWave);
      const unsigned long long tied = __ballot(my_c == low_c && my_c < kMaxPerLane);
      if (tied != 0 && lane == __builtin_ctzll(tied)) {
#pragma unroll
        for (int c = 0; c < kMaxPerLane; ++c)
          if (c == low_c) {
            key[c] = 0;
            taken |= 1u << c;
            if (COMPACT) {
              const size_t slot = static_cast<size_t>(t0 + row) * a.k + pass;
              a.ids[slot] = c * kWave + lane;
              if (a.weights) a.weights[slot] = weight[c];
            }
          }
      }
    }
    if (!COMPACT || a.mask) {
#pragma unroll
      for (int c = 0; c < kMaxPerLane; ++c) {
        const int col = c * kWave + lane;
        if (c < per_lane && col < a.E) a.mask[base + col] = (taken >> c) & 1u;
      }
    }
  }
}

}  // namespace
}  // namespace brt

using namespace brt;

namespace {

int launch_gate(GateArgs a, int dtype, bool compact, void* stream) {
  const int T = a.T, E = a.E, k = a.k;
  if (T < 0 || E <= 0 || k < 0 || k > E) return fail(BRT_E_INVALID, "bad shape T=%d E=%d k=%d", T, E, k);
  if (dtype != BRT_F32 && dtype != BRT_F16 && dtype != BRT_BF16)
    return fail(BRT_E_UNSUPPORTED, "dtype %d is not supported", dtype);
  if (E > kWave * kMaxPerLane) return fail(BRT_E_UNSUPPORTED, "more than %d paths", kWave * kMaxPerLane);
  if (static_cast<long>(T) * E >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*E >= 2^31");
  if (T == 0) return BRT_OK;
  if (!a.scores || (compact ? (k > 0 && !a.ids) : !a.mask)) return fail(BRT_E_INVALID, "null argument");
  int shift = 0;
  while ((1 << shift) < std::min(E, kWave)) ++shift;
  a.ep_shift = shift;
  const int rps = E <= kWave ? kWave >> shift : 1;
  // about 8192 wavefronts (the chip a few times over), whole steps per wavefront: a wavefront's
  // steps run one after the other, each a full memory round trip
  long rows = ((T + 8191) / 8192 + rps - 1) / rps * rps;
  rows = std::min<long>(std::max<long>(rows, rps), 16l * rps);
  a.rows_pw = static_cast<int>(rows);
  const long n_waves = (T + a.rows_pw - 1) / a.rows_pw;
  const int waves_pb = kBlock / kWave;
  const dim3 grid(static_cast<unsigned>((n_waves + waves_pb - 1) / waves_pb)), block(kBlock);
  hipStream_t st = as_stream(stream);
#define BRT_GATE_KERNELS(DT, COMPACT)                                                          \
  if (E <= kWave) hipLaunchKernelGGL((topk_mask_kernel<DT, COMPACT>), grid, block, 0, st, a);  \
  else hipLaunchKernelGGL((topk_mask_wide_kernel<DT, COMPACT>), grid, block, 0, st, a);
#define BRT_GATE_LAUNCH(DT)                   \
  if (compact) { BRT_GATE_KERNELS(DT, true) } \
  else { BRT_GATE_KERNELS(DT, false) }
  if (dtype == BRT_F32) { BRT_GATE_LAUNCH(BRT_F32) }
  else if (dtype == BRT_F16) { BRT_GATE_LAUNCH(BRT_F16) }
  else { BRT_GATE_LAUNCH(BRT_BF16) }
#undef BRT_GATE_LAUNCH
#undef BRT_GATE_KERNELS
  return check_launch("topk_mask_kernel");
}

}  // namespace

extern "C" int brt_hip_topk_hot_mask(const void* scores, int32_t* hot_mask, int T, int E, int k,
                                     int dtype, void* stream) {
  GateArgs a{};
  a.scores = scores; a.mask = hot_mask; a.T = T; a.E = E; a.k = k;
  return launch_gate(a, dtype, false, stream);
}

extern "C" int brt_hip_gate_topk(const void* scores, int T, int E, int k, int dtype, int softmax,
                                 int32_t* path_ids, float* weights, int32_t* hot_mask, void* stream) {
  GateArgs a{};
  a.scores = scores; a.mask = hot_mask; a.ids = path_ids; a.weights = weights;
  a.softmax = softmax; a.T = T; a.E = E; a.k = k;
  return launch_gate(a, dtype, true, stream);
}
