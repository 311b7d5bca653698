// Routing on the compact route format: k path ids per cell instead of a dense [T, E] mask.
//
// The reference carries a route as an int32 hot mask of T x E words from the protocol to the
// fabric (python/brt/router/protocol/topk.py:26-31 builds it, src/router/location.cu:212-257
// scans it, src/router/route.cu:13-282 reads the T x E seat matrix again in dispatch and in
// combine).  With k chosen paths per cell the same information is T x k words:
//
//   path_ids   [T, k]  the paths of a cell (all different, any order; an id outside [0, E) is
//                      no route)
//   seat_rows  [T, k]  1-based row of the dispatched buffer that entry (t, j) is copied to,
//                      0 when the entry was dropped (no route, or past the path's load)
//   row_entries[P]     the inverse: 1-based entry number t*k + j + 1 of every dispatched row,
//                      0 for padding rows
//
// route_by_path computes loads, seat_rows and row_entries with the reference's rules: seats in
// ascending cell order per path, loads from the real counts through the capacity menu
// (location.cu:227-254), rows of path e start at the sum of the loads before it or at
// e * max_path_load.  dispatch_by_rows and combine_by_rows move the rows; their results are
// bit-identical to dispatch / combine on the dense seat matrix of the same route.
#include <algorithm>

#include "rows.hpp"

namespace brt {
namespace {

constexpr int kBlock = 256;
constexpr int kRouteWaves = 16;  // one workgroup of 16 wavefronts computes a whole route
constexpr int kRouteBlock = kRouteWaves * kWave;
constexpr int kBatch = 8;        // chunks of 64 entries a wavefront keeps in flight
constexpr int kMaxK = 8;         // paths per cell in combine_by_rows
constexpr int kMaxRoutePaths = 512;  // (kRouteWaves + 3) * E words of LDS

struct RouteArgs {
  const int* ids;
  const int* caps;
  int* loads;
  int* counts;
  int* seat_rows;
  int* row_entries;
  int n, E, C, P, bits, per_wave;
  int capacity_padding, path_wise_padding, max_path_load;
};

// Lanes of the wavefront that hold the same path id as this lane (`bits` low bits compared).
__device__ __forceinline__ unsigned long long same_path_lanes(int e, bool valid, int bits) {
  unsigned long long m = __ballot(valid);
  for (int b = 0; b < bits; ++b) {
    const bool set = (e >> b) & 1;
    const unsigned long long with = __ballot(set);
    m &= set ? with : ~with;
  }
  return m;
}

__device__ __forceinline__ unsigned long long lanes_below(int lane) { return (1ull << lane) - 1ull; }

// One workgroup.  Wavefront w owns the entries [w * per_wave, (w+1) * per_wave), in chunks of 64
// (one entry per lane).  Pass 1 counts entries per (wavefront, path) in LDS: the lanes of a chunk
// that hold the same path are found with one ballot per id bit, and the lowest of them adds their
// number to the wavefront's counter -- no atomics, every counter has one writer.  A column scan
// over the 16 wavefronts turns the counters into each wavefront's first seat per path and gives
// the real count of every path, from which the loads and the first row of every path follow.
// Pass 2 walks the entries again: seat = wavefront's running count + rank among the lanes of the
// chunk with the same path.
__global__ __launch_bounds__(kRouteBlock) void route_by_path_kernel(RouteArgs a) {
  extern __shared__ int lds[];
  const int E = a.E;
  int* s_base = lds;                     // [kRouteWaves][E]
  int* s_load = lds + kRouteWaves * E;   // [E]
  int* s_start = s_load + E;             // [E]
  int* s_kept = s_start + E;             // [E] rows a path really fills
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < kRouteWaves * E; i += kRouteBlock) s_base[i] = 0;
  __syncthreads();

  const int lo = min(a.n, w * a.per_wave), hi = min(a.n, lo + a.per_wave);
  int* mine = s_base + w * E;

  for (int c0 = lo; c0 < hi; c0 += kWave * kBatch) {
    int id[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int i = c0 + b * kWave + lane;
      id[b] = i < hi ? a.ids[i] : -1;
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      if (c0 + b * kWave < hi) {  // same for the whole wavefront
        const int e = id[b];
        const bool valid = e >= 0 && e < E;
        const unsigned long long same = same_path_lanes(e, valid, a.bits);
        if (valid && (same & lanes_below(lane)) == 0) mine[e] += __popcll(same);
      }
    }
  }
  __syncthreads();

  for (int e = threadIdx.x; e < E; e += kRouteBlock) {
    int run = 0;
    for (int v = 0; v < kRouteWaves; ++v) {
      const int c = s_base[v * E + e];
      s_base[v * E + e] = run;
      run += c;
    }
    const int load = finalize_load(run, a.caps, a.C, a.capacity_padding, a.path_wise_padding, e);
    s_load[e] = load;
    s_kept[e] = min(run, a.max_path_load != 0 ? min(load, a.max_path_load) : load);
    a.loads[e] = load;
    if (a.counts) a.counts[e] = run;
  }
  __syncthreads();
  if (w == 0) {  // first row of every path
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += kWave) {
      const int e = e0 + lane;
      const int v = e < E ? s_load[e] : 0;
      const int incl = wave_inclusive_scan(v);
      if (e < E) s_start[e] = a.max_path_load != 0 ? e * a.max_path_load : carry + incl - v;
      carry += __shfl(incl, kWave - 1, kWave);
    }
  }
  __syncthreads();

  for (int c0 = lo; c0 < hi; c0 += kWave * kBatch) {
    int id[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int i = c0 + b * kWave + lane;
      id[b] = i < hi ? a.ids[i] : -1;
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      if (c0 + b * kWave < hi) {
        const int i = c0 + b * kWave + lane;
        const int e = id[b];
        const bool valid = e >= 0 && e < E;
        const unsigned long long same = same_path_lanes(e, valid, a.bits);
        const int rank = __popcll(same & lanes_below(lane));
        const int before = valid ? mine[e] : 0;  // read by every lane before the first of them updates it
        if (valid && rank == 0) mine[e] = before + __popcll(same);
        const int seat = before + rank + 1;
        int row = 0;
        if (valid && seat <= s_kept[e]) row = s_start[e] + seat;
        if (row > a.P) row = 0;
        if (i < hi) a.seat_rows[i] = row;
        if (row != 0) a.row_entries[row - 1] = i + 1;
      }
    }
  }

  // padding rows: between the rows a path filled and the first row of the next path, and
  // behind the last path
  for (int e = w; e < E; e += kRouteWaves) {
    const int first = s_start[e] + s_kept[e];
    const int end = min(a.P, a.max_path_load != 0 ? s_start[e] + a.max_path_load : s_start[e] + s_load[e]);
    for (int r = first + lane; r < end; r += kWave) a.row_entries[r] = 0;
  }
  const int total = a.max_path_load != 0 ? E * a.max_path_load : s_start[E - 1] + s_load[E - 1];
  for (int r = total + threadIdx.x; r < a.P; r += kRouteBlock) a.row_entries[r] = 0;
}

// ---------------------------------------------------------------- rows by entry
struct RowsArgs {
  const void* src;
  void* dst;
  const float* weights;   // [T, k] or null
  const int* row_entries; // dispatch: [P]
  const int* ids;         // combine: [T, k]
  const int* seat_rows;   // combine: [T, k]
  int T, P, k, cpr, rows_pw, is_residual;
};

// dst[r] = src[cell of entry row_entries[r]] (times the entry's weight, one rounding), zeros for
// padding rows.  A group of 1 << LS lanes per row, UPR 16-byte units per lane and step.
template <int DT, int LS, int UPR>
__global__ __launch_bounds__(kBlock) void dispatch_by_rows_kernel(RowsArgs a) {
  using U = u32x4;
  constexpr int NE = 16 / elem_bytes(DT);
  constexpr int LPR = 1 << LS;
  constexpr int GROUPS = kWave >> LS;
  constexpr bool kStream = LS >= 4;  // rows of more than 128 bytes are not read again here
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int gidx = lane >> LS, glane = lane & (LPR - 1);
  const long p0 = wave * a.rows_pw;
  const int np = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.P - p0)));
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  U* __restrict__ dst = static_cast<U*>(a.dst);
  const int n = a.T * a.k;
  for (int rb = 0; rb < np; rb += GROUPS) {
    const int i = rb + gidx;
    const bool live = i < np;
    int entry = live ? a.row_entries[p0 + i] : 0;
    if (entry < 0 || entry > n) entry = 0;
    const bool filled = entry != 0;
    const int cell = filled ? (entry - 1) / a.k : 0;
    const float g = (filled && a.weights) ? a.weights[entry - 1] : 1.0f;
    const size_t from = static_cast<size_t>(cell) * cpr, to = static_cast<size_t>(p0 + i) * cpr;
    for (int off0 = 0; off0 < cpr; off0 += LPR * UPR) {
      U val[UPR];
#pragma unroll
      for (int u = 0; u < UPR; ++u) {
        const int off = off0 + u * LPR + glane;
        val[u] = zero_unit<16>();
        if (filled && off < cpr) val[u] = src[from + off];
      }
#pragma unroll
      for (int u = 0; u < UPR; ++u) {
        const int off = off0 + u * LPR + glane;
        if (live && off < cpr) {
          if (a.weights != nullptr && filled) {
            float x[NE];
            unpack<DT, 16>(val[u], x);
#pragma unroll
            for (int q = 0; q < NE; ++q) x[q] = x[q] * g;
            pack_store<DT, NE, kStream>(dst + to + off, x);
          } else {
            store_unit<kStream>(dst + to + off, val[u]);
          }
        }
      }
    }
  }
}

// dst[t] = sum over the entries of cell t that own a row, in ascending path order, of
// weight * src[row] (fp32, product and sum rounded separately, starting from 0): the order and
// the roundings of the dense combine.  Cells without a row keep dst (is_residual) or get zeros.
template <int IN_DT, int OUT_DT, int LS, int UPR>
__global__ __launch_bounds__(kBlock) void combine_by_rows_kernel(RowsArgs a) {
  using U = u32x4;
  constexpr int NE = 16 / elem_bytes(IN_DT);
  constexpr int OUT_BYTES = NE * elem_bytes(OUT_DT);
  constexpr int LPR = 1 << LS;
  constexpr int GROUPS = kWave >> LS;
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int gidx = lane >> LS, glane = lane & (LPR - 1);
  const long t0 = wave * a.rows_pw;
  const int nt = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - t0)));
  const int cpr = a.cpr, k = a.k;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  char* __restrict__ dst = static_cast<char*>(a.dst);
  for (int tb = 0; tb < nt; tb += GROUPS) {
    const int i = tb + gidx;
    const bool live = i < nt;
    const size_t slot0 = static_cast<size_t>(t0 + i) * k;
    int id[kMaxK], row[kMaxK];
    float g[kMaxK];
    int owned = 0;
#pragma unroll
    for (int j = 0; j < kMaxK; ++j) {
      const bool has = live && j < k;
      row[j] = has ? a.seat_rows[slot0 + j] : 0;
      if (row[j] < 0 || row[j] > a.P) row[j] = 0;
      id[j] = row[j] != 0 ? a.ids[slot0 + j] : 0x7fffffff;
      g[j] = (row[j] != 0 && a.weights) ? a.weights[slot0 + j] : 1.0f;
      owned += row[j] != 0;
    }
    const size_t to = static_cast<size_t>(t0 + i) * cpr;
    for (int off0 = 0; off0 < cpr; off0 += LPR * UPR) {
      float acc[UPR][NE];
#pragma unroll
      for (int u = 0; u < UPR; ++u)
#pragma unroll
        for (int q = 0; q < NE; ++q) acc[u][q] = 0.0f;
      int last = -1;
      for (int pass = 0; pass < owned; ++pass) {
        // the entry with the lowest path id above the last one taken
        int best = 0x7fffffff, sr = 0;
        float gg = 1.0f;
#pragma unroll
        for (int j = 0; j < kMaxK; ++j) {
          const bool better = id[j] > last && id[j] < best;
          best = better ? id[j] : best;
          sr = better ? row[j] : sr;
          gg = better ? g[j] : gg;
        }
        const bool has = best != 0x7fffffff;  // false only for a cell that names a path twice
        last = best;
        U val[UPR];
#pragma unroll
        for (int u = 0; u < UPR; ++u) {
          const int off = off0 + u * LPR + glane;
          if (has && off < cpr) val[u] = src[static_cast<size_t>(sr - 1) * cpr + off];
        }
#pragma unroll
        for (int u = 0; u < UPR; ++u) {
          const int off = off0 + u * LPR + glane;
          if (has && off < cpr) {
            float x[NE];
            unpack<IN_DT, 16>(val[u], x);
#pragma unroll
            for (int q = 0; q < NE; ++q) acc[u][q] = acc[u][q] + x[q] * gg;
          }
        }
      }
      if (live && (owned != 0 || !a.is_residual)) {
#pragma unroll
        for (int u = 0; u < UPR; ++u) {
          const int off = off0 + u * LPR + glane;
          if (off < cpr) pack_store<OUT_DT, NE, IN_DT == OUT_DT && LS >= 4>(dst + (to + off) * OUT_BYTES, acc[u]);
        }
      }
    }
  }
}

int rows_per_wavefront(int cpr, long rows) {
  int r = std::max(1, 384 / cpr);
  while (r > 1 && (rows + r - 1) / r < 4096) r >>= 1;
  return r;
}

}  // namespace
}  // namespace brt

using namespace brt;

extern "C" int brt_hip_route_by_path(const int32_t* path_ids, int T, int k, int E, const int32_t* caps,
                                     int C, int capacity_padding, int path_wise_padding,
                                     int max_path_load, int32_t* loads, int32_t* counts,
                                     int32_t* seat_rows, int32_t* row_entries, int P, void* stream) {
  if (T < 0 || k < 0 || E <= 0 || P < 0 || max_path_load < 0)
    return fail(BRT_E_INVALID, "bad shape T=%d k=%d E=%d P=%d", T, k, E, P);
  if (E > kMaxRoutePaths) return fail(BRT_E_UNSUPPORTED, "more than %d paths", kMaxRoutePaths);
  if (static_cast<long>(T) * k >= (1l << 24))
    return fail(BRT_E_UNSUPPORTED, "T*k = %ld: the single-workgroup route is limited to 2^24 entries",
                static_cast<long>(T) * k);
  if (caps == nullptr) C = 0;
  if (capacity_padding && C < 1)
    return fail(BRT_E_INVALID, "capacity_padding needs at least one supported capacity");
  if (!capacity_padding) path_wise_padding = 0;
  if (path_wise_padding && C < E)
    return fail(BRT_E_INVALID, "path_wise_padding needs one capacity per path (%d < %d)", C, E);
  if (max_path_load != 0 && static_cast<long>(E) * max_path_load >= (1l << 31))
    return fail(BRT_E_UNSUPPORTED, "E * max_path_load >= 2^31");
  const int n = T * k;
  if (!loads || (n > 0 && (!path_ids || !seat_rows)) || (P > 0 && !row_entries))
    return fail(BRT_E_INVALID, "null argument");
  RouteArgs a{};
  a.ids = path_ids; a.caps = caps; a.loads = loads; a.counts = counts;
  a.seat_rows = seat_rows; a.row_entries = row_entries;
  a.n = n; a.E = E; a.C = C; a.P = P;
  a.capacity_padding = capacity_padding; a.path_wise_padding = path_wise_padding;
  a.max_path_load = max_path_load;
  while ((1 << a.bits) < E) ++a.bits;
  const int chunks = (n + kWave - 1) / kWave;
  a.per_wave = (chunks + kRouteWaves - 1) / kRouteWaves * kWave;
  const size_t lds_bytes = static_cast<size_t>(kRouteWaves + 3) * E * sizeof(int);
  hipLaunchKernelGGL(route_by_path_kernel, dim3(1), dim3(kRouteBlock), lds_bytes, as_stream(stream), a);
  return check_launch("route_by_path_kernel");
}

namespace {

// Lane-group shape by row length, as in the dense kernels.
template <typename F>
void with_row_shape(int cpr, F&& launch) {
  using std::integral_constant;
  if (cpr > 2 * kWave) launch(integral_constant<int, 6>{}, integral_constant<int, 4>{});
  else if (cpr > kWave) launch(integral_constant<int, 6>{}, integral_constant<int, 2>{});
  else if (cpr > 32) launch(integral_constant<int, 6>{}, integral_constant<int, 1>{});
  else if (cpr > 16) launch(integral_constant<int, 5>{}, integral_constant<int, 1>{});
  else if (cpr > 8) launch(integral_constant<int, 4>{}, integral_constant<int, 1>{});
  else if (cpr > 4) launch(integral_constant<int, 3>{}, integral_constant<int, 1>{});
  else launch(integral_constant<int, 2>{}, integral_constant<int, 1>{});
}

}  // namespace

extern "C" int brt_hip_dispatch_by_rows(const void* src, void* dst, const float* weights,
                                        const int32_t* row_entries, int P, int T, int k, int cell,
                                        int dtype, void* stream) {
  if (T < 0 || k <= 0 || cell < 0 || P < 0) return fail(BRT_E_INVALID, "bad shape T=%d k=%d cell=%d P=%d", T, k, cell, P);
  if (dtype != BRT_F32 && dtype != BRT_F16 && dtype != BRT_BF16)
    return fail(BRT_E_UNSUPPORTED, "dtype %d is not supported", dtype);
  if (static_cast<long>(T) * k >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*k >= 2^31");
  if (P == 0 || cell == 0) return BRT_OK;
  if (!dst || !row_entries || (T > 0 && !src)) return fail(BRT_E_INVALID, "null argument");
  const size_t row_bytes = static_cast<size_t>(cell) * elem_bytes(dtype);
  if (row_bytes % 16 != 0 || !aligned(src, 16) || !aligned(dst, 16))
    return fail(BRT_E_UNSUPPORTED, "rows must be whole 16-byte units (row is %zu bytes)", row_bytes);
  RowsArgs a{};
  a.src = src; a.dst = dst; a.weights = weights; a.row_entries = row_entries;
  a.T = T; a.P = P; a.k = k;
  a.cpr = static_cast<int>(row_bytes / 16);
  a.rows_pw = rows_per_wavefront(a.cpr, P);
  const long n_waves = (static_cast<long>(P) + a.rows_pw - 1) / a.rows_pw;
  const int waves_pb = kBlock / kWave;
  const dim3 grid(static_cast<unsigned>((n_waves + waves_pb - 1) / waves_pb)), block(kBlock);
  hipStream_t st = as_stream(stream);
#define BRT_LAUNCH(DT)                                                                              \
  with_row_shape(a.cpr, [&](auto ls, auto upr) {                                                    \
    hipLaunchKernelGGL((dispatch_by_rows_kernel<DT, decltype(ls)::value, decltype(upr)::value>),    \
                       grid, block, 0, st, a);                                                      \
  });
  if (dtype == BRT_F32) BRT_LAUNCH(BRT_F32)
  else if (dtype == BRT_F16) BRT_LAUNCH(BRT_F16)
  else BRT_LAUNCH(BRT_BF16)
#undef BRT_LAUNCH
  return check_launch("dispatch_by_rows_kernel");
}

extern "C" int brt_hip_combine_by_rows(const void* src, void* dst, const float* weights,
                                       const int32_t* path_ids, const int32_t* seat_rows, int T,
                                       int k, int cell, int P, int is_residual, int in_dtype,
                                       int out_dtype, void* stream) {
  if (T < 0 || k <= 0 || cell < 0 || P < 0) return fail(BRT_E_INVALID, "bad shape T=%d k=%d cell=%d P=%d", T, k, cell, P);
  if (k > kMaxK) return fail(BRT_E_UNSUPPORTED, "more than %d paths per cell", kMaxK);
  if ((in_dtype != BRT_F32 && in_dtype != BRT_F16 && in_dtype != BRT_BF16) ||
      (out_dtype != in_dtype && out_dtype != BRT_F32))
    return fail(BRT_E_UNSUPPORTED, "dtype pair %d -> %d is not supported", in_dtype, out_dtype);
  if (static_cast<long>(T) * k >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*k >= 2^31");
  if (T == 0 || cell == 0) return BRT_OK;
  if (!dst || !path_ids || !seat_rows || (P > 0 && !src)) return fail(BRT_E_INVALID, "null argument");
  const size_t row_bytes = static_cast<size_t>(cell) * elem_bytes(in_dtype);
  if (row_bytes % 16 != 0 || !aligned(src ? src : dst, 16) || !aligned(dst, 16))
    return fail(BRT_E_UNSUPPORTED, "rows must be whole 16-byte units (row is %zu bytes)", row_bytes);
  RowsArgs a{};
  a.src = src; a.dst = dst; a.weights = weights; a.ids = path_ids; a.seat_rows = seat_rows;
  a.T = T; a.P = P; a.k = k; a.is_residual = is_residual;
  a.cpr = static_cast<int>(row_bytes / 16);
  a.rows_pw = rows_per_wavefront(a.cpr, T);
  const long n_waves = (static_cast<long>(T) + a.rows_pw - 1) / a.rows_pw;
  const int waves_pb = kBlock / kWave;
  const dim3 grid(static_cast<unsigned>((n_waves + waves_pb - 1) / waves_pb)), block(kBlock);
  hipStream_t st = as_stream(stream);
#define BRT_LAUNCH(IN, OUT)                                                                              \
  with_row_shape(a.cpr, [&](auto ls, auto upr) {                                                         \
    hipLaunchKernelGGL((combine_by_rows_kernel<IN, OUT, decltype(ls)::value, decltype(upr)::value>),     \
                       grid, block, 0, st, a);                                                           \
  });
  if (in_dtype == BRT_F32) BRT_LAUNCH(BRT_F32, BRT_F32)
  else if (in_dtype == BRT_F16 && out_dtype == BRT_F16) BRT_LAUNCH(BRT_F16, BRT_F16)
  else if (in_dtype == BRT_F16) BRT_LAUNCH(BRT_F16, BRT_F32)
  else if (out_dtype == BRT_BF16) BRT_LAUNCH(BRT_BF16, BRT_BF16)
  else BRT_LAUNCH(BRT_BF16, BRT_F32)
#undef BRT_LAUNCH
  return check_launch("combine_by_rows_kernel");
}
