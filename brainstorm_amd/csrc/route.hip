// Dispatch (token rows -> path-major buffer) and combine (path-major buffer ->
// token rows, gate-weighted fp32 accumulation).
//
// Semantics follow src/router/route.cu of the reference
// (dispatch_with_{seat,tag}_indices_{1d,2d} :13-206, combine_with_seat_indices
// :208-248, init_with_seat_indices :250-282).  The reference launches a
// (512, E) grid in which every row of blocks re-reads the whole index matrix,
// copies rows with scalar loads, recomputes the path start offsets per thread,
// needs a separate zero-fill pass over the output and accumulates the combine
// with atomicAdd.  Here one block owns a few rows of the index matrix, reads
// them once (coalesced), turns them into a short work list in LDS and then moves
// whole rows with 128-bit accesses; padding rows are zero-filled by the same
// launch and the combine is a gather with register accumulation, so every byte
// of the output is written exactly once.
#include <algorithm>
#include <cstdlib>

#include "common.hpp"

namespace brt {
namespace {

constexpr int kBlock = 256;
constexpr int kUnroll = 4;

template <int BYTES> struct Unit;
template <> struct Unit<16> { using type = uint4; };
template <> struct Unit<8> { using type = uint2; };
template <> struct Unit<4> { using type = uint32_t; };
template <> struct Unit<2> { using type = uint16_t; };

constexpr int elem_bytes(int dt) { return dt == BRT_F32 ? 4 : 2; }

// Unpacks BYTES of DT elements to fp32.
template <int DT, int BYTES>
__device__ __forceinline__ void unpack(const typename Unit<BYTES>::type& v,
                                       float (&x)[BYTES / elem_bytes(DT)]) {
  if constexpr (BYTES == 2) {
    x[0] = half_bits_to_float<DT>(v);
  } else {
    const uint32_t* w = reinterpret_cast<const uint32_t*>(&v);
#pragma unroll
    for (int i = 0; i < BYTES / 4; ++i) {
      if constexpr (DT == BRT_F32) {
        x[i] = __uint_as_float(w[i]);
      } else {
        x[2 * i] = half_bits_to_float<DT>(w[i] & 0xffffu);
        x[2 * i + 1] = half_bits_to_float<DT>(w[i] >> 16);
      }
    }
  }
}

// Packs N fp32 values to DT (round to nearest even) and stores them at p.
template <int DT, int N>
__device__ __forceinline__ void pack_store(void* p, const float (&x)[N]) {
  if constexpr (DT == BRT_F32) {
    if constexpr (N % 4 == 0) {
#pragma unroll
      for (int i = 0; i < N / 4; ++i)
        static_cast<float4*>(p)[i] = make_float4(x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]);
    } else if constexpr (N == 2) {
      *static_cast<float2*>(p) = make_float2(x[0], x[1]);
    } else {
      *static_cast<float*>(p) = x[0];
    }
  } else {
    if constexpr (N == 1) {
      *static_cast<uint16_t*>(p) = static_cast<uint16_t>(float_to_half_bits<DT>(x[0]));
    } else {
      uint32_t w[N / 2];
#pragma unroll
      for (int i = 0; i < N / 2; ++i)
        w[i] = float_to_half_bits<DT>(x[2 * i]) | (float_to_half_bits<DT>(x[2 * i + 1]) << 16);
      if constexpr (N == 8) {
        *static_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
      } else if constexpr (N == 4) {
        *static_cast<uint2*>(p) = make_uint2(w[0], w[1]);
      } else {
        *static_cast<uint32_t*>(p) = w[0];
      }
    }
  }
}

template <int BYTES>
__device__ __forceinline__ typename Unit<BYTES>::type zero_unit() {
  if constexpr (BYTES == 16) return make_uint4(0, 0, 0, 0);
  else if constexpr (BYTES == 8) return make_uint2(0, 0);
  else return 0;
}

// ---------------------------------------------------------------- dispatch
struct DispatchArgs {
  const void* src;
  void* dst;
  const void* gates;
  const int* idx;
  const int* loads;
  const int* counts;
  const int* old_tags;
  int* new_tags;
  int T, E, P, mpl;
  int cpr;       // units (BYTES each) per row
  int rows_pb;   // rows of the index matrix per block
  int list_cap;  // work-list capacity (>= rows_pb * E)
  int is_1d, is_tag_index;
};

// DT < 0: unweighted byte copy; otherwise rows are scaled by the gate in DT.
template <int BYTES, int DT>
__global__ __launch_bounds__(kBlock) void dispatch_kernel(DispatchArgs a) {
  using U = typename Unit<BYTES>::type;
  extern __shared__ int smem[];
  const int E = a.E;
  int* s_loads = smem;
  int* s_start = smem + E;
  int* s_zstart = smem + 2 * E;  // E + 1 entries: padding rows before path e
  int* s_dst = s_zstart + E + 1;
  int* s_src = s_dst + a.list_cap;
  float* s_gate = reinterpret_cast<float*>(s_src + a.list_cap);
  __shared__ int s_n;

  const int tid = threadIdx.x;
  if (tid == 0) s_n = 0;
  load_and_scan_paths(a.loads, s_loads, s_start, E, a.mpl);
  if (a.counts != nullptr && tid < kWave) {
    int carry = 0;
    for (int base = 0; base < E; base += kWave) {
      const int e = base + tid;
      int z = 0;
      if (e < E) {
        const int load = a.loads[e];
        const int alloc = a.mpl != 0 ? a.mpl : load;
        const int filled = max(0, min(min(a.counts[e], load), alloc));
        z = max(0, alloc - filled);
      }
      const int incl = wave_inclusive_scan(z);
      if (e < E) s_zstart[e] = carry + incl - z;
      carry += __shfl(incl, kWave - 1, kWave);
    }
    if (tid == 0) s_zstart[E] = carry;
  }
  __syncthreads();

  // ---- 1. index rows -> work list (destination row, source row, gate) --------
  const int r0 = blockIdx.x * a.rows_pb;
  const int nr = max(0, min(a.rows_pb, a.T - r0));
  const int* idx0 = a.idx + static_cast<size_t>(r0) * E;
  for (int i = tid; i < nr * E; i += kBlock) {
    const int rl = i / E, e = i - rl * E;
    const int r = r0 + rl;
    const int v = idx0[i];
    bool ok;
    int dst_row, tok;
    if (!a.is_tag_index) {  // v = seat of token r on path e
      ok = v >= 1 && v <= s_loads[e];
      dst_row = s_start[e] + v - 1;
      tok = r;
    } else {  // v = 1-based token held by slot r of path e
      ok = r < s_loads[e] && v >= 1 && v <= a.T;
      dst_row = s_start[e] + r;
      tok = v - 1;
      // the reference walks slots r, r+512, ... per block and stops at the first
      // empty one (route.cu:84-92): an empty slot above in that chain hides r
      if (ok)
        for (int k = r - 512; k >= 0; k -= 512)
          if (a.idx[static_cast<size_t>(k) * E + e] == 0) {
            ok = false;
            break;
          }
    }
    ok = ok && dst_row >= 0 && dst_row < a.P;
    if (ok) {
      const int pos = atomicAdd(&s_n, 1);
      s_dst[pos] = dst_row;
      s_src[pos] = a.is_1d ? tok : tok * E + e;
      if constexpr (DT >= 0) s_gate[pos] = load_gate(a.gates, DT, static_cast<size_t>(tok) * E + e);
      if (a.new_tags != nullptr) a.new_tags[dst_row] = a.old_tags ? a.old_tags[tok] : tok + 1;
    }
  }
  __syncthreads();

  // ---- 2. move rows: flat loop over (entry, unit) pairs -----------------------
  const int n = s_n;
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  U* __restrict__ dst = static_cast<U*>(a.dst);
  int ent = tid / cpr, off = tid - ent * cpr;
  const int d_ent = kBlock / cpr, d_off = kBlock - d_ent * cpr;
  while (ent < n) {
    U v[kUnroll];
    size_t to[kUnroll];
    float g[kUnroll];
    bool live[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      live[u] = ent < n;
      if (live[u]) {
        v[u] = src[static_cast<size_t>(s_src[ent]) * cpr + off];
        to[u] = static_cast<size_t>(s_dst[ent]) * cpr + off;
        if constexpr (DT >= 0) g[u] = s_gate[ent];
      }
      ent += d_ent;
      off += d_off;
      if (off >= cpr) {
        off -= cpr;
        ++ent;
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (live[u]) {
        if constexpr (DT >= 0) {
          constexpr int NE = BYTES / elem_bytes(DT);
          float x[NE];
          unpack<DT, BYTES>(v[u], x);
#pragma unroll
          for (int i = 0; i < NE; ++i) x[i] = x[i] * g[u];
          pack_store<DT, NE>(dst + to[u], x);
        } else {
          dst[to[u]] = v[u];
        }
      }
    }
  }

  // ---- 3. zero-fill this block's share of the padding rows ---------------------
  if (a.counts != nullptr) {
    const long Z = s_zstart[E];
    const long z0 = Z * blockIdx.x / gridDim.x;
    const long z1 = Z * (blockIdx.x + 1) / gridDim.x;
    const int wave = tid >> 6, lane = tid & (kWave - 1);
    for (long z = z0 + wave; z < z1; z += kBlock / kWave) {
      int lo = 0, hi = E;  // largest e with s_zstart[e] <= z
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_zstart[mid] <= z) lo = mid; else hi = mid;
      }
      const int e = lo;
      const int pad = s_zstart[e + 1] - s_zstart[e];
      const int alloc = a.mpl != 0 ? a.mpl : s_loads[e];
      const long row = static_cast<long>(s_start[e]) + (alloc - pad) + (z - s_zstart[e]);
      if (row < a.P) {
        for (int o = lane; o < cpr; o += kWave) dst[static_cast<size_t>(row) * cpr + o] = zero_unit<BYTES>();
        if (a.new_tags != nullptr && lane == 0) a.new_tags[row] = 0;
      }
    }
  }
}

// ----------------------------------------------------------------- combine
struct CombineArgs {
  const void* src;
  void* dst;
  const void* gates;
  const int* idx;
  const int* loads;
  int T, E, P, mpl;
  int cpr;      // input units per row
  int rows_pb;  // tokens per block
  int ep_shift; // log2 of E rounded up to a power of two (E <= 64 only)
  int is_residual, gate_dtype;
};

template <int BYTES, int IN_DT, int OUT_DT>
__global__ __launch_bounds__(kBlock) void combine_kernel(CombineArgs a) {
  using U = typename Unit<BYTES>::type;
  constexpr int NE = BYTES / elem_bytes(IN_DT);
  constexpr int OUT_BYTES = NE * elem_bytes(OUT_DT);
  extern __shared__ int smem[];
  const int E = a.E;
  int* s_loads = smem;
  int* s_start = smem + E;
  int* s_cnt = smem + 2 * E;         // valid routes per token
  int* s_row = s_cnt + a.rows_pb;    // [rows_pb][E] source rows, ascending path order
  float* s_gate = reinterpret_cast<float*>(s_row + a.rows_pb * E);

  const int tid = threadIdx.x;
  load_and_scan_paths(a.loads, s_loads, s_start, E, a.mpl);
  __syncthreads();

  // ---- 1. per token: ordered list of valid (source row, gate) ------------------
  // lanes = paths, __ballot + popcount compacts the valid ones in ascending order
  const int t0 = blockIdx.x * a.rows_pb;
  const int nt = min(a.rows_pb, a.T - t0);
  const int wave = tid >> 6, lane = tid & (kWave - 1);
  const unsigned long long lt = (1ull << lane) - 1ull;
  if (E <= kWave) {
    const int ep = 1 << a.ep_shift;  // lanes per token
    const int tpw = kWave >> a.ep_shift;
    const int sub = lane >> a.ep_shift, e = lane & (ep - 1);
    const unsigned long long seg =
        ep == kWave ? ~0ull : (((1ull << ep) - 1ull) << (sub * ep));
    for (int base = wave * tpw; base < nt; base += (kBlock / kWave) * tpw) {
      const int tl = base + sub;
      bool ok = false;
      int row = 0;
      size_t gi = 0;
      if (tl < nt && e < E) {
        gi = static_cast<size_t>(t0 + tl) * E + e;
        const int seat = a.idx[gi];
        row = s_start[e] + seat - 1;
        ok = seat >= 1 && seat <= s_loads[e] && row < a.P;
      }
      const unsigned long long m = __ballot(ok) & seg;
      if (ok) {
        const int pos = __popcll(m & lt);
        s_row[tl * E + pos] = row;
        s_gate[tl * E + pos] = a.gates ? load_gate(a.gates, a.gate_dtype, gi) : 1.0f;
      }
      if (e == 0 && tl < nt) s_cnt[tl] = __popcll(m);
    }
  } else {
    for (int tl = wave; tl < nt; tl += kBlock / kWave) {
      int base = 0;
      for (int e0 = 0; e0 < E; e0 += kWave) {
        const int e = e0 + lane;
        bool ok = false;
        int row = 0;
        size_t gi = 0;
        if (e < E) {
          gi = static_cast<size_t>(t0 + tl) * E + e;
          const int seat = a.idx[gi];
          row = s_start[e] + seat - 1;
          ok = seat >= 1 && seat <= s_loads[e] && row < a.P;
        }
        const unsigned long long m = __ballot(ok);
        if (ok) {
          const int pos = base + __popcll(m & lt);
          s_row[tl * E + pos] = row;
          s_gate[tl * E + pos] = a.gates ? load_gate(a.gates, a.gate_dtype, gi) : 1.0f;
        }
        base += __popcll(m);
      }
      if (lane == 0) s_cnt[tl] = base;
    }
  }
  __syncthreads();

  // ---- 2. gather + fp32 accumulate, flat loop over (token, unit) pairs -----------
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  char* __restrict__ dst = static_cast<char*>(a.dst);
  int tl = tid / cpr, off = tid - tl * cpr;
  const int d_tl = kBlock / cpr, d_off = kBlock - d_tl * cpr;
  while (tl < nt) {
    float acc[kUnroll][NE];
    int n[kUnroll], tok[kUnroll], o[kUnroll];
    int nmax = 0;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      tok[u] = tl;
      o[u] = off;
      n[u] = tl < nt ? s_cnt[tl] : -1;
      nmax = max(nmax, n[u]);
#pragma unroll
      for (int i = 0; i < NE; ++i) acc[u][i] = 0.0f;
      tl += d_tl;
      off += d_off;
      if (off >= cpr) {
        off -= cpr;
        ++tl;
      }
    }
    for (int k = 0; k < nmax; ++k) {
      U v[kUnroll];
      float g[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        if (k < n[u]) {
          v[u] = src[static_cast<size_t>(s_row[tok[u] * E + k]) * cpr + o[u]];
          g[u] = s_gate[tok[u] * E + k];
        }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        if (k < n[u]) {
          float x[NE];
          unpack<IN_DT, BYTES>(v[u], x);
          // one rounding for the product, one for the sum (no fused multiply-add)
#pragma unroll
          for (int i = 0; i < NE; ++i) acc[u][i] = acc[u][i] + x[i] * g[u];
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      // n < 0: past the end; n == 0: token without a valid route
      if (n[u] > 0 || (n[u] == 0 && !a.is_residual)) {
        const size_t at = (static_cast<size_t>(t0 + tok[u]) * cpr + o[u]) * OUT_BYTES;
        pack_store<OUT_DT, NE>(dst + at, acc[u]);
      }
    }
  }
}

// ---------------------------------------------------------------- host side
int pick_unit_bytes(size_t row_bytes, int elem, const void* p0, const void* p1, int out_scale_num,
                    int out_scale_den) {
  for (int b = 16; b >= elem; b >>= 1) {
    const size_t out_b = std::min<size_t>(16, static_cast<size_t>(b) * out_scale_num / out_scale_den);
    if (row_bytes % b == 0 && aligned(p0, b) && aligned(p1, out_b)) return b;
  }
  return 0;
}

int env_int(const char* name, int fallback) {
  const char* v = getenv(name);
  return v ? atoi(v) : fallback;
}

template <int BYTES, int DT>
void launch_dispatch(const DispatchArgs& a, int grid, size_t lds, hipStream_t st) {
  hipLaunchKernelGGL((dispatch_kernel<BYTES, DT>), dim3(grid), dim3(kBlock), lds, st, a);
}

template <int BYTES, int IN_DT, int OUT_DT>
void launch_combine(const CombineArgs& a, int grid, size_t lds, hipStream_t st) {
  hipLaunchKernelGGL((combine_kernel<BYTES, IN_DT, OUT_DT>), dim3(grid), dim3(kBlock), lds, st, a);
}

}  // namespace
}  // namespace brt

using namespace brt;

extern "C" int brt_hip_dispatch(const void* src, void* dst, const void* gates,
                                const int32_t* indices, const int32_t* loads,
                                const int32_t* counts, const int32_t* old_tags, int32_t* new_tags,
                                int T, int cell, int E, int P, int max_path_load,
                                int is_1d_routing, int is_tag_index, int dtype, void* stream) {
  if (T < 0 || E <= 0 || cell < 0 || P < 0 || max_path_load < 0)
    return fail(BRT_E_INVALID, "bad shape T=%d E=%d cell=%d P=%d", T, E, cell, P);
  if (dtype != BRT_F32 && dtype != BRT_F16 && dtype != BRT_BF16)
    return fail(BRT_E_UNSUPPORTED, "dtype %d is not supported", dtype);
  if (gates != nullptr && !is_1d_routing)
    return fail(BRT_E_INVALID, "gates are only supported with 1-d routing");
  if (counts != nullptr && is_tag_index)
    return fail(BRT_E_INVALID, "counts (zero-fill) is only supported with seat indices");
  if (static_cast<long>(T) * E >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*E >= 2^31");
  if (P == 0 || cell == 0) return BRT_OK;
  if (T == 0 && counts == nullptr) return BRT_OK;
  if (!dst || !loads || (T > 0 && (!src || !indices)))
    return fail(BRT_E_INVALID, "null argument");
  const int es = elem_bytes(dtype);
  const size_t row_bytes = static_cast<size_t>(cell) * es;
  const int bytes = pick_unit_bytes(row_bytes, es, src ? src : dst, dst, 1, 1);
  if (bytes == 0) return fail(BRT_E_INVALID, "src/dst are not aligned to the element size");

  DispatchArgs a{};
  a.src = src; a.dst = dst; a.gates = gates; a.idx = indices; a.loads = loads; a.counts = counts;
  a.old_tags = old_tags; a.new_tags = new_tags;
  a.T = T; a.E = E; a.P = P; a.mpl = max_path_load;
  a.cpr = static_cast<int>(row_bytes / bytes);
  a.is_1d = is_1d_routing; a.is_tag_index = is_tag_index;
  // rows of the index matrix per block: enough row bytes to keep 256 threads busy,
  // few enough that the grid covers the chip several times
  int rows = env_int("BRT_DISPATCH_ROWS", 0);
  if (rows <= 0) {
    rows = static_cast<int>(std::max<size_t>(1, 16384 / std::max<size_t>(row_bytes, 1)));
    rows = std::min(rows, 64);
    while (rows > 1 && (T + rows - 1) / rows < 1024) rows >>= 1;
  }
  rows = std::max(1, std::min(rows, std::max(1, 4096 / E)));
  a.rows_pb = rows;
  a.list_cap = rows * E;
  const size_t lds = (static_cast<size_t>(3) * E + 1 + 3 * static_cast<size_t>(a.list_cap)) * 4;
  if (lds > 120 * 1024) return fail(BRT_E_UNSUPPORTED, "E=%d needs too much LDS", E);
  const int grid = std::max(1, (T + rows - 1) / rows);
  hipStream_t st = as_stream(stream);

#define BRT_DISPATCH_CASE(B)                                               \
  case B:                                                                  \
    if (gates == nullptr) launch_dispatch<B, -1>(a, grid, lds, st);         \
    else if (dtype == BRT_F32) {                                           \
      if constexpr (B >= 4) launch_dispatch<(B >= 4 ? B : 4), BRT_F32>(a, grid, lds, st); \
    } else if (dtype == BRT_F16) launch_dispatch<B, BRT_F16>(a, grid, lds, st); \
    else launch_dispatch<B, BRT_BF16>(a, grid, lds, st);                   \
    break;
  switch (bytes) {
    BRT_DISPATCH_CASE(16)
    BRT_DISPATCH_CASE(8)
    BRT_DISPATCH_CASE(4)
    BRT_DISPATCH_CASE(2)
  }
#undef BRT_DISPATCH_CASE
  return check_launch("dispatch_kernel");
}

extern "C" int brt_hip_combine(const void* src, void* dst, const void* gates,
                               const int32_t* indices, const int32_t* loads, int T, int cell,
                               int E, int P, int max_path_load, int is_residual, int in_dtype,
                               int out_dtype, int gate_dtype, void* stream) {
  if (T < 0 || E <= 0 || cell < 0 || P < 0 || max_path_load < 0)
    return fail(BRT_E_INVALID, "bad shape T=%d E=%d cell=%d P=%d", T, E, cell, P);
  const bool in_ok = in_dtype == BRT_F32 || in_dtype == BRT_F16 || in_dtype == BRT_BF16;
  if (!in_ok || !(out_dtype == in_dtype || out_dtype == BRT_F32))
    return fail(BRT_E_UNSUPPORTED, "combine %d -> %d is not supported", in_dtype, out_dtype);
  if (gates != nullptr && gate_dtype != BRT_F32 && gate_dtype != BRT_F16 && gate_dtype != BRT_BF16)
    return fail(BRT_E_UNSUPPORTED, "gate dtype %d is not supported", gate_dtype);
  if (static_cast<long>(T) * E >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*E >= 2^31");
  if (T == 0 || cell == 0) return BRT_OK;
  if (!dst || !indices || !loads || (P > 0 && !src)) return fail(BRT_E_INVALID, "null argument");
  const int es = elem_bytes(in_dtype), os = elem_bytes(out_dtype);
  const size_t row_bytes = static_cast<size_t>(cell) * es;
  const int bytes = pick_unit_bytes(row_bytes, es, src ? src : dst, dst, os, es);
  if (bytes == 0) return fail(BRT_E_INVALID, "src/dst are not aligned to the element size");

  CombineArgs a{};
  a.src = src; a.dst = dst; a.gates = gates; a.idx = indices; a.loads = loads;
  a.T = T; a.E = E; a.P = P; a.mpl = max_path_load;
  a.cpr = static_cast<int>(row_bytes / bytes);
  a.is_residual = is_residual; a.gate_dtype = gate_dtype;
  int shift = 0;
  while ((1 << shift) < std::min(E, 64)) ++shift;
  a.ep_shift = shift;
  int rows = env_int("BRT_COMBINE_ROWS", 0);
  if (rows <= 0) {
    rows = static_cast<int>(std::max<size_t>(1, 16384 / std::max<size_t>(row_bytes, 1)));
    rows = std::min(rows, 64);
    while (rows > 1 && (T + rows - 1) / rows < 1024) rows >>= 1;
  }
  rows = std::max(1, std::min(rows, std::max(1, 4096 / E)));
  a.rows_pb = rows;
  const size_t lds = (static_cast<size_t>(2) * E + rows + 2 * static_cast<size_t>(rows) * E) * 4;
  if (lds > 120 * 1024) return fail(BRT_E_UNSUPPORTED, "E=%d needs too much LDS", E);
  const int grid = (T + rows - 1) / rows;
  hipStream_t st = as_stream(stream);

#define BRT_COMBINE_HALF(B, DT)                                              \
  if (out_dtype == BRT_F32) launch_combine<B, DT, BRT_F32>(a, grid, lds, st); \
  else launch_combine<B, DT, DT>(a, grid, lds, st);
#define BRT_COMBINE_CASE(B)                                                  \
  case B:                                                                    \
    if (in_dtype == BRT_F32) {                                               \
      if constexpr (B >= 4) launch_combine<(B >= 4 ? B : 4), BRT_F32, BRT_F32>(a, grid, lds, st); \
    } else if (in_dtype == BRT_F16) { BRT_COMBINE_HALF(B, BRT_F16) }         \
    else { BRT_COMBINE_HALF(B, BRT_BF16) }                                   \
    break;
  switch (bytes) {
    BRT_COMBINE_CASE(16)
    BRT_COMBINE_CASE(8)
    BRT_COMBINE_CASE(4)
    BRT_COMBINE_CASE(2)
  }
#undef BRT_COMBINE_CASE
#undef BRT_COMBINE_HALF
  return check_launch("combine_kernel");
}
