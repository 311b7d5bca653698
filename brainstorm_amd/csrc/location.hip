// Index / load generation, hot-mask throttling and index-format conversion.
//
// What is computed follows the reference kernels in src/router/location.cu
// (generate_indices_and_loads :212-257, throttle_hotmask :59-130,
// convert_*_indices :259-302); how it is computed does not.  The reference runs
// one 1024-thread block per path and walks the mask column (stride E) in serial
// 1024-row chunks behind 20 block barriers each.
//
// Here lanes are paths: a wavefront reads whole rows of the [T,E] mask with
// coalesced loads (for E < 64 one load covers 64/ep rows, ep = E rounded up to a
// power of two; for E > 64 the columns are walked in chunks of 64) and keeps the
// per-path running sums in registers, so the seat of a row is one add and one
// multiply per lane.  The rows are cut into bands, one per 4-wavefront
// workgroup:
//
//   pass 1  band_count_kernel  per band and path: sum of the mask values
//                              -> partial[band][path]
//   pass 2  band_apply_kernel  offset of a band = sum of the partials of the
//                              bands above it (a few KiB, cache resident; the
//                              four wavefronts split that sum and exchange it,
//                              together with their own column sums, through LDS
//                              behind the kernel's only barrier), then the rows
//                              are walked again and seats / throttled bits / tag
//                              slots are written; the last band also emits
//                              loads, counts and the throttle prefix.
//
// Two launches, no spinning and no state between calls: on this multi-die part
// a device-scope flag takes about as long to become visible to the other dies
// as a kernel boundary costs, so a single-pass chained scan buys nothing at MoE
// sizes (a few MiB) and adds a way to hang.  Up to 16 rows per wavefront stay in
// registers between the two walks of pass 2; longer bands re-read their rows
// (from cache).  The indices are written exactly once.  Masks small enough for one workgroup of
// eight wavefronts to hold in registers skip pass 1: that workgroup is the only band, and its
// wavefronts' column sums meet in LDS (one launch).
#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "rows.hpp"

// Scratch of brt_hip_generate_indices_and_loads_static: the per-band column sums that the first
// kernel of index generation hands to the second, for callers that cannot bring a workspace of
// their own.  Every GPU holds its own copy at its own address for the life of the process; in
// host code the name is only a handle for hipGetSymbolAddress, never an address to pass on.
constexpr size_t kStaticScratchInts = size_t{1} << 18;  // 1 MiB
static __device__ __align__(256) int scratch[kStaticScratchInts];

namespace brt {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPB = kBlock / kWave;
constexpr int kBatch = 16;         // row loads in flight per lane
constexpr int kPartialBatch = 32;  // loads of earlier bands' sums in flight per lane
constexpr int kMaxBands = 512;

enum { kSeat = 0, kTag = 1, kThrottle = 2 };

struct ScanGeometry {
  int ep_shift;  // log2 of the lanes one row occupies (E <= 64), 6 otherwise
  int rows_pw;   // rows per wavefront (multiple of the rows one load covers)
  int bands;     // workgroups
  int waves_pb;  // wavefronts per workgroup: kWavesPB, or kWavesSingle for the one-workgroup form
};

constexpr int kWavesSingle = 8;  // 512 threads: the kernel keeps its 256 registers per lane

ScanGeometry scan_geometry(int T, int E, bool tag_mode) {
  ScanGeometry g;
  int shift = 0;
  while ((1 << shift) < std::min(E, kWave)) ++shift;
  g.ep_shift = shift;
  g.waves_pb = kWavesPB;
  const int rps = kWave >> shift;  // rows per load instruction
  constexpr int forced_bands = 0;  // a fixed number of workgroups, for experiments
  // Small masks (decode-sized batches) take one launch of one workgroup, the column sums of its
  // wavefronts meeting in LDS.  Up to four loads per lane of a 4-wavefront workgroup that is
  // the ordinary kernel with a single band (16 x 8: 4.1 us, 128 x 8: 4.7 us); up to one batch of
  // loads per lane of an 8-wavefront workgroup it is the 512-thread form (128 x 64: 4.7 us,
  // 512 x 16: 6.8 us, against 6.9-7.3 us for two launches).  Tag indices scatter their stores
  // over the whole matrix, which one CU does slowly: beyond 128 rows they take the two launches
  // (512 x 16: 8.9 us against 10.6 us).  Larger masks are faster spread over many CUs, launch
  // cost and all.
  if (forced_bands <= 0 && E <= kWave && static_cast<long>(T) <= 4l * kWavesPB * rps) {
    long rows_pw = (static_cast<long>(T) + kWavesPB - 1) / kWavesPB;
    g.rows_pw = static_cast<int>(std::max<long>((rows_pw + rps - 1) / rps * rps, rps));
    g.bands = 1;
    return g;
  }
  if (forced_bands <= 0 && E <= kWave && (!tag_mode || T <= 128) &&
      static_cast<long>(T) <= static_cast<long>(kWavesSingle) * kBatch * rps) {
    long rows_pw = (static_cast<long>(T) + kWavesSingle - 1) / kWavesSingle;
    rows_pw = std::max<long>((rows_pw + rps - 1) / rps * rps, rps);
    g.rows_pw = static_cast<int>(rows_pw);
    g.bands = 1;
    g.waves_pb = kWavesSingle;
    return g;
  }
  // Enough bands that a wavefront's rows fit one batch of loads, at least 128 (so
  // that many CUs take part) and never more than kMaxBands, which bounds the sum
  // over earlier bands every band has to form.
  const long one_batch = static_cast<long>(kWavesPB) * kBatch * rps;
  const int fit = static_cast<int>(std::min<long>(kMaxBands, (T + one_batch - 1) / one_batch));
  const int want = forced_bands > 0 ? forced_bands : std::max(128, fit);
  long rows_pb = (static_cast<long>(T) + want - 1) / want;
  rows_pb = std::max<long>(rows_pb, (static_cast<long>(T) + kMaxBands - 1) / kMaxBands);
  long rows_pw = (rows_pb + kWavesPB - 1) / kWavesPB;
  rows_pw = (rows_pw + rps - 1) / rps * rps;
  rows_pw = std::max<long>(rows_pw, rps);
  g.rows_pw = static_cast<int>(rows_pw);
  const long per_band = rows_pw * kWavesPB;
  g.bands = static_cast<int>(std::max(1l, (static_cast<long>(T) + per_band - 1) / per_band));
  return g;
}

struct ScanArgs {
  const int* mask;
  int* out;
  int* loads;
  int* counts;
  const int* caps;
  int* prefix;           // throttle only, updated in place
  const int* threshold;  // throttle only
  int* partial;          // [bands][E] per-band column sums
  int* prefix_in;        // throttle only: copy of prefix taken by pass 1 ([E])
  int T, E, C;
  int capacity_padding, path_wise_padding;
  int ep_shift, rows_pw, bands;
  int n_ins;  // loads per lane that cover a wavefront's rows: rows_pw / (rows one load covers)
};

// Sum over the lanes that hold the same path (lanes e, e+ep, e+2ep, ...); every
// lane ends up with the total.
__device__ __forceinline__ int sum_over_rows_in_wave(int v, int ep_shift) {
  for (int d = 1 << ep_shift; d < kWave; d <<= 1) v += __shfl_xor(v, d, kWave);
  return v;
}

// Second walk over one batch of row words held in registers: turns the mask words
// into seats / throttled bits / tag slots.  Rows of one load are ordered by lane
// group; all cross-lane traffic of the batch is issued first and does not depend
// on the running sum (incl = sum over the groups up to and including this
// lane's, tot = sum over all groups).
template <int MODE>
__device__ __forceinline__ void walk_batch(const int (&m)[kBatch], int i0, int n_ins, int& carry,
                                           int thr, int total, long row_w, int rps, int ep, int sub,
                                           int e, int lane, int col, bool col_ok, const ScanArgs& a) {
  int incl[kBatch], tot[kBatch];
#pragma unroll
  for (int u = 0; u < kBatch; ++u) {
    incl[u] = m[u];
    tot[u] = m[u];
    if (rps > 1 && i0 + u < n_ins) {  // wave-uniform
      int x = m[u];
      for (int d = ep; d < kWave; d <<= 1) {
        const int t = __shfl_up(x, d, kWave);
        if (lane >= d) x += t;
      }
      incl[u] = x;
      tot[u] = __shfl(x, (rps - 1) * ep + e, kWave);
    }
  }
  // rows of this wavefront through one 64-bit base and 32-bit offsets: the address of every
  // store is one instruction instead of a 64-bit multiply-add chain
  int* __restrict__ out_w = a.out + row_w * a.E;
  const int rows_here = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - row_w)));
#pragma unroll
  for (int u = 0; u < kBatch; ++u) {
    const int run = carry + incl[u];
    carry += tot[u];
    const int rl = (i0 + u) * rps + sub;  // row within the wavefront's rows
    if (i0 + u < n_ins && col_ok && rl < rows_here) {
      const unsigned at = static_cast<unsigned>(rl) * a.E + col;
      if (MODE == kSeat) {
        out_w[at] = run * m[u];  // location * mask, location.cu:177-178
      } else if (MODE == kThrottle) {
        out_w[at] = (m[u] == 1 && run <= thr) ? 1 : 0;
      } else {
        const int index = run * m[u];
        if (index >= 1 && index <= a.T)
          a.out[static_cast<size_t>(index - 1) * a.E + col] = static_cast<int>(row_w) + rl + 1;
        // slots past the path's last tag are nobody's to write but this row's owner
        if (row_w + rl >= total) out_w[at] = 0;
      }
    }
  }
}

// Loads one batch of row words (zero beyond the band / the matrix).  One 64-bit base per
// wavefront and 32-bit offsets; the loads are unconditional (a word outside the wavefront's rows
// is read from its first row and dropped), so that they issue back to back.
__device__ __forceinline__ void load_batch(int (&v)[kBatch], int i0, int n_ins, long row_w, int rps,
                                           int sub, int col, bool col_ok, const ScanArgs& a) {
  const int* __restrict__ mask_w = a.mask + min(row_w, a.T - 1l) * a.E;
  const int rows_here = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - row_w)));
  bool ok[kBatch];
#pragma unroll
  for (int u = 0; u < kBatch; ++u) {
    const int rl = (i0 + u) * rps + sub;
    ok[u] = i0 + u < n_ins && col_ok && rl < rows_here;
    v[u] = mask_w[ok[u] ? static_cast<unsigned>(rl) * a.E + col : 0u];
  }
#pragma unroll
  for (int u = 0; u < kBatch; ++u) v[u] = ok[u] ? v[u] : 0;
}

// pass 1: column sums of one band
__global__ __launch_bounds__(kBlock) void band_count_kernel(ScanArgs a) {
  __shared__ int s_sum[kWavesPB][kWave];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int E = a.E;
  const int ep = 1 << a.ep_shift, rps = kWave >> a.ep_shift;
  const int e = lane & (ep - 1), sub = lane >> a.ep_shift;
  const long row_w = (static_cast<long>(blockIdx.x) * kWavesPB + wave) * a.rows_pw;
  const int n_ins = a.n_ins;
  for (int c0 = 0; c0 < E; c0 += kWave) {
    const int col = c0 + e;
    const bool col_ok = col < E;
    int sum = 0;
    for (int i0 = 0; i0 < n_ins; i0 += kBatch) {
      int v[kBatch];
      load_batch(v, i0, n_ins, row_w, rps, sub, col, col_ok, a);
#pragma unroll
      for (int u = 0; u < kBatch; ++u) sum += v[u];
    }
    sum = sum_over_rows_in_wave(sum, a.ep_shift);
    if (c0 > 0) __syncthreads();
    if (sub == 0) s_sum[wave][e] = sum;
    __syncthreads();
    if (tid < kWave && c0 + tid < E) {
      int total = 0;
#pragma unroll
      for (int k = 0; k < kWavesPB; ++k) total += s_sum[k][tid];
      a.partial[static_cast<size_t>(blockIdx.x) * E + c0 + tid] = total;
      // pass 2 overwrites prefix[] while other bands may not have started yet
      if (a.prefix != nullptr && blockIdx.x == 0) a.prefix_in[c0 + tid] = a.prefix[c0 + tid];
    }
  }
}

// pass 2: offsets from the bands above, running sums in registers, results out
template <int MODE, int kWavesPB>
__global__ __launch_bounds__(kWavesPB * kWave) void band_apply_kernel(ScanArgs a) {
  __shared__ int s_above[kWavesPB][kWave];  // each wave's share of the sum over earlier bands
  __shared__ int s_own[kWavesPB][kWave];    // column sums of each wave's own rows
  __shared__ int s_below[kWavesPB][kWave];  // tag mode: share of the sum over later bands
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int E = a.E, band = blockIdx.x;
  const int ep = 1 << a.ep_shift, rps = kWave >> a.ep_shift;
  const int e = lane & (ep - 1), sub = lane >> a.ep_shift;
  const long row_w = (static_cast<long>(band) * kWavesPB + wave) * a.rows_pw;
  const int n_ins = a.n_ins;

  for (int c0 = 0; c0 < E; c0 += kWave) {
    const int col = c0 + e;
    const bool col_ok = col < E;
    // ---- own rows: the first batch stays in registers ---------------------------------
    int m0[kBatch];
    load_batch(m0, 0, n_ins, row_w, rps, sub, col, col_ok, a);
    // ---- this wave's share of the offset: bands wave, wave+4, ... above this one ----
    int above = 0, below = 0;
    for (int j0 = wave + sub * kWavesPB; j0 < band; j0 += kWavesPB * rps * kPartialBatch) {
      // unconditional loads through 32-bit offsets (an entry that does not count is read from
      // the head of the table and dropped), so that they issue back to back
      int v[kPartialBatch];
      bool ok[kPartialBatch];
#pragma unroll
      for (int u = 0; u < kPartialBatch; ++u) {
        const int j = j0 + u * kWavesPB * rps;
        ok[u] = j < band && col_ok;
        v[u] = a.partial[ok[u] ? static_cast<unsigned>(j) * E + col : 0u];
      }
#pragma unroll
      for (int u = 0; u < kPartialBatch; ++u) above += ok[u] ? v[u] : 0;
    }
    if (MODE == kTag) {  // the tag list of a path ends at its total: the later bands count too
      for (int j0 = band + 1 + wave + sub * kWavesPB; j0 < a.bands; j0 += kWavesPB * rps * kPartialBatch) {
        int v[kPartialBatch];
        bool ok[kPartialBatch];
#pragma unroll
        for (int u = 0; u < kPartialBatch; ++u) {
          const int j = j0 + u * kWavesPB * rps;
          ok[u] = j < a.bands && col_ok;
          v[u] = a.partial[ok[u] ? static_cast<unsigned>(j) * E + col : 0u];
        }
#pragma unroll
        for (int u = 0; u < kPartialBatch; ++u) below += ok[u] ? v[u] : 0;
      }
      below = sum_over_rows_in_wave(below, a.ep_shift);
    }
    int own = 0;
#pragma unroll
    for (int u = 0; u < kBatch; ++u) own += m0[u];
    for (int i0 = kBatch; i0 < n_ins; i0 += kBatch) {
      int v[kBatch];
      load_batch(v, i0, n_ins, row_w, rps, sub, col, col_ok, a);
#pragma unroll
      for (int u = 0; u < kBatch; ++u) own += v[u];
    }
    above = sum_over_rows_in_wave(above, a.ep_shift);
    own = sum_over_rows_in_wave(own, a.ep_shift);
    // read before the barrier: with a single band the first wavefront overwrites prefix[] at
    // the end of its walk, which no wavefront may overtake
    int thr = 0, pre_in = 0;
    if (MODE == kThrottle && col_ok) {
      pre_in = (a.bands > 1 ? a.prefix_in : a.prefix)[col];
      thr = a.threshold[col];
    }
    if (c0 > 0) __syncthreads();
    if (sub == 0) {
      s_above[wave][e] = above;
      s_own[wave][e] = own;
      if (MODE == kTag) s_below[wave][e] = below;
    }
    __syncthreads();
    int carry = 0, band_total = 0, later = 0;
#pragma unroll
    for (int k = 0; k < kWavesPB; ++k) {
      carry += s_above[k][e];
      band_total += s_own[k][e];
      if (k < wave) carry += s_own[k][e];
      if (MODE == kTag) later += s_below[k][e];
    }
    band_total += carry;
#pragma unroll
    for (int k = 0; k < kWavesPB; ++k)
      if (k < wave) band_total -= s_own[k][e];  // = offset + all four waves
    if (MODE == kThrottle) carry += pre_in;

    // ---- walk the rows again: running sum per path, one result per element ----------
    const int total = band_total + later;  // tag mode: entries of this path's list
    walk_batch<MODE>(m0, 0, n_ins, carry, thr, total, row_w, rps, ep, sub, e, lane, col, col_ok, a);
    for (int i0 = kBatch; i0 < n_ins; i0 += kBatch) {
      int v[kBatch];
      load_batch(v, i0, n_ins, row_w, rps, sub, col, col_ok, a);
      walk_batch<MODE>(v, i0, n_ins, carry, thr, total, row_w, rps, ep, sub, e, lane, col, col_ok, a);
    }

    // ---- totals: loads / counts / throttle prefix (last band only) ---------------------
    if (band == a.bands - 1 && wave == 0 && sub == 0 && col_ok) {
      if (MODE == kThrottle) {
        a.prefix[col] = min(band_total + pre_in, thr);
      } else {
        a.loads[col] =
            finalize_load(band_total, a.caps, a.C, a.capacity_padding, a.path_wise_padding, col);
        if (a.counts) a.counts[col] = band_total;
      }
    }
  }
}

// ---- index generation pass 2 and dispatch in one kernel ---------------------------------------
// What band_apply_kernel<kSeat> writes, and in the same kernel what the dispatch of those indices
// writes (1-d routing, unweighted, un-strided layout): the rows of the wavefront's own cells go to
// start[path] + seat - 1 of the path-major buffer.  A wavefront's cells are one contiguous run of
// 16-byte units; every lane requests its share of them before anything else, so the rows travel
// while the mask words and the sums of the other bands are fetched and walked, and are stored as
// soon as the seats are known.  Every band needs the totals of all paths (for the path starts),
// so it adds up the bands below it as well as those above.  The rows no cell owns (padding rows
// of a path, rows past the last path) are zero-filled by the same launch, dealt evenly to all
// wavefronts.  E <= 64; a wavefront's cells fit kFusedUnits 16-byte units per lane (the host
// picks the rows per wavefront for that).
constexpr int kFusedUnits = 32;  // 16-byte units of row data a lane holds (128 registers)
constexpr int kFusedCaps = 8;    // supported capacities held in registers
constexpr int kFusedPartials = 64;  // band sums a lane adds up (one batch of loads)

struct FusedArgs {
  ScanArgs s;
  const u32x4* src;  // [T, cpr]
  u32x4* dst;        // [P, cpr]
  int* row_tags;     // [P] or null
  int P, cpr;
};

template <bool STREAM, int NV>
__global__ __launch_bounds__(kBlock) void band_apply_dispatch_kernel(FusedArgs f) {
  const ScanArgs& a = f.s;
  __shared__ int s_above[kWavesPB][kWave];
  __shared__ int s_own[kWavesPB][kWave];
  __shared__ int s_below[kWavesPB][kWave];
  __shared__ int s_n[kWavesPB][kBatch * kWave];     // per wavefront: paths that take each of its rows
  __shared__ int s_list[kWavesPB][kBatch * kWave];  // per wavefront: their destination rows, row-major
  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int E = a.E, band = blockIdx.x;
  const int ep = 1 << a.ep_shift, rps = kWave >> a.ep_shift;
  const int e = lane & (ep - 1), sub = lane >> a.ep_shift;
  const long row_w = (static_cast<long>(band) * kWavesPB + wave) * a.rows_pw;
  const int n_ins = a.n_ins;
  const int rows_here = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - row_w)));
  const int cpr = f.cpr;
  const bool col_ok = e < E;

  // Every load of the kernel's first memory round trip is a buffer load: a wave-uniform base and
  // extent per array, a 32-bit offset per lane, and a word outside the extent (a row past the
  // wavefront's rows, a band past the last, a lane past E) reads as zero -- no 64-bit address
  // arithmetic, no branch and no select stands between the loads, so all of them are in flight
  // before the first is used.
  constexpr unsigned kOutside = 0x80000000u;
  auto resource = [](const void* base, size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0,
                                             static_cast<int>(std::min<size_t>(bytes, 0x7fffffff)), 0x00020000);
  };
  // Issue order = order of use (the memory counter retires loads in order): band sums, own mask
  // words, capacities, and last the wavefront's rows, which are stored at the very end.
  // ---- sums of the other bands (the host keeps the bands within kFusedPartials loads per lane) ----
  int part[kFusedPartials];
  const int j_first = wave + sub * kWavesPB, j_step = kWavesPB * rps;
  {
    const __amdgpu_buffer_rsrc_t res_partial = resource(a.partial, static_cast<size_t>(a.bands) * E * 4);
    const unsigned partial_off = col_ok ? (j_first * E + e) * 4 : kOutside;
#pragma unroll
    for (int u = 0; u < kFusedPartials; ++u)
      part[u] = __builtin_amdgcn_raw_buffer_load_b32(res_partial, partial_off + u * j_step * E * 4, 0, 0);
  }
  // ---- own mask words -----------------------------------------------------------------------
  int m0[kBatch];
  {
    const __amdgpu_buffer_rsrc_t res_mask =
        resource(a.mask + (rows_here > 0 ? row_w : 0) * E, static_cast<size_t>(rows_here) * E * 4);
    const unsigned mask_off = col_ok ? (sub * E + e) * 4 : kOutside;
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      m0[u] = __builtin_amdgcn_raw_buffer_load_b32(res_mask, mask_off + u * rps * E * 4, 0, 0);
  }
  // ---- capacity menu: lane i fetches entry i, lane e the path's own capacity (path-wise padding) ----
  const __amdgpu_buffer_rsrc_t res_caps = resource(a.caps, static_cast<size_t>(a.C) * 4);
  const int cap_lane = __builtin_amdgcn_raw_buffer_load_b32(res_caps, lane * 4, 0, 0);
  const int cap_own = __builtin_amdgcn_raw_buffer_load_b32(res_caps, col_ok ? e * 4 : kOutside, 0, 0);
  // ---- the wavefront's rows ------------------------------------------------------------------
  const int n_units = rows_here * cpr;
  const __amdgpu_buffer_rsrc_t res_rows =
      resource(f.src + (rows_here > 0 ? row_w : 0) * cpr, static_cast<size_t>(n_units) * 16);
  u32x4 val[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i)
    val[i] = __builtin_amdgcn_raw_buffer_load_b128(res_rows, (i * kWave + lane) * 16, 0, 0);
  __builtin_amdgcn_sched_barrier(0);  // nothing below is scheduled in between the loads

  int above = 0, below = 0;
#pragma unroll
  for (int u = 0; u < kFusedPartials; ++u) {
    const int j = j_first + u * j_step;
    above += j < band ? part[u] : 0;
    below += j > band ? part[u] : 0;
  }
  int capv[kFusedCaps];
#pragma unroll
  for (int i = 0; i < kFusedCaps; ++i) capv[i] = read_lane(cap_lane, i);
  int own = 0;
#pragma unroll
  for (int u = 0; u < kBatch; ++u) own += m0[u];
  above = sum_over_rows_in_wave(above, a.ep_shift);
  below = sum_over_rows_in_wave(below, a.ep_shift);
  own = sum_over_rows_in_wave(own, a.ep_shift);
  if (sub == 0) {
    s_above[wave][e] = above;
    s_own[wave][e] = own;
    s_below[wave][e] = below;
  }
  __syncthreads();
  int carry = 0, total = 0;
#pragma unroll
  for (int k = 0; k < kWavesPB; ++k) {
    carry += s_above[k][e];
    total += s_above[k][e] + s_own[k][e] + s_below[k][e];
    if (k < wave) carry += s_own[k][e];
  }

  // ---- loads and path starts from the totals (every lane: those of its own path) ------------
  int load_e = 0;
  if (col_ok) {
    if (a.path_wise_padding) load_e = cap_own;
    else if (total == 0 || a.C == 0) load_e = total;
    else {
      load_e = capv[0];  // overwritten below; the last capacity when none holds the count
      bool done = false;
#pragma unroll
      for (int i = 0; i < kFusedCaps; ++i) {
        if (i < a.C) {
          if (!done && total <= capv[i]) {
            load_e = a.capacity_padding ? capv[i] : total;
            done = true;
          }
          if (!done) load_e = capv[i];
        }
      }
    }
  }
  const int incl_l = wave_inclusive_scan(sub == 0 ? load_e : 0);
  const int start_e = __shfl(incl_l - (sub == 0 ? load_e : 0), e, kWave);
  const int sum_loads = read_lane(incl_l, kWave - 1);

  // ---- walk the rows: seats out, destination rows into the wavefront's table ----------------
  {
    int incl[kBatch], tot[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      incl[u] = m0[u];
      tot[u] = m0[u];
      if (rps > 1 && u < n_ins) {
        int x = m0[u];
        for (int d = ep; d < kWave; d <<= 1) {
          const int t = __shfl_up(x, d, kWave);
          if (lane >= d) x += t;
        }
        incl[u] = x;
        tot[u] = __shfl(x, (rps - 1) * ep + e, kWave);
      }
    }
    int* __restrict__ out_w = a.out + row_w * E;
    const unsigned long long seg0 = ep == kWave ? ~0ull : ((1ull << ep) - 1ull);
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      if (u < n_ins) {  // wave-uniform
        const int run = carry + incl[u];
        carry += tot[u];
        const int rl = u * rps + sub;
        const bool mine = col_ok && rl < rows_here;
        const int v = run * m0[u];
        if (mine) out_w[static_cast<unsigned>(rl) * E + e] = v;  // location * mask, location.cu:177-178
        const int dst_row = start_e + v - 1;
        const bool hit = mine && v >= 1 && v <= load_e && dst_row < f.P;
        const unsigned long long seg = (__ballot(hit) >> (sub * ep)) & seg0;
        if (hit) {
          s_list[wave][rl * ep + __popcll(seg & ((1ull << e) - 1ull))] = dst_row;
          if (f.row_tags != nullptr) f.row_tags[dst_row] = static_cast<int>(row_w) + rl + 1;
        }
        if (e == 0) s_n[wave][rl] = __popcll(seg);
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();

  // ---- the rows leave: unit i*64 + lane of the wavefront's run belongs to row (i*64+lane)/cpr ----
  // The table is read for all units at once (one LDS latency instead of two per unit), the first
  // destination of every unit is stored, and only a wavefront that holds a cell on several paths
  // walks the further destinations.
  {
    const int q64 = kWave / cpr, r64 = kWave - q64 * cpr;
    const int row0 = lane / cpr, off0 = lane - row0 * cpr;
    auto advance = [&](int& row, int& off) {
      row += q64;
      off += r64;
      if (off >= cpr) off -= cpr, ++row;
    };
    int n_of[NV], d_of[NV];
    {
      int row = row0, off = off0;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int at = i * kWave + lane < n_units ? row : 0;
        n_of[i] = s_n[wave][at];
        d_of[i] = s_list[wave][at * ep];
        advance(row, off);
      }
    }
    int most = 0;
    {
      int row = row0, off = off0;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        if (i * kWave + lane >= n_units) n_of[i] = 0;
        if (n_of[i] > 0) store_unit<STREAM>(f.dst + static_cast<size_t>(d_of[i]) * cpr + off, val[i]);
        most = max(most, n_of[i]);
        advance(row, off);
      }
    }
    if (__ballot(most > 1) != 0) {
      int row = row0, off = off0;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        for (int j = 1; j < n_of[i]; ++j) {
          const int d = s_list[wave][row * ep + j];
          store_unit<STREAM>(f.dst + static_cast<size_t>(d) * cpr + off, val[i]);
        }
        advance(row, off);
      }
    }
  }

  // ---- rows no cell owns: padding rows of the paths, then the rows past the last path ----------
  {
    const long n_waves = static_cast<long>(gridDim.x) * kWavesPB;
    const long me = static_cast<long>(band) * kWavesPB + wave;
    const bool path_lane = sub == 0 && col_ok;
    const int z = path_lane ? load_e - max(0, min(total, load_e)) : 0;
    const int z_incl = wave_inclusive_scan(z);
    const long Z = read_lane(z_incl, kWave - 1);
    const long tail = max(0l, static_cast<long>(f.P) - sum_loads);
    if (Z + tail > 0) {
      const unsigned nw = static_cast<unsigned>(n_waves), w = static_cast<unsigned>(me);
      const unsigned all = static_cast<unsigned>(Z + tail);
      const unsigned q = all / nw, r = all % nw;
      const long z0 = static_cast<long>(q) * w + min(w, r), z1 = z0 + q + (w < r ? 1 : 0);
      for (long zi = z0; zi < z1; ++zi) {
        long row;
        if (zi < Z) {
          const int pe = __builtin_ctzll(__ballot(z_incl > zi));
          const int pad = read_lane(z, pe);
          row = static_cast<long>(read_lane(start_e, pe)) + (read_lane(load_e, pe) - pad) +
                (zi - (read_lane(z_incl, pe) - pad));
        } else {
          row = sum_loads + (zi - Z);
        }
        if (row < f.P) {
          for (int o = lane; o < cpr; o += kWave) f.dst[static_cast<size_t>(row) * cpr + o] = zero_unit<16>();
          if (f.row_tags != nullptr && lane == 0) f.row_tags[row] = 0;
        }
      }
    }
  }

  // ---- totals (last band only) -----------------------------------------------------------
  if (band == a.bands - 1 && wave == 0 && sub == 0 && col_ok) {
    a.loads[e] = load_e;
    if (a.counts) a.counts[e] = total;
  }
}

__global__ void fill_int_kernel(int* p, int n, int v) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ __launch_bounds__(256) void seat_to_tag_kernel(const int* __restrict__ src,
                                                          int* __restrict__ dst, int T, int E) {
  const size_t total = static_cast<size_t>(T) * E;
  for (size_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
    const int seat = src[i];
    if (seat >= 1 && seat <= T) {
      const int t = static_cast<int>(i / E);
      const int e = static_cast<int>(i - static_cast<size_t>(t) * E);
      dst[static_cast<size_t>(seat - 1) * E + e] = t + 1;
    }
  }
}

__global__ __launch_bounds__(256) void tag_to_seat_kernel(const int* __restrict__ src,
                                                          int* __restrict__ dst,
                                                          const int* __restrict__ loads, int T,
                                                          int E) {
  const size_t total = static_cast<size_t>(T) * E;
  for (size_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
    const int s = static_cast<int>(i / E);
    const int e = static_cast<int>(i - static_cast<size_t>(s) * E);
    if (s >= loads[e]) continue;
    const int tag = src[i];
    if (tag < 1 || tag > T) continue;
    // the reference walks slots s, s+1024, ... per thread and stops at the first
    // empty one (location.cu:289-300): an empty slot above in the chain hides s
    bool visible = true;
    for (int k = s - 1024; k >= 0; k -= 1024)
      if (src[static_cast<size_t>(k) * E + e] == 0) {
        visible = false;
        break;
      }
    if (visible) dst[static_cast<size_t>(tag - 1) * E + e] = s + 1;
  }
}

int launch_scan(int mode, ScanArgs& a, void* workspace, size_t workspace_bytes, void* stream) {
  const ScanGeometry g = scan_geometry(a.T, a.E, mode == kTag);
  const size_t need = brt_hip_scan_workspace_bytes(a.T, a.E);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(BRT_E_WORKSPACE, "scan workspace too small: %zu < %zu bytes", workspace_bytes,
                need);
  if (!aligned(workspace, 4)) return fail(BRT_E_INVALID, "scan workspace must be 4-byte aligned");
  a.partial = static_cast<int*>(workspace);
  a.prefix_in = a.partial + static_cast<size_t>(g.bands) * a.E;
  a.ep_shift = g.ep_shift;
  a.rows_pw = g.rows_pw;
  a.n_ins = g.rows_pw >> (6 - g.ep_shift);
  a.bands = g.bands;
  const dim3 grid(g.bands);
  hipStream_t st = as_stream(stream);
  if (g.waves_pb == kWavesSingle) {
    const dim3 block(kWavesSingle * kWave);
    if (mode == kSeat)
      hipLaunchKernelGGL((band_apply_kernel<kSeat, kWavesSingle>), grid, block, 0, st, a);
    else if (mode == kTag)
      hipLaunchKernelGGL((band_apply_kernel<kTag, kWavesSingle>), grid, block, 0, st, a);
    else
      hipLaunchKernelGGL((band_apply_kernel<kThrottle, kWavesSingle>), grid, block, 0, st, a);
    return check_launch("band_apply_kernel");
  }
  if (g.bands > 1)  // a single band has nothing above it
    hipLaunchKernelGGL(band_count_kernel, grid, dim3(kBlock), 0, st, a);
  if (mode == kSeat)
    hipLaunchKernelGGL((band_apply_kernel<kSeat, kWavesPB>), grid, dim3(kBlock), 0, st, a);
  else if (mode == kTag)
    hipLaunchKernelGGL((band_apply_kernel<kTag, kWavesPB>), grid, dim3(kBlock), 0, st, a);
  else
    hipLaunchKernelGGL((band_apply_kernel<kThrottle, kWavesPB>), grid, dim3(kBlock), 0, st, a);
  return check_launch("band_apply_kernel");
}

// Geometry of the fused kernel: rows per wavefront so that a wavefront's cells fit the units a
// lane holds and, where the batch allows, every CU gets a band.
bool fused_geometry(int T, int E, int cpr, ScanGeometry* g) {
  if (T <= 0 || E <= 0 || E > kWave || cpr <= 0) return false;
  int shift = 0;
  while ((1 << shift) < E) ++shift;
  const int rps = kWave >> shift;
  const long fit = static_cast<long>(kFusedUnits) * kWave / cpr / rps * rps;  // rows a wavefront can hold
  if (fit < rps) return false;
  const long most = std::min<long>(static_cast<long>(kBatch) * rps, fit);
  constexpr long want_bands = 256;  // one per CU: half as many make the kernel a third longer at 8192 x 64
  long rows_pw = (static_cast<long>(T) + want_bands * kWavesPB - 1) / (want_bands * kWavesPB);
  rows_pw = std::min(most, std::max<long>((rows_pw + rps - 1) / rps * rps, rps));
  const long per_band = rows_pw * kWavesPB;
  const long bands = (static_cast<long>(T) + per_band - 1) / per_band;
  if (bands > kMaxBands || bands > static_cast<long>(kFusedPartials) * kWavesPB * rps) return false;
  g->ep_shift = shift;
  g->rows_pw = static_cast<int>(rows_pw);
  g->bands = static_cast<int>(bands);
  g->waves_pb = kWavesPB;
  return true;
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device, resolved once per device.
int static_scratch(void** out) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return fail(BRT_E_LAUNCH, "hipGetDevice: %s", hipGetErrorString(err));
  if (device < 0 || device >= kMaxDevices)
    return fail(BRT_E_UNSUPPORTED, "device ordinal %d outside [0, %d)", device, kMaxDevices);
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr)
      return fail(BRT_E_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", device,
                  hipGetErrorString(err));
    g_scratch_ptr[device] = ptr;
  }
  *out = g_scratch_ptr[device];
  return BRT_OK;
}

}  // namespace
}  // namespace brt

using namespace brt;

extern "C" size_t brt_hip_scan_workspace_bytes(int T, int E) {
  if (T <= 0 || E <= 0) return 0;
  // enough for either index format (tag indices leave the one-workgroup form earlier)
  const int bands = std::max(scan_geometry(T, E, false).bands, scan_geometry(T, E, true).bands);
  return (static_cast<size_t>(bands) + 1) * E * sizeof(int);
}

extern "C" int brt_hip_generate_indices_and_loads(const int32_t* mask, int32_t* indices,
                                                  int32_t* loads, int32_t* counts, int T, int E,
                                                  const int32_t* caps, int C,
                                                  int capacity_padding, int path_wise_padding,
                                                  int is_tag_index, void* workspace,
                                                  size_t workspace_bytes, void* stream) {
  if (T < 0 || E <= 0) return fail(BRT_E_INVALID, "bad shape T=%d E=%d", T, E);
  if (loads == nullptr) return fail(BRT_E_INVALID, "loads is null");
  if (static_cast<long>(T) * E >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*E >= 2^31");
  if (caps == nullptr) C = 0;
  if (capacity_padding && C < 1)
    return fail(BRT_E_INVALID, "capacity_padding needs at least one supported capacity");
  if (!capacity_padding) path_wise_padding = 0;
  if (path_wise_padding && C < E)
    return fail(BRT_E_INVALID, "path_wise_padding needs one capacity per path (%d < %d)", C, E);
  if (T == 0) {
    hipLaunchKernelGGL(fill_int_kernel, dim3((E + 255) / 256), dim3(256), 0, as_stream(stream),
                       loads, E, 0);
    if (counts)
      hipLaunchKernelGGL(fill_int_kernel, dim3((E + 255) / 256), dim3(256), 0, as_stream(stream),
                         counts, E, 0);
    return check_launch("fill_int_kernel");
  }
  if (mask == nullptr || indices == nullptr) return fail(BRT_E_INVALID, "null mask/indices");
  ScanArgs a{};
  a.mask = mask;
  a.out = indices;
  a.loads = loads;
  a.counts = counts;
  a.caps = caps;
  a.C = C;
  a.T = T;
  a.E = E;
  a.capacity_padding = capacity_padding;
  a.path_wise_padding = path_wise_padding;
  return launch_scan(is_tag_index ? kTag : kSeat, a, workspace, workspace_bytes, stream);
}

extern "C" size_t brt_hip_static_scratch_bytes(void) { return kStaticScratchInts * sizeof(int); }

extern "C" int brt_hip_generate_indices_and_loads_static(const int32_t* mask, int32_t* indices,
                                                         int32_t* loads, int32_t* counts, int T,
                                                         int E, const int32_t* caps, int C,
                                                         int capacity_padding,
                                                         int path_wise_padding, int is_tag_index,
                                                         void* stream) {
  if (T < 0 || E <= 0) return fail(BRT_E_INVALID, "bad shape T=%d E=%d", T, E);
  if (static_cast<long>(T) * E >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*E >= 2^31");
  const size_t need = brt_hip_scan_workspace_bytes(T, E);
  if (need > kStaticScratchInts * sizeof(int))
    return fail(BRT_E_WORKSPACE,
                "a [%d,%d] mask needs %zu bytes of scratch, the built-in buffer holds %zu: use "
                "brt_hip_generate_indices_and_loads with a workspace",
                T, E, need, kStaticScratchInts * sizeof(int));
  void* ptr = nullptr;
  if (const int rc = static_scratch(&ptr)) return rc;
  // nothing in the scratch has to start at zero: every word the second kernel reads was written
  // by the first kernel of the same call
  return brt_hip_generate_indices_and_loads(mask, indices, loads, counts, T, E, caps, C,
                                            capacity_padding, path_wise_padding, is_tag_index, ptr,
                                            kStaticScratchInts * sizeof(int), stream);
}

extern "C" int brt_hip_route_and_dispatch_supported(int T, int E, size_t cell_bytes, int C,
                                                    int path_wise_padding) {
  ScanGeometry g;
  if (cell_bytes == 0 || cell_bytes % 16 != 0 || cell_bytes / 16 > 0x7fffffffull) return 0;
  if (!path_wise_padding && C > kFusedCaps) return 0;
  return fused_geometry(T, E, static_cast<int>(cell_bytes / 16), &g) ? 1 : 0;
}

extern "C" size_t brt_hip_route_and_dispatch_workspace_bytes(int T, int E, size_t cell_bytes) {
  ScanGeometry g;
  if (cell_bytes == 0 || cell_bytes % 16 != 0 || cell_bytes / 16 > 0x7fffffffull) return 0;
  if (!fused_geometry(T, E, static_cast<int>(cell_bytes / 16), &g)) return 0;
  return (static_cast<size_t>(g.bands) + 1) * E * sizeof(int);
}

extern "C" int brt_hip_route_and_dispatch(const int32_t* mask, const void* cells, void* rows,
                                          int32_t* indices, int32_t* loads, int32_t* counts,
                                          int32_t* row_tags, int T, int E, int P, size_t cell_bytes,
                                          const int32_t* caps, int C, int capacity_padding,
                                          int path_wise_padding, void* workspace,
                                          size_t workspace_bytes, void* stream) {
  if (T < 0 || E <= 0 || P < 0) return fail(BRT_E_INVALID, "bad shape T=%d E=%d P=%d", T, E, P);
  if (!mask || !cells || !indices || !loads || (!rows && P > 0)) return fail(BRT_E_INVALID, "null argument");
  if (caps == nullptr) C = 0;
  if (capacity_padding && C < 1)
    return fail(BRT_E_INVALID, "capacity_padding needs at least one supported capacity");
  if (!capacity_padding) path_wise_padding = 0;
  if (path_wise_padding && C < E)
    return fail(BRT_E_INVALID, "path_wise_padding needs one capacity per path (%d < %d)", C, E);
  if (!aligned(cells, 16) || !aligned(rows, 16))
    return fail(BRT_E_INVALID, "cells/rows must be 16-byte aligned");
  ScanGeometry g;
  if (!brt_hip_route_and_dispatch_supported(T, E, cell_bytes, C, path_wise_padding) ||
      !fused_geometry(T, E, static_cast<int>(cell_bytes / 16), &g))
    return fail(BRT_E_UNSUPPORTED,
                "route_and_dispatch takes 1..64 paths, cells of a multiple of 16 bytes, at most %d "
                "supported capacities and a batch its bands can hold (T=%d E=%d cell=%zu bytes C=%d): "
                "use brt_hip_generate_indices_and_loads + brt_hip_dispatch",
                kFusedCaps, T, E, cell_bytes, C);
  const size_t need = (static_cast<size_t>(g.bands) + 1) * E * sizeof(int);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(BRT_E_WORKSPACE, "workspace too small: %zu < %zu bytes", workspace_bytes, need);
  if (!aligned(workspace, 4)) return fail(BRT_E_INVALID, "workspace must be 4-byte aligned");
  FusedArgs f{};
  ScanArgs& a = f.s;
  a.mask = mask;
  a.out = indices;
  a.loads = loads;
  a.counts = counts;
  a.caps = caps;
  a.C = C;
  a.T = T;
  a.E = E;
  a.capacity_padding = capacity_padding;
  a.path_wise_padding = path_wise_padding;
  a.partial = static_cast<int*>(workspace);
  a.prefix_in = a.partial + static_cast<size_t>(g.bands) * E;
  a.ep_shift = g.ep_shift;
  a.rows_pw = g.rows_pw;
  a.n_ins = g.rows_pw >> (6 - g.ep_shift);
  a.bands = g.bands;
  f.src = static_cast<const u32x4*>(cells);
  f.dst = static_cast<u32x4*>(rows);
  f.row_tags = row_tags;
  f.P = P;
  f.cpr = static_cast<int>(cell_bytes / 16);
  hipStream_t st = as_stream(stream);
  const dim3 grid(g.bands);
  if (g.bands > 1) hipLaunchKernelGGL(band_count_kernel, grid, dim3(kBlock), 0, st, a);
  // rows of more than 128 bytes leave as streaming stores, shorter ones merge in the L2 (as in dispatch)
  const int units = (g.rows_pw * f.cpr + kWave - 1) / kWave;  // per lane
  auto go = [&](auto stream_t, auto nv_t) {
    hipLaunchKernelGGL((band_apply_dispatch_kernel<decltype(stream_t)::value, decltype(nv_t)::value>), grid,
                       dim3(kBlock), 0, st, f);
  };
  auto by_units = [&](auto stream_t) {
    if (units <= 8) go(stream_t, std::integral_constant<int, 8>{});
    else if (units <= 16) go(stream_t, std::integral_constant<int, 16>{});
    else go(stream_t, std::integral_constant<int, kFusedUnits>{});
  };
  if (f.cpr > 8) by_units(std::true_type{});
  else by_units(std::false_type{});
  return check_launch("band_apply_dispatch_kernel");
}

extern "C" int brt_hip_throttle_hotmask(const int32_t* mask, int32_t* out, int32_t* prefix,
                                        const int32_t* threshold, int T, int E, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  if (T < 0 || E <= 0) return fail(BRT_E_INVALID, "bad shape T=%d E=%d", T, E);
  if (T == 0) return BRT_OK;
  if (!mask || !out || !prefix || !threshold) return fail(BRT_E_INVALID, "null argument");
  if (static_cast<long>(T) * E >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*E >= 2^31");
  ScanArgs a{};
  a.mask = mask;
  a.out = out;
  a.prefix = prefix;
  a.threshold = threshold;
  a.T = T;
  a.E = E;
  return launch_scan(kThrottle, a, workspace, workspace_bytes, stream);
}

extern "C" int brt_hip_convert_index_format(const int32_t* src, int32_t* dst,
                                            const int32_t* loads, int T, int E, int tag_to_seat,
                                            void* stream) {
  if (T < 0 || E <= 0) return fail(BRT_E_INVALID, "bad shape T=%d E=%d", T, E);
  if (T == 0) return BRT_OK;
  if (!src || !dst) return fail(BRT_E_INVALID, "null argument");
  if (tag_to_seat && !loads) return fail(BRT_E_INVALID, "tag->seat conversion needs loads");
  const size_t total = static_cast<size_t>(T) * E;
  const int blocks = static_cast<int>(std::min<size_t>((total + 255) / 256, 4096));
  if (tag_to_seat)
    hipLaunchKernelGGL(tag_to_seat_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), src, dst,
                       loads, T, E);
  else
    hipLaunchKernelGGL(seat_to_tag_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), src, dst,
                       T, E);
  return check_launch("convert_index_format");
}
