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
constexpr int kWholeWaves = 8;    // a small route: one workgroup of 8 wavefronts, one launch
constexpr int kWholeChunks = 32;  // ... up to this many chunks of 64 entries
constexpr int kSplitWaves = 4;    // larger routes: workgroups of 4 wavefronts, two launches
constexpr int kSplitGroups = 32;  // ... in at most this many workgroups
constexpr int kSoloEntries = 65536;  // routes up to this many entries: one launch, every workgroup counts the whole route
constexpr int kSplitWavesLarge = 16;  // ... of 16 wavefronts for routes beyond 32768 entries
constexpr int kBatch = 4;        // chunks of 64 entries a wavefront keeps in flight
constexpr int kMaxK = 8;         // paths per cell in combine_by_rows
constexpr int kMaxRoutePaths = 512;  // (2 * kWholeWaves + 3) * E words of LDS
constexpr int kMaxCapsInLds = 1024;

struct RouteArgs {
  const int* ids;
  const int* caps;
  int* loads;
  int* counts;
  int* seat_rows;
  int* row_entries;
  int* ws;  // [groups][E] + [units][E] counters of the two-launch form
  int units;
  int n, E, C, P, bits, per_wave;
  int caps_in_lds;  // number of capacities staged in LDS (all of them, or 0)
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

// Wavefront (unit) u owns the entries [u * per_wave, (u+1) * per_wave), in chunks of 64
// (one entry per lane), kBatch chunks in flight.  Pass 1 counts entries per (wavefront, path) in
// LDS: the lanes of a chunk that hold the same path are found with one ballot per id bit, and the
// lowest of them adds their number to the wavefront's counter -- no atomics, every counter has
// one writer.  Then every wavefront sums the counters of the units before it (its first
// seat per path) while the first wavefront turns the column totals into loads and first rows.
// Pass 2 walks the entries again: seat = wavefront's running count + rank among the lanes of the
// chunk with the same path.  The first batch of ids stays in registers between the passes; the
// capacities are staged in LDS at the start, off the critical path.  The kernels are kept small
// (loops over batches and path columns are not unrolled): at a few microseconds per launch,
// fetching the code is part of the run time.
struct Batch {
  int id[kBatch];
};

__device__ __forceinline__ Batch load_batch(const int* __restrict__ ids, int c0, int hi, int lane) {
  Batch b;
#pragma unroll
  for (int q = 0; q < kBatch; ++q) {
    const int i = c0 + q * kWave + lane;
    b.id[q] = i < hi ? ids[i] : -1;
  }
  return b;
}

__device__ __forceinline__ void count_batch(const Batch& b, int c0, int hi, int lane, int E, int bits,
                                            int* mine) {
#pragma unroll
  for (int q = 0; q < kBatch; ++q) {
    if (c0 + q * kWave < hi) {  // same for the whole wavefront
      const int e = b.id[q];
      const bool valid = e >= 0 && e < E;
      const unsigned long long same = same_path_lanes(e, valid, bits);
      if (valid && (same & lanes_below(lane)) == 0) mine[e] += __popcll(same);
    }
  }
}

__device__ __forceinline__ void emit_batch(const Batch& b, int c0, int hi, int lane, const RouteArgs& a,
                                           int* mine, const int* s_kept, const int* s_start) {
#pragma unroll
  for (int q = 0; q < kBatch; ++q) {
    if (c0 + q * kWave < hi) {
      const int i = c0 + q * kWave + lane;
      const int e = b.id[q];
      const bool valid = e >= 0 && e < a.E;
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

// Sums, for the paths e = c * 64 + lane, `rows` rows of counters ([rows][E], in LDS or in
// global memory): all of them into total, those before row `mine` into before.  At most MAX rows,
// all loaded before the first is used: one memory round trip.
template <int MAX, typename Ptr>
__device__ __forceinline__ void sum_rows(Ptr cnt, int rows, int mine, int E, int e, int* before,
                                         int* total) {
  // every load is unconditional (row and path clamped into the table, the value dropped
  // afterwards): a load under a condition of its own becomes a branch, and the loads of
  // consecutive branches wait for each other
  const int col = min(e, E - 1);
  int n[MAX];
#pragma unroll
  for (int v = 0; v < MAX; ++v) n[v] = cnt[min(v, rows - 1) * E + col];
#pragma unroll
  for (int v = 0; v < MAX; ++v) {
    const int add = (v < rows && e < E) ? n[v] : 0;
    *before += v < mine ? add : 0;
    *total += add;
  }
}

// kWhole: one workgroup computes the route (small routes: one launch).  kCount + kEmit: the
// same work spread over up to kSplitGroups workgroups in two launches; a unit is a wavefront and
// its contiguous range of entries.  The counters travel through `ws`: [groups][E] sums per
// workgroup, then [units][E] per unit, so that a unit finds its first seats with one round of
// loads: the sums of the workgroups before its own plus the units before it in its own.
// kSolo: middle-sized routes in ONE launch over several workgroups.  A workgroup needs two things from
// the entries it does not own: how many of each path lie before its range (its first seats) and how
// many there are in all (loads and first rows).  Neither depends on the order of those entries, so
// every workgroup takes them from a histogram of the whole id vector (at most 256 KB, read from
// the L2) built with LDS atomics, one add per entry, instead of waiting for a counting kernel; only
// its own range is ranked with the ballots.  No workgroup waits for another.
enum RouteMode { kWhole = 0, kCount = 1, kEmit = 2, kSolo = 3 };

template <int MODE, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void route_kernel(RouteArgs a) {
  extern __shared__ int lds[];
  const int E = a.E;
  constexpr bool kOwnCounts = MODE == kWhole || MODE == kSolo;  // counters of its wavefronts stay in LDS
  int* s_cnt = lds;                                         // [WAVES][E] counters
  int* s_seat = kOwnCounts ? lds + WAVES * E : lds;         // [WAVES][E] running seats of pass 2
  int* s_load = s_seat + WAVES * E;                         // [E]
  int* s_start = s_load + E;                                // [E]
  int* s_kept = s_start + E;                                // [E] rows a path really fills
  int* s_hist = s_kept + E;                                 // kSolo: [2][E] entries before this workgroup's range / from it on
  int* s_caps = s_hist + (MODE == kSolo ? 2 * E : 0);       // [caps_in_lds]
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x >> 6;
  const int unit = blockIdx.x * WAVES + w;
  constexpr int kStep = kWave * kBatch;

  const int lo = static_cast<int>(min(static_cast<long>(a.n), static_cast<long>(unit) * a.per_wave));
  const int hi = min(a.n, lo + a.per_wave);
  // the first batch of ids is fetched once, ahead of everything else, and serves both passes
  const Batch first = load_batch(a.ids, lo, hi, lane);
  // per-unit counters lie behind the workgroup sums (two-launch form only)
  int* unit_rows = kOwnCounts ? nullptr : a.ws + static_cast<size_t>(gridDim.x) * E;
  // kEmit: the counters of the first 64 paths are fetched in the same round trip as the ids and
  // the capacities
  int before0 = 0, total0 = 0;
  if constexpr (MODE == kEmit) {
    int own = 0;  // this workgroup's total is part of the workgroup sums already
    sum_rows<kSplitGroups>(a.ws, static_cast<int>(gridDim.x), static_cast<int>(blockIdx.x), E, lane, &before0, &total0);
    sum_rows<WAVES>(unit_rows + static_cast<size_t>(blockIdx.x) * WAVES * E, WAVES, w, E, lane, &before0, &own);
  }
  if (MODE != kCount)
    for (int i = threadIdx.x; i < a.caps_in_lds; i += WAVES * kWave) s_caps[i] = a.caps[i];
  if (MODE != kEmit)
    for (int i = threadIdx.x; i < WAVES * E; i += WAVES * kWave) s_cnt[i] = 0;
  if (MODE == kSolo)
    for (int i = threadIdx.x; i < 2 * E; i += WAVES * kWave) s_hist[i] = 0;
  __syncthreads();
  const int* caps = a.caps_in_lds != 0 ? s_caps : a.caps;

  if constexpr (MODE == kSolo) {
    // histogram of every entry, split at the start of this workgroup's range: 16 ids per lane in
    // flight, one LDS add each (the adds of a wavefront to one counter are serialised by the
    // LDS, which for ids spread over the paths is a handful of passes)
    const int own_lo = static_cast<int>(min(static_cast<long>(a.n), static_cast<long>(blockIdx.x) * WAVES * a.per_wave));
    constexpr int kFlight = 8, kThreads = WAVES * kWave;
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    const bool quads = (reinterpret_cast<uintptr_t>(a.ids) & 15) == 0;  // 16-byte loads of 4 ids
    const int nq = quads ? a.n >> 2 : 0;
    const i32x4* ids4 = reinterpret_cast<const i32x4*>(a.ids);
#pragma unroll 1
    for (int base = 0; base < nq; base += kFlight * kThreads) {
      i32x4 id[kFlight];
#pragma unroll
      for (int q = 0; q < kFlight; ++q) id[q] = ids4[min(base + q * kThreads + static_cast<int>(threadIdx.x), nq - 1)];
#pragma unroll
      for (int q = 0; q < kFlight; ++q) {
        const int i4 = base + q * kThreads + threadIdx.x;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int i = i4 * 4 + c, e = id[q][c];
          if (i4 < nq && e >= 0 && e < E)
            __hip_atomic_fetch_add(&s_hist[(i < own_lo ? 0 : E) + e], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
    for (int i = nq * 4 + threadIdx.x; i < a.n; i += kThreads) {  // the tail, or everything behind a misaligned pointer
      const int e = a.ids[i];
      if (e >= 0 && e < E)
        __hip_atomic_fetch_add(&s_hist[(i < own_lo ? 0 : E) + e], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }

  if (MODE != kEmit) {
    int* mine = s_cnt + w * E;
#pragma unroll 1
    for (int c0 = lo; c0 < hi; c0 += kStep) {
      Batch b = first;
      if (c0 != lo) b = load_batch(a.ids, c0, hi, lane);
      count_batch(b, c0, hi, lane, E, a.bits, mine);
    }
  }
  if (MODE == kCount) {
    const int* mine = s_cnt + w * E;
    for (int e = lane; e < E; e += kWave) unit_rows[static_cast<size_t>(unit) * E + e] = mine[e];
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += WAVES * kWave) {
      int sum = 0;
#pragma unroll
      for (int v = 0; v < WAVES; ++v) sum += s_cnt[v * E + e];
      a.ws[static_cast<size_t>(blockIdx.x) * E + e] = sum;
    }
    return;
  }
  if (kOwnCounts) __syncthreads();

  // first seat of this unit in every path; the first wavefront also finishes the columns
  int* mine = s_seat + w * E;
  int carry = 0;
#pragma unroll 1
  for (int e0 = 0; e0 < E; e0 += kWave) {
    const int e = e0 + lane;
    int before = 0, total = 0;
    if constexpr (MODE == kWhole) {
      sum_rows<WAVES>(s_cnt, WAVES, w, E, e, &before, &total);
    } else if constexpr (MODE == kSolo) {
      int own = 0;
      sum_rows<WAVES>(s_cnt, WAVES, w, E, e, &before, &own);
      before += e < E ? s_hist[e] : 0;
      total = e < E ? s_hist[e] + s_hist[E + e] : 0;
    } else if (e0 == 0) {
      before = before0;
      total = total0;
    } else {
      int own = 0;
      sum_rows<kSplitGroups>(a.ws, static_cast<int>(gridDim.x), static_cast<int>(blockIdx.x), E, e, &before, &total);
      sum_rows<WAVES>(unit_rows + static_cast<size_t>(blockIdx.x) * WAVES * E, WAVES, w, E, e, &before, &own);
    }
    if (e < E) mine[e] = before;
    if (w == 0) {
      const int load = e < E ? finalize_load(total, caps, a.C, a.capacity_padding, a.path_wise_padding, e) : 0;
      const int incl = wave_inclusive_scan(load);
      if (e < E) {
        s_load[e] = load;
        s_kept[e] = min(total, a.max_path_load != 0 ? min(load, a.max_path_load) : load);
        s_start[e] = a.max_path_load != 0 ? e * a.max_path_load : carry + incl - load;
        if (blockIdx.x == 0) {
          a.loads[e] = load;
          if (a.counts) a.counts[e] = total;
        }
      }
      carry += __shfl(incl, kWave - 1, kWave);
    }
  }
  __syncthreads();  // loads and first rows are in place

#pragma unroll 1
  for (int c0 = lo; c0 < hi; c0 += kStep) {
    Batch b = first;
    if (c0 != lo) b = load_batch(a.ids, c0, hi, lane);
    emit_batch(b, c0, hi, lane, a, mine, s_kept, s_start);
  }

  // padding rows: between the rows a path filled and the first row of the next path, and
  // behind the last path
  const int all_units = gridDim.x * WAVES;
  for (int e = unit; e < E; e += all_units) {
    const int from = s_start[e] + s_kept[e];
    const int end = min(a.P, a.max_path_load != 0 ? s_start[e] + a.max_path_load : s_start[e] + s_load[e]);
    for (int r = from + lane; r < end; r += kWave) a.row_entries[r] = 0;
  }
  const int rows = a.max_path_load != 0 ? E * a.max_path_load : s_start[E - 1] + s_load[E - 1];
  for (long r = static_cast<long>(rows) + unit * kWave + lane; r < a.P; r += static_cast<long>(all_units) * kWave)
    a.row_entries[r] = 0;
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
            // The product is an fp32 product, then rounded to the data type.  The empty asm keeps
            // it one: multiply and conversion to fp16 would otherwise be merged into a
            // mixed-precision instruction that rounds the exact product once, which differs from
            // the fp32 product in the last bit now and then (and has no bf16 counterpart).
#pragma unroll
            for (int q = 0; q < NE; ++q) {
              x[q] = x[q] * g;
              asm volatile("" : "+v"(x[q]));
            }
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
// KMAX >= k entries per cell are held in registers and sorted by path id (entries without a row
// last), so the row loads of a cell do not depend on each other.
template <int IN_DT, int OUT_DT, int LS, int UPR, int KMAX>
__global__ __launch_bounds__(kBlock) void combine_by_rows_kernel(RowsArgs a) {
  using U = u32x4;
  constexpr int NE = 16 / elem_bytes(IN_DT);
  constexpr int OUT_BYTES = NE * elem_bytes(OUT_DT);
  constexpr int LPR = 1 << LS;
  constexpr int GROUPS = kWave >> LS;
  constexpr int kNone = 0x7fffffff;
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
    // Entries of the cell: independent loads, one memory round trip before the rows can be
    // fetched.  Every load is unconditional (cell and entry clamped into the tables, the value
    // dropped afterwards): loads under conditions of their own become branches that wait for
    // each other.
    const size_t slot0 = static_cast<size_t>(min(t0 + i, static_cast<long>(a.T) - 1)) * k;
    int id[KMAX], row[KMAX];
    float g[KMAX];
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
      const int jj = min(j, k - 1);
      row[j] = a.seat_rows[slot0 + jj];
      id[j] = a.ids[slot0 + jj];
    }
    if (a.weights != nullptr) {
#pragma unroll
      for (int j = 0; j < KMAX; ++j) g[j] = a.weights[slot0 + min(j, k - 1)];
    } else {
#pragma unroll
      for (int j = 0; j < KMAX; ++j) g[j] = 1.0f;
    }
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
      if (!live || j >= k || row[j] < 1 || row[j] > a.P) id[j] = kNone;
    }
    // ascending path id by odd-even transposition (stable: of two entries that name the same
    // path the first stays first, and only it is used)
#pragma unroll
    for (int round = 0; round < KMAX; ++round) {
#pragma unroll
      for (int j = round & 1; j + 1 < KMAX; j += 2) {
        const bool swap = id[j] > id[j + 1];
        const int ti = id[j], tr = row[j];
        const float tg = g[j];
        id[j] = swap ? id[j + 1] : ti;
        row[j] = swap ? row[j + 1] : tr;
        g[j] = swap ? g[j + 1] : tg;
        id[j + 1] = swap ? ti : id[j + 1];
        row[j + 1] = swap ? tr : row[j + 1];
        g[j + 1] = swap ? tg : g[j + 1];
      }
    }
    bool use[KMAX];
#pragma unroll
    for (int j = 0; j < KMAX; ++j) use[j] = id[j] != kNone && (j == 0 || id[j] != id[j - 1]);
    const size_t to = static_cast<size_t>(t0 + i) * cpr;
    for (int off0 = 0; off0 < cpr; off0 += LPR * UPR) {
      float acc[UPR][NE];
#pragma unroll
      for (int u = 0; u < UPR; ++u)
#pragma unroll
        for (int q = 0; q < NE; ++q) acc[u][q] = 0.0f;
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        U val[UPR];
#pragma unroll
        for (int u = 0; u < UPR; ++u) {
          const int off = off0 + u * LPR + glane;
          if (use[j] && off < cpr) val[u] = src[static_cast<size_t>(row[j] - 1) * cpr + off];
        }
#pragma unroll
        for (int u = 0; u < UPR; ++u) {
          const int off = off0 + u * LPR + glane;
          if (use[j] && off < cpr) {
            float x[NE];
            unpack<IN_DT, 16>(val[u], x);
#pragma unroll
            for (int q = 0; q < NE; ++q) acc[u][q] = acc[u][q] + x[q] * g[j];
          }
        }
      }
      if constexpr (IN_DT != OUT_DT && LS == 6) {
        // 16-bit rows into an fp32 result, a whole wavefront per row: whole-line streaming stores
        const bool row_ok = live && (use[0] || !a.is_residual);  // the same for the whole wavefront
#pragma unroll
        for (int u = 0; u < UPR; ++u)
          store_widened_spread(dst + to * OUT_BYTES, off0 + u * LPR, cpr, row_ok, acc[u]);
      } else if (live && (use[0] || !a.is_residual)) {
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

namespace {

// Wavefronts per workgroup, units and entries per unit of the two-launch form: at most
// kSplitGroups workgroups, of 4 wavefronts while that keeps a unit within one batch of chunks, of
// 16 beyond.
void split_geometry(int n, int* waves, int* units, int* per_wave) {
  const int chunks = (n + kWave - 1) / kWave;
  *waves = chunks <= kSplitGroups * kSplitWaves * kBatch ? kSplitWaves : kSplitWavesLarge;
  const int most = kSplitGroups * *waves;
  const int chunks_pw = std::max(1, (chunks + most - 1) / most);
  const int used = (chunks + chunks_pw - 1) / chunks_pw;
  *units = (used + *waves - 1) / *waves * *waves;
  *per_wave = chunks_pw * kWave;
}

}  // namespace

extern "C" size_t brt_hip_route_by_path_workspace_bytes(int T, int k, int E) {
  if (T <= 0 || k <= 0 || E <= 0 || static_cast<long>(T) * k >= (1l << 31)) return 0;
  int waves, units, per_wave;
  split_geometry(T * k, &waves, &units, &per_wave);
  return static_cast<size_t>(units / waves + units) * E * sizeof(int);
}

extern "C" int brt_hip_route_by_path(const int32_t* path_ids, int T, int k, int E, const int32_t* caps,
                                     int C, int capacity_padding, int path_wise_padding,
                                     int max_path_load, int32_t* loads, int32_t* counts,
                                     int32_t* seat_rows, int32_t* row_entries, int P,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  if (T < 0 || k < 0 || E <= 0 || P < 0 || max_path_load < 0)
    return fail(BRT_E_INVALID, "bad shape T=%d k=%d E=%d P=%d", T, k, E, P);
  if (E > kMaxRoutePaths) return fail(BRT_E_UNSUPPORTED, "more than %d paths", kMaxRoutePaths);
  if (static_cast<long>(T) * k >= (1l << 31)) return fail(BRT_E_UNSUPPORTED, "T*k >= 2^31");
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
  a.caps_in_lds = C <= kMaxCapsInLds ? C : 0;
  hipStream_t st = as_stream(stream);
  const int chunks = (n + kWave - 1) / kWave;
  if (chunks <= kWholeChunks) {
    a.per_wave = (chunks + kWholeWaves - 1) / kWholeWaves * kWave;
    const size_t lds_bytes = (static_cast<size_t>(2 * kWholeWaves + 3) * E + a.caps_in_lds) * sizeof(int);
    hipLaunchKernelGGL((route_kernel<kWhole, kWholeWaves>), dim3(1), dim3(kWholeWaves * kWave), lds_bytes, st, a);
    return check_launch("route_kernel");
  }
  if (n <= kSoloEntries) {
    // one launch: workgroups of 4 wavefronts, each wavefront a whole number of chunks of its own
    const int groups = std::min(kSplitGroups, (chunks + kSplitWaves - 1) / kSplitWaves);
    a.per_wave = (chunks + groups * kSplitWaves - 1) / (groups * kSplitWaves) * kWave;
    const size_t lds_bytes = (static_cast<size_t>(2 * kSplitWaves + 5) * E + a.caps_in_lds) * sizeof(int);
    hipLaunchKernelGGL((route_kernel<kSolo, kSplitWaves>), dim3(groups), dim3(kSplitWaves * kWave), lds_bytes, st, a);
    return check_launch("route_kernel");
  }
  int waves;
  split_geometry(n, &waves, &a.units, &a.per_wave);
  const size_t need = static_cast<size_t>(a.units / waves + a.units) * E * sizeof(int);
  if (workspace == nullptr || workspace_bytes < need || !aligned(workspace, 4))
    return fail(BRT_E_WORKSPACE, "route_by_path needs %zu bytes of workspace, got %zu", need, workspace_bytes);
  a.ws = static_cast<int*>(workspace);
  const dim3 grid(a.units / waves), block(waves * kWave);
  const size_t lds_bytes = (static_cast<size_t>(waves + 3) * E + a.caps_in_lds) * sizeof(int);
  if (waves == kSplitWaves) {
    hipLaunchKernelGGL((route_kernel<kCount, kSplitWaves>), grid, block, lds_bytes, st, a);
    hipLaunchKernelGGL((route_kernel<kEmit, kSplitWaves>), grid, block, lds_bytes, st, a);
  } else {
    hipLaunchKernelGGL((route_kernel<kCount, kSplitWavesLarge>), grid, block, lds_bytes, st, a);
    hipLaunchKernelGGL((route_kernel<kEmit, kSplitWavesLarge>), grid, block, lds_bytes, st, a);
  }
  return check_launch("route_kernel");
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
#define BRT_LAUNCH_K(IN, OUT, KMAX)                                                                          \
  with_row_shape(a.cpr, [&](auto ls, auto upr) {                                                             \
    hipLaunchKernelGGL((combine_by_rows_kernel<IN, OUT, decltype(ls)::value, decltype(upr)::value, KMAX>),   \
                       grid, block, 0, st, a);                                                               \
  });
#define BRT_LAUNCH(IN, OUT)                 \
  if (k == 1) BRT_LAUNCH_K(IN, OUT, 1)      \
  else if (k == 2) BRT_LAUNCH_K(IN, OUT, 2) \
  else BRT_LAUNCH_K(IN, OUT, kMaxK)
  if (in_dtype == BRT_F32) BRT_LAUNCH(BRT_F32, BRT_F32)
  else if (in_dtype == BRT_F16 && out_dtype == BRT_F16) BRT_LAUNCH(BRT_F16, BRT_F16)
  else if (in_dtype == BRT_F16) BRT_LAUNCH(BRT_F16, BRT_F32)
  else if (out_dtype == BRT_BF16) BRT_LAUNCH(BRT_BF16, BRT_BF16)
  else BRT_LAUNCH(BRT_BF16, BRT_F32)
#undef BRT_LAUNCH
#undef BRT_LAUNCH_K
  return check_launch("combine_by_rows_kernel");
}
