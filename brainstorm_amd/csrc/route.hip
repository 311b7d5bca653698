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

#include <type_traits>

#include "common.hpp"
#include "rows.hpp"

namespace brt {
namespace {

constexpr int kBlock = 256;

// ------------------------------------------------------- wave-level plumbing
// Every wavefront works on its own: it owns `rows_pw` consecutive rows of the
// index matrix, keeps its tables in a private slice of LDS and never meets a
// block barrier.  LDS traffic of one wavefront is executed in order, so a
// wave-scope fence between the "write list" and "read list" phases is all the
// synchronisation that is needed.
constexpr int kSteps = 8;  // index words fetched per lane before any is used

__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// How one wave-wide load of 64 index words maps to (row, path): for E <= 64 a
// step covers 64/ep whole rows (ep = E rounded up to a power of two, lanes
// beyond E idle); for E > 64 a row takes ceil(E/64) steps.
struct StepMap {
  int ep_shift;  // log2(ep), E <= 64 only
  int chunks;    // steps per row, E > 64 only (1 otherwise)
  int E;
  __device__ __forceinline__ int rows_per_step() const { return E <= kWave ? kWave >> ep_shift : 1; }
  __device__ __forceinline__ int steps(int rows) const {
    return E <= kWave ? (rows + rows_per_step() - 1) >> (6 - ep_shift) : rows * chunks;
  }
  // row (relative) and path handled by `lane` in `step`; path >= E means idle
  __device__ __forceinline__ void locate(int step, int lane, int& row, int& e) const {
    if (E <= kWave) {
      row = step * rows_per_step() + (lane >> ep_shift);
      e = lane & ((1 << ep_shift) - 1);
    } else {
      row = step / chunks;
      e = (step - row * chunks) * kWave + lane;
    }
  }
  // lanes that belong to the same row as `lane` within a step
  __device__ __forceinline__ unsigned long long segment(int lane) const {
    if (E > kWave || ep_shift == 6) return ~0ull;
    const int ep = 1 << ep_shift;
    return ((1ull << ep) - 1ull) << ((lane >> ep_shift) * ep);
  }
};

// Per-wave copy of loads[] and the path start offsets (exclusive prefix of the
// loads, or e*stride for fixed-stride layouts).
__device__ __forceinline__ void wave_path_tables(const int* __restrict__ loads, int* s_loads,
                                                 int* s_start, int E, int stride, int lane) {
  int carry = 0;
  for (int base = 0; base < E; base += kWave) {
    const int e = base + lane;
    int v = e < E ? loads[e] : 0;
    // fixed stride: a path's block ends at the stride, seats beyond it are dropped (the reference
    // would write them into the next path's block, racing with that path's own rows)
    if (stride != 0) v = min(v, stride);
    const int incl = wave_inclusive_scan(v);
    if (e < E) {
      s_loads[e] = v;
      s_start[e] = stride != 0 ? e * stride : carry + incl - v;
    }
    carry += __shfl(incl, kWave - 1, kWave);
  }
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
  int cpr;      // units (BYTES each) per row
  int rows_pw;  // rows of the index matrix per wavefront
  int lds_pw;   // ints of LDS per wavefront
  StepMap map;
  int is_1d, is_tag_index;
};

// DT < 0: unweighted byte copy; otherwise rows are scaled by the gate in DT.
// This wavefront's share [z0, z1) of Z items dealt evenly to n_waves wavefronts (the first
// Z % n_waves of them take one more).  No division when there is nothing to share -- the usual
// case, a route without padding rows -- and a 32-bit one otherwise: this runs at the end of every
// wavefront's life, where a pair of 64-bit divisions was a third of a microsecond of the kernel.
__device__ __forceinline__ void even_share(long Z, long wave, long n_waves, long* z0, long* z1) {
  *z0 = *z1 = 0;
  if (Z <= 0) return;
  const unsigned nw = static_cast<unsigned>(n_waves), w = static_cast<unsigned>(wave);
  const unsigned q = static_cast<unsigned>(Z) / nw, r = static_cast<unsigned>(Z) % nw;
  *z0 = static_cast<long>(q) * w + min(w, r);
  *z1 = *z0 + q + (w < r ? 1 : 0);
}

template <int BYTES, int DT>
__global__ __launch_bounds__(kBlock) void dispatch_kernel(DispatchArgs a) {
  using U = typename Unit<BYTES>::type;
  extern __shared__ int smem[];
  const int E = a.E;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave_in_block = threadIdx.x >> 6;
  const int waves_pb = blockDim.x >> 6;
  const long wave = static_cast<long>(blockIdx.x) * waves_pb + wave_in_block;
  const long n_waves = static_cast<long>(gridDim.x) * waves_pb;
  int* s_loads = smem + wave_in_block * a.lds_pw;
  int* s_start = s_loads + E;
  int* s_zstart = s_start + E;  // E + 1 entries: padding rows before path e
  int* s_dst = s_zstart + E + 1;
  int* s_src = s_dst + a.rows_pw * E;
  float* s_gate = reinterpret_cast<float*>(s_src + a.rows_pw * E);
  const unsigned long long lt = (1ull << lane) - 1ull;

  const long r0 = wave * a.rows_pw;
  const int nr = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - r0)));
  const int* __restrict__ idx0 = a.idx + r0 * E;
  const int n_steps = a.map.steps(nr);

  // ---- 1. fetch the first batch of index words, then build the path tables ------
  int v[kSteps];
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    int row, e;
    a.map.locate(j, lane, row, e);
    v[j] = (j < n_steps && row < nr && e < E) ? idx0[row * E + e] : 0;
  }
  wave_path_tables(a.loads, s_loads, s_start, E, a.mpl, lane);
  if (a.counts != nullptr) {
    int carry = 0;
    for (int base = 0; base < E; base += kWave) {
      const int e = base + lane;
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
    if (lane == 0) s_zstart[E] = carry;
  }
  wave_sync();

  // ---- 2. index words -> compact list of (destination row, source row, gate) -----
  int n = 0;
  for (int s0 = 0; s0 < n_steps; s0 += kSteps) {
    if (s0 > 0) {
#pragma unroll
      for (int j = 0; j < kSteps; ++j) {
        int row, e;
        a.map.locate(s0 + j, lane, row, e);
        v[j] = (s0 + j < n_steps && row < nr && e < E) ? idx0[row * E + e] : 0;
      }
    }
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      if (s0 + j < n_steps) {  // wave-uniform
        int row, e;
        a.map.locate(s0 + j, lane, row, e);
        bool ok = false;
        int dst_row = 0, tok = 0;
        if (row < nr && e < E) {
          const long r = r0 + row;
          if (!a.is_tag_index) {  // v = seat of token r on path e
            ok = v[j] >= 1 && v[j] <= s_loads[e];
            dst_row = s_start[e] + v[j] - 1;
            tok = static_cast<int>(r);
          } else {  // v = 1-based token held by slot r of path e
            ok = r < s_loads[e] && v[j] >= 1 && v[j] <= a.T;
            dst_row = s_start[e] + static_cast<int>(r);
            tok = v[j] - 1;
            // the reference walks slots r, r+512, ... per block and stops at the
            // first empty one (route.cu:84-92): an empty slot above hides r
            if (ok)
              for (long k = r - 512; k >= 0; k -= 512)
                if (a.idx[k * E + e] == 0) {
                  ok = false;
                  break;
                }
          }
          ok = ok && dst_row >= 0 && dst_row < a.P;
        }
        const unsigned long long m = __ballot(ok);
        if (ok) {
          const int pos = n + __popcll(m & lt);
          s_dst[pos] = dst_row;
          s_src[pos] = a.is_1d ? tok : tok * E + e;
          if constexpr (DT >= 0)
            s_gate[pos] = load_gate(a.gates, DT, static_cast<size_t>(tok) * E + e);
          if (a.new_tags != nullptr) a.new_tags[dst_row] = a.old_tags ? a.old_tags[tok] : tok + 1;
        }
        n += __popcll(m);
      }
    }
  }
  wave_sync();

  // ---- 3. move rows: flat loop over (entry, unit) pairs, loads first ---------------
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  U* __restrict__ dst = static_cast<U*>(a.dst);
  int ent = lane / cpr, off = lane - ent * cpr;
  const int d_ent = kWave / cpr, d_off = kWave - d_ent * cpr;
  while (ent < n) {
    U val[kSteps];
    size_t to[kSteps];
    float g[kSteps];
    bool live[kSteps];
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
      live[u] = ent < n;
      if (live[u]) {
        val[u] = src[static_cast<size_t>(s_src[ent]) * cpr + off];
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
    for (int u = 0; u < kSteps; ++u) {
      if (live[u]) {
        if constexpr (DT >= 0) {
          constexpr int NE = BYTES / elem_bytes(DT);
          float x[NE];
          unpack<DT, BYTES>(val[u], x);
#pragma unroll
          for (int i = 0; i < NE; ++i) x[i] = x[i] * g[u];
          pack_store<DT, NE>(dst + to[u], x);
        } else {
          dst[to[u]] = val[u];
        }
      }
    }
  }

  // ---- 4. zero-fill this wavefront's share of the padding rows ---------------------
  if (a.counts != nullptr) {
    const long Z = s_zstart[E];
    long z0, z1;
    even_share(Z, wave, n_waves, &z0, &z1);
    for (long z = z0; z < z1; ++z) {
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
  int rows_pw;  // tokens per wavefront
  int lds_pw;   // ints of LDS per wavefront
  StepMap map;
  int is_residual, gate_dtype;
};

template <int BYTES, int IN_DT, int OUT_DT>
__global__ __launch_bounds__(kBlock) void combine_kernel(CombineArgs a) {
  using U = typename Unit<BYTES>::type;
  constexpr int NE = BYTES / elem_bytes(IN_DT);
  constexpr int OUT_BYTES = NE * elem_bytes(OUT_DT);
  constexpr int kAcc = 4;  // (token, unit) pairs accumulated concurrently per lane
  extern __shared__ int smem[];
  const int E = a.E;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave_in_block = threadIdx.x >> 6;
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block;
  int* s_loads = smem + wave_in_block * a.lds_pw;
  int* s_start = s_loads + E;
  int* s_cnt = s_start + E;          // valid routes per token
  int* s_row = s_cnt + a.rows_pw;    // [rows_pw][E] source rows, ascending path order
  float* s_gate = reinterpret_cast<float*>(s_row + a.rows_pw * E);
  const unsigned long long lt = (1ull << lane) - 1ull;
  const unsigned long long seg = a.map.segment(lane);

  const long t0 = wave * a.rows_pw;
  const int nt = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - t0)));
  if (nt == 0) return;
  const int* __restrict__ idx0 = a.idx + t0 * E;
  const int n_steps = a.map.steps(nt);

  int v[kSteps];
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    int row, e;
    a.map.locate(j, lane, row, e);
    v[j] = (j < n_steps && row < nt && e < E) ? idx0[row * E + e] : 0;
  }
  wave_path_tables(a.loads, s_loads, s_start, E, a.mpl, lane);
  wave_sync();

  // ---- per token: valid (source row, gate) in ascending path order ---------------
  // lanes = paths; __ballot + popcount compacts the valid ones without reordering
  for (int s0 = 0; s0 < n_steps; s0 += kSteps) {
    if (s0 > 0) {
#pragma unroll
      for (int j = 0; j < kSteps; ++j) {
        int row, e;
        a.map.locate(s0 + j, lane, row, e);
        v[j] = (s0 + j < n_steps && row < nt && e < E) ? idx0[row * E + e] : 0;
      }
    }
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      if (s0 + j < n_steps) {  // wave-uniform
        int row, e;
        a.map.locate(s0 + j, lane, row, e);
        bool ok = false;
        int src_row = 0;
        if (row < nt && e < E) {
          src_row = s_start[e] + v[j] - 1;
          ok = v[j] >= 1 && v[j] <= s_loads[e] && src_row < a.P;
        }
        const unsigned long long m = __ballot(ok) & seg;
        if (row < nt) {
          // a row wider than one step continues where its previous step stopped
          const int base = (E > kWave && e >= kWave) ? s_cnt[row] : 0;
          if (ok) {
            const int pos = base + __popcll(m & lt);
            s_row[row * E + pos] = src_row;
            s_gate[row * E + pos] =
                a.gates ? load_gate(a.gates, a.gate_dtype, static_cast<size_t>(t0 + row) * E + e)
                        : 1.0f;
          }
          wave_sync();
          if ((e & (kWave - 1)) == 0 || (E <= kWave && e == 0)) s_cnt[row] = base + __popcll(m);
        }
      }
    }
  }
  wave_sync();

  // ---- gather + fp32 accumulate, flat loop over (token, unit) pairs -----------------
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  char* __restrict__ dst = static_cast<char*>(a.dst);
  int tl = lane / cpr, off = lane - tl * cpr;
  const int d_tl = kWave / cpr, d_off = kWave - d_tl * cpr;
  while (tl < nt) {
    float acc[kAcc][NE];
    int n[kAcc], tok[kAcc], o[kAcc];
    int nmax = 0;
#pragma unroll
    for (int u = 0; u < kAcc; ++u) {
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
      U val[kAcc];
      float g[kAcc];
#pragma unroll
      for (int u = 0; u < kAcc; ++u)
        if (k < n[u]) {
          val[u] = src[static_cast<size_t>(s_row[tok[u] * E + k]) * cpr + o[u]];
          g[u] = s_gate[tok[u] * E + k];
        }
#pragma unroll
      for (int u = 0; u < kAcc; ++u)
        if (k < n[u]) {
          float x[NE];
          unpack<IN_DT, BYTES>(val[u], x);
          // one rounding for the product, one for the sum (no fused multiply-add)
#pragma unroll
          for (int i = 0; i < NE; ++i) acc[u][i] = acc[u][i] + x[i] * g[u];
        }
    }
#pragma unroll
    for (int u = 0; u < kAcc; ++u) {
      // n < 0: past the end; n == 0: token without a valid route
      if (n[u] > 0 || (n[u] == 0 && !a.is_residual)) {
        const size_t at = (static_cast<size_t>(t0 + tok[u]) * cpr + o[u]) * OUT_BYTES;
        pack_store<OUT_DT, NE>(dst + at, acc[u]);
      }
    }
  }
}

// ------------------------------------------------ fast path: E <= 64 paths
// With at most 64 paths one wave-wide load covers whole rows of the index
// matrix and everything stays in registers: lane e holds loads[e] and the start
// offset of path e (DPP prefix scan), __ballot marks the valid (row, path)
// pairs, and the wavefront walks the set bits, broadcasting destination/source
// row and gate with v_readlane while all 64 lanes move the row.  No LDS, no
// barrier; `kInFlight` 16-byte accesses per lane are issued before the first
// store.
constexpr int kInFlight = 8;

struct SmallTables {
  int load_e, start_e;  // of the path this lane looks at (e = lane % ep)
  int my_load, my_start;  // of path `lane`
};

__device__ __forceinline__ SmallTables small_tables(const int* __restrict__ loads, int E, int mpl,
                                                    int ep_shift, int lane) {
  SmallTables t;
  t.my_load = lane < E ? loads[lane] : 0;
  if (mpl != 0) t.my_load = min(t.my_load, mpl);  // fixed stride: a path's block ends at the stride
  const int incl = wave_inclusive_scan(t.my_load);
  t.my_start = mpl != 0 ? lane * mpl : incl - t.my_load;
  if (ep_shift == 6) {
    t.load_e = t.my_load;
    t.start_e = t.my_start;
  } else {
    const int e = lane & ((1 << ep_shift) - 1);
    t.load_e = __shfl(t.my_load, e, kWave);
    t.start_e = __shfl(t.my_start, e, kWave);
  }
  return t;
}

// UPR = 16-byte units each lane moves per row and pass (rows of up to 64*UPR
// units take one pass); kInFlight/UPR rows are in flight together.
template <int BYTES, int DT, int UPR>
__global__ __launch_bounds__(kBlock) void dispatch_small_kernel(DispatchArgs a) {
  using U = typename Unit<BYTES>::type;
  constexpr int G = kInFlight / UPR;
  const int E = a.E;
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const long n_waves = static_cast<long>(gridDim.x) * (blockDim.x >> 6);
  const int ep_shift = a.map.ep_shift;
  const int rps = kWave >> ep_shift;  // rows per step
  const int e = lane & ((1 << ep_shift) - 1);
  const int sub = lane >> ep_shift;

  const long r0 = wave * a.rows_pw;
  const int nr = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - r0)));
  const int n_steps = (nr + rps - 1) >> (6 - ep_shift);
  const int* __restrict__ idx0 = a.idx + r0 * E;
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  U* __restrict__ dst = static_cast<U*>(a.dst);

  int v_next = (n_steps > 0 && sub < nr && e < E) ? idx0[sub * E + e] : 0;
  const SmallTables tab = small_tables(a.loads, E, a.mpl, ep_shift, lane);

  for (int step = 0; step < n_steps; ++step) {
    const int v = v_next;
    const int row = step * rps + sub;
    {  // prefetch the next step's index words before the rows of this one move
      const int nrow = row + rps;
      v_next = (step + 1 < n_steps && nrow < nr && e < E) ? idx0[nrow * E + e] : 0;
    }
    bool ok = false;
    int dst_row = 0, src_row = 0;
    float gate = 1.0f;
    if (row < nr && e < E) {
      const long r = r0 + row;
      int tok;
      if (!a.is_tag_index) {  // v = seat of token r on path e
        ok = v >= 1 && v <= tab.load_e;
        dst_row = tab.start_e + v - 1;
        tok = static_cast<int>(r);
      } else {  // v = 1-based token held by slot r of path e
        ok = r < tab.load_e && v >= 1 && v <= a.T;
        dst_row = tab.start_e + static_cast<int>(r);
        tok = v - 1;
        if (ok)  // stop rule of the reference, see dispatch_kernel
          for (long k = r - 512; k >= 0; k -= 512)
            if (a.idx[k * E + e] == 0) {
              ok = false;
              break;
            }
      }
      ok = ok && dst_row >= 0 && dst_row < a.P;
      if (ok) {
        src_row = a.is_1d ? tok : tok * E + e;
        if constexpr (DT >= 0) gate = load_gate(a.gates, DT, static_cast<size_t>(tok) * E + e);
        if (a.new_tags != nullptr) a.new_tags[dst_row] = a.old_tags ? a.old_tags[tok] : tok + 1;
      }
    }
    unsigned long long m = __ballot(ok);
    while (m != 0) {  // wave-uniform: up to G rows per trip
      int d[G], sr[G];
      float g[G];
      int nb = 0;
#pragma unroll
      for (int i = 0; i < G; ++i) {
        d[i] = 0; sr[i] = 0; g[i] = 1.0f;
        if (m != 0) {
          const int b = __builtin_ctzll(m);
          m &= m - 1;
          d[i] = read_lane(dst_row, b);
          sr[i] = read_lane(src_row, b);
          if constexpr (DT >= 0) g[i] = read_lane(gate, b);
          nb = i + 1;
        }
      }
      for (int off0 = 0; off0 < cpr; off0 += kWave * UPR) {
        U val[G][UPR];
#pragma unroll
        for (int i = 0; i < G; ++i)
#pragma unroll
          for (int u = 0; u < UPR; ++u) {
            const int off = off0 + u * kWave + lane;
            if (i < nb && off < cpr) val[i][u] = src[static_cast<size_t>(sr[i]) * cpr + off];
          }
#pragma unroll
        for (int i = 0; i < G; ++i)
#pragma unroll
          for (int u = 0; u < UPR; ++u) {
            const int off = off0 + u * kWave + lane;
            if (i < nb && off < cpr) {
              U* to = dst + static_cast<size_t>(d[i]) * cpr + off;
              if constexpr (DT >= 0) {
                constexpr int NE = BYTES / elem_bytes(DT);
                float x[NE];
                unpack<DT, BYTES>(val[i][u], x);
#pragma unroll
                for (int q = 0; q < NE; ++q) x[q] = x[q] * g[i];
                pack_store<DT, NE>(to, x);
              } else {
                *to = val[i][u];
              }
            }
          }
      }
    }
  }

  // ---- zero-fill this wavefront's share of the padding rows ------------------------
  if (a.counts != nullptr) {
    int z = 0;
    if (lane < E) {
      const int alloc = a.mpl != 0 ? a.mpl : tab.my_load;
      const int filled = max(0, min(min(a.counts[lane], tab.my_load), alloc));
      z = max(0, alloc - filled);
    }
    const int z_incl = wave_inclusive_scan(z);
    const long Z = read_lane(z_incl, kWave - 1);
    long z0, z1;
    even_share(Z, wave, n_waves, &z0, &z1);
    for (long zi = z0; zi < z1; ++zi) {
      // path of padding row zi: first lane whose inclusive count exceeds zi
      const int pe = __builtin_ctzll(__ballot(z_incl > zi));
      const int pad = read_lane(z, pe);
      const int alloc = a.mpl != 0 ? a.mpl : read_lane(tab.my_load, pe);
      const long row = static_cast<long>(read_lane(tab.my_start, pe)) + (alloc - pad) +
                       (zi - (read_lane(z_incl, pe) - pad));
      if (row < a.P) {
        for (int o = lane; o < cpr; o += kWave) dst[static_cast<size_t>(row) * cpr + o] = zero_unit<BYTES>();
        if (a.new_tags != nullptr && lane == 0) a.new_tags[row] = 0;
      }
    }
  }
}

template <int BYTES, int IN_DT, int OUT_DT, int UPR>
__global__ __launch_bounds__(kBlock) void combine_small_kernel(CombineArgs a) {
  using U = typename Unit<BYTES>::type;
  constexpr int NE = BYTES / elem_bytes(IN_DT);
  constexpr int OUT_BYTES = NE * elem_bytes(OUT_DT);
  constexpr int G = 4 / UPR;  // tokens accumulated together (UPR <= 4)
  const int E = a.E;
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int ep_shift = a.map.ep_shift;
  const int ep = 1 << ep_shift;
  const int rps = kWave >> ep_shift;  // tokens per step
  const int e = lane & (ep - 1);
  const int sub = lane >> ep_shift;
  const unsigned long long seg0 = ep == kWave ? ~0ull : ((1ull << ep) - 1ull);

  const long t0 = wave * a.rows_pw;
  const int nt = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - t0)));
  if (nt == 0) return;
  const int n_steps = (nt + rps - 1) >> (6 - ep_shift);
  const int* __restrict__ idx0 = a.idx + t0 * E;
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  char* __restrict__ dst = static_cast<char*>(a.dst);

  int v_next = (sub < nt && e < E) ? idx0[sub * E + e] : 0;
  const SmallTables tab = small_tables(a.loads, E, a.mpl, ep_shift, lane);

  for (int step = 0; step < n_steps; ++step) {
    const int v = v_next;
    const int row = step * rps + sub;
    {
      const int nrow = row + rps;
      v_next = (step + 1 < n_steps && nrow < nt && e < E) ? idx0[nrow * E + e] : 0;
    }
    bool ok = false;
    int src_row = 0;
    float gate = 1.0f;
    if (row < nt && e < E) {
      src_row = tab.start_e + v - 1;
      ok = v >= 1 && v <= tab.load_e && src_row < a.P;
      if (ok && a.gates != nullptr)
        gate = load_gate(a.gates, a.gate_dtype, static_cast<size_t>(t0 + row) * E + e);
    }
    // bit (i*ep + e) set <=> token i of this step has a valid route on path e;
    // walking a token's bits from the lowest keeps the ascending path order
    const unsigned long long m = __ballot(ok);
    const int tokens = min(rps, nt - step * rps);
    for (int tg = 0; tg < tokens; tg += G) {
      unsigned long long rem0[G];
      int kmax = 0;
#pragma unroll
      for (int i = 0; i < G; ++i) {
        rem0[i] = (tg + i < tokens) ? ((m >> ((tg + i) * ep)) & seg0) << ((tg + i) * ep) : 0ull;
        kmax = max(kmax, static_cast<int>(__popcll(rem0[i])));
      }
      for (int off0 = 0; off0 < cpr; off0 += kWave * UPR) {
        float acc[G][UPR][NE];
#pragma unroll
        for (int i = 0; i < G; ++i)
#pragma unroll
          for (int u = 0; u < UPR; ++u)
#pragma unroll
            for (int q = 0; q < NE; ++q) acc[i][u][q] = 0.0f;
        unsigned long long rem[G];
#pragma unroll
        for (int i = 0; i < G; ++i) rem[i] = rem0[i];
        for (int k = 0; k < kmax; ++k) {
          U val[G][UPR];
          float g[G];
          bool live[G];
#pragma unroll
          for (int i = 0; i < G; ++i) {
            live[i] = rem[i] != 0;
            g[i] = 1.0f;
            if (live[i]) {
              const int b = __builtin_ctzll(rem[i]);
              rem[i] &= rem[i] - 1;
              const int sr = read_lane(src_row, b);
              g[i] = read_lane(gate, b);
#pragma unroll
              for (int u = 0; u < UPR; ++u) {
                const int off = off0 + u * kWave + lane;
                if (off < cpr) val[i][u] = src[static_cast<size_t>(sr) * cpr + off];
              }
            }
          }
#pragma unroll
          for (int i = 0; i < G; ++i)
            if (live[i]) {
#pragma unroll
              for (int u = 0; u < UPR; ++u) {
                const int off = off0 + u * kWave + lane;
                if (off < cpr) {
                  float x[NE];
                  unpack<IN_DT, BYTES>(val[i][u], x);
                  // one rounding for the product, one for the sum (no fused multiply-add)
#pragma unroll
                  for (int q = 0; q < NE; ++q) acc[i][u][q] = acc[i][u][q] + x[q] * g[i];
                }
              }
            }
        }
#pragma unroll
        for (int i = 0; i < G; ++i) {
          const bool routed = rem0[i] != 0;
          if (tg + i < tokens && (routed || !a.is_residual)) {
            const long t = t0 + step * rps + tg + i;
#pragma unroll
            for (int u = 0; u < UPR; ++u) {
              const int off = off0 + u * kWave + lane;
              if (off < cpr)
                pack_store<OUT_DT, NE>(dst + (static_cast<size_t>(t) * cpr + off) * OUT_BYTES,
                                       acc[i][u]);
            }
          }
        }
      }
    }
  }
}

// --------------------------------- lean kernels for the fused MoE fabrics
// Seat indices, 1-d routing, no tag generation, E <= 64, 16-byte units: the
// shape every fused_dispatch / fused_combine call has.  Same scheme as the
// fast path above with everything optional compiled out.  A row is moved by a
// group of LPR = 2^LS lanes (64 for rows of >= 64 units, fewer for short rows, so
// that a wavefront moves 64/LPR rows at a time); each group walks the set bits
// of its own token's slice of the ballot mask and fetches the destination row
// from the lane that computed it with ds_bpermute.
template <int DT, int LS, int UPR>
__global__ __launch_bounds__(kBlock, 8) void dispatch_lean_kernel(DispatchArgs a) {
  using U = u32x4;
  constexpr int LPR = 1 << LS;
  constexpr int GROUPS = kWave >> LS;
  const int E = a.E;
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int ep_shift = a.map.ep_shift;
  const int ep = 1 << ep_shift;
  const int rps = kWave >> ep_shift;
  const int e = lane & (ep - 1);
  const int sub = lane >> ep_shift;
  const int gidx = lane >> LS, glane = lane & (LPR - 1);
  const unsigned long long seg0 = ep == kWave ? ~0ull : ((1ull << ep) - 1ull);

  const long r0 = wave * a.rows_pw;
  const int nr = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - r0)));
  const int n_steps = (nr + rps - 1) >> (6 - ep_shift);
  const int* __restrict__ idx0 = a.idx + r0 * E;
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  U* __restrict__ dst = static_cast<U*>(a.dst);

  // Rows of more than 128 bytes (lane groups of 16 and more) are written with streaming stores;
  // shorter rows are scattered partial lines, which are faster merged in the L2 (measured: 16- and
  // 32-byte rows lose 5-10 % when streamed, 80-byte rows 12 % in the combine; rows of 144 bytes and
  // more gain 5-20 %).  The
  // choice is a compile-time property of the shape: chosen by a branch at run time, the compiler
  // merges the two stores into an ordinary one.
  constexpr bool kStream = LS >= 4;
  int v_next = (n_steps > 0 && sub < nr && e < E) ? idx0[sub * E + e] : 0;
  const int my_count = (a.counts != nullptr && lane < E) ? a.counts[lane] : 0;
  const SmallTables tab = small_tables(a.loads, E, a.mpl, ep_shift, lane);

// In seat mode the source row of a token is the token itself, so its units are
  // fetched before the index words have even arrived and are reused for every
  // path the token is routed to (a top-k token is read once and stored k times).
  auto load_units = [&](int i, int tokens, int step, int off0, bool wanted, U (&val)[UPR]) {
    const size_t from = static_cast<size_t>(r0 + step * rps + i) * cpr;
#pragma unroll
    for (int u = 0; u < UPR; ++u) {
      const int off = off0 + u * LPR + glane;
      if (wanted && i < tokens && off < cpr) val[u] = src[from + off];
    }
  };

  for (int step = 0; step < n_steps; ++step) {
    const int tokens = min(rps, nr - step * rps);
    U val[UPR];
    // The rows of the first cells of a step are requested before anything is known about them;
    // the other cells of the step (and the later units of long rows) only if a path kept them:
    // a cell dropped by the capacities is then not read at all.  (Holding back the first request
    // of a step as well, until its index words -- requested a step earlier -- say that a path
    // kept the cell, takes the top-2 route with 56 % of its entries dropped from 15.1 to 14.3 us,
    // and costs the benchmark layer's dispatch, which drops nothing, half a microsecond.)
    load_units(gidx, tokens, step, 0, true, val);
    const int v = v_next;
    const int row = step * rps + sub;
    {
      const int nrow = row + rps;
      v_next = (step + 1 < n_steps && nrow < nr && e < E) ? idx0[nrow * E + e] : 0;
    }
    const int dst_row = tab.start_e + v - 1;
    const bool ok = row < nr && e < E && v >= 1 && v <= tab.load_e && dst_row < a.P;
    const unsigned long long m = __ballot(ok);
    float gate = 1.0f;
    if constexpr (DT >= 0) {
      if (ok) gate = load_gate(a.gates, DT, static_cast<size_t>(r0 + row) * E + e);
    }
    if (a.new_tags != nullptr && ok) {  // the lane that holds (token, path) tags the row
      const int tok = static_cast<int>(r0) + row;
      a.new_tags[dst_row] = a.old_tags != nullptr ? a.old_tags[tok] : tok + 1;
    }
    for (int tb = 0; tb < tokens; tb += GROUPS) {
      const int i = tb + gidx;  // token of this lane group
      const unsigned long long mine = i < tokens ? (m >> (i * ep)) & seg0 : 0ull;
      for (int off0 = 0; off0 < cpr; off0 += LPR * UPR) {
        if (tb != 0 || off0 != 0) load_units(i, tokens, step, off0, mine != 0, val);
        unsigned long long rem = mine;
        while (__ballot(rem != 0) != 0) {
          const bool has = rem != 0;
          const int b = i * ep + __builtin_ctzll(rem | (1ull << 63));
          rem &= rem - 1;
          const int d = __builtin_amdgcn_ds_bpermute(b << 2, dst_row);
          float g = 1.0f;
          if constexpr (DT >= 0)
            g = __int_as_float(__builtin_amdgcn_ds_bpermute(b << 2, __float_as_int(gate)));
#pragma unroll
          for (int u = 0; u < UPR; ++u) {
            const int off = off0 + u * LPR + glane;
            if (has && off < cpr) {
              U* to = dst + static_cast<size_t>(d) * cpr + off;
              if constexpr (DT >= 0) {
                constexpr int NE = 16 / elem_bytes(DT);
                float x[NE];
                unpack<DT, 16>(val[u], x);
#pragma unroll
                for (int q = 0; q < NE; ++q) x[q] = x[q] * g;
                pack_store<DT, NE, kStream>(to, x);
              } else {
                // streaming store: the row is not read again by this kernel, and written through the
                // L2 like an ordinary store it evicts source rows and index words still to be read
                store_unit<kStream>(to, val[u]);
              }
            }
          }
        }
      }
    }
  }

  if (a.counts != nullptr) {  // zero-fill this wavefront's share of the padding rows
    const long n_waves = static_cast<long>(gridDim.x) * (blockDim.x >> 6);
    int z = 0;
    if (lane < E) {
      const int alloc = a.mpl != 0 ? a.mpl : tab.my_load;
      const int filled = max(0, min(min(my_count, tab.my_load), alloc));
      z = max(0, alloc - filled);
    }
    const int z_incl = wave_inclusive_scan(z);
    const long Z = read_lane(z_incl, kWave - 1);
    long z0, z1;
    even_share(Z, wave, n_waves, &z0, &z1);
    for (long zi = z0; zi < z1; ++zi) {
      const int pe = __builtin_ctzll(__ballot(z_incl > zi));
      const int pad = read_lane(z, pe);
      const int alloc = a.mpl != 0 ? a.mpl : read_lane(tab.my_load, pe);
      const long row = static_cast<long>(read_lane(tab.my_start, pe)) + (alloc - pad) +
                       (zi - (read_lane(z_incl, pe) - pad));
      if (row < a.P) {
        for (int o = lane; o < cpr; o += kWave) dst[static_cast<size_t>(row) * cpr + o] = zero_unit<16>();
        if (a.new_tags != nullptr && lane == 0) a.new_tags[row] = 0;
      }
    }
  }
}

template <int IN_DT, int OUT_DT, int LS, int UPR>
__global__ __launch_bounds__(kBlock) void combine_lean_kernel(CombineArgs a) {
  using U = u32x4;
  constexpr int NE = 16 / elem_bytes(IN_DT);
  constexpr int OUT_BYTES = NE * elem_bytes(OUT_DT);
  constexpr int LPR = 1 << LS;
  constexpr int GROUPS = kWave >> LS;
  const int E = a.E;
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int ep_shift = a.map.ep_shift;
  const int ep = 1 << ep_shift;
  const int rps = kWave >> ep_shift;
  const int e = lane & (ep - 1);
  const int sub = lane >> ep_shift;
  const int gidx = lane >> LS, glane = lane & (LPR - 1);
  const unsigned long long seg0 = ep == kWave ? ~0ull : ((1ull << ep) - 1ull);

  const long t0 = wave * a.rows_pw;
  const int nt = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.T - t0)));
  if (nt == 0) return;
  const int n_steps = (nt + rps - 1) >> (6 - ep_shift);
  const int* __restrict__ idx0 = a.idx + t0 * E;
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  char* __restrict__ dst = static_cast<char*>(a.dst);

  // Index words are fetched two steps ahead and the first row of a step one step ahead: while
  // the rows of step s are added up and stored, the row loads of step s + 1 (which need its index
  // words) are already in flight, so a wavefront keeps two rows' worth of loads outstanding
  // instead of waiting out the index round trip and the row round trip of every cell in turn.
  auto index_word = [&](int step) {
    const int r = step * rps + sub;
    return (step < n_steps && r < nt && e < E) ? idx0[r * E + e] : 0;
  };
  int v_ahead1 = index_word(1);
  const int v_first = index_word(0);
  const SmallTables tab = small_tables(a.loads, E, a.mpl, ep_shift, lane);

  struct Step {
    unsigned long long m;  // (cell, path) pairs of the step that own a row
    int src_row;
    float gate;
    int tokens;
  };
  auto prepare = [&](int step, int v) {
    Step s;
    const int row = step * rps + sub;
    s.src_row = tab.start_e + v - 1;
    const bool ok = row < nt && e < E && v >= 1 && v <= tab.load_e && s.src_row < a.P;
    s.gate = 1.0f;
    if (ok && a.gates != nullptr)
      s.gate = load_gate(a.gates, a.gate_dtype, static_cast<size_t>(t0 + row) * E + e);
    s.m = __ballot(ok);
    s.tokens = min(rps, nt - step * rps);
    return s;
  };
  // the units of the first row of this lane group's first cell of the step (lowest path)
  auto first_row = [&](const Step& s, U (&val)[UPR]) {
    const int i = gidx;
    const unsigned long long mine = i < s.tokens ? (s.m >> (i * ep)) & seg0 : 0ull;
    const bool has = mine != 0;
    const int b = i * ep + __builtin_ctzll(mine | (1ull << 63));
    const int sr = __builtin_amdgcn_ds_bpermute(b << 2, s.src_row);
#pragma unroll
    for (int u = 0; u < UPR; ++u) {
      const int off = u * LPR + glane;
      if (has && off < cpr) val[u] = src[static_cast<size_t>(sr) * cpr + off];
    }
  };

  Step cur = prepare(0, v_first);
  U val_cur[UPR];
  first_row(cur, val_cur);
  for (int step = 0; step < n_steps; ++step) {
    Step nxt = cur;
    U val_nxt[UPR];
    if (step + 1 < n_steps) {
      const int v = v_ahead1;
      v_ahead1 = index_word(step + 2);
      nxt = prepare(step + 1, v);
      first_row(nxt, val_nxt);
    }
    const unsigned long long m = cur.m;
    const int src_row = cur.src_row;
    const float gate = cur.gate;
    const int tokens = cur.tokens;
    for (int tb = 0; tb < tokens; tb += GROUPS) {
      const int i = tb + gidx;
      const unsigned long long mine = i < tokens ? (m >> (i * ep)) & seg0 : 0ull;
      const size_t to = static_cast<size_t>(t0 + step * rps + i) * cpr;
      // No gates and no cell of this pass on more than one path: the sum of a cell is its one row
      // (0 + 1 * x), so the row is moved as it is, minus zeros cleared as the sum would clear them
      // (65536 rows of 1.5 KB: 50.9 -> 46.8 us).  Only for rows of more than 1 KB, one per wavefront at a
      // time: the second path through the loop costs registers, and the short-row shapes, which
      // live on their 7 wavefronts per SIMD, lose more to that than the conversions cost them
      // (100352 rows of 192 bytes: 11.9 -> 13.7 us with it).
      bool moves_rows = false;
      if constexpr (IN_DT == OUT_DT && LS == 6 && UPR >= 2)
        moves_rows = a.gates == nullptr && __ballot((mine & (mine - 1)) != 0) == 0;
      if (moves_rows) {
        const bool has = mine != 0;
        const int b = i * ep + __builtin_ctzll(mine | (1ull << 63));
        const int sr = __builtin_amdgcn_ds_bpermute(b << 2, src_row);
        for (int off0 = 0; off0 < cpr; off0 += LPR * UPR) {
          U val[UPR];
          if (tb == 0 && off0 == 0) {
#pragma unroll
            for (int u = 0; u < UPR; ++u) val[u] = val_cur[u];
          } else {
#pragma unroll
            for (int u = 0; u < UPR; ++u) {
              const int off = off0 + u * LPR + glane;
              if (has && off < cpr) val[u] = src[static_cast<size_t>(sr) * cpr + off];
            }
          }
          if (i < tokens && (has || !a.is_residual)) {
#pragma unroll
            for (int u = 0; u < UPR; ++u) {
              const int off = off0 + u * LPR + glane;
              if (off < cpr) {
                U v = {};
                if (has) {
#pragma unroll
                  for (int q = 0; q < 4; ++q) v[q] = plus_zero<IN_DT>(val[u][q]);
                }
                store_unit<true>(reinterpret_cast<U*>(dst + (to + off) * OUT_BYTES), v);
              }
            }
          }
        }
        continue;
      }
      for (int off0 = 0; off0 < cpr; off0 += LPR * UPR) {
        float acc[UPR][NE];
#pragma unroll
        for (int u = 0; u < UPR; ++u)
#pragma unroll
          for (int q = 0; q < NE; ++q) acc[u][q] = 0.0f;
        unsigned long long rem = mine;
        bool fetched = tb == 0 && off0 == 0;  // the first row of the first cell is in val_cur already
        while (__ballot(rem != 0) != 0) {  // ascending path order: lowest set bit first
          const bool has = rem != 0;
          const int b = i * ep + __builtin_ctzll(rem | (1ull << 63));
          rem &= rem - 1;
          const int sr = __builtin_amdgcn_ds_bpermute(b << 2, src_row);
          const float g = __int_as_float(__builtin_amdgcn_ds_bpermute(b << 2, __float_as_int(gate)));
          U val[UPR];
          if (fetched) {
#pragma unroll
            for (int u = 0; u < UPR; ++u) val[u] = val_cur[u];
          } else {
#pragma unroll
            for (int u = 0; u < UPR; ++u) {
              const int off = off0 + u * LPR + glane;
              if (has && off < cpr) val[u] = src[static_cast<size_t>(sr) * cpr + off];
            }
          }
          fetched = false;
#pragma unroll
          for (int u = 0; u < UPR; ++u) {
            const int off = off0 + u * LPR + glane;
            if (has && off < cpr) {
              float x[NE];
              unpack<IN_DT, 16>(val[u], x);
              // one rounding for the product, one for the sum (no fused multiply-add)
#pragma unroll
              for (int q = 0; q < NE; ++q) acc[u][q] = acc[u][q] + x[q] * g;
            }
          }
        }
        if constexpr (IN_DT != OUT_DT && LS == 6) {
          // 16-bit rows into an fp32 result, a whole wavefront per row: whole-line streaming stores
          const bool row_ok = i < tokens && (mine != 0 || !a.is_residual);  // the same for the whole wavefront
#pragma unroll
          for (int u = 0; u < UPR; ++u)
            store_widened_spread(dst + to * OUT_BYTES, off0 + u * LPR, cpr, row_ok, acc[u]);
        } else if (i < tokens && (mine != 0 || !a.is_residual)) {
#pragma unroll
          for (int u = 0; u < UPR; ++u) {
            const int off = off0 + u * LPR + glane;
            // streamed only when a wavefront's store covers whole lines: rows of up to 128 bytes are
            // scattered partial lines, which are faster merged in the L2
            if (off < cpr) {
              pack_store<OUT_DT, NE, IN_DT == OUT_DT && LS >= 4>(dst + (to + off) * OUT_BYTES, acc[u]);
            }
          }
        }
      }
    }
    cur = nxt;
#pragma unroll
    for (int u = 0; u < UPR; ++u) val_cur[u] = val_nxt[u];
  }
}

// Combine in scatter form for routes where no cell owns more than one row (top-1):
// every source row carries the 1-based tag of the cell it came from (the new_tags
// output of dispatch; 0 marks a padding row), so a row's data and its tag are fetched
// together and the row is stored to dst[tag-1] -- one memory round trip less than the
// gather form, which must read a cell's index words before it knows which row to load.
// Cells without a row are left untouched.
struct CombineRowsArgs {
  const void* src;
  void* dst;
  const int* row_tags;
  int T, P, cpr, rows_pw;
};

template <int IN_DT, int OUT_DT, int LS, int UPR>
__global__ __launch_bounds__(kBlock) void combine_rows_kernel(CombineRowsArgs a) {
  using U = u32x4;
  constexpr int NE = 16 / elem_bytes(IN_DT);
  constexpr int OUT_BYTES = NE * elem_bytes(OUT_DT);
  constexpr int LPR = 1 << LS;
  constexpr int GROUPS = kWave >> LS;
  const int lane = threadIdx.x & (kWave - 1);
  const long wave = static_cast<long>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int gidx = lane >> LS, glane = lane & (LPR - 1);
  const long p0 = wave * a.rows_pw;
  const int np = static_cast<int>(max(0l, min(static_cast<long>(a.rows_pw), a.P - p0)));
  const int cpr = a.cpr;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  char* __restrict__ dst = static_cast<char*>(a.dst);
  for (int rb = 0; rb < np; rb += GROUPS) {
    const int i = rb + gidx;
    const bool live = i < np;
    const int tag_loaded = live ? a.row_tags[p0 + i] : 0;
    const size_t from = static_cast<size_t>(p0 + i) * cpr;
    for (int off0 = 0; off0 < cpr; off0 += LPR * UPR) {
      U val[UPR];
#pragma unroll
      for (int u = 0; u < UPR; ++u) {
        const int off = off0 + u * LPR + glane;
        if (live && off < cpr) val[u] = src[from + off];
      }
      // The tag is first used here, behind the row loads: left alone, the compiler computes the
      // destination address ahead of the loop and so waits for the tag before it issues the row
      // loads -- two memory round trips instead of one.
      int tag = tag_loaded;
      asm volatile("" : "+v"(tag) : : "memory");
      if (tag >= 1 && tag <= a.T) {
        const size_t to = static_cast<size_t>(tag - 1) * cpr;
#pragma unroll
        for (int u = 0; u < UPR; ++u) {
          const int off = off0 + u * LPR + glane;
          if (off < cpr) {
            if constexpr (IN_DT == OUT_DT) {
              // streaming store, as in dispatch (rows of more than 128 bytes): nothing here reads the row again
              // (a row that is summed into a zero accumulator comes out with +0 for every -0)
              U v = val[u];
#pragma unroll
              for (int q = 0; q < 4; ++q) v[q] = plus_zero<IN_DT>(v[q]);
              store_unit<LS >= 4>(reinterpret_cast<U*>(dst + (to + off) * 16), v);
            } else {
              float x[NE];
              unpack<IN_DT, 16>(val[u], x);
#pragma unroll
              for (int q = 0; q < NE; ++q) x[q] = x[q] + 0.0f;  // -0 -> +0, as the sum would
              pack_store<OUT_DT, NE>(dst + (to + off) * OUT_BYTES, x);
            }
          }
        }
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

// Launch shape constants (0 = chosen per launch from the shape).
struct Knobs {
  int dispatch_rows = 0;
  int combine_rows = 0;
  int waves_pb = kBlock / kWave;
  bool no_lean = false;
};
const Knobs& knobs() {
  static const Knobs k;
  return k;
}

StepMap make_step_map(int E) {
  StepMap m{};
  m.E = E;
  m.chunks = E <= kWave ? 1 : (E + kWave - 1) / kWave;
  int shift = 0;
  while ((1 << shift) < std::min(E, kWave)) ++shift;
  m.ep_shift = shift;
  return m;
}

// Rows of the index matrix per wavefront: enough units that each lane has a
// handful of 16-byte accesses in flight, few enough index words that one batch
// of kSteps loads covers them.
int rows_per_wave(int forced_rows, int cpr, int E, long T, long min_waves = 4096) {
  int rows = forced_rows;
  if (rows <= 0) {
    rows = std::max(1, 384 / std::max(cpr, 1));
    while (rows > 1 && (T + rows - 1) / rows < min_waves) rows >>= 1;  // keep every SIMD busy
  }
  const StepMap m = make_step_map(E);
  if (E <= kWave) {  // register path: whole steps of 64 >> ep_shift rows
    const int rps = kWave >> m.ep_shift;
    return std::max(rps, rows / rps * rps);
  }
  rows = std::min(rows, std::max(1, kSteps / m.chunks));
  rows = std::min(rows, std::max(1, 2048 / E));  // bounds the per-wave list in LDS
  return std::max(1, rows);
}

struct LaunchShape {
  int waves_pb, grid;
  size_t lds;
};

// Packs as many wavefronts into a block as the LDS budget allows (at most 4).
bool launch_shape(long T, int rows_pw, int lds_pw_ints, LaunchShape* out) {
  const size_t per_wave = static_cast<size_t>(lds_pw_ints) * 4;
  if (per_wave > 60 * 1024) return false;
  int waves = std::max(1, std::min(kBlock / kWave, knobs().waves_pb));
  while (waves > 1 && per_wave * waves > 60 * 1024) waves >>= 1;
  const long n_waves = std::max(1l, (T + rows_pw - 1) / rows_pw);
  out->waves_pb = waves;
  out->grid = static_cast<int>((n_waves + waves - 1) / waves);
  out->lds = per_wave * waves;
  return true;
}

// Lanes per row (log2) and units per lane for the lean kernels.
#define BRT_LEAN_SHAPES(LAUNCH)                        \
  if (a.cpr > 2 * kWave) { LAUNCH(6, 4) }              \
  else if (a.cpr > kWave) { LAUNCH(6, 2) }             \
  else if (a.cpr > 32) { LAUNCH(6, 1) }                \
  else if (a.cpr > 16) { LAUNCH(5, 1) }                \
  else if (a.cpr > 8) { LAUNCH(4, 1) }                 \
  else if (a.cpr > 4) { LAUNCH(3, 1) }                 \
  else { LAUNCH(2, 1) }

template <int BYTES, int DT>
void launch_dispatch(const DispatchArgs& a, const LaunchShape& sh, hipStream_t st) {
  const dim3 grid(sh.grid), block(sh.waves_pb * kWave);
  if constexpr (BYTES == 16) {
    if (a.E <= kWave && a.is_1d && !a.is_tag_index && !knobs().no_lean) {
#define BRT_LAUNCH(LS, UPR) \
  hipLaunchKernelGGL((dispatch_lean_kernel<DT, LS, UPR>), grid, block, 0, st, a);
      BRT_LEAN_SHAPES(BRT_LAUNCH)
#undef BRT_LAUNCH
      return;
    }
  }
  if (a.E > kWave) {
    hipLaunchKernelGGL((dispatch_kernel<BYTES, DT>), grid, block, sh.lds, st, a);
  } else if (BYTES == 16 && a.cpr <= kWave) {
    hipLaunchKernelGGL((dispatch_small_kernel<BYTES, DT, 1>), grid, block, 0, st, a);
  } else if (BYTES == 16 && a.cpr <= 2 * kWave) {
    hipLaunchKernelGGL((dispatch_small_kernel<BYTES, DT, 2>), grid, block, 0, st, a);
  } else {
    hipLaunchKernelGGL((dispatch_small_kernel<BYTES, DT, 4>), grid, block, 0, st, a);
  }
}

template <int BYTES, int IN_DT, int OUT_DT>
void launch_combine(const CombineArgs& a, const LaunchShape& sh, hipStream_t st) {
  const dim3 grid(sh.grid), block(sh.waves_pb * kWave);
  if constexpr (BYTES == 16) {
    if (a.E <= kWave && !knobs().no_lean) {
#define BRT_LAUNCH(LS, UPR) \
  hipLaunchKernelGGL((combine_lean_kernel<IN_DT, OUT_DT, LS, UPR>), grid, block, 0, st, a);
      BRT_LEAN_SHAPES(BRT_LAUNCH)
#undef BRT_LAUNCH
      return;
    }
  }
  if (a.E > kWave) {
    hipLaunchKernelGGL((combine_kernel<BYTES, IN_DT, OUT_DT>), grid, block, sh.lds, st, a);
  } else if (BYTES == 16 && a.cpr <= kWave) {
    hipLaunchKernelGGL((combine_small_kernel<BYTES, IN_DT, OUT_DT, 1>), grid, block, 0, st, a);
  } else if (BYTES == 16 && a.cpr <= 2 * kWave) {
    hipLaunchKernelGGL((combine_small_kernel<BYTES, IN_DT, OUT_DT, 2>), grid, block, 0, st, a);
  } else {
    hipLaunchKernelGGL((combine_small_kernel<BYTES, IN_DT, OUT_DT, 4>), grid, block, 0, st, a);
  }
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
  a.map = make_step_map(E);
  a.rows_pw = rows_per_wave(knobs().dispatch_rows, a.cpr, E, T);
  a.lds_pw = 3 * E + 1 + 3 * a.rows_pw * E;
  LaunchShape sh;
  if (!launch_shape(T, a.rows_pw, a.lds_pw, &sh))
    return fail(BRT_E_UNSUPPORTED, "E=%d needs too much LDS", E);
  hipStream_t st = as_stream(stream);

#define BRT_DISPATCH_CASE(B)                                               \
  case B:                                                                  \
    if (gates == nullptr) launch_dispatch<B, -1>(a, sh, st);                \
    else if (dtype == BRT_F32) launch_dispatch<(B >= 4 ? B : 4), BRT_F32>(a, sh, st); \
    else if (dtype == BRT_F16) launch_dispatch<B, BRT_F16>(a, sh, st);     \
    else launch_dispatch<B, BRT_BF16>(a, sh, st);                          \
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
  a.map = make_step_map(E);
  // a gather makes two dependent memory round trips per cell: twice the wavefronts of dispatch
  // to hide them (5.8 -> 5.6 us at 8192 x 768 bf16, 8.5 -> 8.3 us at 100352 x 96 fp16)
  a.rows_pw = rows_per_wave(knobs().combine_rows, a.cpr, E, T, 8192);
  a.lds_pw = 2 * E + a.rows_pw + 2 * a.rows_pw * E;
  LaunchShape sh;
  if (!launch_shape(T, a.rows_pw, a.lds_pw, &sh))
    return fail(BRT_E_UNSUPPORTED, "E=%d needs too much LDS", E);
  hipStream_t st = as_stream(stream);

#define BRT_COMBINE_HALF(B, DT)                                        \
  if (out_dtype == BRT_F32) launch_combine<B, DT, BRT_F32>(a, sh, st); \
  else launch_combine<B, DT, DT>(a, sh, st);
#define BRT_COMBINE_CASE(B)                                            \
  case B:                                                              \
    if (in_dtype == BRT_F32) launch_combine<(B >= 4 ? B : 4), BRT_F32, BRT_F32>(a, sh, st); \
    else if (in_dtype == BRT_F16) { BRT_COMBINE_HALF(B, BRT_F16) }     \
    else { BRT_COMBINE_HALF(B, BRT_BF16) }                             \
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

extern "C" int brt_hip_combine_by_tags(const void* src, void* dst, const int32_t* row_tags, int P,
                                       int cell, int T, int in_dtype, int out_dtype, void* stream) {
  if (T < 0 || cell < 0 || P < 0) return fail(BRT_E_INVALID, "bad shape T=%d cell=%d P=%d", T, cell, P);
  if ((in_dtype != BRT_F32 && in_dtype != BRT_F16 && in_dtype != BRT_BF16) ||
      (out_dtype != in_dtype && out_dtype != BRT_F32))
    return fail(BRT_E_UNSUPPORTED, "dtype pair %d -> %d is not supported", in_dtype, out_dtype);
  if (P == 0 || cell == 0 || T == 0) return BRT_OK;
  if (!src || !dst || !row_tags) return fail(BRT_E_INVALID, "null argument");
  const size_t row_bytes = static_cast<size_t>(cell) * elem_bytes(in_dtype);
  if (row_bytes % 16 != 0 || !aligned(src, 16) || !aligned(dst, 16))
    return fail(BRT_E_UNSUPPORTED, "rows must be whole 16-byte units (row is %zu bytes)", row_bytes);
  CombineRowsArgs a{};
  a.src = src; a.dst = dst; a.row_tags = row_tags; a.T = T; a.P = P;
  a.cpr = static_cast<int>(row_bytes / 16);
  int rows = knobs().combine_rows;
  if (rows <= 0) {
    rows = std::max(1, 384 / a.cpr);
    while (rows > 1 && (P + rows - 1) / rows < 4096) rows >>= 1;
  }
  a.rows_pw = rows;
  const long n_waves = (static_cast<long>(P) + rows - 1) / rows;
  const int waves_pb = kBlock / kWave;
  const dim3 grid(static_cast<unsigned>((n_waves + waves_pb - 1) / waves_pb)), block(kBlock);
  hipStream_t st = as_stream(stream);
#define BRT_ROWS_LAUNCH(IN, OUT)                                                          \
  {                                                                                       \
    auto launch = [&](auto ls, auto upr) {                                                \
      hipLaunchKernelGGL((combine_rows_kernel<IN, OUT, decltype(ls)::value, decltype(upr)::value>), \
                         grid, block, 0, st, a);                                          \
    };                                                                                    \
    using std::integral_constant;                                                         \
    if (a.cpr > 2 * kWave) launch(integral_constant<int, 6>{}, integral_constant<int, 4>{});        \
    else if (a.cpr > kWave) launch(integral_constant<int, 6>{}, integral_constant<int, 2>{});       \
    else if (a.cpr > 32) launch(integral_constant<int, 6>{}, integral_constant<int, 1>{});          \
    else if (a.cpr > 16) launch(integral_constant<int, 5>{}, integral_constant<int, 1>{});          \
    else if (a.cpr > 8) launch(integral_constant<int, 4>{}, integral_constant<int, 1>{});           \
    else if (a.cpr > 4) launch(integral_constant<int, 3>{}, integral_constant<int, 1>{});           \
    else launch(integral_constant<int, 2>{}, integral_constant<int, 1>{});                          \
  }
  if (in_dtype == BRT_F32) BRT_ROWS_LAUNCH(BRT_F32, BRT_F32)
  else if (in_dtype == BRT_F16 && out_dtype == BRT_F16) BRT_ROWS_LAUNCH(BRT_F16, BRT_F16)
  else if (in_dtype == BRT_F16) BRT_ROWS_LAUNCH(BRT_F16, BRT_F32)
  else if (out_dtype == BRT_BF16) BRT_ROWS_LAUNCH(BRT_BF16, BRT_BF16)
  else BRT_ROWS_LAUNCH(BRT_BF16, BRT_F32)
#undef BRT_ROWS_LAUNCH
  return check_launch("combine_rows_kernel");
}
