// Tag-index gather: merging the rows that several paths produced for the same cell.
//
// The reference does this with library calls (src/backend/torch/router.cc): the per-path tag
// vectors are concatenated and passed to `_unique(sorted, return_inverse)` (:348-369), a sort;
// the inverse is then expanded to one int64 index per *element* (`repeat`, :451) and the rows are
// summed with `scatter_reduce` (:449-472), whose atomics add in no fixed order.
//
// Here neither step sorts or expands anything.
//   * unique: the tags lie in a known range [lo, hi]; a presence table over that range, one
//     prefix sum over it (which is the rank of every tag in the sorted unique list) and a lookup
//     per row give the unique tags and the inverse.
//   * sum: every row is pushed on a linked list of its output row with one atomic exchange; a
//     wavefront per output row walks its list (one hop per contributing path), orders the row
//     numbers in registers and adds the rows in ascending row order in fp32, so the result does
//     not depend on the order in which the atomics landed and every output row is written once.
#include <algorithm>
#include <climits>

#include "common.hpp"
#include "rows.hpp"

namespace brt {
namespace {

constexpr int kScanThreads = 1024;
constexpr int kScanItems = 8;
constexpr int kScanChunk = kScanThreads * kScanItems;
constexpr long kMaxRange = 1l << 25;  // 4096 scan blocks; each block adds up the totals before it

__global__ void fill_zero_kernel(int* __restrict__ p, long n) {
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

template <typename K>
__global__ void mark_present_kernel(const K* __restrict__ keys, long n, long lo, long range,
                                    int* __restrict__ present) {
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long k = static_cast<long>(keys[i]) - lo;
  if (k >= 0 && k < range) present[k] = 1;  // every writer stores the same value
}

// Sum of one block's chunk of the presence table.
__global__ __launch_bounds__(kScanThreads) void chunk_total_kernel(const int* __restrict__ present,
                                                                   long range, int* __restrict__ totals) {
  __shared__ int s_wave[kScanThreads / kWave];
  const long base = static_cast<long>(blockIdx.x) * kScanChunk + threadIdx.x * kScanItems;
  int v = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i)
    if (base + i < range) v += present[base + i];
  const int incl = wave_inclusive_scan(v);
  if (lane_id() == kWave - 1) s_wave[threadIdx.x >> 6] = incl;
  __syncthreads();
  if (threadIdx.x == 0) {
    int t = 0;
    for (int w = 0; w < kScanThreads / kWave; ++w) t += s_wave[w];
    totals[blockIdx.x] = t;
  }
}

// Turns the presence table into ranks (exclusive prefix sums, in place) and writes the present
// keys, in ascending order, to `unique`; the last block stores how many there are.
template <typename K>
__global__ __launch_bounds__(kScanThreads) void rank_emit_kernel(int* __restrict__ table, long range,
                                                                 const int* __restrict__ totals, long lo,
                                                                 K* __restrict__ unique,
                                                                 int* __restrict__ n_unique) {
  __shared__ int s_wave[kScanThreads / kWave];
  __shared__ int s_before;
  const int tid = threadIdx.x, wave = tid >> 6;
  // keys of the blocks before this one
  if (wave == 0) {
    int t = 0;
    for (int b = tid; b < static_cast<int>(blockIdx.x); b += kWave) t += totals[b];
    const int incl = wave_inclusive_scan(t);
    if (tid == kWave - 1) s_before = incl;
  }
  const long base = static_cast<long>(blockIdx.x) * kScanChunk + tid * kScanItems;
  int flag[kScanItems];
  int mine = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    flag[i] = base + i < range ? table[base + i] : 0;
    mine += flag[i];
  }
  const int incl = wave_inclusive_scan(mine);
  if (lane_id() == kWave - 1) s_wave[wave] = incl;
  __syncthreads();
  int rank = s_before + incl - mine;
  for (int w = 0; w < wave; ++w) rank += s_wave[w];
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    if (base + i < range) {
      table[base + i] = rank;
      if (flag[i]) unique[rank] = static_cast<K>(lo + base + i);
      rank += flag[i];
    }
  }
  if (blockIdx.x == gridDim.x - 1 && tid == kScanThreads - 1) *n_unique = rank;
}

template <typename K>
__global__ void inverse_kernel(const K* __restrict__ keys, long n, long lo, long range,
                               const int* __restrict__ rank, int64_t* __restrict__ inverse) {
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long k = static_cast<long>(keys[i]) - lo;
  inverse[i] = (k >= 0 && k < range) ? rank[k] : -1;
}

// The whole unique in one workgroup, the table in LDS: for ranges of up to kSmallRange tags and
// inputs short enough for 1024 threads to walk twice.
constexpr int kSmallRange = 32768;
constexpr long kSmallCount = 1l << 15;

constexpr int kKeysInFlight = 8;

template <typename K>
__global__ __launch_bounds__(kScanThreads) void unique_small_kernel(const K* __restrict__ keys, int n,
                                                                    long lo, int range,
                                                                    K* __restrict__ unique,
                                                                    int64_t* __restrict__ inverse,
                                                                    int* __restrict__ n_unique) {
  extern __shared__ int s_table[];
  __shared__ int s_wave[kScanThreads / kWave];
  const int tid = threadIdx.x, wave = tid >> 6;
  // The keys are fetched in batches of kKeysInFlight loads per thread (unconditional: an index
  // past the end reads the last key again and is dropped), all in flight together; one at a
  // time, every key would be a memory round trip of its own for this one workgroup.  The first
  // batch stays in registers for the inverse at the end.
  auto key_batch = [&](int base, K (&v)[kKeysInFlight]) {
#pragma unroll
    for (int j = 0; j < kKeysInFlight; ++j) v[j] = keys[min(base + j * kScanThreads + tid, n - 1)];  // n >= 1
  };
  K held[kKeysInFlight];
  key_batch(0, held);
  for (int i = tid; i < range; i += kScanThreads) s_table[i] = 0;
  __syncthreads();
  for (int base = 0; base < n; base += kKeysInFlight * kScanThreads) {
    K v[kKeysInFlight];
    if (base == 0) {
#pragma unroll
      for (int j = 0; j < kKeysInFlight; ++j) v[j] = held[j];
    } else {
      key_batch(base, v);
    }
#pragma unroll
    for (int j = 0; j < kKeysInFlight; ++j) {
      const long k = static_cast<long>(v[j]) - lo;
      if (base + j * kScanThreads + tid < n && k >= 0 && k < range) s_table[k] = 1;
    }
  }
  __syncthreads();
  // every thread scans a run of consecutive entries; an odd run length keeps the lanes of a
  // wavefront on different LDS banks
  const int run = ((range + kScanThreads - 1) / kScanThreads) | 1;
  const int first = min(tid * run, range), last = min(first + run, range);
  int mine = 0;
  for (int i = first; i < last; ++i) mine += s_table[i];
  const int incl = wave_inclusive_scan(mine);
  if (lane_id() == kWave - 1) s_wave[wave] = incl;
  __syncthreads();
  int rank = incl - mine;
  for (int w = 0; w < wave; ++w) rank += s_wave[w];
  for (int i = first; i < last; ++i) {
    const int flag = s_table[i];
    s_table[i] = rank;
    if (flag) unique[rank] = static_cast<K>(lo + i);
    rank += flag;
  }
  if (tid == kScanThreads - 1) *n_unique = rank;
  __syncthreads();
  for (int base = 0; base < n; base += kKeysInFlight * kScanThreads) {
    K v[kKeysInFlight];
    if (base == 0) {
#pragma unroll
      for (int j = 0; j < kKeysInFlight; ++j) v[j] = held[j];
    } else {
      key_batch(base, v);
    }
#pragma unroll
    for (int j = 0; j < kKeysInFlight; ++j) {
      const int i = base + j * kScanThreads + tid;
      const long k = static_cast<long>(v[j]) - lo;
      if (i < n) inverse[i] = (k >= 0 && k < range) ? s_table[k] : -1;
    }
  }
}

// Pushes row p on the list of output row index[p]: head[r] is 1 + the row pushed last (0: empty),
// next[p] is 1 + the row pushed before p.  Rows with an index outside [0, n_out) are left out.
template <typename K>
__global__ void link_rows_kernel(const K* __restrict__ index, int P, int n_out, int* __restrict__ head,
                                 int* __restrict__ next) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const long r = static_cast<long>(index[p]);
  next[p] = (r >= 0 && r < n_out) ? atomicExch(&head[r], p + 1) : 0;
}

// The same with the clearing of the heads in the same launch: one workgroup, for inputs so small
// that every thread issues one exchange (a second launch costs more than that; beyond it the
// exchanges of one workgroup queue up behind each other).
constexpr int kSmallLinkRows = 1024, kSmallLinkOut = 4096;

template <typename K>
__global__ __launch_bounds__(kScanThreads) void clear_and_link_kernel(const K* __restrict__ index, int P,
                                                                      int n_out, int* __restrict__ head,
                                                                      int* __restrict__ next) {
  for (int r = threadIdx.x; r < n_out; r += kScanThreads) head[r] = 0;
  __syncthreads();  // the stores above have reached memory before any exchange below
  for (int p = threadIdx.x; p < P; p += kScanThreads) {
    const long r = static_cast<long>(index[p]);
    next[p] = (r >= 0 && r < n_out) ? atomicExch(&head[r], p + 1) : 0;
  }
}

struct SumArgs {
  const void* src;
  void* dst;
  const int* head;
  const int* next;
  int n_out, cpr;  // cpr: copy units per row
};

// One wavefront per output row.  The contributing rows are collected from the list into lanes
// (lane i holds the i-th row met), ranked against each other and moved to ascending order with
// one cross-lane permute; a list longer than a wavefront is summed by repeated search instead
// (for every next row, walk the list for the smallest row number above the last one).
template <int BYTES, int IN_DT, int OUT_DT>
__global__ __launch_bounds__(256) void sum_rows_by_index_kernel(SumArgs a) {
  using U = typename Unit<BYTES>::type;
  constexpr int NE = BYTES / elem_bytes(IN_DT);
  constexpr int OUT_BYTES = NE * elem_bytes(OUT_DT);
  constexpr int kAhead = 4;
  const int lane = lane_id();
  const int r = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (r >= a.n_out) return;
  const U* __restrict__ src = static_cast<const U*>(a.src);
  char* __restrict__ dst = static_cast<char*>(a.dst) + static_cast<size_t>(r) * a.cpr * OUT_BYTES;

  int cur = __builtin_amdgcn_readfirstlane(a.head[r]);
  int count = 0, mine = INT_MAX;
  while (cur != 0 && count < kWave) {
    if (lane == count) mine = cur - 1;
    cur = __builtin_amdgcn_readfirstlane(a.next[cur - 1]);
    ++count;
  }
  count = __builtin_amdgcn_readfirstlane(count);
  const bool longer = cur != 0;
  int ordered = mine;
  if (!longer && count > 1) {
    int below = 0;
    for (int j = 0; j < count; ++j) below += read_lane(mine, j) < mine ? 1 : 0;
    // lanes past the list all rank `count`; whichever of them lands there carries INT_MAX
    ordered = __builtin_amdgcn_ds_permute(min(below, kWave - 1) << 2, mine);
  }

  for (int off0 = 0; off0 < a.cpr; off0 += kWave) {
    const int off = off0 + lane;
    const bool live = off < a.cpr;
    float acc[NE];
#pragma unroll
    for (int q = 0; q < NE; ++q) acc[q] = 0.0f;
    if (!longer) {
      for (int i0 = 0; i0 < count; i0 += kAhead) {
        U val[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
          if (i0 + u < count) {
            const int p = read_lane(ordered, i0 + u);
            if (live) val[u] = src[static_cast<size_t>(p) * a.cpr + off];
          }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
          if (i0 + u < count && live) {
            float x[NE];
            unpack<IN_DT, BYTES>(val[u], x);
#pragma unroll
            for (int q = 0; q < NE; ++q) acc[q] += x[q];
          }
        }
      }
    } else {
      int last = -1;
      while (true) {
        int best = INT_MAX;
        for (int c = __builtin_amdgcn_readfirstlane(a.head[r]); c != 0;
             c = __builtin_amdgcn_readfirstlane(a.next[c - 1])) {
          const int p = c - 1;
          if (p > last && p < best) best = p;
        }
        if (best == INT_MAX) break;
        last = best;
        if (live) {
          float x[NE];
          unpack<IN_DT, BYTES>(src[static_cast<size_t>(best) * a.cpr + off], x);
#pragma unroll
          for (int q = 0; q < NE; ++q) acc[q] += x[q];
        }
      }
    }
    // streamed when not widening and the rows are whole 16-byte units (the case of the expert
    // outputs this op exists for); narrower units mean short or odd rows, better merged in the L2
    if (live) pack_store<OUT_DT, NE, IN_DT == OUT_DT && BYTES == 16>(dst + static_cast<size_t>(off) * OUT_BYTES, acc);
  }
}

template <int IN_DT, int OUT_DT>
void launch_sum(int unit, const SumArgs& a, hipStream_t st) {
  const dim3 grid((a.n_out + 3) / 4), block(256);
  if (unit == 16) hipLaunchKernelGGL((sum_rows_by_index_kernel<16, IN_DT, OUT_DT>), grid, block, 0, st, a);
  else if (unit == 8) hipLaunchKernelGGL((sum_rows_by_index_kernel<8, IN_DT, OUT_DT>), grid, block, 0, st, a);
  else if (unit == 4) hipLaunchKernelGGL((sum_rows_by_index_kernel<4, IN_DT, OUT_DT>), grid, block, 0, st, a);
  else if constexpr (IN_DT != BRT_F32)
    hipLaunchKernelGGL((sum_rows_by_index_kernel<2, IN_DT, OUT_DT>), grid, block, 0, st, a);
}

long scan_blocks(long range) { return (range + kScanChunk - 1) / kScanChunk; }

}  // namespace
}  // namespace brt

using namespace brt;

extern "C" size_t brt_hip_unique_tags_workspace_bytes(long lo, long hi) {
  if (hi < lo) return 16;
  const long range = hi - lo + 1;
  if (range > kMaxRange) return 0;
  return static_cast<size_t>(range + scan_blocks(range)) * sizeof(int) + 16;
}

extern "C" int brt_hip_unique_tags(const void* tags, int tag_bits, long n, long lo, long hi,
                                   void* workspace, size_t workspace_bytes, void* unique_tags,
                                   int64_t* inverse, int32_t* n_unique, void* stream) {
  if (tag_bits != 32 && tag_bits != 64) return fail(BRT_E_INVALID, "tag_bits must be 32 or 64, got %d", tag_bits);
  if (n < 0 || hi < lo) return fail(BRT_E_INVALID, "bad arguments n=%ld lo=%ld hi=%ld", n, lo, hi);
  if (!n_unique) return fail(BRT_E_INVALID, "null n_unique");
  hipStream_t st = as_stream(stream);
  const long range = hi - lo + 1;
  if (range > kMaxRange)
    return fail(BRT_E_UNSUPPORTED, "tag range %ld exceeds %ld", range, kMaxRange);
  if (!tags || !workspace || !unique_tags || !inverse) return fail(BRT_E_INVALID, "null argument");
  const size_t need = brt_hip_unique_tags_workspace_bytes(lo, hi);
  if (workspace_bytes < need || !aligned(workspace, 4))
    return fail(BRT_E_INVALID, "workspace of %zu bytes, need %zu", workspace_bytes, need);
  if (range <= kSmallRange && n >= 1 && n <= kSmallCount) {  // (no keys: the general path below)
    const size_t lds = static_cast<size_t>(range) * sizeof(int);
    // more than 64 KB of dynamic LDS has to be allowed once per device and kernel
    static bool configured[2][64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 63;
    const int which = tag_bits == 32 ? 0 : 1;
    if (!configured[which][dev] || dev == 63) {
      const void* fn = which == 0 ? reinterpret_cast<const void*>(&unique_small_kernel<int32_t>)
                                  : reinterpret_cast<const void*>(&unique_small_kernel<int64_t>);
      if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                              kSmallRange * static_cast<int>(sizeof(int))) != hipSuccess)
        return fail(BRT_E_LAUNCH, "cannot reserve %d bytes of LDS", kSmallRange * 4);
      configured[which][dev] = true;
    }
    if (tag_bits == 32)
      hipLaunchKernelGGL(unique_small_kernel<int32_t>, dim3(1), dim3(kScanThreads), lds, st,
                         static_cast<const int32_t*>(tags), static_cast<int>(n), lo, static_cast<int>(range),
                         static_cast<int32_t*>(unique_tags), inverse, n_unique);
    else
      hipLaunchKernelGGL(unique_small_kernel<int64_t>, dim3(1), dim3(kScanThreads), lds, st,
                         static_cast<const int64_t*>(tags), static_cast<int>(n), lo, static_cast<int>(range),
                         static_cast<int64_t*>(unique_tags), inverse, n_unique);
    return check_launch("unique_small_kernel");
  }
  int* table = static_cast<int*>(workspace);
  const long blocks = scan_blocks(range);
  int* totals = table + range;
  hipLaunchKernelGGL(fill_zero_kernel, dim3(static_cast<unsigned>((range + 255) / 256)), dim3(256), 0, st,
                     table, range);
  if (n > 0) {
    const dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
    if (tag_bits == 32)
      hipLaunchKernelGGL(mark_present_kernel<int32_t>, grid, block, 0, st,
                         static_cast<const int32_t*>(tags), n, lo, range, table);
    else
      hipLaunchKernelGGL(mark_present_kernel<int64_t>, grid, block, 0, st,
                         static_cast<const int64_t*>(tags), n, lo, range, table);
  }
  if (blocks > 1)
    hipLaunchKernelGGL(chunk_total_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kScanThreads), 0, st,
                       table, range, totals);
  if (tag_bits == 32)
    hipLaunchKernelGGL(rank_emit_kernel<int32_t>, dim3(static_cast<unsigned>(blocks)), dim3(kScanThreads), 0,
                       st, table, range, totals, lo, static_cast<int32_t*>(unique_tags), n_unique);
  else
    hipLaunchKernelGGL(rank_emit_kernel<int64_t>, dim3(static_cast<unsigned>(blocks)), dim3(kScanThreads), 0,
                       st, table, range, totals, lo, static_cast<int64_t*>(unique_tags), n_unique);
  if (n > 0) {
    const dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
    if (tag_bits == 32)
      hipLaunchKernelGGL(inverse_kernel<int32_t>, grid, block, 0, st, static_cast<const int32_t*>(tags), n,
                         lo, range, table, inverse);
    else
      hipLaunchKernelGGL(inverse_kernel<int64_t>, grid, block, 0, st, static_cast<const int64_t*>(tags), n,
                         lo, range, table, inverse);
  }
  return check_launch("unique_tags");
}

extern "C" size_t brt_hip_combine_by_index_workspace_bytes(int P, int n_out) {
  return (static_cast<size_t>(std::max(P, 0)) + static_cast<size_t>(std::max(n_out, 0))) * sizeof(int) + 16;
}

extern "C" int brt_hip_combine_by_index(const void* in_data, void* out_data, const void* index,
                                        int index_bits, int P, int cell, int n_out, void* workspace,
                                        size_t workspace_bytes, int in_dtype, int out_dtype,
                                        void* stream) {
  if (index_bits != 32 && index_bits != 64)
    return fail(BRT_E_INVALID, "index_bits must be 32 or 64, got %d", index_bits);
  if (P < 0 || cell < 0 || n_out < 0) return fail(BRT_E_INVALID, "bad shape P=%d cell=%d n_out=%d", P, cell, n_out);
  const bool same = in_dtype == out_dtype;
  const bool widen = (in_dtype == BRT_F16 || in_dtype == BRT_BF16) && out_dtype == BRT_F32;
  if ((in_dtype != BRT_F32 && in_dtype != BRT_F16 && in_dtype != BRT_BF16) || !(same || widen))
    return fail(BRT_E_UNSUPPORTED, "dtype pair %d -> %d", in_dtype, out_dtype);
  if (n_out == 0 || cell == 0) return BRT_OK;
  if (!out_data || !workspace || (P > 0 && (!in_data || !index))) return fail(BRT_E_INVALID, "null argument");
  const size_t need = brt_hip_combine_by_index_workspace_bytes(P, n_out);
  if (workspace_bytes < need || !aligned(workspace, 4))
    return fail(BRT_E_INVALID, "workspace of %zu bytes, need %zu", workspace_bytes, need);
  const int es = elem_bytes(in_dtype), os = elem_bytes(out_dtype);
  const size_t row_bytes = static_cast<size_t>(cell) * es;
  int unit = 0;
  for (int b = 16; b >= es && unit == 0; b >>= 1)
    if (row_bytes % b == 0 && aligned(in_data, b) && aligned(out_data, std::min(16, b * os / es))) unit = b;
  if (unit == 0) return fail(BRT_E_INVALID, "rows are not aligned to their element size");
  hipStream_t st = as_stream(stream);
  int* head = static_cast<int*>(workspace);
  int* next = head + n_out;
  const bool small = P <= kSmallLinkRows && n_out <= kSmallLinkOut;
  if (small) {
    if (index_bits == 32)
      hipLaunchKernelGGL(clear_and_link_kernel<int32_t>, dim3(1), dim3(kScanThreads), 0, st,
                         static_cast<const int32_t*>(index), P, n_out, head, next);
    else
      hipLaunchKernelGGL(clear_and_link_kernel<int64_t>, dim3(1), dim3(kScanThreads), 0, st,
                         static_cast<const int64_t*>(index), P, n_out, head, next);
  } else {
    hipLaunchKernelGGL(fill_zero_kernel, dim3((n_out + 255) / 256), dim3(256), 0, st, head, static_cast<long>(n_out));
  }
  if (P > 0 && !small) {
    const dim3 grid((P + 255) / 256), block(256);
    if (index_bits == 32)
      hipLaunchKernelGGL(link_rows_kernel<int32_t>, grid, block, 0, st, static_cast<const int32_t*>(index), P,
                         n_out, head, next);
    else
      hipLaunchKernelGGL(link_rows_kernel<int64_t>, grid, block, 0, st, static_cast<const int64_t*>(index), P,
                         n_out, head, next);
  }
  SumArgs a{in_data, out_data, head, next, n_out, static_cast<int>(row_bytes / unit)};
  if (in_dtype == BRT_F32) launch_sum<BRT_F32, BRT_F32>(unit, a, st);
  else if (in_dtype == BRT_F16 && same) launch_sum<BRT_F16, BRT_F16>(unit, a, st);
  else if (in_dtype == BRT_F16) launch_sum<BRT_F16, BRT_F32>(unit, a, st);
  else if (same) launch_sum<BRT_BF16, BRT_BF16>(unit, a, st);
  else launch_sum<BRT_BF16, BRT_F32>(unit, a, st);
  return check_launch("combine_by_index");
}
