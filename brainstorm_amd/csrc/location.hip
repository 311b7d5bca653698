// Index / load generation, hot-mask throttling and index-format conversion.
//
// What is computed follows the reference kernels in src/router/location.cu
// (generate_indices_and_loads :212-257, throttle_hotmask :59-130,
// convert_*_indices :259-302); how it is computed does not.  The reference runs
// one 1024-thread block per path and walks the mask column (stride E) in serial
// 1024-row chunks.  Here the [T,E] mask is cut into row tiles that are read
// ONCE with coalesced 128-bit loads, scanned per column inside LDS, and chained
// across tiles with a single-pass decoupled look-back over per-(tile, column)
// records, so the whole op is one launch that moves 4*T*E bytes in and 4*T*E
// bytes out.
//
// Scan workspace layout (64-bit words):
//   [0, kMaxStrips)      ticket of strip s: (epoch << 32) | next tile id
//   [kMaxStrips]         sticky error flag (look-back spin bound exceeded)
//   [kHeaderWords, ...)  records: rec[strip][tile][col] = (tag << 32) | value,
//                        tag = (epoch << 2) | status, status 1 = tile aggregate,
//                        2 = inclusive prefix up to and including the tile
// A strip is a group of up to 256 adjacent columns; E <= 256 is one strip whose
// tiles are contiguous in memory.  Tile ids are handed out by the ticket in
// launch order, so a tile only ever waits for tiles that are already running.
// The block that draws the last tile id re-arms the ticket with epoch+1; stale
// records of earlier launches never match the current epoch, so the workspace
// is zeroed once and then reused without clearing.
#include <algorithm>

#include "common.hpp"

namespace brt {
namespace {

constexpr int kBlock = 256;
constexpr int kStripCols = 256;
constexpr int kTileIntsMax = 8192;  // 32 KiB of LDS per tile
constexpr int kTileIntsMin = 2048;
constexpr int kMaxStrips = 64;
constexpr int kHeaderWords = 128;  // 1 KiB
constexpr int kWindowMax = 16;     // look-back records fetched per thread and round
constexpr int kSpinLimit = 1 << 20;

enum { kSeat = 0, kTag = 1, kThrottle = 2 };

typedef int v4i __attribute__((ext_vector_type(4)));  // one 128-bit access

struct ScanGeometry {
  int strips;     // column strips
  int strip_cols; // columns per strip (last strip may hold fewer)
  int tile_rows;  // rows per tile (multiple of 4)
  int tiles;      // tiles per strip
  int chunk_rows; // rows scanned by one thread
};

ScanGeometry scan_geometry(int T, int E) {
  ScanGeometry g;
  g.strip_cols = std::min(E, kStripCols);
  g.strips = (E + kStripCols - 1) / kStripCols;
  // Large tiles keep the look-back short (each tile publishes strip_cols
  // records); small problems get smaller tiles so that more CUs take part.
  long total = static_cast<long>(T) * g.strip_cols;
  int tile_ints = kTileIntsMax;
  while (tile_ints > kTileIntsMin && total / tile_ints < 96) tile_ints >>= 1;
  int rows = std::max(4, (tile_ints / g.strip_cols) & ~3);
  g.tile_rows = rows;
  g.tiles = std::max(1, (T + rows - 1) / rows);
  const int slots = kBlock / g.strip_cols;  // row chunks scanned in parallel
  int chunk = (rows + slots - 1) / slots;
  // For narrow strips several row chunks share a wavefront; an odd chunk length
  // spreads their LDS addresses over the banks.
  if (g.strip_cols < 32 && (chunk & 1) == 0) chunk += 1;
  g.chunk_rows = chunk;
  return g;
}

struct ScanArgs {
  const int* mask;
  int* out;
  int* loads;
  int* counts;
  const int* caps;
  int* prefix;            // throttle only, updated in place
  const int* threshold;   // throttle only
  unsigned long long* ws;
  int T, E, C;
  int capacity_padding, path_wise_padding;
  int tile_rows, tiles, strip_cols, chunk_rows;
  int first_window;  // records per thread in the first look-back round
  int vec_ok;        // mask/out 16-byte aligned -> 128-bit tile copies
};

__device__ __forceinline__ unsigned long long ld_record(unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_record(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ int finalize_load(int real, const int* caps, int C, int cap_pad,
                                             int path_pad, int col) {
  if (path_pad) return caps[col];  // unconditional, even for an empty path
  if (real == 0) return 0;
  if (C == 0) return real;
  for (int i = 0; i < C; ++i)
    if (real <= caps[i]) return cap_pad ? caps[i] : real;
  return caps[C - 1];
}

template <int MODE>
__global__ __launch_bounds__(kBlock) void scan_kernel(ScanArgs a) {
  __shared__ __attribute__((aligned(16))) int s_tile[kTileIntsMax];
  __shared__ int s_cnt[kBlock];     // per (row chunk, column) local sums
  __shared__ int s_agg[kStripCols]; // tile aggregate per column
  __shared__ int s_acc[kStripCols]; // exclusive prefix of earlier tiles per column
  __shared__ int s_hi[kStripCols];  // nearest earlier tile not yet consumed
  __shared__ int s_done[kStripCols];
  __shared__ int s_psum[kBlock];
  __shared__ int s_pflag[kBlock];
  __shared__ int s_pre[kStripCols]; // throttle: incoming prefix
  __shared__ int s_thr[kStripCols]; // throttle: threshold
  __shared__ unsigned long long s_ticket;

  const int tid = threadIdx.x;
  const int strip = blockIdx.y;
  const int col0 = strip * kStripCols;
  const int cw = min(kStripCols, a.E - col0);  // columns of this strip
  const int E = a.E;

  if (tid == 0) {
    s_ticket = __hip_atomic_fetch_add(a.ws + strip, 1ull, __ATOMIC_RELAXED,
                                      __HIP_MEMORY_SCOPE_AGENT);
  }
  if (MODE == kThrottle && tid < cw) {
    s_pre[tid] = a.prefix[col0 + tid];
    s_thr[tid] = a.threshold[col0 + tid];
  }
  __syncthreads();
  const unsigned long long ticket = s_ticket;
  const int tile = static_cast<int>(ticket & 0xffffffffull);
  const unsigned epoch = static_cast<unsigned>(ticket >> 32);
  if (tile >= a.tiles) return;  // workspace was not prepared; never happens in normal use
  if (tid == 0 && tile == a.tiles - 1) {
    // every other block of this strip has drawn its ticket already
    st_record(a.ws + strip, static_cast<unsigned long long>(epoch + 1u) << 32);
  }
  const unsigned tag_agg = ((epoch & 0x3fffffffu) << 2) | 1u;
  const unsigned tag_pre = ((epoch & 0x3fffffffu) << 2) | 2u;
  unsigned long long* rec =
      a.ws + kHeaderWords + static_cast<size_t>(strip) * a.tiles * a.strip_cols;

  const int row0 = tile * a.tile_rows;
  const int rows = min(a.tile_rows, a.T - row0);
  const int n = rows * cw;
  const bool contiguous = (cw == E);

  // ---- 1. tile -> LDS ---------------------------------------------------------
  if (contiguous && a.vec_ok) {
    const v4i* src4 = reinterpret_cast<const v4i*>(a.mask + static_cast<size_t>(row0) * E);
    v4i* lds4 = reinterpret_cast<v4i*>(s_tile);
    const int nvec = n >> 2;
    constexpr int kIter = kTileIntsMax / (kBlock * 4);
    v4i r[kIter];
#pragma unroll
    for (int k = 0; k < kIter; ++k) {
      const int i = tid + k * kBlock;
      if (i < nvec) r[k] = __builtin_nontemporal_load(src4 + i);
    }
#pragma unroll
    for (int k = 0; k < kIter; ++k) {
      const int i = tid + k * kBlock;
      if (i < nvec) lds4[i] = r[k];
    }
    for (int i = (nvec << 2) + tid; i < n; i += kBlock)
      s_tile[i] = a.mask[static_cast<size_t>(row0) * E + i];
  } else {
    for (int i = tid; i < n; i += kBlock) {
      const int r = i / cw, c = i - r * cw;
      s_tile[i] = a.mask[static_cast<size_t>(row0 + r) * E + col0 + c];
    }
  }
  __syncthreads();

  // ---- 2. per-column scan inside the tile --------------------------------------
  // thread = (row chunk s, column c); consecutive lanes touch consecutive LDS words
  const int s = tid / cw, c = tid - s * cw;
  const int r_begin = s * a.chunk_rows;
  const int r_end = min(rows, r_begin + a.chunk_rows);
  const bool scanning = r_begin < rows && s * cw + cw <= kBlock;
  int local = 0;
  if (scanning)
    for (int r = r_begin; r < r_end; ++r) local += s_tile[r * cw + c];
  s_cnt[tid] = scanning ? local : 0;
  __syncthreads();
  int offset = 0;  // sum of the chunks above this one in the same column
  if (scanning)
    for (int k = 0; k < s; ++k) offset += s_cnt[k * cw + c];
  if (tid < cw) {
    int total = 0;
    const int slots = kBlock / cw;
    for (int k = 0; k < slots; ++k) total += s_cnt[k * cw + tid];
    s_agg[tid] = total;
    s_acc[tid] = 0;
    s_hi[tid] = tile - 1;
    s_done[tid] = (tile == 0);
    // publish: tile 0 knows its inclusive prefix already
    st_record(rec + static_cast<size_t>(tile) * a.strip_cols + tid,
              (static_cast<unsigned long long>(tile == 0 ? tag_pre : tag_agg) << 32) |
                  static_cast<unsigned>(total));
  }
  __syncthreads();

  // ---- 3. decoupled look-back over earlier tiles ---------------------------------
  if (tile > 0) {
    const int W = kBlock / cw;  // threads cooperating on one column
    const int w = s;
    for (int round = 0;; ++round) {
      const int U = round == 0 ? a.first_window : kWindowMax;
      if (w < W && !s_done[c]) {
        const int near = s_hi[c] - w * U;  // this thread covers tiles near, near-1, ...
        unsigned long long r[kWindowMax];
#pragma unroll
        for (int u = 0; u < kWindowMax; ++u) {
          const int j = near - u;
          if (u < U && j >= 0) r[u] = ld_record(rec + static_cast<size_t>(j) * a.strip_cols + c);
        }
        int sum = 0, flag = 0;  // flag: 0 all aggregates, 1 reached a prefix, 2 not ready
#pragma unroll
        for (int u = 0; u < kWindowMax; ++u) {
          const int j = near - u;
          if (u < U && flag == 0) {
            if (j < 0) {
              flag = 1;  // ran past tile 0: nothing more to add
            } else {
              const unsigned tag = static_cast<unsigned>(r[u] >> 32);
              const int val = static_cast<int>(r[u] & 0xffffffffull);
              if (tag == tag_agg) {
                sum += val;
              } else if (tag == tag_pre) {
                sum += val;
                flag = 1;
              } else {
                flag = 2;
              }
            }
          }
        }
        s_psum[tid] = sum;
        s_pflag[tid] = flag;
      }
      __syncthreads();
      if (tid < cw && !s_done[tid]) {
        int total = 0, state = 0;
        for (int k = 0; k < W; ++k) {
          const int f = s_pflag[k * cw + tid];
          if (f == 2) {
            state = 2;
            break;
          }
          total += s_psum[k * cw + tid];
          if (f == 1) {
            state = 1;
            break;
          }
        }
        if (state != 2) {  // state 2: a record was not published yet, poll again
          s_acc[tid] += total;
          if (state == 1)
            s_done[tid] = 1;
          else
            s_hi[tid] -= W * U;
        }
      }
      const int pending = __syncthreads_count(tid < cw && !s_done[tid]);
      if (pending == 0) break;
      if (round >= kSpinLimit) {  // give up instead of hanging; result is invalid
        if (tid == 0) st_record(a.ws + kMaxStrips, 1ull);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    if (tid < cw) {
      st_record(rec + static_cast<size_t>(tile) * a.strip_cols + tid,
                (static_cast<unsigned long long>(tag_pre) << 32) |
                    static_cast<unsigned>(s_acc[tid] + s_agg[tid]));
    }
  }

  // ---- 4. rewrite the tile in LDS (or scatter tags) --------------------------------
  if (scanning) {
    int run = s_acc[c] + offset;
    if (MODE == kThrottle) run += s_pre[c];
    const int thr = MODE == kThrottle ? s_thr[c] : 0;
    for (int r = r_begin; r < r_end; ++r) {
      const int m = s_tile[r * cw + c];
      run += m;
      if (MODE == kSeat) {
        s_tile[r * cw + c] = run * m;
      } else if (MODE == kThrottle) {
        s_tile[r * cw + c] = (m == 1 && run <= thr) ? 1 : 0;
      } else {
        const int index = run * m;
        if (index >= 1 && index <= a.T)
          a.out[static_cast<size_t>(index - 1) * E + col0 + c] = row0 + r + 1;
      }
    }
  }

  // ---- 5. totals: loads / counts / throttle prefix (last tile only) ------------------
  if (tile == a.tiles - 1 && tid < cw) {
    const int total = s_acc[tid] + s_agg[tid];
    if (MODE == kThrottle) {
      a.prefix[col0 + tid] = min(s_pre[tid] + total, s_thr[tid]);
    } else {
      a.loads[col0 + tid] =
          finalize_load(total, a.caps, a.C, a.capacity_padding, a.path_wise_padding, col0 + tid);
      if (a.counts) a.counts[col0 + tid] = total;
    }
  }
  if (MODE == kTag) return;
  __syncthreads();

  // ---- 6. LDS -> out -------------------------------------------------------------------
  if (contiguous && a.vec_ok) {
    v4i* dst4 = reinterpret_cast<v4i*>(a.out + static_cast<size_t>(row0) * E);
    const v4i* lds4 = reinterpret_cast<const v4i*>(s_tile);
    const int nvec = n >> 2;
    for (int i = tid; i < nvec; i += kBlock) dst4[i] = lds4[i];
    for (int i = (nvec << 2) + tid; i < n; i += kBlock)
      a.out[static_cast<size_t>(row0) * E + i] = s_tile[i];
  } else {
    for (int i = tid; i < n; i += kBlock) {
      const int r = i / cw, cc = i - r * cw;
      a.out[static_cast<size_t>(row0 + r) * E + col0 + cc] = s_tile[i];
    }
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
  const ScanGeometry g = scan_geometry(a.T, a.E);
  if (g.strips > kMaxStrips) return fail(BRT_E_UNSUPPORTED, "E=%d exceeds %d paths", a.E,
                                         kMaxStrips * kStripCols);
  const size_t need = brt_hip_scan_workspace_bytes(a.T, a.E);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(BRT_E_WORKSPACE, "scan workspace too small: %zu < %zu bytes", workspace_bytes,
                need);
  if (!aligned(workspace, 8)) return fail(BRT_E_INVALID, "scan workspace must be 8-byte aligned");
  a.ws = static_cast<unsigned long long*>(workspace);
  a.tile_rows = g.tile_rows;
  a.tiles = g.tiles;
  a.strip_cols = g.strip_cols;
  a.chunk_rows = g.chunk_rows;
  // When every tile is resident at once, nobody has an inclusive prefix yet on
  // the first poll, so fetch a wide window straight away; in a long stream of
  // tiles the nearest predecessors have usually finished and a narrow first
  // window saves record traffic.
  a.first_window = g.tiles <= 1024 ? kWindowMax : 2;
  a.vec_ok = aligned(a.mask, 16) && aligned(a.out, 16);
  const dim3 grid(g.tiles, g.strips);
  hipStream_t st = as_stream(stream);
  if (mode == kSeat)
    hipLaunchKernelGGL(scan_kernel<kSeat>, grid, dim3(kBlock), 0, st, a);
  else if (mode == kTag)
    hipLaunchKernelGGL(scan_kernel<kTag>, grid, dim3(kBlock), 0, st, a);
  else
    hipLaunchKernelGGL(scan_kernel<kThrottle>, grid, dim3(kBlock), 0, st, a);
  return check_launch("scan_kernel");
}

}  // namespace
}  // namespace brt

using namespace brt;

extern "C" size_t brt_hip_scan_workspace_bytes(int T, int E) {
  if (T <= 0 || E <= 0) return kHeaderWords * 8;
  const ScanGeometry g = scan_geometry(T, E);
  return (static_cast<size_t>(kHeaderWords) +
          static_cast<size_t>(g.strips) * g.tiles * g.strip_cols) * 8;
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
