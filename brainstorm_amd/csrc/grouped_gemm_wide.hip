// Grouped expert GEMM, second kernel: 256 x 256 output tiles for loads that give an expert
// several hundred rows and more (ragged task-MoE batches, top-2 routes with large capacities).
//
// Same contract as grouped_gemm.hip (out[rows of e] = act(x[rows of e] @ W_e^T + b_e), one launch,
// loads read on the device).  What differs is what bounds it: with many rows per expert the weights
// are re-used and the matrix units become the limit, so the tile is the one that feeds them best.
//
//   - A workgroup is 4 wavefronts in a 2 x 2 arrangement, each owning 128 x 128 outputs: 16
//     accumulator tiles of v_mfma_f32_32x32x16_bf16 (256 accumulator registers), 8 fragment reads
//     per 16 MFMAs.  LDS read bandwidth, which bounds the 160-row kernel at 7 reads per 10 MFMAs,
//     is half used.
//   - Operands go from global memory straight into LDS (buffer_load ... lds, 16 bytes per lane):
//     no staging registers, no LDS write instructions.  The destination of such a load is
//     M0 + 16 * lane, so the swizzle that keeps the fragment reads free of bank conflicts is
//     applied on the global side: the lane that fills slot s of tile row r fetches chunk
//     s ^ ((r >> 2) & 3) of that row.
//   - LDS is a ring of four K-steps of 32 (32 KiB each: 256 activation rows and 256 weight rows of
//     64 bytes).  While K-step kt is multiplied, kt+1 is complete or landing and kt+2, kt+3 are in
//     flight; the wait for a step counts the wavefront's own loads (s_waitcnt vmcnt with the
//     number of younger loads that may stay outstanding) and one workgroup barrier per K-step both
//     publishes the step that has landed and frees the one that was read last.  The loads are
//     issued from inline assembly, so the compiler neither waits for them before every LDS read
//     nor drains them at a barrier.
//   - Tiles are numbered so that the 32 workgroups an XCD runs at one time form a patch of one
//     expert's output -- 4 row blocks x 8 column tiles where the expert has that many row blocks
//     -- and share both operands through that XCD's L2: a weight tile is fetched from memory once
//     per four row blocks, not once per row block.
//   - A wavefront multiplies only the 32-row tiles that hold rows (1, 2 or 4 of its 4): experts
//     with a handful of rows stream their weights at the rate of the memory, not of the MFMAs.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "common.hpp"
#include "grouped_gemm.hpp"

namespace brt {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const bf16x4 __attribute__((address_space(1)))* global_bf16x4;
typedef const __bf16 __attribute__((address_space(1)))* global_bf16;

constexpr int kBM = 256, kBN = 256, kBK = 64, kStages = 2;
constexpr int kRowB = kBK * 2;                      // bytes of one tile row in one stage: one cache line
constexpr int kChunks = kRowB / 16;                 // 16-byte chunks of a tile row
constexpr int kStageRows = kBM + kBN;               // activation rows first, then weight rows
constexpr int kStageB = kStageRows * kRowB;         // 64 KiB
constexpr int kLdsBytes = kStages * kStageB;        // 128 KiB
constexpr int kRowsPerLoad = 64 / kChunks;          // tile rows one load instruction fills: 8
constexpr int kLoadsPW = kStageRows / kRowsPerLoad / 4;  // loads per wavefront and stage: 16
constexpr int kSub = kBK / 16;                      // MFMA k-steps per stage
constexpr int kGroup = 4;                           // row blocks of one expert that run side by side
constexpr uint32_t kOutOfRange = 0x80000000u;       // buffer offset past any extent: reads as zero
constexpr int kXcds = 8, kCusPerXcd = 32;

// Raw buffer resource: base, no stride, extent in bytes, 32-bit raw data format.
__device__ __forceinline__ i32x4 make_rsrc(const void* p, size_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  i32x4 r;
  r[0] = static_cast<int>(a);
  r[1] = static_cast<int>((a >> 32) & 0xffff);
  r[2] = static_cast<int>(bytes > 0x7fffffffull ? 0x7fffffffull : bytes);
  r[3] = 0x00020000;
  return r;
}

// 16 bytes per lane from the buffer straight into LDS at lds_base + 16 * lane (wave-uniform
// lds_base in M0).  Counts on vmcnt like any load; the compiler does not know it touches LDS.
__device__ __forceinline__ void load_to_lds(const i32x4& rsrc, uint32_t voffset, uint32_t soffset,
                                            uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
               : "memory");
}

// Store of 16 output bytes with the streaming policy and system scope (as in the 160-row kernel).
__device__ __forceinline__ void stream_out(const u32x4& v, u32x4* p) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(p), "v"(v) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_loads() {  // at most N of this wavefront's loads still in flight
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

__device__ __forceinline__ void wait_lds_reads() {
  asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
}

__device__ __forceinline__ void block_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int ACT>
__global__ __launch_bounds__(256) void grouped_gemm_wide_kernel(GemmArgs a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  __shared__ int s_tile[4];  // expert, first row, rows, column tile

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // ---- which tile ------------------------------------------------------------------------
  // hardware deals workgroups round-robin over the XCDs (workgroup b runs on XCD b % 8); the 32
  // workgroups with consecutive b / 8 on one XCD take 32 consecutive tiles of the ordered list
  const int b = blockIdx.x;
  const int within = b >> 3;
  const int t = (((within >> 5) * kXcds + (b & 7)) << 5) + (within & 31);
  if (tid < kWave) {
    int carry_t = 0, carry_m = 0;
    bool found = false;
    for (int base = 0; base < a.E && !found; base += kWave) {
      const int e = base + lane;
      const int m = e < a.E ? a.loads[e] : 0;
      const int blocks = (m + kBM - 1) / kBM;
      const int tiles = blocks * a.tiles_n;
      const int incl_t = wave_inclusive_scan(tiles), incl_m = wave_inclusive_scan(m);
      const int first = carry_t + incl_t - tiles;
      const bool hit = t >= first && t < first + tiles;
      if (__ballot(hit) != 0) {
        found = true;
        if (hit) {
          // order inside an expert: groups of kGroup row blocks; inside a group the row block
          // changes fastest, then the column tile
          const int local = t - first, per_group = kGroup * a.tiles_n;
          const int full = blocks / kGroup;
          const int g = local / per_group;
          int col, block;
          if (g < full) {
            const int r = local - g * per_group;
            col = r / kGroup;
            block = g * kGroup + r % kGroup;
          } else {
            const int last = blocks - full * kGroup;
            const int r = local - full * per_group;
            col = r / last;
            block = full * kGroup + r % last;
          }
          s_tile[0] = e;
          s_tile[1] = carry_m + incl_m - m + block * kBM;
          s_tile[2] = min(kBM, m - block * kBM);
          s_tile[3] = col;
        }
      }
      carry_t += __shfl(incl_t, kWave - 1, kWave);
      carry_m += __shfl(incl_m, kWave - 1, kWave);
    }
    if (!found && lane == 0) s_tile[0] = -1;
  }
  __syncthreads();
  const int e = __builtin_amdgcn_readfirstlane(s_tile[0]);
  if (e < 0) return;  // beyond the last tile
  const int row0 = __builtin_amdgcn_readfirstlane(s_tile[1]);
  const int rows = min(__builtin_amdgcn_readfirstlane(s_tile[2]), a.P - row0);
  const int n0 = __builtin_amdgcn_readfirstlane(s_tile[3]) * kBN;
  const int K = a.K;
  const int k_tiles = K / kBK;

  // ---- global -> LDS --------------------------------------------------------------------
  // Load i of wavefront w fills the 8 tile rows of group i * 4 + w (groups 0..31: activation
  // rows, 32..63: weight rows), a whole 128-byte line of each.  Lane l lands at slot l & 7 of row
  // l >> 3 of the group and fetches chunk (l & 7) ^ ((row >> 1) & 7) of that row; with
  // row = 8 * group + (l >> 3), (row >> 1) & 7 = 4 * (w & 1) + (l >> 4).
  const __bf16* const w_e = a.w[e];
  const i32x4 res_a = make_rsrc(a.x + static_cast<size_t>(row0) * K, static_cast<size_t>(a.P - row0) * K * 2);
  const i32x4 res_b = make_rsrc(w_e + static_cast<size_t>(n0) * K, static_cast<size_t>(a.N - n0) * K * 2);
  const uint32_t chunk = (lane & 7) ^ (((wave & 1) << 2) | (lane >> 4));
  uint32_t off[kLoadsPW];
#pragma unroll
  for (int i = 0; i < kLoadsPW; ++i) {
    const int r = ((i * 4 + wave) & 31) * kRowsPerLoad + (lane >> 3);  // row inside the operand's 256 rows
    off[i] = (static_cast<uint32_t>(r) * K + chunk * 8) * 2;
    if (i < kLoadsPW / 2 && r >= rows) off[i] = kOutOfRange;  // no row: zeros, no memory request
  }
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
  const uint32_t lds_w = __builtin_amdgcn_readfirstlane(lds0) + wave * 1024;
  auto issue = [&](int kt) {
    const uint32_t base = lds_w + (kt & (kStages - 1)) * kStageB;
    const uint32_t k_bytes = kt * kRowB;
#pragma unroll
    for (int i = 0; i < kLoadsPW; ++i)
      load_to_lds(i < kLoadsPW / 2 ? res_a : res_b, off[i], k_bytes, base + i * 4096);
  };

  // ---- fragments ------------------------------------------------------------------------
  // MFMA operand: this lane feeds row (lane % 32), k-half (lane / 32) of a 32 x 16 block; chunk
  // ks * 2 + lane / 32 of the row sits in slot chunk ^ ((row >> 1) & 7)
  const int frag_row = lane & 31, frag_k = lane >> 5;
  char* const lds = smem;
  const int frag_x = (wm * 128 + frag_row) * kRowB;
  const int frag_w = (kBM + wn * 128 + frag_row) * kRowB;
  const int swz = (frag_row >> 1) & 7;

  // row tiles of 32 this wavefront has rows in: 0, 1, 2 or 4 (3 runs as 4)
  const int mine = rows - wm * 128;
  const int row_tiles = mine <= 0 ? 0 : mine <= 32 ? 1 : mine <= 64 ? 2 : 4;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x16{};

  // K loop.  Stage kt & 1 holds K-step kt.  Fragments are read one MFMA k-step ahead of their
  // use; before the last k-step of a stage every fragment of the stage is in registers, so that
  // is where the wavefronts meet: the next stage has landed (each waits for its own loads, the
  // barrier publishes them) and this stage can take the K-step after next.
  auto k_loop = [&](auto mt_tag) {
    constexpr int MT = decltype(mt_tag)::value;
    bf16x8 fw[2][4], fx[2][MT > 0 ? MT : 1];
    auto read_frags = [&](int stage, int ks, int buf) {
      const char* s = lds + stage * kStageB + (((ks * 2 + frag_k) ^ swz) << 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) fw[buf][j] = *reinterpret_cast<const bf16x8*>(s + frag_w + j * 32 * kRowB);
#pragma unroll
      for (int i = 0; i < MT; ++i) fx[buf][i] = *reinterpret_cast<const bf16x8*>(s + frag_x + i * 32 * kRowB);
    };
    auto multiply = [&](int buf) {
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[buf][j], fx[buf][i], acc[i][j], 0, 0, 0);
    };
    issue(0);
    wait_loads<0>();
    block_barrier();
    if (k_tiles > 1) issue(1);
    if (MT > 0) read_frags(0, 0, 0);
    for (int kt = 0; kt < k_tiles; ++kt) {
      const int stage = kt & 1;
#pragma unroll
      for (int ks = 0; ks < kSub; ++ks) {
        if (ks + 1 < kSub) {
          if (MT > 0) read_frags(stage, ks + 1, (ks + 1) & 1);
        } else {
          wait_lds_reads();   // every fragment of this stage is in registers
          wait_loads<0>();    // the next stage has landed
          block_barrier();
          if (kt + 2 < k_tiles) issue(kt + 2);
          if (MT > 0 && kt + 1 < k_tiles) read_frags(stage ^ 1, 0, 0);
        }
        if (MT > 0) multiply(ks & 1);
      }
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I4 = std::integral_constant<int, 4>;
  if (row_tiles == 4) k_loop(I4{});
  else if (row_tiles == 2) k_loop(I2{});
  else if (row_tiles == 1) k_loop(I1{});
  else k_loop(I0{});

  // ---- epilogue: bias + activation, bf16, through this wavefront's quarter of LDS ---------
  // Behind the last barrier of the K loop no wavefront reads or loads LDS any more.  Transposed
  // accumulator: element r of tile (i, j) is output row 32 i + lane % 32 and column
  // 32 j + 8 (r / 4) + 4 (lane / 32) + r % 4 of this wavefront's 128 x 128 block, i.e. a lane holds
  // 4 consecutive columns (8 bytes) of its row.  They go to a 128 x 256-byte image of the block:
  // 16-byte chunk c of row r at slot c ^ (r & 15), its two halves swapped for r & 16, which makes
  // the 8-byte writes of 32 lanes and the 16-byte reads of 16 lanes hit every bank once.  The
  // image is then read a row at a time (16 lanes x 16 bytes) and stored as whole 256-byte rows.
  const global_bf16 bias = a.bias != nullptr ? (global_bf16)(a.bias[e]) : (global_bf16)nullptr;
  char* const image = lds + wave * (128 * 256);
  const int col_w = n0 + wn * 128;  // first column of this wavefront
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int col = j * 32 + 8 * g + 4 * frag_k;  // inside the wavefront's 128 columns
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (bias != nullptr && col_w + col < a.N) {
        const bf16x4 b4 = *(global_bf16x4)(bias + col_w + col);
#pragma unroll
        for (int q = 0; q < 4; ++q) bv[q] = static_cast<float>(b4[q]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (i < row_tiles) {
          const int r = i * 32 + frag_row;
          bf16x4 o;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            o[q] = static_cast<__bf16>(apply_act<ACT>(acc[i][j][4 * g + q] + bv[q]));
          *reinterpret_cast<bf16x4*>(image + r * 256 + (((j * 4 + g) ^ (frag_row & 15)) << 4) +
                                     ((frag_k ^ (frag_row >> 4)) << 3)) = o;
        }
      }
    }
  }
  __bf16* const out_w = a.out + (static_cast<size_t>(row0) + wm * 128) * a.N + col_w;
  const int c16 = lane & 15;
  const bool col_ok = col_w + c16 * 8 < a.N;
  for (int r = lane >> 4; r < min(mine, row_tiles * 32); r += 4) {
    u32x4 v = *reinterpret_cast<const u32x4*>(image + r * 256 + ((c16 ^ (r & 15)) << 4));
    if (r & 16) v = u32x4{v[2], v[3], v[0], v[1]};
    if (col_ok) stream_out(v, reinterpret_cast<u32x4*>(out_w + static_cast<size_t>(r) * a.N + c16 * 8));
  }
}

template <int ACT>
int launch_wide(GemmArgs& a, hipStream_t st) {
  a.tiles_n = (a.N + kBN - 1) / kBN;
  // the sum over experts of ceil(M_e / 256) never exceeds P / 256 + E; whole rounds of XCD patches
  const long tiles_max = (static_cast<long>(a.P + kBM - 1) / kBM + a.E) * a.tiles_n;
  const long round = kXcds * kCusPerXcd;
  const long grid = (tiles_max + round - 1) / round * round;
  auto* fn = &grouped_gemm_wide_kernel<ACT>;
  static bool configured[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 63;
  if (!configured[dev] || dev == 63) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess)
      return fail(BRT_E_LAUNCH, "cannot reserve %d bytes of LDS", kLdsBytes);
    configured[dev] = true;
  }
  hipLaunchKernelGGL(fn, dim3(static_cast<unsigned>(grid)), dim3(256), kLdsBytes, st, a);
  return check_launch("grouped_gemm_wide_kernel");
}

}  // namespace

// The wide tiles pay when experts have more rows than one 160-row block on average; the routed
// forms and K that is not whole K-steps stay with the 160-row kernel.
bool wide_gemm_applies(const GemmArgs& a) {
  static const int forced = std::getenv("BRT_GEMM_WIDE") ? std::atoi(std::getenv("BRT_GEMM_WIDE")) : -1;
  if (a.tags != nullptr || a.K % kBK != 0 || a.K < kBK) return false;
  if (forced >= 0) return forced != 0;
  return false;  // while the kernel is being tuned
}

int launch_wide_gemm(GemmArgs& a, int act, hipStream_t st) {
  if (act == BRT_ACT_GELU) return launch_wide<BRT_ACT_GELU>(a, st);
  if (act == BRT_ACT_RELU) return launch_wide<BRT_ACT_RELU>(a, st);
  return launch_wide<BRT_ACT_NONE>(a, st);
}

}  // namespace brt
