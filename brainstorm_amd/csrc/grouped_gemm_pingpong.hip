// Grouped expert GEMM, second kernel: 256 x 256 output tiles multiplied by two groups of
// wavefronts in ping-pong, for shapes that give an expert hundreds of rows and more (ragged
// task-MoE batches, top-2 routes with large capacities), where the matrix units and not the weight
// stream set the pace.
//
// Same contract as grouped_gemm.hip (out[rows of e] = act(x[rows of e] @ W_e^T + b_e), one launch,
// loads read on the device; reference: src/jit/compiler.cu:151-246).  What differs:
//
//   - A workgroup is 8 wavefronts, two per SIMD, each owning 128 x 64 outputs (8 accumulator tiles
//     of v_mfma_f32_32x32x16_bf16 = 128 registers, and the 24 fragments of a whole K-step of 64 in
//     96 more).  The wavefronts of a SIMD belong to two groups that run half a K-step apart: while
//     one group issues its 32 MFMAs (C phase), the other reads its fragments from LDS and requests
//     operands from memory (M phase); a workgroup barrier separates the phases.  The matrix pipe
//     of a SIMD therefore always has a wavefront that does nothing but multiply, and the memory
//     instructions of the other one never stand between two MFMAs.
//   - Operands go from global memory straight into LDS (buffer_load ... lds): no staging
//     registers.  The destination of such a load is M0 + 16 * lane, so the swizzle that keeps the
//     fragment reads free of bank conflicts is applied on the global side: the lane that fills
//     slot s of tile row r fetches chunk s ^ ((r >> 1) & 7) of that row.
//   - All 160 KB of LDS are operand stages: a ring of three K-steps of activation rows (32 KB
//     each) and a ring of two of weight rows.  Group 0 requests the activation rows two K-steps
//     ahead, into the slot both groups finished reading two phases earlier; group 1 requests the
//     weight rows two K-steps ahead into the slot it has just read itself (group 0 read the same
//     rows one phase earlier), once its own weight fragments are in registers.  Every request has
//     three to four phases to land, and each wavefront issues its 8 loads of a K-step in its M
//     phase, between fragment reads.  A K-step is 2 x 1024 clocks of MFMA per SIMD and measures
//     about 2100 (s_memtime at the phase boundaries: M phase 820-865, C phase's MFMAs back to back),
//     at a shader clock of 1.3-1.6 GHz under this load (boxes differ): time, not clocks, is what is left to win,
//     i.e. less energy per K-step.  Its 64 KB of loads alone take 0.62 us per CU when the rows are up to 8 KB apart and 1.08 us when they
//     are 16 KB apart (K = 8192: the 512 rows of a tile pair then lie in 128 regions of 64 KB,
//     more than a CU's address translation holds), so the load stream has to be fed in every
//     phase and must not wait for anything.
//   - Waits count the wavefront's own loads (s_waitcnt vmcnt(8): everything but the 8 loads of
//     this K-step has landed); the barrier that ends a phase publishes the data.
//   - Workgroups are numbered in patch order (see grouped_gemm.hip): 4 row blocks x 8 column tiles
//     of one expert on an XCD at a time, sharing both operands through that XCD's L2.
//   - The epilogue sends the tile out 32 rows at a time through each wavefront's own corner of
//     LDS (the stages are dead by then), full 128-byte rows per store.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "common.hpp"
#include "grouped_gemm.hpp"
#include "rows.hpp"

namespace brt {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef const bf16x4 __attribute__((address_space(1)))* global_bf16x4;
typedef const __bf16 __attribute__((address_space(1)))* global_bf16;

constexpr int kWaves = 8;
constexpr int kMT = 4, kNT = 2;                       // 32 x 32 tiles per wavefront: 128 x 64
constexpr int kBM = 256, kBN = 256, kBK = 64;
constexpr int kRowB = kBK * 2;                        // bytes of one tile row in one stage: one cache line
constexpr int kTileB = kBM * kRowB;                   // one operand of one K-step: 32 KB
constexpr int kAStages = 3, kBStages = 2;
constexpr int kBBase = kAStages * kTileB;             // the weight ring follows the activation ring
constexpr int kLdsBytes = (kAStages + kBStages) * kTileB;  // 163840: all of a CU's LDS
constexpr int kSub = kBK / 16;                        // MFMA k-steps per stage
constexpr int kHead = 4;                              // MFMAs of a C phase issued ahead of the barrier
constexpr uint32_t kOutOfRange = 0x80000000u;         // buffer offset past any extent: reads as zero
constexpr int kXcds = 8, kCusPerXcd = 32, kPatchRows = 4;
constexpr int kImageRow = kNT * 32 * 2 + 16;          // padded row of a wavefront's 32-row output image
constexpr int kImageB = 32 * kImageRow;
static_assert(kWaves * kImageB <= kLdsBytes, "the output images must fit the stages");

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
// lds_base in M0).  Counts on vmcnt like any load; the compiler does not know it touches LDS,
// so every wait for such a load is written out below.
__device__ __forceinline__ void load_to_lds(const i32x4& rsrc, uint32_t voffset, uint32_t soffset,
                                            uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
               : "memory");
}

__device__ __forceinline__ void stream_out(const u32x4& v, u32x4* p) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(p), "v"(v) : "memory");
}

__device__ __forceinline__ void wait_loads_all() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); }
// everything but the 8 loads this wavefront issued in the current K-step has landed
__device__ __forceinline__ void wait_loads_but_8() { asm volatile("s_waitcnt vmcnt(8)" : : : "memory"); }
__device__ __forceinline__ void wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }
__device__ __forceinline__ void block_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
__device__ __forceinline__ void wave_fence() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

template <int ACT>
__global__ __launch_bounds__(kWaves * 64) void grouped_gemm_pingpong_kernel(GemmArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // the tile's coordinates pass through the first bytes of the stages, before any load lands there
  int* const s_tile = reinterpret_cast<int*>(smem);  // expert, first row, valid rows, column tile

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Wavefronts w and w + 4 share a SIMD: wm is the half of the tile's rows a wavefront owns and
  // also its ping-pong group; wn is its 64 columns.
  const int wm = wave >> 2, wn = wave & 3;

  // ---- which tile: patch order (grouped_gemm.hip) ----------------------------------------------
  const int xcd = blockIdx.x % kXcds, idx = blockIdx.x / kXcds;
  const int t = ((idx / kCusPerXcd) * kXcds + xcd) * kCusPerXcd + idx % kCusPerXcd;
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
          const int local = t - first, per_group = kPatchRows * a.tiles_n;
          const int full = blocks / kPatchRows;
          const int g = local / per_group;
          int col, block;
          if (g < full) {
            const int r = local - g * per_group;
            col = r / kPatchRows;
            block = g * kPatchRows + r % kPatchRows;
          } else {
            const int last = blocks - full * kPatchRows;
            const int r = local - full * per_group;
            col = r / last;
            block = full * kPatchRows + r % last;
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
  if (e < 0) return;  // beyond the last entry of the list
  const int row0 = __builtin_amdgcn_readfirstlane(s_tile[1]);
  const int rows = min(__builtin_amdgcn_readfirstlane(s_tile[2]), a.P - row0);
  const int n0 = __builtin_amdgcn_readfirstlane(s_tile[3]) * kBN;
  const int K = a.K;
  const int k_tiles = K / kBK;
  __syncthreads();  // everyone has read the coordinates; the loads may overwrite them

  // ---- global -> LDS ---------------------------------------------------------------------------
  // A load fills one row group: 8 tile rows, a whole 128-byte line of each.  Group 0 loads the
  // activation rows, wavefront wn taking row groups wn + 4 i (i = 0..7); group 1 the weight rows,
  // wavefront wn taking the 64 rows of its own columns, row groups 8 wn + i.  Lane l lands at slot
  // l & 7 of row l >> 3 of the group and fetches chunk (l & 7) ^ ((row >> 1) & 7) of that row.  The
  // lane's row inside the group and its chunk are the vector offset; the row group and the K-step
  // go into the scalar offset, so no per-load register stays live.  A row that does not exist
  // (past the expert's last row, past N) gets an offset past any extent: zeros, no memory request.
  const __bf16* const w_e = a.w[e];
  const i32x4 res_a = make_rsrc(a.x + static_cast<size_t>(row0) * K, static_cast<size_t>(a.P - row0) * K * 2);
  const i32x4 res_b = make_rsrc(w_e + static_cast<size_t>(n0) * K, static_cast<size_t>(a.N - n0) * K * 2);
  const int cols = a.N - n0;  // weight rows that exist from n0 on
  const uint32_t chunk_a = (lane & 7) ^ (((wn & 1) << 2) | (lane >> 4));
  const int row_a = wn * 8 + (lane >> 3);
  const uint32_t off_a = (static_cast<uint32_t>(row_a) * K + chunk_a * 8) * 2;
  const uint32_t step_a = static_cast<uint32_t>(32) * K * 2;  // 4 row groups further
  const uint32_t chunk_b = (lane & 7) ^ (lane >> 4);           // even row group; odd ones flip bit 2 (byte 64)
  const int row_b = wn * 64 + (lane >> 3);
  const uint32_t off_b = (static_cast<uint32_t>(row_b) * K + chunk_b * 8) * 2;
  const uint32_t step_b = static_cast<uint32_t>(8) * K * 2;   // 1 row group further
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem)));
  auto load_a = [&](int kt, uint32_t slot, int i) {
    const uint32_t off = row_a + i * 32 < rows ? off_a : kOutOfRange;
    load_to_lds(res_a, off, kt * kRowB + i * step_a, lds0 + slot + (wn + 4 * i) * 1024);
  };
  auto load_b = [&](int kt, uint32_t slot, int i) {
    const uint32_t off = row_b + i * 8 < cols ? off_b ^ ((i & 1) << 6) : kOutOfRange;
    load_to_lds(res_b, off, kt * kRowB + i * step_b, lds0 + kBBase + slot + (wn * 8 + i) * 1024);
  };

  // ---- fragments -------------------------------------------------------------------------------
  // MFMA operand: this lane feeds row (lane % 32), k-half (lane / 32) of a 32 x 16 block; chunk
  // ks * 2 + lane / 32 of the row sits in slot chunk ^ ((row >> 1) & 7)
  const int frag_row = lane & 31, frag_k = lane >> 5;
  const int swz = (frag_row >> 1) & 7;
  const int frag_x = (wm * kMT * 32 + frag_row) * kRowB;
  const int frag_w = kBBase + (wn * kNT * 32 + frag_row) * kRowB;
  auto frag_off = [&](int ks) { return ((ks * 2 + frag_k) ^ swz) << 4; };

  f32x16 acc[kMT][kNT];
#pragma unroll
  for (int i = 0; i < kMT; ++i)
#pragma unroll
    for (int j = 0; j < kNT; ++j) acc[i][j] = f32x16{};
  bf16x8 fw[kSub][kNT], fx[kSub][kMT];
  // row tiles of this wavefront that hold rows (wave-uniform)
  const int n_i = __builtin_amdgcn_readfirstlane(min(max((rows - wm * kMT * 32 + 31) >> 5, 0), kMT));

  // prologue: K-steps 0 and 1
  if (wm == 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) load_a(0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) load_a(1, kTileB, i);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) load_b(0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) load_b(1, kTileB, i);
  }
  wait_loads_all();
  block_barrier();
  // Group 1 starts one phase late.  From here on a barrier ends group 0's M phase and group 1's C
  // phase, the next one group 0's C phase and group 1's M phase, and so on.
  if (wm == 1) block_barrier();
  // The K loop, for a wavefront whose first NI row tiles hold rows.  A ragged expert's last row
  // block reads no fragments and issues no MFMAs for the other row tiles, so a block of few rows
  // runs at the pace of its weight stream instead of that of 256 rows of matrix work.  The
  // wavefronts of a workgroup may run different instances: the barriers and the requests are the same in all.
  auto k_loop = [&](auto ni_tag) {
    constexpr int NI = decltype(ni_tag)::value;
    uint32_t a_cur = 0, a_load = 2 * kTileB;  // ring slots: the K-step being read, the one being requested
    for (int kt = 0; kt < k_tiles; ++kt) {
      const uint32_t b_cur = (kt & 1) * kTileB;
      const bool more = kt + 2 < k_tiles;
      const char* const pa = smem + a_cur + frag_x;
      const char* const pb = smem + b_cur + frag_w;
      // ---- M phase: fragments of K-step kt into registers, requests for K-step kt + 2 ----------
      if constexpr (NI > 0) {
#pragma unroll
        for (int ks = 0; ks < kSub; ++ks)
#pragma unroll
          for (int j = 0; j < kNT; ++j) fw[ks][j] = *reinterpret_cast<const bf16x8*>(pb + frag_off(ks) + j * 32 * kRowB);
      }
      if (wm == 0) {
        // the activation rows go into the slot that held K-step kt - 1: both groups have read it
#pragma unroll
        for (int ks = 0; ks < kSub; ++ks) {
#pragma unroll
          for (int i = 0; i < kMT; ++i) {
            if constexpr (NI > 0) {
              if (i < NI) fx[ks][i] = *reinterpret_cast<const bf16x8*>(pa + frag_off(ks) + i * 32 * kRowB);
            }
            if ((i & 1) && more) load_a(kt + 2, a_load, ks * 2 + (i >> 1));
          }
        }
        wait_lds();
      } else {
        // the weight rows go into the slot this wavefront is reading: group 0 read these rows a
        // phase ago, and this wavefront's own weight fragments are in registers after the wait
        wait_lds();
#pragma unroll
        for (int ks = 0; ks < kSub; ++ks) {
#pragma unroll
          for (int i = 0; i < kMT; ++i) {
            if constexpr (NI > 0) {
              if (i < NI) fx[ks][i] = *reinterpret_cast<const bf16x8*>(pa + frag_off(ks) + i * 32 * kRowB);
            }
            if ((i & 1) && more) load_b(kt + 2, b_cur, ks * 2 + (i >> 1));
          }
        }
        wait_lds();
        // the weight rows of K-step kt + 1 have landed (group 0 reads them after this barrier)
        if (more) wait_loads_but_8();
        else wait_loads_all();
      }
      // MFMAs [first, last) of the K-step's 8 x NI, in (ks, i, j) order
      auto multiply = [&](auto first_tag, auto last_tag) {
        constexpr int kFirst = decltype(first_tag)::value, kLast = decltype(last_tag)::value;
#pragma unroll
        for (int ks = 0; ks < kSub; ++ks)
#pragma unroll
          for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < kNT; ++j) {
              const int n = (ks * NI + i) * kNT + j;
              if (n >= kFirst && n < kLast)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[ks][j], fx[ks][i], acc[i][j], 0, 0, 0);
            }
      };
      // ---- C phase: nothing but the MFMAs of the K-step.  The first kHead of them are issued
      // before the barrier: they queue up behind the other group's last MFMAs and keep the matrix
      // pipe fed while the barrier lets both groups through (2.5 % on every shape measured; with 8
      // instead of 4 the group reaches the barrier too late for the other one's M phase).
      __builtin_amdgcn_sched_barrier(0);
      multiply(std::integral_constant<int, 0>{}, std::integral_constant<int, kHead>{});
      __builtin_amdgcn_sched_barrier(0);
      block_barrier();
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(1);
      multiply(std::integral_constant<int, kHead>{}, std::integral_constant<int, kSub * kMT * kNT>{});
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      if (wm == 0) {  // the activation rows of K-step kt + 1 have landed
        if (more) wait_loads_but_8();
        else wait_loads_all();
      }
      block_barrier();
      a_cur = a_cur == 2 * kTileB ? 0 : a_cur + kTileB;
      a_load = a_load == 2 * kTileB ? 0 : a_load + kTileB;
    }
  };
  const long long clock0 = __builtin_amdgcn_s_memtime(), tick0 = __builtin_amdgcn_s_memrealtime();
  if (n_i > 2) k_loop(std::integral_constant<int, 4>{});
  else if (n_i > 0) k_loop(std::integral_constant<int, 2>{});
  else k_loop(std::integral_constant<int, 0>{});
  if (a.clocks != nullptr && t == 0 && tid == 0) {  // measurement aid: this wavefront's K loop
    a.clocks[0] = __builtin_amdgcn_s_memtime() - clock0;
    a.clocks[1] = __builtin_amdgcn_s_memrealtime() - tick0;
    a.clocks[2] = k_tiles;
  }
  if (wm == 0) block_barrier();  // group 1's last C phase
  block_barrier();               // no wavefront reads a stage any more: the epilogue may write over them

  // ---- epilogue: bias + activation, bf16, 32 rows at a time through this wavefront's image -----
  // transposed accumulator: element r of tile (i, j) is output row 32 i + lane % 32, column (of the
  // wavefront's 32 j .. 32 j + 31) 8 * (r / 4) + 4 * (lane / 32) + r % 4, i.e. a lane holds 4
  // consecutive columns (8 bytes) of its row.
  const global_bf16 bias = a.bias != nullptr ? (global_bf16)(a.bias[e]) : (global_bf16)nullptr;
  char* const image = smem + wave * kImageB;
  const int mine = rows - wm * kMT * 32;  // rows of the tile this wavefront holds
  const int col_w = n0 + wn * kNT * 32;   // first column of this wavefront
  __bf16* const out_w = a.out + (static_cast<size_t>(row0) + wm * kMT * 32) * a.N + col_w;
  constexpr int kChunksPerRow = kNT * 32 / 8;  // 8 chunks of 16 bytes
  // the bias of this lane's columns, all eight loads in one round trip
  bf16x4 bv[kNT][4];
#pragma unroll
  for (int j = 0; j < kNT; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int col = col_w + j * 32 + 8 * g + 4 * frag_k;
      bv[j][g] = bf16x4{};
      if (bias != nullptr && col < a.N) bv[j][g] = *(global_bf16x4)(bias + col);
    }
#pragma unroll
  for (int i = 0; i < kMT; ++i) {
    if (i * 32 >= mine) break;  // wave-uniform
#pragma unroll
    for (int j = 0; j < kNT; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = j * 32 + 8 * g + 4 * frag_k;  // inside the wavefront's 64 columns
        const bf16x4 b4 = bv[j][g];
        bf16x4 o;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          o[q] = static_cast<__bf16>(apply_act<ACT>(acc[i][j][4 * g + q] + static_cast<float>(b4[q])));
        *reinterpret_cast<bf16x4*>(image + frag_row * kImageRow + col * 2) = o;
      }
    }
    wave_fence();
    const int rows_i = min(32, mine - i * 32);
    for (int q = lane; q < rows_i * kChunksPerRow; q += kWave) {
      const int rl = q / kChunksPerRow, c = q - rl * kChunksPerRow;
      if (col_w + c * 8 < a.N) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(image + rl * kImageRow + c * 16);
        u32x4* to = reinterpret_cast<u32x4*>(out_w + static_cast<size_t>(i * 32 + rl) * a.N + c * 8);
        if (a.plain_out) *to = v;
        else stream_out(v, to);
      }
    }
    wave_fence();
  }
}

template <int ACT>
int launch_pingpong(GemmArgs& a, hipStream_t st) {
  a.tiles_n = (a.N + kBN - 1) / kBN;
  // the sum over experts of ceil(M_e / 256) never exceeds P / 256 + E; whole rounds of XCD patches
  const long entries = (static_cast<long>(a.P + kBM - 1) / kBM + a.E) * a.tiles_n;
  const long round = kXcds * kCusPerXcd;
  const long grid = (entries + round - 1) / round * round;
  auto* fn = &grouped_gemm_pingpong_kernel<ACT>;
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(fn), kLdsBytes); rc != BRT_OK) return rc;
  hipLaunchKernelGGL(fn, dim3(static_cast<unsigned>(grid)), dim3(kWaves * 64), kLdsBytes, st, a);
  return check_launch("grouped_gemm_pingpong_kernel");
}

}  // namespace

// Shapes the ping-pong tiles take: plain bf16 GEMMs (no gather / scatter, no fp32 output) with K
// in whole K-steps of 64 and at least two of them.
bool pingpong_gemm_applies(const GemmArgs& a) {
  return a.tags == nullptr && a.out_f32 == nullptr && a.gates == nullptr && a.K % kBK == 0 && a.K >= 2 * kBK;
}

int launch_pingpong_gemm(GemmArgs& a, int act, hipStream_t st) {
  if (act == BRT_ACT_GELU) return launch_pingpong<BRT_ACT_GELU>(a, st);
  if (act == BRT_ACT_RELU) return launch_pingpong<BRT_ACT_RELU>(a, st);
  return launch_pingpong<BRT_ACT_NONE>(a, st);
}

}  // namespace brt
