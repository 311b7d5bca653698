// Grouped expert GEMM: out[rows of expert e] = act(x[rows of e] @ W_e^T + b_e) for
// every expert in ONE launch, ragged row counts read from the device.
//
// Call contract of the reference's homo-fused kernel (python/brt/jit/compiler.py:29-31,
// src/backend/torch/jit.cc:54-75, src/jit/compiler.cu:151-246): shared input and
// output buffers hold the experts' rows back to back in expert order, per-expert
// weights are separate tensors in torch Linear layout [N,K].  The reference glues
// per-capacity TVM fp32 kernels together and needs the capacities on the host;
// here the tile -> (expert, row block) map is computed on the device from
// `loads`, so any non-negative loads work and nothing is copied to the host.
//
// Tiling (CDNA4, wave64).  The expert FFN is a skinny GEMM (at most a few hundred
// rows per expert) whose cost is streaming the weights, so the tile is chosen to
// read them once: a workgroup owns BM = 32*MT rows (160 covers a whole capacity-
// padded Switch expert) by BN = 32*WAVES columns, every wavefront owning all BM
// rows of its own 32 columns.  Both operands are K-contiguous in memory, which is
// the MFMA operand layout (a lane feeds 8 consecutive k of one row), so tiles
// travel global -> registers -> LDS as 16-byte chunks without any transpose and
// come back as ds_read_b128 fragments; chunk c of row r lives in slot
// c ^ ((r >> 1) & 7), so that any 16 consecutive rows read at the same k cover all
// 64 banks exactly once (a row is 32 banks wide: even and odd rows take the two
// halves, and the 8 rows of one parity take 8 different slots) without padding.  The loop is bound by memory latency, not by MFMA issue, so it
// keeps two K-steps in flight in registers on top of the two LDS stages (one
// barrier per K-step of 64).  v_mfma_f32_32x32x16_bf16 is issued with the weight
// fragment as its first operand: the accumulator then holds the transposed tile,
// i.e. four consecutive output columns of one row per lane, which makes the
// epilogue (bias, GELU/ReLU, round to bf16) an 8-byte LDS write per group and the
// final stores full 16-byte, row-contiguous accesses.
//
// Workgroups are renumbered so that the column tiles of one row block run on the
// same XCD (hardware deals workgroups round-robin over the 8 XCDs) and share that
// XCD's L2 copy of the activation rows, while row blocks alternate between XCDs.
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
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
// Pointers read from the per-expert table are generic to the compiler, which would
// make every weight load a flat load counted on the LDS counter as well; the
// explicit global address space keeps weight loads off the LDS wait path.
typedef const __bf16 __attribute__((address_space(1)))* global_bf16;
typedef const u32x4 __attribute__((address_space(1)))* global_u32x4;
typedef const bf16x4 __attribute__((address_space(1)))* global_bf16x4;

constexpr int kBK = 64;               // k elements per stage
constexpr int kChunks = kBK / 8;      // 16-byte chunks per tile row
constexpr int kRowBytes = kBK * 2;    // LDS row (swizzled, unpadded)
constexpr int kXcds = 8;

// Cache policy of the weight loads (auxiliary operand of the buffer load: bit 1 = non-temporal on
// gfx94x/gfx950).  Every weight byte is read exactly once per launch; loaded as a stream it does
// not push the activation rows, which the column tiles of a row block share, out of the L2.
constexpr int kStreamingLoad = 2;

// Store of 16 output bytes with the streaming policy and system scope (`sc1 nt`): written
// through at once, the tile leaves no dirty lines behind for the end of the kernel to write back.
// The next kernel starts that much sooner: the two GEMMs of the benchmark FFN launched back to
// back take 143.7 us with this policy, 148.6 us with `nt` alone (what __builtin_nontemporal_store
// gives), 152 us with `sc1` or `sc0 sc1`, 160 us with ordinary stores; each GEMM on its own takes
// the same time with `nt` and `sc1 nt`.  There is no builtin for the pair of bits.
__device__ __forceinline__ void stream_out(const u32x4& v, u32x4* p) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(p), "v"(v) : "memory");
}

template <int N>
struct Staged {
  u32x4 v[N];
};

template <int MT, int NT, int WAVES, int ACT, bool WALKS, bool WSTREAM, bool OUTF32 = false>
__global__ __launch_bounds__(WAVES * 64) void grouped_gemm_kernel(GemmArgs a) {
  static_assert(!(OUTF32 && WALKS), "the fp32 epilogue is built for one column tile per workgroup");
  constexpr int THREADS = WAVES * 64;
  constexpr int BM = MT * 32, WN = NT * 32, BN = WAVES * WN;
  constexpr int TILE_ROWS = BM + BN;  // activation rows first, then weight rows
  constexpr int STAGE = TILE_ROWS * kRowBytes;
  constexpr int ROWS_PER_PASS = THREADS / kChunks;  // rows one load instruction of the block covers
  constexpr int A_LOADS = (BM + ROWS_PER_PASS - 1) / ROWS_PER_PASS;
  constexpr int B_LOADS = BN / ROWS_PER_PASS;
  constexpr bool A_EXACT = BM % ROWS_PER_PASS == 0;
  static_assert(BN % ROWS_PER_PASS == 0 && ROWS_PER_PASS % 8 == 0, "tile shape");
  constexpr int OUT_ROW = BN * 2 + 16;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  __shared__ int s_tile[5];  // expert, first row, valid rows, first row counted inside the expert, column group (patch order)
  __shared__ int s_cell[BM];  // routed forms: 0-based cell behind each row of the tile, -1 = empty slot
  __shared__ float s_gate[BM];  // accumulate form: the weight of each row of the tile

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- which tile: XCD-aware renumbering, then expert lookup from the loads ----------
  // hardware deals workgroups round-robin over the XCDs: workgroup b runs on XCD b % 8.
  // Row blocks are dealt round-robin too (row block m on XCD m % 8, so the row blocks
  // that really exist -- only the device knows how many -- spread evenly), and the
  // column tiles of one row block are consecutive workgroups of that XCD.
  const int xcd = blockIdx.x % kXcds, idx = blockIdx.x / kXcds;
  int mt = 0, nt_first = 0;
  if (a.patch == 0) {
    mt = (idx / a.groups_n) * kXcds + xcd;
    nt_first = (idx % a.groups_n) * a.walk;
    if (mt >= a.tiles_m_max) return;
    if (tid < kWave) {
      int carry_t = 0, carry_m = 0;
      bool found = false;
      for (int base = 0; base < a.E && !found; base += kWave) {
        const int e = base + lane;
        const int m = e < a.E ? a.loads[e] : 0;
        const int tiles = (m + BM - 1) / BM;
        const int incl_t = wave_inclusive_scan(tiles), incl_m = wave_inclusive_scan(m);
        const int first_tile = carry_t + incl_t - tiles;
        const bool hit = mt >= first_tile && mt < first_tile + tiles;
        const unsigned long long b = __ballot(hit);
        if (b != 0) {
          found = true;
          if (hit) {
            const int local = mt - first_tile;
            s_tile[0] = e;
            s_tile[1] = carry_m + incl_m - m + local * BM;
            s_tile[2] = min(BM, m - local * BM);
            s_tile[3] = local * BM;
          }
        }
        carry_t += __shfl(incl_t, kWave - 1, kWave);
        carry_m += __shfl(incl_m, kWave - 1, kWave);
      }
      if (!found && lane == 0) {  // beyond the last row block: how far, and where the rows end
        s_tile[0] = -1;
        s_tile[1] = carry_m;
        s_tile[2] = mt - carry_t;
      }
    }
  } else {
    // Patch order, for experts with several row blocks (plain form only): the workgroups are an
    // ordered list -- expert by expert; inside an expert groups of kPatchRows row blocks; inside
    // a group the row block changes fastest, then the column group -- and the 32 workgroups an XCD
    // runs at one time take 32 consecutive entries: kPatchRows row blocks x 8 column groups of one
    // expert, which share the activation rows AND the weight tiles through that XCD's L2.  With
    // the row blocks of an expert dealt round-robin over the XCDs (the order above) every row
    // block streams the expert's weights from memory again.
    constexpr int kPatchRows = 4, kCusPerXcd = 32;
    const int t = ((idx / kCusPerXcd) * kXcds + xcd) * kCusPerXcd + idx % kCusPerXcd;
    if (tid < kWave) {
      int carry_t = 0, carry_m = 0;
      bool found = false;
      for (int base = 0; base < a.E && !found; base += kWave) {
        const int e = base + lane;
        const int m = e < a.E ? a.loads[e] : 0;
        const int blocks = (m + BM - 1) / BM;
        const int tiles = blocks * a.groups_n;
        const int incl_t = wave_inclusive_scan(tiles), incl_m = wave_inclusive_scan(m);
        const int first = carry_t + incl_t - tiles;
        const bool hit = t >= first && t < first + tiles;
        if (__ballot(hit) != 0) {
          found = true;
          if (hit) {
            const int local = t - first, per_group = kPatchRows * a.groups_n;
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
            s_tile[1] = carry_m + incl_m - m + block * BM;
            s_tile[2] = min(BM, m - block * BM);
            s_tile[3] = block * BM;
            s_tile[4] = col;
          }
        }
        carry_t += __shfl(incl_t, kWave - 1, kWave);
        carry_m += __shfl(incl_m, kWave - 1, kWave);
      }
      if (!found && lane == 0) s_tile[0] = -2;  // beyond the last entry of the list
    }
  }
  __syncthreads();
  const int e = __builtin_amdgcn_readfirstlane(s_tile[0]);
  if (e == -2) return;
  if (a.patch != 0) nt_first = __builtin_amdgcn_readfirstlane(s_tile[4]) * a.walk;
  const int nt_end = WALKS ? min(nt_first + a.walk, a.tiles_n) : nt_first + 1;  // this workgroup's column tiles
  if (e < 0) {
    // The row blocks past the last one clear the tags of the rows no path owns (the layout may be
    // allocated for more rows than the loads add up to): surplus block j takes rows
    // [total + j * BM, total + (j + 1) * BM); there are at least (P - total) / BM of them.
    if (a.row_tags_out != nullptr && nt_first == 0) {
      const long first = static_cast<long>(s_tile[1]) + static_cast<long>(s_tile[2]) * BM;
      for (long r = first + tid; r < min(first + BM, static_cast<long>(a.P)); r += THREADS) a.row_tags_out[r] = 0;
    }
    return;
  }
  const int row0 = __builtin_amdgcn_readfirstlane(s_tile[1]);
  const int rows = __builtin_amdgcn_readfirstlane(s_tile[2]);
  const int seat0 = __builtin_amdgcn_readfirstlane(s_tile[3]);
  const int row_tiles = (rows + 31) >> 5;
  int n0 = nt_first * BN;
  const int K = a.K;

  // ---- global -> register staging ------------------------------------------------
  // Thread t owns 16-byte chunk t%8 of rows t/8 + i*ROWS_PER_PASS of the activation
  // tile and of the weight tile.  Rows past the expert's last row or past N address
  // past the buffer extent and read as zeros (their products land in output
  // rows/columns that are never stored, and all MT row tiles are always multiplied:
  // the inner loop stays one branch-free block); a K tail that is not a multiple of
  // 64 is zeroed when it is written to LDS.
  const int lc = tid % kChunks, lr = tid / kChunks;
  // Buffer loads: a wave-uniform resource (base, byte extent) per operand, a 32-bit
  // per-lane byte offset and the K offset as the scalar offset, so the loop carries no
  // 64-bit address arithmetic; reads past the extent return zero instead of faulting.
  // Gather mode: row s of expert e is cell tags[s,e]-1 of x (the dispatch is folded into the
  // operand load); an empty tag addresses past the extent and so reads a row of zeros, which
  // is what dispatch writes for a padding row.
  const bool gather = a.gather != 0;
  // Routed forms: the 0-based cell behind every row of this tile (-1 for an empty slot), from
  // the tag matrix (seat seat0 + r of column e) or from the row-entry vector of the compact route
  // (entry t*k+j+1 of row row0 + r of the dispatched layout).  One load per row, all of them in
  // one memory round trip, kept in LDS for the operand offsets below and for the store loop of
  // the epilogue.
  if (a.tags != nullptr) {
    for (int r = tid; r < rows; r += THREADS) {
      int cell;
      size_t gate_at;  // accumulate form: where the row's weight stands
      if (a.tag_vector) {
        const int entry = a.tags[static_cast<size_t>(row0) + r];
        cell = a.tag_div > 1 ? (entry - 1) / a.tag_div : entry - 1;
        cell = (entry >= 1 && cell < a.T) ? cell : -1;
        gate_at = static_cast<size_t>(max(entry, 1)) - 1;
      } else {
        // the tag matrix has T rows; a load padded beyond T (capacity above the batch size) names
        // slots that do not exist: they are empty, as in dispatch (route.cu:84-92 bounds the slot
        // by the cell count)
        const int slot = seat0 + r;
        const int tag = slot < a.T ? a.tags[static_cast<size_t>(slot) * a.E + e] : 0;
        cell = (tag >= 1 && tag <= a.T) ? tag - 1 : -1;
        gate_at = static_cast<size_t>(max(cell, 0)) * a.E + e;
      }
      s_cell[r] = cell;
      if (a.gates != nullptr) s_gate[r] = a.gates[cell >= 0 ? gate_at : 0];  // entry 0 for an empty slot: never used
      // side output for a combine that runs later: the cell of every row, written once per row block
      if (a.row_tags_out != nullptr && nt_first == 0) a.row_tags_out[static_cast<size_t>(row0) + r] = cell + 1;
    }
    __syncthreads();
  }
  const char* xa = reinterpret_cast<const char*>(gather ? a.x : a.x + static_cast<size_t>(row0) * K);
  const __bf16* const w_e = a.w[e];
  const size_t xa_bytes = static_cast<size_t>(gather ? a.T : a.P - row0) * K * 2;
  const __amdgpu_buffer_rsrc_t res_a = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(xa), 0, static_cast<int>(std::min<size_t>(xa_bytes, 0x7fffffff)), 0x00020000);
  // weight rows from column `first` on; rows past N lie past the extent and read as zeros
  auto weight_rows = [&](int first) {
    const size_t bytes = static_cast<size_t>(a.N - first) * K * 2;
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(reinterpret_cast<const char*>(w_e + static_cast<size_t>(first) * K)), 0,
        static_cast<int>(std::min<size_t>(bytes, 0x7fffffff)), 0x00020000);
  };
  __amdgpu_buffer_rsrc_t res_b = weight_rows(n0);
  // when ROWS_PER_PASS does not divide BM only the lower wavefronts take the last pass
  const bool a_last = A_EXACT || lr + (A_LOADS - 1) * ROWS_PER_PASS < BM;
  uint32_t off_a[A_LOADS], off_b[B_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    // rows past the expert's last one address past the extent: they read as zeros and cost no
    // memory request (their products land in output rows that are never stored)
    const int r = lr + i * ROWS_PER_PASS;
    const bool in_tile = r < rows;
    if (gather) {
      const int cell = in_tile ? s_cell[r] : -1;
      off_a[i] = cell >= 0 ? (static_cast<uint32_t>(cell) * K + lc * 8) * 2 : 0x80000000u;
    } else {
      off_a[i] = in_tile ? (static_cast<uint32_t>(r) * K + lc * 8) * 2 : 0x80000000u;
    }
  }
#pragma unroll
  for (int i = 0; i < B_LOADS; ++i)
    off_b[i] = (static_cast<uint32_t>(lr + i * ROWS_PER_PASS) * K + lc * 8) * 2;
  // LDS slot of chunk c of row r is c ^ ((r >> 1) & 7).  A thread's rows are ROWS_PER_PASS
  // apart; the pass offset changes the swizzle term by a compile-time constant (0, or 4 for
  // every other pass of the 3-wavefront tile), i.e. it flips one bit of the slot.
  const int slot = lr * kRowBytes + ((lc ^ ((lr >> 1) & 7)) << 4);
  auto pass_flip = [](int first_row) { return (((first_row >> 1) & 7) << 4); };  // xor on the byte offset
  static_assert(ROWS_PER_PASS % 8 == 0 && BM % 16 == 0, "the pass offset must flip whole slot bits");
  const bool k_tail = (K % kBK) != 0;

  using Yes = std::integral_constant<bool, true>;
  using No = std::integral_constant<bool, false>;
  constexpr int LOADS = A_LOADS + B_LOADS;
  constexpr int kSteps = kBK / 16;
  // Loads and LDS writes are issued in kSteps slices so that they can be spread over
  // the k-steps of the multiply; slice p covers loads [p*LOADS/kSteps, (p+1)*LOADS/kSteps).
  auto fetch_slice = [&](Staged<LOADS>& s, int k0, int p) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      if (i < p * LOADS / kSteps || i >= (p + 1) * LOADS / kSteps) continue;
      if (i < A_LOADS) {
        if (i + 1 < A_LOADS || a_last)
          s.v[i] = __builtin_amdgcn_raw_buffer_load_b128(res_a, off_a[i < A_LOADS ? i : 0], k0 * 2, 0);
      } else {
        s.v[i] = __builtin_amdgcn_raw_buffer_load_b128(res_b, off_b[i >= A_LOADS ? i - A_LOADS : 0],
                                                       k0 * 2, WSTREAM ? kStreamingLoad : 0);
      }
    }
  };
  // the K tail (only ever in the last tile) is zeroed here, when the data is in registers
  auto stash_slice = [&](const Staged<LOADS>& s, int stage, int k0, int p, auto may_be_last) {
    char* stage_base = smem + stage * STAGE;
    const bool k_ok = !decltype(may_be_last)::value || !k_tail || k0 + lc * 8 < K;
    const u32x4 z = {};
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      if (i < p * LOADS / kSteps || i >= (p + 1) * LOADS / kSteps) continue;
      const u32x4 v = k_ok ? s.v[i] : z;
      if (i < A_LOADS) {
        if (i + 1 < A_LOADS || a_last)
          *reinterpret_cast<u32x4*>(stage_base + ((slot ^ pass_flip(i * ROWS_PER_PASS)) +
                                                  i * ROWS_PER_PASS * kRowBytes)) = v;
      } else {
        *reinterpret_cast<u32x4*>(stage_base + ((slot ^ pass_flip(BM + (i - A_LOADS) * ROWS_PER_PASS)) +
                                                (BM + (i - A_LOADS) * ROWS_PER_PASS) * kRowBytes)) = v;
      }
    }
  };

  f32x16 acc[MT][NT];

  // MFMA operand: this lane feeds row (lane % 32), k-half (lane / 32) of a 32 x 16 block
  const int frag_row = lane & 31, frag_k = lane >> 5;

  // One K-step of 64: multiply the tile in LDS stage `stage`; meanwhile write the tile
  // that has arrived in `arrived` (K offset k_arrived) to the other stage and start
  // loading the tile after that (K offset k_fetch) into `incoming`.  With one wavefront
  // per SIMD nothing hides a stalled instruction stream, so every 16-wide k-step is
  // issued as MFMA, memory op, MFMA, memory op, ...: the global loads, the fragment
  // reads of the next k-step and the LDS writes each ride behind an MFMA that keeps the
  // matrix pipe busy while they issue.
  auto step = [&](int stage, Staged<LOADS>& incoming, const Staged<LOADS>& arrived, int k_fetch,
                  int k_arrived, auto do_fetch, auto do_stash, auto last_tile) {
    constexpr bool kFetch = decltype(do_fetch)::value, kStash = decltype(do_stash)::value;
    const char* sa = smem + stage * STAGE + frag_row * kRowBytes;
    const char* sb = sa + (BM + wave * WN) * kRowBytes;
    bf16x8 fw[2][NT], fx[2][MT];
    auto read_frags = [&](int ks, int buf) {
      const int phys = ((ks * 2 + frag_k) ^ ((frag_row >> 1) & 7)) << 4;
#pragma unroll
      for (int j = 0; j < NT; ++j)
        fw[buf][j] = *reinterpret_cast<const bf16x8*>(sb + j * 32 * kRowBytes + phys);
#pragma unroll
      for (int i = 0; i < MT; ++i)
        fx[buf][i] = *reinterpret_cast<const bf16x8*>(sa + i * 32 * kRowBytes + phys);
    };
    read_frags(0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks) {
      if constexpr (kFetch) fetch_slice(incoming, k_fetch, ks);
      if (ks + 1 < kSteps) read_frags(ks + 1, (ks + 1) & 1);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[ks & 1][j], fx[ks & 1][i],
                                                              acc[i][j], 0, 0, 0);
      if constexpr (kStash) stash_slice(arrived, stage ^ 1, k_arrived, ks, last_tile);
      // issue order of this k-step: one MFMA, then at most one op of each memory kind
      constexpr int kSlice = (LOADS + kSteps - 1) / kSteps;
      constexpr int kReads = MT + NT;
#pragma unroll
      for (int m = 0; m < MT * NT; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                     // MFMA
        if (m < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      // LDS read
        if (kFetch && m < kSlice) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // global load
        if (kStash && m >= MT * NT - kSlice) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // LDS write
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- K loop: tile kt in LDS stage kt&1, tile kt+1 in one register set (written to LDS
  // during step kt), tile kt+2 being loaded into the other ------------------------------
  // A workgroup walks `walk` column tiles of its row block.  When K is a whole, even number
  // of K-steps the load stream does not stop at a tile boundary: the last two K-steps of a
  // tile already fetch the first two of the next one (same activation rows, next weight
  // rows), so the expert lookup and the two exposed load latencies are paid once per
  // workgroup and the next tile's operands arrive while the epilogue runs.
  const int k_tiles = (K + kBK - 1) / kBK;
  const bool seamless = !k_tail && (k_tiles & 1) == 0 && k_tiles >= 2;
  const global_bf16 bias = a.bias != nullptr ? (global_bf16)(a.bias[e]) : (global_bf16)nullptr;
  Staged<LOADS> s0, s1;
  // first K-step of the first tile into LDS stage 0
#pragma unroll
  for (int p = 0; p < kSteps; ++p) fetch_slice(s0, 0, p);
  if (!WALKS && k_tiles > 1) {  // one tile per workgroup: the second K-step starts right away
#pragma unroll
    for (int p = 0; p < kSteps; ++p) fetch_slice(s1, kBK, p);
  }
#pragma unroll
  for (int p = 0; p < kSteps; ++p) stash_slice(s0, 0, 0, p, Yes{});
  __syncthreads();
  for (int nt = nt_first; nt < nt_end; ++nt, n0 += BN) {
    // here LDS stage 0 holds the first K-step of this tile; the second one starts now.
    // Nothing is carried in registers from one tile to the next: a staged set or an
    // accumulator that lives around the tile loop costs the K loop more registers than
    // it has.
    if (WALKS && k_tiles > 1) {
#pragma unroll
      for (int p = 0; p < kSteps; ++p) fetch_slice(s1, kBK, p);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[i][j] = f32x16{};
    const bool ahead = seamless && nt + 1 < nt_end;  // the tail fetches into the next tile
    int kt = 0;
    for (; kt + 3 < k_tiles; kt += 2) {
      step(0, s0, s1, (kt + 2) * kBK, (kt + 1) * kBK, Yes{}, Yes{}, No{});
      __syncthreads();
      step(1, s1, s0, (kt + 3) * kBK, (kt + 2) * kBK, Yes{}, Yes{}, No{});
      __syncthreads();
    }
    if (ahead) {  // two K-steps left: the first K-step of the next tile rides along
      res_b = weight_rows(n0 + BN);
      step(0, s0, s1, 0, (kt + 1) * kBK, Yes{}, Yes{}, No{});
      __syncthreads();
      step(1, s1, s0, 0, 0, No{}, Yes{}, Yes{});
      __syncthreads();
    } else {
      const int left = k_tiles - kt;  // 1, 2 or 3 tiles; kt is even, so the next tile is in stage 0
      if (left == 3) {
        step(0, s0, s1, (kt + 2) * kBK, (kt + 1) * kBK, Yes{}, Yes{}, No{});
        __syncthreads();
        step(1, s1, s0, 0, (kt + 2) * kBK, No{}, Yes{}, Yes{});
        __syncthreads();
        step(0, s0, s1, 0, 0, No{}, No{}, No{});
      } else if (left == 2) {
        step(0, s0, s1, 0, (kt + 1) * kBK, No{}, Yes{}, Yes{});
        __syncthreads();
        step(1, s1, s0, 0, 0, No{}, No{}, No{});
      } else {
        step(0, s0, s1, 0, 0, No{}, No{}, No{});
      }
      __syncthreads();
    }

    // ---- epilogue: bias + activation, bf16, through LDS, 16-byte row stores -------------
    // transposed accumulator: element r of tile (i, j) is output row 32 i + lane%32, column
    // (of this wavefront's 32 j .. 32 j + 31) 8*(r/4) + 4*(lane/32) + r%4.
    // A walking workgroup sends the tile out in two passes of row tiles through LDS stage 1
    // only: stage 0 may already hold the first K-step of the next tile.  With one tile per
    // workgroup the whole tile is staged at once.
    // The per-lane addresses of the epilogue are recomputed from an opaque copy of the thread
    // index for every tile: as loop invariants of the column walk they would be hoisted into
    // registers that stay live across the K loop, which has none to spare.
    int tid_e = tid;
    asm volatile("" : "+v"(tid_e));
    const int frag_row_e = tid_e & 31, frag_k_e = (tid_e >> 5) & 1;
    float bv[NT][4][4];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = n0 + wave * WN + j * 32 + 8 * g + 4 * frag_k_e;
        bf16x4 b4 = {};
        if (a.bias != nullptr && col < a.N) b4 = *(global_bf16x4)(bias + col);
#pragma unroll
        for (int q = 0; q < 4; ++q) bv[j][g][q] = static_cast<float>(b4[q]);
      }
    }
    if constexpr (OUTF32) {
      // fp32 output (the contract of the reference's expert kernel): the accumulator leaves as it
      // is, 4 consecutive columns (16 bytes) per lane and store, no LDS.
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int r = i * 32 + frag_row_e;
        long to = a.scatter ? (r < rows ? s_cell[r] : -1) : static_cast<long>(row0) + r;
        if (i >= row_tiles || r >= rows || to < 0) continue;
        float* const orow = a.out_f32 + static_cast<size_t>(to) * a.N;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int col = n0 + wave * WN + j * 32 + 8 * g + 4 * frag_k_e;
            if (col >= a.N) continue;
            f32x4 o;
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = apply_act<ACT>(acc[i][j][4 * g + q] + bv[j][g][q]) + 0.0f;  // -0 -> +0, as a combine would
            *reinterpret_cast<f32x4*>(orow + col) = o;
          }
        }
      }
      continue;
    }
    constexpr int OUT_CHUNKS = BN / 8;
    constexpr int kPasses = WALKS ? 2 : 1;
    constexpr int kPassTiles = (MT + kPasses - 1) / kPasses;
    static_assert(!WALKS || kPassTiles * 32 * OUT_ROW <= STAGE, "half an output tile must fit one LDS stage");
    char* const stage_out = WALKS ? smem + STAGE : smem;
    // Scatter mode: row s of expert e goes to cell tags[s,e]-1 of out (the combine of a
    // single-path route is folded into the store); rows without a tag are dropped.
    __bf16* __restrict__ oc = a.out + (a.scatter ? 0 : static_cast<size_t>(row0) * a.N) + n0;
#pragma unroll
    for (int pass = 0; pass < kPasses; ++pass) {
      const int i_lo = pass * kPassTiles, i_hi = pass + 1 < kPasses ? kPassTiles : MT;
      if (pass == 1) __syncthreads();  // the first half has left LDS
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        if (i < i_lo || i >= i_hi) continue;
        if (i < row_tiles) {
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            char* dst = stage_out + ((i - i_lo) * 32 + frag_row_e) * OUT_ROW + (wave * WN + j * 32 + 4 * frag_k_e) * 2;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              bf16x4 o;
#pragma unroll
              for (int q = 0; q < 4; ++q)
                o[q] = static_cast<__bf16>(apply_act<ACT>(acc[i][j][4 * g + q] + bv[j][g][q]));
              *reinterpret_cast<bf16x4*>(dst + 16 * g) = o;
            }
          }
        }
      }
      __syncthreads();
      const int r_lo = i_lo * 32, r_hi = min(rows, i_hi * 32);
      if (a.gates != nullptr) {
        // Accumulate form: the weighted combine of a route with several paths per cell is folded
        // into the store (route.cu:236-243: `in * gate`, then an atomic add per element).  The
        // value is the row as the separate GEMM would have stored it (rounded to bf16), times the
        // gate in fp32, added to the fp32 output; 64 consecutive columns of one row per wavefront
        // and instruction.  Two addends per cell give the same bits in either order.
        float* const of = a.acc_out + n0;
        for (int q = tid_e; q < (r_hi - r_lo) * BN; q += THREADS) {
          const int rl = q / BN, c = q - rl * BN;
          const int r = r_lo + rl;
          const int to = s_cell[r];
          if (to >= 0 && n0 + c < a.N) {
            const float v = static_cast<float>(*reinterpret_cast<const __bf16*>(stage_out + rl * OUT_ROW + c * 2));
            unsafeAtomicAdd(of + static_cast<size_t>(to) * a.N + c, v * s_gate[r]);
          }
        }
        continue;
      }
      for (int q = tid_e; q < (r_hi - r_lo) * OUT_CHUNKS; q += THREADS) {
        const int rl = q / OUT_CHUNKS, c = q - rl * OUT_CHUNKS;
        const int r = r_lo + rl;
        long to = r;
        if (a.scatter) to = s_cell[r];
        // streaming stores: the output is not read again by this kernel, and written through the
        // L2 like ordinary stores it pushes the operand lines out that the column tiles share
        if (to >= 0 && n0 + c * 8 < a.N) {
          u32x4 v = *reinterpret_cast<const u32x4*>(stage_out + rl * OUT_ROW + c * 16);
          if (a.scatter) {  // the combine this store stands for adds the row to zero: -0 becomes +0
#pragma unroll
            for (int w = 0; w < 4; ++w) v[w] = plus_zero<BRT_BF16>(v[w]);
          }
          if (a.plain_out) *reinterpret_cast<u32x4*>(oc + static_cast<size_t>(to) * a.N + c * 8) = v;  // kept in the caches
          else stream_out(v, reinterpret_cast<u32x4*>(oc + static_cast<size_t>(to) * a.N + c * 8));
        }
      }
    }
    if (nt + 1 < nt_end) {
      __syncthreads();  // stage 1 is written again by the first K-step of the next tile
      if (!ahead) {  // K does not allow the seamless tail: load the next tile's first K-step now
        res_b = weight_rows(n0 + BN);
#pragma unroll
        for (int p = 0; p < kSteps; ++p) fetch_slice(s0, 0, p);
#pragma unroll
        for (int p = 0; p < kSteps; ++p) stash_slice(s0, 0, 0, p, Yes{});
        __syncthreads();
      }
    }
  }
}

int device_cus() {
  static const int cus = [] {
    int dev = 0, n = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    return std::max(n, 1);
  }();
  return cus;
}

// row blocks of 160 a capacity-filled route has; the loads themselves live on the device
long estimated_row_blocks(int P, int E) { return std::max<long>((P + 159) / 160, std::min(E, P)); }

template <int MT, int NT, int WAVES, int ACT>
int launch_act(GemmArgs& a, hipStream_t st) {
  constexpr int BM = MT * 32, BN = WAVES * NT * 32;
  constexpr int STAGE = (BM + BN) * kRowBytes;
  constexpr int OUT_BYTES = BM * (BN * 2 + 16);  // the epilogue stages the output tile in the same memory
  const size_t lds = std::max(2 * STAGE, OUT_BYTES);
  a.tiles_n = (a.N + BN - 1) / BN;
  // sum over experts of ceil(M_e/BM) never exceeds P/BM + E; rounded up to whole XCD rounds
  a.tiles_m_max = ((a.P + BM - 1) / BM + a.E + kXcds - 1) / kXcds * kXcds;
  // Column tiles one workgroup walks: the largest number that neither leaves CUs without a
  // workgroup nor adds a round of tiles to the busiest CU (estimated like the tile shape,
  // from the row blocks a capacity-filled route has; the loads themselves live on the device).
  constexpr int forced_walk = 0;  // a fixed walk length, for experiments
  a.walk = 1;
  if (WAVES == 4) {  // the narrower tiles stage more per thread and have no registers left for it
    const long slots = static_cast<long>(device_cus()) * (WAVES == 2 ? 2 : 1);
    const long row_blocks = estimated_row_blocks(a.P, a.E);
    const long plain = (row_blocks * a.tiles_n + slots - 1) / slots;
    for (int w = a.tiles_n; w > 1; --w) {
      const long groups = (a.tiles_n + w - 1) / w;
      if (row_blocks * groups >= slots && (row_blocks * groups + slots - 1) / slots * w <= plain) {
        a.walk = w;
        break;
      }
    }
  }
  if (forced_walk > 0) a.walk = std::min(forced_walk, a.tiles_n);
  a.groups_n = (a.tiles_n + a.walk - 1) / a.walk;
  // Weight loads are streamed (non-temporal) when a weight tile is read about once per launch:
  // experts of at most one row block on average.  Experts with many row blocks read their
  // weights once per row block, and those re-reads are served by the caches only if the first
  // read left the lines there.
  const bool stream_weights = static_cast<long>(a.P) <= static_cast<long>(a.E) * BM;
  // only the 4-wavefront tiles have the registers to walk column tiles
  constexpr bool kCanWalk = WAVES == 4;
  if (!kCanWalk) a.walk = 1, a.groups_n = a.tiles_n;
  // Experts with several row blocks (and no routing through tags): patch order, so that the row
  // blocks of an expert that run side by side on an XCD share its weight tiles.  Measured against
  // the round-robin order in one process: the ragged task-MoE shape (128 experts, Dirichlet loads)
  // 1652 -> 1596 us and 1443 -> 1379 us, 8 experts x 4096 rows 1106 -> 1053 us and 1019 -> 999 us,
  // the top-2 shape with three row blocks per expert the same within 2 %; 2, 8 or 16 row blocks per
  // patch instead of 4 change these by less than 1 %.
  a.patch = (a.tags == nullptr && !stream_weights) ? 1 : 0;
  long grid_wgs = static_cast<long>(a.tiles_m_max) * a.groups_n;
  if (a.patch) grid_wgs = (grid_wgs + 255) / 256 * 256;  // whole rounds of 32 workgroups per XCD
  const dim3 blocks(static_cast<unsigned>(grid_wgs)), threads(WAVES * 64);
  auto run = [&](auto walks, auto wstream) -> int {
    auto* fn = &grouped_gemm_kernel<MT, NT, WAVES, ACT, decltype(walks)::value, decltype(wstream)::value>;
    if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(fn), static_cast<int>(lds)); rc != BRT_OK) return rc;
    hipLaunchKernelGGL(fn, blocks, threads, lds, st, a);
    return check_launch("grouped_gemm_kernel");
  };
  using Yes = std::integral_constant<bool, true>;
  using No = std::integral_constant<bool, false>;
  if constexpr (kCanWalk) {
    if (a.walk > 1) return stream_weights ? run(Yes{}, Yes{}) : run(Yes{}, No{});
  }
  return stream_weights ? run(No{}, Yes{}) : run(No{}, No{});
}

// fp32 output: the 4-wavefront tile, one column tile per workgroup, ordinary weight loads
template <int ACT>
int launch_f32(GemmArgs& a, hipStream_t st) {
  constexpr int MT = 5, NT = 2, WAVES = 4, BM = MT * 32, BN = WAVES * NT * 32;
  constexpr int STAGE = (BM + BN) * kRowBytes;
  a.tiles_n = (a.N + BN - 1) / BN;
  a.tiles_m_max = ((a.P + BM - 1) / BM + a.E + kXcds - 1) / kXcds * kXcds;
  a.walk = 1;
  a.groups_n = a.tiles_n;
  auto* fn = &grouped_gemm_kernel<MT, NT, WAVES, ACT, false, false, true>;
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(fn), 2 * STAGE); rc != BRT_OK) return rc;
  const long grid_wgs = static_cast<long>(a.tiles_m_max) * a.groups_n;
  hipLaunchKernelGGL(fn, dim3(static_cast<unsigned>(grid_wgs)), dim3(WAVES * 64), 2 * STAGE, st, a);
  return check_launch("grouped_gemm_kernel (fp32 output)");
}

template <int MT, int NT, int WAVES>
int launch(GemmArgs& a, int act, hipStream_t st) {
  if (act == BRT_ACT_GELU) return launch_act<MT, NT, WAVES, BRT_ACT_GELU>(a, st);
  if (act == BRT_ACT_RELU) return launch_act<MT, NT, WAVES, BRT_ACT_RELU>(a, st);
  return launch_act<MT, NT, WAVES, BRT_ACT_NONE>(a, st);
}

}  // namespace
}  // namespace brt

using namespace brt;

namespace {

int grouped_gemm_impl(const void* x, const void* const* weights, const void* const* biases, void* out,
                      const int32_t* loads, const int32_t* tags, int entries_per_cell, int E, int P,
                      int T, int K, int N, int act, int gather_in, int scatter_out, void* stream,
                      bool out_is_f32 = false, int32_t* row_tags_out = nullptr,
                      const float* gates = nullptr, long long* clocks = nullptr) {
  if (E <= 0 || P < 0 || K <= 0 || N <= 0 || T < 0)
    return fail(BRT_E_INVALID, "bad shape E=%d P=%d T=%d K=%d N=%d", E, P, T, K, N);
  if (K % 8 != 0 || N % 8 != 0)
    return fail(BRT_E_UNSUPPORTED, "K and N must be multiples of 8 (16-byte rows), got K=%d N=%d", K, N);
  if (act != BRT_ACT_NONE && act != BRT_ACT_GELU && act != BRT_ACT_RELU)
    return fail(BRT_E_INVALID, "unknown activation %d", act);
  if (P == 0) return BRT_OK;
  if ((gather_in || scatter_out) && T == 0) return BRT_OK;
  if (!x || !weights || !out || !loads) return fail(BRT_E_INVALID, "null argument");
  if ((gather_in || scatter_out) && !tags) return fail(BRT_E_INVALID, "gather/scatter need the tag matrix");
  if (gather_in && static_cast<size_t>(T) * K * 2 > 0x7fffffffull)
    return fail(BRT_E_UNSUPPORTED, "gathered input of %d x %d exceeds 2 GiB", T, K);
  if (!aligned(x, 16) || !aligned(out, 16)) return fail(BRT_E_INVALID, "x/out must be 16-byte aligned");
  if (gates != nullptr && (!scatter_out || out_is_f32 || !aligned(gates, 4)))
    return fail(BRT_E_INVALID, "the accumulate form scatters into an fp32 output and needs 4-byte aligned gates");
  GemmArgs a{};
  a.x = static_cast<const __bf16*>(x);
  a.w = reinterpret_cast<const __bf16* const*>(weights);
  a.bias = reinterpret_cast<const __bf16* const*>(biases);
  a.out = (out_is_f32 || gates != nullptr) ? nullptr : static_cast<__bf16*>(out);
  a.out_f32 = out_is_f32 ? static_cast<float*>(out) : nullptr;
  a.gates = gates;
  a.acc_out = gates != nullptr ? static_cast<float*>(out) : nullptr;
  a.row_tags_out = tags != nullptr ? row_tags_out : nullptr;
  a.loads = loads;
  a.tags = tags;
  a.tag_vector = entries_per_cell > 0;
  a.tag_div = entries_per_cell;
  a.E = E; a.P = P; a.K = K; a.N = N; a.T = T;
  a.gather = gather_in != 0; a.scatter = scatter_out != 0;
  // Output stores.  A large output (the expanding GEMM of an FFN) is written with the streaming
  // policy: it would only push the operands out of the caches.  A small one that the next kernel
  // reads at once (the contracting GEMM: its rows go straight into the combine) is written with
  // ordinary stores and stays in the last-level cache: the benchmark layer's combine then costs
  // 4.9 us instead of 5.9 us and the GEMM itself nothing (measured inside the step; with ordinary
  // stores in the expanding GEMM that GEMM takes 102 us instead of 87 us).
  a.plain_out = N < K && static_cast<size_t>(P) * N * 2 <= (size_t{32} << 20);
  if (clocks != nullptr) {  // the timed form: the ping-pong kernel or nothing
    if (!pingpong_gemm_applies(a) || out_is_f32)
      return fail(BRT_E_UNSUPPORTED, "the timed form runs the ping-pong kernel only (bf16 output, no tags, K a multiple of 64 and >= 128)");
    a.clocks = clocks;
    return launch_pingpong_gemm(a, act, as_stream(stream));
  }
  if (out_is_f32) {
    if (act == BRT_ACT_GELU) return launch_f32<BRT_ACT_GELU>(a, as_stream(stream));
    if (act == BRT_ACT_RELU) return launch_f32<BRT_ACT_RELU>(a, as_stream(stream));
    return launch_f32<BRT_ACT_NONE>(a, as_stream(stream));
  }
  // Kernel choice.  Experts that average more than one row block take the ping-pong kernel
  // (grouped_gemm_pingpong.hip), whose 256 x 256 tile moves a third fewer operand bytes per flop,
  // when its tiles come in whole rounds over the CUs: at least two rounds, or one round that most
  // CUs take part in.  In between (one to two tiles per CU) a CU with two tiles sets the time and
  // the smaller tiles of the 160-row kernel spread better.  The tile count is an estimate: the
  // loads are on the device; an expert's last row block is taken as half full.  Measured in one
  // process against the 160-row kernel: 8 experts x 4096 rows 2048 -> 8192 -> 2048 1165 / 993 ->
  // 962 / 793 us, the ragged task-MoE shape 1585 / 1374 -> 1355 / 1211 us, the top-2 shape's
  // expanding GEMM (1232 tiles) 212 -> 166 us, 8 x 1824 rows 4096 -> 1024 (256 tiles) 146 -> 99 us;
  // the top-2 shape's contracting GEMM (308 tiles on 256 CUs) 162 -> 173 us.
  if (pingpong_gemm_applies(a) && static_cast<long>(P) > static_cast<long>(E) * 160) {
    const long tiles = (static_cast<long>(P + 255) / 256 + (E + 1) / 2) * ((N + 255) / 256);
    const long cus = device_cus();
    if (tiles >= 2 * cus || (4 * tiles >= 3 * cus && tiles <= cus))
      return launch_pingpong_gemm(a, act, as_stream(stream));
  }
  // Tile choice.  A wavefront owns 160 x 64 outputs (7 LDS fragment reads feed 10 MFMAs); a
  // workgroup is 2, 3 or 4 of them side by side.  The kernel is bound by how fast a CU can fill
  // its L1 (about 29 KB/us, L2 hits included), so the shape is the one that gives the busiest CU
  // the fewest operand bytes: wide tiles re-read the activation rows less often, narrow ones
  // keep all CUs busy when there are few tiles (only the 2-wavefront tile fits twice on a CU).
  constexpr int forced = 0;  // a fixed tile shape (21..24), for experiments
  int shape = forced;
  if (shape == 0) {
    const int cus = device_cus();
    const long row_blocks = estimated_row_blocks(P, E);
    double best = 0;
    for (int waves = 4; waves >= 2; --waves) {
      const long tiles = row_blocks * ((N + 64 * waves - 1) / (64 * waves));
      const long slots = static_cast<long>(cus) * (waves == 2 ? 2 : 1);
      const double rounds = static_cast<double>((tiles + slots - 1) / slots) * (waves == 2 ? 2 : 1);
      const double cost = rounds * (160 + 64 * waves);  // operand rows the busiest CU streams per K
      if (shape == 0 || cost < best) { best = cost; shape = 20 + waves; }
    }
  }
  if (shape == 24) return launch<5, 2, 4>(a, act, as_stream(stream));
  if (shape == 23) return launch<5, 2, 3>(a, act, as_stream(stream));
  if (shape == 22) return launch<5, 2, 2>(a, act, as_stream(stream));
  return launch<5, 1, 4>(a, act, as_stream(stream));
}

}  // namespace

extern "C" int brt_hip_grouped_gemm(const void* x, const void* const* weights,
                                    const void* const* biases, void* out, const int32_t* loads,
                                    int E, int P, int K, int N, int act, void* stream) {
  return grouped_gemm_impl(x, weights, biases, out, loads, nullptr, 0, E, P, 0, K, N, act, 0, 0, stream);
}

extern "C" int brt_hip_grouped_gemm_timed(const void* x, const void* const* weights, const void* const* biases,
                                          void* out, const int32_t* loads, int E, int P, int K, int N, int act,
                                          long long* clocks, void* stream) {
  if (clocks == nullptr) return fail(BRT_E_INVALID, "grouped_gemm_timed: clocks is null");
  return grouped_gemm_impl(x, weights, biases, out, loads, nullptr, 0, E, P, 0, K, N, act, 0, 0, stream, false,
                                nullptr, nullptr, clocks);
}

extern "C" int brt_hip_grouped_gemm_f32out(const void* x, const void* const* weights,
                                           const void* const* biases, float* out,
                                           const int32_t* loads, int E, int P, int K, int N, int act,
                                           void* stream) {
  return grouped_gemm_impl(x, weights, biases, out, loads, nullptr, 0, E, P, 0, K, N, act, 0, 0, stream, true);
}

extern "C" int brt_hip_grouped_gemm_routed(const void* x, const void* const* weights,
                                           const void* const* biases, void* out,
                                           const int32_t* loads, const int32_t* tags, int E, int P,
                                           int T, int K, int N, int act, int gather_in,
                                           int scatter_out, int32_t* row_tags_out, void* stream) {
  return grouped_gemm_impl(x, weights, biases, out, loads, tags, 0, E, P, T, K, N, act, gather_in,
                           scatter_out, stream, false, row_tags_out);
}

extern "C" int brt_hip_grouped_gemm_routed_f32out(const void* x, const void* const* weights,
                                                  const void* const* biases, float* out,
                                                  const int32_t* loads, const int32_t* tags, int E,
                                                  int P, int T, int K, int N, int act, int gather_in,
                                                  int scatter_out, int32_t* row_tags_out, void* stream) {
  return grouped_gemm_impl(x, weights, biases, out, loads, tags, 0, E, P, T, K, N, act, gather_in,
                           scatter_out, stream, true, row_tags_out);
}

namespace {
// 8 values per thread: two 16-byte loads, one 16-byte store
__global__ __launch_bounds__(256) void cast_f32_to_bf16_kernel(const float* __restrict__ src, __bf16* __restrict__ dst, size_t n) {
  const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
  if (i + 8 <= n) {
    const f32x4 lo = *reinterpret_cast<const f32x4*>(src + i), hi = *reinterpret_cast<const f32x4*>(src + i + 4);
    bf16x8 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = static_cast<__bf16>(lo[q]), o[4 + q] = static_cast<__bf16>(hi[q]);
    *reinterpret_cast<bf16x8*>(dst + i) = o;
  } else {
    for (size_t j = i; j < n; ++j) dst[j] = static_cast<__bf16>(src[j]);
  }
}
}  // namespace

extern "C" int brt_hip_cast_f32_to_bf16(const float* src, void* dst, size_t n, void* stream) {
  if (n == 0) return BRT_OK;
  if (!src || !dst) return fail(BRT_E_INVALID, "null argument");
  if (!aligned(src, 16) || !aligned(dst, 16)) return fail(BRT_E_INVALID, "src/dst must be 16-byte aligned");
  const size_t blocks = (n + 2047) / 2048;
  if (blocks > 0x7fffffffull) return fail(BRT_E_UNSUPPORTED, "%zu elements are too many for one launch", n);
  hipLaunchKernelGGL(cast_f32_to_bf16_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                     as_stream(stream), src, static_cast<__bf16*>(dst), n);
  return check_launch("cast_f32_to_bf16_kernel");
}

extern "C" int brt_hip_grouped_gemm_accumulate(const void* x, const void* const* weights,
                                               const void* const* biases, float* out,
                                               const int32_t* loads, const int32_t* tags,
                                               int entries_per_cell, const float* gates, int E, int P,
                                               int T, int K, int N, int act, int gather_in,
                                               void* stream) {
  if (entries_per_cell < 0) return fail(BRT_E_INVALID, "entries per cell must not be negative, got %d", entries_per_cell);
  if (!gates) return fail(BRT_E_INVALID, "the accumulate form needs the gates");
  return grouped_gemm_impl(x, weights, biases, out, loads, tags, entries_per_cell, E, P, T, K, N, act,
                           gather_in, 1, stream, false, nullptr, gates);
}

extern "C" int brt_hip_grouped_gemm_by_rows(const void* x, const void* const* weights,
                                            const void* const* biases, void* out,
                                            const int32_t* loads, const int32_t* row_entries, int k,
                                            int E, int P, int T, int K, int N, int act,
                                            int gather_in, int scatter_out, void* stream) {
  if (k <= 0) return fail(BRT_E_INVALID, "entries per cell must be positive, got %d", k);
  if (scatter_out && k != 1)
    return fail(BRT_E_UNSUPPORTED, "scatter_out needs one path per cell (k = %d)", k);
  return grouped_gemm_impl(x, weights, biases, out, loads, row_entries, k, E, P, T, K, N, act,
                           gather_in, scatter_out, stream);
}
