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
// Tiling (CDNA4, wave64): a 256-thread workgroup owns a BM x BN output tile and
// walks K in steps of 64.  Both operands are K-contiguous in memory, which is the
// MFMA operand layout (each lane feeds 8 consecutive k of one row/column), so
// tiles go global -> registers -> LDS as 16-byte chunks without any transpose and
// come back out of LDS as ds_read_b128 fragments.  LDS rows are padded by 16 bytes
// so that 8 consecutive rows hit 8 distinct bank groups.  Two LDS stages: the next
// K-step is in flight in registers while the current one feeds
// v_mfma_f32_32x32x16_bf16 (fp32 accumulate); one barrier per K-step.  The
// epilogue (bias, GELU/ReLU, round to bf16) goes through LDS so that the stores
// are full 16-byte, row-contiguous accesses.
//
// Workgroups are renumbered so that consecutive logical tiles run on the same
// XCD (hardware deals workgroups round-robin over the 8 XCDs): the BN-wide column
// tiles of one row block then share that XCD's L2 copy of the activation rows.
#include <algorithm>
#include <cstdlib>

#include "common.hpp"

namespace brt {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kBK = 64;                    // k elements per stage
constexpr int kChunks = kBK / 8;           // 16-byte chunks per tile row
constexpr int kRowBytes = kBK * 2 + 16;    // padded LDS row
constexpr int kXcds = 8;

struct GemmArgs {
  const __bf16* x;
  const __bf16* const* w;
  const __bf16* const* bias;
  __bf16* out;
  const int* loads;
  int E, P, K, N;
  int tiles_n, tiles_m_max;
  int act;
};

__device__ __forceinline__ float apply_act(float v, int act) {
  if (act == BRT_ACT_GELU) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
  if (act == BRT_ACT_RELU) return fmaxf(v, 0.0f);
  return v;
}

template <int BM, int BN>
__global__ __launch_bounds__(kThreads) void grouped_gemm_kernel(GemmArgs a) {
  constexpr int WM = BM / 2, WN = BN / 2;  // 2 x 2 wavefronts
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes;
  constexpr int STAGE = A_BYTES + B_BYTES;
  constexpr int A_LOADS = BM * kChunks / kThreads, B_LOADS = BN * kChunks / kThreads;
  constexpr int OUT_ROW = BN * 2 + 16;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  __shared__ int s_tile[3];  // expert, first row, valid rows

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // ---- which tile: XCD-aware renumbering, then expert lookup from the loads ----------
  const int per_xcd = gridDim.x / kXcds;
  const int logical = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
  const int mt = logical / a.tiles_n, nt = logical - mt * a.tiles_n;
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
        }
      }
      carry_t += __shfl(incl_t, kWave - 1, kWave);
      carry_m += __shfl(incl_m, kWave - 1, kWave);
    }
    if (!found && lane == 0) s_tile[0] = -1;
  }
  __syncthreads();
  const int e = s_tile[0];
  if (e < 0) return;  // beyond the last tile
  const int row0 = s_tile[1], rows = s_tile[2];
  const int n0 = nt * BN;
  const int K = a.K;

  const __bf16* __restrict__ xa = a.x + static_cast<size_t>(row0) * K;
  const __bf16* __restrict__ wb = a.w[e] + static_cast<size_t>(n0) * K;

  // global -> register staging: thread t owns chunk (t % 8) of rows t/8 + 32 i
  const int lc = tid % kChunks, lr = tid / kChunks;
  u32x4 ra[A_LOADS], rb[B_LOADS];
  auto fetch = [&](int k0) {
    const bool k_ok = k0 + lc * 8 < K;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int r = lr + i * (kThreads / kChunks);
      u32x4 z = {};
      ra[i] = (k_ok && r < rows)
                  ? *reinterpret_cast<const u32x4*>(xa + static_cast<size_t>(r) * K + k0 + lc * 8)
                  : z;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int r = lr + i * (kThreads / kChunks);
      u32x4 z = {};
      rb[i] = (k_ok && n0 + r < a.N)
                  ? *reinterpret_cast<const u32x4*>(wb + static_cast<size_t>(r) * K + k0 + lc * 8)
                  : z;
    }
  };
  auto stash = [&](int stage) {
    char* sa = smem + stage * STAGE;
    char* sb = sa + A_BYTES;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int r = lr + i * (kThreads / kChunks);
      *reinterpret_cast<u32x4*>(sa + r * kRowBytes + lc * 16) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int r = lr + i * (kThreads / kChunks);
      *reinterpret_cast<u32x4*>(sb + r * kRowBytes + lc * 16) = rb[i];
    }
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = f32x16{};

  const int wm = wave >> 1, wn = wave & 1;
  const int frag_row = lane & 31, frag_k = lane >> 5;  // MFMA operand: row / k-half of this lane

  fetch(0);
  stash(0);
  __syncthreads();
  const int k_tiles = (K + kBK - 1) / kBK;
  for (int kt = 0; kt < k_tiles; ++kt) {
    if (kt + 1 < k_tiles) fetch((kt + 1) * kBK);
    const char* sa = smem + (kt & 1) * STAGE;
    const char* sb = sa + A_BYTES;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      bf16x8 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa[i] = *reinterpret_cast<const bf16x8*>(
            sa + (wm * WM + i * 32 + frag_row) * kRowBytes + (ks * 2 + frag_k) * 16);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        fb[j] = *reinterpret_cast<const bf16x8*>(
            sb + (wn * WN + j * 32 + frag_row) * kRowBytes + (ks * 2 + frag_k) * 16);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < k_tiles) stash((kt + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue: bias + activation, bf16, through LDS, 16-byte row stores ---------------
  // accumulator r of a 32x32 tile: row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
  const __bf16* bias = a.bias != nullptr ? a.bias[e] : nullptr;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = wn * WN + j * 32 + (lane & 31);
      const float b = (bias != nullptr && n0 + col < a.N) ? static_cast<float>(bias[n0 + col]) : 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wm * WM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
        const float v = apply_act(acc[i][j][r] + b, a.act);
        *reinterpret_cast<__bf16*>(smem + row * OUT_ROW + col * 2) = static_cast<__bf16>(v);
      }
    }
  __syncthreads();
  constexpr int OUT_CHUNKS = BN / 8;
  __bf16* __restrict__ oc = a.out + static_cast<size_t>(row0) * a.N + n0;
  for (int q = tid; q < BM * OUT_CHUNKS; q += kThreads) {
    const int r = q / OUT_CHUNKS, c = q - r * OUT_CHUNKS;
    if (r < rows && n0 + c * 8 < a.N)
      *reinterpret_cast<u32x4*>(oc + static_cast<size_t>(r) * a.N + c * 8) =
          *reinterpret_cast<const u32x4*>(smem + r * OUT_ROW + c * 16);
  }
}

template <int BM, int BN>
int launch(GemmArgs& a, hipStream_t st) {
  constexpr int STAGE = (BM + BN) * kRowBytes;
  constexpr int OUT_BYTES = BM * (BN * 2 + 16);
  const size_t lds = std::max(2 * STAGE, OUT_BYTES);
  a.tiles_n = (a.N + BN - 1) / BN;
  a.tiles_m_max = (a.P + BM - 1) / BM + a.E;  // sum over experts of ceil(M_e/BM) never exceeds this
  long grid = static_cast<long>(a.tiles_m_max) * a.tiles_n;
  grid = (grid + kXcds - 1) / kXcds * kXcds;
  static bool configured = false;
  if (!configured) {
    hipFuncSetAttribute(reinterpret_cast<const void*>(&grouped_gemm_kernel<BM, BN>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    configured = true;
  }
  hipLaunchKernelGGL((grouped_gemm_kernel<BM, BN>), dim3(static_cast<unsigned>(grid)),
                     dim3(kThreads), lds, st, a);
  return check_launch("grouped_gemm_kernel");
}

}  // namespace
}  // namespace brt

using namespace brt;

extern "C" int brt_hip_grouped_gemm(const void* x, const void* const* weights,
                                    const void* const* biases, void* out, const int32_t* loads,
                                    int E, int P, int K, int N, int act, void* stream) {
  if (E <= 0 || P < 0 || K <= 0 || N <= 0) return fail(BRT_E_INVALID, "bad shape E=%d P=%d K=%d N=%d", E, P, K, N);
  if (K % 8 != 0 || N % 8 != 0)
    return fail(BRT_E_UNSUPPORTED, "K and N must be multiples of 8 (16-byte rows), got K=%d N=%d", K, N);
  if (act != BRT_ACT_NONE && act != BRT_ACT_GELU && act != BRT_ACT_RELU)
    return fail(BRT_E_INVALID, "unknown activation %d", act);
  if (P == 0) return BRT_OK;
  if (!x || !weights || !out || !loads) return fail(BRT_E_INVALID, "null argument");
  if (!aligned(x, 16) || !aligned(out, 16)) return fail(BRT_E_INVALID, "x/out must be 16-byte aligned");
  GemmArgs a{};
  a.x = static_cast<const __bf16*>(x);
  a.w = reinterpret_cast<const __bf16* const*>(weights);
  a.bias = reinterpret_cast<const __bf16* const*>(biases);
  a.out = static_cast<__bf16*>(out);
  a.loads = loads;
  a.E = E; a.P = P; a.K = K; a.N = N; a.act = act;
  return launch<128, 128>(a, as_stream(stream));
}
