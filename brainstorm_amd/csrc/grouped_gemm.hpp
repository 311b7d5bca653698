// Shared by the grouped GEMM kernels: argument block, activation epilogue.
#pragma once

#include "common.hpp"

namespace brt {

struct GemmArgs {
  const __bf16* x;
  const __bf16* const* w;
  const __bf16* const* bias;
  __bf16* out;
  float* out_f32;      // non-null: the output is fp32 (the accumulator after bias and activation), `out` is unused
  int* row_tags_out;   // non-null (routed forms): [P], the 1-based cell behind every row of the layout, 0 = empty slot
  const int* loads;
  const int* tags;  // [T,E] tag matrix (column e: 1-based cells of path e in seat order), or the
                    // row-entry vector [P] of the compact route (1-based entry t*k+j+1 per row), or null
  int tag_vector;   // tags is the row-entry vector
  int tag_div;      // entries per cell (k) of the row-entry vector
  int E, P, K, N, T;
  int plain_out;  // ordinary output stores instead of streaming ones (a small output that is read at once)
  int gather, scatter;  // rows of x / of out are addressed through the tags
  // accumulate form (scatter only): non-null gates turn the store of a row into
  // acc_out[cell] += gate * (the row rounded to bf16), fp32 atomic adds; gate of the row's cell on
  // this path from the [T,E] gate matrix, or by the row's entry from the [T*k] weights of the compact route
  const float* gates;
  float* acc_out;
  int tiles_n, tiles_m_max;
  int walk, groups_n;  // column tiles one workgroup walks, ceil(tiles_n / walk)
  int patch;           // workgroups in patch order (experts with several row blocks), see the kernel
  // measurement aid (ping-pong kernel only): non-null, the workgroup of the first tile writes the
  // shader clocks (s_memtime) and the ticks of the constant 100 MHz counter (s_memrealtime) its
  // first wavefront spent in the K loop, and the number of K-steps, into clocks[0..2]
  long long* clocks;
};

// The 256 x 256 ping-pong kernel (grouped_gemm_pingpong.hip): the shapes it takes, and its launch.
bool pingpong_gemm_applies(const GemmArgs& a);
int launch_pingpong_gemm(GemmArgs& a, int act, hipStream_t st);

// GELU(v) = v * Phi(v) = max(v, 0) - |v| * Phi(-|v|), branch free.  The tail probability is
// exp2(Q(|v|)) with Q a degree-7 fit of log2 Phi(-x) on [0, 8] (|Q - log2 Phi| < 5e-5 there, so the
// tail is good to 3.5e-5 relative; beyond 8 the product is below 5e-15 and Q keeps falling to -inf).
// Against the erf form in double the result is within 4.3e-6 absolute everywhere, two orders below
// half a bf16 step at the values where that bound is reached.  The clamp keeps +-inf inputs from
// turning inf * 0 into NaN.  Cost per element: seven multiply-adds, one exp2, min, max, one more fma.
__device__ __forceinline__ float gelu_erf(float v) {
  const float av = fminf(fabsf(v), 1e30f);
  float q = -1.262479145e-06f;
  q = __builtin_fmaf(q, av, 4.820351751e-05f);
  q = __builtin_fmaf(q, av, -8.072460769e-04f);
  q = __builtin_fmaf(q, av, 7.944535464e-03f);
  q = __builtin_fmaf(q, av, -5.263513327e-02f);
  q = __builtin_fmaf(q, av, -4.599574506e-01f);
  q = __builtin_fmaf(q, av, -1.150609374e+00f);
  q = __builtin_fmaf(q, av, -1.000043273e+00f);
  return __builtin_fmaf(-av, __builtin_amdgcn_exp2f(q), fmaxf(v, 0.0f));
}

template <int ACT>
__device__ __forceinline__ float apply_act(float v) {
  if (ACT == BRT_ACT_GELU) return gelu_erf(v);
  if (ACT == BRT_ACT_RELU) return fmaxf(v, 0.0f);
  return v;
}

}  // namespace brt
