// Shared host/device helpers for libbrt_hip.so (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "brt_hip.h"

namespace brt {

// ---- host side: per-thread error text -------------------------------------
int fail(int code, const char* fmt, ...);  // records the message, returns code
int check_launch(const char* what);        // hipGetLastError -> BRT_E_LAUNCH
// More than 64 KB of dynamic LDS has to be allowed once per kernel and device.  Thread-safe; the
// first call for a kernel on a device changes a function attribute, so it must not happen while a
// stream is being captured into a graph (make the first call of each op outside the capture).
int allow_dynamic_lds(const void* kernel, int bytes);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// ---- device side ------------------------------------------------------------
constexpr int kWave = 64;

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Inclusive prefix sum across the 64 lanes of a wavefront, on the DPP network
// (no LDS, no cross-lane memory traffic): Kogge-Stone inside each row of 16 lanes
// with row_shr, then the row totals are carried over with row_bcast15/31.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 -> rows 1,3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 -> rows 2,3
  return v;
}

// All-reduce of a commutative `op` over aligned segments of `width` lanes (a power of two; the
// same for the whole wavefront): the xor butterfly, with its first four steps on the DPP network
// instead of the LDS crossbar.  Step d pairs lane i with lane i ^ d; quad_perm does that for
// d = 1, 2, and because the values are uniform over aligned groups of d lanes once step d is
// reached, row_half_mirror (i -> 7 - i) and row_mirror (i -> 15 - i) do it for d = 4, 8.
template <typename Op>
__device__ __forceinline__ int segment_all_reduce(int v, int width, Op op) {
  if (width > 1) v = op(v, __builtin_amdgcn_mov_dpp(v, 0xB1, 0xf, 0xf, true));   // quad_perm:[1,0,3,2]
  if (width > 2) v = op(v, __builtin_amdgcn_mov_dpp(v, 0x4E, 0xf, 0xf, true));   // quad_perm:[2,3,0,1]
  if (width > 4) v = op(v, __builtin_amdgcn_mov_dpp(v, 0x141, 0xf, 0xf, true));  // row_half_mirror
  if (width > 8) v = op(v, __builtin_amdgcn_mov_dpp(v, 0x140, 0xf, 0xf, true));  // row_mirror
  if (width > 16) v = op(v, __shfl_xor(v, 16, kWave));
  if (width > 32) v = op(v, __shfl_xor(v, 32, kWave));
  return v;
}
template <typename Op>
__device__ __forceinline__ float segment_all_reduce(float v, int width, Op op) {
  return __int_as_float(segment_all_reduce(__float_as_int(v), width, [&](int x, int y) {
    return __float_as_int(op(__int_as_float(x), __int_as_float(y)));
  }));
}

// Value of `v` held by lane `src_lane`; src_lane must be wave-uniform.
__device__ __forceinline__ int read_lane(int v, int src_lane) {
  return __builtin_amdgcn_readlane(v, src_lane);
}
__device__ __forceinline__ float read_lane(float v, int src_lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}

// bf16 <-> fp32 (round to nearest even; NaN stays NaN).
__device__ __forceinline__ float bf16_to_float(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t float_to_bf16(float f) {
  // gfx950 converts in hardware (v_cvt_pk_bf16_f32, round to nearest even)
  union { __bf16 h; uint16_t u; } c;
  c.h = static_cast<__bf16>(f);
  return c.u;
}
__device__ __forceinline__ float f16_to_float(uint32_t h) {
  union { uint16_t u; _Float16 f; } c;
  c.u = static_cast<uint16_t>(h);
  return static_cast<float>(c.f);
}
__device__ __forceinline__ uint32_t float_to_f16(float f) {
  union { uint16_t u; _Float16 f; } c;
  c.f = static_cast<_Float16>(f);
  return c.u;
}

template <int DT>
__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
  return DT == BRT_F16 ? f16_to_float(h) : bf16_to_float(h);
}
template <int DT>
__device__ __forceinline__ uint32_t float_to_half_bits(float f) {
  return DT == BRT_F16 ? float_to_f16(f) : float_to_bf16(f);
}

// Scalar load of one gate value of a runtime dtype.
__device__ __forceinline__ float load_gate(const void* gates, int dtype, size_t i) {
  if (dtype == BRT_F32) return static_cast<const float*>(gates)[i];
  uint32_t h = static_cast<const uint16_t*>(gates)[i];
  return dtype == BRT_F16 ? f16_to_float(h) : bf16_to_float(h);
}

// Load of a path from its real row count (src/router/location.cu:227-254): the path's own
// capacity when padding path-wise (even for an empty path); 0 for an empty path; the count itself
// without a capacity menu; else the smallest capacity that holds the count (the count itself when
// not padding), and the last capacity when none does.
__device__ __forceinline__ int finalize_load(int real, const int* caps, int C, int cap_pad,
                                             int path_pad, int col) {
  if (path_pad) return caps[col];  // unconditional, even for an empty path
  if (real == 0) return 0;
  if (C == 0) return real;
  for (int i = 0; i < C; ++i)
    if (real <= caps[i]) return cap_pad ? caps[i] : real;
  return caps[C - 1];
}

// Fills s_val[e] = g[e] and s_start[e] = exclusive prefix of g (or e*stride when
// stride != 0) for e < E, using the first wavefront of the block.  The caller
// must __syncthreads() afterwards.
__device__ __forceinline__ void load_and_scan_paths(const int* __restrict__ g, int* s_val,
                                                    int* s_start, int E, int stride) {
  if (threadIdx.x < kWave) {
    const int lane = threadIdx.x;
    int carry = 0;
    for (int base = 0; base < E; base += kWave) {
      const int e = base + lane;
      const int v = e < E ? g[e] : 0;
      const int incl = wave_inclusive_scan(v);
      if (e < E) {
        s_val[e] = v;
        s_start[e] = stride != 0 ? e * stride : carry + incl - v;
      }
      carry += __shfl(incl, kWave - 1, kWave);
    }
  }
}

}  // namespace brt
