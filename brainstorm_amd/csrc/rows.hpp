// Row-copy helpers shared by the routing kernels: 2..16-byte copy units as native vector
// types, and conversion of a unit of fp32 / fp16 / bf16 elements to and from fp32.
#pragma once

#include "common.hpp"

namespace brt {

// Copy units are native vector types, so that arrays of them live in registers.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

template <int BYTES> struct Unit;
template <> struct Unit<16> { using type = u32x4; };
template <> struct Unit<8> { using type = u32x2; };
template <> struct Unit<4> { using type = uint32_t; };
template <> struct Unit<2> { using type = uint16_t; };

template <int BYTES>
__device__ __forceinline__ uint32_t unit_word(const typename Unit<BYTES>::type& v, int i) {
  if constexpr (BYTES >= 8) return v[i];
  else return v;
}

// A word of DT elements with every -0 turned into +0, all other bit patterns kept: what adding the
// element to a zero accumulator does to it (0 + -0 = +0), for kernels that move a row instead of
// summing it.  16-bit halves: flip the sign bits, find the halves that are now zero without a carry
// crossing between them, clear the sign of exactly those.
template <int DT>
__device__ __forceinline__ uint32_t plus_zero(uint32_t w) {
  if constexpr (DT == BRT_F32) {
    return w == 0x80000000u ? 0u : w;
  } else {
    const uint32_t t = w ^ 0x80008000u;
    const uint32_t nonzero = (((t & 0x7fff7fffu) + 0x7fff7fffu) | t) & 0x80008000u;
    return w & ~(nonzero ^ 0x80008000u);
  }
}

constexpr int elem_bytes(int dt) { return dt == BRT_F32 ? 4 : 2; }

// Unpacks BYTES of DT elements to fp32.
template <int DT, int BYTES>
__device__ __forceinline__ void unpack(const typename Unit<BYTES>::type& v,
                                       float (&x)[BYTES / elem_bytes(DT)]) {
  if constexpr (BYTES == 2) {
    x[0] = half_bits_to_float<DT>(v);
  } else {
#pragma unroll
    for (int i = 0; i < BYTES / 4; ++i) {
      const uint32_t w = unit_word<BYTES>(v, i);
      if constexpr (DT == BRT_F32) {
        x[i] = __uint_as_float(w);
      } else {
        x[2 * i] = half_bits_to_float<DT>(w & 0xffffu);
        x[2 * i + 1] = half_bits_to_float<DT>(w >> 16);
      }
    }
  }
}

// One store of a native unit; STREAM marks it non-temporal (written past the L2: for rows that
// the kernel does not read again, so that they do not evict data it still has to read).
template <bool STREAM, typename V>
__device__ __forceinline__ void store_unit(V* p, const V& v) {
  if constexpr (STREAM) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// Packs N fp32 values to DT (round to nearest even) and stores them at p.
template <int DT, int N, bool STREAM = false>
__device__ __forceinline__ void pack_store(void* p, const float (&x)[N]) {
  if constexpr (DT == BRT_F32) {
    if constexpr (N % 4 == 0) {
#pragma unroll
      for (int i = 0; i < N / 4; ++i) {
        f32x4 o = {x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]};
        store_unit<STREAM>(static_cast<f32x4*>(p) + i, o);
      }
    } else if constexpr (N == 2) {
      f32x2 o = {x[0], x[1]};
      store_unit<STREAM>(static_cast<f32x2*>(p), o);
    } else {
      store_unit<STREAM>(static_cast<float*>(p), x[0]);
    }
  } else {
    if constexpr (N == 1) {
      store_unit<STREAM>(static_cast<uint16_t*>(p), static_cast<uint16_t>(float_to_half_bits<DT>(x[0])));
    } else {
      uint32_t w[N / 2];
#pragma unroll
      for (int i = 0; i < N / 2; ++i)
        w[i] = float_to_half_bits<DT>(x[2 * i]) | (float_to_half_bits<DT>(x[2 * i + 1]) << 16);
      if constexpr (N == 8) {
        u32x4 o = {w[0], w[1], w[2], w[3]};
        store_unit<STREAM>(static_cast<u32x4*>(p), o);
      } else if constexpr (N == 4) {
        u32x2 o = {w[0], w[1]};
        store_unit<STREAM>(static_cast<u32x2*>(p), o);
      } else {
        store_unit<STREAM>(static_cast<uint32_t*>(p), w[0]);
      }
    }
  }
}

// Widening store of a whole wavefront's row segment (16-bit input units, fp32 output): lane l
// holds the 8 fp32 values of unit `first_unit + l`, i.e. 32 contiguous bytes of the output row, so
// two plain 16-byte stores per lane would each write every other 16 bytes of the segment (halves
// that have to meet in the L2).  The values are spread over the lanes first -- lane l takes half
// l & 1 of lane l / 2 (first store) and of lane 32 + l / 2 (second store) -- and each store then
// covers 1 KB of whole lines, streamed.  All 64 lanes must call it; `row_ok` (the row is written at
// all) must be the same for the whole wavefront, units at or past `units_in_row` are not written.
__device__ __forceinline__ void store_widened_spread(char* row_base, int first_unit, int units_in_row,
                                                     bool row_ok, const float (&x)[8]) {
  const int lane = lane_id();
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int from = 32 * half + (lane >> 1);
    f32x4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int lo = __builtin_amdgcn_ds_bpermute(from << 2, __float_as_int(x[q]));
      const int hi = __builtin_amdgcn_ds_bpermute(from << 2, __float_as_int(x[4 + q]));
      o[q] = __int_as_float((lane & 1) ? hi : lo);
    }
    const int unit = first_unit + from;
    if (row_ok && unit < units_in_row)
      store_unit<true>(reinterpret_cast<f32x4*>(row_base + static_cast<size_t>(unit) * 32 + (lane & 1) * 16), o);
  }
}

template <int BYTES>
__device__ __forceinline__ typename Unit<BYTES>::type zero_unit() {
  typename Unit<BYTES>::type z = {};
  return z;
}

}  // namespace brt
