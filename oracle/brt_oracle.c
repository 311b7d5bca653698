/*
 * CPU oracle for the MoE routing hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * Sequential, plain-C restatement of what the reference's CUDA kernels compute,
 * written from their source text (paths are relative to the reference tree):
 *
 *   src/router/location.cu   generate_indices_and_loads, throttle_hotmask,
 *                            convert_{seat_to_tag,tag_to_seat}_indices
 *   src/router/route.cu      dispatch_with_{seat,tag}_indices_{1d,2d},
 *                            combine_with_seat_indices, init_with_seat_indices
 *   src/backend/torch/router.cc   shape/dtype conventions around them
 *   python/brt/router/protocol/topk.py:26-31   top-k hot mask (torch.topk + scatter_)
 *   src/backend/torch/router.cc:348-369,449-472   tag-index gather (_unique + scatter_reduce)
 *   the same route held as k path ids per cell (compact format; restated from the dense ops)
 *
 * Only tests, the smoke check and the bench's cpu_baseline leg may link or call
 * this file; the product path never does.
 *
 * Parity status: every function here is pinned by checks that do not retype
 * its formula (reference notebook vectors, the reference test-suite's own
 * closed forms, permutation/round-trip invariants, brute force on tiny
 * inputs); see tests/test_oracle_*.py.  No function is "parity unpinned".
 *
 * Index conventions (location.cu:132-195): all index tensors are int32
 * row-major [T,E]; values are 1-based and 0 means "not routed / empty slot".
 *
 * Build: gcc -O2 -ffp-contract=off -shared -fPIC (no FMA contraction, so the
 * fp32 combine keeps one rounding per multiply and one per add, like the
 * reference's `in * gate` followed by atomicAdd, route.cu:236-243).
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>
#include <math.h>

enum { ORACLE_F32 = 0, ORACLE_F16 = 1, ORACLE_BF16 = 2 };

/* ---------- 16-bit float helpers (round-to-nearest-even) ---------- */

static float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

static float bf16_to_float(uint16_t h) { return bits_to_float((uint32_t)h << 16); }

static uint16_t float_to_bf16(float f) {
  uint32_t u = float_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

static float f16_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_to_float(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * (1.0f / 16777216.0f);
    return sign ? -v : v;
  }
  if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
  return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

static uint16_t float_to_f16(float f) {
  uint32_t u = float_to_bits(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  /* NaN */
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 (or inf) -> inf */
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds up to inf */
  if (a < 0x33000001u) return sign;                        /* <= 2^-25 rounds to zero */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;                                /* bits dropped from m */
  uint32_t hexp;
  if (e < -14) { /* subnormal half */
    shift = 13 + (-14 - e);
    hexp = 0;
  } else {
    shift = 13;
    hexp = (uint32_t)(e + 15);
  }
  uint32_t kept = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) kept++;
  uint32_t out;
  if (hexp == 0) {
    out = kept; /* may carry into exponent 1: correct encoding */
  } else {
    out = ((hexp - 1u) << 10) + kept; /* kept includes the hidden bit (1<<10) */
  }
  return (uint16_t)(sign | out);
}

static size_t elem_size(int dtype) { return dtype == ORACLE_F32 ? 4 : 2; }

static float load_elem(const void* p, int dtype, size_t i) {
  if (dtype == ORACLE_F32) return ((const float*)p)[i];
  if (dtype == ORACLE_F16) return f16_to_float(((const uint16_t*)p)[i]);
  return bf16_to_float(((const uint16_t*)p)[i]);
}

static void store_elem(void* p, int dtype, size_t i, float v) {
  if (dtype == ORACLE_F32)
    ((float*)p)[i] = v;
  else if (dtype == ORACLE_F16)
    ((uint16_t*)p)[i] = float_to_f16(v);
  else
    ((uint16_t*)p)[i] = float_to_bf16(v);
}

/* exported so tests can pin the converters against numpy/torch */
float oracle_f16_to_float(uint16_t h) { return f16_to_float(h); }
uint16_t oracle_float_to_f16(float f) { return float_to_f16(f); }
float oracle_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
uint16_t oracle_float_to_bf16(float f) { return float_to_bf16(f); }

/* ---------- location.cu ---------- */

/*
 * generate_indices_and_loads  (location.cu:132-257, launcher :335-379)
 *
 * Per column e: a running inclusive sum of the mask values ("location"),
 * index = location * mask (location.cu:177-178).  Seat mode writes it at
 * [t,e]; tag mode writes t+1 at [index-1,e] (:180-185).  `indices` must be
 * zero-filled by the caller (router.cc:74).  Load rules: location.cu:222-256;
 * path_wise_padding is honoured only together with capacity_padding (:349-358).
 */
void oracle_generate_indices_and_loads(const int32_t* mask, int32_t* indices, int32_t* loads,
                                       int T, int E, const int32_t* caps, int C,
                                       int capacity_padding, int path_wise_padding,
                                       int is_tag_index) {
  if (caps == NULL) C = 0;
  if (!capacity_padding) path_wise_padding = 0;
  for (int e = 0; e < E; ++e) {
    int prefix = 0;
    for (int t = 0; t < T; ++t) {
      int m = mask[(size_t)t * E + e];
      prefix += m;
      int index = prefix * m;
      if (index != 0) {
        if (is_tag_index) {
          if (index >= 1 && index <= T) indices[(size_t)(index - 1) * E + e] = t + 1;
        } else {
          indices[(size_t)t * E + e] = index;
        }
      }
    }
    int real_load = prefix;
    if (path_wise_padding) {
      loads[e] = caps[e];
      continue;
    }
    if (real_load == 0) {
      loads[e] = 0;
      continue;
    }
    if (capacity_padding) {
      int v = caps[C - 1];
      for (int i = 0; i < C; ++i)
        if (real_load <= caps[i]) {
          v = caps[i];
          break;
        }
      loads[e] = v;
    } else {
      if (C == 0) {
        loads[e] = real_load;
        continue;
      }
      int v = caps[C - 1];
      for (int i = 0; i < C; ++i)
        if (real_load <= caps[i]) {
          v = real_load;
          break;
        }
      loads[e] = v;
    }
  }
}

/*
 * throttle_hotmask  (location.cu:59-130)
 *
 * The reference walks each column in chunks of 1024 rows; inside a chunk a row
 * is kept iff mask==1 and prefix+rank <= threshold; after a chunk, the running
 * prefix absorbs the chunk's sum and the walk stops once it reaches the
 * threshold (then prefix := threshold).  `out` must be zero-filled by the
 * caller (router.cc:26); prefix is updated in place.
 */
void oracle_throttle_hotmask(const int32_t* mask, int32_t* out, int32_t* prefix,
                             const int32_t* threshold, int T, int E) {
  const int chunk = 1024;
  for (int e = 0; e < E; ++e) {
    int run = prefix[e];
    int thr = threshold[e];
    for (int s = 0; s < T; s += chunk) {
      int loc = run;
      int end = s + chunk < T ? s + chunk : T;
      for (int t = s; t < end; ++t) {
        int m = mask[(size_t)t * E + e];
        loc += m;
        if (m == 1 && loc <= thr) out[(size_t)t * E + e] = 1;
      }
      run = loc;
      if (run >= thr) {
        run = thr;
        break;
      }
    }
    prefix[e] = run;
  }
}

/*
 * convert_seat_to_tag_indices (location.cu:259-278): tag[seat-1,e] = t+1.
 * convert_tag_to_seat_indices (location.cu:280-302): slot s (< loads[e]) is
 * handled by thread s%1024, which walks s, s+1024, ... and stops at its first
 * zero tag; so slot s is converted iff tags at s, s-1024, s-2048, ... are all
 * non-zero.  `dst` must be zero-filled by the caller (router.cc:102).
 */
void oracle_convert_index_format(const int32_t* src, int32_t* dst, const int32_t* loads, int T,
                                 int E, int tag_to_seat) {
  if (!tag_to_seat) {
    for (int e = 0; e < E; ++e)
      for (int t = 0; t < T; ++t) {
        int seat = src[(size_t)t * E + e];
        if (seat != 0 && seat >= 1 && seat <= T) dst[(size_t)(seat - 1) * E + e] = t + 1;
      }
    return;
  }
  for (int e = 0; e < E; ++e) {
    int load = loads[e];
    if (load > T) load = T;
    for (int lane = 0; lane < 1024; ++lane)
      for (int s = lane; s < load; s += 1024) {
        int tag = src[(size_t)s * E + e];
        if (tag == 0) break;
        if (tag >= 1 && tag <= T) dst[(size_t)(tag - 1) * E + e] = s + 1;
      }
  }
}

/* ---------- route.cu ---------- */

static void copy_row(const void* src, size_t src_row, void* dst, size_t dst_row, int cell,
                     int dtype, int weighted, float gate) {
  size_t es = elem_size(dtype);
  if (!weighted) {
    memcpy((char*)dst + dst_row * cell * es, (const char*)src + src_row * cell * es, cell * es);
    return;
  }
  for (int j = 0; j < cell; ++j) {
    float v = load_elem(src, dtype, src_row * cell + j) * gate;
    store_elem(dst, dtype, dst_row * cell + j, v);
  }
}

/*
 * dispatch_with_indices_and_loads  (route.cu:13-206; shapes router.cc:131-273)
 *
 *   src   1-d: [T, cell];  2-d: [T, E, cell] (expert e reads slice [:, e, :];
 *         the binding transposes to [E,T,cell] first, router.cc:212)
 *   dst   [P, cell], zero-filled by the caller (router.cc:219)
 *   gates [T, E] in the data dtype or NULL (1-d only, route.cu:362)
 *   start[e] = e*max_path_load when max_path_load != 0, else sum(loads[:e])
 *   seat mode: every (t,e) with 1 <= idx <= loads[e] copies row t to
 *         start[e]+idx-1 (route.cu:37-50)
 *   tag mode: slot i < loads[e] is handled by block i%512, which walks
 *         i, i+512, ... and stops at its first zero tag (route.cu:84-92);
 *         dst row start[e]+i receives row tag-1
 *   new_tags (zero-filled by the caller) receive old_tags[source row]
 *         (route.cu:51-53); old_tags NULL means "no tag generation".
 *   Rows >= P are never written (guard added here; the reference would write
 *   out of bounds).  With a fixed stride (max_path_load != 0) seats beyond the
 *   stride are dropped: the reference would write them into the next path's
 *   block, racing with that path's own rows (route.cu:37-50 has no such guard),
 *   so there is no defined result to reproduce.
 */
void oracle_dispatch(const void* src, void* dst, const void* gates, const int32_t* idx,
                     const int32_t* loads, const int32_t* old_tags, int32_t* new_tags, int T,
                     int cell, int E, int P, int max_path_load, int is_1d, int is_tag_index,
                     int dtype) {
  int weighted = gates != NULL;
  long start = 0;
  for (int e = 0; e < E; ++e) {
    long load_start = max_path_load != 0 ? (long)e * max_path_load : start;
    int path_load = loads[e];
    if (max_path_load != 0 && path_load > max_path_load) path_load = max_path_load;
    if (!is_tag_index) {
      for (int t = 0; t < T; ++t) {
        int seat = idx[(size_t)t * E + e];
        if (seat == 0 || seat > path_load || seat < 0) continue;
        long row = load_start + seat - 1;
        if (row >= P) continue;
        size_t src_row = is_1d ? (size_t)t : (size_t)t * E + e;
        float g = weighted ? load_elem(gates, dtype, (size_t)t * E + e) : 1.0f;
        copy_row(src, src_row, dst, (size_t)row, cell, dtype, weighted, g);
        if (old_tags) new_tags[row] = old_tags[t];
      }
    } else {
      for (int blk = 0; blk < 512; ++blk)
        for (int i = blk; i < T; i += 512) {
          if (i >= path_load) continue;
          int tag = idx[(size_t)i * E + e];
          if (tag == 0) break;
          if (tag < 1 || tag > T) continue;
          long row = load_start + i;
          if (row >= P) continue;
          int t = tag - 1;
          size_t src_row = is_1d ? (size_t)t : (size_t)t * E + e;
          float g = weighted ? load_elem(gates, dtype, (size_t)t * E + e) : 1.0f;
          copy_row(src, src_row, dst, (size_t)row, cell, dtype, weighted, g);
          if (old_tags) new_tags[row] = old_tags[t];
        }
    }
    start += path_load;
  }
}

/*
 * combine_with_indices_and_loads, seat mode  (route.cu:208-282, 467-518)
 *
 *   src [P, cell] in in_dtype; dst [T, cell] in out_dtype; gates [T,E] in
 *   gate_dtype or NULL.
 *   For token t the accumulator starts at 0 (non-residual: dst is torch::zeros,
 *   router.cc:460; residual: init_with_seat_indices zeroes the rows of routed
 *   tokens, route.cu:250-282) and adds, for e ascending with
 *   1 <= idx <= loads[e], src[start[e]+idx-1] * gate: one fp32 multiply, then
 *   one fp32 add (the atomicAdd of route.cu:243 is issued by one thread per
 *   element in program order, so the order is ascending e).  Residual rows of
 *   tokens with no valid route are left untouched.
 *   The reference binding only instantiates fp32 (router.cc:435,443); for
 *   16-bit inputs this oracle defines: widen to fp32, accumulate in fp32 in the
 *   same order, round once on store.
 */
void oracle_combine(const void* src, void* dst, const void* gates, const int32_t* idx,
                    const int32_t* loads, int T, int cell, int E, int P, int max_path_load,
                    int is_residual, int in_dtype, int out_dtype, int gate_dtype) {
  for (int t = 0; t < T; ++t) {
    int routed = 0;
    for (int j = 0; j < cell; ++j) {
      float acc = 0.0f;
      long start = 0;
      int any = 0;
      for (int e = 0; e < E; ++e) {
        int seat = idx[(size_t)t * E + e];
        int load = loads[e];
        long load_start = max_path_load != 0 ? (long)e * max_path_load : start;
        start += load;
        /* fixed stride: a path's block ends at the stride (see oracle_dispatch) */
        if (max_path_load != 0 && load > max_path_load) load = max_path_load;
        if (seat == 0 || seat > load || seat < 0) continue;
        long row = load_start + seat - 1;
        if (row >= P) continue;
        any = 1;
        float v = load_elem(src, in_dtype, (size_t)row * cell + j);
        if (gates) {
          float g = load_elem(gates, gate_dtype, (size_t)t * E + e);
          v = v * g;
        }
        acc = acc + v;
      }
      routed = any;
      if (any || !is_residual) store_elem(dst, out_dtype, (size_t)t * cell + j, acc);
    }
    (void)routed;
  }
}


/* ---------- gate front-end: top-k hot mask ----------
 * python/brt/router/protocol/topk.py:26-31:
 *   hot_mask = zeros_like(score, int32).scatter_(1, topk(score, k, dim=1).indices, 1)
 * torch.topk orders NaN above every number; which of several equal scores it returns is
 * not specified, here the lowest column wins.  Scores arrive as fp32 (16-bit inputs are
 * widened exactly by the caller).  Selection by k passes of "largest remaining". */
static int score_greater(float a, float b) { /* a strictly above b in topk's order */
  const int a_nan = a != a, b_nan = b != b;
  if (a_nan || b_nan) return a_nan && !b_nan;
  return a > b;
}

void oracle_topk_hot_mask(const float* score, int32_t* mask, int T, int E, int k) {
  for (int t = 0; t < T; ++t) {
    const float* row = score + (size_t)t * E;
    int32_t* out = mask + (size_t)t * E;
    for (int e = 0; e < E; ++e) out[e] = 0;
    for (int pass = 0; pass < k && pass < E; ++pass) {
      int best = -1;
      for (int e = 0; e < E; ++e) {
        if (out[e]) continue;
        if (best < 0 || score_greater(row[e], row[best])) best = e;
      }
      out[best] = 1;
    }
  }
}

/* ---------- compact route format ----------
 * The same route as the dense mask / seat matrix, held as k path ids per cell.  No function of
 * the reference has this signature; each restates what the reference computes on the dense
 * form and is pinned by converting to and from that form (tests/test_oracle.py):
 *   gate_topk       topk.py:26-31 (selection), switch_transformer.py:240-253 (softmax in fp32)
 *   route_by_path   location.cu:132-257 (seats in ascending cell order, load rules :222-256)
 *   dispatch_by_rows / combine_by_rows   route.cu:13-282 on rows named directly */
void oracle_gate_topk(const float* score, int T, int E, int k, int softmax, int32_t* ids,
                      float* weights) {
  char* taken = (char*)malloc((size_t)(E > 0 ? E : 1));
  for (int t = 0; t < T; ++t) {
    const float* row = score + (size_t)t * E;
    double top = -HUGE_VAL, sum = 0.0;
    if (softmax) {
      for (int e = 0; e < E; ++e) if (row[e] > top) top = row[e];
      for (int e = 0; e < E; ++e) sum += exp((double)row[e] - top);
    }
    memset(taken, 0, (size_t)E);
    for (int pass = 0; pass < k && pass < E; ++pass) {
      int best = -1;
      for (int e = 0; e < E; ++e) {
        if (taken[e]) continue;
        if (best < 0 || score_greater(row[e], row[best])) best = e;
      }
      taken[best] = 1;
      ids[(size_t)t * k + pass] = best;
      if (weights)
        weights[(size_t)t * k + pass] =
            softmax ? (float)(exp((double)row[best] - top) / sum) : row[best];
    }
  }
  free(taken);
}

void oracle_route_by_path(const int32_t* ids, int T, int k, int E, const int32_t* caps, int C,
                          int capacity_padding, int path_wise_padding, int max_path_load,
                          int32_t* loads, int32_t* counts, int32_t* seat_rows,
                          int32_t* row_entries, int P) {
  /* the dense mask of the same route, then the dense scan (pinned above) on it */
  int32_t* mask = (int32_t*)calloc((size_t)T * E + 1, sizeof(int32_t));
  int32_t* seats = (int32_t*)calloc((size_t)T * E + 1, sizeof(int32_t));
  for (int t = 0; t < T; ++t)
    for (int j = 0; j < k; ++j) {
      int e = ids[(size_t)t * k + j];
      if (e >= 0 && e < E) mask[(size_t)t * E + e] = 1;
    }
  oracle_generate_indices_and_loads(mask, seats, loads, T, E, caps, C, capacity_padding,
                                    path_wise_padding, 0);
  for (int e = 0; e < E; ++e) {
    int c = 0;
    for (int t = 0; t < T; ++t) c += mask[(size_t)t * E + e];
    if (counts) counts[e] = c;
  }
  for (int r = 0; r < P; ++r) row_entries[r] = 0;
  for (int t = 0; t < T; ++t)
    for (int j = 0; j < k; ++j) {
      int e = ids[(size_t)t * k + j];
      int32_t row = 0;
      if (e >= 0 && e < E) {
        long start = 0;
        for (int q = 0; q < e; ++q) start += loads[q];
        if (max_path_load != 0) start = (long)e * max_path_load;
        int seat = seats[(size_t)t * E + e];
        int limit = loads[e];
        if (max_path_load != 0 && limit > max_path_load) limit = max_path_load;
        if (seat >= 1 && seat <= limit && start + seat <= P) row = (int32_t)(start + seat);
      }
      seat_rows[(size_t)t * k + j] = row;
      if (row != 0) row_entries[row - 1] = t * k + j + 1;
    }
  free(mask);
  free(seats);
}

void oracle_dispatch_by_rows(const void* src, void* dst, const float* weights,
                             const int32_t* row_entries, int P, int T, int k, int cell, int dtype) {
  for (int r = 0; r < P; ++r) {
    int entry = row_entries[r];
    for (int j = 0; j < cell; ++j) {
      float v = 0.0f;
      if (entry >= 1 && entry <= T * k) {
        v = load_elem(src, dtype, (size_t)((entry - 1) / k) * cell + j);
        if (weights) v = v * weights[entry - 1];
      }
      store_elem(dst, dtype, (size_t)r * cell + j, v);
    }
  }
}

void oracle_combine_by_rows(const void* src, void* dst, const float* weights, const int32_t* ids,
                            const int32_t* seat_rows, int T, int k, int cell, int P,
                            int is_residual, int in_dtype, int out_dtype) {
  for (int t = 0; t < T; ++t)
    for (int j = 0; j < cell; ++j) {
      float acc = 0.0f;
      int any = 0, last = -1;
      for (;;) { /* entries with a row, by ascending path id */
        int pick = -1;
        for (int q = 0; q < k; ++q) {
          int row = seat_rows[(size_t)t * k + q], e = ids[(size_t)t * k + q];
          if (row < 1 || row > P || e <= last) continue;
          if (pick < 0 || e < ids[(size_t)t * k + pick]) pick = q;
        }
        if (pick < 0) break;
        last = ids[(size_t)t * k + pick];
        float v = load_elem(src, in_dtype, (size_t)(seat_rows[(size_t)t * k + pick] - 1) * cell + j);
        if (weights) v = v * weights[(size_t)t * k + pick];
        acc = acc + v;
        any = 1;
      }
      if (any || !is_residual) store_elem(dst, out_dtype, (size_t)t * cell + j, acc);
    }
}

/* ---------- tag-index gather (router.cc:348-369, 449-472) ----------
 * fuse_split_cells_from_paths hands the concatenated tags to `_unique(sorted, return_inverse)`:
 * the distinct values in ascending order and, for every input element, the position of its
 * value in that list.  Restated the way the library does it: sort a copy, drop repeats, then
 * look every element up by bisection. */
static int cmp_i64(const void* a, const void* b) {
  int64_t x = *(const int64_t*)a, y = *(const int64_t*)b;
  return (x > y) - (x < y);
}

int64_t oracle_unique_tags(const int64_t* tags, int64_t n, int64_t* unique, int64_t* inverse) {
  if (n <= 0) return 0;
  memcpy(unique, tags, (size_t)n * sizeof(int64_t));
  qsort(unique, (size_t)n, sizeof(int64_t), cmp_i64);
  int64_t m = 0;
  for (int64_t i = 0; i < n; ++i)
    if (i == 0 || unique[i] != unique[m - 1]) unique[m++] = unique[i];
  for (int64_t i = 0; i < n; ++i) {
    int64_t lo = 0, hi = m - 1;
    while (lo < hi) {
      int64_t mid = (lo + hi) / 2;
      if (unique[mid] < tags[i]) lo = mid + 1; else hi = mid;
    }
    inverse[i] = lo;
  }
  return m;
}

/* The tag-mode combine is zeros(n_out, cell).scatter_reduce(0, index per element, in, "sum")
 * (router.cc:451,459-460): out[index[p]] += in[p].  The reference's atomics add in arrival
 * order; the order is fixed here to ascending p, with an fp32 accumulator that starts at zero
 * and one rounding to the output type at the end. */
void oracle_combine_by_index(const void* src, void* dst, const int64_t* index, int P, int cell,
                             int n_out, int in_dtype, int out_dtype) {
  float* acc = (float*)calloc((size_t)(cell > 0 ? cell : 1), sizeof(float));
  for (int r = 0; r < n_out; ++r) {
    for (int c = 0; c < cell; ++c) acc[c] = 0.0f;
    for (int p = 0; p < P; ++p) {
      if (index[p] != r) continue;
      for (int c = 0; c < cell; ++c) acc[c] += load_elem(src, in_dtype, (size_t)p * cell + c);
    }
    for (int c = 0; c < cell; ++c) store_elem(dst, out_dtype, (size_t)r * cell + c, acc[c]);
  }
  free(acc);
}
