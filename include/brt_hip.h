/*
 * libbrt_hip.so -- C ABI of the MI355X (gfx950) MoE routing hot path.
 *
 * Each entry point replaces one raw-pointer launcher of the reference's native
 * layer (paths relative to the reference tree); the reference-side binding
 * that would call it is the torch extension src/backend/torch/router.cc.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; `stream` is a
 *     hipStream_t passed as void* (NULL = the null stream);
 *   - index tensors are int32 row-major [T,E], values 1-based, 0 = not routed;
 *   - entry points return 0 on success and a negative BRT_E_* code otherwise
 *     (brt_hip_last_error() gives the message of the calling thread's last
 *     failure); they never throw, never allocate device memory, never
 *     synchronise the stream, and only enqueue work on `stream`;
 *   - the caller owns every buffer, including workspaces;
 *   - sizes: element counts of index-shaped arguments (T*E, T*k) must stay
 *     below 2^31 (BRT_E_UNSUPPORTED otherwise); row buffers may be of any
 *     size, their offsets are 64-bit.
 */
#ifndef BRT_HIP_H_
#define BRT_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  BRT_OK = 0,
  BRT_E_INVALID = -1,     /* bad argument (shape, flag combination, null pointer) */
  BRT_E_WORKSPACE = -2,   /* workspace missing or too small */
  BRT_E_LAUNCH = -3,      /* HIP reported a launch error */
  BRT_E_UNSUPPORTED = -4  /* dtype / layout not implemented */
};

enum { BRT_F32 = 0, BRT_F16 = 1, BRT_BF16 = 2 };

/* activation fused into the grouped GEMM epilogue */
enum { BRT_ACT_NONE = 0, BRT_ACT_GELU = 1, BRT_ACT_RELU = 2 };

/* Message of this thread's most recent failing call ("" if none). */
const char* brt_hip_last_error(void);

/* Library version, "major.minor". */
const char* brt_hip_version(void);

/*
 * Bytes of scratch memory brt_hip_generate_indices_and_loads /
 * brt_hip_throttle_hotmask need for a [T,E] mask (per-band column sums handed
 * from their first to their second kernel).  The content needs no
 * initialisation and carries nothing from one call to the next; one workspace
 * must not be used by two calls that can run concurrently (two streams).
 */
size_t brt_hip_scan_workspace_bytes(int T, int E);

/*
 * Replaces router::GenerateIndicesAndLoads (include/brt/router/location.h:28-38,
 * src/router/location.cu:212-257,335-379).
 *
 *   mask     [T,E] int32 hot mask
 *   indices  [T,E] int32 out; every element is written, no pre-zeroing needed.
 *            Seat mode (is_tag_index=0): cumsum(mask,0)*mask.  Tag mode: slot
 *            [s-1,e] receives row+1 of the s-th routed row of column e, the
 *            slots past a column's last tag receive 0.
 *   loads    [E] int32 out, after the capacity rules of location.cu:222-256
 *   counts   [E] int32 out or NULL: the un-clipped, un-padded per-path counts
 *            (sum(mask,0)); brt_hip_dispatch uses them to zero-fill padding rows
 *   caps     [C] int32 ascending supported capacities or NULL (C=0)
 *   capacity_padding requires C>=1; path_wise_padding is honoured only together
 *   with capacity_padding and requires C>=E (location.cu:349-358,227-230).
 *   T==0 writes loads=counts=0.
 */
int brt_hip_generate_indices_and_loads(const int32_t* mask, int32_t* indices, int32_t* loads,
                                       int32_t* counts, int T, int E, const int32_t* caps, int C,
                                       int capacity_padding, int path_wise_padding,
                                       int is_tag_index, void* workspace, size_t workspace_bytes,
                                       void* stream);

/*
 * brt_hip_generate_indices_and_loads for callers that cannot allocate (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results without the workspace: the per-band column sums go
 * through a buffer built into the library (brt_hip_static_scratch_bytes() bytes, 1 MiB, held on
 * every GPU the library runs on until the process ends).  The entry point calls no allocating
 * routine.  A mask whose brt_hip_scan_workspace_bytes(T, E) exceeds the buffer is refused with
 * BRT_E_WORKSPACE (nothing is launched); [8192,64], [100352,8] and [1<<20,64] fit.  The buffer
 * carries nothing from call to call and needs no clearing, but every call on one GPU uses the
 * same buffer: calls that can overlap on one GPU (two streams, two threads) race.  The first
 * call on a device looks the buffer's address up (hipGetSymbolAddress); make that call outside
 * graph capture.
 */
size_t brt_hip_static_scratch_bytes(void);
int brt_hip_generate_indices_and_loads_static(const int32_t* mask, int32_t* indices,
                                              int32_t* loads, int32_t* counts, int T, int E,
                                              const int32_t* caps, int C, int capacity_padding,
                                              int path_wise_padding, int is_tag_index,
                                              void* stream);

/*
 * Replaces router::ThrottleHotmask (location.h:13-19, location.cu:59-130,304-315).
 *   out[t,e] = 1 iff mask[t,e]==1 and prefix[e] + cumsum(mask)[t,e] <= threshold[e]
 *   prefix[e] <- min(prefix[e] + sum(mask[:,e]), threshold[e])   (in place)
 * `out` is fully written (no pre-zeroing needed).  T==0 leaves prefix untouched.
 */
int brt_hip_throttle_hotmask(const int32_t* mask, int32_t* out, int32_t* prefix,
                             const int32_t* threshold, int T, int E, void* workspace,
                             size_t workspace_bytes, void* stream);

/*
 * Replaces router::ConvertIndexFormat (location.h:21-27, location.cu:259-302,317-333).
 *   tag_to_seat=0: dst[src[t,e]-1, e] = t+1 for src[t,e] != 0
 *   tag_to_seat=1: dst[src[s,e]-1, e] = s+1 for s < loads[e], under the
 *                  reference's stop rule (slot s is converted iff the tags at
 *                  s, s-1024, s-2048, ... are all non-zero)
 * `dst` must be zero-filled by the caller.  `loads` is only read when
 * tag_to_seat=1.
 */
int brt_hip_convert_index_format(const int32_t* src, int32_t* dst, const int32_t* loads, int T,
                                 int E, int tag_to_seat, void* stream);

/*
 * Replaces router::DispatchWithIndicesAndLoads<dtype> (include/brt/router/route.h:14-28,
 * src/router/route.cu:13-206,284-465).
 *
 *   src       1-d routing: [T, cell]; 2-d routing: [T, E, cell] (path e reads
 *             src[:, e, :]; no transposed copy is needed)
 *   dst       [P, cell]
 *   gates     [T,E] in `dtype`, or NULL (unweighted); 1-d routing only
 *   indices   [T,E] seat indices (is_tag_index=0) or tag lists (is_tag_index=1)
 *   loads     [E]
 *   counts    [E] or NULL.  Non-NULL (seat mode only): the routed rows of path e
 *             are exactly seats 1..min(counts[e],loads[e]); the kernel then
 *             writes every row of dst (data rows, and zeros for the padding
 *             rows) and dst/new_tags need no pre-zeroing.  NULL: dst and
 *             new_tags must be zero-filled by the caller (the reference's
 *             contract, router.cc:219,246).
 *   old_tags  [T] or NULL; new_tags [P] or NULL.  new_tags non-NULL enables tag
 *             generation: new_tags[row] = old_tags ? old_tags[t] : t+1.
 *   cell      elements per row, in units of `dtype`
 *   P         rows of dst (rows >= P are never written)
 *   max_path_load  0 = paths packed back to back (start[e] = sum(loads[:e]));
 *             otherwise start[e] = e*max_path_load and seats beyond max_path_load are
 *             dropped (a path's block ends at the stride; brt_hip_combine applies the
 *             same bound)
 *   Weighted rows are src*gate rounded once to `dtype`; unweighted rows are
 *   byte copies.
 */
int brt_hip_dispatch(const void* src, void* dst, const void* gates, const int32_t* indices,
                     const int32_t* loads, const int32_t* counts, const int32_t* old_tags,
                     int32_t* new_tags, int T, int cell, int E, int P, int max_path_load,
                     int is_1d_routing, int is_tag_index, int dtype, void* stream);

/*
 * Index generation and dispatch in one dependent step: what
 * brt_hip_generate_indices_and_loads (seat indices) followed by brt_hip_dispatch (1-d routing,
 * unweighted, counts given, max_path_load = 0) write, from two launches instead of three -- the
 * second pass of the scan moves the rows of its own cells as soon as it knows their seats.  Fuses
 * src/router/location.cu:212-257 with src/router/route.cu:13-103 (the reference runs them as
 * separate kernels, router.cc:100-140,180-250); results are bit-identical to the two calls.
 *
 *   mask      [T,E] int32 hot mask of zeros and ones (what brt_hip_dispatch assumes when it is
 *             given counts); cells [T, cell_bytes]: rows of any dtype, 16-byte aligned
 *   rows      [P, cell_bytes] out: EVERY row is written -- routed rows, zeros for the padding
 *             rows of a path and for the rows past the last path (P may exceed sum(loads):
 *             a caller that cannot read the loads back allocates an upper bound)
 *   indices   [T,E] out, loads [E] out, counts [E] out or NULL: as brt_hip_generate_indices_and_loads
 *   row_tags  [P] out or NULL: 1-based cell of every row, 0 for rows no cell owns (the new_tags
 *             of brt_hip_dispatch; what brt_hip_combine_by_tags reads)
 *   caps, C, capacity_padding, path_wise_padding: the capacity rules of location.cu:222-256
 *   workspace at least brt_hip_route_and_dispatch_workspace_bytes(T, E, cell_bytes) bytes
 *
 * Shapes it takes: 1 <= E <= 64, T >= 1, cell_bytes a multiple of 16, at most 8 supported
 * capacities unless padding path-wise, and a batch whose bands can hold its cells
 * (brt_hip_route_and_dispatch_supported() returns 1; e.g. up to 16384 cells of 1536 bytes over 64 paths, or
 * 262144 cells of 192 bytes over 8 paths).  Anything else is refused with BRT_E_UNSUPPORTED and nothing is launched:
 * make the two calls.
 */
int brt_hip_route_and_dispatch_supported(int T, int E, size_t cell_bytes, int C,
                                         int path_wise_padding);
size_t brt_hip_route_and_dispatch_workspace_bytes(int T, int E, size_t cell_bytes);
int brt_hip_route_and_dispatch(const int32_t* mask, const void* cells, void* rows,
                               int32_t* indices, int32_t* loads, int32_t* counts,
                               int32_t* row_tags, int T, int E, int P, size_t cell_bytes,
                               const int32_t* caps, int C, int capacity_padding,
                               int path_wise_padding, void* workspace, size_t workspace_bytes,
                               void* stream);

/*
 * Replaces router::CombineWithIndicesAndLoads<dtype>, seat-index mode
 * (route.h:30-44, route.cu:208-282,467-518).
 *
 *   src [P, cell] in in_dtype; dst [T, cell] in out_dtype; gates [T,E] in
 *   gate_dtype or NULL.
 *   dst[t] = sum over e ascending with 1 <= indices[t,e] <= loads[e] of
 *            src[start[e]+indices[t,e]-1] (* gates[t,e]),
 *   each product rounded to fp32, accumulated in fp32 in that order from 0, and
 *   rounded once to out_dtype.  is_residual=0: tokens without a valid route get
 *   a zero row (dst needs no pre-zeroing).  is_residual=1: such rows of dst are
 *   left untouched, rows of routed tokens are overwritten.
 */
int brt_hip_combine(const void* src, void* dst, const void* gates, const int32_t* indices,
                    const int32_t* loads, int T, int cell, int E, int P, int max_path_load,
                    int is_residual, int in_dtype, int out_dtype, int gate_dtype, void* stream);

/*
 * Combine for routes in which no cell owns more than one row (top-1 protocols),
 * driven by the per-row tags that dispatch generates (new_tags above; the
 * reference produces them with tag_generating=true, router.cc:235-250, and carries
 * them on the tag stack of the routed tensor).  Gives exactly the rows that
 * brt_hip_combine(..., gates=NULL, is_residual=1) gives for such a route, with
 * one memory round trip less: a row and its tag are fetched together, nothing has
 * to be looked up in the [T,E] index matrix first.  "Exactly" includes the zero that a
 * sum starting at zero makes of a -0 (0 + -0 = +0): a -0 element is stored as +0.
 *
 *   src       [P, cell] in in_dtype
 *   dst       [T, cell] in out_dtype (= in_dtype, or BRT_F32); rows of cells that
 *             own no row are left untouched
 *   row_tags  [P]: 1-based cell of row p, 0 for a padding row; tags > T are ignored
 *   Rows must be whole 16-byte units (BRT_E_UNSUPPORTED otherwise: use brt_hip_combine).
 *   If two rows carry the same tag the result is unspecified (one of them wins).
 */
int brt_hip_combine_by_tags(const void* src, void* dst, const int32_t* row_tags, int P, int cell,
                            int T, int in_dtype, int out_dtype, void* stream);

/*
 * Gate front-end (the three torch launches of TopKProtocol.make_route_decision,
 * python/brt/router/protocol/topk.py:26-31: topk, zeros_like, scatter_, in one pass):
 *   hot_mask[t,e] = 1 if scores[t,e] is among the k largest of row t, else 0.
 *   scores [T,E] in `dtype`, hot_mask [T,E] int32 (every element is written).
 *   NaN ranks above every number (torch.topk); among equal scores the lowest
 *   column wins (torch leaves that choice unspecified).  0 <= k <= E <= 1024.
 */
int brt_hip_topk_hot_mask(const void* scores, int32_t* hot_mask, int T, int E, int k, int dtype,
                          void* stream);

/*
 * Replaces the homo-fused expert kernel launch jit::CUDACompiler::HomoExecute
 * (src/jit/compiler.cu:151-246, binding src/backend/torch/jit.cc:54-75) for
 * Linear branches (python/brt/jit/modules/linear.py:15-61):
 *
 *   out[start[e] : start[e]+loads[e], :] =
 *        act( x[start[e] : start[e]+loads[e], :] @ W_e^T + b_e ),  start[e] = sum(loads[:e])
 *
 *   x [P,K], out [P,N] bf16 row-major; `weights` is a device array of E
 *   pointers to W_e [N,K] bf16 row-major (torch Linear layout); `biases` is a
 *   device array of E pointers to b_e [N] bf16, or NULL; `loads` [E] int32 is
 *   read on the device (no host copy, any non-negative values, sum <= P).
 *   One launch covers all experts; accumulation is fp32 on the bf16 MFMA units.
 *   K and N must be multiples of 8 (16-byte rows; BRT_E_UNSUPPORTED otherwise), x and out
 *   16-byte aligned.  `act` is one of BRT_ACT_*; GELU is the erf form
 *   (v * Phi(v), to 4.3e-6 absolute before the rounding to bf16).
 *   The GEMM kernels use more than 64 KB of LDS, which has to be allowed once per kernel and
 *   device (a function attribute, set under a lock on the first launch): make the first call of
 *   every GEMM entry point on a device outside a graph capture, as for the static scratch above.
 */
int brt_hip_grouped_gemm(const void* x, const void* const* weights, const void* const* biases,
                         void* out, const int32_t* loads, int E, int P, int K, int N, int act,
                         void* stream);

/*
 * The same grouped GEMM with the routing folded into it (no counterpart in the
 * reference, which dispatches, runs the expert kernel and combines in separate
 * launches; this is the fusion of src/router/route.cu:13-282 into the operand load
 * and the result store of the expert kernel).  `tags` is the [T,E] tag-index matrix
 * that brt_hip_generate_indices_and_loads writes with is_tag_index=1: column e
 * lists, in seat order, the 1-based cells routed to path e; 0 = empty slot.
 *
 *   gather_in=1   x is the cell-major tensor [T,K]; row s of expert e is
 *                 x[tags[s,e]-1] (what dispatch would have copied there), an empty
 *                 slot is a row of zeros.  gather_in=0: x is [P,K] as above.
 *   scatter_out=1 out is cell-major [T,N]; row s of expert e is stored to
 *                 out[tags[s,e]-1] (what combine does for a route in which no cell is
 *                 on more than one path, without gates, with out as the residual,
 *                 including +0 for a -0 element); rows of empty slots are dropped.  scatter_out=0: out is [P,N].
 *   Only rows s < min(loads[e], T) of column e are used, so a clipped capacity drops the
 *   overflow exactly as seat indices beyond loads[e] do, and a load padded beyond the T rows
 *   the tag matrix has (a capacity above the batch size) names empty slots.  With gather_in the cell-major
 *   input is limited to 2 GiB.
 *   row_tags_out  NULL, or [P] int32: receives the 1-based cell behind every row of the path-major
 *                 layout (0 for an empty slot and for the rows past sum(loads)), which is what
 *                 brt_hip_dispatch writes as new_tags; brt_hip_combine_by_tags takes it, so a
 *                 route that gathers in the first GEMM never runs dispatch at all.
 */
int brt_hip_grouped_gemm_routed(const void* x, const void* const* weights,
                                const void* const* biases, void* out, const int32_t* loads,
                                const int32_t* tags, int E, int P, int T, int K, int N, int act,
                                int gather_in, int scatter_out, int32_t* row_tags_out, void* stream);

/*
 * brt_hip_grouped_gemm with an fp32 result: out [P,N] float receives the fp32 accumulator after
 * bias and activation, which is the output type of the reference's expert kernel
 * (benchmark/switch_moe/switch_expert.py:74-92 allocates fp32 outputs, test/python/jit_test.py:157-203
 * compares in fp32).  x and the weights stay bf16: brt_hip_cast_f32_to_bf16 converts fp32 operands.
 */
int brt_hip_grouped_gemm_f32out(const void* x, const void* const* weights, const void* const* biases,
                                float* out, const int32_t* loads, int E, int P, int K, int N, int act,
                                void* stream);
/* brt_hip_grouped_gemm_routed with the fp32 result of brt_hip_grouped_gemm_f32out. */
int brt_hip_grouped_gemm_routed_f32out(const void* x, const void* const* weights,
                                       const void* const* biases, float* out, const int32_t* loads,
                                       const int32_t* tags, int E, int P, int T, int K, int N, int act,
                                       int gather_in, int scatter_out, int32_t* row_tags_out,
                                       void* stream);

/*
 * dst[i] = bf16(src[i]) (round to nearest even), n elements; both 16-byte aligned.  For callers that
 * hold the reference's fp32 activations or weights (no counterpart in the reference, whose kernels
 * compute in fp32).
 */
int brt_hip_cast_f32_to_bf16(const float* src, void* dst, size_t n, void* stream);

/*
 * The routed grouped GEMM on the compact route (no counterpart in the reference): as
 * brt_hip_grouped_gemm_routed, with the rows named by the row_entries vector [P] that
 * brt_hip_route_by_path writes (1-based entry t*k+j+1 of each row of the dispatched layout,
 * 0 = padding row) instead of the [T,E] tag matrix.  Row r of the layout is cell
 * (row_entries[r]-1)/k of x (gather_in) or of out (scatter_out; k must be 1).  Rows of path e
 * start at sum(loads[:e]) (no max_path_load layout).
 */
int brt_hip_grouped_gemm_by_rows(const void* x, const void* const* weights,
                                 const void* const* biases, void* out, const int32_t* loads,
                                 const int32_t* row_entries, int k, int E, int P, int T, int K,
                                 int N, int act, int gather_in, int scatter_out, void* stream);

/*
 * The routed grouped GEMM with the WEIGHTED combine of a route with several paths per cell folded
 * into its store (the weighted branch of combine_with_seat_indices, src/router/route.cu:236-243:
 * `in * gate`, then one atomic add per element): for every row r of the dispatched layout that a
 * cell c owns on path e,
 *     out[c, :] += gates(c, e) * bf16(act(x_row @ W_e^T + b_e))
 * with fp32 atomic adds into the fp32 matrix out [T,N], which the caller has filled with zeros (or
 * with what the sums are to be added to) before the call; cells without a row are not touched.  The
 * addend is exactly what brt_hip_grouped_gemm_routed would store for the row (rounded to bf16)
 * times the fp32 gate, so the result equals brt_hip_combine on that GEMM's output with fp32 gates
 * and fp32 out: bit for bit with at most two paths per cell (an fp32 sum of two does not depend on
 * the order), to the last bits of an fp32 sum in another order with more.
 * entries_per_cell = 0: tags is the [T,E] tag matrix and gates the [T,E] fp32 gate matrix;
 * entries_per_cell = k > 0: tags is the row-entry vector [P] of brt_hip_route_by_path and gates its
 * [T,k] fp32 weights (the weight of a row is gates[entry-1]).  gather_in as in
 * brt_hip_grouped_gemm_routed.  Calls that add into the same out on different streams at the same
 * time are summed correctly; nothing else may write out meanwhile.
 */
int brt_hip_grouped_gemm_accumulate(const void* x, const void* const* weights,
                                    const void* const* biases, float* out, const int32_t* loads,
                                    const int32_t* tags, int entries_per_cell, const float* gates,
                                    int E, int P, int T, int K, int N, int act, int gather_in,
                                    void* stream);

/* ---------------------------------------------------------------------------
 * Tag-index gather (the default GatherRouter path of the reference).
 *
 * brt_hip_unique_tags replaces the `_unique(cat(tags), sorted, return_inverse)` call of
 *   fuse_split_cells_from_paths (src/backend/torch/router.cc:348-369): `tags` [n] (int32 or
 *   int64, `tag_bits` 32 or 64) with every value in [lo, hi] (the caller's min and max; values
 *   outside get inverse -1 and are left out) -> `unique_tags` (same element type, room for
 *   min(n, hi-lo+1) values, ascending), `inverse` [n] int64 (position of tags[i] in
 *   unique_tags), `n_unique` [1] int32 on the device.  No sort: a presence table over the range
 *   and one prefix sum.  hi-lo+1 may be at most 2^25 (BRT_E_UNSUPPORTED beyond; the workspace
 *   size query returns 0 then).
 *
 * brt_hip_combine_by_index replaces the tag-mode branch of combine_with_indices_and_loads
 *   (router.cc:449-472: `repeat` of the index to one int64 per element + `scatter_reduce`
 *   "sum" into zeros): out_data[r] = sum of in_data[p] over the rows p with index[p] == r, for
 *   r < n_out; rows nobody points to become zero, rows with an index outside [0, n_out) are
 *   left out.  `index` is int32 or int64 (`index_bits`).  The sum runs in ascending p in fp32 and
 *   is rounded once, so it is reproducible (the reference's atomics add in arrival order).
 *   dtypes as brt_hip_combine: fp32, fp16, bf16, or a 16-bit input with fp32 output.
 *   out_data is written whole; it needs no zero fill.
 *
 * Both take a caller-provided workspace (4-byte aligned, size from the query functions) and
 * queue 1 to 5 small launches on `stream` (small inputs are handled by a single workgroup).
 */
size_t brt_hip_unique_tags_workspace_bytes(long lo, long hi);
int brt_hip_unique_tags(const void* tags, int tag_bits, long n, long lo, long hi, void* workspace,
                        size_t workspace_bytes, void* unique_tags, int64_t* inverse,
                        int32_t* n_unique, void* stream);
size_t brt_hip_combine_by_index_workspace_bytes(int P, int n_out);
int brt_hip_combine_by_index(const void* in_data, void* out_data, const void* index, int index_bits,
                             int P, int cell, int n_out, void* workspace, size_t workspace_bytes,
                             int in_dtype, int out_dtype, void* stream);

/* ---------------------------------------------------------------------------
 * Compact route format (no counterpart in the reference's extension; it replaces, for routes
 * with k chosen paths per cell, the dense [T,E] hot mask and seat matrix that the reference
 * passes from protocol to fabric: python/brt/router/protocol/topk.py:26-31,
 * src/router/location.cu:212-257, src/router/route.cu:13-282).
 *
 *   path_ids    [T,k] int32  paths of a cell, all different; an id outside [0,E) is no route
 *   weights     [T,k] fp32   gate value of each entry
 *   seat_rows   [T,k] int32  1-based row of the dispatched buffer of entry (t,j); 0 = dropped
 *   row_entries [P]   int32  1-based entry number t*k+j+1 of each dispatched row; 0 = padding
 *                            (for k == 1 this is the new_tags output of brt_hip_dispatch)
 *
 * brt_hip_gate_topk: scores [T,E] (fp32/fp16/bf16) -> path_ids in the order of selection
 *   (largest first, NaN above every number, lowest column among equals, as
 *   brt_hip_topk_hot_mask), weights (or NULL) = the chosen scores as fp32, or with softmax != 0
 *   their softmax over the row (fp32, exp(x - max) / sum: the Switch router's probabilities,
 *   benchmark/switch_moe/switch_transformer.py:240-253), and optionally the dense hot_mask
 *   (or NULL).  One launch; E <= 1024.
 *
 * brt_hip_route_by_path: what brt_hip_generate_indices_and_loads computes from the mask,
 *   from path_ids: loads [E] by the same capacity rules, counts [E] (or NULL) the real row
 *   counts, seat_rows and row_entries.  Seats of a path go to its cells in ascending cell
 *   order; entry (t,j) of path e with seat s <= loads[e] owns row start[e] + s, start[e] = sum
 *   of the loads before e, or e * max_path_load when max_path_load != 0 (seats beyond
 *   max_path_load are dropped then).  Rows beyond P are dropped; row_entries is written whole
 *   ([0,P)), it needs no zero fill.  E <= 512.  Routes of up to 2048 entries take one launch of
 *   one workgroup; larger ones two launches that pass per-wavefront counters through the
 *   workspace (size from brt_hip_route_by_path_workspace_bytes, 4-byte aligned, uninitialised,
 *   not shared between calls that run at the same time).
 *
 * brt_hip_dispatch_by_rows: dst[r] = src[(row_entries[r]-1) / k] (times weights[row_entries[r]-1]
 *   when weights != NULL: an fp32 product, then rounded to the data type), zero rows where
 *   row_entries[r] == 0.
 *   dst [P,cell] is written whole.  Rows must be whole 16-byte units.
 *
 * brt_hip_combine_by_rows: dst[t] = sum over the entries j of cell t with seat_rows[t,j] != 0,
 *   in ascending path id, of weights[t,j] * src[seat_rows[t,j]-1] (weights NULL = 1), in fp32 from 0
 *   with product and sum rounded separately: the order and roundings of brt_hip_combine.  Cells
 *   without a row keep dst when is_residual != 0 and are zeroed otherwise.  k <= 8; dtypes as
 *   brt_hip_combine.
 */
int brt_hip_gate_topk(const void* scores, int T, int E, int k, int dtype, int softmax,
                      int32_t* path_ids, float* weights, int32_t* hot_mask, void* stream);
size_t brt_hip_route_by_path_workspace_bytes(int T, int k, int E);
int brt_hip_route_by_path(const int32_t* path_ids, int T, int k, int E, const int32_t* caps, int C,
                          int capacity_padding, int path_wise_padding, int max_path_load,
                          int32_t* loads, int32_t* counts, int32_t* seat_rows,
                          int32_t* row_entries, int P, void* workspace, size_t workspace_bytes,
                          void* stream);
int brt_hip_dispatch_by_rows(const void* src, void* dst, const float* weights,
                             const int32_t* row_entries, int P, int T, int k, int cell, int dtype,
                             void* stream);
int brt_hip_combine_by_rows(const void* src, void* dst, const float* weights,
                            const int32_t* path_ids, const int32_t* seat_rows, int T, int k,
                            int cell, int P, int is_residual, int in_dtype, int out_dtype,
                            void* stream);

/*
 * Measurement aid (no counterpart in the reference; bench.py reports what it reads beside the
 * compute-bound shapes): brt_hip_grouped_gemm through the 256 x 256 ping-pong kernel, whatever the
 * shape (BRT_E_UNSUPPORTED when that kernel does not take it: K must be a multiple of 64 and at
 * least 128), which also writes into clocks[0..2] (device, 8-byte aligned) what the first
 * wavefront of the first tile's workgroup spent in its K loop: shader clocks (s_memtime), ticks of
 * the constant 100 MHz counter (s_memrealtime), and the number of K-steps of 64.  A full tile
 * issues 2 x 1024 clocks of MFMA per SIMD and K-step, so clocks[0] / clocks[2] says how much of
 * the loop is matrix work and clocks[0] / clocks[1] at which clock the part ran it.  The output is
 * that of brt_hip_grouped_gemm, bit for bit.
 */
int brt_hip_grouped_gemm_timed(const void* x, const void* const* weights, const void* const* biases,
                               void* out, const int32_t* loads, int E, int P, int K, int N, int act,
                               long long* clocks, void* stream);

/*
 * Measurement aid (no counterpart in the reference; bench.py's `ceilings` uses it): `workgroups`
 * workgroups of four wavefronts, one per SIMD, each issue iters x 8 v_mfma_f32_32x32x16_bf16
 * (32768 flop per wavefront and instruction) on register operands of random bit patterns and touch
 * no memory.  clocks[0] (device, 8-byte aligned) receives the shader clocks the first wavefront
 * spent in its loop; clocks[1] is reserved and never written in practice.  Launch time and
 * clocks[0] give the rate the matrix pipes sustain under the part's power limit and the shader
 * clock they sustain it at.  workgroups 1..65536, iters >= 1.
 */
int brt_hip_probe_mfma_rate(int workgroups, int iters, long long* clocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BRT_HIP_H_ */
