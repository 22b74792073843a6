/*
 * sgnn.h -- C ABI of libsgnn_hip.so: the MI355X (gfx950) implementation of SuperGNN's
 * data-parallel hot path.
 *
 *   1. CSR SpMM neighbour aggregation        out (+)= A * X          (fp32, sum / mean)
 *   2. boundary-row quantize + bit-pack      fp32 -> int8/int4/int2  (per-row min/scale)
 *   3. unpack + dequantize                   int8/int4/int2 -> fp32
 *   4. fused unpack + dequantize + SpMM      remote columns arrive packed
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - the caller allocates every output; functions write in place (the reference extension has
 *     the same ownership rule: super_gnn/ops/csrc/spmm.h:3-6, quantization_arm.h:5-10);
 *   - `stream` is a hipStream_t passed as void*; work is enqueued asynchronously on it;
 *   - the return value is 0 on success and negative on error; sgnn_last_error() then returns a
 *     message for the calling thread (the reference raises through AT_ASSERTM / TORCH_CHECK,
 *     super_gnn/ops/csrc/utils.h:12-13);
 *   - reference citations are relative to the reference checkout.
 */
#ifndef SGNN_H
#define SGNN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SGNN_OK 0
#define SGNN_ERR_ARG (-1)     /* bad argument (null pointer, size, alignment, bits) */
#define SGNN_ERR_HIP (-2)     /* a HIP runtime call failed                          */
#define SGNN_ERR_RANGE (-3)   /* an index in the input is out of range              */

typedef void *sgnn_stream_t; /* hipStream_t */

/* Message of the last error raised on the calling thread ("" if none). */
const char *sgnn_last_error(void);

/* ABI version, bumped on any signature change. */
int sgnn_version(void);

/* ---------------------------------------------------------------------------------------------
 * SpMM
 * ------------------------------------------------------------------------------------------- */

/* Per-matrix schedule: 32-bit column indices, the row classes and their work lists.
 *   short rows : chunks of consecutive rows (about 64 edges), one lane group per chunk;
 *   long rows  : edges regrouped by column class (a hash of col, 8 classes) and cut into pieces, one
 *                lane group per piece, workgroup i serving class i % 8 so that each XCD's L2 caches
 *                its own class of dense rows; partial sums land in a buffer owned by the plan.  The
 *                regrouping is skipped when column popularity is essentially uniform (it then only
 *                costs): pieces are cut from the CSR order instead;
 *   empty rows : a list, used only by the modes that must write them.
 * Plays the role of the row_splits the reference computes once per matrix and caches on it
 * (super_gnn/ops/spmm_kernel.py:49-58, distribute_work_for_row :8-29).
 * The plan owns device copies of rowptr and of the (narrowed) column indices. */
typedef struct sgnn_spmm_plan sgnn_spmm_plan;

/* rowptr: int64[M+1] (device). col: int64[nnz] if col_is_i64 else int32[nnz] (device).
 * K = number of sparse columns = rows of the dense operand.  M and K must be below 2^31 (the
 * reference's kernel computes its offsets in 32-bit int as well, super_gnn/ops/csrc/spmm.cpp:30,94).
 * nnz may be larger: a matrix of 2^31 edges or more is held as consecutive row blocks of fewer edges,
 * each scheduled on its own, and every call on the plan runs the blocks one after the other on the
 * caller's stream (same results; a single row must still have fewer than 2^31 edges).
 * Every col must lie in [0, K) and rowptr must be non-decreasing with rowptr[0] == 0: both are
 * checked (SGNN_ERR_RANGE).
 * long_row_threshold: rows with more edges take the long-row path (<= 0: default 128).
 * piece_edges: minimum edges per long-row piece (<= 0: default 96).
 * Synchronises the stream (the work lists are built on the host). */
int sgnn_spmm_plan_create(const int64_t *rowptr, const void *col, int col_is_i64, int64_t M,
                          int64_t K, int64_t nnz, int long_row_threshold, int piece_edges,
                          sgnn_stream_t stream, sgnn_spmm_plan **plan_out);

int sgnn_spmm_plan_destroy(sgnn_spmm_plan *plan);

/* info[0]=M, [1]=K, [2]=nnz, [3]=#long rows, [4]=#pieces, [5]=edges in long rows,
 * [6]=long_row_threshold, [7]=piece_edges, [8]=1 if the long rows were regrouped by column class,
 * [9]=share of all edges that point at the 16384 most popular columns, in parts per million (0 when
 * it was not measured). */
int sgnn_spmm_plan_info(const sgnn_spmm_plan *plan, int64_t info[10]);

/* Which schedule sgnn_spmm_csr_f32 takes for a dense operand of F contiguous, 16-byte aligned fp32 columns:
 * info[0] = 1 for the band schedule, 0 for the row-class schedule above.  The band schedule is for
 * dense-degree matrices whose dense operand does not fit the L2 caches (e.g. 233 k nodes with ~490 edges
 * per row at F = 602): the column space is cut into bands of info[1] columns (info[2] bands), the product
 * is one launch per band accumulating onto out, and inside a launch the eight XCDs split the feature axis
 * into info[3] slices so that each L2 holds one band of one slice and every repeated gather hits it.  It
 * needs column-sorted rows (checked on first use; unsorted matrices keep the row-class schedule) and is
 * built on the first call that wants it.  A row's edges are summed in CSR order with one fma per edge
 * starting from the old out value, so its results are bit-identical to the reference's for every row
 * length.  Replaces the per-64-column re-walk of the edge list in the reference's kernel
 * (super_gnn/ops/csrc/spmm.cpp:502-510). */
int sgnn_spmm_plan_schedule(const sgnn_spmm_plan *plan, int64_t F, int64_t info[4]);

/* Optional: declare an edge-value array constant until the next bind.  The plan keeps a copy of the
 * long rows' values in its own (regrouped) edge order, and later sgnn_spmm_csr_f32 /
 * sgnn_spmm_csr_dq*_f32 calls that pass the SAME pointer read that copy contiguously instead of
 * going through the edge permutation (-8 % on the long-row kernel of the power-law graph).  The
 * caller must bind again after changing the array's contents (also after freeing it and getting the same
 * address back from an allocator); val == NULL unbinds.  Nothing is ever bound implicitly: a run call
 * only compares the pointer it is given with the bound one, and a different pointer is read in place.
 * A plan holds per-call state (partial sums, the restaged operand, these copies): use it, and bind it,
 * from one stream at a time, or order the streams yourself.  The reference
 * passes `value` on every call (super_gnn/ops/spmm_kernel.py:60-65) but never changes it after the
 * graph is built (DataProcessor.py:112,119), which is what this exploits. */
int sgnn_spmm_plan_bind_values(sgnn_spmm_plan *plan, const float *val, sgnn_stream_t stream);

/* out[M,F] (+)= A[M,K] * x[K,F], fp32, row-major, leading dimensions ldx / ldo (in floats).
 *
 * Replaces supergnn_ops.spmm (super_gnn/ops/csrc/spmm.cpp:594-608):
 *   accumulate != 0 : out[m,:] += sum_e val[e]*x[col[e],:], rows without edges untouched --
 *                     spmm_cpu_optimized_no_tile_v1 (spmm.cpp:348-539, empty-row skip :486);
 *   accumulate == 0 : out[m,:]  = sum_e val[e]*x[col[e],:], rows without edges zeroed --
 *                     spmm_cpu + Reducer<SUM> (spmm.cpp:177-271, reducer.h:70-74).
 * val == NULL means all ones.  row_div != NULL fuses the mean epilogue
 * out[m,:] = (...) / row_div[m] for EVERY row m (super_gnn/layers/sageconv.py:78).
 * Short rows are summed in CSR edge order with one fused multiply-add per edge starting from
 * the old out value, as the reference does (bit-identical results); long rows are summed per piece
 * and the piece partials are added in piece order (deterministic, no atomics).
 * When F >= 256, the dense operand is large (K * F * 4 bytes >= 0.9 GB) and x, out, ldx, ldo allow
 * 16-byte accesses, the product runs as consecutive feature slices of 128 ... 192 columns (same kernels
 * on column windows of x and out, same results): a gathered row then leaves 512 ... 768 bytes in the
 * caches instead of 4F, and the same cache holds more rows.  The reference walks the feature axis in
 * tiles of 64 columns for its own caches (spmm.cpp:502-510). */
int sgnn_spmm_csr_f32(sgnn_spmm_plan *plan, const float *val, const float *x, float *out,
                      int64_t F, int64_t ldx, int64_t ldo, int accumulate, const float *row_div,
                      sgnn_stream_t stream);

/* sgnn_spmm_csr_f32 for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same
 * arguments, same kernels and same results, bit for bit, as sgnn_spmm_csr_f32, but the call
 * performs no hipMalloc / hipFree and creates no stream or event: the partial sums of the long rows
 * go to a 64 MiB scratch array that lives inside the library's code object (one copy per GPU, held
 * until the process ends) instead of the plan's growable buffer.
 *   - limit: (#long-row pieces of the plan) * F * 4 bytes <= 64 MiB (sgnn_spmm_plan_info, info[4]);
 *     a larger product is refused with SGNN_ERR_ARG and nothing is launched.  Matrices without long
 *     rows never touch the scratch and have no limit.  A product that runs as feature slices (see
 *     sgnn_spmm_csr_f32) needs the partial sums of one slice at a time, and the limit then applies to
 *     the width of a slice;
 *   - every call on one GPU shares that GPU's scratch: two calls whose kernels may overlap in time
 *     (different streams, different host threads) race on it.  Calls queued on one stream are safe.
 *     Nothing in the scratch has to start at zero: each call writes every partial it later reads;
 *   - a matrix that sgnn_spmm_plan_schedule reports as band-scheduled runs that schedule here only if earlier
 *     sgnn_spmm_csr_f32 calls on this plan have already built everything it needs (building allocates): the
 *     band-major edge copy for this product's band width (info[1] of sgnn_spmm_plan_schedule; every F > 512
 *     shares one, narrower products have one per padded slice width), a restaged-operand workspace at least as
 *     large as this F needs, and the chunk list for the same kind of weights (val given or NULL: the two cut the
 *     bands into different chunks).  The simple way to guarantee that is one sgnn_spmm_csr_f32 call with the same
 *     F and the same kind of weights beforehand.  Otherwise the row-class kernels run: same result on rows of up
 *     to 128 edges, bit for bit; longer rows are summed per piece instead of in one chain (within the fp32
 *     tolerance, not the same bits);
 *   - the scratch address is looked up when a plan is created, so the call itself performs no lazy symbol
 *     lookup, and it records no profiling events (sgnn_profile_enable does not see its kernels). */
int sgnn_spmm_csr_f32_noalloc(sgnn_spmm_plan *plan, const float *val, const float *x, float *out,
                              int64_t F, int64_t ldx, int64_t ldo, int accumulate,
                              const float *row_div, sgnn_stream_t stream);

/* 1 if the reference's spmm() would take its overwrite branch for this shape
 * (float(nnz)/M/K <= 1e-4 && F > 256, super_gnn/ops/csrc/spmm.cpp:601-602), else 0. */
int sgnn_spmm_reference_overwrites(int64_t nnz, int64_t M, int64_t K, int64_t F);

/* ---------------------------------------------------------------------------------------------
 * Row-group quantization (the live training path)
 * ------------------------------------------------------------------------------------------- */

/* Packed-row offset of each segment: pseg_host[p] = sum_{q<p} ceil((seg[q+1]-seg[q]) / (8/bits)),
 * p = 0..P.  Host-only helper (no GPU work); returns the total number of packed rows or a
 * negative error.  Restates the layout rule of divide_work_v1
 * (super_gnn/ops/csrc/quantization_arm.cpp:21-77) and get_quantized_splits
 * (super_gnn/quantizer.py:91-92). */
int64_t sgnn_quant_segment_offsets(const int32_t *seg_host, int P, int bits, int32_t *pseg_host);

/* Fused per-row min/max -> (zero_point, scale) -> RNE((x-zp)/scale) -> bit-pack.
 * x f32[n,F]; q u8[pseg[P],F]; params f32[n,2] = (zero_point, scale) per row;
 * seg i32[P+1] cumulative row ranges, pseg i32[P+1] from sgnn_quant_segment_offsets (both device).
 * bits in {8,4,2}.  Packed row g of segment p holds that segment's rows g*EPB+k, first row in
 * the most significant bits; a short last group leaves its low bits zero.
 * Replaces quantize_tensor_for_all_procs and, with P == 1, quantize_tensor
 * (super_gnn/ops/csrc/quantization_arm.cpp:496-578, :433-464, kernel :79-301). */
int sgnn_quant_pack_rows_f32(const float *x, uint8_t *q, float *params, const int32_t *seg,
                             const int32_t *pseg, int P, int64_t n_rows, int64_t n_packed_rows,
                             int64_t F, int bits, sgnn_stream_t stream);

/* Inverse: x[r,:] = fma(code, scale, zero_point) for every row of every segment.
 * Replaces dequantize_tensor_for_all_procs / dequantize_tensor
 * (super_gnn/ops/csrc/quantization_arm.cpp:580-633, :466-494, kernel :303-431). */
int sgnn_unpack_dequant_rows_f32(const uint8_t *q, float *x, const float *params,
                                 const int32_t *seg, const int32_t *pseg, int P, int64_t n_rows,
                                 int64_t n_packed_rows, int64_t F, int bits, sgnn_stream_t stream);

/* The same two kernels with the operands as they sit either side of the boundary exchange:
 *   - row_index (i64[n_rows], device, nullable): row r of the quantizer's input is
 *     x[row_index[r] * ldx ...] -- the index_select into send_buf that precedes quantization in
 *     the plain (non pre-aggregated) mode, super_gnn/aggregator.py:48, folded into the load.
 *     Entries must lie in [0, n_src_rows); an entry outside reads row 0 instead of faulting.
 *     NULL: rows are x[r * ldx ...] and n_src_rows is ignored.
 *   - params_bf16 = 1: params is bf16[n,2] instead of f32[n,2] -- the form in which the reference
 *     ships (zero_point, scale), super_gnn/communicator.py:283-294 (copy_ to the bf16 buffer,
 *     all_to_all, copy_ back).  Codes are computed from the fp32 values; only the stored pair is
 *     rounded (to nearest even, NaN kept quiet), and the receiver widens it exactly. */
int sgnn_quant_pack_rows_wire_f32(const float *x, int64_t ldx, const int64_t *row_index,
                                  int64_t n_src_rows, uint8_t *q, void *params, int params_bf16,
                                  const int32_t *seg, const int32_t *pseg, int P, int64_t n_rows,
                                  int64_t n_packed_rows, int64_t F, int bits, sgnn_stream_t stream);

int sgnn_unpack_dequant_rows_wire_f32(const uint8_t *q, float *x, const void *params,
                                      int params_bf16, const int32_t *seg, const int32_t *pseg,
                                      int P, int64_t n_rows, int64_t n_packed_rows, int64_t F,
                                      int bits, sgnn_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Fused unpack + dequantize + SpMM (pre/post-aggregation mode)
 * ------------------------------------------------------------------------------------------- */

/* row_slot[r] = pseg[p] * EPB + (r - seg[p]) for the segment p that holds row r: the position of
 * row r in the padded row space of the packed buffer (packed row = slot / EPB, position inside the
 * byte = slot % EPB).  seg, pseg, row_slot are device arrays.  When every segment but the last
 * holds a multiple of EPB rows the table is the identity and callers may pass NULL instead. */
int sgnn_quant_row_slots(const int32_t *seg, const int32_t *pseg, int P, int bits, int64_t n_rows,
                         int32_t *row_slot, sgnn_stream_t stream);

/* out[M,F] (+)= A[M,K] * dequant(q)[K,F]: the dense operand is handed over as it arrives from the
 * boundary exchange -- packed codes q u8[n_packed,F] in the row-group layout plus params f32[K,2] --
 * and is decoded inside the gather, value = fma(code, scale, zero_point), then one fma per edge.
 * Replaces the pair "dequantize into recv_buf, then SPMM_forward(remote graph, recv_buf, out)" of
 * super_gnn/aggregator.py:72-93 (forward) and :159-171 (backward); no fp32 recv_buf is written or
 * re-read.  The result is bit-identical to running sgnn_unpack_dequant_rows_f32 followed by
 * sgnn_spmm_csr_f32 with the same plan.  F must be even (F % 4 == 0 takes four-code lanes, other even widths such
 * as 602 two-code lanes; an odd F is refused: dequantize, then multiply); other arguments as in
 * sgnn_spmm_csr_f32.  row_slot: see sgnn_quant_row_slots (NULL = identity). */
int sgnn_spmm_csr_dq_f32(sgnn_spmm_plan *plan, const float *val, const uint8_t *q, const float *params,
                         const int32_t *row_slot, int bits, float *out, int64_t F, int64_t ldo,
                         int accumulate, const float *row_div, sgnn_stream_t stream);

/* The fused calls below never look row_slot up per gathered row: the plan keeps
 * row_slot[col[e]] for each of its edges, streamed next to the column indices (a table lookup in
 * front of every packed-row fetch cost +23 % on the remote step).  That per-edge stream is built by
 * this call -- or by the first fused call that sees a new row_slot POINTER -- and reused while
 * the same pointer comes back: a table is taken to be constant (a partition's segment table is fixed
 * when its graph is built, super_gnn/data_manager/CommBuffer.py:37-44).  Call this again after
 * changing a table in place; row_slot == NULL drops the stream. */
int sgnn_spmm_plan_bind_row_slots(sgnn_spmm_plan *plan, const int32_t *row_slot, sgnn_stream_t stream);

/* sgnn_spmm_csr_dq_f32 with params in either form (params_bf16: see
 * sgnn_quant_pack_rows_wire_f32).  With a 0/1 selection matrix as A this is also the scatter of the
 * plain mode's backward pass, local_grad.index_add_(0, idx, dequantize(q))
 * (super_gnn/aggregator.py:159-175), summed in index order and free of atomics. */
int sgnn_spmm_csr_dq_wire_f32(sgnn_spmm_plan *plan, const float *val, const uint8_t *q,
                              const void *params, int params_bf16, const int32_t *row_slot, int bits,
                              float *out, int64_t F, int64_t ldo, int accumulate,
                              const float *row_div, sgnn_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Feature-packed mixed-bit quantization ("v1")
 * ------------------------------------------------------------------------------------------- */

/* params f32[n,3] = (bits, zero_point, scale): bits is read, zero_point/scale are written.
 * range i64[n+1]: row i's bytes are q[range[i] .. range[i+1]).  The table is trusted, as in the reference:
 * range[i+1] - range[i] must be at least ceil(F * bits_i / 8), or a row's bytes spill into the next row's
 * (the Python layer checks this once per (params, range) pair).  Rows may lie anywhere in q; where the ranges
 * of consecutive rows follow one another without gaps (range[i+1] - range[i] == ceil(F * bits_i / 8), the
 * layout the reference builds) the bytes of several rows leave the GPU as one run of stores.  A row whose bits
 * is not 8, 4 or 2 is left untouched (the reference prints an error and skips it, quantization_x86.cpp:244-245).
 * Replaces quantize_tensor_v1 (super_gnn/ops/csrc/quantization_arm.cpp:635-702). */
int sgnn_quant_v1_f32(const float *x, uint8_t *q, const int64_t *range, float *params, int64_t n,
                      int64_t F, sgnn_stream_t stream);

/* Replaces dequantize_tensor_v1 (super_gnn/ops/csrc/quantization_arm.cpp:704-757). */
int sgnn_dequant_v1_f32(const uint8_t *q, float *x, const int64_t *range, const float *params,
                        int64_t n, int64_t F, sgnn_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Measurement helpers (no reference counterpart; the reference times with std::chrono under
 * #define PROFILE, super_gnn/ops/csrc/spmm.cpp:12,352-354,518-523)
 * ------------------------------------------------------------------------------------------- */

/* on != 0: drop earlier records and start recording one HIP event pair around every kernel
 * launch, on the stream the kernel is launched on.  on == 0: stop recording (records kept). */
int sgnn_profile_enable(int on);

/* Waits for the recorded launches of kernel_id and returns their count and summed duration. */
int sgnn_profile_read(int kernel_id, int64_t *launches, double *total_ms);

/* Kernel ids are 0 .. sgnn_profile_kernel_count()-1; the name is the __global__ function's. */
const char *sgnn_profile_kernel_name(int kernel_id);
int sgnn_profile_kernel_count(void);

/* dst[0..n) = src[0..n) with 128-bit non-temporal accesses: the attainable-bandwidth yardstick
 * and the calibration kernel for hardware traffic counters.  n % 4 == 0, 16-byte aligned. */
int sgnn_stream_copy_f32(const float *src, float *dst, int64_t n, sgnn_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SGNN_H */
