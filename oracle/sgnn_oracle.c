/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Plain-C CPU restatement of the SuperGNN hot path (CSR SpMM neighbour aggregation and the
 * boundary-row quantize / bit-pack / unpack / dequantize pipeline).  It exists so that the HIP
 * kernels can be checked against the reference's arithmetic on identical inputs, and so that
 * bench.py can time a CPU baseline beside the GPU number.  Only tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg may load this library; the product path never does.
 *
 * Every function names the reference lines (paths relative to the reference checkout) whose
 * arithmetic it restates.  No reference source text is reproduced: loops are rewritten scalar.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   orc_spmm_accumulate / orc_spmm_overwrite / orc_spmm_dispatch
 *       - the reference's own x86 extension built into oracle/_ref (bit-for-bit on the
 *         accumulate branch, allclose on the overwrite branch), scipy CSR @ dense, an fp64
 *         accumulation, brute force on tiny inputs, and algebraic invariants.
 *   orc_quant_rows / orc_dequant_rows
 *       - hand-derived known-answer vectors, torch.round((x-min)/scale) in fp32, the x86
 *         reference quantize_tensor/dequantize_tensor in oracle/_ref (bytes bit-exact given the
 *         same min/scale), and the reference's segment-concatenation invariant
 *         (tests/test_quantization_ops.py:214-228 of the reference).
 *   orc_quant_v1 / orc_dequant_v1
 *       - golden bytes/params in the reference's tests/test_quantizer.py:57-114 and the x86
 *         reference in oracle/_ref.
 *
 * Build: see oracle/Makefile (gcc -O3 -mavx2 -mfma -fopenmp -ffp-contract=off).
 * -ffp-contract=off matters: every fused multiply-add below is an explicit fmaf().
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------------------------------
 * Thread split balanced by nnz.  Restates the intent of distribute_work_for_row
 * (super_gnn/ops/spmm_kernel.py:8-29): contiguous row ranges of roughly equal edge count.
 * The split only decides which thread computes a row; it never changes a result.
 * ---------------------------------------------------------------------------------------- */
static void nnz_balanced_split(const int64_t *rowptr, int64_t M, int T, int64_t *split) {
    int64_t nnz = rowptr[M] - rowptr[0];
    split[0] = 0;
    int64_t m = 0;
    for (int t = 1; t < T; t++) {
        int64_t target = rowptr[0] + (nnz * t) / T;
        while (m < M && rowptr[m] < target) m++;
        split[t] = m;
    }
    split[T] = M;
}

/* ------------------------------------------------------------------------------------------
 * out[m,:] += sum_e val[e] * x[col[e],:]  for every NON-EMPTY row m; empty rows are untouched.
 *
 * Follows spmm_cpu_optimized_no_tile_v1 (super_gnn/ops/csrc/spmm.cpp:348-539) with its inner
 * kernel_1xN (spmm.cpp:87-162): the accumulator of feature f starts from out[m,f]
 * (spmm.cpp:98-113), walks the row's edges in CSR order (spmm.cpp:116), does ONE fused
 * multiply-add per edge (spmm.cpp:142-145), and is stored back (spmm.cpp:148-161).  The
 * reference tiles the feature axis by 64 and re-walks the edges per tile (spmm.cpp:502-510);
 * features are independent, so the per-feature result does not depend on the tiling.
 * Empty rows are skipped by the test at spmm.cpp:486.
 * ---------------------------------------------------------------------------------------- */
void orc_spmm_accumulate(const int64_t *rowptr, const int64_t *col, const float *val,
                         const float *x, float *out, int64_t M, int64_t F) {
    int T = orc_num_threads();
    int64_t *split = (int64_t *)malloc(sizeof(int64_t) * (size_t)(T + 1));
    nnz_balanced_split(rowptr, M, T, split);
#pragma omp parallel num_threads(T)
    {
#ifdef _OPENMP
        int t = omp_get_thread_num();
#else
        int t = 0;
#endif
        for (int64_t m = split[t]; m < split[t + 1]; m++) {
            int64_t b = rowptr[m], e = rowptr[m + 1];
            if (e <= b) continue;
            float *o = out + m * F;
            for (int64_t f0 = 0; f0 < F; f0 += 64) {
                int64_t w = F - f0 < 64 ? F - f0 : 64;
                float acc[64];
                for (int64_t f = 0; f < w; f++) acc[f] = o[f0 + f];
                for (int64_t j = b; j < e; j++) {
                    const float a = val[j];
                    const float *xr = x + col[j] * F + f0;
                    for (int64_t f = 0; f < w; f++) acc[f] = fmaf(a, xr[f], acc[f]);
                }
                for (int64_t f = 0; f < w; f++) o[f0 + f] = acc[f];
            }
        }
    }
    free(split);
}

/* ------------------------------------------------------------------------------------------
 * out[m,:] = sum_e val[e] * x[col[e],:]  for EVERY row (empty rows become 0).
 *
 * Follows spmm_cpu (super_gnn/ops/csrc/spmm.cpp:177-271) with Reducer<float,SUM>
 * (super_gnn/ops/csrc/reducer.h:43-84): accumulator starts at 0 (reducer.h:44-52), each edge adds
 * the rounded product val*x (spmm.cpp:245-246, reducer.h:57-58), result is written, not
 * accumulated (reducer.h:70-74).  val may be NULL (spmm.cpp:247-249: plain sum of rows).
 * Whether a compiler contracts "acc + a*b" into an FMA there is build dependent; this
 * restatement keeps the source's two roundings.
 * ---------------------------------------------------------------------------------------- */
void orc_spmm_overwrite(const int64_t *rowptr, const int64_t *col, const float *val,
                        const float *x, float *out, int64_t M, int64_t F) {
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t m = 0; m < M; m++) {
        float *o = out + m * F;
        for (int64_t f = 0; f < F; f++) o[f] = 0.0f;
        for (int64_t j = rowptr[m]; j < rowptr[m + 1]; j++) {
            const float *xr = x + col[j] * F;
            if (val) {
                const float a = val[j];
                for (int64_t f = 0; f < F; f++) {
                    float p = a * xr[f];
                    o[f] = o[f] + p;
                }
            } else {
                for (int64_t f = 0; f < F; f++) o[f] = o[f] + xr[f];
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * The dispatch rule of spmm() (super_gnn/ops/csrc/spmm.cpp:594-608): the generic overwrite
 * kernel is taken iff  float(nnz)/M/K <= 1e-4  and  F > 256 ; otherwise the accumulate kernel.
 * Returns 1 when the overwrite branch is the one the reference would take.
 * ---------------------------------------------------------------------------------------- */
int orc_spmm_takes_overwrite_branch(int64_t nnz, int64_t M, int64_t K, int64_t F) {
    float sparsity = (float)nnz / (float)M / (float)K;
    return (sparsity <= 0.0001f && F > 256) ? 1 : 0;
}

void orc_spmm_dispatch(const int64_t *rowptr, const int64_t *col, const float *val,
                       const float *x, float *out, int64_t M, int64_t K, int64_t F) {
    int64_t nnz = rowptr[M];
    if (orc_spmm_takes_overwrite_branch(nnz, M, K, F))
        orc_spmm_overwrite(rowptr, col, val, x, out, M, F);
    else
        orc_spmm_accumulate(rowptr, col, val, x, out, M, F);
}

/* fp64 accumulation of the same sum (no reference counterpart): the adjudicator for rows so
 * long that the reference's own sequential fp32 rounding error nears the comparison tolerance. */
void orc_spmm_f64(const int64_t *rowptr, const int64_t *col, const float *val, const float *x,
                  const float *out_init, double *out, int64_t M, int64_t F) {
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t m = 0; m < M; m++) {
        double *o = out + m * F;
        for (int64_t f = 0; f < F; f++) o[f] = out_init ? (double)out_init[m * F + f] : 0.0;
        for (int64_t j = rowptr[m]; j < rowptr[m + 1]; j++) {
            const double a = val ? (double)val[j] : 1.0;
            const float *xr = x + col[j] * F;
            for (int64_t f = 0; f < F; f++) o[f] += a * (double)xr[f];
        }
    }
}

/* mean epilogue: out[m,:] /= deg[m]  (super_gnn/layers/sageconv.py:78, true division). */
void orc_row_divide(float *out, const float *deg, int64_t M, int64_t F) {
#pragma omp parallel for
    for (int64_t m = 0; m < M; m++)
        for (int64_t f = 0; f < F; f++) out[m * F + f] = out[m * F + f] / deg[m];
}

/* ------------------------------------------------------------------------------------------
 * Per-row quantization parameters.
 * Follows quantize_tensor_kernel (super_gnn/ops/csrc/quantization_arm.cpp:93-113 and again
 * :262-279): min and max by sequential STRICT compares starting from element 0 (first
 * occurrence wins among compare-equal values such as -0/+0; a NaN is sticky only as element 0),
 * zero_point = min, scale = (max - min) / float(2^bits - 1), scale == 0 -> 1.
 * ---------------------------------------------------------------------------------------- */
static void row_params(const float *row, int64_t F, int bits, float *zp, float *scale) {
    float mx = row[0], mn = row[0];
    for (int64_t k = 1; k < F; k++) {
        float v = row[k];
        if (v > mx) mx = v;
        if (v < mn) mn = v;
    }
    float s = (mx - mn) / (float)((1 << bits) - 1);
    if (s == 0) s = 1.0f;
    *zp = mn;
    *scale = s;
}

/* code = RNE((x - zp) / scale) with IEEE subtraction and division: the form of the remainder
 * path (quantization_arm.cpp:293), of the x86 build (quantization_x86.cpp:73,93) and of both
 * v1 builds (quantization_arm.cpp:693).  The SVE full-group path multiplies by a reciprocal
 * ESTIMATE (quantization_arm.cpp:157-165) that only exists on A64FX and is not restated. */
static inline uint32_t code_of(float x, float zp, float scale) {
    float q = (x - zp) / scale;
    float r = nearbyintf(q); /* default rounding mode = to nearest even */
    if (!(r >= 0.0f)) return 0u; /* NaN or negative: svcvt_u32_f32 saturates to 0 */
    if (r > 4294967040.0f) return 0xFFFFFFFFu;
    return (uint32_t)r;
}

/* ------------------------------------------------------------------------------------------
 * Row-group quantize + pack over P independent segments.
 *
 * Layout (quantize_tensor_for_all_procs, quantization_arm.cpp:496-578, with divide_work_v1
 * :21-77 and quantize_tensor_kernel :79-301): segment p = rows [seg[p], seg[p+1]); its packed
 * rows start at  sum_{q<p} ceil(n_q / EPB)  and every segment's grouping restarts at its own
 * first row.  Packed row g of a segment holds rows g*EPB+k, k = 0..EPB-1, first row in the most
 * significant bits:  byte[g,j] = OR_k code[g*EPB+k, j] << ((EPB-1-k)*bits)
 * (quantization_arm.cpp:177-185, :217-221, :249, :294-295).  A short last group leaves its low
 * bits zero (:288-298).  params[i] = (zero_point, scale) (:112-113).
 * P = 1 with seg = {0, n} is quantize_tensor (quantization_arm.cpp:433-464) with `bits`
 * honoured (the ARM build hard-codes 2 there, :447-448; the x86 build honours it,
 * quantization_x86.cpp:33).
 * ---------------------------------------------------------------------------------------- */
void orc_quant_rows(const float *x, uint8_t *q, float *params, const int32_t *seg, int P,
                    int64_t F, int bits) {
    const int EPB = 8 / bits;
    int64_t *pbase = (int64_t *)malloc(sizeof(int64_t) * (size_t)(P + 1));
    pbase[0] = 0;
    for (int p = 0; p < P; p++) pbase[p + 1] = pbase[p] + (seg[p + 1] - seg[p] + EPB - 1) / EPB;
    for (int p = 0; p < P; p++) {
        const int64_t r0 = seg[p], n = seg[p + 1] - seg[p];
        const int64_t ng = (n + EPB - 1) / EPB;
#pragma omp parallel for schedule(static)
        for (int64_t g = 0; g < ng; g++) {
            uint8_t *qo = q + (pbase[p] + g) * F;
            memset(qo, 0, (size_t)F);
            for (int k = 0; k < EPB; k++) {
                int64_t i = g * EPB + k;
                if (i >= n) break;
                const float *row = x + (r0 + i) * F;
                float zp, sc;
                row_params(row, F, bits, &zp, &sc);
                params[(r0 + i) * 2 + 0] = zp;
                params[(r0 + i) * 2 + 1] = sc;
                const int sh = (EPB - 1 - k) * bits;
                for (int64_t j = 0; j < F; j++)
                    qo[j] = (uint8_t)(qo[j] | (uint8_t)(code_of(row[j], zp, sc) << sh));
            }
        }
    }
    free(pbase);
}

/* Same packing with caller-supplied min/scale per row: the x86 build's 5-argument
 * quantize_tensor (super_gnn/ops/csrc/quantization_x86.cpp:17-103).  Single segment. */
void orc_quant_rows_given_params(const float *x, uint8_t *q, const float *mn, const float *sc,
                                 int64_t n, int64_t F, int bits) {
    const int EPB = 8 / bits;
    const int64_t ng = (n + EPB - 1) / EPB;
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < ng; g++) {
        uint8_t *qo = q + g * F;
        memset(qo, 0, (size_t)F);
        for (int k = 0; k < EPB; k++) {
            int64_t i = g * EPB + k;
            if (i >= n) break;
            const int sh = (EPB - 1 - k) * bits;
            for (int64_t j = 0; j < F; j++)
                qo[j] = (uint8_t)(qo[j] | (uint8_t)(code_of(x[i * F + j], mn[i], sc[i]) << sh));
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Unpack + dequantize, the inverse layout walk.
 * Follows dequantize_tensor_kernel (quantization_arm.cpp:303-431): code = (byte >> ((EPB-1-k)*
 * bits)) & (2^bits-1) (:323-331, :416-417), value = fma(float(code), scale, zero_point)
 * (:349-352, :425); only rows inside the segment are written (:406-429).
 * ---------------------------------------------------------------------------------------- */
void orc_dequant_rows(const uint8_t *q, float *x, const float *params, const int32_t *seg, int P,
                      int64_t F, int bits) {
    const int EPB = 8 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    int64_t pbase = 0;
    for (int p = 0; p < P; p++) {
        const int64_t r0 = seg[p], n = seg[p + 1] - seg[p];
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n; i++) {
            const uint8_t *qi = q + (pbase + i / EPB) * F;
            const int sh = (EPB - 1 - (int)(i % EPB)) * bits;
            const float zp = params[(r0 + i) * 2], sc = params[(r0 + i) * 2 + 1];
            float *o = x + (r0 + i) * F;
            for (int64_t j = 0; j < F; j++) o[j] = fmaf((float)((qi[j] >> sh) & mask), sc, zp);
        }
        pbase += (n + EPB - 1) / EPB;
    }
}

/* ------------------------------------------------------------------------------------------
 * Feature-packed mixed-bit quantization ("v1").
 * Follows quantize_tensor_v1 (super_gnn/ops/csrc/quantization_arm.cpp:635-702; x86 twin
 * quantization_x86.cpp:170-246): per row i, bits b = int(params[i,0]); min/max as above;
 * params[i,1] = zero_point, params[i,2] = scale (:682-683); byte t of row i =
 * OR_k lrintf((x[i, t*epb+k] - zp)/scale) << ((epb-1-k)*b) for the features that exist
 * (:686-699); row i's bytes start at range[i].
 * ---------------------------------------------------------------------------------------- */
void orc_quant_v1(const float *x, uint8_t *q, const int64_t *range, float *params, int64_t n,
                  int64_t F) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const int b = (int)params[i * 3];
        const float *row = x + i * F;
        float zp, sc;
        row_params(row, F, b, &zp, &sc);
        params[i * 3 + 1] = zp;
        params[i * 3 + 2] = sc;
        const int epb = 8 / b;
        uint8_t *qo = q + range[i];
        for (int64_t j = 0; j < F; j += epb) {
            int rem = (int)(F - j < epb ? F - j : epb);
            uint8_t pk = 0;
            for (int k = 0; k < rem; k++)
                pk = (uint8_t)(pk | (uint8_t)(code_of(row[j + k], zp, sc) << ((epb - 1 - k) * b)));
            qo[j / epb] = pk;
        }
    }
}

/* Follows dequantize_tensor_v1 (quantization_arm.cpp:704-757): value = code*scale + zero_point
 * written as mul then add in the source (:747); the x86 build compiles that line with
 * contraction allowed, so the comparison tolerance for dequantized floats is rel 1e-6, never
 * bit-exact.  Stops at F (:744). */
void orc_dequant_v1(const uint8_t *q, float *x, const int64_t *range, const float *params,
                    int64_t n, int64_t F) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const int b = (int)params[i * 3];
        const float zp = params[i * 3 + 1], sc = params[i * 3 + 2];
        const int epb = 8 / b;
        const uint32_t mask = (1u << b) - 1u;
        const int64_t len = range[i + 1] - range[i];
        for (int64_t j = 0; j < len; j++) {
            const uint8_t pk = q[range[i] + j];
            for (int k = 0; k < epb && j * epb + k < F; k++) {
                float c = (float)((pk >> ((epb - 1 - k) * b)) & mask);
                float prod = c * sc;
                x[i * F + j * epb + k] = prod + zp;
            }
        }
    }
}
