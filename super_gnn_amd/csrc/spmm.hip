// CSR SpMM neighbour aggregation for gfx950:  out (+)= A * X, fp32.
//
// Replaces supergnn_ops.spmm (super_gnn/ops/csrc/spmm.cpp:594-608 of the reference) and the two
// kernels it dispatches to (accumulate: spmm.cpp:348-539; overwrite: spmm.cpp:177-271).
//
// The work is a random gather of dense rows, bound by memory bandwidth and latency; there is no
// MFMA here.  Scheduling is by row class:
//   * short rows (degree <= threshold): one group of G lanes owns one row.  G*VEC*NV floats cover
//     the feature axis (F=128: 32 lanes x float4, two rows per wavefront).  The group fetches its
//     (col,val) pairs G at a time with one coalesced load and broadcasts them lane by lane, so
//     every gather instruction moves whole 128-bit pieces of one dense row and U rows are in
//     flight per group.  Edges are summed in CSR order with one fma per edge, starting from the
//     old out value: the same operation sequence as the reference's kernel_1xN (spmm.cpp:87-162).
//   * long rows (power-law hubs): the edge list is cut into segments; one workgroup per segment,
//     its lane groups take contiguous sub-ranges, partial sums are combined through LDS in a
//     fixed order and written to a partial buffer; a last small kernel adds a row's partials in
//     segment order.  No float atomics: results are reproducible run to run.
#include <algorithm>
#include <vector>

#include "common.hpp"

namespace sgnn {

constexpr int kBlock = 256;
constexpr int kDefaultLongThreshold = 512;
constexpr int kDefaultSegmentEdges = 512;

__host__ __device__ constexpr int unroll_of(int nv) { return nv == 1 ? 8 : nv == 2 ? 4 : nv == 3 ? 3 : 2; }

template <int G>
__device__ __forceinline__ int group_bcast_i(int v, int src) {
    if constexpr (G == 64) {
        return __builtin_amdgcn_readlane(v, src);
    } else {
        return __shfl(v, src, G);
    }
}
template <int G>
__device__ __forceinline__ float group_bcast_f(float v, int src) {
    return __int_as_float(group_bcast_i<G>(__float_as_int(v), src));
}

__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Accumulate `deg` edges starting at colp/valp into acc for one feature tile.
template <int VEC, int G, int NV>
__device__ __forceinline__ void gather_edges(float (&acc)[NV][VEC], const int32_t *__restrict__ colp,
                                             const float *__restrict__ valp, int deg,
                                             const float *__restrict__ x, int64_t ldx, const int (&off)[NV],
                                             const bool (&act)[NV], int lig) {
    constexpr int U = unroll_of(NV);
    for (int base = 0; base < deg; base += G) {
        const int idx = base + lig;
        int myc = 0;
        float myw = 0.0f;
        if (idx < deg) {
            myc = __builtin_nontemporal_load(colp + idx);
            myw = valp ? __builtin_nontemporal_load(valp + idx) : 1.0f;
        }
        const int cnt = deg - base < G ? deg - base : G;
        int j = 0;
        for (; j + U <= cnt; j += U) {
            float xv[U][NV][VEC];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = group_bcast_i<G>(myc, j + u);
                const float *xr = x + (int64_t)c * ldx;
#pragma unroll
                for (int v = 0; v < NV; ++v)
                    if (act[v]) vec_load<VEC>(xv[u][v], xr + off[v]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float w = group_bcast_f<G>(myw, j + u);
#pragma unroll
                for (int v = 0; v < NV; ++v)
#pragma unroll
                    for (int k = 0; k < VEC; ++k) acc[v][k] = fmaf(w, xv[u][v][k], acc[v][k]);
            }
        }
        for (; j < cnt; ++j) {
            const int c = group_bcast_i<G>(myc, j);
            const float w = group_bcast_f<G>(myw, j);
            const float *xr = x + (int64_t)c * ldx;
            float xv[NV][VEC];
#pragma unroll
            for (int v = 0; v < NV; ++v)
                if (act[v]) vec_load<VEC>(xv[v], xr + off[v]);
#pragma unroll
            for (int v = 0; v < NV; ++v)
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[v][k] = fmaf(w, xv[v][k], acc[v][k]);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Short rows: one lane group per row.
// ------------------------------------------------------------------------------------------------
template <int VEC, int G, int NV>
__global__ __launch_bounds__(kBlock) void spmm_short_kernel(
    const int64_t *__restrict__ rowptr, const int32_t *__restrict__ col, const float *__restrict__ val,
    const float *__restrict__ x, float *__restrict__ out, int64_t M, int F, int64_t ldx, int64_t ldo,
    int accumulate, const float *__restrict__ row_div, int long_thresh, uint32_t nblocks) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    const uint32_t lb = xcd_contiguous_block(blockIdx.x, nblocks);
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    int64_t row = (int64_t)lb * GPB + gid;
    if (row >= M) return;
    int64_t b = rowptr[row], e = rowptr[row + 1];
    if constexpr (G == 64) {
        row = uniform64(row);
        b = uniform64(b);
        e = uniform64(e);
    }
    if (e - b > (int64_t)long_thresh) return;  // handled by the segment kernels
    const int deg = (int)(e - b);
    if (deg == 0 && accumulate && row_div == nullptr) return;  // reference skips empty rows
    const int32_t *colp = col + b;
    const float *valp = val ? val + b : nullptr;
    float *orow = out + row * ldo;
    float div = 1.0f;
    if (row_div) div = row_div[row];

    for (int f0 = 0; f0 < F; f0 += TILE) {
        int off[NV];
        bool act[NV];
        float acc[NV][VEC];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            off[v] = f0 + (v * G + lig) * VEC;
            act[v] = off[v] < F;
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[v][k] = 0.0f;
            if (accumulate && act[v]) vec_load_nt<VEC>(acc[v], orow + off[v]);
        }
        gather_edges<VEC, G, NV>(acc, colp, valp, deg, x, ldx, off, act, lig);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
            if (row_div) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[v][k] = acc[v][k] / div;
            }
            vec_store_nt<VEC>(orow + off[v], acc[v]);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Long rows, step 1: one workgroup per edge segment -> partial[s, :].
// ------------------------------------------------------------------------------------------------
template <int VEC, int G, int NV>
__global__ __launch_bounds__(kBlock) void spmm_segment_kernel(
    const int32_t *__restrict__ col, const float *__restrict__ val, const float *__restrict__ x,
    float *__restrict__ partial, const int64_t *__restrict__ seg_begin, const int32_t *__restrict__ seg_len,
    int F, int64_t ldx) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    __shared__ float red[GPB][TILE];
    const int s = blockIdx.x;
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int64_t b = uniform64(seg_begin[s]);
    const int len = __builtin_amdgcn_readfirstlane(seg_len[s]);
    const int per = (len + GPB - 1) / GPB;
    int my_b = gid * per;
    int my_e = my_b + per < len ? my_b + per : len;
    if constexpr (G == 64) {
        my_b = __builtin_amdgcn_readfirstlane(my_b);
        my_e = __builtin_amdgcn_readfirstlane(my_e);
    }
    const int my_deg = my_e > my_b ? my_e - my_b : 0;
    const int32_t *colp = col + b + my_b;
    const float *valp = val ? val + b + my_b : nullptr;

    for (int f0 = 0; f0 < F; f0 += TILE) {
        int off[NV];
        bool act[NV];
        float acc[NV][VEC];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            off[v] = f0 + (v * G + lig) * VEC;
            act[v] = off[v] < F;
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[v][k] = 0.0f;
        }
        gather_edges<VEC, G, NV>(acc, colp, valp, my_deg, x, ldx, off, act, lig);
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int k = 0; k < VEC; ++k) red[gid][(v * G + lig) * VEC + k] = acc[v][k];
        __syncthreads();
        const int width = F - f0 < TILE ? F - f0 : TILE;
        for (int i = threadIdx.x; i < width; i += kBlock) {
            float sum = red[0][i];
#pragma unroll
            for (int g = 1; g < GPB; ++g) sum += red[g][i];
            partial[(int64_t)s * F + f0 + i] = sum;
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------------
// Long rows, step 2: add a row's segment partials in segment order, epilogue, store.
// ------------------------------------------------------------------------------------------------
template <int VEC, int G, int NV>
__global__ __launch_bounds__(kBlock) void spmm_long_final_kernel(
    const int32_t *__restrict__ long_rows, const int32_t *__restrict__ long_segptr,
    const float *__restrict__ partial, float *__restrict__ out, int n_long, int F, int64_t ldo,
    int accumulate, const float *__restrict__ row_div) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int li = blockIdx.x * GPB + gid;
    if (li >= n_long) return;
    const int64_t row = long_rows[li];
    const int s0 = long_segptr[li], s1 = long_segptr[li + 1];
    float *orow = out + row * ldo;
    const float div = row_div ? row_div[row] : 1.0f;
    for (int f0 = 0; f0 < F; f0 += TILE) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int off = f0 + (v * G + lig) * VEC;
            if (off >= F) continue;
            float acc[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
            if (accumulate) vec_load_nt<VEC>(acc, orow + off);
            for (int s = s0; s < s1; ++s) {
                float p[VEC];
                vec_load<VEC>(p, partial + (int64_t)s * F + off);
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] += p[k];
            }
            if (row_div) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] = acc[k] / div;
            }
            vec_store_nt<VEC>(orow + off, acc);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Column index narrowing + range check.
// ------------------------------------------------------------------------------------------------
template <typename SrcT>
__global__ __launch_bounds__(kBlock) void narrow_cols_kernel(const SrcT *__restrict__ src, int32_t *__restrict__ dst,
                                                             int64_t n, int64_t K, int *__restrict__ bad) {
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    bool any_bad = false;
    for (; i < n; i += stride) {
        const int64_t c = (int64_t)src[i];
        if (c < 0 || c >= K) any_bad = true;
        dst[i] = (int32_t)c;
    }
    if (any_bad) atomicOr(bad, 1);
}

// ------------------------------------------------------------------------------------------------
// Launch tables.
// ------------------------------------------------------------------------------------------------
struct ShortArgs {
    const int64_t *rowptr; const int32_t *col; const float *val; const float *x; float *out;
    int64_t M; int F; int64_t ldx, ldo; int accumulate; const float *row_div; int long_thresh;
};
struct SegArgs {
    const int32_t *col; const float *val; const float *x; float *partial; const int64_t *seg_begin;
    const int32_t *seg_len; int n_seg; int F; int64_t ldx;
};
struct FinalArgs {
    const int32_t *long_rows; const int32_t *long_segptr; const float *partial; float *out; int n_long;
    int F; int64_t ldo; int accumulate; const float *row_div;
};

template <int VEC, int G, int NV>
static void launch_all(const ShortArgs &a, const SegArgs &s, const FinalArgs &f, hipStream_t st) {
    constexpr int GPB = kBlock / G;
    if (a.M > 0) {
        const uint32_t nb = (uint32_t)((a.M + GPB - 1) / GPB);
        ProfScope prof(K_SPMM_SHORT, st);
        hipLaunchKernelGGL((spmm_short_kernel<VEC, G, NV>), dim3(nb), dim3(kBlock), 0, st, a.rowptr, a.col, a.val, a.x,
                           a.out, a.M, a.F, a.ldx, a.ldo, a.accumulate, a.row_div, a.long_thresh, nb);
    }
    if (s.n_seg > 0) {
        {
            ProfScope prof(K_SPMM_SEGMENT, st);
            hipLaunchKernelGGL((spmm_segment_kernel<VEC, G, NV>), dim3(s.n_seg), dim3(kBlock), 0, st, s.col, s.val,
                               s.x, s.partial, s.seg_begin, s.seg_len, s.F, s.ldx);
        }
        const uint32_t nb = (uint32_t)((f.n_long + GPB - 1) / GPB);
        ProfScope prof(K_SPMM_LONG_FINAL, st);
        hipLaunchKernelGGL((spmm_long_final_kernel<VEC, G, NV>), dim3(nb), dim3(kBlock), 0, st, f.long_rows,
                           f.long_segptr, f.partial, f.out, f.n_long, f.F, f.ldo, f.accumulate, f.row_div);
    }
}

template <int VEC>
static int dispatch_shape(int nvec, const ShortArgs &a, const SegArgs &s, const FinalArgs &f, hipStream_t st) {
    if (nvec <= 8) launch_all<VEC, 8, 1>(a, s, f, st);
    else if (nvec <= 16) launch_all<VEC, 16, 1>(a, s, f, st);
    else if (nvec <= 32) launch_all<VEC, 32, 1>(a, s, f, st);
    else if (nvec <= 64) launch_all<VEC, 64, 1>(a, s, f, st);
    else if (nvec <= 128) launch_all<VEC, 64, 2>(a, s, f, st);
    else if (nvec <= 192) launch_all<VEC, 64, 3>(a, s, f, st);
    else if (nvec <= 256) launch_all<VEC, 64, 4>(a, s, f, st);
    else if (nvec <= 320) launch_all<VEC, 64, 5>(a, s, f, st);
    else if (nvec <= 384) launch_all<VEC, 64, 6>(a, s, f, st);
    else launch_all<VEC, 64, 8>(a, s, f, st);  // feature axis walked in tiles of 512 vectors
    return SGNN_OK;
}

}  // namespace sgnn

using namespace sgnn;

struct sgnn_spmm_plan {
    int device = 0;
    int64_t M = 0, K = 0, nnz = 0;
    int long_thresh = 0, seg_edges = 0;
    int64_t *rowptr = nullptr;  // device, owned
    int32_t *col = nullptr;     // device, owned
    int64_t n_long = 0, n_seg = 0, long_edges = 0;
    int32_t *long_rows = nullptr;    // [n_long]
    int32_t *long_segptr = nullptr;  // [n_long + 1]
    int64_t *seg_begin = nullptr;    // [n_seg]
    int32_t *seg_len = nullptr;      // [n_seg]
    float *partial = nullptr;        // [n_seg * F], grown on demand
    size_t partial_floats = 0;
};

extern "C" int sgnn_spmm_plan_destroy(sgnn_spmm_plan *p) {
    if (!p) return SGNN_OK;
    (void)hipFree(p->rowptr);
    (void)hipFree(p->col);
    (void)hipFree(p->long_rows);
    (void)hipFree(p->long_segptr);
    (void)hipFree(p->seg_begin);
    (void)hipFree(p->seg_len);
    (void)hipFree(p->partial);
    delete p;
    return SGNN_OK;
}

static int plan_create_impl(sgnn_spmm_plan *p, const int64_t *rowptr, const void *col, int col_is_i64,
                            int long_row_threshold, int segment_edges, hipStream_t st) {
    const int64_t M = p->M, K = p->K, nnz = p->nnz;
    SGNN_HIP_CHECK(hipGetDevice(&p->device));
    p->long_thresh = long_row_threshold > 0 ? long_row_threshold : kDefaultLongThreshold;
    p->seg_edges = segment_edges > 0 ? segment_edges : kDefaultSegmentEdges;

    std::vector<int64_t> h_rowptr((size_t)M + 1);
    SGNN_HIP_CHECK(hipMemcpyAsync(h_rowptr.data(), rowptr, sizeof(int64_t) * (size_t)(M + 1), hipMemcpyDeviceToHost, st));
    SGNN_HIP_CHECK(hipStreamSynchronize(st));
    if (h_rowptr[0] != 0) return fail(SGNN_ERR_RANGE, "rowptr[0] = %lld, expected 0", (long long)h_rowptr[0]);
    for (int64_t m = 0; m < M; ++m)
        if (h_rowptr[m + 1] < h_rowptr[m]) return fail(SGNN_ERR_RANGE, "rowptr decreases at row %lld", (long long)m);
    if (h_rowptr[M] != nnz)
        return fail(SGNN_ERR_RANGE, "rowptr[M] = %lld but nnz = %lld", (long long)h_rowptr[M], (long long)nnz);

    std::vector<int32_t> long_rows, long_segptr, seg_len;
    std::vector<int64_t> seg_begin;
    long_segptr.push_back(0);
    for (int64_t m = 0; m < M; ++m) {
        const int64_t b = h_rowptr[m], deg = h_rowptr[m + 1] - b;
        if (deg <= p->long_thresh) continue;
        long_rows.push_back((int32_t)m);
        for (int64_t o = 0; o < deg; o += p->seg_edges) {
            seg_begin.push_back(b + o);
            seg_len.push_back((int32_t)std::min<int64_t>(p->seg_edges, deg - o));
        }
        if (seg_begin.size() > (size_t)INT32_MAX) return fail(SGNN_ERR_ARG, "too many long-row segments");
        long_segptr.push_back((int32_t)seg_begin.size());
        p->long_edges += deg;
    }
    p->n_long = (int64_t)long_rows.size();
    p->n_seg = (int64_t)seg_begin.size();

    SGNN_HIP_CHECK(hipMalloc(&p->rowptr, sizeof(int64_t) * (size_t)(M + 1)));
    SGNN_HIP_CHECK(hipMemcpyAsync(p->rowptr, rowptr, sizeof(int64_t) * (size_t)(M + 1), hipMemcpyDeviceToDevice, st));
    SGNN_HIP_CHECK(hipMalloc(&p->col, sizeof(int32_t) * (size_t)std::max<int64_t>(nnz, 1)));
    if (nnz > 0) {
        int *bad = nullptr;
        SGNN_HIP_CHECK(hipMalloc(&bad, sizeof(int)));
        SGNN_HIP_CHECK(hipMemsetAsync(bad, 0, sizeof(int), st));
        const int nb = (int)std::min<int64_t>((nnz + kBlock - 1) / kBlock, 65536);
        if (col_is_i64)
            hipLaunchKernelGGL((narrow_cols_kernel<int64_t>), dim3(nb), dim3(kBlock), 0, st, (const int64_t *)col, p->col, nnz, K, bad);
        else
            hipLaunchKernelGGL((narrow_cols_kernel<int32_t>), dim3(nb), dim3(kBlock), 0, st, (const int32_t *)col, p->col, nnz, K, bad);
        int h_bad = 0;
        hipError_t e1 = hipGetLastError();
        hipError_t e2 = hipMemcpyAsync(&h_bad, bad, sizeof(int), hipMemcpyDeviceToHost, st);
        hipError_t e3 = hipStreamSynchronize(st);
        (void)hipFree(bad);
        SGNN_HIP_CHECK(e1);
        SGNN_HIP_CHECK(e2);
        SGNN_HIP_CHECK(e3);
        if (h_bad) return fail(SGNN_ERR_RANGE, "a column index lies outside [0, %lld)", (long long)K);
    }
    if (p->n_long > 0) {
        SGNN_HIP_CHECK(hipMalloc(&p->long_rows, sizeof(int32_t) * long_rows.size()));
        SGNN_HIP_CHECK(hipMalloc(&p->long_segptr, sizeof(int32_t) * long_segptr.size()));
        SGNN_HIP_CHECK(hipMalloc(&p->seg_begin, sizeof(int64_t) * seg_begin.size()));
        SGNN_HIP_CHECK(hipMalloc(&p->seg_len, sizeof(int32_t) * seg_len.size()));
        SGNN_HIP_CHECK(hipMemcpyAsync(p->long_rows, long_rows.data(), sizeof(int32_t) * long_rows.size(), hipMemcpyHostToDevice, st));
        SGNN_HIP_CHECK(hipMemcpyAsync(p->long_segptr, long_segptr.data(), sizeof(int32_t) * long_segptr.size(), hipMemcpyHostToDevice, st));
        SGNN_HIP_CHECK(hipMemcpyAsync(p->seg_begin, seg_begin.data(), sizeof(int64_t) * seg_begin.size(), hipMemcpyHostToDevice, st));
        SGNN_HIP_CHECK(hipMemcpyAsync(p->seg_len, seg_len.data(), sizeof(int32_t) * seg_len.size(), hipMemcpyHostToDevice, st));
        SGNN_HIP_CHECK(hipStreamSynchronize(st));  // the host vectors die at return
    }
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_create(const int64_t *rowptr, const void *col, int col_is_i64, int64_t M, int64_t K,
                                     int64_t nnz, int long_row_threshold, int segment_edges, sgnn_stream_t stream,
                                     sgnn_spmm_plan **plan_out) {
    SGNN_REQUIRE(plan_out != nullptr, "plan_out is null");
    *plan_out = nullptr;
    SGNN_REQUIRE(rowptr != nullptr, "rowptr is null");
    SGNN_REQUIRE(M >= 0 && K >= 0 && nnz >= 0, "negative size (M=%lld K=%lld nnz=%lld)", (long long)M, (long long)K, (long long)nnz);
    SGNN_REQUIRE(M < INT32_MAX && K < INT32_MAX, "M and K must fit 31 bits (M=%lld K=%lld)", (long long)M, (long long)K);
    SGNN_REQUIRE(nnz == 0 || col != nullptr, "col is null with nnz=%lld", (long long)nnz);
    sgnn_spmm_plan *p = new sgnn_spmm_plan();
    p->M = M; p->K = K; p->nnz = nnz;
    const int rc = plan_create_impl(p, rowptr, col, col_is_i64, long_row_threshold, segment_edges, (hipStream_t)stream);
    if (rc != SGNN_OK) {
        sgnn_spmm_plan_destroy(p);
        return rc;
    }
    *plan_out = p;
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_info(const sgnn_spmm_plan *p, int64_t info[8]) {
    SGNN_REQUIRE(p != nullptr && info != nullptr, "null argument");
    info[0] = p->M; info[1] = p->K; info[2] = p->nnz; info[3] = p->n_long; info[4] = p->n_seg;
    info[5] = p->long_edges; info[6] = p->long_thresh; info[7] = p->seg_edges;
    return SGNN_OK;
}

extern "C" int sgnn_spmm_reference_overwrites(int64_t nnz, int64_t M, int64_t K, int64_t F) {
    if (M <= 0 || K <= 0) return 0;
    const float sparsity = (float)nnz / (float)M / (float)K;
    return (sparsity <= 0.0001f && F > 256) ? 1 : 0;
}

extern "C" int sgnn_spmm_csr_f32(sgnn_spmm_plan *p, const float *val, const float *x, float *out, int64_t F,
                                 int64_t ldx, int64_t ldo, int accumulate, const float *row_div,
                                 sgnn_stream_t stream) {
    SGNN_REQUIRE(p != nullptr, "plan is null");
    SGNN_REQUIRE(F > 0 && F < (1 << 24), "feature width F=%lld out of range", (long long)F);
    SGNN_REQUIRE(ldx >= F && ldo >= F, "leading dimension smaller than F (ldx=%lld ldo=%lld F=%lld)", (long long)ldx, (long long)ldo, (long long)F);
    if (p->M == 0) return SGNN_OK;
    SGNN_REQUIRE(out != nullptr, "out is null");
    SGNN_REQUIRE(x != nullptr || p->nnz == 0, "x is null");
    hipStream_t st = (hipStream_t)stream;
    int dev = 0;
    SGNN_HIP_CHECK(hipGetDevice(&dev));
    SGNN_REQUIRE(dev == p->device, "plan was created on device %d, current device is %d", p->device, dev);

    if (p->n_seg > 0) {
        const size_t need = (size_t)p->n_seg * (size_t)F;
        if (need > p->partial_floats) {
            // The old buffer may still be read by work queued on another stream: drain first.
            SGNN_HIP_CHECK(hipDeviceSynchronize());
            (void)hipFree(p->partial);
            p->partial = nullptr;
            p->partial_floats = 0;
            SGNN_HIP_CHECK(hipMalloc(&p->partial, need * sizeof(float)));
            p->partial_floats = need;
        }
    }
    int vec = 1;
    if (F % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 && aligned(x, 16) && aligned(out, 16)) vec = 4;
    else if (F % 2 == 0 && ldx % 2 == 0 && ldo % 2 == 0 && aligned(x, 8) && aligned(out, 8)) vec = 2;
    const int nvec = (int)(F / vec);
    ShortArgs a{p->rowptr, p->col, val, x, out, p->M, (int)F, ldx, ldo, accumulate, row_div, p->long_thresh};
    SegArgs s{p->col, val, x, p->partial, p->seg_begin, p->seg_len, (int)p->n_seg, (int)F, ldx};
    FinalArgs f{p->long_rows, p->long_segptr, p->partial, out, (int)p->n_long, (int)F, ldo, accumulate, row_div};
    if (vec == 4) dispatch_shape<4>(nvec, a, s, f, st);
    else if (vec == 2) dispatch_shape<2>(nvec, a, s, f, st);
    else dispatch_shape<1>(nvec, a, s, f, st);
    SGNN_HIP_CHECK(hipGetLastError());
    return SGNN_OK;
}
