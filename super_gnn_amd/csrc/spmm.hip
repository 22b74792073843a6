// CSR SpMM neighbour aggregation for gfx950:  out (+)= A * X, fp32.
//
// Replaces supergnn_ops.spmm (super_gnn/ops/csrc/spmm.cpp:594-608 of the reference) and the two
// kernels it dispatches to (accumulate: spmm.cpp:348-539; overwrite: spmm.cpp:177-271).
//
// The work is a random gather of dense rows, bound by memory bandwidth and latency; there is no
// MFMA here.  Scheduling is by row class:
//   * short rows (degree <= threshold): consecutive rows are cut into chunks of ~128 edges; one
//     group of G lanes owns one chunk.  G*VEC*NV floats cover the feature axis (F=128: 32 lanes x
//     float4, two chunks per wavefront).  Because the edges of consecutive CSR rows are contiguous,
//     the group streams the chunk's (col,val) pairs G at a time with one coalesced load, broadcasts
//     them lane by lane and keeps U whole-row gathers in flight regardless of where rows begin
//     and end; a row boundary only switches the accumulator (store the finished row, continue with
//     the next one, whose old value was prefetched).  Edges are summed in CSR order with one fma
//     per edge, starting from the old out value: the same operation sequence as the reference's
//     kernel_1xN (spmm.cpp:87-162), so these rows are bit-identical to the reference.
//   * long rows (power-law hubs): the edge list is cut into segments; one workgroup per segment,
//     its lane groups take contiguous sub-ranges, partial sums are combined through LDS in a
//     fixed order and written to a partial buffer; a last small kernel adds a row's partials in
//     segment order.  No float atomics: results are reproducible run to run.
#include <algorithm>
#include <cstdlib>
#include <functional>
#include <vector>

#include "common.hpp"

namespace sgnn {

constexpr int kBlock = 256;
constexpr int kDefaultLongThreshold = 128;
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
template <int VEC, int G, int NV, bool FLAVOURS>
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
                const int cf = group_bcast_i<G>(myc, j + u);
                const float *xr = x + (int64_t)(cf & 0x7fffffff) * ldx;
                if (FLAVOURS && cf < 0) {
#pragma unroll
                    for (int v = 0; v < NV; ++v)
                        if (act[v]) vec_load_nt<VEC>(xv[u][v], xr + off[v]);
                } else {
#pragma unroll
                    for (int v = 0; v < NV; ++v)
                        if (act[v]) vec_load<VEC>(xv[u][v], xr + off[v]);
                }
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
            const int cf = group_bcast_i<G>(myc, j);
            const float w = group_bcast_f<G>(myw, j);
            const float *xr = x + (int64_t)(cf & 0x7fffffff) * ldx;
            float xv[NV][VEC];
            if (FLAVOURS && cf < 0) {
#pragma unroll
                for (int v = 0; v < NV; ++v)
                    if (act[v]) vec_load_nt<VEC>(xv[v], xr + off[v]);
            } else {
#pragma unroll
                for (int v = 0; v < NV; ++v)
                    if (act[v]) vec_load<VEC>(xv[v], xr + off[v]);
            }
#pragma unroll
            for (int v = 0; v < NV; ++v)
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[v][k] = fmaf(w, xv[v][k], acc[v][k]);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Short rows: one lane group per chunk of consecutive rows.
// ------------------------------------------------------------------------------------------------
template <int G>
__device__ __forceinline__ uint32_t group_ballot(bool pred) {
    const unsigned long long m = __ballot(pred);
    if constexpr (G == 64) {
        return (uint32_t)m;  // only the low 32 lanes carry row flags
    } else {
        const int base = threadIdx.x & 63 & ~(G - 1);
        return (uint32_t)(m >> base) & (G == 32 ? 0xffffffffu : ((1u << G) - 1u));
    }
}

// Rows per chunk: each of the first nr+1 lanes of the group holds one rowptr entry.
__host__ __device__ constexpr int chunk_row_limit(int G) { return (G < 32 ? G : 32) - 1; }

template <int VEC, int G, int NV>
__global__ __launch_bounds__(kBlock) void spmm_short_kernel(
    const int64_t *__restrict__ rowptr, const int32_t *__restrict__ col, const float *__restrict__ val,
    const float *__restrict__ x, float *__restrict__ out, const int2 *__restrict__ chunks, int n_chunks, int F,
    int64_t ldx, int64_t ldo, int accumulate, const float *__restrict__ row_div, uint32_t nblocks) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    constexpr int U = unroll_of(NV);
    const uint32_t lb = xcd_contiguous_block(blockIdx.x, nblocks);
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int ci = (int)lb * GPB + gid;
    if (ci >= n_chunks) return;
    int2 ch = chunks[ci];
    if constexpr (G == 64) {
        ch.x = __builtin_amdgcn_readfirstlane(ch.x);
        ch.y = __builtin_amdgcn_readfirstlane(ch.y);
    }
    const int rb = ch.x, nr = ch.y;  // rows rb .. rb+nr-1, first and last non-empty, 1 <= nr <= limit

    // Lane i holds rowptr[rb+i] relative to the chunk's first edge (lanes >= nr hold the end).
    const int64_t rp = rowptr[rb + (lig < nr ? lig : nr)];
    int64_t B = rp;
    {
        const int lo = group_bcast_i<G>((int)(uint32_t)rp, 0), hi = group_bcast_i<G>((int)(uint32_t)((uint64_t)rp >> 32), 0);
        B = (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo);
    }
    const int rel = (int)(rp - B);
    const int rel_next = __shfl_down(rel, 1, G);
    const uint32_t mask = group_ballot<G>(lig < nr && rel_next > rel);  // bit i: row rb+i has edges
    const int E = group_bcast_i<G>(rel, nr);
    const float mydiv = (row_div && lig < nr) ? row_div[rb + lig] : 1.0f;
    const int32_t *colp = col + B;
    const float *valp = val ? val + B : nullptr;

    for (int f0 = 0; f0 < F; f0 += TILE) {
        int off[NV];
        bool act[NV];
        float acc[NV][VEC], nxt_old[NV][VEC];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            off[v] = f0 + (v * G + lig) * VEC;
            act[v] = off[v] < F;
        }
        int cur = __builtin_ctz(mask);
        int cur_end = group_bcast_i<G>(rel, cur + 1);
        uint32_t rest = mask & ~((2u << cur) - 1u);
        int nxt = rest ? __builtin_ctz(rest) : -1;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                acc[v][k] = 0.0f;
                nxt_old[v][k] = 0.0f;
            }
            if (accumulate && act[v]) {
                vec_load_nt<VEC>(acc[v], out + (int64_t)(rb + cur) * ldo + off[v]);
                if (nxt >= 0) vec_load_nt<VEC>(nxt_old[v], out + (int64_t)(rb + nxt) * ldo + off[v]);
            }
        }

        for (int base = 0; base < E; base += G) {
            const int idx = base + lig;
            int myc = 0;
            float myw = 1.0f;
            if (idx < E) {
                myc = __builtin_nontemporal_load(colp + idx) & 0x7fffffff;
                if (valp) myw = __builtin_nontemporal_load(valp + idx);
            }
            const int cnt = E - base < G ? E - base : G;
            for (int j = 0; j < cnt; j += U) {
                float xv[U][NV][VEC];
                // U gathers back to back.  Past the end of the chunk the last edge's row is
                // fetched again (a cache hit) so that no branch separates the loads.
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int src = j + u < cnt ? j + u : cnt - 1;
                    const int c = group_bcast_i<G>(myc, src);
                    const float *xr = x + (int64_t)c * ldx;
#pragma unroll
                    for (int v = 0; v < NV; ++v)
                        if (act[v]) vec_load<VEC>(xv[u][v], xr + off[v]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (j + u < cnt) {
                        if (base + j + u == cur_end) {
                            // first edge of the next non-empty row: retire the finished one
                            const float div = row_div ? group_bcast_f<G>(mydiv, cur) : 1.0f;
#pragma unroll
                            for (int v = 0; v < NV; ++v) {
                                if (!act[v]) continue;
                                if (row_div) {
#pragma unroll
                                    for (int k = 0; k < VEC; ++k) acc[v][k] = acc[v][k] / div;
                                }
                                vec_store_nt<VEC>(out + (int64_t)(rb + cur) * ldo + off[v], acc[v]);
#pragma unroll
                                for (int k = 0; k < VEC; ++k) acc[v][k] = nxt_old[v][k];
                            }
                            cur = nxt;
                            cur_end = group_bcast_i<G>(rel, cur + 1);
                            rest = mask & ~((2u << cur) - 1u);
                            nxt = rest ? __builtin_ctz(rest) : -1;
                            if (accumulate && nxt >= 0) {
#pragma unroll
                                for (int v = 0; v < NV; ++v)
                                    if (act[v]) vec_load_nt<VEC>(nxt_old[v], out + (int64_t)(rb + nxt) * ldo + off[v]);
                            }
                        }
                        const float w = group_bcast_f<G>(myw, j + u);
#pragma unroll
                        for (int v = 0; v < NV; ++v)
#pragma unroll
                            for (int k = 0; k < VEC; ++k) acc[v][k] = fmaf(w, xv[u][v][k], acc[v][k]);
                    }
                }
            }
        }
        const float div = row_div ? group_bcast_f<G>(mydiv, cur) : 1.0f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
            if (row_div) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[v][k] = acc[v][k] / div;
            }
            vec_store_nt<VEC>(out + (int64_t)(rb + cur) * ldo + off[v], acc[v]);
        }
    }
}

// Rows without edges, only needed when they must be written: overwrite mode (zeros) or the mean
// epilogue (old value / divisor).  One lane group per empty row.
template <int VEC, int G, int NV>
__global__ __launch_bounds__(kBlock) void spmm_empty_rows_kernel(const int32_t *__restrict__ empty_rows, int n_empty,
                                                                 float *__restrict__ out, int F, int64_t ldo,
                                                                 int accumulate, const float *__restrict__ row_div) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int i = blockIdx.x * GPB + gid;
    if (i >= n_empty) return;
    const int64_t row = empty_rows[i];
    const float div = row_div ? row_div[row] : 1.0f;
    for (int f0 = 0; f0 < F; f0 += TILE) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int off = f0 + (v * G + lig) * VEC;
            if (off >= F) continue;
            float a[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) a[k] = 0.0f;
            if (accumulate) vec_load_nt<VEC>(a, out + row * ldo + off);
            if (row_div) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) a[k] = a[k] / div;
            }
            vec_store_nt<VEC>(out + row * ldo + off, a);
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
        gather_edges<VEC, G, NV, true>(acc, colp, valp, my_deg, x, ldx, off, act, lig);
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
                                                             int64_t n, int64_t K, int *__restrict__ bad,
                                                             int *__restrict__ popularity) {
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    bool any_bad = false;
    for (; i < n; i += stride) {
        const int64_t c = (int64_t)src[i];
        if (c < 0 || c >= K) {
            any_bad = true;
        } else if (popularity) {
            atomicAdd(popularity + c, 1);
        }
        dst[i] = (int32_t)c;
    }
    if (any_bad) atomicOr(bad, 1);
}

// Marks the gathers of unpopular dense rows as streaming (sign bit of the stored column index):
// they are fetched with non-temporal loads so that they do not evict the popular rows from L2.
__global__ __launch_bounds__(kBlock) void mark_cold_cols_kernel(int32_t *__restrict__ col, int64_t n,
                                                                const int *__restrict__ popularity, int hot_min) {
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (; i < n; i += stride) {
        const int32_t c = col[i];
        if (popularity[c] < hot_min) col[i] = c | (int32_t)0x80000000;
    }
}

// ------------------------------------------------------------------------------------------------
// Launch tables.
// ------------------------------------------------------------------------------------------------
struct ShortArgs {
    const int64_t *rowptr; const int32_t *col; const float *val; const float *x; float *out;
    const int2 *chunks; int n_chunks; const int32_t *empty_rows; int n_empty;
    int F; int64_t ldx, ldo; int accumulate; const float *row_div;
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
    if (a.n_chunks > 0) {
        const uint32_t nb = (uint32_t)((a.n_chunks + GPB - 1) / GPB);
        ProfScope prof(K_SPMM_SHORT, st);
        hipLaunchKernelGGL((spmm_short_kernel<VEC, G, NV>), dim3(nb), dim3(kBlock), 0, st, a.rowptr, a.col, a.val, a.x,
                           a.out, a.chunks, a.n_chunks, a.F, a.ldx, a.ldo, a.accumulate, a.row_div, nb);
    }
    if (a.n_empty > 0 && (!a.accumulate || a.row_div)) {
        const uint32_t nb = (uint32_t)((a.n_empty + GPB - 1) / GPB);
        ProfScope prof(K_SPMM_EMPTY_ROWS, st);
        hipLaunchKernelGGL((spmm_empty_rows_kernel<VEC, G, NV>), dim3(nb), dim3(kBlock), 0, st, a.empty_rows, a.n_empty,
                           a.out, a.F, a.ldo, a.accumulate, a.row_div);
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

// Lane-group width for a row of nvec vectors (the kernels are instantiated for these shapes).
static int group_width(int nvec) { return nvec <= 8 ? 8 : nvec <= 16 ? 16 : nvec <= 32 ? 32 : 64; }

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

// Number of dense rows treated as "popular" (kept on the normal, cache-retaining load path).
// Everything else is gathered with streaming loads.  0 disables the classification.
static int hot_rows_budget() {
    const char *e = getenv("SGNN_SPMM_HOT_ROWS");
    return e ? atoi(e) : 8192;
}

struct sgnn_spmm_plan {
    int device = 0;
    int64_t M = 0, K = 0, nnz = 0;
    int long_thresh = 0, seg_edges = 0, hot_min = 0;
    int64_t *rowptr = nullptr;  // device, owned
    int32_t *col = nullptr;     // device, owned
    int64_t n_long = 0, n_seg = 0, long_edges = 0;
    int32_t *long_rows = nullptr;    // [n_long]
    int32_t *long_segptr = nullptr;  // [n_long + 1]
    int64_t *seg_begin = nullptr;    // [n_seg]
    int32_t *seg_len = nullptr;      // [n_seg]
    float *partial = nullptr;        // [n_seg * F], grown on demand
    size_t partial_floats = 0;
    int32_t *empty_rows = nullptr;   // [n_empty]
    int64_t n_empty = 0;
    // Short-row chunks, one list per chunk row limit (7, 15, 31), built on first use.
    std::vector<int64_t> h_rowptr;
    int2 *chunks[3] = {nullptr, nullptr, nullptr};
    int64_t n_chunks[3] = {-1, -1, -1};
};

constexpr int kChunkEdges = 128;  // target edges per short-row chunk

// Cuts the short, non-empty rows into chunks of consecutive rows: at most `limit` rows and about
// kChunkEdges edges each, never containing a long row, starting and ending on a non-empty row.
static int build_chunks(sgnn_spmm_plan *p, int which, hipStream_t st) {
    const int limit = which == 0 ? 7 : which == 1 ? 15 : 31;
    const std::vector<int64_t> &rp = p->h_rowptr;
    std::vector<int2> out;
    const int64_t M = p->M;
    int64_t m = 0;
    while (m < M) {
        const int64_t d0 = rp[m + 1] - rp[m];
        if (d0 == 0 || d0 > p->long_thresh) { ++m; continue; }
        const int64_t start = m;
        int64_t last = m, edges = 0;
        while (m < M && m - start < limit && edges < kChunkEdges) {
            const int64_t d = rp[m + 1] - rp[m];
            if (d > p->long_thresh) break;
            if (d > 0) last = m;
            edges += d;
            ++m;
        }
        out.push_back(make_int2((int)start, (int)(last - start + 1)));
    }
    p->n_chunks[which] = (int64_t)out.size();
    if (!out.empty()) {
        SGNN_HIP_CHECK(hipMalloc(&p->chunks[which], sizeof(int2) * out.size()));
        SGNN_HIP_CHECK(hipMemcpyAsync(p->chunks[which], out.data(), sizeof(int2) * out.size(), hipMemcpyHostToDevice, st));
        SGNN_HIP_CHECK(hipStreamSynchronize(st));
    }
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_destroy(sgnn_spmm_plan *p) {
    if (!p) return SGNN_OK;
    (void)hipFree(p->rowptr);
    (void)hipFree(p->col);
    (void)hipFree(p->long_rows);
    (void)hipFree(p->long_segptr);
    (void)hipFree(p->seg_begin);
    (void)hipFree(p->seg_len);
    (void)hipFree(p->partial);
    (void)hipFree(p->empty_rows);
    for (int i = 0; i < 3; ++i) (void)hipFree(p->chunks[i]);
    delete p;
    return SGNN_OK;
}

static int plan_create_impl(sgnn_spmm_plan *p, const int64_t *rowptr, const void *col, int col_is_i64,
                            int long_row_threshold, int segment_edges, hipStream_t st) {
    const int64_t M = p->M, K = p->K, nnz = p->nnz;
    SGNN_HIP_CHECK(hipGetDevice(&p->device));
    p->long_thresh = long_row_threshold > 0 ? long_row_threshold : kDefaultLongThreshold;
    p->seg_edges = segment_edges > 0 ? segment_edges : kDefaultSegmentEdges;

    std::vector<int64_t> &h_rowptr = p->h_rowptr;
    h_rowptr.resize((size_t)M + 1);
    SGNN_HIP_CHECK(hipMemcpyAsync(h_rowptr.data(), rowptr, sizeof(int64_t) * (size_t)(M + 1), hipMemcpyDeviceToHost, st));
    SGNN_HIP_CHECK(hipStreamSynchronize(st));
    if (h_rowptr[0] != 0) return fail(SGNN_ERR_RANGE, "rowptr[0] = %lld, expected 0", (long long)h_rowptr[0]);
    for (int64_t m = 0; m < M; ++m)
        if (h_rowptr[m + 1] < h_rowptr[m]) return fail(SGNN_ERR_RANGE, "rowptr decreases at row %lld", (long long)m);
    if (h_rowptr[M] != nnz)
        return fail(SGNN_ERR_RANGE, "rowptr[M] = %lld but nnz = %lld", (long long)h_rowptr[M], (long long)nnz);

    std::vector<int32_t> long_rows, long_segptr, seg_len, empty_rows;
    std::vector<int64_t> seg_begin;
    long_segptr.push_back(0);
    for (int64_t m = 0; m < M; ++m) {
        const int64_t b = h_rowptr[m], deg = h_rowptr[m + 1] - b;
        if (deg == 0) empty_rows.push_back((int32_t)m);
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
    p->n_empty = (int64_t)empty_rows.size();
    if (p->n_empty > 0) {
        SGNN_HIP_CHECK(hipMalloc(&p->empty_rows, sizeof(int32_t) * empty_rows.size()));
        SGNN_HIP_CHECK(hipMemcpyAsync(p->empty_rows, empty_rows.data(), sizeof(int32_t) * empty_rows.size(), hipMemcpyHostToDevice, st));
        SGNN_HIP_CHECK(hipStreamSynchronize(st));
    }

    SGNN_HIP_CHECK(hipMalloc(&p->rowptr, sizeof(int64_t) * (size_t)(M + 1)));
    SGNN_HIP_CHECK(hipMemcpyAsync(p->rowptr, rowptr, sizeof(int64_t) * (size_t)(M + 1), hipMemcpyDeviceToDevice, st));
    SGNN_HIP_CHECK(hipMalloc(&p->col, sizeof(int32_t) * (size_t)std::max<int64_t>(nnz, 1)));
    if (nnz > 0) {
        int *bad = nullptr;  // [0] = range flag, [1 .. K] = per-column popularity (in-degree)
        const int hot_rows = hot_rows_budget();
        const bool want_pop = hot_rows > 0 && K > hot_rows;
        SGNN_HIP_CHECK(hipMalloc(&bad, sizeof(int) * (size_t)(1 + (want_pop ? K : 0))));
        SGNN_HIP_CHECK(hipMemsetAsync(bad, 0, sizeof(int) * (size_t)(1 + (want_pop ? K : 0)), st));
        int *pop = want_pop ? bad + 1 : nullptr;
        const int nb = (int)std::min<int64_t>((nnz + kBlock - 1) / kBlock, 65536);
        if (col_is_i64)
            hipLaunchKernelGGL((narrow_cols_kernel<int64_t>), dim3(nb), dim3(kBlock), 0, st, (const int64_t *)col, p->col, nnz, K, bad, pop);
        else
            hipLaunchKernelGGL((narrow_cols_kernel<int32_t>), dim3(nb), dim3(kBlock), 0, st, (const int32_t *)col, p->col, nnz, K, bad, pop);
        std::vector<int> h_pop(1 + (want_pop ? (size_t)K : 0));
        hipError_t e1 = hipGetLastError();
        hipError_t e2 = hipMemcpyAsync(h_pop.data(), bad, sizeof(int) * h_pop.size(), hipMemcpyDeviceToHost, st);
        hipError_t e3 = hipStreamSynchronize(st);
        if (e1 == hipSuccess && e2 == hipSuccess && e3 == hipSuccess && h_pop[0] == 0 && want_pop) {
            // popularity of the hot_rows-th most popular column = the admission threshold
            std::vector<int> sorted(h_pop.begin() + 1, h_pop.end());
            std::nth_element(sorted.begin(), sorted.begin() + hot_rows, sorted.end(), std::greater<int>());
            const int hot_min = std::max(sorted[hot_rows] + 1, 2);
            hipLaunchKernelGGL(mark_cold_cols_kernel, dim3(nb), dim3(kBlock), 0, st, p->col, nnz, pop, hot_min);
            e1 = hipGetLastError();
            e3 = hipStreamSynchronize(st);
            p->hot_min = hot_min;
        }
        (void)hipFree(bad);
        SGNN_HIP_CHECK(e1);
        SGNN_HIP_CHECK(e2);
        SGNN_HIP_CHECK(e3);
        if (h_pop[0]) return fail(SGNN_ERR_RANGE, "a column index lies outside [0, %lld)", (long long)K);
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
    const int gw = group_width(nvec);
    const int which = gw == 8 ? 0 : gw == 16 ? 1 : 2;
    if (p->n_chunks[which] < 0) {
        const int rc = build_chunks(p, which, st);
        if (rc != SGNN_OK) return rc;
    }
    ShortArgs a{p->rowptr, p->col, val, x, out, p->chunks[which], (int)p->n_chunks[which], p->empty_rows,
                (int)p->n_empty, (int)F, ldx, ldo, accumulate, row_div};
    SegArgs s{p->col, val, x, p->partial, p->seg_begin, p->seg_len, (int)p->n_seg, (int)F, ldx};
    FinalArgs f{p->long_rows, p->long_segptr, p->partial, out, (int)p->n_long, (int)F, ldo, accumulate, row_div};
    if (vec == 4) dispatch_shape<4>(nvec, a, s, f, st);
    else if (vec == 2) dispatch_shape<2>(nvec, a, s, f, st);
    else dispatch_shape<1>(nvec, a, s, f, st);
    SGNN_HIP_CHECK(hipGetLastError());
    return SGNN_OK;
}
