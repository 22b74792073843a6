// CSR SpMM neighbour aggregation for gfx950:  out (+)= A * X, fp32.
//
// Replaces supergnn_ops.spmm (super_gnn/ops/csrc/spmm.cpp:594-608 of the reference) and the two
// kernels it dispatches to (accumulate: spmm.cpp:348-539; overwrite: spmm.cpp:177-271).
//
// The work is a random gather of dense rows, bound by memory bandwidth and latency; there is no
// MFMA here.  Scheduling is by row class:
//   * short rows (degree <= threshold): consecutive rows are cut into chunks of about 64 edges (fewer
//     on small matrices, so that the chip stays full); one group of G lanes owns one chunk.
//     G*VEC*NV floats cover the feature axis (F=128: 32 lanes x float4, two chunks per wavefront).
//     Because the edges of consecutive CSR rows are contiguous, the group streams the chunk's
//     (col,val) pairs G at a time with one coalesced load, broadcasts them lane by lane and keeps
//     several whole-row gathers in flight regardless of where rows begin and end; a row boundary
//     only switches the accumulator (store the finished row, continue with the next one, whose old
//     value was prefetched).  Edges are summed in CSR order with one fma per edge, starting from
//     the old out value: the same operation sequence as the reference's kernel_1xN
//     (spmm.cpp:87-162), so these rows are bit-identical to the reference.
//   * long rows (power-law hubs): at plan time the row's edges are regrouped by column class (a
//     hash of the column index, 8 classes) and each class run is cut into pieces; one lane group
//     sums one piece into a partial buffer, and a last small kernel adds a row's partials in piece
//     order (deterministic, no float atomics).  Workgroup i only takes pieces of class i % 8, i.e.
//     each XCD gathers only its own class of dense rows, so the eight L2 caches hold disjoint sets
//     of popular rows.
#include <algorithm>
#include <cstdlib>
#include <functional>
#include <mutex>
#include <vector>

#include "common.hpp"

namespace sgnn {

constexpr int kBlock = 256;
constexpr int kDefaultLongThreshold = 128;  // rows with more edges go to the class-partitioned piece path
constexpr int kChunkGroupsWanted = 16384;
constexpr int kDefaultPieceEdges = 32;      // minimum edges per piece of a long row
constexpr int kPopularColumns = 16384;      // size of the "popular" column set the plan looks at
constexpr double kPartitionMinShare = 0.02; // below this share of all edges (popularity ~uniform) leave the long rows as they are

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

// The dense operand of the product: fp32 rows (BITS == 0), or rows that arrive quantized and
// bit-packed in the row-group layout (see quant.hip) and are decoded on the fly.  For those the
// template parameter BITS is a format code: the low four bits are the code width (8, 4 or 2) and
// kBf16Params is added when (zero_point, scale) are bf16 pairs instead of fp32 pairs.
constexpr int kBf16Params = 16;
constexpr int kEdgeSlots = 32;  // added when every edge carries its slot (plan-bound row slots)
struct DenseSrc {
    const float *x;        // fp32: [K, ldx]
    int64_t ldx;
    const uint8_t *q;      // quantized: packed rows of qF bytes
    ParamBuf params;       // quantized: (zero_point, scale) per dense row, fp32 or bf16 pairs
    const int32_t *eslot_csr;   // quantized, ragged segments: position of each edge's dense row in the padded row
                                // space, row_slot[col[e]], in CSR order (bound to the plan) ...
    const int32_t *eslot_long;  // ... and in the regrouped order of the long rows; null = no padding (slot == row)
    int qF;
};

// What one gather of one dense row leaves in a lane's registers: the fp32 values themselves, or
// the packed words plus the row's decode parameters (decoded only when consumed, so that the U
// loads of a batch are all in flight before the first conversion).
template <int VEC, int NV, int BITS>
struct Fetched {
    float f[BITS == 0 ? NV : 1][BITS == 0 ? VEC : 1];
    uint32_t w[BITS == 0 ? 1 : NV];
    float zp, sc;
    int shift;
};

template <int VEC, int NV, int BITS>
__device__ __forceinline__ void fetch_row(Fetched<VEC, NV, BITS> &r, const DenseSrc &d, int c, int edge_slot,
                                          const int (&off)[NV], const bool (&act)[NV]) {
    if constexpr (BITS == 0) {
        const float *xr = d.x + (int64_t)c * d.ldx;
#pragma unroll
        for (int v = 0; v < NV; ++v)
            if (act[v]) vec_load<VEC>(r.f[v], xr + off[v]);
    } else {
        constexpr int NB = BITS & 15;
        constexpr int EPB = 8 / NB;
        const int sl = (BITS & kEdgeSlots) != 0 ? edge_slot : c;  // without a slot stream the row space has no padding
        const float2 ps = load_params_as<(BITS & kBf16Params) != 0>(d.params.p, c);
        r.zp = ps.x;
        r.sc = ps.y;
        r.shift = (EPB - 1 - (sl % EPB)) * NB;
        const uint8_t *qr = d.q + (int64_t)(sl / EPB) * d.qF;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
            if constexpr (VEC == 4) r.w[v] = *reinterpret_cast<const uint32_t *>(qr + off[v]);
            else if constexpr (VEC == 2) r.w[v] = *reinterpret_cast<const uint16_t *>(qr + off[v]);
            else r.w[v] = qr[off[v]];
        }
    }
}

// acc += w * row, one fma per element.  A quantized row is first decoded exactly as the stand-alone
// unpack+dequantize kernel does, fma(code, scale, zero_point), so the fused product equals
// "dequantize, then multiply" bit for bit.
template <int VEC, int NV, int BITS>
__device__ __forceinline__ void fma_row(float (&acc)[NV][VEC], float w, const Fetched<VEC, NV, BITS> &r) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            float xv;
            if constexpr (BITS == 0) {
                xv = r.f[v][k];
            } else {
                const uint32_t code = (r.w[v] >> (8 * k + r.shift)) & ((1u << (BITS & 15)) - 1u);
                xv = fmaf((float)code, r.sc, r.zp);
            }
            acc[v][k] = fmaf(w, xv, acc[v][k]);
        }
    }
}

// Accumulate the `deg` edges listed at colp into acc for one feature tile.  The weight of edge i is
// val[eperm[i]], or val[i] when eperm is null (val may be null = all ones).
template <int VEC, int G, int NV, int BITS, bool PERM>
__device__ __forceinline__ void gather_piece(float (&acc)[NV][VEC], const int32_t *__restrict__ colp,
                                             const int32_t *__restrict__ eperm, const float *__restrict__ val,
                                             const int32_t *__restrict__ slotp, int deg, const DenseSrc &dense,
                                             const int (&off)[NV], const bool (&act)[NV], int lig) {
    constexpr int U = unroll_of(NV);
    // (col,val) pairs are fetched G at a time, one chunk ahead of the gathers that consume them.
    int nc = 0, ns = -1;
    float nw = 1.0f;
    if (lig < deg) {
        nc = __builtin_nontemporal_load(colp + lig);
        if (val) nw = PERM ? val[__builtin_nontemporal_load(eperm + lig)] : __builtin_nontemporal_load(val + lig);
        if constexpr ((BITS & kEdgeSlots) != 0) ns = __builtin_nontemporal_load(slotp + lig);
    }
    for (int base = 0; base < deg; base += G) {
        const int myc = nc, mys = ns;
        const float myw = nw;
        const int nidx = base + G + lig;
        if (nidx < deg) {
            nc = __builtin_nontemporal_load(colp + nidx);
            if (val) nw = PERM ? val[__builtin_nontemporal_load(eperm + nidx)] : __builtin_nontemporal_load(val + nidx);
            if constexpr ((BITS & kEdgeSlots) != 0) ns = __builtin_nontemporal_load(slotp + nidx);
        }
        const int cnt = deg - base < G ? deg - base : G;
        for (int j = 0; j < cnt; j += U) {
            Fetched<VEC, NV, BITS> xv[U];
            // U gathers back to back; past the end the last edge's row is fetched again (a cache
            // hit) so that no branch separates the loads.
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int src = j + u < cnt ? j + u : cnt - 1;
                int es = -1;
                if constexpr ((BITS & kEdgeSlots) != 0) es = group_bcast_i<G>(mys, src);
                fetch_row<VEC, NV, BITS>(xv[u], dense, group_bcast_i<G>(myc, src), es, off, act);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (j + u < cnt) fma_row<VEC, NV, BITS>(acc, group_bcast_f<G>(myw, j + u), xv[u]);
            }
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

template <int VEC, int G, int NV, int BITS>
__global__ __launch_bounds__(kBlock) void spmm_short_kernel(
    const int64_t *__restrict__ rowptr, const int32_t *__restrict__ col, const float *__restrict__ val,
    const DenseSrc dense, float *__restrict__ out, const int4 *__restrict__ chunks, int n_chunks, int F,
    int64_t ldo, int accumulate, const float *__restrict__ row_div, uint32_t nblocks) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    // gathers in flight per lane group: 6 keeps the kernel at 75 VGPRs (6 waves per SIMD); 8 costs 83 (5 waves)
    constexpr int U = NV == 1 ? 6 : unroll_of(NV);
    const uint32_t lb = xcd_contiguous_block(blockIdx.x, nblocks);
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int ci = (int)lb * GPB + gid;
    if (ci >= n_chunks) return;
    // A chunk record is (first row, row count, first edge, edge count): the column/weight loads
    // depend on it alone and are issued before the row pointers come back.
    int4 ch = chunks[ci];
    if constexpr (G == 64) {
        ch.x = __builtin_amdgcn_readfirstlane(ch.x);
        ch.y = __builtin_amdgcn_readfirstlane(ch.y);
        ch.z = __builtin_amdgcn_readfirstlane(ch.z);
        ch.w = __builtin_amdgcn_readfirstlane(ch.w);
    }
    const int rb = ch.x, nr = ch.y;  // rows rb .. rb+nr-1, first and last non-empty, 1 <= nr <= limit
    const int64_t B = ch.z;
    const int E = ch.w;
    const int32_t *colp = col + B;
    const float *valp = val ? val + B : nullptr;
    const int32_t *slotp = nullptr;
    if constexpr ((BITS & kEdgeSlots) != 0) slotp = dense.eslot_csr + B;
    int nc0 = 0, ns0 = -1;
    float nw0 = 1.0f;
    if (lig < E) {
        nc0 = __builtin_nontemporal_load(colp + lig);
        if (valp) nw0 = __builtin_nontemporal_load(valp + lig);
        if constexpr ((BITS & kEdgeSlots) != 0) ns0 = __builtin_nontemporal_load(slotp + lig);
    }

    // Lane i holds rowptr[rb+i] relative to the chunk's first edge (lanes >= nr hold the end).
    const int rel = (int)(rowptr[rb + (lig < nr ? lig : nr)] - B);
    const int rel_next = __shfl_down(rel, 1, G);
    const uint32_t mask = group_ballot<G>(lig < nr && rel_next > rel);  // bit i: row rb+i has edges
    const float mydiv = (row_div && lig < nr) ? row_div[rb + lig] : 1.0f;

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

        int nc = nc0, ns = ns0;
        float nw = nw0;
        if (f0 > 0 && lig < E) {  // a later feature tile walks the chunk's edges again
            nc = __builtin_nontemporal_load(colp + lig);
            if (valp) nw = __builtin_nontemporal_load(valp + lig);
            if constexpr ((BITS & kEdgeSlots) != 0) ns = __builtin_nontemporal_load(slotp + lig);
        }
        for (int base = 0; base < E; base += G) {
            const int myc = nc, mys = ns;
            const float myw = nw;
            const int nidx = base + G + lig;  // next chunk, fetched one chunk ahead of its gathers
            if (nidx < E) {
                nc = __builtin_nontemporal_load(colp + nidx);
                if (valp) nw = __builtin_nontemporal_load(valp + nidx);
                if constexpr ((BITS & kEdgeSlots) != 0) ns = __builtin_nontemporal_load(slotp + nidx);
            }
            const int cnt = E - base < G ? E - base : G;
            for (int j = 0; j < cnt; j += U) {
                Fetched<VEC, NV, BITS> xv[U];
                // U gathers back to back.  Past the end of the chunk the last edge's row is
                // fetched again (a cache hit) so that no branch separates the loads.
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int src = j + u < cnt ? j + u : cnt - 1;
                    int es = -1;
                    if constexpr ((BITS & kEdgeSlots) != 0) es = group_bcast_i<G>(mys, src);
                    fetch_row<VEC, NV, BITS>(xv[u], dense, group_bcast_i<G>(myc, src), es, off, act);
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
                        fma_row<VEC, NV, BITS>(acc, group_bcast_f<G>(myw, j + u), xv[u]);
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
// epilogue (old value / divisor).  One lane group per kEmptyRowsPerGroup empty rows: the row ids (and
// divisors) of all of them are requested before the first store, so a wave pays the latency of the
// dependent id -> address chain once, not once per row.
constexpr int kEmptyRowsPerGroup = 4;
template <int VEC, int G, int NV>
__global__ __launch_bounds__(kBlock) void spmm_empty_rows_kernel(const int32_t *__restrict__ empty_rows, int n_empty,
                                                                 float *__restrict__ out, int F, int64_t ldo,
                                                                 int accumulate, const float *__restrict__ row_div) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    constexpr int R = kEmptyRowsPerGroup;
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int i0 = (blockIdx.x * GPB + gid) * R;
    if (i0 >= n_empty) return;
    int64_t rows[R];
    float divs[R];
#pragma unroll
    for (int r = 0; r < R; ++r) rows[r] = empty_rows[i0 + r < n_empty ? i0 + r : n_empty - 1];
#pragma unroll
    for (int r = 0; r < R; ++r) divs[r] = row_div ? row_div[rows[r]] : 1.0f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (i0 + r >= n_empty) break;
        const int64_t row = rows[r];
        const float div = divs[r];
        // x / 1 == x for every float, so an accumulating call leaves such a row exactly as it is: nothing
        // to read or write (the mean epilogue divides rows without edges by a degree clamped to 1).
        if (accumulate && div == 1.0f) continue;
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
}

// ------------------------------------------------------------------------------------------------
// Long rows, step 1: pieces.  At plan time a long row's edges are regrouped by column class (a hash
// of the column index, 8 classes) and each class run is cut into pieces; a piece is summed by one
// lane group into partial[piece, :].  All pieces a workgroup handles belong to ONE class, and workgroup i takes
// class i % 8: workgroups are dealt round-robin to the 8 XCDs, so every XCD gathers only the dense
// rows of its own class and the eight 4 MB L2s hold eight DISJOINT sets of popular rows instead of
// eight copies of the same set.
// ------------------------------------------------------------------------------------------------
// Lanes whose vector lies past the end of the row do not skip their gathers: they load the tile's
// first vector again (a cache hit) and simply never store.  Every gather is then unconditional;
// per-load lane predicates would fence each one in its own exec-mask region (measured: piece kernel
// 2.08 -> 1.74 ms at F = 128, 2.07 -> 1.70 ms at F = 100).
template <int VEC, int G, int NV, int BITS, bool PERM>
__global__ __launch_bounds__(kBlock) void spmm_piece_kernel(
    const int32_t *__restrict__ col_long, const int32_t *__restrict__ eperm, const float *__restrict__ val,
    const DenseSrc dense, float *__restrict__ partial, const int4 *__restrict__ cls_work, int cls_stride, int F) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int cls = blockIdx.x % kNumXCD;
    const int slot = (int)(blockIdx.x / kNumXCD) * GPB + gid;
    if (slot >= cls_stride) return;
    // One record per piece, (piece id, first edge, edge count): the only load between the start of
    // the wave and its column loads.  Every class's list is padded to cls_stride records.
    const int4 w = cls_work[(int64_t)cls * cls_stride + slot];
    int item = w.x, b = w.y, len = w.z;
    if (len == 0) return;
    if constexpr (G == 64) {
        item = __builtin_amdgcn_readfirstlane(item);
        b = __builtin_amdgcn_readfirstlane(b);
        len = __builtin_amdgcn_readfirstlane(len);
    }
    for (int f0 = 0; f0 < F; f0 += TILE) {
        int off[NV], off_ld[NV];
        bool act[NV], act_ld[NV];
        float acc[NV][VEC];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            off[v] = f0 + (v * G + lig) * VEC;
            act[v] = off[v] < F;
            off_ld[v] = act[v] ? off[v] : f0;
            act_ld[v] = true;
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[v][k] = 0.0f;
        }
        gather_piece<VEC, G, NV, BITS, PERM>(acc, col_long + b, PERM ? eperm + b : nullptr, (PERM || !val) ? val : val + b,
                                             (BITS & kEdgeSlots) != 0 ? dense.eslot_long + b : nullptr, len, dense,
                                             off_ld, act_ld, lig);
#pragma unroll
        for (int v = 0; v < NV; ++v)
            if (act[v]) vec_store<VEC>(partial + (int64_t)item * F + off[v], acc[v]);
    }
}

// ------------------------------------------------------------------------------------------------
// Long rows, step 2: add a row's piece partials in piece order, epilogue, store.
// ------------------------------------------------------------------------------------------------
template <int VEC, int G, int NV>
__global__ __launch_bounds__(kBlock) void spmm_long_final_kernel(
    const int32_t *__restrict__ long_rows, const int32_t *__restrict__ long_pbeg,
    const float *__restrict__ partial, float *__restrict__ out, int n_long, int F, int64_t ldo,
    int accumulate, const float *__restrict__ row_div) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    constexpr int UP = 8;
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int li = blockIdx.x * GPB + gid;
    if (li >= n_long) return;
    const int64_t row = long_rows[li];
    const int s0 = long_pbeg[li], s1 = long_pbeg[li + 1];
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
            for (int s = s0; s < s1; s += UP) {
                float p[UP][VEC];
#pragma unroll
                for (int u = 0; u < UP; ++u) {
                    const int si = s + u < s1 ? s + u : s1 - 1;
                    vec_load<VEC>(p[u], partial + (int64_t)si * F + off);
                }
#pragma unroll
                for (int u = 0; u < UP; ++u) {
                    if (s + u < s1) {
#pragma unroll
                        for (int k = 0; k < VEC; ++k) acc[k] += p[u][k];
                    }
                }
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
// Plan-time: regroup every long row's edges by column class, keeping the CSR order inside a class
// (a stable 8-way split done by one workgroup per row).
// ------------------------------------------------------------------------------------------------
// Column class: a multiplicative hash, NOT col % 8.  Dense row c starts at byte c * 4F, so a class
// taken from the low bits of c would pin address bits that the L2 and HBM channel interleaving
// use, and an XCD would then hammer a fraction of its cache channels.
__device__ __forceinline__ int col_class(int32_t c) {
    return (int)(((uint32_t)c * 0x9E3779B1u) >> 29);
}

__global__ __launch_bounds__(kBlock) void partition_long_rows_kernel(
    const int64_t *__restrict__ rowptr, const int32_t *__restrict__ col, const int32_t *__restrict__ long_rows,
    const int32_t *__restrict__ long_off, int32_t *__restrict__ col_long, int32_t *__restrict__ eperm,
    int32_t *__restrict__ cls_count) {
    __shared__ int cnt[kNumXCD], base[kNumXCD], wave_cnt[kBlock / 64][kNumXCD];
    const int slot = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row = long_rows[slot];
    const int64_t b = rowptr[row];
    const int n = (int)(rowptr[row + 1] - b);
    const int dst0 = long_off[slot];
    if (tid < kNumXCD) cnt[tid] = 0;
    __syncthreads();
    for (int i = tid; i < n; i += kBlock) atomicAdd(&cnt[col_class(col[b + i])], 1);
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int k = 0; k < kNumXCD; ++k) {
            base[k] = run;
            run += cnt[k];
            cls_count[slot * kNumXCD + k] = cnt[k];
        }
    }
    __syncthreads();
    for (int c0 = 0; c0 < n; c0 += kBlock) {
        const int i = c0 + tid;
        const bool valid = i < n;
        const int c = valid ? col[b + i] : 0;
        const int k = col_class(c);
        int my_rank = 0;
#pragma unroll
        for (int kk = 0; kk < kNumXCD; ++kk) {
            const unsigned long long m = __ballot(valid && k == kk);
            if (k == kk) my_rank = __popcll(m & ((1ull << lane) - 1ull));
            if (lane == 0) wave_cnt[wave][kk] = __popcll(m);
        }
        __syncthreads();
        if (valid) {
            int pre = 0;
            for (int w = 0; w < wave; ++w) pre += wave_cnt[w][k];
            const int dst = dst0 + base[k] + pre + my_rank;
            col_long[dst] = c;
            eperm[dst] = (int32_t)(b + i);
        }
        __syncthreads();
        if (tid < kNumXCD) {
            int add = 0;
            for (int w = 0; w < kBlock / 64; ++w) add += wave_cnt[w][tid];
            base[tid] += add;
        }
        __syncthreads();
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

// How often each column occurs (its in-degree): decides at plan time whether regrouping the long
// rows by column class can pay off.
__global__ __launch_bounds__(kBlock) void column_popularity_kernel(const int32_t *__restrict__ col, int64_t n,
                                                                   int *__restrict__ popularity) {
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (; i < n; i += stride) atomicAdd(popularity + col[i], 1);
}

// dst[i] = table[idx[i]]: the per-edge slot stream of a plan (idx = the plan's column array).
__global__ __launch_bounds__(kBlock) void translate_columns_kernel(const int32_t *__restrict__ idx, const int32_t *__restrict__ table,
                                                                   int32_t *__restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) dst[i] = table[__builtin_nontemporal_load(idx + i)];
}

__global__ __launch_bounds__(kBlock) void permute_values_kernel(const float *__restrict__ val, const int32_t *__restrict__ eperm,
                                                                float *__restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) dst[i] = val[__builtin_nontemporal_load(eperm + i)];
}

// ------------------------------------------------------------------------------------------------
// Launch tables.
// ------------------------------------------------------------------------------------------------
struct ShortArgs {
    const int64_t *rowptr; const int32_t *col; const float *val; DenseSrc dense; float *out;
    const int4 *chunks; int n_chunks; const int32_t *empty_rows; int n_empty;
    int F; int64_t ldo; int accumulate; const float *row_div;
};
struct PieceArgs {
    const int32_t *col_long; const int32_t *eperm; const float *val; float *partial;
    const int4 *cls_work;
    int max_cls_items; int F;
    hipStream_t side; hipEvent_t ev_fork, ev_join;  // side != null: long rows run beside the short rows
};
struct FinalArgs {
    const int32_t *long_rows; const int32_t *long_pbeg; const float *partial; float *out; int n_long;
    int F; int64_t ldo; int accumulate; const float *row_div;
};

template <int VEC, int G, int NV, int BITS>
static void launch_all(const ShortArgs &a, const PieceArgs &s, const FinalArgs &f, hipStream_t st) {
    constexpr int GPB = kBlock / G;
    // The long rows (pieces + final sum) and the short rows write disjoint output rows.  With a side
    // stream they are issued side by side: fork after the caller's earlier work, join before returning.
    hipStream_t ls = st;
    if (s.side != nullptr && f.n_long > 0 && a.n_chunks > 0) {
        (void)hipEventRecord(s.ev_fork, st);
        (void)hipStreamWaitEvent(s.side, s.ev_fork, 0);
        ls = s.side;
    }
    if (f.n_long > 0) {
        {
            // workgroup i serves class i % 8: grid = 8 * (workgroups of the fullest class)
            const uint32_t nb = (uint32_t)kNumXCD * (uint32_t)((s.max_cls_items + GPB - 1) / GPB);
            ProfScope prof(BITS == 0 ? K_SPMM_PIECE : K_FUSED_PIECE, ls);
            if (s.eperm)
                hipLaunchKernelGGL((spmm_piece_kernel<VEC, G, NV, BITS, true>), dim3(nb), dim3(kBlock), 0, ls, s.col_long,
                                   s.eperm, s.val, a.dense, s.partial, s.cls_work, s.max_cls_items, s.F);
            else
                hipLaunchKernelGGL((spmm_piece_kernel<VEC, G, NV, BITS, false>), dim3(nb), dim3(kBlock), 0, ls, s.col_long,
                                   s.eperm, s.val, a.dense, s.partial, s.cls_work, s.max_cls_items, s.F);
        }
        const uint32_t nb = (uint32_t)((f.n_long + GPB - 1) / GPB);
        ProfScope prof(K_SPMM_LONG_FINAL, ls);
        hipLaunchKernelGGL((spmm_long_final_kernel<VEC, G, NV>), dim3(nb), dim3(kBlock), 0, ls, f.long_rows,
                           f.long_pbeg, f.partial, f.out, f.n_long, f.F, f.ldo, f.accumulate, f.row_div);
    }
    if (a.n_chunks > 0) {
        const uint32_t nb = (uint32_t)((a.n_chunks + GPB - 1) / GPB);
        ProfScope prof(BITS == 0 ? K_SPMM_SHORT : K_FUSED_SHORT, st);
        hipLaunchKernelGGL((spmm_short_kernel<VEC, G, NV, BITS>), dim3(nb), dim3(kBlock), 0, st, a.rowptr, a.col, a.val,
                           a.dense, a.out, a.chunks, a.n_chunks, a.F, a.ldo, a.accumulate, a.row_div, nb);
    }
    if (a.n_empty > 0 && (!a.accumulate || a.row_div)) {
        const uint32_t nb = (uint32_t)((a.n_empty + GPB * kEmptyRowsPerGroup - 1) / (GPB * kEmptyRowsPerGroup));
        ProfScope prof(K_SPMM_EMPTY_ROWS, st);
        hipLaunchKernelGGL((spmm_empty_rows_kernel<VEC, G, NV>), dim3(nb), dim3(kBlock), 0, st, a.empty_rows, a.n_empty,
                           a.out, a.F, a.ldo, a.accumulate, a.row_div);
    }
    if (ls != st) {
        (void)hipEventRecord(s.ev_join, ls);
        (void)hipStreamWaitEvent(st, s.ev_join, 0);
    }
}

// Lane-group width for a row of nvec vectors (the kernels are instantiated for these shapes).
static int group_width(int nvec) { return nvec <= 8 ? 8 : nvec <= 16 ? 16 : nvec <= 32 ? 32 : 64; }

template <int VEC>
static int dispatch_shape(int nvec, const ShortArgs &a, const PieceArgs &s, const FinalArgs &f, hipStream_t st) {
    if (nvec <= 8) launch_all<VEC, 8, 1, 0>(a, s, f, st);
    else if (nvec <= 16) launch_all<VEC, 16, 1, 0>(a, s, f, st);
    else if (nvec <= 32) launch_all<VEC, 32, 1, 0>(a, s, f, st);
    else if (nvec <= 64) launch_all<VEC, 64, 1, 0>(a, s, f, st);
    else if (nvec <= 128) launch_all<VEC, 64, 2, 0>(a, s, f, st);
    else if (nvec <= 192) launch_all<VEC, 64, 3, 0>(a, s, f, st);
    else if (nvec <= 256) launch_all<VEC, 64, 4, 0>(a, s, f, st);
    else if (nvec <= 320) launch_all<VEC, 64, 5, 0>(a, s, f, st);
    else if (nvec <= 384) launch_all<VEC, 64, 6, 0>(a, s, f, st);
    else launch_all<VEC, 64, 8, 0>(a, s, f, st);  // feature axis walked in tiles of 512 vectors
    return SGNN_OK;
}

// Quantized dense operand: float4-wide lanes only (F % 4 == 0), one packed word per lane and vector.
template <int BITS>
static int dispatch_shape_dq(int nvec, const ShortArgs &a, const PieceArgs &s, const FinalArgs &f, hipStream_t st) {
    if (nvec <= 8) launch_all<4, 8, 1, BITS>(a, s, f, st);
    else if (nvec <= 16) launch_all<4, 16, 1, BITS>(a, s, f, st);
    else if (nvec <= 32) launch_all<4, 32, 1, BITS>(a, s, f, st);
    else if (nvec <= 64) launch_all<4, 64, 1, BITS>(a, s, f, st);
    else if (nvec <= 128) launch_all<4, 64, 2, BITS>(a, s, f, st);
    else if (nvec <= 256) launch_all<4, 64, 4, BITS>(a, s, f, st);
    else launch_all<4, 64, 8, BITS>(a, s, f, st);
    return SGNN_OK;
}

}  // namespace sgnn

using namespace sgnn;

static int env_int(const char *name, int dflt) {
    const char *e = getenv(name);
    return e ? atoi(e) : dflt;
}

// ------------------------------------------------------------------------------------------------
// Scratch of sgnn_spmm_csr_f32_noalloc: the piece partials of the long rows, in a device array the
// code object itself carries (every GPU the library is loaded on holds its own 64 MiB copy until
// the process ends).  In host code the array's NAME is only a handle for hipGetSymbolAddress; the
// address kernels and copies must use is looked up once per device and kept in g_scratch_ptr.
// ------------------------------------------------------------------------------------------------
constexpr size_t kScratchFloats = (size_t)16 << 20;  // 64 MiB
static __device__ __align__(256) float g_spmm_scratch[kScratchFloats];
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static float *g_scratch_ptr[kMaxDevices] = {};

// Address of the CURRENT device's copy of the scratch array (looked up on first use per device).
static int scratch_for_current_device(float **out) {
    int dev = 0;
    SGNN_HIP_CHECK(hipGetDevice(&dev));
    SGNN_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d beyond the %d this library keeps scratch addresses for", dev, kMaxDevices);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        float *ptr = nullptr;
        SGNN_HIP_CHECK(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(g_spmm_scratch)));
        SGNN_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned a null scratch address on device %d", dev);
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return SGNN_OK;
}

struct sgnn_spmm_plan {
    int device = 0;
    int64_t M = 0, K = 0, nnz = 0;
    int long_thresh = 0, piece_edges = 0;
    bool partitioned = false;   // long rows regrouped by column class
    double top_share = 0.0;     // share of all edges that point at the kPopularColumns most popular columns
    int64_t *rowptr = nullptr;  // device, owned
    int32_t *col = nullptr;     // device, owned
    // long rows
    int64_t n_long = 0, n_items = 0, long_edges = 0;
    int max_cls_items = 0;
    int32_t *long_rows = nullptr;   // [n_long] row ids
    int32_t *long_pbeg = nullptr;   // [n_long + 1] first piece of each long row
    int32_t *col_long = nullptr;    // [long_edges] columns regrouped by class inside each long row
    int32_t *eperm = nullptr;       // [long_edges] original edge index of each regrouped edge
    hipStream_t side = nullptr;     // long rows run here, beside the short rows on the caller's stream
    hipEvent_t ev_fork = nullptr, ev_join = nullptr;
    float *val_long = nullptr;      // [long_edges] bound edge values in regrouped order (sgnn_spmm_plan_bind_values)
    const float *bound_val = nullptr;  // the caller's array val_long was taken from
    int32_t *eslot_csr = nullptr;      // [nnz] row_slot[col[e]] in CSR order (sgnn_spmm_plan_bind_row_slots)
    int32_t *eslot_long = nullptr;     // [long_edges] the same in regrouped order (partitioned plans)
    const int32_t *bound_slots = nullptr;  // the caller's table they were taken from
    int4 *cls_work = nullptr;       // [8 * max_cls_items] (piece id, first edge in col_long / eperm, edges, 0) per class, zero-padded
    float *partial = nullptr;       // [n_items * F], grown on demand
    size_t partial_floats = 0;
    // rows without edges
    int32_t *empty_rows = nullptr;
    int64_t n_empty = 0;
    // Short-row chunks, one list per chunk row limit (7, 15, 31), built on first use.
    std::vector<int64_t> h_rowptr;
    int4 *chunks[3] = {nullptr, nullptr, nullptr};
    int64_t n_chunks[3] = {-1, -1, -1};
};

// Cuts the short, non-empty rows into chunks of consecutive rows: at most `limit` rows and about
// `target` edges each, never containing a long row, starting and ending on a non-empty row.
static int build_chunks(sgnn_spmm_plan *p, int which, hipStream_t st) {
    const int limit = which == 0 ? 7 : which == 1 ? 15 : 31;
    // About 64 edges per chunk on large matrices (measured plateau 32-96 on the power-law graph; 128
    // is 4 % slower, 256 15 %), and never so few chunks that the chip idles: a small matrix is cut
    // finer, down to 16 edges, until there are about kChunkGroupsWanted lane groups for the 256 CUs.
    int target = env_int("SGNN_SPMM_CHUNK_EDGES", 0);
    if (target <= 0) {
        const int64_t short_edges = p->nnz - p->long_edges;
        target = (int)std::min<int64_t>(64, std::max<int64_t>(16, short_edges / env_int("SGNN_SPMM_CHUNK_GROUPS", kChunkGroupsWanted)));
    }
    const std::vector<int64_t> &rp = p->h_rowptr;
    std::vector<int4> out;
    const int64_t M = p->M;
    int64_t m = 0;
    while (m < M) {
        const int64_t d0 = rp[m + 1] - rp[m];
        if (d0 == 0 || d0 > p->long_thresh) { ++m; continue; }
        const int64_t start = m;
        int64_t last = m, edges = 0;
        while (m < M && m - start < limit && edges < target) {
            const int64_t d = rp[m + 1] - rp[m];
            if (d > p->long_thresh) break;
            if (d > 0) last = m;
            edges += d;
            ++m;
        }
        out.push_back(make_int4((int)start, (int)(last - start + 1), (int)rp[start], (int)(rp[last + 1] - rp[start])));
    }
    p->n_chunks[which] = (int64_t)out.size();
    if (!out.empty()) {
        SGNN_HIP_CHECK(hipMalloc(&p->chunks[which], sizeof(int4) * out.size()));
        SGNN_HIP_CHECK(hipMemcpyAsync(p->chunks[which], out.data(), sizeof(int4) * out.size(), hipMemcpyHostToDevice, st));
        SGNN_HIP_CHECK(hipStreamSynchronize(st));
    }
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_destroy(sgnn_spmm_plan *p) {
    if (!p) return SGNN_OK;
    (void)hipFree(p->rowptr);
    (void)hipFree(p->col);
    (void)hipFree(p->long_rows);
    (void)hipFree(p->long_pbeg);
    if (p->col_long != p->col) (void)hipFree(p->col_long);
    (void)hipFree(p->eperm);
    (void)hipFree(p->cls_work);
    (void)hipFree(p->val_long);
    (void)hipFree(p->eslot_csr);
    (void)hipFree(p->eslot_long);
    if (p->ev_fork) (void)hipEventDestroy(p->ev_fork);
    if (p->ev_join) (void)hipEventDestroy(p->ev_join);
    if (p->side) (void)hipStreamDestroy(p->side);
    (void)hipFree(p->partial);
    (void)hipFree(p->empty_rows);
    for (int i = 0; i < 3; ++i) (void)hipFree(p->chunks[i]);
    delete p;
    return SGNN_OK;
}

// A plan-time device temporary, freed on every way out of the scope.
template <typename T>
struct DevTmp {
    T *p = nullptr;
    ~DevTmp() { (void)hipFree(p); }
};

template <typename T>
static int upload(T **dst, const std::vector<T> &src, hipStream_t st) {
    if (src.empty()) return SGNN_OK;
    SGNN_HIP_CHECK(hipMalloc(dst, sizeof(T) * src.size()));
    SGNN_HIP_CHECK(hipMemcpyAsync(*dst, src.data(), sizeof(T) * src.size(), hipMemcpyHostToDevice, st));
    return SGNN_OK;
}

static int plan_create_impl(sgnn_spmm_plan *p, const int64_t *rowptr, const void *col, int col_is_i64,
                            hipStream_t st) {
    const int64_t M = p->M, K = p->K, nnz = p->nnz;
    SGNN_HIP_CHECK(hipGetDevice(&p->device));

    std::vector<int64_t> &h_rowptr = p->h_rowptr;
    h_rowptr.resize((size_t)M + 1);
    SGNN_HIP_CHECK(hipMemcpyAsync(h_rowptr.data(), rowptr, sizeof(int64_t) * (size_t)(M + 1), hipMemcpyDeviceToHost, st));
    SGNN_HIP_CHECK(hipStreamSynchronize(st));
    if (h_rowptr[0] != 0) return fail(SGNN_ERR_RANGE, "rowptr[0] = %lld, expected 0", (long long)h_rowptr[0]);
    for (int64_t m = 0; m < M; ++m)
        if (h_rowptr[m + 1] < h_rowptr[m]) return fail(SGNN_ERR_RANGE, "rowptr decreases at row %lld", (long long)m);
    if (h_rowptr[M] != nnz)
        return fail(SGNN_ERR_RANGE, "rowptr[M] = %lld but nnz = %lld", (long long)h_rowptr[M], (long long)nnz);

    // ---- row classes ------------------------------------------------------------------------
    std::vector<int32_t> long_rows, long_off, empty_rows;
    for (int64_t m = 0; m < M; ++m) {
        const int64_t deg = h_rowptr[m + 1] - h_rowptr[m];
        if (deg == 0) empty_rows.push_back((int32_t)m);
        if (deg <= p->long_thresh) continue;
        long_rows.push_back((int32_t)m);
        long_off.push_back((int32_t)p->long_edges);
        p->long_edges += deg;
    }
    p->n_long = (int64_t)long_rows.size();
    p->n_empty = (int64_t)empty_rows.size();

    // ---- device copies: rowptr, narrowed + range-checked columns -------------------------------
    SGNN_HIP_CHECK(hipMalloc(&p->rowptr, sizeof(int64_t) * (size_t)(M + 1)));
    SGNN_HIP_CHECK(hipMemcpyAsync(p->rowptr, rowptr, sizeof(int64_t) * (size_t)(M + 1), hipMemcpyDeviceToDevice, st));
    SGNN_HIP_CHECK(hipMalloc(&p->col, sizeof(int32_t) * (size_t)std::max<int64_t>(nnz, 1)));
    int rc = upload(&p->empty_rows, empty_rows, st);
    if (rc != SGNN_OK) return rc;
    if (nnz > 0) {
        DevTmp<int> bad;
        SGNN_HIP_CHECK(hipMalloc(&bad.p, sizeof(int)));
        SGNN_HIP_CHECK(hipMemsetAsync(bad.p, 0, sizeof(int), st));
        const int nb = (int)std::min<int64_t>((nnz + kBlock - 1) / kBlock, 65536);
        if (col_is_i64)
            hipLaunchKernelGGL((narrow_cols_kernel<int64_t>), dim3(nb), dim3(kBlock), 0, st, (const int64_t *)col, p->col, nnz, K, bad.p);
        else
            hipLaunchKernelGGL((narrow_cols_kernel<int32_t>), dim3(nb), dim3(kBlock), 0, st, (const int32_t *)col, p->col, nnz, K, bad.p);
        int h_bad = 0;
        SGNN_HIP_CHECK(hipGetLastError());
        SGNN_HIP_CHECK(hipMemcpyAsync(&h_bad, bad.p, sizeof(int), hipMemcpyDeviceToHost, st));
        SGNN_HIP_CHECK(hipStreamSynchronize(st));
        if (h_bad) return fail(SGNN_ERR_RANGE, "a column index lies outside [0, %lld)", (long long)K);
    }

    // ---- long rows: regroup by column class (when popular columns exist), cut into pieces --------
    if (p->n_long > 0) {
        if ((rc = upload(&p->long_rows, long_rows, st)) != SGNN_OK) return rc;
        // Regrouping lets each XCD's L2 keep its own slice of the popular dense rows; it pays when a
        // modest set of columns receives a large share of the gathers (power-law graphs) and costs
        // ~15% (smaller pieces, permuted val reads) when no column is popular.  Measure it.
        const int part_env = env_int("SGNN_SPMM_PARTITION", -1);
        if (part_env >= 0) {
            p->partitioned = part_env != 0;
        } else if (K <= kPopularColumns) {
            p->partitioned = true;  // every dense row is "popular": eight disjoint slices beat eight full copies
        } else {
            DevTmp<int> pop;
            SGNN_HIP_CHECK(hipMalloc(&pop.p, sizeof(int) * (size_t)K));
            SGNN_HIP_CHECK(hipMemsetAsync(pop.p, 0, sizeof(int) * (size_t)K, st));
            const int nb = (int)std::min<int64_t>((nnz + kBlock - 1) / kBlock, 65536);
            hipLaunchKernelGGL(column_popularity_kernel, dim3(nb), dim3(kBlock), 0, st, p->col, nnz, pop.p);
            std::vector<int> h_pop((size_t)K);
            SGNN_HIP_CHECK(hipGetLastError());
            SGNN_HIP_CHECK(hipMemcpyAsync(h_pop.data(), pop.p, sizeof(int) * h_pop.size(), hipMemcpyDeviceToHost, st));
            SGNN_HIP_CHECK(hipStreamSynchronize(st));
            std::nth_element(h_pop.begin(), h_pop.begin() + kPopularColumns, h_pop.end(), std::greater<int>());
            int64_t top = 0;
            for (int i = 0; i < kPopularColumns; ++i) top += h_pop[i];
            p->top_share = (double)top / (double)nnz;
            // a clearly popular set, or at least non-uniform popularity with enough reuse per column to matter
            p->partitioned = p->top_share >= 0.2 || (p->top_share >= kPartitionMinShare && nnz >= 8 * K);
        }
        std::vector<int32_t> cls_count;
        if (p->partitioned) {
            DevTmp<int32_t> d_long_off, d_cls_count;
            if ((rc = upload(&d_long_off.p, long_off, st)) != SGNN_OK) return rc;
            SGNN_HIP_CHECK(hipMalloc(&d_cls_count.p, sizeof(int32_t) * (size_t)p->n_long * kNumXCD));
            SGNN_HIP_CHECK(hipMalloc(&p->col_long, sizeof(int32_t) * (size_t)p->long_edges));
            SGNN_HIP_CHECK(hipMalloc(&p->eperm, sizeof(int32_t) * (size_t)p->long_edges));
            hipLaunchKernelGGL(partition_long_rows_kernel, dim3((uint32_t)p->n_long), dim3(kBlock), 0, st, p->rowptr, p->col,
                               p->long_rows, d_long_off.p, p->col_long, p->eperm, d_cls_count.p);
            cls_count.resize((size_t)p->n_long * kNumXCD);
            SGNN_HIP_CHECK(hipGetLastError());
            SGNN_HIP_CHECK(hipMemcpyAsync(cls_count.data(), d_cls_count.p, sizeof(int32_t) * cls_count.size(), hipMemcpyDeviceToHost, st));
            SGNN_HIP_CHECK(hipStreamSynchronize(st));
        } else {
            p->col_long = p->col;  // pieces index the CSR arrays directly; no permutation
            p->eperm = nullptr;
        }

        std::vector<int32_t> item_begin, item_len, long_pbeg;
        std::vector<std::vector<int32_t>> cls_items(kNumXCD);
        std::vector<uint32_t> item_key;  // partitioned pieces: position of the piece inside its (row, class) run, 16.16
        long_pbeg.push_back(0);
        int rr = 0;  // round-robin class for unpartitioned pieces (balances the eight work lists)
        for (int64_t slot = 0; slot < p->n_long; ++slot) {
            if (!p->partitioned) {
                const int64_t b = h_rowptr[long_rows[slot]], n = h_rowptr[long_rows[slot] + 1] - b;
                const int64_t len = std::max<int64_t>(std::max(p->piece_edges, 64), (n + 255) / 256);
                for (int64_t o = 0; o < n; o += len) {
                    cls_items[rr].push_back((int32_t)item_begin.size());
                    rr = (rr + 1) % kNumXCD;
                    item_begin.push_back((int32_t)(b + o));
                    item_len.push_back((int32_t)std::min<int64_t>(len, n - o));
                }
                long_pbeg.push_back((int32_t)item_begin.size());
                continue;
            }
            int32_t base = long_off[slot];
            for (int c = 0; c < kNumXCD; ++c) {
                const int32_t n = cls_count[slot * kNumXCD + c];
                if (n == 0) continue;
                // at most 32 pieces per (row, class) so that the final sum stays short
                const int32_t len = std::max<int32_t>(p->piece_edges, (n + 31) / 32);
                for (int32_t o = 0; o < n; o += len) {
                    cls_items[c].push_back((int32_t)item_begin.size());
                    item_key.push_back((uint32_t)(((uint64_t)o << 16) / (uint64_t)n));
                    item_begin.push_back(base + o);
                    item_len.push_back(std::min<int32_t>(len, n - o));
                }
                base += n;
            }
            if (item_begin.size() > (size_t)INT32_MAX / 2) return fail(SGNN_ERR_ARG, "too many long-row pieces");
            long_pbeg.push_back((int32_t)item_begin.size());
        }
        p->n_items = (int64_t)item_begin.size();
        // Work order inside a class: by the piece's relative position in its (row, class) run.  Columns
        // ascend along a run, so pieces at the same relative position gather from similar column bands
        // and the workgroups running together on an XCD sweep the dense matrix band by band instead of
        // touching all of it at once (measured: -3 % piece-kernel time on the power-law graph; sorting by
        // the exact first column instead piles the hot low columns into the same moment and costs +5 %).
        if (p->partitioned && env_int("SGNN_SPMM_PIECE_ORDER", 1) >= 1) {
            for (int c = 0; c < kNumXCD; ++c)
                std::stable_sort(cls_items[c].begin(), cls_items[c].end(),
                                 [&](int32_t a, int32_t b) { return item_key[a] < item_key[b]; });
        }
        for (int c = 0; c < kNumXCD; ++c) p->max_cls_items = std::max<int>(p->max_cls_items, (int)cls_items[c].size());
        std::vector<int4> cls_work((size_t)kNumXCD * (size_t)p->max_cls_items, make_int4(0, 0, 0, 0));
        for (int c = 0; c < kNumXCD; ++c)
            for (size_t i = 0; i < cls_items[c].size(); ++i) {
                const int32_t it = cls_items[c][i];
                cls_work[(size_t)c * p->max_cls_items + i] = make_int4(it, item_begin[it], item_len[it], 0);
            }
        if ((rc = upload(&p->long_pbeg, long_pbeg, st)) != SGNN_OK) return rc;
        if ((rc = upload(&p->cls_work, cls_work, st)) != SGNN_OK) return rc;
    }
    SGNN_HIP_CHECK(hipStreamSynchronize(st));  // the host vectors die at return
    // The short-row chunk lists of all three lane-group shapes (a few MB in total): no later call has
    // to build, and therefore allocate, one.
    for (int which = 0; which < 3; ++which)
        if ((rc = build_chunks(p, which, st)) != SGNN_OK) return rc;
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_create(const int64_t *rowptr, const void *col, int col_is_i64, int64_t M, int64_t K,
                                     int64_t nnz, int long_row_threshold, int piece_edges,
                                     sgnn_stream_t stream, sgnn_spmm_plan **plan_out) {
    SGNN_REQUIRE(plan_out != nullptr, "plan_out is null");
    *plan_out = nullptr;
    SGNN_REQUIRE(rowptr != nullptr, "rowptr is null");
    SGNN_REQUIRE(M >= 0 && K >= 0 && nnz >= 0, "negative size (M=%lld K=%lld nnz=%lld)", (long long)M, (long long)K, (long long)nnz);
    SGNN_REQUIRE(M < INT32_MAX && K < INT32_MAX && nnz < INT32_MAX,
                 "M, K and nnz must fit 31 bits (M=%lld K=%lld nnz=%lld)", (long long)M, (long long)K, (long long)nnz);
    SGNN_REQUIRE(nnz == 0 || col != nullptr, "col is null with nnz=%lld", (long long)nnz);
    sgnn_spmm_plan *p = new sgnn_spmm_plan();
    p->M = M; p->K = K; p->nnz = nnz;
    p->long_thresh = long_row_threshold > 0 ? long_row_threshold : env_int("SGNN_SPMM_LONG_THRESHOLD", kDefaultLongThreshold);
    p->piece_edges = piece_edges > 0 ? piece_edges : env_int("SGNN_SPMM_PIECE_EDGES", kDefaultPieceEdges);
    const int rc = plan_create_impl(p, rowptr, col, col_is_i64, (hipStream_t)stream);
    if (rc != SGNN_OK) {
        sgnn_spmm_plan_destroy(p);
        return rc;
    }
    *plan_out = p;
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_info(const sgnn_spmm_plan *p, int64_t info[10]) {
    SGNN_REQUIRE(p != nullptr && info != nullptr, "null argument");
    info[0] = p->M; info[1] = p->K; info[2] = p->nnz; info[3] = p->n_long; info[4] = p->n_items;
    info[5] = p->long_edges; info[6] = p->long_thresh; info[7] = p->piece_edges;
    info[8] = p->partitioned ? 1 : 0; info[9] = (int64_t)(p->top_share * 1e6);
    return SGNN_OK;
}

extern "C" int sgnn_spmm_reference_overwrites(int64_t nnz, int64_t M, int64_t K, int64_t F) {
    if (M <= 0 || K <= 0) return 0;
    const float sparsity = (float)nnz / (float)M / (float)K;
    return (sparsity <= 0.0001f && F > 256) ? 1 : 0;
}

// scratch != null: the call must not allocate.  The piece partials then go to `scratch` (scratch_floats
// floats) instead of the plan's own, growable buffer, and nothing is created on the way.
static int spmm_run(sgnn_spmm_plan *p, const float *val, const DenseSrc &dense, int bits, float *out, int64_t F,
                    int64_t ldo, int accumulate, const float *row_div, hipStream_t st, float *scratch = nullptr,
                    size_t scratch_floats = 0) {
    SGNN_REQUIRE(p != nullptr, "plan is null");
    SGNN_REQUIRE(F > 0 && F < (1 << 24), "feature width F=%lld out of range", (long long)F);
    SGNN_REQUIRE(ldo >= F, "leading dimension smaller than F (ldo=%lld F=%lld)", (long long)ldo, (long long)F);
    if (p->M == 0) return SGNN_OK;
    SGNN_REQUIRE(out != nullptr, "out is null");
    int dev = 0;
    SGNN_HIP_CHECK(hipGetDevice(&dev));
    SGNN_REQUIRE(dev == p->device, "plan was created on device %d, current device is %d", p->device, dev);

    float *partial = p->partial;
    if (scratch != nullptr) {
        const size_t need = (size_t)p->n_items * (size_t)F;
        SGNN_REQUIRE(need <= scratch_floats,
                     "the long rows of this matrix need %zu bytes of partial sums at F=%lld; the scratch of the "
                     "non-allocating entry point holds %zu bytes (use sgnn_spmm_csr_f32)",
                     need * sizeof(float), (long long)F, scratch_floats * sizeof(float));
        partial = scratch;
    } else if (p->n_items > 0) {
        const size_t need = (size_t)p->n_items * (size_t)F;
        if (need > p->partial_floats) {
            // The old buffer may still be read by work queued on another stream: drain first.
            SGNN_HIP_CHECK(hipDeviceSynchronize());
            (void)hipFree(p->partial);
            p->partial = nullptr;
            p->partial_floats = 0;
            SGNN_HIP_CHECK(hipMalloc(&p->partial, need * sizeof(float)));
            p->partial_floats = need;
        }
        partial = p->partial;
    }
    int vec = 1;
    if (bits != 0) {
        vec = 4;  // checked by the caller: F % 4 == 0 and 4-byte aligned packed rows
        SGNN_REQUIRE(ldo % 4 == 0 && aligned(out, 16), "out must be 16-byte aligned with ldo %% 4 == 0 for the fused path");
    } else if (F % 4 == 0 && dense.ldx % 4 == 0 && ldo % 4 == 0 && aligned(dense.x, 16) && aligned(out, 16)) {
        vec = 4;
    } else if (F % 2 == 0 && dense.ldx % 2 == 0 && ldo % 2 == 0 && aligned(dense.x, 8) && aligned(out, 8)) {
        vec = 2;
    }
    const int nvec = (int)(F / vec);
    const int gw = group_width(nvec);
    const int which = gw == 8 ? 0 : gw == 16 ? 1 : 2;
    SGNN_REQUIRE(p->n_chunks[which] >= 0, "plan has no chunk list for this feature width (plan creation failed?)");
    ShortArgs a{p->rowptr, p->col, val, dense, out, p->chunks[which], (int)p->n_chunks[which], p->empty_rows,
                (int)p->n_empty, (int)F, ldo, accumulate, row_div};
    if (scratch == nullptr && p->side == nullptr && p->n_long > 0 && env_int("SGNN_SPMM_OVERLAP", 0) != 0) {
        SGNN_HIP_CHECK(hipStreamCreateWithFlags(&p->side, hipStreamNonBlocking));  // default priority
        SGNN_HIP_CHECK(hipEventCreateWithFlags(&p->ev_fork, hipEventDisableTiming));
        SGNN_HIP_CHECK(hipEventCreateWithFlags(&p->ev_join, hipEventDisableTiming));
    }
    PieceArgs s{p->col_long, p->eperm, val, partial, p->cls_work, p->max_cls_items, (int)F,
                scratch == nullptr ? p->side : nullptr, p->ev_fork, p->ev_join};
    if (val != nullptr && val == p->bound_val && p->val_long != nullptr) {
        s.eperm = nullptr;   // values already sit in regrouped order: contiguous reads, no indirection
        s.val = p->val_long;
    }
    FinalArgs f{p->long_rows, p->long_pbeg, partial, out, (int)p->n_long, (int)F, ldo, accumulate, row_div};
    if (bits != 0) {
        const int fmt = bits + (dense.params.bf16 ? kBf16Params : 0) + (dense.eslot_csr ? kEdgeSlots : 0);
        switch (fmt) {
#define SGNN_DQ(FMT) case FMT: dispatch_shape_dq<FMT>(nvec, a, s, f, st); break
            SGNN_DQ(8); SGNN_DQ(4); SGNN_DQ(2);
            SGNN_DQ(8 + kBf16Params); SGNN_DQ(4 + kBf16Params); SGNN_DQ(2 + kBf16Params);
            SGNN_DQ(8 + kEdgeSlots); SGNN_DQ(4 + kEdgeSlots); SGNN_DQ(2 + kEdgeSlots);
            SGNN_DQ(8 + kBf16Params + kEdgeSlots); SGNN_DQ(4 + kBf16Params + kEdgeSlots); SGNN_DQ(2 + kBf16Params + kEdgeSlots);
#undef SGNN_DQ
            default: return fail(SGNN_ERR_ARG, "unsupported quantized format %d", fmt);
        }
    }
    else if (vec == 4) dispatch_shape<4>(nvec, a, s, f, st);
    else if (vec == 2) dispatch_shape<2>(nvec, a, s, f, st);
    else dispatch_shape<1>(nvec, a, s, f, st);
    SGNN_HIP_CHECK(hipGetLastError());
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_bind_values(sgnn_spmm_plan *p, const float *val, sgnn_stream_t stream) {
    SGNN_REQUIRE(p != nullptr, "plan is null");
    p->bound_val = nullptr;
    if (val == nullptr || !p->partitioned || p->long_edges == 0) return SGNN_OK;  // nothing to regroup
    if (p->val_long == nullptr) SGNN_HIP_CHECK(hipMalloc(&p->val_long, sizeof(float) * (size_t)p->long_edges));
    const int64_t nb = (p->long_edges + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(permute_values_kernel, dim3((uint32_t)nb), dim3(kBlock), 0, (hipStream_t)stream, val, p->eperm,
                       p->val_long, p->long_edges);
    SGNN_HIP_CHECK(hipGetLastError());
    p->bound_val = val;
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_bind_row_slots(sgnn_spmm_plan *p, const int32_t *row_slot, sgnn_stream_t stream) {
    SGNN_REQUIRE(p != nullptr, "plan is null");
    p->bound_slots = nullptr;
    if (row_slot == nullptr || p->nnz == 0) return SGNN_OK;
    hipStream_t st = (hipStream_t)stream;
    if (p->eslot_csr == nullptr) SGNN_HIP_CHECK(hipMalloc(&p->eslot_csr, sizeof(int32_t) * (size_t)p->nnz));
    hipLaunchKernelGGL(translate_columns_kernel, dim3((uint32_t)((p->nnz + kBlock - 1) / kBlock)), dim3(kBlock), 0, st, p->col,
                       row_slot, p->eslot_csr, p->nnz);
    if (p->partitioned && p->long_edges > 0) {
        if (p->eslot_long == nullptr) SGNN_HIP_CHECK(hipMalloc(&p->eslot_long, sizeof(int32_t) * (size_t)p->long_edges));
        hipLaunchKernelGGL(translate_columns_kernel, dim3((uint32_t)((p->long_edges + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                           st, p->col_long, row_slot, p->eslot_long, p->long_edges);
    }
    SGNN_HIP_CHECK(hipGetLastError());
    p->bound_slots = row_slot;
    return SGNN_OK;
}

extern "C" int sgnn_spmm_csr_f32(sgnn_spmm_plan *p, const float *val, const float *x, float *out, int64_t F,
                                 int64_t ldx, int64_t ldo, int accumulate, const float *row_div,
                                 sgnn_stream_t stream) {
    SGNN_REQUIRE(p != nullptr, "plan is null");
    SGNN_REQUIRE(ldx >= F, "leading dimension smaller than F (ldx=%lld F=%lld)", (long long)ldx, (long long)F);
    SGNN_REQUIRE(x != nullptr || p->nnz == 0 || p->M == 0, "x is null");
    DenseSrc d{x, ldx, nullptr, ParamBuf{nullptr, 0}, nullptr, nullptr, 0};
    return spmm_run(p, val, d, 0, out, F, ldo, accumulate, row_div, (hipStream_t)stream);
}

extern "C" int sgnn_spmm_csr_f32_noalloc(sgnn_spmm_plan *p, const float *val, const float *x, float *out, int64_t F,
                                         int64_t ldx, int64_t ldo, int accumulate, const float *row_div,
                                         sgnn_stream_t stream) {
    SGNN_REQUIRE(p != nullptr, "plan is null");
    SGNN_REQUIRE(ldx >= F, "leading dimension smaller than F (ldx=%lld F=%lld)", (long long)ldx, (long long)F);
    SGNN_REQUIRE(x != nullptr || p->nnz == 0 || p->M == 0, "x is null");
    float *scratch = nullptr;
    const int rc = scratch_for_current_device(&scratch);
    if (rc != SGNN_OK) return rc;
    DenseSrc d{x, ldx, nullptr, ParamBuf{nullptr, 0}, nullptr, nullptr, 0};
    return spmm_run(p, val, d, 0, out, F, ldo, accumulate, row_div, (hipStream_t)stream, scratch, kScratchFloats);
}

static int spmm_dq_impl(sgnn_spmm_plan *p, const float *val, const uint8_t *q, const void *params, int params_bf16,
                       const int32_t *row_slot, int bits, float *out, int64_t F, int64_t ldo, int accumulate,
                       const float *row_div, sgnn_stream_t stream) {
    SGNN_REQUIRE(p != nullptr, "plan is null");
    SGNN_REQUIRE(bits == 8 || bits == 4 || bits == 2, "bits=%d, expected 8, 4 or 2", bits);
    SGNN_REQUIRE(params_bf16 == 0 || params_bf16 == 1, "params_bf16=%d, expected 0 or 1", params_bf16);
    SGNN_REQUIRE(F % 4 == 0, "the fused path needs F %% 4 == 0 (F=%lld): dequantize, then call sgnn_spmm_csr_f32", (long long)F);
    SGNN_REQUIRE((q != nullptr && params != nullptr) || p->nnz == 0 || p->M == 0, "q / params is null");
    SGNN_REQUIRE(aligned(q, 4) && aligned(params, params_bf16 ? 4 : 8), "q must be 4-byte and params %d-byte aligned",
                 params_bf16 ? 4 : 8);
    DenseSrc d{nullptr, 0, q, ParamBuf{const_cast<void *>(params), params_bf16}, nullptr, nullptr, (int)F};
    if (row_slot != nullptr && p->nnz > 0) {
        // Every edge carries its slot next to its column, so a gather never looks the table up.  The
        // per-edge stream is built the first time a table is seen and kept while the same pointer
        // comes back (the table is taken to be constant; sgnn_spmm_plan_bind_row_slots refreshes it).
        if (row_slot != p->bound_slots) {
            const int rc = sgnn_spmm_plan_bind_row_slots(p, row_slot, stream);
            if (rc != SGNN_OK) return rc;
        }
        d.eslot_csr = p->eslot_csr;
        d.eslot_long = p->eslot_long ? p->eslot_long : p->eslot_csr;  // unregrouped long rows index the CSR arrays
    }
    return spmm_run(p, val, d, bits, out, F, ldo, accumulate, row_div, (hipStream_t)stream);
}

extern "C" int sgnn_spmm_csr_dq_f32(sgnn_spmm_plan *p, const float *val, const uint8_t *q, const float *params,
                                    const int32_t *row_slot, int bits, float *out, int64_t F, int64_t ldo,
                                    int accumulate, const float *row_div, sgnn_stream_t stream) {
    return spmm_dq_impl(p, val, q, params, 0, row_slot, bits, out, F, ldo, accumulate, row_div, stream);
}

extern "C" int sgnn_spmm_csr_dq_wire_f32(sgnn_spmm_plan *p, const float *val, const uint8_t *q, const void *params,
                                         int params_bf16, const int32_t *row_slot, int bits, float *out, int64_t F,
                                         int64_t ldo, int accumulate, const float *row_div, sgnn_stream_t stream) {
    return spmm_dq_impl(p, val, q, params, params_bf16, row_slot, bits, out, F, ldo, accumulate, row_div, stream);
}
