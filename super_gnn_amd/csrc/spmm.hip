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
#include <list>
#include <memory>
#include <mutex>
#include <vector>

#include "common.hpp"

namespace sgnn {

constexpr int kBlock = 256;
constexpr int kDefaultLongThreshold = 128;  // rows with more edges go to the class-partitioned piece path
constexpr int kChunkGroupsWanted = 16384;
constexpr int kDefaultPieceEdges = 96;      // minimum edges per piece of a long row (a class run shorter than this stays one piece)
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
            // (ordinary loads: marking the code rows non-temporal, to keep the (zero_point, scale) table in the L2, cut the
            // fetched bytes by 4 % and cost 10 % of the kernel's time: rows that share a packed row hit in cache)
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
        // all codes of the word moved to the bottom of their bytes with one shift and one mask; each then
        // converts with a single byte-to-float instruction
        uint32_t wm = 0;
        if constexpr (BITS != 0) wm = (r.w[v] >> r.shift) & (((1u << (BITS & 15)) - 1u) * 0x01010101u);
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            float xv;
            if constexpr (BITS == 0) {
                xv = r.f[v][k];
            } else {
                xv = fmaf((float)((wm >> (8 * k)) & 0xffu), r.sc, r.zp);
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
        return (uint32_t)(m >> base) & (uint32_t)((1ull << G) - 1ull);
    }
}

// Rows per chunk: each of the first nr+1 lanes of the group holds one rowptr entry.
__host__ __device__ constexpr int chunk_row_limit(int G) { return (G < 32 ? G : 32) - 1; }

// One lane group walks one chunk of consecutive rows for the feature columns [f_lo, f_hi) (both multiples
// of VEC).  RP is the row-pointer type: the caller's int64 array, or the 32-bit per-band row pointers of a
// band schedule.
template <int VEC, int G, int NV, int BITS, typename RP, int UF = 0>
__device__ __forceinline__ void short_chunk_body(
    const RP *__restrict__ rowptr, const int32_t *__restrict__ col, const float *__restrict__ val,
    const DenseSrc &dense, float *__restrict__ out, int4 ch, int f_lo, int f_hi,
    int64_t ldo, int accumulate, const float *__restrict__ row_div, int lig) {
    constexpr int TILE = G * VEC * NV;
    // gathers in flight per lane group: 6 keeps the kernel at 75 VGPRs (6 waves per SIMD); 8 costs 83 (5 waves)
    constexpr int U = UF > 0 ? UF : NV == 1 ? 6 : unroll_of(NV);
    const int F = f_hi;
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

    for (int f0 = f_lo; f0 < F; f0 += TILE) {
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
        if (f0 > f_lo && lig < E) {  // a later feature tile walks the chunk's edges again
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

template <int VEC, int G, int NV, int BITS>
__global__ __launch_bounds__(kBlock) void spmm_short_kernel(
    const int64_t *__restrict__ rowptr, const int32_t *__restrict__ col, const float *__restrict__ val,
    const DenseSrc dense, float *__restrict__ out, const int4 *__restrict__ chunks, int n_chunks, int F,
    int64_t ldo, int accumulate, const float *__restrict__ row_div, uint32_t nblocks) {
    constexpr int GPB = kBlock / G;
    const uint32_t lb = xcd_contiguous_block(blockIdx.x, nblocks);
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int ci = (int)lb * GPB + gid;
    if (ci >= n_chunks) return;
    // A chunk record is (first row, row count, first edge, edge count): the column/weight loads
    // depend on it alone and are issued before the row pointers come back.
    short_chunk_body<VEC, G, NV, BITS, int64_t>(rowptr, col, val, dense, out, chunks[ci], 0, F, ldo, accumulate, row_div, lig);
}

// ------------------------------------------------------------------------------------------------
// Band schedule (dense-degree matrices whose dense operand does not fit the L2 caches).
//
// The column space is cut into bands of band_cols columns; band b of the matrix is a CSR matrix of its
// own (32-bit row pointers, edges stored band-major), and the product is a sequence of launches, one per
// band, each accumulating its band's contribution onto `out` in place.  Inside one launch the eight XCDs
// split the FEATURE axis: workgroup i runs on XCD i % 8 and only touches feature slice (i % 8) % n_slices,
// so an XCD's L2 has to hold band_cols x (slice bytes) of the dense operand -- sized to fit -- and every
// gather after the first touch of a dense row slice is an L2 hit.  All workgroups of a launch work on the
// same band (the kernel boundary is the synchronisation), the accumulators travel through `out` between
// bands (read-modify-write of one row slice per band, a stream), and a row's edges are still summed in CSR
// order with one fma per edge starting from the old value: with column-sorted rows the result is the
// reference's, bit for bit, whatever the row length.
// ------------------------------------------------------------------------------------------------
// Upper limits of a chunk of the band kernel: rows, and staged (row offset, val) pairs.  What a launch uses is
// decided from the lane-group shape and the LDS it leaves (band_chunk_caps).
#ifndef SGNN_BAND_ROWS
#define SGNN_BAND_ROWS 16
#endif
#ifndef SGNN_BAND_EDGES
#define SGNN_BAND_EDGES 448
#endif
#ifndef SGNN_BAND_U
#define SGNN_BAND_U 8
#endif
constexpr int kBandRows = SGNN_BAND_ROWS;
constexpr int kBandEdges = SGNN_BAND_EDGES;
// With edge values a chunk keeps twice the words per edge in flight and in LDS: lower limits keep the kernel's
// registers (all of a chunk's HBM loads are in flight at once) within two waves per SIMD.
constexpr int kBandRowsWeighted = kBandRows < 12 ? kBandRows : 12;
constexpr int kBandEdgesWeighted = kBandEdges < 320 ? kBandEdges : 320;
constexpr int kBandWindow = SGNN_BAND_U;  // gathers in flight per lane group
constexpr int kBandPad = 16;              // staging entries past the last pair (>= the gather window)
#ifndef SGNN_BAND_BLOCK
#define SGNN_BAND_BLOCK 256
#endif
constexpr int kBandBlock = SGNN_BAND_BLOCK;  // threads per workgroup of the band kernel
static_assert(kBandWindow <= kBandPad, "gather window wider than the staging pad");
// LDS floats of one lane group: the output tile, the staged row offsets of the edges and, for a weighted matrix, their values.
__host__ __device__ constexpr int band_group_floats(int tile_stride, int rows_cap, int edge_cap, bool weighted) {
    return rows_cap * tile_stride + (weighted ? 2 : 1) * (edge_cap + kBandPad);
}

// The dense operand restaged for the band kernel: xs[slice][column][slice_pad floats], slice_pad a multiple of
// 16 floats.  Every row of a slice then starts on a 64-byte boundary, a group of slice_pad / 4 lanes reads it
// with aligned 128-bit loads, and four neighbouring lanes cover exactly one 64-byte sector.  That matters
// because the L1 looks up one sector per cycle: gathered straight out of rows of 602 floats (2408 bytes, only
// 8-byte aligned) a wave instruction of three 304-byte slices touched 23 sectors and held the address path for
// 36 cycles; restaged it touches 15.  One pass over X per product (about 2 % of the product's time).
// Floats past the end of a slice or of the row are zero.
__global__ __launch_bounds__(kBlock) void band_restage_kernel(const float *__restrict__ x, int64_t ldx, float *__restrict__ xs,
                                                               int64_t K, int F, int slice_floats, int slice_pad, int n_slices) {
    const int vpr = slice_pad / 4;  // float4 per restaged row
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= (int64_t)n_slices * K * vpr) return;
    const int v = (int)(i % vpr);
    const int64_t sc = i / vpr;
    const int64_t c = sc % K;
    const int sl = (int)(sc / K);
    const int f0 = sl * slice_floats + 4 * v;
    const float *row = x + c * ldx;
    float r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = (4 * v + e < slice_floats && f0 + e < F) ? row[f0 + e] : 0.0f;
    reinterpret_cast<float4 *>(xs)[i] = make_float4(r[0], r[1], r[2], r[3]);
}

// Old / new values of `out` for one lane: nf (0..4) floats at p.  EVEN: rows start on 8-byte boundaries and F is
// even, so nf is 4 or 2 and 128-bit accesses that need only 8-byte alignment are used (a lane with two floats
// loads the four floats that END at p + 2 and keeps the upper two, so no access crosses the end of its row).
template <bool EVEN>
__device__ __forceinline__ void out_load(float (&r)[4], const float *p, int nf) {
    if constexpr (EVEN) {
        typedef float f4 __attribute__((ext_vector_type(4), aligned(8)));
        const bool half = nf == 2;
        const f4 v = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(p - (half ? 2 : 0)));
        r[0] = half ? v.z : v.x;
        r[1] = half ? v.w : v.y;
        r[2] = v.z;
        r[3] = v.w;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = e < nf ? __builtin_nontemporal_load(p + e) : 0.0f;
    }
}
template <bool EVEN>
__device__ __forceinline__ void out_store(float *p, const float (&r)[4], int nf) {
    if constexpr (EVEN) {
        typedef float f4 __attribute__((ext_vector_type(4), aligned(8)));
        typedef float f2 __attribute__((ext_vector_type(2), aligned(8)));
        if (nf == 2) {
            f2 v = {r[0], r[1]};
            __builtin_nontemporal_store(v, reinterpret_cast<f2 *>(p));
        } else {
            f4 v = {r[0], r[1], r[2], r[3]};
            __builtin_nontemporal_store(v, reinterpret_cast<f4 *>(p));
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < nf) __builtin_nontemporal_store(r[e], p + e);
    }
}

// A chunk is a run of consecutive rows of one band: at most rows_cap rows and edge_cap edges (a single row may
// have more).  Its record is four int4: (first row, rows, first edge, edges), then 24 16-bit edge offsets
// relative to the first edge: entry i belongs to row i of the chunk, entries from `rows` on hold the number of
// edges (a one-row chunk may have more than 65535 edges: its two offsets are taken from the header instead).
constexpr int kBandOffsets = 24;
static_assert(kBandEdges <= 65535 && kBandRows < kBandOffsets && kBandRows <= 16, "row offsets of a chunk are 16-bit, 24 per record");

// One lane group per chunk.  A group is
// G = slice_pad / 4 lanes (any value from 16 to 64, not only powers of two), one float4 of the restaged slice
// each, and a wavefront carries 64 / G groups: a vector memory instruction occupies a CU's address path for as
// long whether 20 or 64 of its lanes are active, so what a gather costs is decided by how many gathers share one
// instruction.  At F = 602 a slice is 76 floats padded to 80, G = 20, and three gathers travel together.
// Three phases per chunk:
//   1. everything that comes from HBM is requested in ONE batch right after the chunk's record has arrived, so a
//      chunk pays two memory latencies in all: the old `out` values of all its rows for this feature slice go to
//      LDS (the output tile of the chunk), and so do its (row offset, val) pairs;
//   2. the gather loop: a rolling window of kBandWindow gathers of dense-row slices, all of them L2 hits, one fma
//      per edge in CSR order; a row boundary swaps the accumulator through the LDS tile.  Nothing slow sits in
//      the vector memory queue during this phase: loads return in order, and one HBM-latency load between two
//      gathers would stall every gather behind it;
//   3. the tile rows that received edges are written back.
// A tile column belongs to one lane and a group to one wavefront: the kernel has no workgroup barrier.
template <bool EVEN, bool OFF32, bool WEIGHTED>
__global__ __launch_bounds__(kBandBlock) __attribute__((amdgpu_waves_per_eu(2))) void spmm_band_kernel(
    const int32_t *__restrict__ col_bm, const float *__restrict__ val_bm, const float *__restrict__ xs, int64_t K,
    float *__restrict__ out, const int4 *__restrict__ chunks, int n_chunks, int F, int64_t ldo, int slice_floats,
    int slice_pad, int n_slices, int G, int rows_cap, int edge_cap) {
    extern __shared__ float band_lds[];
    constexpr int U = kBandWindow;
    constexpr int kRows = WEIGHTED ? kBandRowsWeighted : kBandRows;
    constexpr int kKeyRounds = ((WEIGHTED ? kBandEdgesWeighted : kBandEdges) + kBandPad + 63) / 64;
    const int tile_stride = G * 4;
    const int gpw = 64 / G;                       // groups per wavefront
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int gsub = lane / G, lig = lane - gsub * G;
    const int gbase = gsub * G;                   // first lane of this group inside the wavefront
    const int gid = wave * gpw + gsub;            // group inside the workgroup
    const int xcd = blockIdx.x % kNumXCD;
    const int slice = xcd % n_slices, rg = xcd / n_slices, n_rg = kNumXCD / n_slices;
    const int ci = ((int)(blockIdx.x / kNumXCD) * n_rg + rg) * ((kBandBlock / 64) * gpw) + gid;
    const int f_lo = slice * slice_floats;        // first feature column of this slice
    const int vpr = slice_pad / 4;                // float4 per restaged row
    const bool valid = gsub < gpw && ci < n_chunks && f_lo < F;
    float *tile = band_lds + (size_t)(gsub < gpw ? gid : 0) * band_group_floats(tile_stride, rows_cap, edge_cap, WEIGHTED);
    int *lkey = reinterpret_cast<int *>(tile + rows_cap * tile_stride);
    float *lval = reinterpret_cast<float *>(lkey + edge_cap + kBandPad);   // only there (and only used) for a weighted matrix
    const float *xslice = xs + (int64_t)slice * K * slice_pad;

    int4 ch = make_int4(0, 0, 0, 0);
    int rel16 = 0;
    if (valid) {
        const int4 *rec = chunks + 4 * (int64_t)ci;
        ch = rec[0];
        rel16 = reinterpret_cast<const uint16_t *>(rec + 1)[lig < kBandOffsets - 1 ? lig : kBandOffsets - 1];
    }
    const int rb = ch.x, nr = ch.y, E = ch.w;  // rows rb .. rb+nr-1 (first and last non-empty in this band), E edges
    const int64_t B = ch.z;
    const int32_t *colp = col_bm + B;
    const float *valp = WEIGHTED ? val_bm + B : nullptr;
    // Lane i of the group holds the offset of row rb+i relative to the chunk's first edge (lanes >= nr hold the end).
    int rel = 0;
    if (valid) rel = nr == 1 ? (lig == 0 ? 0 : E) : rel16;
    const int rel_next = __shfl(rel, lane + 1 < 64 ? lane + 1 : 63);
    const unsigned long long bal = __ballot(valid && lig < nr && rel_next > rel);
    const uint32_t mask = (uint32_t)(bal >> gbase) & ((1u << rows_cap) - 1u);  // bit i: row rb+i has edges in this band

    for (int t0 = 0; t0 < vpr; t0 += G) {             // slices wider than 64 float4 are walked in tiles
        const int vi = t0 + lig;                      // this lane's float4 of the slice
        const int off = f_lo + 4 * vi;                // its first feature column
        int nf = slice_floats - 4 * vi < F - off ? slice_floats - 4 * vi : F - off;
        nf = !valid || vi >= vpr || nf < 0 ? 0 : nf > 4 ? 4 : nf;  // floats of `out` this lane owns (EVEN: 0, 2 or 4)
        const bool act = nf > 0;
        // This lane's column of the tile.  Lanes that own nothing point at column 0 and never write (a write
        // through "their" offset would land in the next row or in the staged pairs).
        float *tcol = tile + (act ? lig * 4 : 0);
        // ---- phase 1: one batch of loads: old out values of the chunk's rows, the first edge_cap pairs -------------
        const int se0 = E < edge_cap ? E : edge_cap;
        {
            float old[kRows][4];
            if (act) {
#pragma unroll
                for (int k = 0; k < kRows; ++k) {
                    const int r = k < nr ? k : nr - 1;
                    out_load<EVEN>(old[k], out + (int64_t)(rb + r) * ldo + off, nf);
                }
            }
            // Four pairs per lane and load.  The window below gathers up to U pairs past the chunk's last one (never
            // consumed): those are the next edges of the band-major arrays, valid columns all, and the arrays end
            // in kBandPad + 4 zero entries.
            int c[kKeyRounds][4];
            float w[kKeyRounds][4];
            if (valid) {
#pragma unroll
                for (int q = 0; q < kKeyRounds; ++q) {
                    const int i = 4 * lig + 4 * G * q;
#pragma unroll
                    for (int e = 0; e < 4; ++e) { c[q][e] = 0; w[q][e] = 1.0f; }
                    if (i < se0 + U) {
                        typedef int i4 __attribute__((ext_vector_type(4), aligned(4)));
                        typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
                        const i4 cv = __builtin_nontemporal_load(reinterpret_cast<const i4 *>(colp + i));
                        c[q][0] = cv.x; c[q][1] = cv.y; c[q][2] = cv.z; c[q][3] = cv.w;
                        if constexpr (WEIGHTED) {
                            const f4 wv4 = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(valp + i));
                            w[q][0] = wv4.x; w[q][1] = wv4.y; w[q][2] = wv4.z; w[q][3] = wv4.w;
                        }
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // the previous tile's LDS reads are done
            if (act) {
#pragma unroll
                for (int k = 0; k < kRows; ++k) {
                    if (k < nr) *reinterpret_cast<float4 *>(tcol + k * tile_stride) = make_float4(old[k][0], old[k][1], old[k][2], old[k][3]);
                }
            }
            if (valid) {
#pragma unroll
                for (int q = 0; q < kKeyRounds; ++q) {
                    const int i = 4 * lig + 4 * G * q;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (i + e < se0 + U) {
                            lkey[i + e] = OFF32 ? (int)((uint32_t)c[q][e] * (uint32_t)slice_pad * 4u) : c[q][e];
                            if constexpr (WEIGHTED) lval[i + e] = w[q][e];
                        }
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        }
        // ---- phase 2: gathers ------------------------------------------------------------------------------
        if (valid) {
            // every lane of the group loads: the restaged rows are padded, so a lane that owns nothing reads zeros
            const float *xlane = xslice + 4 * (vi < vpr ? vi : t0);
            int cur = __builtin_ctz(mask);
            int cur_end = __shfl(rel, gbase + cur + 1);
            float4 acc = *reinterpret_cast<const float4 *>(tcol + cur * tile_stride);
            // The chunk's (row offset, val) pairs are staged in LDS, edge_cap at a time (more than one round only
            // for a row longer than that).  A group lives inside one wavefront, whose LDS operations execute in
            // order: a wavefront-level fence is all the staging needs.
            for (int seg = 0; seg < E; seg += edge_cap) {
                const int se = E - seg < edge_cap ? E - seg : edge_cap;
                if (seg > 0) {   // a later round of a row longer than edge_cap: stage its pairs now
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                    for (int i = 4 * lig; i < se + U; i += 4 * G) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (i + e < se + U) {
                                const int cc = __builtin_nontemporal_load(colp + seg + i + e);
                                lkey[i + e] = OFF32 ? (int)((uint32_t)cc * (uint32_t)slice_pad * 4u) : cc;
                                if constexpr (WEIGHTED) lval[i + e] = __builtin_nontemporal_load(valp + seg + i + e);
                            }
                        }
                    }
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                }
                // A rolling window of U gathers: slot u is refilled with the edge U further on as soon as its value
                // has been consumed, so U - 1 gathers are in flight at all times (loads return in order).
                float4 xv[U];
                float wv[U];
                auto gather = [&](int u, int key) {
                    const float *p;
                    if constexpr (OFF32) p = reinterpret_cast<const float *>(reinterpret_cast<const char *>(xlane) + (uint32_t)key);
                    else p = xlane + (int64_t)key * slice_pad;
                    xv[u] = *reinterpret_cast<const float4 *>(p);
                };
                auto consume = [&](int edge, int u) {
                    if (edge == cur_end) {  // first edge of the next non-empty row: swap accumulators through the tile
                        if (act) *reinterpret_cast<float4 *>(tcol + cur * tile_stride) = acc;
                        const uint32_t rest = mask & ~((2u << cur) - 1u);
                        cur = __builtin_ctz(rest);
                        cur_end = __shfl(rel, gbase + cur + 1);
                        acc = *reinterpret_cast<const float4 *>(tcol + cur * tile_stride);
                    }
                    const float wu = WEIGHTED ? wv[u] : 1.0f;   // fma(1, x, acc) is the chain the reference computes with unit weights
                    acc.x = fmaf(wu, xv[u].x, acc.x);
                    acc.y = fmaf(wu, xv[u].y, acc.y);
                    acc.z = fmaf(wu, xv[u].z, acc.z);
                    acc.w = fmaf(wu, xv[u].w, acc.w);
                };
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if constexpr (WEIGHTED) wv[u] = lval[u];
                    gather(u, lkey[u]);
                }
                int base = 0;
                // full rounds: every slot holds a real edge and is refilled unconditionally (no branch around a load:
                // the compiler then counts outstanding loads exactly instead of draining the queue at every join)
                for (; base + U < se; base += U) {
                    const int *lk = lkey + base + U;
                    const float *lv = lval + base + U;
                    int kn[U];
                    float wn[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) {  // the next round's pairs, read from LDS ahead of their use
                        kn[u] = lk[u];
                        if constexpr (WEIGHTED) wn[u] = lv[u];
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        consume(seg + base + u, u);
                        if constexpr (WEIGHTED) wv[u] = wn[u];
                        gather(u, kn[u]);
                    }
                }
                // last round: the window drains
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (base + u < se) consume(seg + base + u, u);
                }
            }
            if (act) *reinterpret_cast<float4 *>(tcol + cur * tile_stride) = acc;
        }
        // ---- phase 3: rows that received edges go back to out ---------------------------------------------
        if (act) {
            uint32_t m = mask;
            while (m) {
                const int r = __builtin_ctz(m);
                m &= m - 1;
                const float4 t = *reinterpret_cast<const float4 *>(tcol + r * tile_stride);
                const float v[4] = {t.x, t.y, t.z, t.w};
                out_store<EVEN>(out + (int64_t)(rb + r) * ldo + off, v, nf);
            }
        }
    }
}

// out[r, 0..F) = 0 (overwrite mode of the band schedule) or out[r, :] /= row_div[r] (mean epilogue), for all rows.
template <int VEC, bool DIV>
__global__ __launch_bounds__(kBlock) void rows_fill_or_divide_kernel(float *__restrict__ out, int64_t M, int F, int64_t ldo,
                                                                     const float *__restrict__ row_div) {
    const int nvec = F / VEC;
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= M * nvec) return;
    const int64_t r = i / nvec;
    float *p = out + r * ldo + (i - r * nvec) * VEC;
    float a[VEC];
    if constexpr (DIV) {
        vec_load_nt<VEC>(a, p);
        const float d = row_div[r];
#pragma unroll
        for (int k = 0; k < VEC; ++k) a[k] = a[k] / d;
    } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) a[k] = 0.0f;
    }
    vec_store_nt<VEC>(p, a);
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
            if (act[v]) vec_store_nt<VEC>(partial + (int64_t)item * F + off[v], acc[v]);
    }
}

// ------------------------------------------------------------------------------------------------
// Long rows the other way, for comparison only (SGNN_SPMM_HUB_LDS=1): ONE WORKGROUP PER LONG ROW.  The row's
// edges, in CSR order, are cut into eight contiguous parts shared out to the lane groups; the partial sums
// meet in LDS and are added in part order onto the old output row.  No plan-time regrouping, no partial buffer,
// no second kernel -- and a 95,000-edge row is one workgroup's work while every XCD gathers every popular
// dense row (on the 2.45 M-node power-law graph the long rows take 4.2 ms this way against 1.9 ms as pieces by
// column class plus the final sum: 5.5 against 3.2 ms per step).
// ------------------------------------------------------------------------------------------------
template <int VEC, int G, int NV>
__global__ __launch_bounds__(kBlock) void spmm_hubrow_lds_kernel(
    const int64_t *__restrict__ rowptr, const int32_t *__restrict__ col, const float *__restrict__ val, const DenseSrc dense,
    const int32_t *__restrict__ long_rows, float *__restrict__ out, int F, int64_t ldo, int accumulate,
    const float *__restrict__ row_div) {
    constexpr int GPB = kBlock / G;
    constexpr int TILE = G * VEC * NV;
    constexpr int kParts = 8;  // a row is always cut the same way, whatever the lane-group shape: same sums for every layout of X
    __shared__ float red[kParts][TILE];
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int64_t row = long_rows[blockIdx.x];
    const int64_t b = rowptr[row];
    const int n = (int)(rowptr[row + 1] - b);
    const int part = (n + kParts - 1) / kParts;
    float *orow = out + row * ldo;
    const float div = row_div ? row_div[row] : 1.0f;
    for (int f0 = 0; f0 < F; f0 += TILE) {
        for (int pp = gid; pp < kParts; pp += GPB) {
            const int my_off = pp * part;
            const int my_len = n - my_off < 0 ? 0 : n - my_off < part ? n - my_off : part;
            int off_ld[NV];
            bool act_ld[NV];
            float acc[NV][VEC];
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const int off = f0 + (v * G + lig) * VEC;
                off_ld[v] = off < F ? off : f0;
                act_ld[v] = true;
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[v][k] = 0.0f;
            }
            if (my_len > 0)
                gather_piece<VEC, G, NV, 0, false>(acc, col + b + my_off, nullptr, val ? val + b + my_off : nullptr, nullptr, my_len,
                                                   dense, off_ld, act_ld, lig);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) red[pp][(v * G + lig) * VEC + k] = acc[v][k];
            }
        }
        __syncthreads();
        for (int e = threadIdx.x; e < TILE && f0 + e < F; e += kBlock) {
            float sum = accumulate ? orow[f0 + e] : 0.0f;
#pragma unroll
            for (int g = 0; g < kParts; ++g) sum += red[g][e];
            orow[f0 + e] = row_div ? sum / div : sum;
        }
        __syncthreads();
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
                    vec_load_nt<VEC>(p[u], partial + (int64_t)si * F + off);
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
// Band schedule, plan-time kernels.
// ------------------------------------------------------------------------------------------------
// flag = 1 if some row's columns are not in non-decreasing order (16 lanes per row).
__global__ __launch_bounds__(kBlock) void check_rows_sorted_kernel(const int64_t *__restrict__ rowptr,
                                                                   const int32_t *__restrict__ col, int64_t M,
                                                                   int *__restrict__ flag) {
    const int64_t r = (int64_t)blockIdx.x * (kBlock / 16) + threadIdx.x / 16;
    if (r >= M) return;
    const int64_t b = rowptr[r], e = rowptr[r + 1];
    bool bad = false;
    for (int64_t i = b + (threadIdx.x % 16); i + 1 < e; i += 16) bad |= col[i] > col[i + 1];
    if (bad) atomicOr(flag, 1);
}

// lo[r, b] = index of row r's first edge whose column is >= b * band_cols (b = 0 .. n_bands), and the
// per-band edge counts transposed, cnt_t[b, r] = lo[r, b+1] - lo[r, b].  Rows are column-sorted.
__global__ __launch_bounds__(kBlock) void band_bounds_kernel(const int64_t *__restrict__ rowptr,
                                                             const int32_t *__restrict__ col, int64_t M, int n_bands,
                                                             int band_cols, int32_t *__restrict__ lo) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= M * (n_bands + 1)) return;
    const int64_t r = i / (n_bands + 1);
    const int b = (int)(i - r * (n_bands + 1));
    int64_t a = rowptr[r], z = rowptr[r + 1];
    if (b == n_bands) a = z;
    else if (b > 0) {
        const int64_t key = (int64_t)b * band_cols;
        while (a < z) {
            const int64_t mid = (a + z) >> 1;
            if (col[mid] < key) a = mid + 1; else z = mid;
        }
    }
    lo[i] = (int32_t)a;
}
__global__ __launch_bounds__(kBlock) void band_counts_kernel(const int32_t *__restrict__ lo, int64_t M, int n_bands,
                                                             int32_t *__restrict__ cnt_t) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= M * n_bands) return;
    const int b = (int)(i / M);
    const int64_t r = i - (int64_t)b * M;
    cnt_t[i] = lo[r * (n_bands + 1) + b + 1] - lo[r * (n_bands + 1) + b];
}

// Copies the edges into band-major order: band b's edges of row r go to rowptr_bm[b, r] ... in CSR order.
__global__ __launch_bounds__(kBlock) void band_scatter_kernel(const int64_t *__restrict__ rowptr,
                                                              const int32_t *__restrict__ col, int64_t M, int n_bands,
                                                              int band_cols, const int32_t *__restrict__ lo,
                                                              const int32_t *__restrict__ rowptr_bm,
                                                              int32_t *__restrict__ col_bm, int32_t *__restrict__ eperm_bm) {
    const int64_t r = (int64_t)blockIdx.x * (kBlock / 16) + threadIdx.x / 16;
    if (r >= M) return;
    const int64_t b0 = rowptr[r], e0 = rowptr[r + 1];
    for (int64_t i = b0 + (threadIdx.x % 16); i < e0; i += 16) {
        const int32_t c = col[i];
        const int b = c / band_cols;
        const int64_t dst = (int64_t)rowptr_bm[(int64_t)b * (M + 1) + r] + (i - lo[r * (n_bands + 1) + b]);
        col_bm[dst] = c;
        eperm_bm[dst] = (int32_t)i;
    }
}

// ------------------------------------------------------------------------------------------------
// Launch tables.
// ------------------------------------------------------------------------------------------------
struct ShortArgs {
    const int64_t *rowptr; const int32_t *col; const float *val; DenseSrc dense; float *out;
    const int4 *chunks; int n_chunks; const int32_t *empty_rows; int n_empty;
    int F; int64_t ldo; int accumulate; const float *row_div;
    bool prof;   // false: no profiling events (the non-allocating entry point creates nothing)
};
struct PieceArgs {
    const int32_t *col_long; const int32_t *eperm; const float *val; float *partial;
    const int4 *cls_work;
    int max_cls_items; int F;
};
struct FinalArgs {
    const int32_t *long_rows; const int32_t *long_pbeg; const float *partial; float *out; int n_long;
    int F; int64_t ldo; int accumulate; const float *row_div;
};

template <int VEC, int G, int NV, int BITS>
static void launch_all(const ShortArgs &a, const PieceArgs &s, const FinalArgs &f, hipStream_t st) {
    constexpr int GPB = kBlock / G;
    // The long rows (pieces + final sum) and the short rows write disjoint output rows; all kernels go to the
    // caller's stream one after the other (issuing the long rows on a second stream measured -1 ... +5 %).
    hipStream_t ls = st;
    const char *hub_env = getenv("SGNN_SPMM_HUB_LDS");
    const bool hub_lds = hub_env != nullptr && atoi(hub_env) != 0;
    if (BITS == 0 && hub_lds && f.n_long > 0) {
        ProfScope prof(K_SPMM_PIECE, ls, a.prof);
        hipLaunchKernelGGL((spmm_hubrow_lds_kernel<VEC, G, NV>), dim3((uint32_t)f.n_long), dim3(kBlock), 0, ls, a.rowptr, a.col, a.val,
                           a.dense, f.long_rows, f.out, f.F, f.ldo, f.accumulate, f.row_div);
    } else if (f.n_long > 0) {
        {
            // workgroup i serves class i % 8: grid = 8 * (workgroups of the fullest class)
            const uint32_t nb = (uint32_t)kNumXCD * (uint32_t)((s.max_cls_items + GPB - 1) / GPB);
            ProfScope prof(BITS == 0 ? K_SPMM_PIECE : K_FUSED_PIECE, ls, a.prof);
            if (s.eperm)
                hipLaunchKernelGGL((spmm_piece_kernel<VEC, G, NV, BITS, true>), dim3(nb), dim3(kBlock), 0, ls, s.col_long,
                                   s.eperm, s.val, a.dense, s.partial, s.cls_work, s.max_cls_items, s.F);
            else
                hipLaunchKernelGGL((spmm_piece_kernel<VEC, G, NV, BITS, false>), dim3(nb), dim3(kBlock), 0, ls, s.col_long,
                                   s.eperm, s.val, a.dense, s.partial, s.cls_work, s.max_cls_items, s.F);
        }
        const uint32_t nb = (uint32_t)((f.n_long + GPB - 1) / GPB);
        ProfScope prof(K_SPMM_LONG_FINAL, ls, a.prof);
        hipLaunchKernelGGL((spmm_long_final_kernel<VEC, G, NV>), dim3(nb), dim3(kBlock), 0, ls, f.long_rows,
                           f.long_pbeg, f.partial, f.out, f.n_long, f.F, f.ldo, f.accumulate, f.row_div);
    }
    if (a.n_chunks > 0) {
        const uint32_t nb = (uint32_t)((a.n_chunks + GPB - 1) / GPB);
        ProfScope prof(BITS == 0 ? K_SPMM_SHORT : K_FUSED_SHORT, st, a.prof);
        hipLaunchKernelGGL((spmm_short_kernel<VEC, G, NV, BITS>), dim3(nb), dim3(kBlock), 0, st, a.rowptr, a.col, a.val,
                           a.dense, a.out, a.chunks, a.n_chunks, a.F, a.ldo, a.accumulate, a.row_div, nb);
    }
    if (a.n_empty > 0 && (!a.accumulate || a.row_div)) {
        const uint32_t nb = (uint32_t)((a.n_empty + GPB * kEmptyRowsPerGroup - 1) / (GPB * kEmptyRowsPerGroup));
        ProfScope prof(K_SPMM_EMPTY_ROWS, st, a.prof);
        hipLaunchKernelGGL((spmm_empty_rows_kernel<VEC, G, NV>), dim3(nb), dim3(kBlock), 0, st, a.empty_rows, a.n_empty,
                           a.out, a.F, a.ldo, a.accumulate, a.row_div);
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

// Lane slots (of VEC codes each) the fused kernels' lane-group shape for a row of nvec vectors holds: the shapes
// instantiated in dispatch_shape_dq.
static int dq_slots(int vec, int nvec) {
    if (nvec <= 8) return 8;
    if (nvec <= 16) return 16;
    if (nvec <= 32) return 32;
    if (nvec <= 64) return 64;
    if (nvec <= 128) return 128;
    if (vec == 2) return nvec <= 320 ? 320 : (nvec + 511) / 512 * 512;
    return nvec <= 256 ? 256 : (nvec + 511) / 512 * 512;
}

// Quantized dense operand: one packed word of VEC codes per lane and vector.  VEC = 4 when F % 4 == 0,
// VEC = 2 for the other even widths (F = 602: 301 two-float lanes slots, five per lane).
template <int BITS>
static int dispatch_shape_dq(int vec, int nvec, const ShortArgs &a, const PieceArgs &s, const FinalArgs &f, hipStream_t st) {
    if (vec == 2) {
        if (nvec <= 8) launch_all<2, 8, 1, BITS>(a, s, f, st);
        else if (nvec <= 16) launch_all<2, 16, 1, BITS>(a, s, f, st);
        else if (nvec <= 32) launch_all<2, 32, 1, BITS>(a, s, f, st);
        else if (nvec <= 64) launch_all<2, 64, 1, BITS>(a, s, f, st);
        else if (nvec <= 128) launch_all<2, 64, 2, BITS>(a, s, f, st);
        else if (nvec <= 320) launch_all<2, 64, 5, BITS>(a, s, f, st);
        else launch_all<2, 64, 8, BITS>(a, s, f, st);
        return SGNN_OK;
    }
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

// The matrix cut into column bands, each band a CSR matrix of its own (see spmm_band_kernel).
struct BandSchedule {
    int band_cols = 0, n_bands = 0;
    int32_t *col_bm = nullptr;         // [nnz] columns, band-major (+ kBandPad + 4 zero entries)
    int32_t *eperm_bm = nullptr;       // [nnz] CSR index of each band-major edge
    float *val_bm = nullptr;           // [nnz] edge values in band-major order
    uint64_t val_gen = 0;              // plan bind generation val_bm was filled under (0 = not from a bound array)
    uint64_t last_use = 0;             // the plan's band_use_clock at this schedule's last product
    int64_t M = 0, K = 0;
    std::vector<int32_t> h_rowptr_bm;  // host: [n_bands * (M+1)] where each (band, row) starts in the band-major arrays
    // The bands cut into chunks, for one pair of limits (rows, edges per chunk); a launch picks the limits from
    // its lane-group shape and from whether edge values are staged, so a schedule may hold more than one list.
    struct ChunkList {
        int rows_cap = 0, edge_cap = 0;
        int4 *chunks = nullptr;            // all bands' chunk records (four int4 each, see spmm_band_kernel), band after band
        std::vector<int64_t> chunk_off;    // [n_bands + 1] each band's range of chunks
    };
    std::list<ChunkList> lists;   // (a list: launches keep pointers to its elements while further lists are built)
    ~BandSchedule() {
        (void)hipFree(col_bm); (void)hipFree(eperm_bm); (void)hipFree(val_bm);
        for (ChunkList &l : lists) (void)hipFree(l.chunks);
    }
};

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
    // Band schedules (dense-degree matrices), built on first use for a band width.
    int cols_sorted = -1;           // -1 unknown, 0 some row's columns are out of order, 1 every row is column-sorted
    uint64_t bind_gen = 1;          // bumped by every sgnn_spmm_plan_bind_values
    std::vector<BandSchedule *> bands;
    float *band_xs = nullptr;       // the dense operand restaged slice by slice (see band_restage_kernel), grown on demand
    size_t band_xs_floats = 0;
    // A matrix with 2^31 edges or more is held as consecutive row blocks, each a plan of its own with fewer
    // edges than that (the kernels' edge offsets are 32-bit); every call on the whole runs the blocks in turn.
    std::vector<sgnn_spmm_plan *> parts;
    std::vector<int64_t> part_row0, part_edge0;
    sgnn_spmm_plan *whole = nullptr;   // a row block: the plan it belongs to, which owns the restaged-operand workspace
    uint64_t call_serial = 0;          // products run on this (whole) plan so far
    uint64_t xs_serial = 0;            // the product whose dense operand band_xs holds ...
    int xs_F = 0, xs_slice_pad = 0, xs_slices = 0;  // ... and in which slice layout
    uint64_t band_use_clock = 0;       // counts band-schedule products (least-recently-used eviction of schedules)
    // Short-row chunks, one list per chunk row limit (7, 15, 31).
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
    const int64_t short_edges = p->nnz - p->long_edges;
    const int target = (int)std::min<int64_t>(64, std::max<int64_t>(16, short_edges / kChunkGroupsWanted));
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
    for (sgnn_spmm_plan *part : p->parts) (void)sgnn_spmm_plan_destroy(part);
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
    (void)hipFree(p->partial);
    (void)hipFree(p->empty_rows);
    for (int i = 0; i < 3; ++i) (void)hipFree(p->chunks[i]);
    for (BandSchedule *b : p->bands) delete b;
    (void)hipFree(p->band_xs);
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
        if (p->partitioned) {
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

// Most edges one plan holds (the kernels address edges with 32-bit offsets).  SGNN_SPMM_PART_EDGES lowers it so
// that the row-block path can be exercised on small matrices.
static int64_t part_edge_cap() {
    const int64_t dflt = (int64_t)INT32_MAX - ((int64_t)1 << 20);
    const char *e = getenv("SGNN_SPMM_PART_EDGES");
    const int64_t v = e ? atoll(e) : 0;
    return v > 0 && v < dflt ? v : dflt;
}

// A matrix with more edges than one plan holds: consecutive row blocks of at most `cap` edges, each a plan of its
// own over a rebased copy of its slice of rowptr.  A single row longer than the cap is refused.
static int plan_create_parts(sgnn_spmm_plan *p, const int64_t *rowptr, const void *col, int col_is_i64, int64_t cap,
                             hipStream_t st) {
    const int64_t M = p->M;
    SGNN_HIP_CHECK(hipGetDevice(&p->device));
    std::vector<int64_t> h((size_t)M + 1);
    SGNN_HIP_CHECK(hipMemcpyAsync(h.data(), rowptr, sizeof(int64_t) * h.size(), hipMemcpyDeviceToHost, st));
    SGNN_HIP_CHECK(hipStreamSynchronize(st));
    if (h[0] != 0) return fail(SGNN_ERR_RANGE, "rowptr[0] = %lld, expected 0", (long long)h[0]);
    for (int64_t m = 0; m < M; ++m)
        if (h[m + 1] < h[m]) return fail(SGNN_ERR_RANGE, "rowptr decreases at row %lld", (long long)m);
    if (h[M] != p->nnz) return fail(SGNN_ERR_RANGE, "rowptr[M] = %lld but nnz = %lld", (long long)h[M], (long long)p->nnz);
    const size_t col_bytes = col_is_i64 ? sizeof(int64_t) : sizeof(int32_t);
    int64_t r0 = 0;
    while (r0 < M) {
        // the longest run of rows from r0 on with at most `cap` edges
        int64_t r1 = std::upper_bound(h.begin() + r0, h.end(), h[r0] + cap) - h.begin() - 1;
        if (r1 <= r0)
            return fail(SGNN_ERR_ARG, "row %lld has %lld edges, more than one plan holds (%lld)", (long long)r0,
                        (long long)(h[r0 + 1] - h[r0]), (long long)cap);
        if (r1 > M) r1 = M;
        std::vector<int64_t> rebased((size_t)(r1 - r0) + 1);
        for (int64_t i = r0; i <= r1; ++i) rebased[(size_t)(i - r0)] = h[i] - h[r0];
        DevTmp<int64_t> d_rp;
        int rc = upload(&d_rp.p, rebased, st);
        if (rc != SGNN_OK) return rc;
        sgnn_spmm_plan *part = new sgnn_spmm_plan();
        p->parts.push_back(part);  // owned from here on: destroyed with the whole
        p->part_row0.push_back(r0);
        p->part_edge0.push_back(h[r0]);
        part->whole = p;
        part->M = r1 - r0; part->K = p->K; part->nnz = h[r1] - h[r0];
        part->long_thresh = p->long_thresh; part->piece_edges = p->piece_edges;
        rc = plan_create_impl(part, d_rp.p, (const char *)col + (size_t)h[r0] * col_bytes, col_is_i64, st);
        if (rc != SGNN_OK) return rc;
        SGNN_HIP_CHECK(hipStreamSynchronize(st));  // the rebased row pointers die at the end of the iteration
        r0 = r1;
    }
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_create(const int64_t *rowptr, const void *col, int col_is_i64, int64_t M, int64_t K,
                                     int64_t nnz, int long_row_threshold, int piece_edges,
                                     sgnn_stream_t stream, sgnn_spmm_plan **plan_out) {
    SGNN_REQUIRE(plan_out != nullptr, "plan_out is null");
    *plan_out = nullptr;
    SGNN_REQUIRE(rowptr != nullptr, "rowptr is null");
    SGNN_REQUIRE(M >= 0 && K >= 0 && nnz >= 0, "negative size (M=%lld K=%lld nnz=%lld)", (long long)M, (long long)K, (long long)nnz);
    SGNN_REQUIRE(M < INT32_MAX && K < INT32_MAX, "M and K must fit 31 bits (M=%lld K=%lld)", (long long)M, (long long)K);
    SGNN_REQUIRE(nnz == 0 || col != nullptr, "col is null with nnz=%lld", (long long)nnz);
    sgnn_spmm_plan *p = new sgnn_spmm_plan();
    p->M = M; p->K = K; p->nnz = nnz;
    p->long_thresh = long_row_threshold > 0 ? long_row_threshold : kDefaultLongThreshold;
    p->piece_edges = piece_edges > 0 ? piece_edges : kDefaultPieceEdges;
    const int64_t part_cap = part_edge_cap();
    const int rc = nnz <= part_cap ? plan_create_impl(p, rowptr, col, col_is_i64, (hipStream_t)stream)
                                   : plan_create_parts(p, rowptr, col, col_is_i64, part_cap, (hipStream_t)stream);
    if (rc != SGNN_OK) {
        sgnn_spmm_plan_destroy(p);
        return rc;
    }
    // The non-allocating entry point must not be the first to look the scratch array's address up (a lazy symbol
    // lookup inside what may be a graph capture): plan creation, which synchronises and allocates anyway, does it.
    float *scratch = nullptr;
    (void)scratch_for_current_device(&scratch);
    *plan_out = p;
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_info(const sgnn_spmm_plan *p, int64_t info[10]) {
    SGNN_REQUIRE(p != nullptr && info != nullptr, "null argument");
    info[0] = p->M; info[1] = p->K; info[2] = p->nnz; info[3] = p->n_long; info[4] = p->n_items;
    info[5] = p->long_edges; info[6] = p->long_thresh; info[7] = p->piece_edges;
    info[8] = p->partitioned ? 1 : 0; info[9] = (int64_t)(p->top_share * 1e6);
    for (const sgnn_spmm_plan *part : p->parts) {  // row blocks: counts add up, the flags are those of any block
        info[3] += part->n_long; info[4] += part->n_items; info[5] += part->long_edges;
        info[8] |= part->partitioned ? 1 : 0;
        info[9] = std::max<int64_t>(info[9], (int64_t)(part->top_share * 1e6));
    }
    return SGNN_OK;
}

extern "C" int sgnn_spmm_reference_overwrites(int64_t nnz, int64_t M, int64_t K, int64_t F) {
    if (M <= 0 || K <= 0) return 0;
    const float sparsity = (float)nnz / (float)M / (float)K;
    return (sparsity <= 0.0001f && F > 256) ? 1 : 0;
}

// ------------------------------------------------------------------------------------------------
// Band schedule, host side.
// ------------------------------------------------------------------------------------------------
constexpr int kBandL2BudgetKB = 4096;   // per-XCD bytes of the restaged dense operand in one band: the whole 4 MB L2 measured best (the other streams pass through)
constexpr double kBandMinRowEdges = 6;  // average edges per row and band below which the per-band read-modify-write of out dominates
constexpr int64_t kBandMinDenseBytes = (int64_t)48 << 20;  // a dense operand this small lives in the L2s anyway

struct BandShape {
    bool even;         // X-independent: out rows on 8-byte boundaries, F even and >= 4 (128-bit accesses to out)
    int n_slices;      // feature slices = XCDs that split the feature axis (8, 4, 2 or 1)
    int slice_floats;  // feature columns per slice (a multiple of 4)
    int slice_pad;     // floats per restaged slice row (a multiple of 16: rows on 64-byte boundaries)
    int G;             // lanes per group: slice_pad / 4, at least 16, at most 64 (wider slices are walked in tiles)
    int band_cols, n_bands;
    int f0, F;         // the feature columns [f0, f0 + F) of the product this shape covers (one window)
    size_t xs_off;     // where this window's restaged operand starts in the workspace, in floats
};

// Feature columns per window of a wide product.  Slices of exactly 64 floats are the band kernel's most efficient
// shape (a wavefront instruction carries four gathers of 256 bytes, every lane busy), and a window of 512 columns
// is eight of them, one per XCD.  Wider products run as consecutive windows over the same bands: the reference
// tiles the feature axis of every row in the same way (spmm.cpp:502-510).
constexpr int kBandWindowCols = 512;
constexpr int kBandMinGroup = 8;   // lanes per group, at least (lane i of a group holds row i's offset: up to 7 rows per chunk)
constexpr int kMaxBandSchedules = 3;   // band widths a plan keeps schedules for (each holds ~12 bytes per edge)
constexpr int kBandMaxWindows = 64;

// How a product of feature width F is cut into feature windows, slices and column bands.  Products of up to
// kBandWindowCols columns are one window whose slices share the eight XCDs evenly.  Wider products take windows
// of kBandWindowCols columns and a remainder window with slices of at most 64 floats; every window uses the
// bands of a 64-float slice, so one band-major copy of the edges serves them all.
struct BandWindows {
    int n = 0;
    BandShape w[kBandMaxWindows];
    size_t xs_floats = 0;   // restaged operand of all windows
    int total_slices = 0;
};

static BandShape band_window_shape(const sgnn_spmm_plan *p, int f0, int Fw, bool even_out, bool windowed) {
    BandShape b{};
    b.f0 = f0;
    b.F = Fw;
    b.even = even_out && Fw % 2 == 0 && Fw >= 4 && f0 % 2 == 0;
    const int nvec = (Fw + 3) / 4;
    if (windowed) {
        // At most 16 float4 per slice (the bands are sized for 64-float slices).  A gather instruction costs the same
        // whatever its lanes carry, so the cut that needs the fewest of them wins: slices / (lane groups per wavefront).
        // A remainder of 90 columns takes 2 slices of 12 float4, five lane groups per wavefront (0.4 instructions per
        // edge against 0.5 for 2 slices in groups of 16 lanes or 4 slices of 6 float4).
        double best = 1e30;
        for (int n = 1; n <= kNumXCD; n *= 2) {
            const int vps = (nvec + n - 1) / n;
            if (vps > 16) continue;
            const int g = std::max(kBandMinGroup, (4 * vps + 15) / 16 * 4);
            const double cost = (double)n / (64 / g);
            if (cost < best - 1e-9) { best = cost; b.n_slices = n; }
        }
    } else {
        b.n_slices = kNumXCD;
        while (b.n_slices > 1 && (nvec + b.n_slices - 1) / b.n_slices < 16) b.n_slices /= 2;
        const int forced = env_int("SGNN_SPMM_BAND_SLICES", 0);
        if (forced == 1 || forced == 2 || forced == 4 || forced == 8) b.n_slices = forced;
    }
    b.slice_floats = 4 * ((nvec + b.n_slices - 1) / b.n_slices);
    b.slice_pad = (b.slice_floats + 15) / 16 * 16;
    b.G = std::max(windowed ? kBandMinGroup : 16, std::min(64, b.slice_pad / 4));
    int cols = env_int("SGNN_SPMM_BAND_COLS", 0);
    if (cols <= 0) {
        const int pad = windowed ? 64 : b.slice_pad;   // windows share the bands of a full 64-float slice
        cols = (int)std::max<int64_t>(256, (int64_t)env_int("SGNN_SPMM_BAND_KB", kBandL2BudgetKB) * 1024 / (pad * 4) / 256 * 256);
    }
    b.band_cols = cols;
    b.n_bands = (int)std::max<int64_t>(1, (p->K + cols - 1) / cols);
    return b;
}

static BandWindows band_windows(const sgnn_spmm_plan *p, int64_t F, bool even_out) {
    BandWindows bw;
    const int win = env_int("SGNN_SPMM_BAND_WINDOW", kBandWindowCols);   // 0 = never cut a product into windows
    const bool windowed = win >= 64 && win % 64 == 0 && F > win && (F + win - 1) / win <= kBandMaxWindows;
    if (!windowed) {
        bw.n = 1;
        bw.w[0] = band_window_shape(p, 0, (int)F, even_out, false);
    } else {
        for (int64_t f0 = 0; f0 < F; f0 += win)
            bw.w[bw.n++] = band_window_shape(p, (int)f0, (int)std::min<int64_t>(win, F - f0), even_out, true);
    }
    for (int i = 0; i < bw.n; ++i) {
        bw.w[i].xs_off = bw.xs_floats;
        bw.xs_floats += (size_t)bw.w[i].n_slices * (size_t)p->K * (size_t)bw.w[i].slice_pad;
        bw.total_slices += bw.w[i].n_slices;
    }
    return bw;
}

// Whether the band schedule is the one to use: the dense operand does not fit the caches, and every row has
// enough edges per band to pay for carrying its accumulator through `out` from band to band.
static bool band_wanted(const sgnn_spmm_plan *p, int64_t F, const BandShape &b) {
    const int mode = env_int("SGNN_SPMM_BAND", -1);
    if (mode == 0 || p->nnz == 0 || p->M == 0) return false;
    if (mode > 0) return true;
    if (b.n_bands < 3 || p->K * F * 4 < kBandMinDenseBytes) return false;
    return (double)p->nnz / (double)p->M / (double)b.n_bands >= kBandMinRowEdges;
}

static int band_rows_sorted(sgnn_spmm_plan *p, hipStream_t st, bool *sorted) {
    if (p->cols_sorted < 0) {
        DevTmp<int> flag;
        SGNN_HIP_CHECK(hipMalloc(&flag.p, sizeof(int)));
        SGNN_HIP_CHECK(hipMemsetAsync(flag.p, 0, sizeof(int), st));
        hipLaunchKernelGGL(check_rows_sorted_kernel, dim3((uint32_t)((p->M + 15) / 16)), dim3(kBlock), 0, st, p->rowptr, p->col,
                           p->M, flag.p);
        SGNN_HIP_CHECK(hipGetLastError());
        int h = 0;
        SGNN_HIP_CHECK(hipMemcpyAsync(&h, flag.p, sizeof(int), hipMemcpyDeviceToHost, st));
        SGNN_HIP_CHECK(hipStreamSynchronize(st));
        p->cols_sorted = h ? 0 : 1;
    }
    *sorted = p->cols_sorted == 1;
    return SGNN_OK;
}

// The chunk list of every band for the given limits: consecutive rows, at most rows_cap rows and edge_cap edges
// (one row may have more), first and last row non-empty in the band.
static int band_build_chunks(BandSchedule *bs, int rows_cap, int edge_cap, hipStream_t st, const BandSchedule::ChunkList **res) {
    const int64_t M = bs->M;
    std::vector<int4> out;   // four per chunk
    BandSchedule::ChunkList list;
    list.rows_cap = rows_cap;
    list.edge_cap = edge_cap;
    list.chunk_off.assign((size_t)bs->n_bands + 1, 0);
    for (int b = 0; b < bs->n_bands; ++b) {
        const int32_t *rp = bs->h_rowptr_bm.data() + (size_t)b * (size_t)(M + 1);
        int64_t m = 0;
        while (m < M) {
            if (rp[m + 1] == rp[m]) { ++m; continue; }
            const int64_t start = m;
            int64_t last = m, edges = 0;
            while (m < M && m - start < rows_cap) {
                const int64_t d = rp[m + 1] - rp[m];
                if (m > start && edges + d > edge_cap) break;
                if (d > 0) last = m;
                edges += d;
                ++m;
            }
            const int nr = (int)(last - start + 1);
            const int64_t E = rp[last + 1] - rp[start];
            uint32_t w[kBandOffsets / 2] = {};   // 16-bit offsets of the chunk's rows, entries >= nr hold the edge count
            for (int i = 0; i < kBandOffsets; ++i) {
                const int64_t rel = i < nr ? rp[start + i] - rp[start] : E;
                w[i >> 1] |= (uint32_t)(rel & 0xffff) << (16 * (i & 1));   // (more than 65535 only in a one-row chunk)
            }
            out.push_back(make_int4((int)start, nr, rp[start], (int)E));
            for (int q = 0; q < 3; ++q) out.push_back(make_int4((int)w[4 * q], (int)w[4 * q + 1], (int)w[4 * q + 2], (int)w[4 * q + 3]));
        }
        list.chunk_off[(size_t)b + 1] = (int64_t)(out.size() / 4);
    }
    if (!out.empty()) {
        SGNN_HIP_CHECK(hipMalloc(&list.chunks, sizeof(int4) * out.size()));
        const hipError_t e = hipMemcpyAsync(list.chunks, out.data(), sizeof(int4) * out.size(), hipMemcpyHostToDevice, st);
        const hipError_t e2 = e == hipSuccess ? hipStreamSynchronize(st) : e;
        if (e2 != hipSuccess) {
            (void)hipFree(list.chunks);
            SGNN_HIP_CHECK(e2);
        }
    }
    bs->lists.push_back(std::move(list));
    *res = &bs->lists.back();
    return SGNN_OK;
}

// Device allocations of the band schedule: running out of memory is not an error of the product (the row-class
// schedule needs none of this), so it is told apart from other failures.
static thread_local bool g_band_oom = false;
static bool band_build_out_of_memory() {
    const bool r = g_band_oom;
    g_band_oom = false;
    return r;
}
#define SGNN_BAND_ALLOC(pp, bytes)                                                             \
    do {                                                                                       \
        const hipError_t _me = hipMalloc((pp), (bytes));                                       \
        if (_me == hipErrorOutOfMemory) {                                                      \
            (void)hipGetLastError();                                                           \
            g_band_oom = true;                                                                 \
            return ::sgnn::fail(SGNN_ERR_HIP, "band schedule: out of device memory");          \
        }                                                                                      \
        SGNN_HIP_CHECK(_me);                                                                   \
    } while (0)

static int band_build(sgnn_spmm_plan *p, int band_cols, int n_bands, hipStream_t st, BandSchedule **out) {
    const int64_t M = p->M, nnz = p->nnz;
    std::unique_ptr<BandSchedule> bs(new BandSchedule());
    bs->band_cols = band_cols;
    bs->n_bands = n_bands;
    bs->M = M;
    bs->K = p->K;
    SGNN_REQUIRE((int64_t)n_bands * (M + 1) < INT32_MAX && M * ((int64_t)n_bands + 1) < INT32_MAX * (int64_t)4,
                 "band schedule too large (%d bands x %lld rows)", n_bands, (long long)M);
    DevTmp<int32_t> lo, cnt_t;
    const int64_t n_lo = M * ((int64_t)n_bands + 1), n_cnt = M * (int64_t)n_bands;
    SGNN_BAND_ALLOC(&lo.p, sizeof(int32_t) * (size_t)n_lo);
    SGNN_BAND_ALLOC(&cnt_t.p, sizeof(int32_t) * (size_t)n_cnt);
    hipLaunchKernelGGL(band_bounds_kernel, dim3((uint32_t)((n_lo + kBlock - 1) / kBlock)), dim3(kBlock), 0, st, p->rowptr, p->col, M,
                       n_bands, band_cols, lo.p);
    hipLaunchKernelGGL(band_counts_kernel, dim3((uint32_t)((n_cnt + kBlock - 1) / kBlock)), dim3(kBlock), 0, st, lo.p, M, n_bands,
                       cnt_t.p);
    SGNN_HIP_CHECK(hipGetLastError());
    std::vector<int32_t> h_cnt((size_t)n_cnt);
    SGNN_HIP_CHECK(hipMemcpyAsync(h_cnt.data(), cnt_t.p, sizeof(int32_t) * h_cnt.size(), hipMemcpyDeviceToHost, st));
    SGNN_HIP_CHECK(hipStreamSynchronize(st));
    std::vector<int32_t> rp((size_t)n_bands * (size_t)(M + 1));
    int64_t run = 0;
    for (int b = 0; b < n_bands; ++b) {
        int32_t *row = rp.data() + (size_t)b * (size_t)(M + 1);
        const int32_t *c = h_cnt.data() + (size_t)b * (size_t)M;
        for (int64_t r = 0; r < M; ++r) {
            row[r] = (int32_t)run;
            run += c[r];
        }
        row[M] = (int32_t)run;
    }
    if (run != nnz) return fail(SGNN_ERR_RANGE, "band schedule: %lld of %lld edges fall into the bands", (long long)run, (long long)nnz);
    DevTmp<int32_t> rowptr_bm;   // [n_bands * (M+1)] where each (band, row) starts in the band-major arrays
    SGNN_BAND_ALLOC(&rowptr_bm.p, sizeof(int32_t) * rp.size());
    SGNN_HIP_CHECK(hipMemcpyAsync(rowptr_bm.p, rp.data(), sizeof(int32_t) * rp.size(), hipMemcpyHostToDevice, st));
    // the kernel reads up to kBandPad + 3 entries past a chunk's last pair: zero entries (column 0) close the arrays
    const size_t tail = (size_t)kBandPad + 4;
    SGNN_BAND_ALLOC(&bs->col_bm, sizeof(int32_t) * ((size_t)nnz + tail));
    SGNN_BAND_ALLOC(&bs->eperm_bm, sizeof(int32_t) * (size_t)nnz);
    SGNN_BAND_ALLOC(&bs->val_bm, sizeof(float) * ((size_t)nnz + tail));
    SGNN_HIP_CHECK(hipMemsetAsync(bs->col_bm + nnz, 0, sizeof(int32_t) * tail, st));
    SGNN_HIP_CHECK(hipMemsetAsync(bs->val_bm + nnz, 0, sizeof(float) * tail, st));
    hipLaunchKernelGGL(band_scatter_kernel, dim3((uint32_t)((M + 15) / 16)), dim3(kBlock), 0, st, p->rowptr, p->col, M, n_bands,
                       band_cols, lo.p, rowptr_bm.p, bs->col_bm, bs->eperm_bm);
    SGNN_HIP_CHECK(hipGetLastError());
    SGNN_HIP_CHECK(hipStreamSynchronize(st));
    bs->h_rowptr_bm = std::move(rp);
    *out = bs.release();
    return SGNN_OK;
}

// Limits of a chunk for one launch shape.  Two workgroups per CU is what the kernel's registers allow, so a lane
// group may use 80 KB / (groups per workgroup) of LDS: its output tile (rows_cap rows of the slice) and the staged
// edges (4 bytes each, 8 with values).  Large chunks matter: every chunk costs a fixed set-up, measured on the
// 233 k-node / 114 M-edge graph at F = 602 as time = 14.7 ms + 590 ms / (edges per chunk).  The rows are sized so
// that a chunk of average rows fills the edge budget.
struct BandCaps { int rows, edges; };
static BandCaps band_chunk_caps(const sgnn_spmm_plan *p, const BandShape &sh, bool weighted) {
    const int gpb = (kBandBlock / 64) * (64 / sh.G);
    const int64_t budget = (int64_t)80 * 1024 / gpb, row_bytes = (int64_t)sh.G * 16, bpe = weighted ? 8 : 4;
    const int64_t avg = std::max<int64_t>(1, p->nnz / std::max<int64_t>(1, p->M) / std::max(1, sh.n_bands));
    // (the kernel stages a chunk's pairs in a fixed number of rounds of 4 * G pairs: narrow groups stage fewer)
    constexpr int kRoundsU = (kBandEdges + kBandPad + 63) / 64, kRoundsW = (kBandEdgesWeighted + kBandPad + 63) / 64;
    const int rows_lim = weighted ? kBandRowsWeighted : kBandRows;
    const int edges_lim = std::min(weighted ? kBandEdgesWeighted : kBandEdges,
                                   ((weighted ? kRoundsW : kRoundsU) * 4 * sh.G - kBandPad - kBandWindow) / 16 * 16);
    const int rows_max = std::min(rows_lim, sh.G - 1);   // lane i of a group holds row i's offset, lane `rows` the end
    int rows = (int)std::max<int64_t>(1, std::min<int64_t>(rows_max, (budget - kBandPad * bpe) / (row_bytes + bpe * avg)));
    int edges = 0;
    for (;; --rows) {
        edges = (int)std::min<int64_t>(edges_lim, ((budget - rows * row_bytes) / bpe - kBandPad) / 16 * 16);
        if (edges >= 64 || rows == 1) break;
    }
    edges = std::max(edges, 16);
    const int er = env_int("SGNN_SPMM_BAND_CHUNK_ROWS", 0), ee = env_int("SGNN_SPMM_BAND_CHUNK_EDGES", 0);
    if (er > 0) rows = std::min(er, rows_max);
    if (ee > 0) edges = std::max(16, std::min(ee, edges_lim) / 16 * 16);   // the next group's float4 tile starts right behind the staged edges
    return BandCaps{rows, edges};
}

template <bool EVEN, bool WEIGHTED>
static int launch_band(const BandSchedule *bs, const BandSchedule::ChunkList *cl, const BandShape &sh, int b, const float *val_bm,
                       const float *xs, float *out, int64_t ldo, hipStream_t st, int device) {
    const int64_t c0 = cl->chunk_off[(size_t)b], c1 = cl->chunk_off[(size_t)b + 1];
    if (c1 == c0) return SGNN_OK;
    const int gpb = (kBandBlock / 64) * (64 / sh.G);  // lane groups per workgroup
    const int n_rg = kNumXCD / sh.n_slices;
    const int64_t wgs = (c1 - c0 + gpb - 1) / gpb;
    const uint32_t nb = (uint32_t)((wgs + n_rg - 1) / n_rg) * kNumXCD;
    const size_t lds = sizeof(float) * (size_t)gpb * (size_t)band_group_floats(sh.G * 4, cl->rows_cap, cl->edge_cap, WEIGHTED);
    // every restaged row of a slice within 4 GB of the slice's start: 32-bit gather offsets
    // (SGNN_SPMM_BAND_OFF64=1 forces the 64-bit variant so that tests reach it at small sizes)
    const bool off32 = (uint64_t)bs->K * (uint64_t)sh.slice_pad * 4u < ((uint64_t)1 << 32) && env_int("SGNN_SPMM_BAND_OFF64", 0) == 0;
    auto kernel = off32 ? spmm_band_kernel<EVEN, true, WEIGHTED> : spmm_band_kernel<EVEN, false, WEIGHTED>;
    // the dynamic-LDS limit of a kernel is a per-device setting: remember what each device has been told
    static std::mutex mu;
    static size_t lds_allowed[64][2];
    {
        std::lock_guard<std::mutex> lock(mu);
        size_t &allowed = lds_allowed[device & 63][off32];
        if (lds > std::max<size_t>(allowed, 48 * 1024)) {
            SGNN_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            allowed = lds;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(nb), dim3(kBandBlock), lds, st, bs->col_bm, val_bm, xs + sh.xs_off, bs->K, out + sh.f0,
                       cl->chunks + 4 * c0, (int)(c1 - c0), sh.F, ldo, sh.slice_floats, sh.slice_pad, sh.n_slices, sh.G, cl->rows_cap,
                       cl->edge_cap);
    return SGNN_OK;
}

template <int VEC>
static void launch_fill_or_divide(float *out, int64_t M, int F, int64_t ldo, const float *row_div, hipStream_t st) {
    const int64_t n = M * (F / VEC);
    const uint32_t nb = (uint32_t)((n + kBlock - 1) / kBlock);
    if (row_div) hipLaunchKernelGGL((rows_fill_or_divide_kernel<VEC, true>), dim3(nb), dim3(kBlock), 0, st, out, M, F, ldo, row_div);
    else hipLaunchKernelGGL((rows_fill_or_divide_kernel<VEC, false>), dim3(nb), dim3(kBlock), 0, st, out, M, F, ldo, row_div);
}

// The product through the band schedule.  may_build = false (the non-allocating entry point): use a schedule
// only if an earlier call has built it; *done tells whether the product was carried out here.
static int spmm_run_band(sgnn_spmm_plan *p, const BandWindows &bw, const float *val, const DenseSrc &dense, float *out, int64_t F,
                         int64_t ldo, int accumulate, const float *row_div, hipStream_t st, bool may_build, bool *done) {
    *done = false;
    const BandShape &sh0 = bw.w[0];
    BandSchedule *bs = nullptr;
    for (BandSchedule *c : p->bands)
        if (c->band_cols == sh0.band_cols) bs = c;
    // The restaged operand lives in the plan the caller holds: the row blocks of a large matrix share one copy,
    // restaged by the first block of a product that takes the band schedule.
    sgnn_spmm_plan *root = p->whole ? p->whole : p;
    const size_t xs_floats = bw.xs_floats;
    if (bs == nullptr || xs_floats > root->band_xs_floats) {
        if (!may_build) return SGNN_OK;
        bool sorted = false;
        int rc = band_rows_sorted(p, st, &sorted);
        if (rc != SGNN_OK) return rc;
        if (!sorted) return SGNN_OK;  // band edges of a row would not be contiguous: the other schedules take it
        if (bs == nullptr) {
            // A plan keeps the schedules of at most kMaxBandSchedules band widths (each holds a band-major copy of
            // the edge list): the one used longest ago makes room.
            if (p->bands.size() >= (size_t)kMaxBandSchedules) {
                SGNN_HIP_CHECK(hipDeviceSynchronize());   // queued launches may still read it
                size_t victim = 0;
                for (size_t i = 1; i < p->bands.size(); ++i)
                    if (p->bands[i]->last_use < p->bands[victim]->last_use) victim = i;
                delete p->bands[victim];
                p->bands.erase(p->bands.begin() + (long)victim);
            }
            rc = band_build(p, sh0.band_cols, sh0.n_bands, st, &bs);
            if (rc == SGNN_ERR_HIP && band_build_out_of_memory()) return SGNN_OK;  // no room for the band-major copy: the row-class schedule runs
            if (rc != SGNN_OK) return rc;
            p->bands.push_back(bs);
        }
        if (xs_floats > root->band_xs_floats) {
            SGNN_HIP_CHECK(hipDeviceSynchronize());  // the old workspace may still be read by queued work
            (void)hipFree(root->band_xs);
            root->band_xs = nullptr;
            root->band_xs_floats = 0;
            root->xs_serial = 0;
            if (hipMalloc(&root->band_xs, xs_floats * sizeof(float)) != hipSuccess) {
                (void)hipGetLastError();
                root->band_xs = nullptr;
                return SGNN_OK;   // no room for the restaged operand: the row-class schedule runs
            }
            root->band_xs_floats = xs_floats;
        }
    }
    const bool weighted = val != nullptr;
    const BandSchedule::ChunkList *cls[kBandMaxWindows];
    for (int w = 0; w < bw.n; ++w) {
        const BandCaps caps = band_chunk_caps(p, bw.w[w], weighted);
        const BandSchedule::ChunkList *cl = nullptr;
        for (const BandSchedule::ChunkList &l : bs->lists)
            if (l.rows_cap == caps.rows && l.edge_cap == caps.edges) cl = &l;
        if (cl == nullptr) {
            if (!may_build) return SGNN_OK;
            const int rc = band_build_chunks(bs, caps.rows, caps.edges, st, &cl);
            if (rc != SGNN_OK) return rc;
        }
        cls[w] = cl;
    }
    const float *val_bm = nullptr;
    if (weighted) {
        const bool bound = val == p->bound_val;
        if (!(bound && bs->val_gen == p->bind_gen)) {
            hipLaunchKernelGGL(permute_values_kernel, dim3((uint32_t)((p->nnz + kBlock - 1) / kBlock)), dim3(kBlock), 0, st, val,
                               bs->eperm_bm, bs->val_bm, p->nnz);
            bs->val_gen = bound ? p->bind_gen : 0;
        }
        val_bm = bs->val_bm;
    }
    const int iF = (int)F;
    if (p->whole == nullptr) ++root->call_serial;  // (a plan of row blocks counts its products in spmm_run)
    bs->last_use = ++root->band_use_clock;
    if (!(root->xs_serial == root->call_serial && root->xs_F == iF && root->xs_slice_pad == sh0.slice_pad && root->xs_slices == bw.total_slices)) {
        ProfScope prof(K_SPMM_BAND_RESTAGE, st, may_build);
        for (int w = 0; w < bw.n; ++w) {
            const BandShape &sh = bw.w[w];
            const int64_t n = (int64_t)sh.n_slices * p->K * (sh.slice_pad / 4);
            hipLaunchKernelGGL(band_restage_kernel, dim3((uint32_t)((n + kBlock - 1) / kBlock)), dim3(kBlock), 0, st, dense.x + sh.f0,
                               dense.ldx, root->band_xs + sh.xs_off, p->K, sh.F, sh.slice_floats, sh.slice_pad, sh.n_slices);
        }
        root->xs_serial = root->call_serial;
        root->xs_F = iF; root->xs_slice_pad = sh0.slice_pad; root->xs_slices = bw.total_slices;
    }
    // vector width of the fill / divide passes over whole rows of out
    const int ev = (ldo % 2 == 0 && F % 2 == 0 && F >= 4 && aligned(out, 8)) ? 2 : 1;
    if (!accumulate) {
        if (ev == 2) launch_fill_or_divide<2>(out, p->M, iF, ldo, nullptr, st);
        else launch_fill_or_divide<1>(out, p->M, iF, ldo, nullptr, st);
    }
    {
        ProfScope prof(K_SPMM_BAND, st, may_build);
        // window after window, band after band: a window's accumulators make all their trips through `out` while
        // its columns of `out` are the only ones in flight
        for (int w = 0; w < bw.n; ++w) {
            const BandShape &sh = bw.w[w];
            for (int b = 0; b < bs->n_bands; ++b) {
                int rc;
                if (val_bm) rc = sh.even ? launch_band<true, true>(bs, cls[w], sh, b, val_bm, root->band_xs, out, ldo, st, p->device)
                                         : launch_band<false, true>(bs, cls[w], sh, b, val_bm, root->band_xs, out, ldo, st, p->device);
                else rc = sh.even ? launch_band<true, false>(bs, cls[w], sh, b, val_bm, root->band_xs, out, ldo, st, p->device)
                                  : launch_band<false, false>(bs, cls[w], sh, b, val_bm, root->band_xs, out, ldo, st, p->device);
                if (rc != SGNN_OK) return rc;
            }
        }
    }
    if (row_div) {
        if (ev == 2) launch_fill_or_divide<2>(out, p->M, iF, ldo, row_div, st);
        else launch_fill_or_divide<1>(out, p->M, iF, ldo, row_div, st);
    }
    SGNN_HIP_CHECK(hipGetLastError());
    *done = true;
    return SGNN_OK;
}

extern "C" int sgnn_spmm_plan_schedule(const sgnn_spmm_plan *p, int64_t F, int64_t info[4]) {
    SGNN_REQUIRE(p != nullptr && info != nullptr, "null argument");
    SGNN_REQUIRE(F > 0 && F < (1 << 24), "feature width F=%lld out of range", (long long)F);
    if (!p->parts.empty()) p = p->parts[0];  // row blocks decide one by one; the first one's answer is reported
    const BandWindows bw = band_windows(p, F, true);
    info[0] = (band_wanted(p, F, bw.w[0]) && p->cols_sorted != 0) ? 1 : 0;
    info[1] = bw.w[0].band_cols; info[2] = bw.w[0].n_bands; info[3] = bw.total_slices;
    return SGNN_OK;
}

// scratch != null: the call must not allocate.  The piece partials then go to `scratch` (scratch_floats
// floats) instead of the plan's own, growable buffer, and nothing is created on the way.
// Width of the feature slices of a wide fp32 product (a multiple of 4; >= F means one slice).  Slices pay once the
// dense operand is too large for the caches to hold its popular rows -- measured on power-law graphs of 0.15 M to
// 2.45 M nodes at F = 256 and 512: with K * F * 4 bytes of 1.25 GB and more two to four slices take 0.78-0.92 of
// the time of one piece, with 0.63 GB and less 1.07-1.30 (a second pass over the edge stream and a second tail
// for nothing).  Multiples of 128 floats go in slices of 128 (two row chunks per wavefront, the shape of the
// headline width); other widths from 256 floats up in equal slices of at most 192.
// SGNN_SPMM_SLICE=<floats> forces slices of that width at any size (0 = never slice).
static int64_t slice_width(int64_t F, int64_t K) {
    const int e = env_int("SGNN_SPMM_SLICE", -1);
    if (e == 0) return F;
    if (e > 0) return std::max<int64_t>(4, (e + 3) / 4 * 4);
    if (F < 256 || K * F * 4 < 900000000ll) return F;
    if (F % 128 == 0) return 128;
    const int64_t n = (F + 191) / 192;
    return ((F + n - 1) / n + 3) / 4 * 4;
}

static int spmm_run(sgnn_spmm_plan *p, const float *val, const DenseSrc &dense, int bits, float *out, int64_t F,
                    int64_t ldo, int accumulate, const float *row_div, hipStream_t st, float *scratch = nullptr,
                    size_t scratch_floats = 0, bool is_slice = false) {
    SGNN_REQUIRE(p != nullptr, "plan is null");
    SGNN_REQUIRE(F > 0 && F < (1 << 24), "feature width F=%lld out of range", (long long)F);
    SGNN_REQUIRE(ldo >= F, "leading dimension smaller than F (ldo=%lld F=%lld)", (long long)ldo, (long long)F);
    if (p->M == 0) return SGNN_OK;
    SGNN_REQUIRE(out != nullptr, "out is null");
    if (!p->parts.empty()) {  // row blocks, one after the other on the caller's stream
        ++p->call_serial;     // one product: the blocks that take the band schedule share one restaged operand
        for (size_t i = 0; i < p->parts.size(); ++i) {
            sgnn_spmm_plan *part = p->parts[i];
            DenseSrc d = dense;
            if (d.eslot_csr != nullptr) {  // per-edge slot streams belong to the block
                d.eslot_csr = part->eslot_csr;
                d.eslot_long = part->eslot_long ? part->eslot_long : part->eslot_csr;
            }
            const int rc = spmm_run(part, val ? val + p->part_edge0[i] : nullptr, d, bits, out + p->part_row0[i] * ldo, F, ldo,
                                    accumulate, row_div ? row_div + p->part_row0[i] : nullptr, st, scratch, scratch_floats);
            if (rc != SGNN_OK) return rc;
        }
        return SGNN_OK;
    }
    int dev = 0;
    SGNN_HIP_CHECK(hipGetDevice(&dev));
    SGNN_REQUIRE(dev == p->device, "plan was created on device %d, current device is %d", p->device, dev);

    int vec = 1;
    if (bits != 0) {
        vec = F % 4 == 0 ? 4 : 2;  // checked by the caller: F even, 4-byte aligned packed buffer
        // With a dense-degree matrix the fused kernels are bound by instruction issue (two fmas and a conversion
        // per element), so idle lane slots cost time: F = 600 fills 150 of the 256 four-code slots of its lane-group
        // shape but 300 of the 320 two-code slots (measured on the 114 M-edge community graph: 11.7 -> 10.5 ms).
        if (vec == 4 && dq_slots(2, (int)(F / 2)) * 2 < dq_slots(4, (int)(F / 4)) * 4 * 0.8) vec = 2;
        SGNN_REQUIRE(ldo % vec == 0 && aligned(out, 4 * vec),
                     "the fused path at F=%lld needs out %d-byte aligned with ldo %% %d == 0", (long long)F, 4 * vec, vec);
    } else if (F % 4 == 0 && dense.ldx % 4 == 0 && ldo % 4 == 0 && aligned(dense.x, 16) && aligned(out, 16)) {
        vec = 4;
    } else if (F % 2 == 0 && dense.ldx % 2 == 0 && ldo % 2 == 0 && aligned(dense.x, 8) && aligned(out, 8)) {
        vec = 2;
    }
    if (bits == 0 && !is_slice) {
        const BandWindows bw = band_windows(p, F, ldo % 2 == 0 && aligned(out, 8));
        if (band_wanted(p, F, bw.w[0])) {
            bool done = false;
            const int rc = spmm_run_band(p, bw, val, dense, out, F, ldo, accumulate, row_div, st, scratch == nullptr, &done);
            if (rc != SGNN_OK || done) return rc;
        }
        // Wide fp32 rows of a large operand: one product per slice of the feature axis, one after the other.  The rows
        // a gather leaves in the caches are then 512 ... 768 bytes instead of 4F, so the same cache holds more of them:
        // on the 62 M-edge power-law graph F = 256 takes 6.3 ms in two slices against 7.3 ms in one, F = 512
        // 13.0 against 16.7, F = 1024 27.4 against 35.2 (the edge stream is read once per slice: +8 bytes on
        // 4 * slice bytes per edge).  A slice is the same arithmetic on its own columns: results do not change.
        const int64_t sw = slice_width(F, p->K);
        if (vec == 4 && sw < F) {
            for (int64_t s0 = 0; s0 < F; s0 += sw) {
                DenseSrc d = dense;
                d.x = dense.x + s0;
                const int rc = spmm_run(p, val, d, 0, out + s0, std::min(sw, F - s0), ldo, accumulate, row_div, st, scratch,
                                        scratch_floats, true);
                if (rc != SGNN_OK) return rc;
            }
            return SGNN_OK;
        }
    }
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
    const int nvec = (int)(F / vec);
    const int gw = group_width(nvec);
    const int which = gw == 8 ? 0 : gw == 16 ? 1 : 2;
    SGNN_REQUIRE(p->n_chunks[which] >= 0, "plan has no chunk list for this feature width (plan creation failed?)");
    ShortArgs a{p->rowptr, p->col, val, dense, out, p->chunks[which], (int)p->n_chunks[which], p->empty_rows,
                (int)p->n_empty, (int)F, ldo, accumulate, row_div, scratch == nullptr};
    PieceArgs s{p->col_long, p->eperm, val, partial, p->cls_work, p->max_cls_items, (int)F};
    if (val != nullptr && val == p->bound_val && p->val_long != nullptr) {
        s.eperm = nullptr;   // values already sit in regrouped order: contiguous reads, no indirection
        s.val = p->val_long;
    }
    FinalArgs f{p->long_rows, p->long_pbeg, partial, out, (int)p->n_long, (int)F, ldo, accumulate, row_div};
    if (bits != 0) {
        const int fmt = bits + (dense.params.bf16 ? kBf16Params : 0) + (dense.eslot_csr ? kEdgeSlots : 0);
        switch (fmt) {
#define SGNN_DQ(FMT) case FMT: dispatch_shape_dq<FMT>(vec, nvec, a, s, f, st); break
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
    for (size_t i = 0; i < p->parts.size(); ++i) {
        const int rc = sgnn_spmm_plan_bind_values(p->parts[i], val ? val + p->part_edge0[i] : nullptr, stream);
        if (rc != SGNN_OK) return rc;
    }
    if (!p->parts.empty()) return SGNN_OK;
    p->bound_val = nullptr;
    ++p->bind_gen;  // band schedules refill their value copies on their next use
    if (val == nullptr) return SGNN_OK;
    if (!p->partitioned || p->long_edges == 0) {  // nothing to regroup for the piece path
        p->bound_val = val;
        return SGNN_OK;
    }
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
    for (sgnn_spmm_plan *part : p->parts) {
        const int rc = sgnn_spmm_plan_bind_row_slots(part, row_slot, stream);
        if (rc != SGNN_OK) return rc;
    }
    if (!p->parts.empty()) {
        p->bound_slots = row_slot;
        return SGNN_OK;
    }
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
    SGNN_REQUIRE(F % 2 == 0, "the fused path needs an even feature width (F=%lld): dequantize, then call sgnn_spmm_csr_f32", (long long)F);
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
        if (!p->parts.empty()) {
            // "slots are bound": spmm_run takes each row block's own streams
            for (const sgnn_spmm_plan *part : p->parts)
                if (part->eslot_csr != nullptr) { d.eslot_csr = d.eslot_long = part->eslot_csr; break; }
        } else {
            d.eslot_csr = p->eslot_csr;
            d.eslot_long = p->eslot_long ? p->eslot_long : p->eslot_csr;  // unregrouped long rows index the CSR arrays
        }
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
