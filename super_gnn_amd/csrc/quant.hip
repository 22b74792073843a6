// Boundary-row quantize -> bit-pack -> unpack -> dequantize for gfx950.
//
// Row-group layout ("rows"): replaces quantize_tensor(_for_all_procs) / dequantize_tensor(_for_all_procs)
// of the reference (super_gnn/ops/csrc/quantization_arm.cpp:79-301, :303-431, :433-633).
// Feature-packed mixed-bit layout ("v1"): replaces quantize_tensor_v1 / dequantize_tensor_v1
// (quantization_arm.cpp:635-757).
//
// Every kernel here streams its input once and is bound by HBM bandwidth.  The fused
// quantize+pack kernel keeps the rows it packs in registers between the min/max reduction and the
// quantization, so the fp32 input is read from memory exactly once.
#include <algorithm>
#include <climits>
#include <cstdlib>

#include "common.hpp"

namespace sgnn {

constexpr int kQBlock = 256;
constexpr int kRowsPerGroup = 4;  // fp32 rows one lane group handles: keeps >= 4 loads in flight per lane

// ---- cross-lane helpers ---------------------------------------------------------------------
// DPP controls (GFX9): quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_mirror = 0x140,
// row_half_mirror = 0x141.  Four butterfly steps make a value uniform over each row of 16 lanes.
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xF, 0xF, false);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(dpp_i<CTRL>(__float_as_int(v)));
}

struct OpMinF { __device__ static float f(float a, float b) { return fminf(a, b); } };
struct OpMaxF { __device__ static float f(float a, float b) { return fmaxf(a, b); } };

// All-reduce over a group of G consecutive lanes (G in {1, 2, 4, 8, 16, 32, 64}); every lane gets the result.
template <int G, typename Op>
__device__ __forceinline__ float group_allreduce_f(float v) {
    if constexpr (G == 1) return v;
    v = Op::f(v, dpp_f<0xB1>(v));
    if constexpr (G == 2) return v;
    v = Op::f(v, dpp_f<0x4E>(v));
    if constexpr (G == 4) return v;
    v = Op::f(v, dpp_f<0x141>(v));
    if constexpr (G == 8) return v;
    v = Op::f(v, dpp_f<0x140>(v));
    if constexpr (G == 16) {
        return v;
    } else {
        const int iv = __float_as_int(v);
        const float a0 = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
        const float a1 = __int_as_float(__builtin_amdgcn_readlane(iv, 16));
        const float a2 = __int_as_float(__builtin_amdgcn_readlane(iv, 32));
        const float a3 = __int_as_float(__builtin_amdgcn_readlane(iv, 48));
        if constexpr (G == 32) {
            const float lo = Op::f(a0, a1), hi = Op::f(a2, a3);
            return (threadIdx.x & 32) ? hi : lo;
        } else {
            return Op::f(Op::f(a0, a1), Op::f(a2, a3));
        }
    }
}

template <int G>
__device__ __forceinline__ int group_allmin_i(int v) {
    if constexpr (G == 1) return v;
    v = min(v, dpp_i<0xB1>(v));
    if constexpr (G == 2) return v;
    v = min(v, dpp_i<0x4E>(v));
    if constexpr (G == 4) return v;
    v = min(v, dpp_i<0x141>(v));
    if constexpr (G == 8) return v;
    v = min(v, dpp_i<0x140>(v));
    if constexpr (G == 16) {
        return v;
    } else {
        const int a0 = __builtin_amdgcn_readlane(v, 0), a1 = __builtin_amdgcn_readlane(v, 16);
        const int a2 = __builtin_amdgcn_readlane(v, 32), a3 = __builtin_amdgcn_readlane(v, 48);
        if constexpr (G == 32) {
            const int lo = min(a0, a1), hi = min(a2, a3);
            return (threadIdx.x & 32) ? hi : lo;
        } else {
            return min(min(a0, a1), min(a2, a3));
        }
    }
}

// Segment of packed row gp: the p with pseg[p] <= gp < pseg[p+1].
__device__ __forceinline__ int find_segment(const int32_t *__restrict__ pseg, int P, int gp) {
    int lo = 0, hi = P - 1;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (pseg[mid + 1] > gp) hi = mid; else lo = mid + 1;
    }
    return lo;
}

// The segment p with keys[p] <= key < keys[p + 1] for a wave-uniform key (keys ascending, P + 1 entries,
// keys[0] <= key < keys[P]; empty segments allowed), with the segment's two ends in `keys` and in the companion
// table `other`.  Call it with all 64 lanes active.  Up to 63 segments cost one round of loads: lane i fetches
// entry i of both tables, a ballot counts the entries that do not exceed the key, and the four ends are read out
// of the lanes that hold them -- where a binary search makes log2(P) dependent loads, plus one more round for
// the ends, before a wavefront can issue its first data load (eight segments: quantize+pack of 4 M x 64 int2
// 0.218 -> 0.198 ms).  Longer tables are first narrowed to 63 segments by a binary search over every 63rd entry.
struct WaveSegment { int p, k0, k1, o0, o1; };
__device__ __forceinline__ WaveSegment wave_find_segment(const int32_t *__restrict__ keys, const int32_t *__restrict__ other,
                                                         int P, int key) {
    const int lane = threadIdx.x & 63;
    int base = 0;
    if (P > 63) {
        int lo = 0, hi = (P - 1) / 63;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (keys[mid * 63] <= key) lo = mid; else hi = mid - 1;
        }
        base = lo * 63;
    }
    const int idx = base + lane <= P ? base + lane : P;
    const int mk = keys[idx], mo = other[idx];
    int k = __popcll(__ballot(lane >= 1 && base + lane <= P && mk <= key));
    k = k > 62 ? 62 : k;
    WaveSegment w;
    w.p = base + k;
    w.k0 = __builtin_amdgcn_readlane(mk, k);
    w.k1 = __builtin_amdgcn_readlane(mk, k + 1);
    w.o0 = __builtin_amdgcn_readlane(mo, k);
    w.o1 = __builtin_amdgcn_readlane(mo, k + 1);
    return w;
}

// First fp32 row held by packed row g, and the end of the segment it belongs to.  With a single
// segment (single_rows >= 0, the row count) nothing is read from memory, so a wave's first loads are
// its data loads.  With several segments the table is searched once per wavefront, for g_wave (a
// wave-uniform packed row <= g, so the search runs on scalar loads), and only a lane whose packed
// row lies beyond that segment searches again on its own.
__device__ __forceinline__ void locate_packed_row(const int32_t *__restrict__ seg, const int32_t *__restrict__ pseg,
                                                  int P, int64_t single_rows, int g, int g_wave, int epb,
                                                  int64_t &row0, int64_t &rend) {
    if (single_rows >= 0) {
        row0 = (int64_t)g * epb;
        rend = single_rows;
        return;
    }
    const int pw = find_segment(pseg, P, g_wave);
    const int ps0 = pseg[pw], ps1 = pseg[pw + 1], s0 = seg[pw], s1 = seg[pw + 1];
    if (g < ps1) {
        row0 = (int64_t)s0 + (int64_t)(g - ps0) * epb;
        rend = s1;
    } else {
        const int p = find_segment(pseg, P, g);
        row0 = (int64_t)seg[p] + (int64_t)(g - pseg[p]) * epb;
        rend = seg[p + 1];
    }
}

// The same with the wavefront's segment already found (wave_find_segment on pseg with seg as the companion).
__device__ __forceinline__ void locate_packed_row_w(const int32_t *__restrict__ seg, const int32_t *__restrict__ pseg,
                                                    int P, int64_t single_rows, int g, const WaveSegment &w, int epb,
                                                    int64_t &row0, int64_t &rend) {
    if (single_rows >= 0) {
        row0 = (int64_t)g * epb;
        rend = single_rows;
    } else if (g < w.k1) {
        row0 = (int64_t)w.o0 + (int64_t)(g - w.k0) * epb;
        rend = w.o1;
    } else {
        const int p = find_segment(pseg, P, g);
        row0 = (int64_t)seg[p] + (int64_t)(g - pseg[p]) * epb;
        rend = seg[p + 1];
    }
}

// code = RNE((x - zp) / scale), IEEE subtraction and division (no reciprocal shortcut).
__device__ __forceinline__ uint32_t quant_code(float x, float zp, float sc) {
    const float q = (x - zp) / sc;
    return __float2uint_rn(q);  // saturating: NaN and negatives give 0
}

// ------------------------------------------------------------------------------------------------
// Fused quantize + pack, row-group layout.  One group of G lanes handles kRowsPerGroup fp32 rows
// (= 1 packed row at int2, 2 at int4, 4 at int8); G*VEC*NV >= F so a row lives in registers.
// ------------------------------------------------------------------------------------------------
// RAGGED (VEC == 4 only): any F and any 4-byte aligned row start -- 16-byte loads at their natural addresses, the
// vector that reaches past the end of the row read and written element by element (see quant_pack_rows16_kernel).
template <int BITS, int VEC, int G, int NV, bool kForceExactDivision, bool RAGGED = false>
__global__ __launch_bounds__(kQBlock) void quant_pack_rows_kernel(
    const RowSrc xs, uint8_t *__restrict__ q, const ParamBuf pb,
    const int32_t *__restrict__ seg, const int32_t *__restrict__ pseg, int P, int64_t single_rows, int n_packed, int F,
    int n_units) {
    constexpr int EPB = 8 / BITS;
    constexpr int R = kRowsPerGroup;
    constexpr int NPR = R / EPB;  // packed rows per group
    constexpr int GPB = kQBlock / G;
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int unit = blockIdx.x * GPB + gid;
    if (unit >= n_units) return;

    int64_t row[R];
    bool valid[R];
#pragma unroll
    for (int pi = 0; pi < NPR; ++pi) {
        const int gp = unit * NPR + pi;
        int64_t row0 = 0, rend = 0;
        if (gp < n_packed) {
            locate_packed_row(seg, pseg, P, single_rows, gp, __builtin_amdgcn_readfirstlane(gp), EPB, row0, rend);
        }
#pragma unroll
        for (int k = 0; k < EPB; ++k) {
            row[pi * EPB + k] = row0 + k;
            valid[pi * EPB + k] = row0 + k < rend;
        }
    }

    int off[NV];
    bool act[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        off[v] = (v * G + lig) * VEC;
        act[v] = off[v] < F;
    }

    float xv[R][NV][VEC];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (!valid[r]) continue;
        const float *xr = row_ptr(xs, row[r]);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
            if constexpr (RAGGED) {
                if (off[v] + VEC <= F) {
                    vec4_load_nt_unaligned(xv[r][v], xr + off[v]);
                } else {  // the row's short last vector: its elements one by one (padded below, once every load is out)
#pragma unroll
                    for (int k = 0; k < VEC; ++k)
                        if (off[v] + k < F) xv[r][v][k] = xr[off[v] + k];
                }
            } else {
                vec_load_nt<VEC>(xv[r][v], xr + off[v]);
            }
        }
    }
    if constexpr (RAGGED) {
        // missing elements: copies of the vector's first one (they change neither min nor max nor the first zero).  Done
        // after the loads: a use of a loaded value between two loads would make every load wait for the one before.
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                if (valid[r] && act[v] && off[v] + VEC > F) {
#pragma unroll
                    for (int k = 1; k < VEC; ++k)
                        if (off[v] + k >= F) xv[r][v][k] = xv[r][v][0];
                }
            }
        }
    }

    float zp[R], sc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        zp[r] = 0.0f;
        sc[r] = 1.0f;
        if (!valid[r]) continue;
        float mn = INFINITY, mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                mn = fminf(mn, xv[r][v][k]);
                mx = fmaxf(mx, xv[r][v][k]);
            }
        }
        mn = group_allreduce_f<G, OpMinF>(mn);
        mx = group_allreduce_f<G, OpMaxF>(mx);
        if (mn == 0.0f || mx == 0.0f) {
            // Among compare-equal zeros the reference keeps the FIRST one it meets
            // (strict compares, quantization_arm.cpp:98-101): recover that zero's sign.
            int key = INT_MAX;
#pragma unroll
            for (int v = NV - 1; v >= 0; --v) {
                if (!act[v]) continue;
#pragma unroll
                for (int k = VEC - 1; k >= 0; --k)
                    if (xv[r][v][k] == 0.0f) key = ((off[v] + k) << 1) | (int)(__float_as_uint(xv[r][v][k]) >> 31);
            }
            key = group_allmin_i<G>(key);
            const float z = (key & 1) ? -0.0f : 0.0f;
            if (mn == 0.0f) mn = z;
            if (mx == 0.0f) mx = z;
        }
        // A NaN is sticky only as element 0 (every later compare against it is false).
        const unsigned long long nanmask = __ballot(lig == 0 && xv[r][0][0] != xv[r][0][0]);
        if ((nanmask >> (threadIdx.x & 63 & ~(G - 1))) & 1ull) {
            mn = __int_as_float(0x7fc00000);
            mx = mn;
        }
        float s = (mx - mn) / (float)((1 << BITS) - 1);
        if (s == 0.0f) s = 1.0f;
        zp[r] = mn;
        sc[r] = s;
        if (lig == 0) store_params(pb, row[r], mn, s);
    }

    // Codes.  The reference's code is RNE(RN((x - zp) / scale)).  A correctly rounded fp32 division
    // costs ~15 instructions per element, which would make this streaming kernel ALU-bound, so the
    // quotient is first formed as (x - zp) * RN(1/scale): that product is within 2^-23 relative of
    // the true quotient, the IEEE quotient within 2^-24, and both are below 256, so the two differ
    // by less than 2^-14.  If the product is further than 2^-14 from every half-integer, rounding
    // it gives the same integer as rounding the IEEE quotient.  Any lane that sees an element
    // inside that guard band (about 1 in 8000), or a row whose scale is outside the range where
    // the reciprocal is a normal number, recomputes its elements with the IEEE division, so the
    // stored bytes are always those of the exact formula.
    float rinv[R];
    bool lane_exact = kForceExactDivision;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        rinv[r] = 1.0f / sc[r];
        if (valid[r] && !(sc[r] >= 0x1p-100f && sc[r] <= 0x1p100f)) lane_exact = true;
    }
    uint32_t words[NPR][NV];
#pragma unroll
    for (int pi = 0; pi < NPR; ++pi) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            uint32_t word = 0;
            if (act[v]) {
#pragma unroll
                for (int k = 0; k < EPB; ++k) {
                    const int r = pi * EPB + k;
                    if (!valid[r]) continue;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float qf = (xv[r][v][e] - zp[r]) * rinv[r];
                        const float ri = rintf(qf);
                        if (!(fabsf(qf - ri) < 0.5f - 0x1p-14f)) lane_exact = true;
                        word |= (uint32_t)ri << (8 * e + (EPB - 1 - k) * BITS);
                    }
                }
            }
            words[pi][v] = word;
        }
    }
    if (lane_exact) {
#pragma unroll
        for (int pi = 0; pi < NPR; ++pi) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                uint32_t word = 0;
                if (act[v]) {
#pragma unroll
                    for (int k = 0; k < EPB; ++k) {
                        const int r = pi * EPB + k;
                        if (!valid[r]) continue;
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            word |= quant_code(xv[r][v][e], zp[r], sc[r]) << (8 * e + (EPB - 1 - k) * BITS);
                    }
                }
                words[pi][v] = word;
            }
        }
    }
#pragma unroll
    for (int pi = 0; pi < NPR; ++pi) {
        const int gp = unit * NPR + pi;
        if (gp >= n_packed) continue;
        uint8_t *qr = q + (int64_t)gp * F;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
            const uint32_t word = words[pi][v];
            if constexpr (RAGGED) {
                uint8_t *dst = qr + off[v];
                const uintptr_t al = reinterpret_cast<uintptr_t>(dst) & 3;
                if (off[v] + VEC <= F && al == 0) {
                    __builtin_nontemporal_store(word, reinterpret_cast<uint32_t *>(dst));
                } else if (off[v] + VEC <= F && al == 2) {
                    __builtin_nontemporal_store((uint16_t)word, reinterpret_cast<uint16_t *>(dst));
                    __builtin_nontemporal_store((uint16_t)(word >> 16), reinterpret_cast<uint16_t *>(dst) + 1);
                } else {
                    for (int k = 0; k < VEC && off[v] + k < F; ++k) dst[k] = (uint8_t)(word >> (8 * k));
                }
            } else if constexpr (VEC == 4) __builtin_nontemporal_store(word, reinterpret_cast<uint32_t *>(qr + off[v]));
            else if constexpr (VEC == 2) __builtin_nontemporal_store((uint16_t)word, reinterpret_cast<uint16_t *>(qr + off[v]));
            else qr[off[v]] = (uint8_t)word;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Fused quantize + pack, row-group layout, one fp32 row per L = 16 lanes (float4 lanes, F <= 1024) or,
// for rows of up to 128 floats, per L = 8 lanes.
//
// L lanes inside one 16-lane DPP row own one fp32 row (NV float4 per lane), so the per-row min/max
// reductions are four (three) DPP butterfly steps with no cross-row traffic, and the per-row scalars
// (zero_point, scale, reciprocal) are computed once per lane instead of once per row per lane.  A wavefront
// handles 64/L * RL consecutive rows (RL rows per lane, chosen so that every lane keeps >= 4 loads in
// flight); neighbouring lane groups hold consecutive fp32 rows, i.e. exactly the rows that share a packed
// byte (four at int2, two at int4), so packing is a shift in each lane followed by an OR across lane
// groups.  Narrow rows take L = 8: the work per row (reductions, scale, reciprocal, parameter store) is
// then spread over twice as many elements per lane, which is what limits rows of 64 and 128 floats.  Rows
// of at most 16, 8 and 4 floats take L = 4, 2 and 1, so that a lane group has no idle lanes.
// ------------------------------------------------------------------------------------------------
// FULL: F == 4 * L * NV, every lane's every vector lies inside the row (no per-load lane predicates).
// RAGGED: any F and any 4-byte aligned row start (F = 602, F = 123, a window with an odd leading dimension):
// the float4 loads and the 4-byte code stores are issued at their natural (unaligned) addresses, and the one
// vector per row that reaches past the end of the row is loaded and stored element by element, its missing
// elements filled with copies of its first one (copies change neither min nor max nor the first-zero rule).
// STAGED: the packed bytes of a wavefront (RL * 64 / L consecutive fp32 rows = consecutive packed rows, one
// contiguous run of the output) first go to a wave-private piece of LDS and are then written with 4-byte stores
// over that run, 256 consecutive bytes per store instruction, instead of one 64-byte piece per lane group and
// vector.  For rows that do not start on cache lines the many short, oddly aligned pieces are what limits the
// kernel (F = 602 int2: 5.2 -> 6.4 TB/s with the output redirected into a cache-resident window).
constexpr int kStageBytes = 4096 + 16;  // per wavefront: at most 4 packed rows of 1024 bytes (int8, F = 1024)
template <int BITS, int NV, int RL, bool kForceExactDivision, bool FULL = false, int L = 16, bool RAGGED = false,
          bool STAGED = false>
__global__ __launch_bounds__(kQBlock) void quant_pack_rows16_kernel(
    const RowSrc xs, uint8_t *__restrict__ q, const ParamBuf pb,
    const int32_t *__restrict__ seg, const int32_t *__restrict__ pseg, int P, int64_t single_rows, int n_packed, int F,
    int n_units) {
    constexpr int EPB = 8 / BITS;
    constexpr int VEC = 4;
    constexpr int RW = 64 / L;  // fp32 rows of a wavefront per round
    const int lane = threadIdx.x & 63, d = lane / L, l16 = lane % L;  // lane group (= row) inside the wavefront, lane inside the group
    const int unit = blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    if (unit >= n_units) return;  // wave-uniform

    int64_t row[RL];
    bool valid[RL];
    int gp[RL];
    WaveSegment ws{0, 0, 0, 0, 0};
    const int unit_w = __builtin_amdgcn_readfirstlane(unit);
    if (single_rows < 0) ws = wave_find_segment(pseg, seg, P, (unit_w * RL * RW) / EPB);  // wave-uniform branch
#pragma unroll
    for (int rl = 0; rl < RL; ++rl) {
        const int pr = (unit * RL + rl) * RW + d;  // row index in the padded (EPB rows per packed row) space
        const int g = pr / EPB, k = pr % EPB;
        gp[rl] = g;
        valid[rl] = false;
        row[rl] = 0;
        if (rl > 0 && single_rows < 0) {  // a later round that starts beyond the segment found: look again (wave-uniform)
            const int g_first = ((unit_w * RL + rl) * RW) / EPB;
            if (g_first >= ws.k1 && g_first < n_packed) ws = wave_find_segment(pseg, seg, P, g_first);
        }
        if (g < n_packed) {
            int64_t row0, rend;
            locate_packed_row_w(seg, pseg, P, single_rows, g, ws, EPB, row0, rend);
            row[rl] = row0 + k;
            valid[rl] = row[rl] < rend;
        }
    }
    int off[NV];
    bool act[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        off[v] = (v * L + l16) * VEC;
        act[v] = FULL ? true : off[v] < F;
    }
    float xv[RL][NV][VEC];
#pragma unroll
    for (int rl = 0; rl < RL; ++rl) {
        if (!valid[rl]) continue;
        const float *xr = row_ptr(xs, row[rl]);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
            if constexpr (RAGGED) {
                if (off[v] + VEC <= F) {
                    vec4_load_nt_unaligned(xv[rl][v], xr + off[v]);
                } else {  // the row's short last vector: its elements one by one (padded below, once every load is out)
#pragma unroll
                    for (int k = 0; k < VEC; ++k)
                        if (off[v] + k < F) xv[rl][v][k] = xr[off[v] + k];
                }
            } else {
                vec_load_nt<VEC>(xv[rl][v], xr + off[v]);
            }
        }
    }
    if constexpr (RAGGED) {
        // missing elements: copies of the vector's first one.  Done after the loads: a use of a loaded value between two
        // loads would make every load wait for the one before.
#pragma unroll
        for (int rl = 0; rl < RL; ++rl) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                if (valid[rl] && act[v] && off[v] + VEC > F) {
#pragma unroll
                    for (int k = 1; k < VEC; ++k)
                        if (off[v] + k >= F) xv[rl][v][k] = xv[rl][v][0];
                }
            }
        }
    }

    float zp[RL], sc[RL], rinv[RL];
    bool lane_exact = kForceExactDivision;
#pragma unroll
    for (int rl = 0; rl < RL; ++rl) {
        zp[rl] = 0.0f;
        sc[rl] = 1.0f;
        rinv[rl] = 1.0f;
        if (!valid[rl]) continue;  // uniform within a DPP row: the row-level DPP steps below see full rows
        float mn = INFINITY, mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                mn = fminf(mn, xv[rl][v][k]);
                mx = fmaxf(mx, xv[rl][v][k]);
            }
        }
        mn = group_allreduce_f<L, OpMinF>(mn);
        mx = group_allreduce_f<L, OpMaxF>(mx);
        if (mn == 0.0f || mx == 0.0f) {
            // first-occurrence rule for compare-equal zeros (quantization_arm.cpp:98-101)
            int key = INT_MAX;
#pragma unroll
            for (int v = NV - 1; v >= 0; --v) {
                if (!act[v]) continue;
#pragma unroll
                for (int k = VEC - 1; k >= 0; --k)
                    if (xv[rl][v][k] == 0.0f) key = ((off[v] + k) << 1) | (int)(__float_as_uint(xv[rl][v][k]) >> 31);
            }
            key = group_allmin_i<L>(key);
            const float z = (key & 1) ? -0.0f : 0.0f;
            if (mn == 0.0f) mn = z;
            if (mx == 0.0f) mx = z;
        }
        // a NaN is sticky only as element 0, which lane 0 of the lane group holds
        const unsigned long long nanmask = __ballot(l16 == 0 && xv[rl][0][0] != xv[rl][0][0]);
        if ((nanmask >> (lane & ~(L - 1))) & 1ull) {
            mn = __int_as_float(0x7fc00000);
            mx = mn;
        }
        float s = (mx - mn) / (float)((1 << BITS) - 1);
        if (s == 0.0f) s = 1.0f;
        zp[rl] = mn;
        sc[rl] = s;
        rinv[rl] = __builtin_amdgcn_rcpf(s);  // hardware reciprocal, within 1 ulp of 1/s
        if (!(s >= 0x1p-100f && s <= 0x1p100f)) lane_exact = true;
        if (l16 == 0) store_params(pb, row[rl], mn, s);
    }

    // Codes.  The reference's code is RNE(RN(d / scale)) with d = RN(x - zp).  The quotient is first formed
    // as RN(d * r) with r the hardware reciprocal of the scale (within 1 ulp of 1/scale): d * r differs from
    // d / scale by at most 2^-23 relative, and each of the two roundings adds 2^-24, so the product and the
    // IEEE quotient differ by less than 2^-22 relative -- in absolute terms less than qmax * 2^-22, since
    // neither exceeds qmax = 2^bits - 1 by more than a rounding: 2^-14 at int8, 2^-18.1 at int4, 2^-20.4 at
    // int2.  If the product is further than kGuard (twice that bound or more) from every half-integer,
    // rounding it gives the same integer as rounding the IEEE quotient; a lane that sees an element inside
    // the guard band (1 element in 4000 at int8, 1 in 33 000 at int4, 1 in 130 000 at int2), or a scale whose
    // reciprocal is not a normal number, redoes its elements with the IEEE division.  The stored bytes are
    // always the exact formula's.
    constexpr float kGuard = BITS == 8 ? 0x1p-13f : BITS == 4 ? 0x1p-17f : 0x1p-19f;
    const int shift = (EPB - 1 - (d % EPB)) * BITS;
    uint32_t words[RL][NV];
#pragma unroll
    for (int rl = 0; rl < RL; ++rl) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            uint32_t word = 0;
            if (valid[rl] && act[v]) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float qf = (xv[rl][v][e] - zp[rl]) * rinv[rl];
                    const float ri = rintf(qf);
                    if (!(fabsf(qf - ri) < 0.5f - kGuard)) lane_exact = true;  // also true for a NaN quotient
                    // ri is an integer in [0, 255] whenever the lane stays on this path: one instruction
                    // converts it and drops it into byte e of the word
                    word = __builtin_amdgcn_cvt_pk_u8_f32(ri, e, word);
                }
            }
            words[rl][v] = word;
        }
    }
    if (lane_exact) {
#pragma unroll
        for (int rl = 0; rl < RL; ++rl) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                uint32_t word = 0;
                if (valid[rl] && act[v]) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) word |= quant_code(xv[rl][v][e], zp[rl], sc[rl]) << (8 * e);
                }
                words[rl][v] = word;
            }
        }
    }
    // Pack: shift to the row's bit position, OR across the DPP rows that share a packed row, store.
    __shared__ __align__(16) uint8_t stage_all[STAGED ? kQBlock / 64 : 1][STAGED ? kStageBytes : 16];
    uint8_t *stage = stage_all[STAGED ? (threadIdx.x >> 6) : 0];
    const int gp_first = (unit * RL * RW) / EPB;                       // the wavefront's first packed row
    const int64_t run_lo = (int64_t)gp_first * F;                      // byte offset of its output run
    const int mis = (int)((reinterpret_cast<uintptr_t>(q) + (uint64_t)run_lo) & 3);  // the LDS copy keeps the run's alignment modulo 4
#pragma unroll
    for (int rl = 0; rl < RL; ++rl) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            uint32_t w = words[rl][v] << shift;
            if constexpr (L == 16) {
                if constexpr (EPB >= 2) w |= (uint32_t)__shfl_xor((int)w, 16, 64);
                if constexpr (EPB == 4) w |= (uint32_t)__shfl_xor((int)w, 32, 64);
            } else if constexpr (L == 8) {  // the neighbouring row sits in the other half of the DPP row (row_ror:8 swaps the halves)
                if constexpr (EPB >= 2) w |= (uint32_t)dpp_i<0x128>((int)w);
                if constexpr (EPB == 4) w |= (uint32_t)__shfl_xor((int)w, 16, 64);
            } else {  // L lanes per row, L in {1, 2, 4}: the rows of a packed byte sit L and 2 L lanes apart
                if constexpr (EPB >= 2) w |= (uint32_t)__shfl_xor((int)w, L, 64);
                if constexpr (EPB == 4) w |= (uint32_t)__shfl_xor((int)w, 2 * L, 64);
            }
            const bool mine = EPB == 1 ? true : EPB == 2 ? ((d & 1) == (v & 1)) : ((d & 3) == (v & 3));
            if constexpr (STAGED) {
                if (mine && act[v] && gp[rl] < n_packed) {
                    uint8_t *dst = stage + mis + (gp[rl] - gp_first) * F + off[v];
                    const int nb = RAGGED ? (F - off[v] < VEC ? F - off[v] : VEC) : VEC;
                    const uintptr_t al = reinterpret_cast<uintptr_t>(dst) & 3;
                    if (nb == VEC && al == 0) {
                        *reinterpret_cast<uint32_t *>(dst) = w;
                    } else if (nb == VEC && al == 2) {
                        reinterpret_cast<uint16_t *>(dst)[0] = (uint16_t)w;
                        reinterpret_cast<uint16_t *>(dst)[1] = (uint16_t)(w >> 16);
                    } else {
                        for (int k = 0; k < nb; ++k) dst[k] = (uint8_t)(w >> (8 * k));
                    }
                }
                continue;
            }
            if (mine && act[v] && gp[rl] < n_packed) {
                uint8_t *dst = q + (int64_t)gp[rl] * F + off[v];
                if constexpr (RAGGED) {
                    if (off[v] + VEC <= F) {
                        // a 4-byte store that is not 4-byte aligned is slower than two aligned 2-byte stores
                        const uintptr_t al = reinterpret_cast<uintptr_t>(dst) & 3;
                        if (al == 0) {
                            __builtin_nontemporal_store(w, reinterpret_cast<uint32_t *>(dst));
                        } else if (al == 2) {
                            __builtin_nontemporal_store((uint16_t)w, reinterpret_cast<uint16_t *>(dst));
                            __builtin_nontemporal_store((uint16_t)(w >> 16), reinterpret_cast<uint16_t *>(dst) + 1);
                        } else {
                            for (int k = 0; k < 4; ++k) dst[k] = (uint8_t)(w >> (8 * k));
                        }
                    } else {
                        for (int k = 0; off[v] + k < F; ++k) dst[k] = (uint8_t)(w >> (8 * k));
                    }
                } else {
                    __builtin_nontemporal_store(w, reinterpret_cast<uint32_t *>(dst));
                }
            }
        }
    }
    if constexpr (STAGED) {
        // LDS operations of one wavefront complete in program order; the fence keeps the compiler from moving
        // the reads below above the writes of other lanes.
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        int gp_end = gp_first + RL * RW / EPB;
        if (gp_end > n_packed) gp_end = n_packed;
        const int nbytes = (gp_end - gp_first) * F;                    // the run [run_lo, run_lo + nbytes)
        uint8_t *qo = q + run_lo;
        int head = (4 - mis) & 3;
        if (head > nbytes) head = nbytes;
        const int ndw = (nbytes - head) >> 2;
        const int tail_bytes = nbytes - head - 4 * ndw;
        if (lane < head) qo[lane] = stage[mis + lane];
        const uint32_t *s32 = reinterpret_cast<const uint32_t *>(stage + mis + head);   // (mis + head) % 4 == 0 whenever ndw > 0
        uint32_t *q32 = reinterpret_cast<uint32_t *>(qo + head);
        for (int i = lane; i < ndw; i += 64) __builtin_nontemporal_store(s32[i], q32 + i);
        if (lane < tail_bytes) qo[head + 4 * ndw + lane] = stage[mis + head + 4 * ndw + lane];
    }
}

// ------------------------------------------------------------------------------------------------
// Fused quantize + pack over a run of consecutive row slots: any row width from 9 floats; the rows themselves are
// consecutive in memory (the fast case) or found through a table (a row index, a pitch, a chunk across two segments).
//
// A wavefront takes `gw` consecutive packed rows, i.e. gw * EPB fp32 rows (at most 64), which lie one after the
// other in memory.  Each row is cut into VPR = ceil(F / 4) float4 vectors and the chunk's rows * VPR vectors are
// dealt to the lanes in order: lane l holds vectors l, l + 64, ... .  A load instruction therefore fetches 64
// consecutive vectors -- 1 KB of consecutive bytes when F % 4 == 0, a few rows' worth of them otherwise -- and no
// lane slot idles because a row is not a whole number of lane-group passes (the lane-group kernels leave 25 of 32
// slots busy at F = 100).  What those kernels get from their fixed row -> lane mapping goes through a
// wave-private piece of LDS here:
//   A  every lane reduces each of its vectors to (min, max) and writes the pair to LDS;
//   B  the lanes are regrouped, 64 / rows lanes per row: each group reduces its row's pairs, computes zero_point,
//      scale and the reciprocal, stores the params and leaves them in a row table in LDS;
//   C  every lane quantizes its vectors with their rows' table entries and writes the four code bytes of each
//      to a code array in LDS (int8 with F % 4 == 0: straight to memory);
//   D  the lanes walk the output run (gw * F consecutive bytes) in aligned 4-byte words, 256 bytes per store
//      instruction: a word is the OR of the EPB rows' code words, fetched from the code array at their byte
//      offsets and shifted to their bit positions.
// The last vector of a row with F % 4 != 0 is loaded whole (it reaches into the next row) and, once every load is
// out, cut back to its F % 4 elements and padded with copies of its first element (copies change neither min nor
// max nor the first-zero rule).  Vector slots behind the chunk's last row (the rest of the lane's last vector or
// two, or the row slots a segment's short last group leaves empty) repeat the chunk's last vector, so that no load
// needs a predicate; phase B never reads their pairs and phase C clears their code words.
// The kernel is sized so that it waits on memory and not on instruction issue (~66 vector instructions per float4
// at int2): no lane predicates or row bookkeeping around the loads (the row slot of a vector is one 24-bit
// multiply), the rule for a NaN as a row's first element looked at only when some vector starts with a NaN, one
// guard-band test per lane instead of one per element.
// Signed zeros: v_min_f32 / v_max_f32 order -0 < +0, so a zero minimum is -0 exactly when the row holds a -0
// and a zero maximum is +0 exactly when it holds a +0; the sign of the row's FIRST zero (what the reference's
// strict compares keep, quantization_arm.cpp:98-101) needs a second pass over the elements only when a row
// may hold zeros of both signs.
// ------------------------------------------------------------------------------------------------
// v_min_f32 / v_max_f32 as they are: fminf / fmaxf quiet their operands first (one more instruction each), which
// results of earlier min / max operations do not need.  A NaN operand loses against a number, as in fminf / fmaxf.
__device__ __forceinline__ float min_bare(float a, float b) {
    float r;
    asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float max_bare(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
constexpr int kStreamRows = 64;   // fp32 rows per wavefront chunk, at most (one lane per row in the set-up)
// Four bytes of LDS at any byte address: gfx950's LDS serves a misaligned 32-bit access in one instruction.
__device__ __forceinline__ uint32_t lds_load_u32_unaligned(const uint8_t *p) {
    typedef uint32_t u32u __attribute__((aligned(1)));
    return *reinterpret_cast<const u32u *>(p);
}
__device__ __forceinline__ void lds_store_u32_unaligned(uint8_t *p, uint32_t v) {
    typedef uint32_t u32u __attribute__((aligned(1)));
    *reinterpret_cast<u32u *>(p) = v;
}
__host__ __device__ constexpr int stream_wave_bytes(int nv) {
    // (min, max) pair per vector -- later the code bytes, which need half of it (+ 16 for the funnel reads) --, row
    // table (float4; empty row slots keep a neutral entry), row ids, row flags, source rows
    return nv * 512 + 16 + kStreamRows * 16 + kStreamRows * (4 + 4 + 4);
}

// RAGGED: F % 4 != 0, or an output buffer that is not 4-byte aligned.
template <int BITS, int NV, bool RAGGED, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void quant_pack_stream_kernel(
    const RowSrc xs, uint8_t *__restrict__ q, const ParamBuf pb, const int32_t *__restrict__ seg,
    const int32_t *__restrict__ pseg, int P, int64_t single_rows, int n_packed, int F, int gw, int n_units,
    uint32_t vpr_magic) {
    constexpr int EPB = 8 / BITS;
    constexpr int kWaveBytes = stream_wave_bytes(NV);
    const float *__restrict__ x = xs.x;
    const int n_rows = (int)xs.n_src;   // rows of the source tensor (the launcher keeps them below 2^31)
    static_assert(kWaveBytes % 16 == 0, "wave pieces of LDS must keep 16-byte alignment");
    static_assert(WAVES * kWaveBytes <= 64 * 1024, "static LDS of a workgroup");
    __shared__ __align__(16) uint8_t lds_all[WAVES * kWaveBytes];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int unit = blockIdx.x * WAVES + wv;
    if (unit >= n_units) return;   // wave-uniform
    uint8_t *base = lds_all + wv * kWaveBytes;
    float2 *ent = reinterpret_cast<float2 *>(base);
    float4 *rowtab = reinterpret_cast<float4 *>(base + NV * 512 + 16);   // (zero_point, scale, 1 / scale, needs the exact division)
    int *rowid = reinterpret_cast<int *>(rowtab + kStreamRows);   // the row whose params a row slot writes, -1: empty slot
    int *rowflag = rowid + kStreamRows;
    int *rowsrc = rowflag + kStreamRows;                                // the row of x it reads (the same without a row index)
    uint8_t *codes = base;   // the pairs are dead by the time the codes are written

    const int g0 = __builtin_amdgcn_readfirstlane(unit) * gw;
    const int ng = n_packed - g0 < gw ? n_packed - g0 : gw;
    const int npr = ng * EPB;          // fp32 row slots of the chunk (the last group of a segment may leave some empty)
    const int VPR = (F + 3) >> 2;      // vectors per row; npr * VPR <= NV * 64

    // ---- the chunk's rows: lane i looks up row slot i --------------------------------------------------------
    int my_row = -1, my_src = -1;
    {
        WaveSegment ws{0, 0, 0, 0, 0};
        if (single_rows < 0) ws = wave_find_segment(pseg, seg, P, g0);
        if (lane < npr) {
            int64_t row0, rend;
            locate_packed_row_w(seg, pseg, P, single_rows, g0 + lane / EPB, ws, EPB, row0, rend);
            const int64_t r = row0 + lane % EPB;
            if (r < rend) my_row = (int)r;
        }
        my_src = my_row;
        if (xs.index != nullptr && my_row >= 0) {
            const int64_t r = xs.index[my_row];
            my_src = (uint64_t)r < (uint64_t)xs.n_src ? (int)r : 0;   // (as row_ptr() treats an index out of range)
        }
        rowid[lane] = my_row;
        rowsrc[lane] = my_src;
        rowflag[lane] = 0;
        rowtab[lane] = make_float4(0.0f, 1.0f, 1.0f, 0.0f);
    }
    const unsigned long long vb = __ballot(my_row >= 0);
    const int n_valid = __popcll(vb);
    const int r_first = __builtin_amdgcn_readfirstlane(my_row);
    // rows consecutive in memory, empty slots only at the end: row slot p holds row r_first + p for p < n_valid
    const bool run = xs.index == nullptr && xs.ld == F && (vb & (vb + 1)) == 0 && (vb & 1) &&
                     __ballot(my_row >= 0 && my_row != r_first + lane) == 0;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");

    // ---- loads ------------------------------------------------------------------------------------------------
    // Vector slot v * 64 + lane of the chunk is vector (slot % VPR) of row slot (slot / VPR); the quotient comes from
    // one 24-bit multiply (vpr_magic = ceil(2^21 / VPR), exact for slot * VPR < 2^21).
    int prv[NV];
    float xv[NV][4];
    // run: slots up to `last` hold vectors; the slots behind them (the rest of the last one or two of the lane's
    // vectors) repeat the last vector, so that their loads need no predicate, and their code words are cleared in C.
    const int n_sv = run ? n_valid * VPR : 0;
    const int last = run ? n_sv - 1 : INT_MAX;
    const int n_full = run ? n_sv >> 6 : NV;   // the lane's vectors below this index are real in every lane (wave-uniform)
    uint32_t dead_mask = 0;                    // table path: bit v = the lane's vector v belongs to no row
    if (run) {
        // The common case: one base address, 32-bit element offsets, every vector a 16-byte load -- a row's short last
        // vector too, which then reaches into the next row and is cut back after all loads are out; only the one that
        // would reach past the end of the tensor is moved back to end with it.
        const float *xb = x + (int64_t)r_first * F;
        // (a chunk is far smaller than 2^31 elements; the rest of the tensor need not be)
        const int64_t e_rest = (int64_t)(n_rows - r_first) * F - 4;
        const uint32_t eo_max = e_rest < 0x7fffffff ? (uint32_t)e_rest : 0x7fffffffu;
        const int pad = 4 * VPR - F;   // elements a row's last vector lacks
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int sl = v * 64 + lane < last ? v * 64 + lane : last;
            const int pr = (int)(__umul24((uint32_t)sl, vpr_magic) >> 21);
            prv[v] = pr;
            uint32_t eo = 4u * (uint32_t)sl;
            if constexpr (RAGGED) {
                eo -= (uint32_t)(pr * pad);
                eo = eo < eo_max ? eo : eo_max;
            }
            // (a 32-bit byte offset from the chunk's first row: base register + lane offset addressing)
            vec4_load_nt_unaligned(xv[v], reinterpret_cast<const float *>(reinterpret_cast<const char *>(xb) + 4u * eo));
        }
        if constexpr (RAGGED) {
            const int nt = F & 3;
            if (nt != 0) {   // cut the short vectors back to their F % 4 elements, padded with copies of the first
                if (r_first + n_valid == n_rows) {   // the tensor's last vector was loaded `pad` elements early
#pragma unroll
                    for (int v = 0; v < NV; ++v) {
                        const int sl = v * 64 + lane < last ? v * 64 + lane : last;
                        if (sl == last) {
                            const float a1 = xv[v][1], a2 = xv[v][2], a3 = xv[v][3];
                            xv[v][0] = pad == 1 ? a1 : pad == 2 ? a2 : a3;
                            xv[v][1] = pad == 1 ? a2 : a3;
                            xv[v][2] = a3;
                        }
                    }
                }
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    const int sl = v * 64 + lane < last ? v * 64 + lane : last;
                    const bool sh = sl - prv[v] * VPR == VPR - 1;
#pragma unroll
                    for (int t = 1; t < 4; ++t) xv[v][t] = (sh && t >= nt) ? xv[v][0] : xv[v][t];
                }
            }
        }
    } else {
        // Rows anywhere -- a row index, rows with a pitch, a chunk that spans the end of a segment: every vector finds
        // its row in the chunk's table.  Slots of empty row slots and behind the chunk read the chunk's first row
        // (their codes are cleared in C), so that here too no load needs a predicate.
        const int src_any = __builtin_amdgcn_readlane(my_src, __builtin_ctzll(vb));   // some row of the chunk (vb != 0)
        const int n_sl = npr * VPR;
        const int pad = 4 * VPR - F;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int sl = v * 64 + lane < n_sl ? v * 64 + lane : n_sl - 1;
            const int pr = (int)(__umul24((uint32_t)sl, vpr_magic) >> 21);
            const int cv = sl - pr * VPR;
            prv[v] = pr;
            int src = rowsrc[pr];
            if (src < 0 || v * 64 + lane >= n_sl) dead_mask |= 1u << v;
            if (src < 0) src = src_any;
            int64_t eo = (int64_t)src * xs.ld + 4 * cv;
            // the short last vector of the tensor's last row is loaded `pad` elements early (cut back below)
            if (RAGGED && pad != 0 && cv == VPR - 1 && src == n_rows - 1) eo -= pad;
            vec4_load_nt_unaligned(xv[v], x + eo);
        }
        if constexpr (RAGGED) {
            const int nt = F & 3;
            if (nt != 0) {
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    const int sl = v * 64 + lane < n_sl ? v * 64 + lane : n_sl - 1;
                    const bool sh = sl - prv[v] * VPR == VPR - 1;
                    if (sh && rowsrc[prv[v]] == n_rows - 1) {
                        const float a1 = xv[v][1], a2 = xv[v][2], a3 = xv[v][3];
                        xv[v][0] = pad == 1 ? a1 : pad == 2 ? a2 : a3;
                        xv[v][1] = pad == 1 ? a2 : a3;
                        xv[v][2] = a3;
                    }
#pragma unroll
                    for (int t = 1; t < 4; ++t) xv[v][t] = (sh && t >= nt) ? xv[v][0] : xv[v][t];
                }
            }
        }
    }

    // ---- A: (min, max) of every vector -----------------------------------------------------------------------
    bool nan0 = false;   // a NaN is sticky only as element 0 of its row: look closer when some vector starts with one
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const float m = fminf(fminf(xv[v][0], xv[v][1]), fminf(xv[v][2], xv[v][3]));
        const float M = fmaxf(fmaxf(xv[v][0], xv[v][1]), fmaxf(xv[v][2], xv[v][3]));
        ent[v * 64 + lane] = make_float2(m, M);
        nan0 |= xv[v][0] != xv[v][0];
    }
    if (__ballot(nan0) != 0) {   // wave-uniform, rare
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int sl = v * 64 + lane;
            if (sl <= last && !((dead_mask >> v) & 1u) && sl - prv[v] * VPR == 0 && xv[v][0] != xv[v][0]) rowflag[prv[v]] = 1;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ---- B: per-row reduction, LR lanes per row --------------------------------------------------------------
    int lr_shift = 0;   // LR = largest power of two <= 64 / npr
    while ((npr << (lr_shift + 1)) <= 64) ++lr_shift;
    const int LR = 1 << lr_shift;
    const int row_b = lane >> lr_shift, li = lane & (LR - 1);
    const bool has_row = row_b < npr;
    const int e_lo = has_row ? row_b * VPR : 0, e_hi = has_row ? e_lo + VPR : 0;   // the row's vectors
    float mn = INFINITY, mx = -INFINITY;
    // (the pairs are results of min / max already: the bare instructions, without a quieting pass over their operands)
    for (int e = e_lo + li; e < e_hi; e += LR) {
        const float2 p = ent[e];
        mn = min_bare(mn, p.x);
        mx = max_bare(mx, p.y);
    }
    for (int o = 1; o < LR; o <<= 1) {
        mn = min_bare(mn, __shfl_xor(mn, o, 64));
        mx = max_bare(mx, __shfl_xor(mx, o, 64));
    }
    const bool row_valid = has_row && rowid[has_row ? row_b : 0] >= 0;
    // the sign of the row's first zero, where both signs may occur (see the header)
    {
        const bool mn0 = mn == 0.0f, mx0 = mx == 0.0f;
        const bool neg0 = mn0 && (__float_as_uint(mn) >> 31) != 0;     // the row holds a -0 (known when mn == 0)
        const bool pos0 = mx0 && (__float_as_uint(mx) >> 31) == 0;     // the row holds a +0 (known when mx == 0)
        const bool unsure = row_valid && ((mn0 && neg0 && !(mx0 && !pos0)) || (mx0 && pos0 && !(mn0 && !neg0)));
        if (__ballot(unsure) != 0) {   // wave-uniform, rare: first zero of every row by position
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                int k0 = INT_MAX;
#pragma unroll
                for (int t = 3; t >= 0; --t)
                    if (xv[v][t] == 0.0f) k0 = (((v * 64 + lane) * 4 + t) << 1) | (int)(__float_as_uint(xv[v][t]) >> 31);
                ent[v * 64 + lane].x = __int_as_float(k0);
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            int key = INT_MAX;
            for (int e = e_lo + li; e < e_hi; e += LR) key = min(key, __float_as_int(ent[e].x));
            for (int o = 1; o < LR; o <<= 1) key = min(key, __shfl_xor(key, o, 64));
            const float z = (key & 1) ? -0.0f : 0.0f;
            if (mn0) mn = z;
            if (mx0) mx = z;
        }   // (else every zero of the row has the sign the reduction shows)
    }
    if (has_row && rowflag[has_row ? row_b : 0] != 0) {
        mn = __int_as_float(0x7fc00000);
        mx = mn;
    }
    {
        float s = (mx - mn) / (float)((1 << BITS) - 1);
        if (s == 0.0f) s = 1.0f;
        const bool exact_row = !(s >= 0x1p-100f && s <= 0x1p100f);
        if (row_valid && li == 0) {   // (empty row slots keep their neutral entry)
            rowtab[row_b] = make_float4(mn, s, __builtin_amdgcn_rcpf(s), exact_row ? 1.0f : 0.0f);
            store_params(pb, rowid[row_b], mn, s);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ---- C: codes (the guard-band reciprocal of quant_pack_rows16_kernel) -------------------------------------
    constexpr float kGuard = BITS == 8 ? 0x1p-13f : BITS == 4 ? 0x1p-17f : 0x1p-19f;
    uint8_t *out_run = q + (int64_t)g0 * F;                         // the chunk's ng * F output bytes
    const int mis = RAGGED ? (int)(reinterpret_cast<uintptr_t>(out_run) & 3) : 0;
    bool lane_exact = false;
    uint32_t words[NV];
    // The largest distance of a quotient from its rounded value over all of the lane's elements decides once for the
    // lane.  A NaN quotient (a NaN element behind the first of its row) drops out of the maximum: its code is 0 from
    // the conversion here as from the saturating conversion of quant_code.
    float far = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const float4 ta = rowtab[prv[v]];
        if (ta.w != 0.0f) lane_exact = true;
        uint32_t word = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float qf = (xv[v][t] - ta.x) * ta.z;
            const float ri = rintf(qf);
            far = fmaxf(far, fabsf(qf - ri));
            word = __builtin_amdgcn_cvt_pk_u8_f32(ri, t, word);
        }
        words[v] = word;
    }
    if (!(far < 0.5f - kGuard)) lane_exact = true;
    if (lane_exact) {   // this lane redoes its elements with the IEEE division
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const float4 ta = rowtab[prv[v]];
            uint32_t word = 0;
#pragma unroll
            for (int t = 0; t < 4; ++t) word |= quant_code(xv[v][t], ta.x, ta.y) << (8 * t);
            words[v] = word;
        }
    }
#pragma unroll
    for (int v = 0; v < NV; ++v)   // slots behind the chunk's last vector hold copies of it: their codes are zero
        if ((v >= n_full && v * 64 + lane > last) || ((dead_mask >> v) & 1u)) words[v] = 0;
    if constexpr (EPB == 1 && RAGGED) {
        // int8, rows that are not whole words or an output that is not word-aligned: code byte j of row slot p is
        // output byte p * F + j, so every lane stores its words where they belong, at whatever alignment.  A row's
        // short last word is filled up with the first bytes of the next row's first word (the next vector slot:
        // the next lane, or lane 0's next vector), which that slot writes too -- the same bytes, so the order of
        // the two stores does not matter; the chunk's last row has no next one and goes out byte by byte.
        const int nt = F & 3;
        const int n_sl = ng * VPR;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int sl = v * 64 + lane;
            const int pr = prv[v];
            const int cv = (sl < n_sl ? sl : n_sl - 1) - pr * VPR;
            uint32_t w = words[v];
            const bool sh = nt != 0 && cv == VPR - 1;
            if (nt != 0) {
                uint32_t nxt = (uint32_t)__shfl_down((int)words[v], 1, 64);
                if (v + 1 < NV) {
                    const uint32_t first_of_next = (uint32_t)__builtin_amdgcn_readfirstlane((int)words[v + 1]);
                    if (lane == 63) nxt = first_of_next;
                }
                if (sh) w = (w & ((1u << (8 * nt)) - 1u)) | (nxt << (8 * nt));
            }
            if (sl < n_sl) {
                uint8_t *dst = out_run + pr * F + 4 * cv;
                if (sh && pr == ng - 1) {
                    for (int t = 0; t < nt; ++t) dst[t] = (uint8_t)(w >> (8 * t));
                } else {
                    u32_store_nt_unaligned(dst, w);
                }
            }
        }
        return;
    }
    if (EPB == 1 && !RAGGED) {   // code words are output words
        uint32_t *q32 = reinterpret_cast<uint32_t *>(out_run);
#pragma unroll
        for (int v = 0; v < NV; ++v)
            if (v * 64 + lane < npr * VPR) __builtin_nontemporal_store(words[v], q32 + v * 64 + lane);
        return;
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) reinterpret_cast<uint32_t *>(codes)[v * 64 + lane] = words[v];
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ---- D: pack and store ------------------------------------------------------------------------------------
    // code word w of row slot p: codes32[p * VPR + w]
    const int nbytes = ng * F;
    const int nw = (mis + nbytes + 3) >> 2;
    const uint32_t *codes32 = reinterpret_cast<const uint32_t *>(codes);
    uint32_t *q32 = reinterpret_cast<uint32_t *>(out_run - mis);
    const int n_pw = ng * VPR;   // words of the packed rows, a row's last one short when F % 4 != 0
    if constexpr (!RAGGED) {
        // F % 4 == 0: packed word s of the chunk is output word s
        for (int s = lane; s < n_pw; s += 64) {
            const int g = (int)(__umul24((uint32_t)s, vpr_magic) >> 21);
            const uint32_t *cw = codes32 + s * EPB - (s - g * VPR) * (EPB - 1);   // (g * EPB) * VPR + word in the row
            uint32_t word = 0;
#pragma unroll
            for (int k = 0; k < EPB; ++k) word |= cw[k * VPR] << ((EPB - 1 - k) * BITS);
            __builtin_nontemporal_store(word, q32 + s);
        }
    } else if constexpr (EPB < 4) {
        // The lanes walk the output run in aligned words; a word's bytes are gathered from the code words of its
        // packed row -- or, where it straddles two, of both -- at their byte offsets.  (For int8 and int4 this is
        // cheaper than the extra pass through LDS below: F = 123 int8 5.5 against 4.7 TB/s.)
        const int pitch = 4 * VPR;
        // (packed row, column) of the LAST byte of a lane's word (never negative): advanced by 256 bytes per round
        const int dgr = 256 / F, djc = 256 % F;
        int b0 = 4 * lane - mis;
        int gr = (b0 + 3) / F, jc = b0 + 3 - gr * F;
        for (int w = lane; w < nw; w += 64) {
            if (b0 >= 0 && b0 + 3 < nbytes) {
                // jc >= 3: four bytes of packed row gr; else the first 3 - jc bytes are the end of packed row gr - 1
                const int nA = jc >= 3 ? 0 : 3 - jc;
                const uint32_t keep = 0xffffffffu << (8 * nA);
                uint32_t word = 0;
#pragma unroll
                for (int k = 0; k < EPB; ++k) {
                    const uint32_t c = lds_load_u32_unaligned(codes + (gr * EPB + k) * pitch + jc - 3);
                    word |= (c & keep) << ((EPB - 1 - k) * BITS);
                }
                if (nA != 0) {
#pragma unroll
                    for (int k = 0; k < EPB; ++k) {
                        const uint32_t c = lds_load_u32_unaligned(codes + ((gr - 1) * EPB + k) * pitch + F + jc - 3);
                        word |= (c & ~keep) << ((EPB - 1 - k) * BITS);
                    }
                }
                __builtin_nontemporal_store(word, q32 + w);
            } else {   // the first or the last word of the run, partly outside it
                for (int t = 0; t < 4; ++t) {
                    const int b = b0 + t;
                    if (b < 0 || b >= nbytes) continue;
                    const int c = jc - 3 + t;
                    const int g = c < 0 ? gr - 1 : gr, j = c < 0 ? c + F : c;
                    uint32_t byte = 0;
#pragma unroll
                    for (int k = 0; k < EPB; ++k) byte |= (uint32_t)codes[(g * EPB + k) * pitch + j] << ((EPB - 1 - k) * BITS);
                    out_run[b] = (uint8_t)byte;
                }
            }
            b0 += 256;
            gr += dgr;
            jc += djc;
            if (jc >= F) { jc -= F; ++gr; }
        }
    } else {
        // int2: the packed rows are first laid out byte after byte in LDS (behind the code words): a row's last word is
        // written before the other words of the round, so that the bytes it spills into the next row are overwritten
        // by that row's first word (same round, or a later one).  The run then goes out in aligned words.
        uint8_t *packed = base + NV * 256;
        for (int s0 = 0; s0 < n_pw; s0 += 64) {
            const int s = s0 + lane < n_pw ? s0 + lane : n_pw - 1;
            const int g = (int)(__umul24((uint32_t)s, vpr_magic) >> 21), wv = s - g * VPR;
            const uint32_t *cw = codes32 + s * EPB - wv * (EPB - 1);
            uint32_t word = 0;
#pragma unroll
            for (int k = 0; k < EPB; ++k) word |= cw[k * VPR] << ((EPB - 1 - k) * BITS);
            uint8_t *dst = packed + g * F + 4 * wv;
            const bool live = s0 + lane < n_pw, tail = wv == VPR - 1;
            if (live && tail) lds_store_u32_unaligned(dst, word);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // (keeps the two stores apart and in this order)
            if (live && !tail) lds_store_u32_unaligned(dst, word);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (int w = lane; w < nw; w += 64) {
            const int b0 = 4 * w - mis;
            if (b0 >= 0 && b0 + 3 < nbytes) {
                __builtin_nontemporal_store(lds_load_u32_unaligned(packed + b0), q32 + w);
            } else {   // the first or the last word of the run, partly outside it
                for (int t = 0; t < 4; ++t)
                    if (b0 + t >= 0 && b0 + t < nbytes) out_run[b0 + t] = packed[b0 + t];
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Unpack + dequantize, row-group layout.  Same work decomposition as the quantize kernel.
// ------------------------------------------------------------------------------------------------
template <int BITS, int VEC, int G, int NV>
__global__ __launch_bounds__(kQBlock) void unpack_dequant_rows_kernel(
    const uint8_t *__restrict__ q, float *__restrict__ x, const ParamBuf pb,
    const int32_t *__restrict__ seg, const int32_t *__restrict__ pseg, int P, int64_t single_rows, int n_packed, int F,
    int n_units) {
    constexpr int EPB = 8 / BITS;
    constexpr int R = kRowsPerGroup;
    constexpr int NPR = R / EPB;
    constexpr int GPB = kQBlock / G;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int gid = threadIdx.x / G, lig = threadIdx.x % G;
    const int unit = blockIdx.x * GPB + gid;
    if (unit >= n_units) return;

#pragma unroll
    for (int pi = 0; pi < NPR; ++pi) {
        const int gp = unit * NPR + pi;
        if (gp >= n_packed) continue;
        int64_t row0, rend;
        locate_packed_row(seg, pseg, P, single_rows, gp, __builtin_amdgcn_readfirstlane(gp), EPB, row0, rend);
        const uint8_t *qr = q + (int64_t)gp * F;
        float zp[EPB], sc[EPB];
#pragma unroll
        for (int k = 0; k < EPB; ++k) {
            zp[k] = 0.0f;
            sc[k] = 0.0f;
            if (row0 + k < rend) {
                const float2 ps = load_params(pb, row0 + k);
                zp[k] = ps.x;
                sc[k] = ps.y;
            }
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int off = (v * G + lig) * VEC;
            if (off >= F) continue;
            uint32_t word;
            if constexpr (VEC == 4) word = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(qr + off));
            else if constexpr (VEC == 2) word = __builtin_nontemporal_load(reinterpret_cast<const uint16_t *>(qr + off));
            else word = qr[off];
#pragma unroll
            for (int k = 0; k < EPB; ++k) {
                if (row0 + k >= rend) continue;
                float o[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const uint32_t c = (word >> (8 * e + (EPB - 1 - k) * BITS)) & MASK;
                    o[e] = fmaf((float)c, sc[k], zp[k]);
                }
                vec_store_nt<VEC>(x + (row0 + k) * F + off, o);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Unpack + dequantize over the flat output (F % 4 == 0, any F): the fp32 output is one contiguous
// array of n*F/4 float4, and every wavefront store covers 64 consecutive float4 = 1 KB of it,
// whatever the row width (a 512-byte row: two rows per store; a 4-KB row: a quarter row).  A lane
// derives (row, column) from its flat index, fetches the packed word that holds its four codes and
// the row's params, and writes.  Rows that share a packed word re-read it from the cache.  Waves are
// short (R stores each) and carry no loop: measured on MI355X this shape streams writes faster than
// longer-lived or persistent waves.
// ------------------------------------------------------------------------------------------------
template <int BITS, int R, bool POW2, bool SEGMENTED>
__global__ __launch_bounds__(kQBlock) void unpack_dequant_flat_kernel(
    const uint8_t *__restrict__ q, float *__restrict__ x, const ParamBuf pb, const int32_t *__restrict__ seg,
    const int32_t *__restrict__ pseg, int P, int G /* float4 per row */, int g_shift, int64_t n_vec) {
    constexpr int EPB = 8 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    const int64_t base = wave * (R * 64) + lane;
    uint32_t word[R];
    float2 ps[R];
    int shift[R];
    // The segment that holds the wave's first row, searched once per wave on wave-uniform values
    // (scalar loads); lanes further on fall back to their own search.
    int w_p = 0, w_s0 = 0, w_s1 = 0, w_ps0 = 0;
    if constexpr (SEGMENTED) {
        const int64_t i0 = ((int64_t)blockIdx.x * (kQBlock / 64) + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6))) * (R * 64);
        const int row_w = (int)(POW2 ? (i0 >> g_shift) : (i0 / G));
        const WaveSegment ws = wave_find_segment(seg, pseg, P, row_w);  // the wave's first vector exists, so row_w < seg[P]
        w_p = ws.p;
        w_s0 = ws.k0;
        w_s1 = ws.k1;
        w_ps0 = ws.o0;
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t i = base + u * 64;
        word[u] = 0;
        ps[u] = make_float2(0.0f, 0.0f);
        shift[u] = 0;
        if (i >= n_vec) continue;
        int row, c;
        if constexpr (POW2) {
            row = (int)(i >> g_shift);
            c = (int)(i & (G - 1));
        } else {
            row = (int)(i / G);
            c = (int)(i - (int64_t)row * G);
        }
        int slot = row;
        if constexpr (SEGMENTED) {  // sub-byte codes and more than one segment: segments start on packed-row boundaries
            if (row < w_s1) {
                slot = w_ps0 * EPB + (row - w_s0);
            } else {             // this lane's row lies beyond the segment the wave starts in
                int lo = w_p, hi = P - 1;
                while (lo < hi) {
                    const int mid = (lo + hi) >> 1;
                    if (seg[mid + 1] > row) hi = mid; else lo = mid + 1;
                }
                slot = pseg[lo] * EPB + (row - seg[lo]);
            }
        }
        ps[u] = load_params(pb, row);
        shift[u] = (EPB - 1 - (slot % EPB)) * BITS;
        word[u] = reinterpret_cast<const uint32_t *>(q)[(int64_t)(slot / EPB) * G + c];  // cacheable on purpose
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t i = base + u * 64;
        if (i >= n_vec) continue;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = fmaf((float)((word[u] >> (8 * e + shift[u])) & MASK), ps[u].y, ps[u].x);
        vec_store_nt<4>(x + i * 4, o);
    }
}

// ------------------------------------------------------------------------------------------------
// The same flat decomposition for widths that are not a multiple of four (F = 602, F = 123 ...): the
// output is still written as 16-byte vectors over the flat array, but a vector may now straddle a row
// boundary, so it is made of 4 / VEC pieces of VEC floats (VEC = 2 for even F, 1 for odd F), each with
// its own (row, column), its own VEC code bytes and its own params.  The last vector of the array may be
// partial and is written element by element.  x must be 16-byte aligned (the row-tiled kernels take
// other cases).
// ------------------------------------------------------------------------------------------------
template <int BITS, int VEC, int R, bool SEGMENTED>
__global__ __launch_bounds__(kQBlock) void unpack_dequant_flat_ragged_kernel(
    const uint8_t *__restrict__ q, float *__restrict__ x, const ParamBuf pb, const int32_t *__restrict__ seg,
    const int32_t *__restrict__ pseg, int P, int F, int64_t n_elem) {
    constexpr int EPB = 8 / BITS;
    constexpr int NP = 4 / VEC;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    const int64_t base = wave * (R * 64) + lane;
    const int64_t n_vec = (n_elem + 3) >> 2;
    uint32_t word[R][NP];
    float2 ps[R][NP];
    int shift[R][NP];
    int w_p = 0, w_s0 = 0, w_s1 = 0, w_ps0 = 0;
    if constexpr (SEGMENTED) {  // the segment of the wave's first row, found on wave-uniform values
        const int64_t i0 = ((int64_t)blockIdx.x * (kQBlock / 64) + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6))) * (R * 64);
        const int row_w = (int)((i0 * 4) / F);
        const WaveSegment ws = wave_find_segment(seg, pseg, P, row_w);  // the wave's first vector exists, so row_w < seg[P]
        w_p = ws.p;
        w_s0 = ws.k0;
        w_s1 = ws.k1;
        w_ps0 = ws.o0;
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t i = base + u * 64;
        int row = 0, c = 0;
        if (i < n_vec) {
            const int64_t e0 = i * 4;
            row = (int)(e0 / F);
            c = (int)(e0 - (int64_t)row * F);
        }
        // When no vector of the wavefront straddles a row boundary -- most wavefronts of a wide row -- a lane's two
        // pieces share row, slot and params, and one 4-byte load at the bytes' natural address fetches both.
        const bool whole = c + 4 <= F;
        if (VEC == 2 && __ballot(i < n_vec && !whole) == 0ull) {
            word[u][0] = word[u][NP - 1] = 0;
            ps[u][0] = ps[u][NP - 1] = make_float2(0.0f, 0.0f);
            shift[u][0] = shift[u][NP - 1] = 0;
            if (i < n_vec) {
                int slot = row;
                if constexpr (SEGMENTED) {
                    if (row < w_s1) {
                        slot = w_ps0 * EPB + (row - w_s0);
                    } else {
                        int lo = w_p, hi = P - 1;
                        while (lo < hi) {
                            const int mid = (lo + hi) >> 1;
                            if (seg[mid + 1] > row) hi = mid; else lo = mid + 1;
                        }
                        slot = pseg[lo] * EPB + (row - seg[lo]);
                    }
                }
                typedef uint32_t u32u __attribute__((aligned(2)));
                const uint32_t w = *reinterpret_cast<const u32u *>(q + (int64_t)(slot / EPB) * F + c);
                word[u][0] = w & 0xffffu;
                word[u][NP - 1] = w >> 16;
                ps[u][0] = ps[u][NP - 1] = load_params(pb, row);
                shift[u][0] = shift[u][NP - 1] = (EPB - 1 - (slot % EPB)) * BITS;
            }
            continue;
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            word[u][p] = 0;
            ps[u][p] = make_float2(0.0f, 0.0f);
            shift[u][p] = 0;
            if (i < n_vec && i * 4 + p * VEC < n_elem) {
                int slot = row;
                if constexpr (SEGMENTED) {
                    if (row < w_s1) {
                        slot = w_ps0 * EPB + (row - w_s0);
                    } else {
                        int lo = w_p, hi = P - 1;
                        while (lo < hi) {
                            const int mid = (lo + hi) >> 1;
                            if (seg[mid + 1] > row) hi = mid; else lo = mid + 1;
                        }
                        slot = pseg[lo] * EPB + (row - seg[lo]);
                    }
                }
                ps[u][p] = load_params(pb, row);
                shift[u][p] = (EPB - 1 - (slot % EPB)) * BITS;
                const uint8_t *src = q + (int64_t)(slot / EPB) * F + c;  // cacheable: rows that share a byte hit in cache
                if constexpr (VEC == 2) word[u][p] = *reinterpret_cast<const uint16_t *>(src);
                else word[u][p] = *src;
            }
            c += VEC;
            if (c >= F) { c = 0; ++row; }  // F % VEC == 0: a piece never straddles a row boundary
        }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t i = base + u * 64;
        if (i >= n_vec) continue;
        float o[4];
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                o[p * VEC + e] = fmaf((float)((word[u][p] >> (8 * e + shift[u][p])) & MASK), ps[u][p].y, ps[u][p].x);
        if (i * 4 + 4 <= n_elem) {
            vec_store_nt<4>(x + i * 4, o);
        } else {
            for (int e = 0; e < 4; ++e)
                if (i * 4 + e < n_elem) x[i * 4 + e] = o[e];
        }
    }
}

// Odd F >= 4: the four floats of a 16-byte vector lie in at most two rows, A (the first n_a of them) and the
// row after it, so a lane looks up two rows (slot, params) instead of four and fetches its four code bytes from
// the one or two places they sit in.
template <int BITS, int R, bool SEGMENTED>
__global__ __launch_bounds__(kQBlock) void unpack_dequant_flat_odd_kernel(
    const uint8_t *__restrict__ q, float *__restrict__ x, const ParamBuf pb, const int32_t *__restrict__ seg,
    const int32_t *__restrict__ pseg, int P, int F, int n_rows, int64_t n_elem, int n_packed) {
    constexpr int EPB = 8 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    const int64_t base = wave * (R * 64) + lane;
    const int64_t n_vec = (n_elem + 3) >> 2;
    WaveSegment ws{0, 0, 0, 0, 0};
    if constexpr (SEGMENTED) {  // the segment of the wave's first row
        const int64_t i0 = ((int64_t)blockIdx.x * (kQBlock / 64) + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6))) * (R * 64);
        const int row_w = (int)((i0 * 4) / F);
        ws = wave_find_segment(seg, pseg, P, row_w < n_rows ? row_w : n_rows - 1);
    }
    auto slot_of = [&](int row) {
        if constexpr (!SEGMENTED) return row;
        if (row < ws.k1) return ws.o0 * EPB + (row - ws.k0);
        int lo = ws.p, hi = P - 1;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (seg[mid + 1] > row) hi = mid; else lo = mid + 1;
        }
        return pseg[lo] * EPB + (row - seg[lo]);
    };
    // (row, column) of each vector's first element: one division for the lane's first vector, then 256 elements per round
    const int dr = 256 / F, dc = 256 % F;
    int row_a = (int)((base * 4) / F);
    int c_a = (int)(base * 4 - (int64_t)row_a * F);
    const int64_t q_bytes = (int64_t)n_packed * F;   // (at least 4: F >= 4 on this path)
    typedef uint32_t u32u __attribute__((aligned(1)));
    uint32_t wa[R], wb[R];
    int sh_a[R], sh_b[R];
    float2 psa[R], psb[R];
    int na[R];
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t i = base + u * 64;
        na[u] = 4;
        psa[u] = psb[u] = make_float2(0.0f, 0.0f);
        wa[u] = wb[u] = 0;
        sh_a[u] = sh_b[u] = 0;
        if (i < n_vec) {
            na[u] = F - c_a < 4 ? F - c_a : 4;
            const int slot_a = slot_of(row_a);
            psa[u] = load_params(pb, row_a);
            sh_a[u] = (EPB - 1 - (slot_a % EPB)) * BITS;
            // The vector's four code bytes with one 4-byte load at their natural address (bytes past the end of row A, if
            // any, are not used).  A load that would reach past the end of the buffer starts d bytes earlier and is
            // shifted back; no branch around a load, so all of a lane's loads are in flight together.
            const int64_t off_a = (int64_t)(slot_a / EPB) * F + c_a;
            const int64_t off_ac = off_a < q_bytes - 4 ? off_a : q_bytes - 4;
            wa[u] = *reinterpret_cast<const u32u *>(q + off_ac) >> (8 * (int)(off_a - off_ac));
            if (na[u] < 4 && row_a + 1 < n_rows) {   // the vector's tail lies in the next row: its columns 0 ... 3 - n_a
                const int slot_b = slot_of(row_a + 1);
                psb[u] = load_params(pb, row_a + 1);
                sh_b[u] = (EPB - 1 - (slot_b % EPB)) * BITS;
                // piece k of row B is its column k - n_a: a load that would start before the buffer starts at its
                // first byte and is shifted forth
                const int64_t off_b = (int64_t)(slot_b / EPB) * F - na[u];
                const int64_t off_bc = off_b > 0 ? off_b : 0;
                wb[u] = *reinterpret_cast<const u32u *>(q + off_bc) << (8 * (int)(off_bc - off_b));
            }
        }
        row_a += dr;
        c_a += dc;
        if (c_a >= F) { c_a -= F; ++row_a; }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t i = base + u * 64;
        if (i >= n_vec) continue;
        float o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const bool in_a = k < na[u];
            const uint32_t c = ((in_a ? wa[u] : wb[u]) >> (8 * k + (in_a ? sh_a[u] : sh_b[u]))) & MASK;
            const float2 ps = in_a ? psa[u] : psb[u];
            o[k] = fmaf((float)c, ps.y, ps.x);
        }
        if (i * 4 + 4 <= n_elem) {
            vec_store_nt<4>(x + i * 4, o);
        } else {
            for (int k = 0; k < 4; ++k)
                if (i * 4 + k < n_elem) x[i * 4 + k] = o[k];
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Any-F fallbacks (F wider than a register tile): one wavefront per packed row, two passes.
// ------------------------------------------------------------------------------------------------
template <int BITS>
__global__ __launch_bounds__(kQBlock) void quant_pack_rows_wide_kernel(
    const RowSrc xs, uint8_t *__restrict__ q, const ParamBuf pb,
    const int32_t *__restrict__ seg, const int32_t *__restrict__ pseg, int P, int64_t single_rows, int n_packed, int F) {
    constexpr int EPB = 8 / BITS;
    const int lane = threadIdx.x & 63;
    const int gp = blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    if (gp >= n_packed) return;
    int64_t row0, rend;
    locate_packed_row(seg, pseg, P, single_rows, gp, __builtin_amdgcn_readfirstlane(gp), EPB, row0, rend);
    // Both passes walk a row in 16-byte vectors at their natural (4-byte aligned) addresses, several loads in flight
    // per lane (slots past the last whole vector repeat it: a repeat changes neither min nor max nor the first zero);
    // the F % 4 elements behind the last whole vector are taken one by one.  The second pass finds the rows in cache.
    const int nvf = F >> 2;                     // whole vectors of a row (at least 128: narrower rows never come here)
    const int n_tail = F & 3;
    constexpr int U1 = 8, U2 = BITS == 2 ? 2 : BITS == 4 ? 4 : 8;   // vectors in flight per lane: first / second pass (x EPB rows)
    constexpr float kGuard = BITS == 8 ? 0x1p-13f : BITS == 4 ? 0x1p-17f : 0x1p-19f;
    float zp[EPB], sc[EPB], rinv[EPB];
    const float *xr[EPB];
#pragma unroll
    for (int k = 0; k < EPB; ++k) {
        zp[k] = 0.0f;
        sc[k] = 1.0f;
        rinv[k] = 1.0f;
        xr[k] = nullptr;
        if (row0 + k >= rend) continue;
        xr[k] = row_ptr(xs, row0 + k);
        float mn = INFINITY, mx = -INFINITY;
        int key = INT_MAX;
        for (int j0 = lane; j0 < nvf; j0 += 64 * U1) {
            float v[U1][4];
#pragma unroll
            for (int u = 0; u < U1; ++u) {
                const int j = j0 + 64 * u < nvf ? j0 + 64 * u : nvf - 1;
                vec4_load_nt_unaligned(v[u], xr[k] + 4 * j);
            }
#pragma unroll
            for (int u = 0; u < U1; ++u) {
                const int j = j0 + 64 * u < nvf ? j0 + 64 * u : nvf - 1;
#pragma unroll
                for (int t = 3; t >= 0; --t) {
                    mn = fminf(mn, v[u][t]);
                    mx = fmaxf(mx, v[u][t]);
                }
                if (key == INT_MAX) {
#pragma unroll
                    for (int t = 3; t >= 0; --t)
                        if (v[u][t] == 0.0f) key = ((4 * j + t) << 1) | (int)(__float_as_uint(v[u][t]) >> 31);
                }
            }
        }
        if (lane < n_tail) {
            const float e = xr[k][4 * nvf + lane];
            mn = fminf(mn, e);
            mx = fmaxf(mx, e);
            if (e == 0.0f) key = min(key, ((4 * nvf + lane) << 1) | (int)(__float_as_uint(e) >> 31));
        }
        mn = group_allreduce_f<64, OpMinF>(mn);
        mx = group_allreduce_f<64, OpMaxF>(mx);
        key = group_allmin_i<64>(key);
        const float z = (key & 1) ? -0.0f : 0.0f;
        if (mn == 0.0f) mn = z;
        if (mx == 0.0f) mx = z;
        const float first = xr[k][0];
        if (first != first) { mn = first; mx = first; }
        float s = (mx - mn) / (float)((1 << BITS) - 1);
        if (s == 0.0f) s = 1.0f;
        zp[k] = mn;
        sc[k] = s;
        rinv[k] = __builtin_amdgcn_rcpf(s);
        if (lane == 0) store_params(pb, row0 + k, mn, s);
    }
    uint8_t *qr = q + (int64_t)gp * F;
    // product with the hardware reciprocal first, IEEE division only when an element lies inside the guard band
    // around a rounding tie (same argument and bands as in quant_pack_rows16_kernel)
    auto codes4 = [&](const float (&v)[4], int k) {
        uint32_t w = 0;
        bool redo = !(sc[k] >= 0x1p-100f && sc[k] <= 0x1p100f);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float qf = (v[t] - zp[k]) * rinv[k];
            const float ri = rintf(qf);
            if (!(fabsf(qf - ri) < 0.5f - kGuard)) redo = true;
            w = __builtin_amdgcn_cvt_pk_u8_f32(ri, t, w);
        }
        if (redo) {
            w = 0;
#pragma unroll
            for (int t = 0; t < 4; ++t) w |= quant_code(v[t], zp[k], sc[k]) << (8 * t);
        }
        return w;
    };
    for (int j0 = lane; j0 < nvf; j0 += 64 * U2) {
        float v[U2][EPB][4];
#pragma unroll
        for (int u = 0; u < U2; ++u) {
            const int j = j0 + 64 * u < nvf ? j0 + 64 * u : nvf - 1;
#pragma unroll
            for (int k = 0; k < EPB; ++k) {
                if (row0 + k < rend) vec4_load_nt_unaligned(v[u][k], xr[k] + 4 * j);
            }
        }
#pragma unroll
        for (int u = 0; u < U2; ++u) {
            const int j = j0 + 64 * u;
            if (j >= nvf) continue;
            uint32_t word = 0;
#pragma unroll
            for (int k = 0; k < EPB; ++k) {
                if (row0 + k < rend) word |= codes4(v[u][k], k) << ((EPB - 1 - k) * BITS);
            }
            u32_store_nt_unaligned(qr + 4 * j, word);
        }
    }
    if (lane < n_tail) {
        const int c = 4 * nvf + lane;
        uint32_t byte = 0;
#pragma unroll
        for (int k = 0; k < EPB; ++k) {
            if (row0 + k < rend) byte |= quant_code(xr[k][c], zp[k], sc[k]) << ((EPB - 1 - k) * BITS);
        }
        qr[c] = (uint8_t)byte;
    }
}

// ------------------------------------------------------------------------------------------------
// Rows too wide for a wavefront's registers: one workgroup per packed row, the row kept in the registers of its TB
// threads.  Thread t holds vectors t, t + TB, ... (NVT of them) of each of the EPB rows, so the fp32 rows are read
// once, the per-row min / max is a reduction over the workgroup (DPP inside a wavefront, a few words of LDS across
// wavefronts), and a thread packs its own output words: the EPB code words it needs sit in its own registers.
// F <= 4 * TB * NVT, i.e. up to 8192 floats.  (The two-pass kernel above reads the rows twice, and at these widths the
// second read no longer finds them in a cache: F = 3703 int2 2.7 TB/s.)
// ------------------------------------------------------------------------------------------------
template <int BITS, int TB, int NVT>
__global__ __launch_bounds__(TB) void quant_pack_rows_block_kernel(
    const RowSrc xs, uint8_t *__restrict__ q, const ParamBuf pb,
    const int32_t *__restrict__ seg, const int32_t *__restrict__ pseg, int P, int64_t single_rows, int n_packed, int F) {
    constexpr int EPB = 8 / BITS;
    constexpr int NW = TB / 64;
    __shared__ float red_mn[NW][EPB], red_mx[NW][EPB];
    __shared__ int red_key[NW][EPB];
    __shared__ float4 rowpar[EPB];   // (zero_point, scale, 1 / scale, needs the exact division)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gp = blockIdx.x;
    int64_t row0, rend;
    locate_packed_row(seg, pseg, P, single_rows, gp, gp, EPB, row0, rend);
    const int nvf = F >> 2, n_tail = F & 3;   // whole vectors of a row (1 <= nvf <= TB * NVT), elements behind them
    // (a row slot the segment's short last group leaves empty reads the group's first row again, so that no load
    //  sits behind a condition; nothing of it is used.  Vector slots behind the row repeat its last whole vector:
    //  a repeat changes neither min nor max nor the first zero, and is not stored.)
    const float *xr[EPB];
    float v[NVT][EPB][4], e_tail[EPB];
#pragma unroll
    for (int k = 0; k < EPB; ++k) xr[k] = row_ptr(xs, row0 + k < rend ? row0 + k : row0);
#pragma unroll
    for (int u = 0; u < NVT; ++u) {
        const int j = u * TB + tid < nvf ? u * TB + tid : nvf - 1;
#pragma unroll
        for (int k = 0; k < EPB; ++k) vec4_load_nt_unaligned(v[u][k], xr[k] + 4 * j);
    }
#pragma unroll
    for (int k = 0; k < EPB; ++k) e_tail[k] = tid < n_tail ? xr[k][4 * nvf + tid] : 0.0f;
#pragma unroll
    for (int k = 0; k < EPB; ++k) {
        float mn = INFINITY, mx = -INFINITY;
        int key = INT_MAX;
#pragma unroll
        for (int u = 0; u < NVT; ++u) {
            const int j = u * TB + tid < nvf ? u * TB + tid : nvf - 1;
#pragma unroll
            for (int t = 3; t >= 0; --t) {
                mn = fminf(mn, v[u][k][t]);
                mx = fmaxf(mx, v[u][k][t]);
            }
            if (key == INT_MAX) {
#pragma unroll
                for (int t = 3; t >= 0; --t)
                    if (v[u][k][t] == 0.0f) key = ((4 * j + t) << 1) | (int)(__float_as_uint(v[u][k][t]) >> 31);
            }
        }
        if (tid < n_tail) {
            mn = fminf(mn, e_tail[k]);
            mx = fmaxf(mx, e_tail[k]);
            if (e_tail[k] == 0.0f) key = min(key, ((4 * nvf + tid) << 1) | (int)(__float_as_uint(e_tail[k]) >> 31));
        }
        mn = group_allreduce_f<64, OpMinF>(mn);
        mx = group_allreduce_f<64, OpMaxF>(mx);
        key = group_allmin_i<64>(key);
        if (lane == 0) {
            red_mn[wave][k] = mn;
            red_mx[wave][k] = mx;
            red_key[wave][k] = key;
        }
    }
    __syncthreads();
    if (tid < EPB && row0 + tid < rend) {
        const int k = tid;
        float mn = red_mn[0][k], mx = red_mx[0][k];
        int key = red_key[0][k];
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            mn = fminf(mn, red_mn[w][k]);
            mx = fmaxf(mx, red_mx[w][k]);
            key = min(key, red_key[w][k]);
        }
        const float z = (key & 1) ? -0.0f : 0.0f;
        if (mn == 0.0f) mn = z;
        if (mx == 0.0f) mx = z;
        const float first = row_ptr(xs, row0 + k)[0];
        if (first != first) { mn = first; mx = first; }
        float s = (mx - mn) / (float)((1 << BITS) - 1);
        if (s == 0.0f) s = 1.0f;
        rowpar[k] = make_float4(mn, s, __builtin_amdgcn_rcpf(s), (s >= 0x1p-100f && s <= 0x1p100f) ? 0.0f : 1.0f);
        store_params(pb, row0 + k, mn, s);
    }
    __syncthreads();
    constexpr float kGuard = BITS == 8 ? 0x1p-13f : BITS == 4 ? 0x1p-17f : 0x1p-19f;
    float4 par[EPB];
#pragma unroll
    for (int k = 0; k < EPB; ++k) par[k] = rowpar[k];
    uint8_t *qr = q + (int64_t)gp * F;
#pragma unroll
    for (int u = 0; u < NVT; ++u) {
        const int j = u * TB + tid;
        uint32_t word = 0;
#pragma unroll
        for (int k = 0; k < EPB; ++k) {
            if (row0 + k >= rend) continue;
            uint32_t w = 0;
            bool redo = par[k].w != 0.0f;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float qf = (v[u][k][t] - par[k].x) * par[k].z;
                const float ri = rintf(qf);
                if (!(fabsf(qf - ri) < 0.5f - kGuard)) redo = true;
                w = __builtin_amdgcn_cvt_pk_u8_f32(ri, t, w);
            }
            if (redo) {
                w = 0;
#pragma unroll
                for (int t = 0; t < 4; ++t) w |= quant_code(v[u][k][t], par[k].x, par[k].y) << (8 * t);
            }
            word |= w << ((EPB - 1 - k) * BITS);
        }
        if (j < nvf) u32_store_nt_unaligned(qr + 4 * j, word);
    }
    if (tid < n_tail) {
        uint32_t byte = 0;
#pragma unroll
        for (int k = 0; k < EPB; ++k) {
            if (row0 + k < rend) byte |= quant_code(e_tail[k], par[k].x, par[k].y) << ((EPB - 1 - k) * BITS);
        }
        qr[4 * nvf + tid] = (uint8_t)byte;
    }
}

template <int BITS>
__global__ __launch_bounds__(kQBlock) void unpack_dequant_rows_wide_kernel(
    const uint8_t *__restrict__ q, float *__restrict__ x, const ParamBuf pb,
    const int32_t *__restrict__ seg, const int32_t *__restrict__ pseg, int P, int64_t single_rows, int n_packed, int F) {
    constexpr int EPB = 8 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int lane = threadIdx.x & 63;
    const int gp = blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    if (gp >= n_packed) return;
    int64_t row0, rend;
    locate_packed_row(seg, pseg, P, single_rows, gp, __builtin_amdgcn_readfirstlane(gp), EPB, row0, rend);
    const uint8_t *qr = q + (int64_t)gp * F;
#pragma unroll
    for (int k = 0; k < EPB; ++k) {
        if (row0 + k >= rend) continue;
        const float2 ps = load_params(pb, row0 + k);
        const float zp = ps.x, sc = ps.y;
        for (int j = lane; j < F; j += 64)
            x[(row0 + k) * F + j] = fmaf((float)((qr[j] >> ((EPB - 1 - k) * BITS)) & MASK), sc, zp);
    }
}

// ------------------------------------------------------------------------------------------------
// Feature-packed mixed-bit layout ("v1"): one wavefront per row; bits differ row to row.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kQBlock) void quant_v1_kernel(const float *__restrict__ x, uint8_t *__restrict__ q,
                                                           const int64_t *__restrict__ range,
                                                           float *__restrict__ params, int64_t n, int F) {
    const int lane = threadIdx.x & 63;
    const int64_t i = (int64_t)blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    if (i >= n) return;
    const int b = (int)params[i * 3];
    if (b != 8 && b != 4 && b != 2) return;  // the reference prints an error and leaves the row (quantization_x86.cpp:244-245)
    const float *xr = x + i * F;
    float mn = INFINITY, mx = -INFINITY;
    int key = INT_MAX;
    for (int j = lane; j < F; j += 64) {
        const float v = xr[j];
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
        if (v == 0.0f && key == INT_MAX) key = (j << 1) | (int)(__float_as_uint(v) >> 31);
    }
    mn = group_allreduce_f<64, OpMinF>(mn);
    mx = group_allreduce_f<64, OpMaxF>(mx);
    key = group_allmin_i<64>(key);
    const float z = (key & 1) ? -0.0f : 0.0f;
    if (mn == 0.0f) mn = z;
    if (mx == 0.0f) mx = z;
    const float first = xr[0];
    if (first != first) { mn = first; mx = first; }
    float s = (mx - mn) / (float)((1 << b) - 1);
    if (s == 0.0f) s = 1.0f;
    if (lane == 0) { params[i * 3 + 1] = mn; params[i * 3 + 2] = s; }
    const int epb = 8 / b;
    const int nbytes = (F + epb - 1) / epb;
    uint8_t *qo = q + range[i];
    for (int t = lane; t < nbytes; t += 64) {
        uint32_t byte = 0;
        for (int k = 0; k < epb; ++k) {
            const int j = t * epb + k;
            if (j < F) byte |= quant_code(xr[j], mn, s) << ((epb - 1 - k) * b);
        }
        qo[t] = (uint8_t)byte;
    }
}

__global__ __launch_bounds__(kQBlock) void dequant_v1_kernel(const uint8_t *__restrict__ q, float *__restrict__ x,
                                                             const int64_t *__restrict__ range,
                                                             const float *__restrict__ params, int64_t n, int F) {
    const int lane = threadIdx.x & 63;
    const int64_t i = (int64_t)blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    if (i >= n) return;
    const int b = (int)params[i * 3];
    if (b != 8 && b != 4 && b != 2) return;
    const float zp = params[i * 3 + 1], sc = params[i * 3 + 2];
    const int epb = 8 / b;
    const uint32_t mask = (1u << b) - 1u;
    const uint8_t *qi = q + range[i];
    const int nbytes = (int)(range[i + 1] - range[i]);
    float *xo = x + i * F;
    for (int j = lane; j < F; j += 64) {
        const int t = j / epb, k = j % epb;
        if (t < nbytes) xo[j] = fmaf((float)((qi[t] >> ((epb - 1 - k) * b)) & mask), sc, zp);
    }
}

// The same two operations with float4 lanes (F % 4 == 0, F <= 256 * NV, 16-byte aligned fp32 rows): a
// wavefront takes R consecutive rows, each row read once into registers, 64-lane DPP reductions, and the
// four codes of a lane packed into one 32/16/8-bit store (int8/int4/int2).  A row's layout depends on
// two loaded values (its bit width and its byte offset range[i]); all R rows' values are requested
// before the first is used, so the wave pays that latency once per R KB instead of once per row.
// A row's bytes need not start 4- or 2-byte aligned; such a row falls back to byte stores / loads.
template <int NV, int R>
__global__ __launch_bounds__(kQBlock) void quant_v1_vec_kernel(const float *__restrict__ x, uint8_t *__restrict__ q,
                                                               const int64_t *__restrict__ range,
                                                               float *__restrict__ params, int64_t n, int F) {
    const int lane = threadIdx.x & 63;
    const int64_t i0 = ((int64_t)blockIdx.x * (kQBlock / 64) + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6))) * R;
    if (i0 >= n) return;
    float bits_f[R];
    int64_t r0[R];
    float xv[R][NV][4];
    int off[NV];
    bool act[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        off[v] = (v * 64 + lane) * 4;
        act[v] = off[v] < F;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t i = i0 + r < n ? i0 + r : n - 1;  // a short last wave repeats the last row's loads
        bits_f[r] = params[i * 3];
        r0[r] = range[i];
#pragma unroll
        for (int v = 0; v < NV; ++v) vec_load_nt<4>(xv[r][v], x + i * F + (act[v] ? off[v] : 0));  // unconditional
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t i = i0 + r;
        if (i >= n) break;
        const int b = (int)bits_f[r];
        if (b != 8 && b != 4 && b != 2) continue;  // the reference prints an error and leaves the row (quantization_x86.cpp:244-245)
        float mn = INFINITY, mx = -INFINITY;
        int key = INT_MAX;
#pragma unroll
        for (int v = NV - 1; v >= 0; --v) {
            if (!act[v]) continue;
#pragma unroll
            for (int k = 3; k >= 0; --k) {
                mn = fminf(mn, xv[r][v][k]);
                mx = fmaxf(mx, xv[r][v][k]);
                if (xv[r][v][k] == 0.0f) key = ((off[v] + k) << 1) | (int)(__float_as_uint(xv[r][v][k]) >> 31);
            }
        }
        mn = group_allreduce_f<64, OpMinF>(mn);
        mx = group_allreduce_f<64, OpMaxF>(mx);
        key = group_allmin_i<64>(key);
        const float z = (key & 1) ? -0.0f : 0.0f;
        if (mn == 0.0f) mn = z;
        if (mx == 0.0f) mx = z;
        const float first = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(xv[r][0][0])));
        if (first != first) { mn = first; mx = first; }
        float s = (mx - mn) / (float)((1 << b) - 1);
        if (s == 0.0f) s = 1.0f;
        if (lane == 0) { params[i * 3 + 1] = mn; params[i * 3 + 2] = s; }
        const float rinv = __builtin_amdgcn_rcpf(s);
        uint8_t *qo = q + r0[r];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
            // product with the hardware reciprocal first, IEEE division only for a lane that sees an
            // element within 2^-13 of a rounding tie (same argument as in quant_pack_rows16_kernel)
            uint32_t c[4];
            bool redo = !(s >= 0x1p-100f && s <= 0x1p100f);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float qf = (xv[r][v][k] - mn) * rinv;
                const float ri = rintf(qf);
                if (!(fabsf(qf - ri) < 0.5f - 0x1p-13f)) redo = true;
                c[k] = (uint32_t)ri;
            }
            if (redo) {
#pragma unroll
                for (int k = 0; k < 4; ++k) c[k] = quant_code(xv[r][v][k], mn, s);
            }
            if (b == 8) {
                uint8_t *dst = qo + off[v];
                if ((r0[r] & 3) == 0) {
                    __builtin_nontemporal_store(c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24), reinterpret_cast<uint32_t *>(dst));
                } else {
#pragma unroll
                    for (int k = 0; k < 4; ++k) dst[k] = (uint8_t)c[k];
                }
            } else if (b == 4) {
                uint8_t *dst = qo + off[v] / 2;
                const uint32_t b0 = (c[0] << 4) | c[1], b1 = (c[2] << 4) | c[3];
                if ((r0[r] & 1) == 0) {
                    __builtin_nontemporal_store((uint16_t)(b0 | (b1 << 8)), reinterpret_cast<uint16_t *>(dst));
                } else {
                    dst[0] = (uint8_t)b0;
                    dst[1] = (uint8_t)b1;
                }
            } else {
                qo[off[v] / 4] = (uint8_t)((c[0] << 6) | (c[1] << 4) | (c[2] << 2) | c[3]);
            }
        }
    }
}

// SGNN_V1_STAGED=0 at build time restores the direct stores of the v1 quantizer (for comparison).
#ifndef SGNN_V1_STAGED
#define SGNN_V1_STAGED 1
#endif
constexpr bool kV1Staged = SGNN_V1_STAGED;

// True when the byte ranges [r0, r1) of a wavefront's rows (row index = round * RW + lane group) follow one another
// without gaps: each row ends where the next begins.  Wave-uniform.
template <int R>
__device__ __forceinline__ bool contiguous_rows(const int64_t (&r0)[R], const int64_t (&r1)[R], int L) {
    const int lane = threadIdx.x & 63;
    bool ok = true;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // the next row sits L lanes further on, or in lane group 0 of the next round
        const int64_t nxt_same = __shfl_down(r0[r], L, 64);
        const int64_t nxt_round = __shfl(r0[r + 1 < R ? r + 1 : r], lane % L, 64);
        if (lane + L < 64) ok = ok && r1[r] == nxt_same;
        else if (r + 1 < R) ok = ok && r1[r] == nxt_round;
    }
    return __ballot(!ok) == 0ull;
}

// The four codes of one lane of a v1 row, packed and stored at the row's byte position for columns off .. off+3:
// 4 / 2 / 1 bytes at 8 / 4 / 2 bits, in one store when the address allows it.  NT: non-temporal (global memory).
template <bool NT>
__device__ __forceinline__ void store_v1_codes(uint8_t *row_bytes, int off, int b, const uint32_t (&c)[4]) {
    if (b == 8) {
        uint8_t *dst = row_bytes + off;
        const uint32_t w = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
        if ((reinterpret_cast<uintptr_t>(dst) & 3) == 0) {
            if constexpr (NT) __builtin_nontemporal_store(w, reinterpret_cast<uint32_t *>(dst));
            else *reinterpret_cast<uint32_t *>(dst) = w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) dst[k] = (uint8_t)c[k];
        }
    } else if (b == 4) {
        uint8_t *dst = row_bytes + off / 2;
        const uint32_t b0 = (c[0] << 4) | c[1], b1 = (c[2] << 4) | c[3];
        if ((reinterpret_cast<uintptr_t>(dst) & 1) == 0) {
            if constexpr (NT) __builtin_nontemporal_store((uint16_t)(b0 | (b1 << 8)), reinterpret_cast<uint16_t *>(dst));
            else *reinterpret_cast<uint16_t *>(dst) = (uint16_t)(b0 | (b1 << 8));
        } else {
            dst[0] = (uint8_t)b0;
            dst[1] = (uint8_t)b1;
        }
    } else {
        row_bytes[off / 4] = (uint8_t)((c[0] << 6) | (c[1] << 4) | (c[2] << 2) | c[3]);
    }
}

// The quantizer once more with L = 16 or 8 lanes per row instead of a whole wavefront (F <= 4 * L * NV): the
// min/max/zero-sign reductions stay inside a DPP row (four or three butterfly steps, no readlane round trips), a
// wavefront carries 64/L rows side by side and R such rounds, and rows of different bit widths simply take
// different store paths.  Same arithmetic and same bytes as quant_v1_vec_kernel.
template <int NV, int R, int L>
__global__ __launch_bounds__(kQBlock) void quant_v1_group_kernel(const float *__restrict__ x, uint8_t *__restrict__ q,
                                                                 const int64_t *__restrict__ range,
                                                                 float *__restrict__ params, int64_t n, int F) {
    constexpr int RW = 64 / L;
    const int lane = threadIdx.x & 63, d = lane / L, ll = lane % L;
    const int64_t unit = (int64_t)blockIdx.x * (kQBlock / 64) + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int64_t i0 = unit * (RW * R);
    if (i0 >= n) return;  // wave-uniform
    float bits_f[R];
    int64_t r0[R], r1[R];
    float xv[R][NV][4];
    int off[NV];
    bool act[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        off[v] = (v * L + ll) * 4;
        act[v] = off[v] < F;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t i = i0 + r * RW + d < n ? i0 + r * RW + d : n - 1;  // rows past the end repeat the last row's loads
        bits_f[r] = params[i * 3];
        r0[r] = range[i];
        r1[r] = range[i + 1];
#pragma unroll
        for (int v = 0; v < NV; ++v) vec_load_nt<4>(xv[r][v], x + i * F + (act[v] ? off[v] : 0));  // unconditional
    }
    // The wavefront's rows are consecutive, and so -- in the layout the reference builds (row i's bytes end where
    // row i + 1's begin) -- are their packed bytes: one run of the output.  When every row of the wavefront exists,
    // has a legal bit width and lies where that layout puts it, the codes go to a wave-private piece of LDS first
    // and then out as 4-byte stores over the run (256 consecutive bytes per instruction instead of one 8- to
    // 64-byte piece per lane group and vector: F = 128 at 8 bits 3.9 -> 6.2 TB/s, mixed widths 4.4 -> 6.3);
    // otherwise the lanes store their pieces themselves.
    constexpr int kStage = RW * R * L * NV * 4;   // bytes of the wavefront's rows at 8 bits
    __shared__ __align__(16) uint8_t stage_all[kQBlock / 64][kStage + 16];
    uint8_t *stage = stage_all[threadIdx.x >> 6];
    bool lane_ok = true;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int b = (int)bits_f[r];
        const bool legal = b == 8 || b == 4 || b == 2;
        lane_ok = lane_ok && i0 + r * RW + d < n && legal && r1[r] - r0[r] == (int64_t)((F * (legal ? b : 8) + 7) / 8);
    }
    const int64_t run_lo = uniform64(r0[0]);                                             // lane 0 holds the wavefront's first row
    const int64_t run_hi = range[i0 + RW * R < n ? i0 + RW * R : n];
    const bool rows_ok = __ballot(!lane_ok) == 0ull;
    const bool staged = kV1Staged && contiguous_rows<R>(r0, r1, L) && rows_ok && run_hi - run_lo <= (int64_t)kStage;
    const int mis = (int)((reinterpret_cast<uintptr_t>(q) + (uint64_t)run_lo) & 3);     // the LDS copy keeps the run's alignment modulo 4
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t i = i0 + r * RW + d;
        const int b = (int)bits_f[r];
        float mn = INFINITY, mx = -INFINITY;
        int key = INT_MAX;
#pragma unroll
        for (int v = NV - 1; v >= 0; --v) {
            if (!act[v]) continue;
#pragma unroll
            for (int k = 3; k >= 0; --k) {
                mn = fminf(mn, xv[r][v][k]);
                mx = fmaxf(mx, xv[r][v][k]);
                if (xv[r][v][k] == 0.0f) key = ((off[v] + k) << 1) | (int)(__float_as_uint(xv[r][v][k]) >> 31);
            }
        }
        mn = group_allreduce_f<L, OpMinF>(mn);
        mx = group_allreduce_f<L, OpMaxF>(mx);
        key = group_allmin_i<L>(key);
        const float first = __shfl(xv[r][0][0], lane & ~(L - 1));  // element 0 of the row
        // everything from here on is private to a row's lanes
        if (i >= n || (b != 8 && b != 4 && b != 2)) continue;  // the reference prints an error and leaves the row (quantization_x86.cpp:244-245)
        const float z = (key & 1) ? -0.0f : 0.0f;
        if (mn == 0.0f) mn = z;
        if (mx == 0.0f) mx = z;
        if (first != first) { mn = first; mx = first; }
        float s = (mx - mn) / (float)((1 << b) - 1);
        if (s == 0.0f) s = 1.0f;
        if (ll == 0) { params[i * 3 + 1] = mn; params[i * 3 + 2] = s; }
        const float rinv = __builtin_amdgcn_rcpf(s);
        uint8_t *qo = q + r0[r];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (!act[v]) continue;
            // product with the hardware reciprocal first, IEEE division only for a lane that sees an
            // element within 2^-13 of a rounding tie (same argument as in quant_pack_rows16_kernel)
            uint32_t c[4];
            bool redo = !(s >= 0x1p-100f && s <= 0x1p100f);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float qf = (xv[r][v][k] - mn) * rinv;
                const float ri = rintf(qf);
                if (!(fabsf(qf - ri) < 0.5f - 0x1p-13f)) redo = true;
                c[k] = (uint32_t)ri;
            }
            if (redo) {
#pragma unroll
                for (int k = 0; k < 4; ++k) c[k] = quant_code(xv[r][v][k], mn, s);
            }
            if (staged) store_v1_codes<false>(stage + mis + (int)(r0[r] - run_lo), off[v], b, c);
            else store_v1_codes<true>(qo, off[v], b, c);
        }
    }
    if (staged) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // LDS operations of one wavefront complete in program order
        __builtin_amdgcn_wave_barrier();
        const int nbytes = (int)(run_hi - run_lo);
        uint8_t *qrun = q + run_lo;
        int head = (4 - mis) & 3;
        if (head > nbytes) head = nbytes;
        const int ndw = (nbytes - head) >> 2;
        const int tail_bytes = nbytes - head - 4 * ndw;
        if (lane < head) qrun[lane] = stage[mis + lane];
        const uint32_t *s32 = reinterpret_cast<const uint32_t *>(stage + mis + head);
        uint32_t *q32 = reinterpret_cast<uint32_t *>(qrun + head);
        for (int i = lane; i < ndw; i += 64) __builtin_nontemporal_store(s32[i], q32 + i);
        if (lane < tail_bytes) qrun[head + 4 * ndw + lane] = stage[mis + head + 4 * ndw + lane];
    }
}

template <int NV, int R>
__global__ __launch_bounds__(kQBlock) void dequant_v1_vec_kernel(const uint8_t *__restrict__ q, float *__restrict__ x,
                                                                 const int64_t *__restrict__ range,
                                                                 const float *__restrict__ params, int64_t n, int F) {
    const int lane = threadIdx.x & 63;
    const int64_t i0 = ((int64_t)blockIdx.x * (kQBlock / 64) + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6))) * R;
    if (i0 >= n) return;
    float bits_f[R], zp[R], sc[R];
    int64_t r0[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t i = i0 + r < n ? i0 + r : n - 1;
        bits_f[r] = params[i * 3];
        zp[r] = params[i * 3 + 1];
        sc[r] = params[i * 3 + 2];
        r0[r] = range[i];
    }
    uint32_t w[R][NV];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int b = (int)bits_f[r];
        const uint8_t *qi = q + r0[r];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int off = (v * 64 + lane) * 4;
            w[r][v] = 0;
            if (off >= F || i0 + r >= n) continue;
            if (b == 8) {
                const uint8_t *src = qi + off;
                if ((r0[r] & 3) == 0) w[r][v] = *reinterpret_cast<const uint32_t *>(src);
                else w[r][v] = src[0] | (src[1] << 8) | (src[2] << 16) | ((uint32_t)src[3] << 24);
            } else if (b == 4) {
                const uint8_t *src = qi + off / 2;
                if ((r0[r] & 1) == 0) w[r][v] = *reinterpret_cast<const uint16_t *>(src);
                else w[r][v] = src[0] | (src[1] << 8);
            } else if (b == 2) {
                w[r][v] = qi[off / 4];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t i = i0 + r;
        if (i >= n) break;
        const int b = (int)bits_f[r];
        if (b != 8 && b != 4 && b != 2) continue;
        float *xo = x + i * F;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int off = (v * 64 + lane) * 4;
            if (off >= F) continue;
            const uint32_t ww = w[r][v];
            uint32_t c[4];
            if (b == 8) {
#pragma unroll
                for (int k = 0; k < 4; ++k) c[k] = (ww >> (8 * k)) & 255u;
            } else if (b == 4) {
                c[0] = (ww >> 4) & 15u; c[1] = ww & 15u; c[2] = (ww >> 12) & 15u; c[3] = (ww >> 8) & 15u;
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) c[k] = (ww >> (6 - 2 * k)) & 3u;
            }
            float o[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) o[k] = fmaf((float)c[k], sc[r], zp[r]);
            vec_store_nt<4>(xo + off, o);
        }
    }
}

// The v1 dequantizer over the flat output (F % 4 == 0): as in unpack_dequant_flat_kernel every wavefront store
// covers 1 KB of consecutive output whatever the row width, and a lane looks up what it needs for its four
// elements -- its row's bit width, params and byte offset, then one to four code bytes -- with cacheable
// loads.  Narrow rows no longer leave most of a wavefront idle (F = 64: a wavefront-per-row kernel has 16 of
// 64 lanes at work).
template <int R>
__global__ __launch_bounds__(kQBlock) void dequant_v1_flat_kernel(const uint8_t *__restrict__ q, float *__restrict__ x,
                                                                  const int64_t *__restrict__ range,
                                                                  const float *__restrict__ params, int64_t n_vec, int G) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kQBlock / 64) + (threadIdx.x >> 6);
    const int64_t base = wave * (R * 64) + lane;
    uint32_t w[R];
    float zp[R], sc[R];
    int b[R];
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t i = base + u * 64;
        w[u] = 0; zp[u] = 0.0f; sc[u] = 0.0f; b[u] = 0;
        if (i >= n_vec) continue;
        const int64_t row = i / G;
        const int col = (int)(i - row * G) * 4;
        b[u] = (int)params[row * 3];
        zp[u] = params[row * 3 + 1];
        sc[u] = params[row * 3 + 2];
        const int64_t r0 = range[row];
        const uint8_t *qi = q + r0;
        if (b[u] == 8) {
            const uint8_t *src = qi + col;
            if ((r0 & 3) == 0) w[u] = *reinterpret_cast<const uint32_t *>(src);
            else w[u] = src[0] | (src[1] << 8) | (src[2] << 16) | ((uint32_t)src[3] << 24);
        } else if (b[u] == 4) {
            const uint8_t *src = qi + col / 2;
            if ((r0 & 1) == 0) w[u] = *reinterpret_cast<const uint16_t *>(src);
            else w[u] = src[0] | (src[1] << 8);
        } else if (b[u] == 2) {
            w[u] = qi[col / 4];
        }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const int64_t i = base + u * 64;
        if (i >= n_vec || (b[u] != 8 && b[u] != 4 && b[u] != 2)) continue;  // other widths: the row is left alone
        const uint32_t ww = w[u];
        uint32_t c[4];
        if (b[u] == 8) {
#pragma unroll
            for (int k = 0; k < 4; ++k) c[k] = (ww >> (8 * k)) & 255u;
        } else if (b[u] == 4) {
            c[0] = (ww >> 4) & 15u; c[1] = ww & 15u; c[2] = (ww >> 12) & 15u; c[3] = (ww >> 8) & 15u;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) c[k] = (ww >> (6 - 2 * k)) & 3u;
        }
        float o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = fmaf((float)c[k], sc[u], zp[u]);
        vec_store_nt<4>(x + i * 4, o);
    }
}

// Position of every row in the padded row space (EPB rows per packed row, every segment starting
// on a packed-row boundary): slot[r] = pseg[p] * EPB + (r - seg[p]) for the segment p holding r.
// Packed row = slot / EPB, position inside the byte = slot % EPB.
__global__ __launch_bounds__(kQBlock) void row_slots_kernel(const int32_t *__restrict__ seg,
                                                            const int32_t *__restrict__ pseg, int P, int epb,
                                                            int64_t n_rows, int32_t *__restrict__ slot) {
    const int64_t r = (int64_t)blockIdx.x * kQBlock + threadIdx.x;
    if (r >= n_rows) return;
    int lo = 0, hi = P - 1;  // the p with seg[p] <= r < seg[p+1]
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (seg[mid + 1] > r) hi = mid; else lo = mid + 1;
    }
    slot[r] = pseg[lo] * epb + (int32_t)(r - seg[lo]);
}

// ------------------------------------------------------------------------------------------------
// Launch tables.
// ------------------------------------------------------------------------------------------------
static int env_flag(const char *name, int dflt) {
    const char *e = getenv(name);
    return e ? atoi(e) : dflt;
}

struct RowsArgs {
    RowSrc x_in; uint8_t *q_out;                                     // quantize
    const uint8_t *q_in; float *x_out;                               // dequantize
    ParamBuf params;                                                 // written by quantize, read by dequantize
    const int32_t *seg; const int32_t *pseg; int P; int n_packed; int F; bool quantize;
    int64_t single_rows;  // the row count when P == 1 (kernels then read no segment table), else -1
    bool flat;            // dequantize over the flat output (default) vs the row-tiled kernels
    bool exact_division;  // diagnostic: IEEE division for every element (the results are identical either way)
};

// ONLY = 1: shapes the quantizer never takes (rows of up to 1024 aligned floats go to the sixteen-lane and stream
// kernels); ONLY = 2: shapes the dequantizer never takes.
template <int BITS, int VEC, int G, int NV, int ONLY = 0>
static void launch_rows(const RowsArgs &a, hipStream_t st) {
    constexpr int NPR = kRowsPerGroup / (8 / BITS);
    constexpr int GPB = kQBlock / G;
    const int n_units = (a.n_packed + NPR - 1) / NPR;
    const int nb = (n_units + GPB - 1) / GPB;
    ProfScope prof(a.quantize ? K_QUANT_PACK_ROWS : K_UNPACK_DEQUANT_ROWS, st);
    if constexpr (ONLY != 1) {
        if (a.quantize && a.exact_division) {
            hipLaunchKernelGGL((quant_pack_rows_kernel<BITS, VEC, G, NV, true>), dim3(nb), dim3(kQBlock), 0, st, a.x_in,
                               a.q_out, a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, n_units);
            return;
        }
        if (a.quantize) {
            hipLaunchKernelGGL((quant_pack_rows_kernel<BITS, VEC, G, NV, false>), dim3(nb), dim3(kQBlock), 0, st, a.x_in,
                               a.q_out, a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, n_units);
            return;
        }
    }
    if constexpr (ONLY != 2)
        hipLaunchKernelGGL((unpack_dequant_rows_kernel<BITS, VEC, G, NV>), dim3(nb), dim3(kQBlock), 0, st, a.q_in,
                           a.x_out, a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, n_units);
}

// Rows that are not a whole number of lane-group passes (every width but 4 * L * NV floats) write their packed
// bytes through the wave-private LDS stage.  Measured on MI355X at 256 M elements against stores straight from the
// lanes: F = 300 / 600 / 1000 5.2-5.9 -> 6.0-6.2 TB/s, F = 602 4.7-5.2 -> 5.6-5.9 TB/s; rows that are whole passes
// (F = 64 ... 1024 in steps of the lane-group width) gain nothing from it and keep the direct stores.
template <int BITS, int NV, int L>
static void launch_quant16_ragged(const RowsArgs &a, hipStream_t st) {
    constexpr int RL = NV >= 4 ? 1 : 4 / NV;
    constexpr int EPB = 8 / BITS;
    constexpr int RW = 64 / L;
    const int64_t padded = (int64_t)a.n_packed * EPB;
    const int n_units = (int)((padded + RW * RL - 1) / (RW * RL));
    const int nb = (n_units + kQBlock / 64 - 1) / (kQBlock / 64);
    ProfScope prof(K_QUANT_PACK_ROWS, st);
    hipLaunchKernelGGL((quant_pack_rows16_kernel<BITS, NV, RL, false, false, L, true, true>), dim3(nb), dim3(kQBlock), 0, st,
                       a.x_in, a.q_out, a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, n_units);
}

// The same for rows of 1025 ... 2560 floats: a wavefront holds four rows in registers, NV vectors per lane each.
template <int BITS, int NV>
static void launch_rows_ragged(const RowsArgs &a, hipStream_t st) {
    constexpr int NPR = kRowsPerGroup / (8 / BITS);
    constexpr int GPB = kQBlock / 64;
    const int n_units = (a.n_packed + NPR - 1) / NPR;
    const int nb = (n_units + GPB - 1) / GPB;
    ProfScope prof(K_QUANT_PACK_ROWS, st);
    hipLaunchKernelGGL((quant_pack_rows_kernel<BITS, 4, 64, NV, false, true>), dim3(nb), dim3(kQBlock), 0, st, a.x_in, a.q_out,
                       a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, n_units);
}
template <int BITS>
static void dispatch_rows_ragged_wide(const RowsArgs &a, hipStream_t st) {
    const int nvec = (a.F + 3) / 4;
    if (nvec <= 320) return launch_rows_ragged<BITS, 5>(a, st);
    if (nvec <= 384) return launch_rows_ragged<BITS, 6>(a, st);
    if (nvec <= 512) return launch_rows_ragged<BITS, 8>(a, st);
    return launch_rows_ragged<BITS, 10>(a, st);
}

// Widths or row starts that are not a multiple of four floats, up to 1024 floats per row.
template <int BITS>
static void dispatch_quant16_ragged(const RowsArgs &a, hipStream_t st) {
    const int nvec = (a.F + 3) / 4;
    if (nvec <= 1) return launch_quant16_ragged<BITS, 1, 1>(a, st);
    if (nvec <= 2) return launch_quant16_ragged<BITS, 1, 2>(a, st);
    if (nvec <= 4) return launch_quant16_ragged<BITS, 1, 4>(a, st);
    if (nvec <= 8) return launch_quant16_ragged<BITS, 1, 8>(a, st);
    if (nvec <= 16) return launch_quant16_ragged<BITS, 2, 8>(a, st);
    if (nvec <= 32) return launch_quant16_ragged<BITS, 4, 8>(a, st);   // (sixteen lanes with two vectors each: 3 ... 20 % slower)
    if (nvec <= 64) return launch_quant16_ragged<BITS, 4, 16>(a, st);
    if (nvec <= 128) return launch_quant16_ragged<BITS, 8, 16>(a, st);
    if (nvec <= 160) return launch_quant16_ragged<BITS, 10, 16>(a, st);
    return launch_quant16_ragged<BITS, 16, 16>(a, st);
}

template <int BITS, int NV, int L = 16>
static void launch_quant16(const RowsArgs &a, hipStream_t st) {
    constexpr int RL = NV >= 4 ? 1 : 4 / NV;
    constexpr int EPB = 8 / BITS;
    constexpr int RW = 64 / L;
    const int64_t padded = (int64_t)a.n_packed * EPB;
    const int n_units = (int)((padded + RW * RL - 1) / (RW * RL));
    const int nb = (n_units + kQBlock / 64 - 1) / (kQBlock / 64);
    ProfScope prof(K_QUANT_PACK_ROWS, st);
    if (a.exact_division)
        hipLaunchKernelGGL((quant_pack_rows16_kernel<BITS, NV, RL, true, false, L>), dim3(nb), dim3(kQBlock), 0, st, a.x_in, a.q_out,
                           a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, n_units);
    else if (a.F == 4 * L * NV)
        hipLaunchKernelGGL((quant_pack_rows16_kernel<BITS, NV, RL, false, true, L>), dim3(nb), dim3(kQBlock), 0, st, a.x_in, a.q_out,
                           a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, n_units);
    else
        hipLaunchKernelGGL((quant_pack_rows16_kernel<BITS, NV, RL, false, false, L, false, true>), dim3(nb), dim3(kQBlock), 0, st,
                           a.x_in, a.q_out, a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, n_units);
}

// Lane-slot shape of the stream quantizer for rows of F floats: NV vectors per lane (one of the instantiated
// values) and gw packed rows per wavefront, chosen to fill the wavefront's NV * 64 vector slots.
static bool stream_shape(int F, int epb, bool ragged, int *nv_out, int *gw_out) {
    // Rows of whole float4: four vectors per lane first.  The kernel then waits on memory, not on instruction issue,
    // and what counts is how many wavefronts a CU holds (15 KB of LDS per workgroup, ~45 registers: F = 128 / 256
    // 5.8-6.1 -> 6.1-6.5 TB/s against eight); eight where four would leave more than 2.5 % more slots empty.  The
    // ragged path does more per wavefront (short vectors, output words that straddle rows) and shares it among eight
    // vectors first (F = 123 / 250: 5.3 / 5.4 -> 5.6 / 5.9 TB/s against four).  Ten and more cost registers and LDS
    // and are taken only for a clearly better fill or when a packed row needs them.
    static const int nvs_aligned[] = {4, 8, 10, 12, 16, 20}, nvs_ragged[] = {8, 4, 10, 12, 16, 20};
    const int *nvs = ragged ? nvs_ragged : nvs_aligned;
    const int vpr = (F + 3) / 4;
    double best = 0.0;
    for (int k = 0; k < 6; ++k) {
        const int nv = nvs[k];
        if (best > 0.0 && (nv > 12 || (nv > 10 && best >= 0.8))) break;   // (twelve still competes with a poor fill)
        const int gw = std::min(nv * 64 / (epb * vpr), kStreamRows / epb);
        if (gw < 1) continue;
        const double fill = (double)gw * epb * vpr / (nv * 64);
        if (fill > best + 0.025) {
            best = fill;
            *nv_out = nv;
            *gw_out = gw;
        }
    }
    return best > 0.0;
}

template <int BITS, int NV, bool RAGGED>
static void launch_quant_stream_nv(const RowsArgs &a, int gw, hipStream_t st) {
    constexpr int WAVES = stream_wave_bytes(NV) * 4 <= 64 * 1024 ? 4 : 2;
    const int n_units = (a.n_packed + gw - 1) / gw;
    const int nb = (n_units + WAVES - 1) / WAVES;
    const uint32_t vpr = (uint32_t)(a.F + 3) / 4;   // (at most NV * 64 <= 1280: the kernel divides slots by it with one multiply)
    ProfScope prof(K_QUANT_PACK_ROWS, st);
    hipLaunchKernelGGL((quant_pack_stream_kernel<BITS, NV, RAGGED, WAVES>), dim3(nb), dim3(64 * WAVES), 0, st, a.x_in, a.q_out,
                       a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F, gw, n_units,
                       (uint32_t)(((1u << 21) + vpr - 1) / vpr));
}

template <int BITS>
static bool launch_quant_stream(const RowsArgs &a, hipStream_t st) {
    int nv = 0, gw = 0;
    // (from 9 floats: three vectors per row fill 3/4 of the slots of 64 rows x four vectors, and the tensor holds the four
    //  floats the last load needs; narrower rows are faster with the lane-group kernels: F = 8 6.6 against 5.9 TB/s)
    if (a.x_in.ld < a.F || a.x_in.n_src >= ((int64_t)1 << 31) || a.F < 9) return false;
    const bool ragged = a.F % 4 != 0 || !aligned(a.q_out, 4);
    if (!stream_shape(a.F, 8 / BITS, ragged, &nv, &gw)) return false;
#define SGNN_STREAM(NV_)                                                       \
    case NV_:                                                                  \
        if (ragged) launch_quant_stream_nv<BITS, NV_, true>(a, gw, st);        \
        else launch_quant_stream_nv<BITS, NV_, false>(a, gw, st);              \
        break
    switch (nv) {
        SGNN_STREAM(4); SGNN_STREAM(8); SGNN_STREAM(10); SGNN_STREAM(12); SGNN_STREAM(16); SGNN_STREAM(20);
        default: return false;
    }
#undef SGNN_STREAM
    return true;
}

template <int BITS, int R>
static void launch_dequant_flat_r(const RowsArgs &a, int64_t n_rows, hipStream_t st) {
    const int G = a.F / 4;
    const int64_t n_vec = n_rows * G;
    const int64_t n_waves = (n_vec + R * 64 - 1) / (R * 64);
    const unsigned nb = (unsigned)((n_waves + kQBlock / 64 - 1) / (kQBlock / 64));
    const bool pow2 = (G & (G - 1)) == 0;
    int g_shift = 0;
    while ((1 << g_shift) < G) ++g_shift;
    const bool segmented = BITS != 8 && a.P > 1;
    ProfScope prof(K_UNPACK_DEQUANT_ROWS, st);
#define SGNN_FLAT(POW2, SEGM)                                                                                        \
    hipLaunchKernelGGL((unpack_dequant_flat_kernel<BITS, R, POW2, SEGM>), dim3(nb), dim3(kQBlock), 0, st, a.q_in, \
                       a.x_out, a.params, a.seg, a.pseg, a.P, G, g_shift, n_vec)
    if (pow2 && segmented) SGNN_FLAT(true, true);
    else if (pow2) SGNN_FLAT(true, false);
    else if (segmented) SGNN_FLAT(false, true);
    else SGNN_FLAT(false, false);
#undef SGNN_FLAT
}

// Measured on MI355X (1 M x 256, 2 M x 128, 1 M x 64, 400 k x 600): ordinary (cacheable) loads of the
// packed words beat non-temporal ones by 15-40 % (rows that share a word hit in cache, and the
// write stream is not disturbed), and the shortest waves win: one 1-KB store per wave for sub-byte
// codes on power-of-two widths, two otherwise.
template <int BITS>
static void launch_dequant_flat(const RowsArgs &a, int64_t n_rows, hipStream_t st) {
    const int G = a.F / 4;
    // With several segments and sub-byte codes every wavefront first looks its segment up, and the shortest waves
    // lose: 1 M x 256 int2 in eight segments 0.194 ms with one store per wave, 0.169 with two, 0.160 with four
    // (one segment: 0.155 / 0.171 / 0.170); int4 0.199 / 0.162 / 0.162.
    int r;
    if (BITS == 8) r = 2;
    else if (a.P <= 1) r = (G & (G - 1)) == 0 ? 1 : BITS == 2 ? 4 : 2;
    else r = BITS == 2 && a.F <= 256 ? 4 : 2;
    if (r == 4) launch_dequant_flat_r<BITS, 4>(a, n_rows, st);
    else if (r == 2) launch_dequant_flat_r<BITS, 2>(a, n_rows, st);
    else launch_dequant_flat_r<BITS, 1>(a, n_rows, st);
}

template <int BITS, int VEC, int R>
static void launch_dequant_flat_ragged_r(const RowsArgs &a, int64_t n_rows, hipStream_t st) {
    const int64_t n_elem = n_rows * (int64_t)a.F;
    const int64_t n_vec = (n_elem + 3) / 4;
    const int64_t n_waves = (n_vec + R * 64 - 1) / (R * 64);
    const unsigned nb = (unsigned)((n_waves + kQBlock / 64 - 1) / (kQBlock / 64));
    ProfScope prof(K_UNPACK_DEQUANT_ROWS, st);
    const char *odd2 = getenv("SGNN_DEQUANT_ODD2");
    const bool two_rows = !(odd2 && odd2[0] == '0');
    if (VEC == 1 && a.F >= 4 && two_rows) {
        if (BITS != 8 && a.P > 1)
            hipLaunchKernelGGL((unpack_dequant_flat_odd_kernel<BITS, R, true>), dim3(nb), dim3(kQBlock), 0, st, a.q_in, a.x_out,
                               a.params, a.seg, a.pseg, a.P, a.F, (int)n_rows, n_elem, a.n_packed);
        else
            hipLaunchKernelGGL((unpack_dequant_flat_odd_kernel<BITS, R, false>), dim3(nb), dim3(kQBlock), 0, st, a.q_in, a.x_out,
                               a.params, a.seg, a.pseg, a.P, a.F, (int)n_rows, n_elem, a.n_packed);
        return;
    }
    if (BITS != 8 && a.P > 1)
        hipLaunchKernelGGL((unpack_dequant_flat_ragged_kernel<BITS, VEC, R, true>), dim3(nb), dim3(kQBlock), 0, st, a.q_in,
                           a.x_out, a.params, a.seg, a.pseg, a.P, a.F, n_elem);
    else
        hipLaunchKernelGGL((unpack_dequant_flat_ragged_kernel<BITS, VEC, R, false>), dim3(nb), dim3(kQBlock), 0, st, a.q_in,
                           a.x_out, a.params, a.seg, a.pseg, a.P, a.F, n_elem);
}

template <int BITS, int VEC>
static void launch_dequant_flat_ragged(const RowsArgs &a, int64_t n_rows, hipStream_t st) {
    // several segments and sub-byte codes: four stores per wavefront per segment lookup (see launch_dequant_flat)
    if (BITS != 8 && a.P > 1) launch_dequant_flat_ragged_r<BITS, VEC, 4>(a, n_rows, st);
    else launch_dequant_flat_ragged_r<BITS, VEC, 2>(a, n_rows, st);
}

// Rows the workgroup-per-packed-row kernel holds in registers: at most 4 * 512 * 4 floats.
static bool rows_fit_block(int F) { return F >= 4 && F / 4 <= 512 * 4; }
template <int BITS>
static void launch_quant_block(const RowsArgs &a, hipStream_t st) {
    const int nvf = a.F / 4;
    ProfScope prof(K_QUANT_PACK_ROWS, st);
#define SGNN_BLOCKQ(TB_, NVT_)                                                                                              \
    hipLaunchKernelGGL((quant_pack_rows_block_kernel<BITS, TB_, NVT_>), dim3(a.n_packed), dim3(TB_), 0, st, a.x_in, a.q_out, \
                       a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F)
    // the fewest vectors per thread that hold the row, in the smaller workgroup where both do
    if (nvf <= 256) SGNN_BLOCKQ(256, 1);
    else if (nvf <= 512) SGNN_BLOCKQ(256, 2);
    else if (nvf <= 768) SGNN_BLOCKQ(256, 3);
    else if (nvf <= 1024) SGNN_BLOCKQ(512, 2);
    else if (nvf <= 1536) SGNN_BLOCKQ(512, 3);
    else SGNN_BLOCKQ(512, 4);
#undef SGNN_BLOCKQ
}

template <int BITS>
static void launch_rows_wide(const RowsArgs &a, hipStream_t st) {
    const int nb = (a.n_packed + kQBlock / 64 - 1) / (kQBlock / 64);
    ProfScope prof(a.quantize ? K_QUANT_PACK_ROWS : K_UNPACK_DEQUANT_ROWS, st);
    if (a.quantize)
        hipLaunchKernelGGL((quant_pack_rows_wide_kernel<BITS>), dim3(nb), dim3(kQBlock), 0, st, a.x_in, a.q_out,
                           a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F);
    else
        hipLaunchKernelGGL((unpack_dequant_rows_wide_kernel<BITS>), dim3(nb), dim3(kQBlock), 0, st, a.q_in, a.x_out,
                           a.params, a.seg, a.pseg, a.P, a.single_rows, a.n_packed, a.F);
}

template <int BITS, int VEC>
static void dispatch_rows_shape(int nvec, const RowsArgs &a, hipStream_t st) {
    if constexpr (VEC == 4) {
        if (a.quantize) {
            // rows of up to 128 floats: eight lanes per row (with the staged output also for rows of 17 ... 31 vectors,
            // whose groups have idle lanes either way: F = 72 / 80 3.8-4.7 -> 4.7-5.7 TB/s, F = 100 / 112 +3 ... 6 %)
            if (nvec <= 1) return launch_quant16<BITS, 1, 1>(a, st);
            if (nvec <= 2) return launch_quant16<BITS, 1, 2>(a, st);
            if (nvec <= 4) return launch_quant16<BITS, 1, 4>(a, st);
            // rows of 5 ... 12 vectors other than the whole eight-lane pass F = 32: four lanes per row (F = 20 / 24:
            // 3.2-4.3 -> 4.1-5.2 TB/s, F = 28 ... 48: +4 ... 17 %; from 13 vectors on eight lanes win, F = 52 ... 64 by
            // 6 ... 18 %)
            if (nvec <= 8 && a.F != 32) return launch_quant16<BITS, 2, 4>(a, st);
            if (nvec > 8 && nvec <= 12) return launch_quant16<BITS, 4, 4>(a, st);
            if (nvec <= 8) return launch_quant16<BITS, 1, 8>(a, st);
            if (nvec <= 16) return launch_quant16<BITS, 2, 8>(a, st);
            if (nvec <= 32) return launch_quant16<BITS, 4, 8>(a, st);
            if (nvec <= 64) return launch_quant16<BITS, 4>(a, st);
            if (nvec <= 128) return launch_quant16<BITS, 8>(a, st);
            if (nvec <= 160) return launch_quant16<BITS, 10>(a, st);
            if (nvec <= 256) return launch_quant16<BITS, 16>(a, st);
        }
    }
    constexpr int kDq = VEC == 4 ? 1 : 0;   // (VEC == 4: the quantizer has returned above for rows of up to 256 vectors)
    if (nvec <= 16) return launch_rows<BITS, VEC, 16, 1, kDq>(a, st);
    if (nvec <= 32) return launch_rows<BITS, VEC, 32, 1, kDq>(a, st);
    if (nvec <= 64) return launch_rows<BITS, VEC, 64, 1, kDq>(a, st);
    if (nvec <= 128) return launch_rows<BITS, VEC, 64, 2, kDq>(a, st);
    if constexpr (VEC == 4) {
        if (nvec <= 192) return launch_rows<BITS, VEC, 64, 3, 1>(a, st);
        if (nvec <= 256) return launch_rows<BITS, VEC, 64, 4, 1>(a, st);
        if (a.quantize) {  // rows of up to 2048 floats still fit a wavefront's registers (four rows, NV vectors per lane each)
            if (nvec <= 320) return launch_rows<BITS, VEC, 64, 5, 2>(a, st);
            if (nvec <= 384) return launch_rows<BITS, VEC, 64, 6, 2>(a, st);
            if (nvec <= 512) return launch_rows<BITS, VEC, 64, 8, 2>(a, st);
            if (nvec <= 640) return launch_rows<BITS, VEC, 64, 10, 2>(a, st);
        }
    } else {
        if (nvec <= 256) return launch_rows<BITS, VEC, 64, 4>(a, st);
        if (nvec <= 512) return launch_rows<BITS, VEC, 64, 8>(a, st);
    }
    launch_rows_wide<BITS>(a, st);
}

template <int BITS>
static void dispatch_rows(int vec, const RowsArgs &a, hipStream_t st) {
    if (vec == 4) dispatch_rows_shape<BITS, 4>(a.F / 4, a, st);
    else if (vec == 2) dispatch_rows_shape<BITS, 2>(a.F / 2, a, st);
    else dispatch_rows_shape<BITS, 1>(a.F, a, st);
}

// Widths the stream quantizer takes by default (measured at 256 M elements per width, all three code widths):
//   - rows of whole float4 in aligned buffers, except the multiples of 64 floats up to 768, which are whole passes of
//     the sixteen-lane kernel (128 ... 768: level with it at int4 / int2 within +-4 %, 3-6 % behind at int8; F = 64 at
//     int4 / int2 is the exception and takes the stream kernel: 6.16 / 5.95 -> 6.27 / 6.34 TB/s).  It gains most where
//     a row leaves lane slots of that kernel idle: F = 20 / 36 / 72 / 100 / 160: 4.4-5.7 -> 5.9-6.3 TB/s;
//   - rows of up to 256 floats that are not whole float4 or sit in unaligned buffers, where the lane-group kernels'
//     per-row 16-byte pieces at 4-byte alignments cost most (F = 123: 4.4-4.8 -> 5.5-5.6 TB/s, F = 37: 3.4-3.9 -> 5.4-5.5);
//     wider ones at int4 / int2 while a packed row fits twelve vectors per lane (F = 602: 5.7 / 5.5 -> 5.9 / 5.9 TB/s; at
//     int8 the lane-group kernels are level or ahead: F = 301 5.9 against 5.5);
//   - beyond 1024 floats every row a wavefront can hold (F = 2050: 3.7 -> 4.7 TB/s at int8 and int4).
//   - rows picked by a row index, or with a pitch: the same up to 256 floats (F = 100 through a sorted index: 4.3-4.6 ->
//     4.9-5.5 TB/s); wider ones keep the lane-group kernels (F = 602 through an index: 5.0-5.6 against 4.9-5.0).
static bool stream_wanted(int F, int vec, int bits, bool rows_by_table) {
    if (F > 1024) return true;
    if (rows_by_table && F > 256) return false;
    if (vec == 4) return !(F % 64 == 0 && F <= 768) || (F == 64 && bits < 8);
    return F <= 256 || (bits < 8 && (F + 3) / 4 * (8 / bits) <= 12 * 64);
}

static int run_rows(const RowsArgs &a, int bits, int64_t n_rows, const void *fp32_ptr, const void *u8_ptr,
                    hipStream_t st) {
    SGNN_REQUIRE(bits == 8 || bits == 4 || bits == 2, "bits=%d, expected 8, 4 or 2", bits);
    SGNN_REQUIRE(a.P >= 1, "P=%d, expected >= 1", a.P);
    SGNN_REQUIRE(a.F > 0, "feature width F=%d out of range", a.F);
    SGNN_REQUIRE(n_rows >= 0 && a.n_packed >= 0, "negative row count");
    if (n_rows == 0 || a.n_packed == 0) return SGNN_OK;
    SGNN_REQUIRE(n_rows * (int64_t)a.F < ((int64_t)1 << 40), "n_rows * F = %lld elements is beyond the supported grid",
                 (long long)(n_rows * (int64_t)a.F));
    SGNN_REQUIRE(a.P > 1 || (int64_t)a.n_packed == (n_rows + 8 / bits - 1) / (8 / bits),
                 "one segment of %lld rows needs %lld packed rows, got %d", (long long)n_rows,
                 (long long)((n_rows + 8 / bits - 1) / (8 / bits)), a.n_packed);
    SGNN_REQUIRE(fp32_ptr && u8_ptr && a.seg && a.pseg, "null pointer argument");
    SGNN_REQUIRE(a.params.p != nullptr, "params is null");
    SGNN_REQUIRE((int64_t)a.n_packed * (8 / bits) < (int64_t)INT32_MAX, "too many rows for 32-bit row units");
    const int64_t ld = a.quantize ? a.x_in.ld : (int64_t)a.F;
    int vec = 1;
    if (a.F % 4 == 0 && ld % 4 == 0 && aligned(fp32_ptr, 16) && aligned(u8_ptr, 4)) vec = 4;
    else if (a.F % 2 == 0 && ld % 2 == 0 && aligned(fp32_ptr, 8) && aligned(u8_ptr, 2)) vec = 2;
    SGNN_REQUIRE(aligned(a.params.p, a.params.bf16 ? 4 : 8), "params must be %d-byte aligned", a.params.bf16 ? 4 : 8);
    const int stream = env_flag("SGNN_QUANT_STREAM", -1);   // 1: every width the stream quantizer can take, 0: never
    bool taken = false;
    const bool block_rows_wanted = a.F > (bits == 2 ? 1280 : 1920) && rows_fit_block(a.F);
    if (a.quantize && !a.exact_division && (stream > 0 || (stream < 0 && !block_rows_wanted && stream_wanted(a.F, vec, bits, a.x_in.index != nullptr || a.x_in.ld != a.F))))
        taken = bits == 8 ? launch_quant_stream<8>(a, st) : bits == 4 ? launch_quant_stream<4>(a, st) : launch_quant_stream<2>(a, st);
    if (taken) {
    } else if (a.quantize && !a.exact_division && block_rows_wanted) {
        // rows a wavefront cannot hold (int2 beyond 1280 floats), or holds only with few wavefronts per CU: a workgroup
        // per packed row, the rows in its registers (F = 2050: 5.0 / 5.0 / 3.5 -> 5.9 / 6.1 / 5.8 TB/s at int8 / int4 / int2,
        // F = 3703: 4.9 / 2.6 / 2.7 -> 5.7 / 5.9 / 5.8, F = 1433 int2: 4.7 -> 5.6; at int8 / int4 the stream kernel is ahead up to
        // about 1900 floats: F = 1700 6.3 / 6.2 against 5.6 / 6.0)
        if (bits == 8) launch_quant_block<8>(a, st);
        else if (bits == 4) launch_quant_block<4>(a, st);
        else launch_quant_block<2>(a, st);
    } else if (!a.quantize && vec == 4 && a.flat) {
        if (bits == 8) launch_dequant_flat<8>(a, n_rows, st);
        else if (bits == 4) launch_dequant_flat<4>(a, n_rows, st);
        else launch_dequant_flat<2>(a, n_rows, st);
    } else if (!a.quantize && a.flat && a.F % 4 != 0 && aligned(fp32_ptr, 16) && (a.F % 2 != 0 || aligned(u8_ptr, 2))) {
        // widths that are not a multiple of four: flat 16-byte stores made of float2 / float pieces
        const bool even = a.F % 2 == 0;
        if (bits == 8) even ? launch_dequant_flat_ragged<8, 2>(a, n_rows, st) : launch_dequant_flat_ragged<8, 1>(a, n_rows, st);
        else if (bits == 4) even ? launch_dequant_flat_ragged<4, 2>(a, n_rows, st) : launch_dequant_flat_ragged<4, 1>(a, n_rows, st);
        else even ? launch_dequant_flat_ragged<2, 2>(a, n_rows, st) : launch_dequant_flat_ragged<2, 1>(a, n_rows, st);
    } else if (a.quantize && vec != 4 && !a.exact_division && a.F <= 1024) {
        if (bits == 8) dispatch_quant16_ragged<8>(a, st);
        else if (bits == 4) dispatch_quant16_ragged<4>(a, st);
        else dispatch_quant16_ragged<2>(a, st);
    } else if (a.quantize && vec != 4 && !a.exact_division && a.F <= 2560) {
        if (bits == 8) dispatch_rows_ragged_wide<8>(a, st);
        else if (bits == 4) dispatch_rows_ragged_wide<4>(a, st);
        else dispatch_rows_ragged_wide<2>(a, st);
    } else if (bits == 8) dispatch_rows<8>(vec, a, st);
    else if (bits == 4) dispatch_rows<4>(vec, a, st);
    else dispatch_rows<2>(vec, a, st);
    SGNN_HIP_CHECK(hipGetLastError());
    return SGNN_OK;
}

}  // namespace sgnn

using namespace sgnn;

extern "C" int64_t sgnn_quant_segment_offsets(const int32_t *seg_host, int P, int bits, int32_t *pseg_host) {
    if (!(bits == 8 || bits == 4 || bits == 2)) return fail(SGNN_ERR_ARG, "bits=%d, expected 8, 4 or 2", bits);
    if (P < 1 || !seg_host || !pseg_host) return fail(SGNN_ERR_ARG, "bad segment table");
    const int epb = 8 / bits;
    if (seg_host[0] != 0) return fail(SGNN_ERR_RANGE, "segment table must start at 0");
    int64_t acc = 0;
    pseg_host[0] = 0;
    for (int p = 0; p < P; ++p) {
        const int64_t n = (int64_t)seg_host[p + 1] - seg_host[p];
        if (n < 0) return fail(SGNN_ERR_RANGE, "segment table decreases at %d", p);
        acc += (n + epb - 1) / epb;
        if (acc > INT32_MAX) return fail(SGNN_ERR_RANGE, "packed row count overflows 31 bits");
        pseg_host[p + 1] = (int32_t)acc;
    }
    return acc;
}

extern "C" int sgnn_quant_row_slots(const int32_t *seg, const int32_t *pseg, int P, int bits, int64_t n_rows,
                                    int32_t *row_slot, sgnn_stream_t stream) {
    SGNN_REQUIRE(bits == 8 || bits == 4 || bits == 2, "bits=%d, expected 8, 4 or 2", bits);
    SGNN_REQUIRE(P >= 1 && n_rows >= 0 && n_rows < INT32_MAX / 4, "bad segment table size");
    if (n_rows == 0) return SGNN_OK;
    SGNN_REQUIRE(seg && pseg && row_slot, "null pointer argument");
    const int64_t nb = (n_rows + kQBlock - 1) / kQBlock;
    hipLaunchKernelGGL(row_slots_kernel, dim3((uint32_t)nb), dim3(kQBlock), 0, (hipStream_t)stream, seg, pseg, P, 8 / bits,
                       n_rows, row_slot);
    SGNN_HIP_CHECK(hipGetLastError());
    return SGNN_OK;
}

static int quant_pack_rows_impl(const RowSrc &src, uint8_t *q, void *params, int params_bf16, const int32_t *seg,
                                const int32_t *pseg, int P, int64_t n_rows, int64_t n_packed_rows, int64_t F, int bits,
                                sgnn_stream_t stream) {
    SGNN_REQUIRE(F > 0 && F < (1 << 24) && n_packed_rows < INT32_MAX, "size out of range");
    SGNN_REQUIRE(src.ld >= F, "row stride %lld is smaller than the feature width %lld", (long long)src.ld, (long long)F);
    SGNN_REQUIRE(src.index == nullptr || src.n_src > 0 || n_rows == 0, "row index given but the source has no rows");
    SGNN_REQUIRE(params_bf16 == 0 || params_bf16 == 1, "params_bf16=%d, expected 0 or 1", params_bf16);
    RowsArgs a{};
    a.x_in = src; a.q_out = q; a.params = ParamBuf{params, params_bf16}; a.seg = seg; a.pseg = pseg; a.P = P;
    a.n_packed = (int)n_packed_rows; a.F = (int)F; a.quantize = true;
    a.single_rows = P == 1 ? n_rows : -1;
    { const char *e = getenv("SGNN_QUANT_EXACT_DIV"); a.exact_division = e && e[0] == '1'; }
    return run_rows(a, bits, n_rows, src.x, q, (hipStream_t)stream);
}

static int unpack_dequant_rows_impl(const uint8_t *q, float *x, const void *params, int params_bf16,
                                    const int32_t *seg, const int32_t *pseg, int P, int64_t n_rows,
                                    int64_t n_packed_rows, int64_t F, int bits, sgnn_stream_t stream) {
    SGNN_REQUIRE(F > 0 && F < (1 << 24) && n_packed_rows < INT32_MAX, "size out of range");
    SGNN_REQUIRE(params_bf16 == 0 || params_bf16 == 1, "params_bf16=%d, expected 0 or 1", params_bf16);
    RowsArgs a{};
    a.q_in = q; a.x_out = x; a.params = ParamBuf{const_cast<void *>(params), params_bf16}; a.seg = seg; a.pseg = pseg;
    a.P = P; a.n_packed = (int)n_packed_rows; a.F = (int)F; a.quantize = false;
    a.single_rows = P == 1 ? n_rows : -1;
    { const char *e = getenv("SGNN_DEQUANT_FLAT"); a.flat = !(e && e[0] == '0'); }
    return run_rows(a, bits, n_rows, x, q, (hipStream_t)stream);
}

extern "C" int sgnn_quant_pack_rows_f32(const float *x, uint8_t *q, float *params, const int32_t *seg,
                                        const int32_t *pseg, int P, int64_t n_rows, int64_t n_packed_rows,
                                        int64_t F, int bits, sgnn_stream_t stream) {
    return quant_pack_rows_impl(RowSrc{x, F, nullptr, n_rows}, q, params, 0, seg, pseg, P, n_rows, n_packed_rows, F,
                                bits, stream);
}

extern "C" int sgnn_quant_pack_rows_wire_f32(const float *x, int64_t ldx, const int64_t *row_index, int64_t n_src_rows,
                                             uint8_t *q, void *params, int params_bf16, const int32_t *seg,
                                             const int32_t *pseg, int P, int64_t n_rows, int64_t n_packed_rows,
                                             int64_t F, int bits, sgnn_stream_t stream) {
    return quant_pack_rows_impl(RowSrc{x, ldx, row_index, row_index ? n_src_rows : n_rows}, q, params, params_bf16,
                                seg, pseg, P, n_rows, n_packed_rows, F, bits, stream);
}

extern "C" int sgnn_unpack_dequant_rows_f32(const uint8_t *q, float *x, const float *params, const int32_t *seg,
                                            const int32_t *pseg, int P, int64_t n_rows, int64_t n_packed_rows,
                                            int64_t F, int bits, sgnn_stream_t stream) {
    return unpack_dequant_rows_impl(q, x, params, 0, seg, pseg, P, n_rows, n_packed_rows, F, bits, stream);
}

extern "C" int sgnn_unpack_dequant_rows_wire_f32(const uint8_t *q, float *x, const void *params, int params_bf16,
                                                 const int32_t *seg, const int32_t *pseg, int P, int64_t n_rows,
                                                 int64_t n_packed_rows, int64_t F, int bits, sgnn_stream_t stream) {
    return unpack_dequant_rows_impl(q, x, params, params_bf16, seg, pseg, P, n_rows, n_packed_rows, F, bits, stream);
}

extern "C" int sgnn_quant_v1_f32(const float *x, uint8_t *q, const int64_t *range, float *params, int64_t n,
                                 int64_t F, sgnn_stream_t stream) {
    SGNN_REQUIRE(n >= 0 && F > 0 && F < (1 << 24), "size out of range");
    if (n == 0) return SGNN_OK;
    SGNN_REQUIRE(x && q && range && params, "null pointer argument");
    const int64_t nb = (n + kQBlock / 64 - 1) / (kQBlock / 64);
    SGNN_REQUIRE(nb < INT32_MAX, "too many rows");
    ProfScope prof(K_QUANT_V1, (hipStream_t)stream);
    const dim3 grid((uint32_t)nb), block(kQBlock);
    const auto grid_r = [&](int rows) { return dim3((uint32_t)((nb + rows - 1) / rows)); };
    hipStream_t st = (hipStream_t)stream;
    if (F % 4 == 0 && F <= 512 && aligned(x, 16)) {   // (wider rows: a wavefront per row is faster)
        const auto grid_g = [&](int rows_per_wave) {
            const int64_t waves = (n + rows_per_wave - 1) / rows_per_wave;
            return dim3((uint32_t)((waves + kQBlock / 64 - 1) / (kQBlock / 64)));
        };
#define SGNN_V1G(NV, R, L) hipLaunchKernelGGL((quant_v1_group_kernel<NV, R, L>), grid_g((64 / L) * R), block, 0, st, x, q, range, params, n, (int)F)
        if (F <= 32) SGNN_V1G(1, 4, 8);
        else if (F <= 64) SGNN_V1G(2, 2, 8);
        else if (F <= 128) SGNN_V1G(4, 1, 8);
        else if (F <= 256) SGNN_V1G(4, 1, 16);
        else SGNN_V1G(8, 1, 16);
#undef SGNN_V1G
    } else if (F % 4 == 0 && F <= 1024 && aligned(x, 16)) {
        if (F <= 256) hipLaunchKernelGGL((quant_v1_vec_kernel<1, 4>), grid_r(4), block, 0, st, x, q, range, params, n, (int)F);
        else if (F <= 512) hipLaunchKernelGGL((quant_v1_vec_kernel<2, 2>), grid_r(2), block, 0, st, x, q, range, params, n, (int)F);
        else hipLaunchKernelGGL((quant_v1_vec_kernel<4, 1>), grid, block, 0, st, x, q, range, params, n, (int)F);
    } else {
        hipLaunchKernelGGL(quant_v1_kernel, grid, block, 0, st, x, q, range, params, n, (int)F);
    }
    SGNN_HIP_CHECK(hipGetLastError());
    return SGNN_OK;
}

extern "C" int sgnn_dequant_v1_f32(const uint8_t *q, float *x, const int64_t *range, const float *params, int64_t n,
                                   int64_t F, sgnn_stream_t stream) {
    SGNN_REQUIRE(n >= 0 && F > 0 && F < (1 << 24), "size out of range");
    if (n == 0) return SGNN_OK;
    SGNN_REQUIRE(x && q && range && params, "null pointer argument");
    const int64_t nb = (n + kQBlock / 64 - 1) / (kQBlock / 64);
    SGNN_REQUIRE(nb < INT32_MAX, "too many rows");
    ProfScope prof(K_DEQUANT_V1, (hipStream_t)stream);
    const dim3 grid((uint32_t)nb), block(kQBlock);
    const auto grid_r = [&](int rows) { return dim3((uint32_t)((nb + rows - 1) / rows)); };
    hipStream_t st = (hipStream_t)stream;
    // narrow rows (a wavefront per row leaves lanes idle) and rows beyond the vector kernel's width: flat output,
    // four stores per wavefront (measured 1-3 % above two and 10-15 % above one)
    if (F % 4 == 0 && aligned(x, 16) && (F <= 128 || F > 1024)) {
        const int64_t n_vec = n * (F / 4);
        const dim3 waves((uint32_t)(((n_vec + 4 * 64 - 1) / (4 * 64) + kQBlock / 64 - 1) / (kQBlock / 64)));
        hipLaunchKernelGGL((dequant_v1_flat_kernel<4>), waves, block, 0, st, q, x, range, params, n_vec, (int)(F / 4));
    } else if (F % 4 == 0 && F <= 1024 && aligned(x, 16)) {
        if (F <= 256) hipLaunchKernelGGL((dequant_v1_vec_kernel<1, 4>), grid_r(4), block, 0, st, q, x, range, params, n, (int)F);
        else if (F <= 512) hipLaunchKernelGGL((dequant_v1_vec_kernel<2, 2>), grid_r(2), block, 0, st, q, x, range, params, n, (int)F);
        else hipLaunchKernelGGL((dequant_v1_vec_kernel<4, 1>), grid, block, 0, st, q, x, range, params, n, (int)F);
    } else {
        hipLaunchKernelGGL(dequant_v1_kernel, grid, block, 0, st, q, x, range, params, n, (int)F);
    }
    SGNN_HIP_CHECK(hipGetLastError());
    return SGNN_OK;
}
