// Shared host/device helpers of libsgnn_hip (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <string>

#include "sgnn.h"

namespace sgnn {

constexpr int kNumXCD = 8;  // MI355X: 8 accelerator dies, each with its own L2

std::string &last_error();
int fail(int code, const char *fmt, ...);

#define SGNN_HIP_CHECK(expr)                                                                  \
    do {                                                                                      \
        hipError_t _e = (expr);                                                               \
        if (_e != hipSuccess)                                                                 \
            return ::sgnn::fail(SGNN_ERR_HIP, "%s failed: %s (%s:%d)", #expr,                 \
                                hipGetErrorString(_e), __FILE__, __LINE__);                   \
    } while (0)

#define SGNN_REQUIRE(cond, ...)                                                               \
    do {                                                                                      \
        if (!(cond)) return ::sgnn::fail(SGNN_ERR_ARG, __VA_ARGS__);                          \
    } while (0)

// Kernels the built-in HIP-event profiler can attribute time to (see sgnn_profile_* in sgnn.h).
enum KernelId {
    K_SPMM_SHORT = 0,
    K_SPMM_PIECE,
    K_SPMM_LONG_FINAL,
    K_QUANT_PACK_ROWS,
    K_UNPACK_DEQUANT_ROWS,
    K_QUANT_V1,
    K_DEQUANT_V1,
    K_STREAM_COPY,
    K_FUSED_SHORT,
    K_FUSED_PIECE,
    K_SPMM_EMPTY_ROWS,
    K_SPMM_BAND,
    K_SPMM_BAND_RESTAGE,
    K_COUNT
};

// Records a HIP event pair around the launches made while it is alive, on the launch stream,
// when profiling is enabled; free otherwise.
struct ProfScope {
    // enabled = false: never records (callers that must not create events, e.g. under graph capture)
    ProfScope(int id, hipStream_t st, bool enabled = true);
    ~ProfScope();
    int id_;
    hipStream_t st_;
    hipEvent_t start_ = nullptr;
};

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Workgroups are dealt round-robin to the XCDs (workgroup i runs on XCD i % 8).  This maps the
// hardware workgroup id to a logical one such that each XCD works on one contiguous range of
// logical ids, so rows that are neighbours in memory share one L2.
__device__ __forceinline__ uint32_t xcd_contiguous_block(uint32_t bid, uint32_t nblocks) {
    const uint32_t per = nblocks / kNumXCD, rem = nblocks % kNumXCD;
    const uint32_t xcd = bid % kNumXCD, idx = bid / kNumXCD;
    return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

// The first active lane's 64-bit value, as a wave-uniform (scalar) value.
__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

template <int VEC>
__device__ __forceinline__ void vec_load(float (&r)[VEC], const float *p) {
    if constexpr (VEC == 4) {
        const float4 v = *reinterpret_cast<const float4 *>(p);
        r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
    } else if constexpr (VEC == 2) {
        const float2 v = *reinterpret_cast<const float2 *>(p);
        r[0] = v.x; r[1] = v.y;
    } else {
        r[0] = *p;
    }
}

// ------------------------------------------------------------------------------------------------
// Operands of the quantize / dequantize kernels as they sit either side of the boundary exchange.
// ------------------------------------------------------------------------------------------------

// fp32 rows to quantize: row r is x[(index ? index[r] : r) * ld ...].  With an index the kernel
// gathers the boundary rows straight out of the feature matrix (the reference first copies them into
// send_buf, super_gnn/aggregator.py:48).  An index outside [0, n_src) reads row 0 instead of faulting.
struct RowSrc {
    const float *x;
    int64_t ld;
    const int64_t *index;
    int64_t n_src;
};
__device__ __forceinline__ const float *row_ptr(const RowSrc &s, int64_t r) {
    if (s.index) {
        r = s.index[r];
        if ((uint64_t)r >= (uint64_t)s.n_src) r = 0;
    }
    return s.x + r * s.ld;
}

// (zero_point, scale) per row, either fp32[n,2] or -- the form the reference puts on the wire,
// super_gnn/communicator.py:283-294 -- bf16[n,2].  Codes are always computed from the fp32 values;
// the bf16 form only changes what is stored and what the receiver multiplies by.
struct ParamBuf {
    void *p;
    int bf16;
};
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {  // round to nearest even, NaN -> quiet NaN
    const uint32_t u = __float_as_uint(f);
    if (f != f) return 0x7fc0u | ((u >> 16) & 0x8000u);
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ void store_params(const ParamBuf &b, int64_t row, float zp, float sc) {
    if (b.bf16) reinterpret_cast<uint32_t *>(b.p)[row] = f32_to_bf16_bits(zp) | (f32_to_bf16_bits(sc) << 16);
    else reinterpret_cast<float2 *>(b.p)[row] = make_float2(zp, sc);
}
template <bool BF16>
__device__ __forceinline__ float2 load_params_as(const void *p, int64_t row) {
    if constexpr (BF16) {
        const uint32_t w = reinterpret_cast<const uint32_t *>(p)[row];
        return make_float2(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u));
    } else {
        return reinterpret_cast<const float2 *>(p)[row];
    }
}
__device__ __forceinline__ float2 load_params(const ParamBuf &b, int64_t row) {
    return b.bf16 ? load_params_as<true>(b.p, row) : load_params_as<false>(b.p, row);
}

template <int VEC>
__device__ __forceinline__ void vec_load_nt(float (&r)[VEC], const float *p) {
    if constexpr (VEC == 4) {
        typedef float f4 __attribute__((ext_vector_type(4)));
        const f4 v = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(p));
        r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
    } else if constexpr (VEC == 2) {
        typedef float f2 __attribute__((ext_vector_type(2)));
        const f2 v = __builtin_nontemporal_load(reinterpret_cast<const f2 *>(p));
        r[0] = v.x; r[1] = v.y;
    } else {
        r[0] = __builtin_nontemporal_load(p);
    }
}

// A 16-byte non-temporal load from an address that is only 4-byte aligned (rows whose width is not a
// multiple of four floats).  Global memory on gfx950 serves such a vector access in one instruction.
__device__ __forceinline__ void vec4_load_nt_unaligned(float (&r)[4], const float *p) {
    typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
    const f4u v = __builtin_nontemporal_load(reinterpret_cast<const f4u *>(p));
    r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
}
// A 4-byte non-temporal store to an address of any alignment.
__device__ __forceinline__ void u32_store_nt_unaligned(uint8_t *p, uint32_t w) {
    typedef uint32_t u32u __attribute__((aligned(1)));
    __builtin_nontemporal_store(w, reinterpret_cast<u32u *>(p));
}

template <int VEC>
__device__ __forceinline__ void vec_store_nt(float *p, const float (&r)[VEC]) {
    if constexpr (VEC == 4) {
        typedef float f4 __attribute__((ext_vector_type(4)));
        f4 v = {r[0], r[1], r[2], r[3]};
        __builtin_nontemporal_store(v, reinterpret_cast<f4 *>(p));
    } else if constexpr (VEC == 2) {
        typedef float f2 __attribute__((ext_vector_type(2)));
        f2 v = {r[0], r[1]};
        __builtin_nontemporal_store(v, reinterpret_cast<f2 *>(p));
    } else {
        __builtin_nontemporal_store(r[0], p);
    }
}

template <int VEC>
__device__ __forceinline__ void vec_store(float *p, const float (&r)[VEC]) {
    if constexpr (VEC == 4) {
        *reinterpret_cast<float4 *>(p) = make_float4(r[0], r[1], r[2], r[3]);
    } else if constexpr (VEC == 2) {
        *reinterpret_cast<float2 *>(p) = make_float2(r[0], r[1]);
    } else {
        *p = r[0];
    }
}

}  // namespace sgnn
