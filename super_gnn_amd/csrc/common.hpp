// Shared host/device helpers of libsgnn_hip (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <string>

#include "sgnn.h"

namespace sgnn {

constexpr int kWave = 64;
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
    K_COUNT
};

// Records a HIP event pair around the launches made while it is alive, on the launch stream,
// when profiling is enabled; free otherwise.
struct ProfScope {
    ProfScope(int id, hipStream_t st);
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

template <int VEC>
struct VecT;
template <>
struct VecT<1> {
    using type = float;
};
template <>
struct VecT<2> {
    using type = float2;
};
template <>
struct VecT<4> {
    using type = float4;
};

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
