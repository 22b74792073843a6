// Error reporting, the HIP-event profiler behind bench.py, the streaming-copy yardstick and the ABI version.
#include <algorithm>
#include <atomic>
#include <mutex>
#include <vector>

#include "common.hpp"

namespace sgnn {

std::string &last_error() {
    static thread_local std::string msg;
    return msg;
}

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

// ---- HIP-event profiler ------------------------------------------------------------------------
struct ProfRecord {
    int id;
    hipEvent_t start, stop;
};
static std::mutex g_prof_mu;
static std::atomic<bool> g_prof_on{false};
static std::vector<ProfRecord> g_prof;

ProfScope::ProfScope(int id, hipStream_t st, bool enabled) : id_(id), st_(st) {
    if (!enabled || !g_prof_on) return;
    if (hipEventCreate(&start_) != hipSuccess) { start_ = nullptr; return; }
    (void)hipEventRecord(start_, st_);
}

ProfScope::~ProfScope() {
    if (!start_) return;
    hipEvent_t stop = nullptr;
    if (hipEventCreate(&stop) != hipSuccess) { (void)hipEventDestroy(start_); return; }
    (void)hipEventRecord(stop, st_);
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof.push_back({id_, start_, stop});
}

static const char *kKernelNames[K_COUNT] = {
    "spmm_short_kernel",  "spmm_piece_kernel", "spmm_long_final_kernel", "quant_pack_rows_kernel",
    "unpack_dequant_rows_kernel", "quant_v1_kernel", "dequant_v1_kernel", "stream_copy_kernel",
    "spmm_short_kernel(dq)", "spmm_piece_kernel(dq)", "spmm_empty_rows_kernel", "spmm_band_kernel", "band_restage_kernel"};

// ---- plain streaming copy: the attainable-bandwidth yardstick and the counter calibration -----
__global__ __launch_bounds__(256) void stream_copy_kernel(const float4 *__restrict__ src, float4 *__restrict__ dst,
                                                          int64_t n4) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    // one float4 per lane and no loop: on MI355X the shortest waves stream fastest (6.5 TB/s against
    // 5.4 TB/s for a grid-stride loop over the same gigabyte)
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) {
        const f4 v = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(src) + i);
        __builtin_nontemporal_store(v, reinterpret_cast<f4 *>(dst) + i);
    }
}

}  // namespace sgnn

using namespace sgnn;

extern "C" int sgnn_profile_enable(int on) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    if (on) {
        for (auto &r : g_prof) { (void)hipEventDestroy(r.start); (void)hipEventDestroy(r.stop); }
        g_prof.clear();
    }
    g_prof_on = on != 0;
    return SGNN_OK;
}

extern "C" int sgnn_profile_read(int kernel_id, int64_t *launches, double *total_ms) {
    SGNN_REQUIRE(kernel_id >= 0 && kernel_id < K_COUNT && launches && total_ms, "bad profile query");
    std::lock_guard<std::mutex> lk(g_prof_mu);
    *launches = 0;
    *total_ms = 0.0;
    for (auto &r : g_prof) {
        if (r.id != kernel_id) continue;
        SGNN_HIP_CHECK(hipEventSynchronize(r.stop));
        float ms = 0.0f;
        SGNN_HIP_CHECK(hipEventElapsedTime(&ms, r.start, r.stop));
        *launches += 1;
        *total_ms += ms;
    }
    return SGNN_OK;
}

extern "C" const char *sgnn_profile_kernel_name(int kernel_id) {
    return (kernel_id >= 0 && kernel_id < K_COUNT) ? kKernelNames[kernel_id] : "";
}

extern "C" int sgnn_profile_kernel_count(void) { return K_COUNT; }

extern "C" int sgnn_stream_copy_f32(const float *src, float *dst, int64_t n, sgnn_stream_t stream) {
    SGNN_REQUIRE(n >= 0 && n % 4 == 0, "n must be a non-negative multiple of 4");
    if (n == 0) return SGNN_OK;
    SGNN_REQUIRE(src && dst && aligned(src, 16) && aligned(dst, 16), "src/dst must be non-null and 16-byte aligned");
    const int64_t n4 = n / 4;
    SGNN_REQUIRE((n4 + 255) / 256 < INT32_MAX, "n too large for one launch");
    const int nb = (int)((n4 + 255) / 256);
    ProfScope prof(K_STREAM_COPY, (hipStream_t)stream);
    hipLaunchKernelGGL(stream_copy_kernel, dim3(nb), dim3(256), 0, (hipStream_t)stream, (const float4 *)src, (float4 *)dst, n4);
    SGNN_HIP_CHECK(hipGetLastError());
    return SGNN_OK;
}

extern "C" const char *sgnn_last_error(void) { return sgnn::last_error().c_str(); }

extern "C" int sgnn_version(void) { return 2; }
