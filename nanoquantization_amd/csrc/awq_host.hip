// Host-side plumbing shared by every entry point: error text, argument checks.
#include <stdarg.h>
#include <stdio.h>

#include "awq_common.hpp"

namespace awq {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(const char* fn, hipError_t e) {
    set_error("%s: HIP error %d (%s)", fn, (int)e, hipGetErrorString(e));
    return AWQ_ERR_HIP;
}

int check_linear_args(const char* fn, const void* x, const int32_t* qweight, const void* qscales,
                      const int32_t* qzeros, const void* y, int64_t M, int64_t N, int64_t K,
                      int64_t g, int dtype) {
    if (!x || !qweight || !qscales || !qzeros || !y) {
        set_error("%s: null pointer argument", fn);
        return AWQ_ERR_INVALID_ARG;
    }
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(qweight) |
         reinterpret_cast<uintptr_t>(qscales) | reinterpret_cast<uintptr_t>(qzeros) |
         reinterpret_cast<uintptr_t>(y)) & 15u) {
        set_error("%s: every tensor must be 16-byte aligned", fn);
        return AWQ_ERR_INVALID_ARG;
    }
    if (dtype != AWQ_F16 && dtype != AWQ_BF16) {
        set_error("%s: dtype must be AWQ_F16 (0) or AWQ_BF16 (1), got %d", fn, dtype);
        return AWQ_ERR_INVALID_ARG;
    }
    if (M <= 0 || N <= 0 || K <= 0 || g <= 0) {
        set_error("%s: M, N, K and group_size must be positive (M=%lld N=%lld K=%lld g=%lld)", fn,
                  (long long)M, (long long)N, (long long)K, (long long)g);
        return AWQ_ERR_INVALID_ARG;
    }
    if (N % 8 != 0) {
        set_error("%s: out_features N=%lld must be divisible by 8", fn, (long long)N);
        return AWQ_ERR_INVALID_ARG;
    }
    if (K % g != 0) {
        set_error("%s: in_features K=%lld must be divisible by group_size %lld", fn, (long long)K,
                  (long long)g);
        return AWQ_ERR_INVALID_ARG;
    }
    if (K * N >= ((int64_t)1 << 40) || M * (N > K ? N : K) >= ((int64_t)1 << 40)) {
        set_error("%s: problem too large", fn);
        return AWQ_ERR_UNSUPPORTED;
    }
    return AWQ_OK;
}

// up to kMaxPrefetchRegions pending regions per thread
static thread_local PrefetchRegions g_pf = {};

void take_prefetch_hint(PrefetchRegions* out) {
    *out = g_pf;
    g_pf.count = 0;
}

}  // namespace awq

extern "C" int awq_prefetch_hint(const void* ptr, size_t bytes) {
    if (!ptr) {
        awq::g_pf.count = 0;
        return AWQ_OK;
    }
    if ((reinterpret_cast<uintptr_t>(ptr) & 127u) != 0) {
        awq::set_error("awq_prefetch_hint: the region must start on a 128-byte boundary");
        return AWQ_ERR_INVALID_ARG;
    }
    if (awq::g_pf.count == awq::kMaxPrefetchRegions) return AWQ_OK;   // a hint is optional: further regions are ignored
    awq::g_pf.ptr[awq::g_pf.count] = static_cast<const char*>(ptr);
    awq::g_pf.bytes[awq::g_pf.count] = (long long)bytes;
    ++awq::g_pf.count;
    return AWQ_OK;
}

extern "C" int awq_prefetch_pending(void) { return awq::g_pf.count; }

extern "C" int awq_hip_version(void) { return 100; }

extern "C" const char* awq_hip_last_error(void) { return awq::g_err; }
