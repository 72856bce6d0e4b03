// Offline path on the device: per-group asymmetric 4-bit min/max quantisation of an fp32 weight
// [N, K] fused with the AWQ packing, producing qweight [K, N/8], qzeros [K/g, N/8] and qscales
// [K/g, N] directly.  The arithmetic is the reference's, operation by operation in fp32 (true
// divisions, round-half-to-even), so the words equal those of its quantise -> transpose -> pack chain.
#include "awq_common.hpp"

namespace awq {
namespace {

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// One wave per (word column i, group kg): 8 output columns n = 8i..8i+7, g input rows k.
// Weight rows are read 64 consecutive floats at a time (coalesced); a lane ends up with the 8
// nibbles of one packed word per k it owns.
template <typename T>
__global__ __launch_bounds__(256) void quantize_pack_kernel(const float* __restrict__ w,
                                                            uint32_t* __restrict__ qweight,
                                                            uint32_t* __restrict__ qzeros,
                                                            uint16_t* __restrict__ qscales, int N, int K, int g) {
    const int lane = threadIdx.x & 63;
    const int words = N >> 3, groups = K / g;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (int64_t)words * groups) return;
    const int i = (int)(item % words), kg = (int)(item / words);
    const float* base = w + (size_t)(8 * i) * K + (size_t)kg * g;

    float s[8], z[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        float lo = INFINITY, hi = -INFINITY;
        for (int kk = lane; kk < g; kk += 64) {
            const float v = base[(size_t)c * K + kk];
            lo = fminf(lo, v);
            hi = fmaxf(hi, v);
        }
        lo = wave_min(lo);
        hi = wave_max(hi);
        s[c] = __fdiv_rn(fmaxf(__fsub_rn(hi, lo), 1e-5f), 15.f);
        z[c] = fminf(fmaxf(-rintf(__fdiv_rn(lo, s[c])), 0.f), 15.f);
    }
    for (int kk = lane; kk < g; kk += 64) {
        uint32_t word = 0;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float v = base[(size_t)c * K + kk];
            const float q = fminf(fmaxf(__fadd_rn(rintf(__fdiv_rn(v, s[c])), z[c]), 0.f), 15.f);
            const float dq = __fmul_rn(__fsub_rn(q, z[c]), s[c]);                 // the fake-quantised weight
            const int iw = (int)rintf(__fadd_rn(__fdiv_rn(dq, s[c]), z[c]));      // re-quantised by the packer
            word |= ((uint32_t)iw & 15u) << nibble_shift(c);
        }
        qweight[(size_t)(kg * g + kk) * words + i] = word;
    }
    if (lane == 0) {
        uint32_t zw = 0;
#pragma unroll
        for (int c = 0; c < 8; ++c) zw |= ((uint32_t)(int)z[c] & 15u) << nibble_shift(c);
        qzeros[(size_t)kg * words + i] = zw;
    }
    if (lane < 8) {
        float sv = s[0];
#pragma unroll
        for (int c = 1; c < 8; ++c) sv = lane == c ? s[c] : sv;
        qscales[(size_t)kg * N + 8 * i + lane] = T::from_f32(sv);
    }
}

}  // namespace
}  // namespace awq

using namespace awq;

extern "C" int awq_quantize_pack(const float* weight, int32_t* qweight, void* qscales, int32_t* qzeros, int64_t N,
                                 int64_t K, int64_t group_size, int dtype, void* stream) {
    const char* fn = "awq_quantize_pack";
    if (!weight || !qweight || !qscales || !qzeros) {
        set_error("%s: null pointer argument", fn);
        return AWQ_ERR_INVALID_ARG;
    }
    if (dtype != AWQ_F16 && dtype != AWQ_BF16) {
        set_error("%s: dtype must be AWQ_F16 (0) or AWQ_BF16 (1), got %d", fn, dtype);
        return AWQ_ERR_INVALID_ARG;
    }
    if (N <= 0 || K <= 0 || group_size <= 0 || N % 8 != 0 || K % group_size != 0) {
        set_error("%s: need N %% 8 == 0 and K %% group_size == 0 (N=%lld K=%lld g=%lld)", fn, (long long)N,
                  (long long)K, (long long)group_size);
        return AWQ_ERR_INVALID_ARG;
    }
    const int64_t items = (N / 8) * (K / group_size);
    if (N > 0x7fffffff || K > 0x7fffffff || cdiv(items, 4) > 0x7fffffff) {
        set_error("%s: problem too large", fn);
        return AWQ_ERR_UNSUPPORTED;
    }
    hipStream_t st = (hipStream_t)stream;
    (void)hipGetLastError();
    const dim3 grid((unsigned)cdiv(items, 4)), block(256);
    if (dtype == AWQ_F16)
        quantize_pack_kernel<F16><<<grid, block, 0, st>>>(weight, (uint32_t*)qweight, (uint32_t*)qzeros,
                                                          (uint16_t*)qscales, (int)N, (int)K, (int)group_size);
    else
        quantize_pack_kernel<BF16><<<grid, block, 0, st>>>(weight, (uint32_t*)qweight, (uint32_t*)qzeros,
                                                           (uint16_t*)qscales, (int)N, (int)K, (int)group_size);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}
