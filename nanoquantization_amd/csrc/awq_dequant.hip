// Kernel (a): standalone int4 unpack + dequantise, bit-exact with
// RN_dtype(float(q - z) * s).
//
// HBM-bound (reads 0.52 B, writes 2 B per weight).  One lane owns one packed
// word column (8 outputs) and walks ROWS rows of one quantisation group, so the
// zero word and the 8 scales are fetched once per ROWS rows; a wavefront writes
// 64 x 16 B = 1 KiB contiguous per row.
#include "awq_common.hpp"

namespace awq {

template <typename T>
struct DequantWord;

// fp16: (w >> 4i) & 0x000F000F holds columns (2i, 2i+1) in the two halves;
// OR-ing 0x6400 makes each half the fp16 number 1024 + q exactly.  The
// difference of two such numbers is exact and the product with the scale pair
// is rounded once -- the same value the reference's int->fp16 promotion gives.
template <>
struct DequantWord<F16> {
    uint32_t zp[4];
    f16x2 sc[4];
    __device__ __forceinline__ void set_group(uint32_t zw, u32x4 sv) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            zp[i] = ((zw >> (4 * i)) & 0x000F000Fu) | 0x64006400u;
            sc[i] = as_f16x2(sv[i]);
        }
    }
    __device__ __forceinline__ u32x4 apply(uint32_t w) const {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t qp = ((w >> (4 * i)) & 0x000F000Fu) | 0x64006400u;
            f16x2 d = as_f16x2(qp) - as_f16x2(zp[i]);
            o[i] = as_u32(d * sc[i]);
        }
        return o;
    }
};

// bf16: the integer difference converts exactly to fp32, the fp32 product with
// the (8-bit significand) scale is exact, and one round-to-nearest-even makes
// the bf16 result.
template <>
struct DequantWord<BF16> {
    int z[8];
    float sc[8];
    __device__ __forceinline__ void set_group(uint32_t zw, u32x4 sv) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            z[c] = (int)((zw >> nibble_shift(c)) & 0xFu);
            uint32_t pair = sv[c >> 1];
            sc[c] = __builtin_bit_cast(float, (c & 1) ? (pair & 0xFFFF0000u) : (pair << 16));
        }
    }
    __device__ __forceinline__ u32x4 apply(uint32_t w) const {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int q0 = (int)((w >> nibble_shift(2 * i)) & 0xFu);
            int q1 = (int)((w >> nibble_shift(2 * i + 1)) & 0xFu);
            float a = (float)(q0 - z[2 * i]) * sc[2 * i];
            float b = (float)(q1 - z[2 * i + 1]) * sc[2 * i + 1];
            o[i] = BF16::pack2(a, b);
        }
        return o;
    }
};

template <typename T, int ROWS>
__global__ __launch_bounds__(256) void dequant_kernel(const uint32_t* __restrict__ qweight,
                                                      const uint16_t* __restrict__ scales,
                                                      const uint32_t* __restrict__ qzeros,
                                                      uint16_t* __restrict__ out, int words, int g) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= words) return;
    const int k0 = blockIdx.y * ROWS;
    // host guarantees g % ROWS == 0 (all ROWS rows share a group) and hence K % ROWS == 0
    const int gi = k0 / g;
    const size_t N = (size_t)words * 8;
    DequantWord<T> dq;
    dq.set_group(qzeros[(size_t)gi * words + c],
                 *reinterpret_cast<const u32x4*>(scales + (size_t)gi * N + (size_t)c * 8));
    uint32_t w[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) w[r] = qweight[(size_t)(k0 + r) * words + c];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
        *reinterpret_cast<u32x4*>(out + (size_t)(k0 + r) * N + (size_t)c * 8) = dq.apply(w[r]);
}

template <typename T>
static int launch_dequant(const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                          void* out, int64_t K, int64_t N, int64_t g, hipStream_t stream) {
    const int words = (int)(N / 8);
    dim3 block(256);
    auto qw = reinterpret_cast<const uint32_t*>(qweight);
    auto qz = reinterpret_cast<const uint32_t*>(qzeros);
    auto sc = reinterpret_cast<const uint16_t*>(qscales);
    auto o = reinterpret_cast<uint16_t*>(out);
    if (g % 16 == 0) {
        dim3 grid((unsigned)cdiv(words, 256), (unsigned)cdiv(K, 16));
        hipLaunchKernelGGL((dequant_kernel<T, 16>), grid, block, 0, stream, qw, sc, qz, o, words, (int)g);
    } else {
        dim3 grid((unsigned)cdiv(words, 256), (unsigned)K);
        hipLaunchKernelGGL((dequant_kernel<T, 1>), grid, block, 0, stream, qw, sc, qz, o, words, (int)g);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail("awq_dequantize", e);
}

}  // namespace awq

extern "C" int awq_dequantize(const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                              void* out, int64_t K, int64_t N, int64_t group_size, int dtype,
                              void* stream) {
    using namespace awq;
    // x is not an argument here: pass `out` twice to reuse the shared checks (M = 1).
    int rc = check_linear_args("awq_dequantize", out, qweight, qscales, qzeros, out, 1, N, K,
                               group_size, dtype);
    if (rc != AWQ_OK) return rc;
    if (K > 65535 * 16 && group_size % 16 == 0) {
        set_error("awq_dequantize: K=%lld exceeds the launch grid", (long long)K);
        return AWQ_ERR_UNSUPPORTED;
    }
    if (group_size % 16 != 0 && K > 65535) {
        set_error("awq_dequantize: K=%lld exceeds the launch grid for group_size %lld",
                  (long long)K, (long long)group_size);
        return AWQ_ERR_UNSUPPORTED;
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    return dtype == AWQ_F16
               ? launch_dequant<F16>(qweight, qscales, qzeros, out, K, N, group_size, s)
               : launch_dequant<BF16>(qweight, qscales, qzeros, out, K, N, group_size, s);
}
