// Shared device/host helpers for the gfx950 AWQ W4A16 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/awq_hip.h"

namespace awq {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

// Bit position of logical column c inside a packed word: the packer stores
// column {0,2,4,6,1,3,5,7}[j] in nibble j, so column c sits at nibble
// 4*(c&1) + (c>>1).
__host__ __device__ constexpr int nibble_shift(int c) { return 4 * (4 * (c & 1) + (c >> 1)); }

struct F16 {
    using vec8 = f16x8;
    static constexpr int id = AWQ_F16;
    static constexpr uint32_t ones2 = 0x3C003C00u;  // (1.0, 1.0)
    static __device__ __forceinline__ float to_f32(uint16_t b) {
        return (float)__builtin_bit_cast(_Float16, b);
    }
    static __device__ __forceinline__ uint16_t from_f32(float f) {
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f16x2 v;
        v.x = (_Float16)lo;
        v.y = (_Float16)hi;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

struct BF16 {
    using vec8 = bf16x8;
    static constexpr int id = AWQ_BF16;
    static constexpr uint32_t ones2 = 0x3F803F80u;
    static __device__ __forceinline__ float to_f32(uint16_t b) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    }
    static __device__ __forceinline__ uint16_t from_f32(float f) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        bf16x2 v;
        v.x = (__bf16)lo;
        v.y = (__bf16)hi;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};

// ---- host-side error plumbing -------------------------------------------
void set_error(const char* fmt, ...);
int check_linear_args(const char* fn, const void* x, const int32_t* qweight, const void* qscales,
                      const int32_t* qzeros, const void* y, int64_t M, int64_t N, int64_t K,
                      int64_t g, int dtype);
int hip_fail(const char* fn, hipError_t e);

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Split-K bookkeeping shared by the GEMV and GEMM kernels.  The workspace is
//   [ int32 counters, one per output tile, padded to 256 B | fp32 partials ]
// Counters start at zero and the last workgroup to arrive at a tile resets its
// counter, so the buffer is reusable without a memset between calls.
static inline size_t counter_bytes(int64_t tiles) { return (size_t)cdiv(tiles * 4, 256) * 256; }

}  // namespace awq
