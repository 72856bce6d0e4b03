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

// Reinterpret one 32-bit register as a pair of halves.  Takes the word BY VALUE:
// __builtin_bit_cast applied directly to a vector element (v[i]) reads element 0.
__device__ __forceinline__ f16x2 as_f16x2(uint32_t w) { return __builtin_bit_cast(f16x2, w); }
__device__ __forceinline__ uint32_t as_u32(f16x2 h) { return __builtin_bit_cast(uint32_t, h); }

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

// ---- split-K exchange between workgroups ----------------------------------
// Partials cross workgroups (and XCDs, each with its own L2) as agent-scope
// relaxed atomic stores/loads: they are written through to, and read from, the
// agent's point of coherence, so no cache write-back or invalidate -- which
// costs every wave of the grid a serialised L2 operation -- is needed.
__device__ __forceinline__ void publish_f32(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16-byte form of publish_f32.  The store is invisible to the compiler's wait-count
// bookkeeping, which is why arrive_last waits for vmcnt = 0 explicitly.  It is invisible to the compiler's
// hazard pass as well: a store of more than 8 bytes reads its data registers up to two wait states after it
// issues (gfx940 and later), and to the compiler those registers are free the moment the statement ends -- it
// has put the next address computation into them one instruction later, and the store then wrote that value
// now and then.  Hence the two wait states inside the statement.
__device__ __forceinline__ void publish_f32x4(float* p, f32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ float fetch_f32(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16-byte form of fetch_f32 that does not wait: the load is invisible to the compiler's wait-count
// bookkeeping, so the values may only be used after fetch_wait() has been given every one of them.
__device__ __forceinline__ f32x4 fetch_f32x4_nowait(const float* p) {
    f32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void fetch_wait(f32x4 (&a)[8], f32x4 (&b)[8]) {
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]),
                   "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7])
                 :
                 : "memory");
}
// All of this workgroup's publish_f32 stores have been acknowledged (vmcnt = 0
// in every wave, then the barrier) before one thread bumps the tile's arrival
// counter; returns true in the workgroup that arrived last.
__device__ __forceinline__ bool arrive_last(int* counter, int splits, int* s_flag) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): also covers the inline-asm stores of publish_f32x4
    __syncthreads();
    if (threadIdx.x == 0) {
        const int prev = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_flag = (prev == splits - 1);
    }
    __syncthreads();
    return *s_flag != 0;
}

// T(a * b) for a genuine fp32 factor: the product is rounded to fp32, then to T, as torch's `x.float() * r`
// followed by `.to(dtype)` does.  Without the barrier the compiler may pick the mixed-precision FMA for fp16, which
// rounds once, and two kernels that should agree bit for bit would depend on its choice.
template <typename T>
__device__ __forceinline__ float mul_round(float a, float b) {
    float p = a * b;
    asm("" : "+v"(p));
    return T::to_f32(T::from_f32(p));
}
// acc + bias with the reference's two rounding points: the product is rounded to T first, then `out.add_(bias)`
// adds in fp32 and rounds again (nanoquantization/layers/gemm.py:561-566).  The caller rounds the returned sum to T.
template <typename T>
__device__ __forceinline__ float add_bias(float acc, float b) {
    return T::to_f32(T::from_f32(acc)) + b;
}
// The same barrier for any fp32 value about to be rounded to T: the value is an fp32 result first.
__device__ __forceinline__ float as_f32_result(float v) {
    asm("" : "+v"(v));
    return v;
}

// Sum of squares of one 128-column tile of a row, 8 consecutive values per lane, 16 lanes (an aligned group) per
// tile: the lane's 8 squares in column order by fused multiply-add, then the lanes by xor 8, 4, 2, 1.  Every
// kernel that produces or consumes RMSNorm statistics uses this order, so their results agree bit for bit.
__device__ __forceinline__ float tile_ssq(const float (&v)[8]) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = __builtin_fmaf(v[e], v[e], ss);
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) ss += __shfl_xor(ss, o);
    return ss;
}

// ---- host-side error plumbing -------------------------------------------
void set_error(const char* fmt, ...);
int check_linear_args(const char* fn, const void* x, const int32_t* qweight, const void* qscales,
                      const int32_t* qzeros, const void* y, int64_t M, int64_t N, int64_t K,
                      int64_t g, int dtype);
int hip_fail(const char* fn, hipError_t e);

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Prefetch hints of the calling thread (awq_prefetch_hint): taken, and cleared, by the next GEMV launch.
constexpr int kMaxPrefetchRegions = 4;
struct PrefetchRegions {
    const char* ptr[kMaxPrefetchRegions];
    long long bytes[kMaxPrefetchRegions];
    int count;
};
void take_prefetch_hint(PrefetchRegions* out);

// Split-K bookkeeping shared by the GEMV and GEMM kernels.  The workspace is
//   [ kMaxSplitTiles int32 arrival counters | fp32 partials [splits][M][N] ]
// The counter region has the same size for every problem, so partials of one
// call never land on counters of the next.  Counters start at zero and the last
// workgroup to arrive at a tile resets its counter: the buffer is reusable
// without a memset between calls.
constexpr int64_t kMaxSplitTiles = 4096;
constexpr size_t kCounterBytes = (size_t)kMaxSplitTiles * sizeof(int);

}  // namespace awq
