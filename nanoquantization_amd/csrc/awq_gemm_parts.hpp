// Pieces shared by the fused dequant+GEMM kernels: the register unpack of packed words into
// k-pairs of dequantised values, and the epilogue: direct store (+ bias) of a workgroup's
// BM x BN tile, or fp32 partials of a K split that a second kernel adds in split order.
#pragma once

#include "awq_common.hpp"

namespace awq {

template <typename T>
struct UnpackRows;

// fp16: returns, for byte-pair i (columns 2i, 2i+1) of one word, the packed
// pair of dequantised halves.
template <>
struct UnpackRows<F16> {
    uint32_t zp[4];
    f16x2 sc[4];
    __device__ __forceinline__ void set_group(uint32_t zw, u32x4 sv) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            zp[i] = ((zw >> (4 * i)) & 0x000F000Fu) | 0x64006400u;
            sc[i] = as_f16x2(sv[i]);
        }
    }
    // out[c] = (W[k, c], W[k+1, c]) for the 8 columns of the word pair (w0 = row k, w1 = row k+1)
    __device__ __forceinline__ void pair(uint32_t w0, uint32_t w1, uint32_t out[8]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t q0 = ((w0 >> (4 * i)) & 0x000F000Fu) | 0x64006400u;
            uint32_t q1 = ((w1 >> (4 * i)) & 0x000F000Fu) | 0x64006400u;
            f16x2 d0 = (as_f16x2(q0) - as_f16x2(zp[i])) * sc[i];
            f16x2 d1 = (as_f16x2(q1) - as_f16x2(zp[i])) * sc[i];
            uint32_t u0 = as_u32(d0), u1 = as_u32(d1);
            // columns 2i (low halves) and 2i+1 (high halves), rows k / k+1
            out[2 * i] = __builtin_amdgcn_perm(u1, u0, 0x05040100u);
            out[2 * i + 1] = __builtin_amdgcn_perm(u1, u0, 0x07060302u);
        }
    }
};

template <>
struct UnpackRows<BF16> {
    float sc[8], nzs[8];  // s and -(z * s), both exact in fp32
    __device__ __forceinline__ void set_group(uint32_t zw, u32x4 sv) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint32_t pr = sv[c >> 1];
            sc[c] = __builtin_bit_cast(float, (c & 1) ? (pr & 0xFFFF0000u) : (pr << 16));
            nzs[c] = -(float)((zw >> nibble_shift(c)) & 0xFu) * sc[c];
        }
    }
    __device__ __forceinline__ void pair(uint32_t w0, uint32_t w1, uint32_t out[8]) const {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float q0 = (float)((w0 >> nibble_shift(c)) & 0xFu);
            const float q1 = (float)((w1 >> nibble_shift(c)) & 0xFu);
            // q*s - z*s: the exact value (q-z)*s has <= 13 significant bits, so the
            // fused multiply-add returns it exactly.
            out[c] = BF16::pack2(__builtin_fmaf(q0, sc[c], nzs[c]), __builtin_fmaf(q1, sc[c], nzs[c]));
        }
    }
};


// Gated epilogue: a lane pair holds a gate word and the up word of the same 8 outputs (already rounded to T); each
// lane of the pair produces four of them (the even lane outputs 0..3, the odd lane 4..7) and stores 8 bytes:
// dtype(SiLU(gate)) * up, the rounding points of F.silu(gate_proj(x)) * up_proj(x).  `mine` is this lane's word,
// `other` its partner's, `odd` says which of the two this lane holds.
template <typename T>
__device__ __forceinline__ void swiglu_pair_store(u32x4 mine, u32x4 other, bool odd, uint16_t* __restrict__ dst) {
    const u32x4 gate = odd ? other : mine, up = odd ? mine : other;
    uint32_t o[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t gw = odd ? gate[2 + i] : gate[i], uw = odd ? up[2 + i] : up[i];
        float r[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float g = T::to_f32((uint16_t)(h ? gw >> 16 : gw & 0xFFFFu));
            const float u = T::to_f32((uint16_t)(h ? uw >> 16 : uw & 0xFFFFu));
            r[h] = T::to_f32(T::from_f32(g / (1.f + __expf(-g)))) * u;
        }
        o[i] = T::pack2(r[0], r[1]);
    }
    *reinterpret_cast<u32x2*>(dst + (odd ? 4 : 0)) = u32x2{o[0], o[1]};
}

// acc[a][b][v] of the 32x32x16 MFMA: row (v/4)*8 + (lane/32)*4 + v%4, column lane%32 of tile
// (a, b) of the wave's sub-tile at (wm0, wn0).
template <typename T, int BM, int BN, int TM, int TN, int NT>
__device__ __forceinline__ void gemm_epilogue(f32x16 (&acc)[TM][TN], const uint16_t* __restrict__ bias,
                                              uint16_t* __restrict__ y, float* __restrict__ partials, int M,
                                              int N, int m0, int n0, int wm0, int wn0, int split, int splits) {
    const int lane = threadIdx.x & 63;
    const int li = lane & 31, kb2 = lane >> 5;
    const bool direct = splits == 1;
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int n = n0 + wn0 + b * 32 + li;
            if (n >= N) continue;
            const bool has_bias = direct && bias;
            const float bv = has_bias ? T::to_f32(bias[n]) : 0.f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm0 + a * 32 + (v >> 2) * 8 + kb2 * 4 + (v & 3);
                if (m >= M) continue;
                if (direct)
                    y[(size_t)m * N + n] = T::from_f32(has_bias ? add_bias<T>(acc[a][b][v], bv) : acc[a][b][v]);
                else
                    partials[((size_t)split * M + m) * N + n] = acc[a][b][v];   // 32 lanes = one 128-byte line
            }
        }
}

// Second pass of a split-K product: y = dtype(sum over splits, in split order, of the fp32
// partials [splits][M][N] (+ bias)).  A thread owns 8 consecutive columns of one row.
template <typename T>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ partials,
                                                                 const uint16_t* __restrict__ bias,
                                                                 uint16_t* __restrict__ y, int64_t M, int N,
                                                                 int splits) {
    const int64_t vec = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int per_row = N >> 3;
    if (vec >= M * per_row) return;
    const int64_t m = vec / per_row;
    const int nn = (int)(vec % per_row) * 8;
    const size_t plane = (size_t)M * N;
    const float* p = partials + (size_t)m * N + nn;
    f32x4 lo = f32x4{0.f, 0.f, 0.f, 0.f}, hi = lo;
    // four splits' loads in flight at a time, added in split order
    for (int s0 = 0; s0 < splits; s0 += 4) {
        f32x4 a[4], b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t off = (size_t)min(s0 + u, splits - 1) * plane;
            a[u] = *reinterpret_cast<const f32x4*>(p + off);
            b[u] = *reinterpret_cast<const f32x4*>(p + off + 4);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (s0 + u < splits) {
                lo += a[u];
                hi += b[u];
            }
    }
    float out[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (bias) {
        const u32x4 bvv = *reinterpret_cast<const u32x4*>(bias + nn);
#pragma unroll
        for (int c = 0; c < 8; ++c)
            out[c] = add_bias<T>(out[c], T::to_f32((uint16_t)((c & 1) ? (bvv[c >> 1] >> 16) : (bvv[c >> 1] & 0xFFFFu))));
    }
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = T::pack2(out[2 * i], out[2 * i + 1]);
    *reinterpret_cast<u32x4*>(y + (size_t)m * N + nn) = o;
}

// Launches the reduction pass on `stream` (after the product kernel that wrote `partials`).
inline hipError_t launch_splitk_reduce(int dtype, const float* partials, const void* bias, void* y, int64_t M, int N,
                                       int splits, hipStream_t stream) {
    const int64_t vecs = M * (N >> 3);
    const dim3 grid((unsigned)cdiv(vecs, 256)), block(256);
    if (dtype == AWQ_F16)
        gemm_splitk_reduce_kernel<F16><<<grid, block, 0, stream>>>(partials, reinterpret_cast<const uint16_t*>(bias),
                                                                   reinterpret_cast<uint16_t*>(y), M, N, splits);
    else
        gemm_splitk_reduce_kernel<BF16><<<grid, block, 0, stream>>>(partials, reinterpret_cast<const uint16_t*>(bias),
                                                                    reinterpret_cast<uint16_t*>(y), M, N, splits);
    return hipGetLastError();
}

// Work split of the 256 x 256 pipelined kernel: `full_tiles` output tiles are computed whole by one
// workgroup each; the `tail_tiles` after them (tile index = m-tile * tiles_n + n-tile) are cut into `splits`
// K slices of `iters_per_split` 64-row steps whose fp32 partials a second kernel adds.
struct PipePlan {
    int tiles_n, full_tiles, tail_tiles, splits, iters_per_split;
    int act;   // 1: gate|up word-interleaved along N, y [M, N/2] = dtype(SiLU(gate)) * up (no bias)
};

// tail_only = false: every tile is cut `split_k` ways (none if that leaves one slice).
// tail_only = true: only the tiles beyond the last full round of 256 workgroups are cut.
inline PipePlan make_pipe_plan(int64_t M, int64_t N, int64_t K, int split_k, bool tail_only) {
    PipePlan p;
    p.tiles_n = (int)cdiv(N, 256);
    const int tiles = (int)(cdiv(M, 256) * p.tiles_n);
    const int total_iters = (int)(K / 64);
    p.iters_per_split = (int)cdiv(total_iters, split_k);
    p.splits = (int)cdiv(total_iters, p.iters_per_split);
    p.tail_tiles = p.splits <= 1 ? 0 : (tail_only ? tiles % 256 : tiles);
    p.full_tiles = tiles - p.tail_tiles;
    if (p.tail_tiles == 0) p.splits = 1;
    p.act = 0;
    return p;
}

inline size_t pipe_ws_bytes(const PipePlan& p) {
    return p.tail_tiles == 0 ? 0 : kCounterBytes + ((size_t)p.splits * p.tail_tiles << 18);
}

// awq_gemm_pipe.hip: the 256 x 256 software-pipelined kernel (same arguments as the tiled launcher).
hipError_t launch_gemm_pipe(int dtype, const void* x, const int32_t* qweight, const void* qscales,
                            const int32_t* qzeros, const void* bias, void* y, int M, int N, int K, int g,
                            void* workspace, int split_k, bool tail_only, hipStream_t stream, int act = 0);

// awq_gemm_pipe.hip: the second pass over the tail tiles of a PipePlan (fp32 partials [slice][tail tile][256][256]
// added in slice order, + bias or the gated product), on `stream` after the kernel that wrote them.
hipError_t launch_pipe_tail_reduce(int dtype, const float* partials, const void* bias, void* y, int M, int N,
                                   const PipePlan& plan, hipStream_t stream);

// awq_gemm_regb.hip: the 256 x 256 kernel that builds its B operands in registers (same arguments; group sizes that are
// multiples of 64 only).
hipError_t launch_gemm_regb(int dtype, const void* x, const int32_t* qweight, const void* qscales,
                            const int32_t* qzeros, const void* bias, void* y, int M, int N, int K, int g,
                            void* workspace, int split_k, bool tail_only, hipStream_t stream, int act = 0);

// awq_gemm_pipe.hip: wt [N][K] = the dequantised weight, transposed (K % 64 == 0, group size a multiple of 64 or
// a divisor of 64 that is a multiple of 8).
hipError_t launch_dequant_transpose(int dtype, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                                    void* wt, int N, int K, int g, hipStream_t stream);

}  // namespace awq
