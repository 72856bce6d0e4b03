// Kernel (b): decode-regime AWQ GEMV, 1 <= M <= 16, split-K.
//
// HBM-bound: the job is to stream 0.52 B per weight and keep everything else
// off the critical path.  The contraction runs on the 16x16x32 MFMA (A = the
// <=16 activation rows, B = 16 output columns x 32 k), because even M = 2
// would saturate the vector ALUs at HBM speed.
//
// Data movement.  A lane is (j = lane % 16, kb = lane / 16).  Per 32-row step
// it loads V packed words from each of rows k0 + 8*kb + 0..7, word columns
// (tile*16 + j)*V .. +V-1: 16 lanes x 4V bytes are contiguous per row.  Those
// 8 rows x V words are 8V columns x 8 consecutive k: exactly the 8 k-slots the
// MFMA B operand wants per lane, once the nibbles of two rows are paired.
//
// In-register transposition.  v_perm_b32 puts byte b of row k into the low
// half and byte b of row k+1 into the high half of one register; a shift and
// one v_and_or_b32 then turn the two low (or high) nibbles into a packed pair
// of 16-bit floats with value 16 + q (the nibble sits in the top mantissa bits
// under the exponent of 16.0) -- no int->float conversion, no LDS.
//
// Scale and zero point are applied per quantisation group, in fp32, on the
// accumulator instead of per weight:
//   y += s[g,n] * ( sum_k x[k]*(16+q[k,n])  -  (16+z[g,n]) * sum_k x[k] )
// where sum_k x[k] comes from one extra MFMA per step against a B operand of
// ones.  The products 16+q are exact, so this differs from the reference's
// "round W to 16 bits, then multiply" only by not rounding W.
//
// Reduction.  Waves of a workgroup own consecutive K sub-slices and are summed
// through LDS in a fixed order; workgroups of different K-splits write fp32
// partials to the workspace and the last one to arrive (an agent-scope counter)
// adds them in split order, so results are bit-stable run to run.
#include "awq_common.hpp"

namespace awq {

template <typename T>
struct Embed;
template <>
struct Embed<F16> {  // 16.0 = 0x4C00, 10 mantissa bits: q << 6
    static constexpr uint32_t mask = 0x03C003C0u, magic = 0x4C004C00u;
    static __device__ __forceinline__ uint32_t lo(uint32_t p) { return ((p << 6) & mask) | magic; }
    static __device__ __forceinline__ uint32_t hi(uint32_t p) { return ((p << 2) & mask) | magic; }
};
template <>
struct Embed<BF16> {  // 16.0 = 0x4180, 7 mantissa bits: q << 3
    static constexpr uint32_t mask = 0x00780078u, magic = 0x41804180u;
    static __device__ __forceinline__ uint32_t lo(uint32_t p) { return ((p << 3) & mask) | magic; }
    static __device__ __forceinline__ uint32_t hi(uint32_t p) { return ((p >> 1) & mask) | magic; }
};

template <int V>
struct WordVec;
template <>
struct WordVec<1> { using type = uint32_t; };
template <>
struct WordVec<2> { using type = u32x2; };
template <>
struct WordVec<4> { using type = u32x4; };

template <int V>
__device__ __forceinline__ uint32_t vget(const typename WordVec<V>::type& v, int i) {
    if constexpr (V == 1) return v; else return v[i];
}

template <int V>
struct StepData {
    typename WordVec<V>::type w[8];  // 8 rows x V words
    u32x4 xa;                        // A operand: x[m = j][k0 + 8kb .. +7]
};

template <int V>
struct GroupData {
    typename WordVec<V>::type zw;  // V zero words
    u32x4 sv[V];                   // 8 scales per word
};

template <typename T, int V, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemv_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, float* __restrict__ partials,
    int* __restrict__ counters, int M, int N, int K, int g, int steps_per_split, int splits) {
    using WV = typename WordVec<V>::type;
    constexpr int NF = 8 * V;  // column fragments per lane
    extern __shared__ float red[];  // [WAVES][NF*4][64]
    __shared__ int s_last;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, kb = lane >> 4;
    const int words = N >> 3;
    const int tile = blockIdx.x, split = blockIdx.y;
    const int c0 = (tile * 16 + j) * V;
    const bool col_ok = c0 < words;  // words % V == 0, so all V words are in or out together

    const int total_steps = K >> 5;
    const int s_begin = split * steps_per_split;
    const int s_end = min(s_begin + steps_per_split, total_steps);
    const int per_wave = (max(s_end - s_begin, 0) + WAVES - 1) / WAVES;
    const int t0 = s_begin + wave * per_wave;
    const int t1 = min(t0 + per_wave, s_end);
    const int steps_per_group = g >> 5;  // host guarantees g % 32 == 0

    f32x4 acc[NF], dg[NF], dones;
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[f] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load_step = [&](int t, StepData<V>& d) {
        const int kbase = t * 32 + kb * 8;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if (col_ok)
                d.w[r] = *reinterpret_cast<const WV*>(qweight + (size_t)(kbase + r) * words + c0);
            else
                d.w[r] = WV{};
        }
        if (j < M)
            d.xa = *reinterpret_cast<const u32x4*>(x + (size_t)j * K + kbase);
        else
            d.xa = u32x4{0u, 0u, 0u, 0u};
    };
    auto load_group = [&](int gi, GroupData<V>& gd) {
        if (col_ok) {
            gd.zw = *reinterpret_cast<const WV*>(qzeros + (size_t)gi * words + c0);
#pragma unroll
            for (int v = 0; v < V; ++v)
                gd.sv[v] = *reinterpret_cast<const u32x4*>(scales + (size_t)gi * N +
                                                           (size_t)(c0 + v) * 8);
        } else {
            gd.zw = WV{};
#pragma unroll
            for (int v = 0; v < V; ++v) gd.sv[v] = u32x4{0u, 0u, 0u, 0u};
        }
    };
    // acc += s * (dg - (16 + z) * dones), one group's worth
    auto flush = [&](const GroupData<V>& gd) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const uint32_t zw = vget<V>(gd.zw, v);
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const float zf = (float)(((zw >> nibble_shift(c)) & 0xFu) | 16u);
                const uint32_t pair = gd.sv[v][c >> 1];
                const float sc = T::to_f32((uint16_t)((c & 1) ? (pair >> 16) : (pair & 0xFFFFu)));
                const int f = v * 8 + c;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[f][r] += sc * (dg[f][r] - zf * dones[r]);
            }
        }
    };

    if (t0 < t1) {
        StepData<V> cur, nxt;
        GroupData<V> gcur, gnxt;
        load_step(t0, cur);
        load_group(t0 / steps_per_group, gcur);
        bool fresh = true;  // dg/dones need zeroing before the next MFMA
        const u32x4 ones = u32x4{T::ones2, T::ones2, T::ones2, T::ones2};
        for (int t = t0; t < t1; ++t) {
            const bool more = t + 1 < t1;
            const bool next_new_group = more && ((t + 1) % steps_per_group == 0);
            if (more) load_step(t + 1, nxt);
            if (next_new_group) load_group((t + 1) / steps_per_group, gnxt);
            if (fresh) {
#pragma unroll
                for (int f = 0; f < NF; ++f) dg[f] = f32x4{0.f, 0.f, 0.f, 0.f};
                dones = f32x4{0.f, 0.f, 0.f, 0.f};
                fresh = false;
            }
#pragma unroll
            for (int v = 0; v < V; ++v) {
                u32x4 bfrag[8];
#pragma unroll
                for (int rp = 0; rp < 4; ++rp) {
                    const uint32_t w0 = vget<V>(cur.w[2 * rp], v);
                    const uint32_t w1 = vget<V>(cur.w[2 * rp + 1], v);
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        // byte b of row 2rp -> bits 0..7, byte b of row 2rp+1 -> bits 16..23
                        const uint32_t p =
                            __builtin_amdgcn_perm(w1, w0, 0x0c000c00u | (uint32_t)b | ((4u + b) << 16));
                        constexpr int kLoCol[4] = {0, 4, 1, 5}, kHiCol[4] = {2, 6, 3, 7};
                        bfrag[kLoCol[b]][rp] = Embed<T>::lo(p);
                        bfrag[kHiCol[b]][rp] = Embed<T>::hi(p);
                    }
                }
#pragma unroll
                for (int c = 0; c < 8; ++c) dg[v * 8 + c] = T::mfma16(cur.xa, bfrag[c], dg[v * 8 + c]);
            }
            dones = T::mfma16(cur.xa, ones, dones);
            if (next_new_group || !more) {
                flush(gcur);
                fresh = true;
                if (next_new_group) gcur = gnxt;
            }
            if (more) cur = nxt;
        }
    }

    // ---- sum the waves of this workgroup through LDS (fixed order) ----------
    // slot q = v*4 + r holds 8 consecutive output columns of row 4*kb + r
    constexpr int NQ = 4 * V;
    if constexpr (WAVES > 1) {
        float* mine = red + (size_t)wave * (NF * 4 * 64);
#pragma unroll
        for (int v = 0; v < V; ++v)
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 8; ++c) mine[((v * 4 + r) * 8 + c) * 64 + lane] = acc[v * 8 + c][r];
        __syncthreads();
    }
    for (int q = wave; q < NQ; q += WAVES) {
        const int v = q >> 2, r = q & 3;
        const int m = 4 * kb + r;
        float out[8];
        if constexpr (WAVES > 1) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) s += red[(size_t)w * (NF * 4 * 64) + (q * 8 + c) * 64 + lane];
                out[c] = s;
            }
        } else {
            // WAVES == 1: q runs over every slot in this wave; pick from registers
#pragma unroll
            for (int vv = 0; vv < V; ++vv)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr)
                    if (vv == v && rr == r)
#pragma unroll
                        for (int c = 0; c < 8; ++c) out[c] = acc[vv * 8 + c][rr];
        }
        if (m < M && col_ok) {
            const size_t n0 = (size_t)(c0 + v) * 8;
            if (splits == 1) {
                if (bias) {
                    const u32x4 bv = *reinterpret_cast<const u32x4*>(bias + n0);
#pragma unroll
                    for (int c = 0; c < 8; ++c)
                        out[c] += T::to_f32((uint16_t)((c & 1) ? (bv[c >> 1] >> 16) : (bv[c >> 1] & 0xFFFFu)));
                }
                u32x4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = T::pack2(out[2 * i], out[2 * i + 1]);
                *reinterpret_cast<u32x4*>(y + (size_t)m * N + n0) = o;
            } else {
                float* p = partials + ((size_t)split * M + m) * N + n0;
                *reinterpret_cast<f32x4*>(p) = f32x4{out[0], out[1], out[2], out[3]};
                *reinterpret_cast<f32x4*>(p + 4) = f32x4{out[4], out[5], out[6], out[7]};
            }
        }
    }
    if (splits == 1) return;

    // ---- cross-workgroup: last arriver sums the partials in split order -----
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        const int prev = __hip_atomic_fetch_add(&counters[tile], 1, __ATOMIC_ACQ_REL,
                                                __HIP_MEMORY_SCOPE_AGENT);
        s_last = (prev == splits - 1);
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    const int tile_words = 16 * V;
    const int w_begin = tile * tile_words;
    const int w_count = min(tile_words, words - w_begin);
    for (int idx = threadIdx.x; idx < M * w_count; idx += 64 * WAVES) {
        const int m = idx / w_count, wc = idx - m * w_count;
        const size_t n0 = (size_t)(w_begin + wc) * 8;
        float out[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < splits; ++s) {
            const float* p = partials + ((size_t)s * M + m) * N + n0;
            const f32x4 a = *reinterpret_cast<const f32x4*>(p);
            const f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                out[c] += a[c];
                out[4 + c] += b[c];
            }
        }
        if (bias) {
            const u32x4 bv = *reinterpret_cast<const u32x4*>(bias + n0);
#pragma unroll
            for (int c = 0; c < 8; ++c)
                out[c] += T::to_f32((uint16_t)((c & 1) ? (bv[c >> 1] >> 16) : (bv[c >> 1] & 0xFFFFu)));
        }
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = T::pack2(out[2 * i], out[2 * i + 1]);
        *reinterpret_cast<u32x4*>(y + (size_t)m * N + n0) = o;
    }
    if (threadIdx.x == 0) counters[tile] = 0;
}

// ---- host side -------------------------------------------------------------
struct GemvVariant {
    const char* name;
    int V, waves;
};
static const GemvVariant kGemvVariants[] = {
    {"v1w4", 1, 4}, {"v1w8", 1, 8}, {"v1w16", 1, 16}, {"v2w4", 2, 4},
    {"v2w8", 2, 8}, {"v4w4", 4, 4}, {"v1w1", 1, 1},  {"v2w1", 2, 1},
};
constexpr int kNumGemvVariants = sizeof(kGemvVariants) / sizeof(kGemvVariants[0]);

template <typename T, int V, int WAVES>
static hipError_t launch_gemv(const void* x, const int32_t* qweight, const void* qscales,
                              const int32_t* qzeros, const void* bias, void* y, int M, int N, int K,
                              int g, void* workspace, int split_k, hipStream_t stream) {
    const int words = N / 8;
    const int tiles = (int)cdiv(words, 16 * V);
    const int total_steps = K / 32;
    const int steps_per_split = (int)cdiv(total_steps, split_k);
    const int splits = (int)cdiv(total_steps, steps_per_split);
    int* counters = reinterpret_cast<int*>(workspace);
    float* partials = workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) +
                                                            counter_bytes(tiles))
                                : nullptr;
    const size_t lds = WAVES > 1 ? (size_t)WAVES * 8 * V * 4 * 64 * sizeof(float) : 0;
    auto kern = gemv_kernel<T, V, WAVES>;
    if (lds > 64 * 1024) {
        // once per process and instantiation; a racing second call only repeats it
        static bool raised = false;
        if (!raised) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(tiles, splits), dim3(64 * WAVES), lds, stream,
                       reinterpret_cast<const uint16_t*>(x),
                       reinterpret_cast<const uint32_t*>(qweight),
                       reinterpret_cast<const uint16_t*>(qscales),
                       reinterpret_cast<const uint32_t*>(qzeros),
                       reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y),
                       partials, counters, M, N, K, g, steps_per_split, splits);
    return hipGetLastError();
}

static int effective_splits(int64_t K, int split_k) {
    const int total_steps = (int)(K / 32);
    const int sps = (int)cdiv(total_steps, split_k);
    return (int)cdiv(total_steps, sps);
}

static size_t gemv_ws_bytes(int64_t M, int64_t N, int64_t K, int variant, int split_k) {
    const GemvVariant& gv = kGemvVariants[variant];
    const int splits = effective_splits(K, split_k);
    if (splits <= 1) return 0;
    const int64_t tiles = cdiv(N / 8, 16 * gv.V);
    return counter_bytes(tiles) + (size_t)splits * M * N * sizeof(float);
}

// Launch shape for the default entry point: enough waves to cover the chip a
// few times over, K-runs per wave as long as that allows.
static void pick_gemv(int64_t M, int64_t N, int64_t K, int* variant, int* split_k) {
    (void)M;
    const int64_t steps = K / 32;
    int v = (N % 16 == 0 && N * K >= (int64_t)4096 * 4096) ? 3 /* v2w4 */ : 0 /* v1w4 */;
    const GemvVariant& gv = kGemvVariants[v];
    const int64_t tiles = cdiv(N / 8, 16 * gv.V);
    // target ~4 waves per SIMD: 256 CUs * 4 SIMDs * 4
    const int64_t want_wgs = (256 * 16) / gv.waves;
    int64_t s = cdiv(want_wgs, tiles);
    const int64_t max_s = steps / gv.waves > 0 ? steps / gv.waves : 1;  // >= 1 step per wave
    if (s > max_s) s = max_s;
    if (s < 1) s = 1;
    if (s > 64) s = 64;
    *variant = v;
    *split_k = (int)s;
}

static int gemv_dispatch(const char* fn, const void* x, const int32_t* qweight, const void* qscales,
                         const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                         int64_t K, int64_t g, int dtype, void* workspace, size_t workspace_bytes,
                         void* stream, int variant, int split_k) {
    int rc = check_linear_args(fn, x, qweight, qscales, qzeros, y, M, N, K, g, dtype);
    if (rc != AWQ_OK) return rc;
    if (M > 16) {
        set_error("%s: M=%lld is outside the decode regime (1..16); use awq_gemm", fn, (long long)M);
        return AWQ_ERR_UNSUPPORTED;
    }
    if (g % 32 != 0 || K % 32 != 0) {
        set_error("%s: group_size %lld must be a multiple of 32", fn, (long long)g);
        return AWQ_ERR_UNSUPPORTED;
    }
    if (bias && (reinterpret_cast<uintptr_t>(bias) & 15u)) {
        set_error("%s: bias must be 16-byte aligned", fn);
        return AWQ_ERR_INVALID_ARG;
    }
    if (variant < 0 || variant >= kNumGemvVariants || split_k < 1) {
        set_error("%s: bad variant %d / split_k %d", fn, variant, split_k);
        return AWQ_ERR_INVALID_ARG;
    }
    const GemvVariant& gv = kGemvVariants[variant];
    if ((N / 8) % gv.V != 0) {
        set_error("%s: variant %s needs N %% %d == 0 (N=%lld)", fn, gv.name, 8 * gv.V, (long long)N);
        return AWQ_ERR_UNSUPPORTED;
    }
    const size_t need = gemv_ws_bytes(M, N, K, variant, split_k);
    if (need > 0 && (!workspace || workspace_bytes < need)) {
        set_error("%s: workspace of %zu bytes needed, %zu given", fn, need, workspace ? workspace_bytes : (size_t)0);
        return AWQ_ERR_WORKSPACE;
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    hipError_t e = hipErrorInvalidValue;
#define AWQ_GEMV_CASE(IDX, VV, WW)                                                                \
    case IDX:                                                                                     \
        e = dtype == AWQ_F16                                                                      \
                ? launch_gemv<F16, VV, WW>(x, qweight, qscales, qzeros, bias, y, (int)M, (int)N,  \
                                           (int)K, (int)g, workspace, split_k, s)                 \
                : launch_gemv<BF16, VV, WW>(x, qweight, qscales, qzeros, bias, y, (int)M, (int)N, \
                                            (int)K, (int)g, workspace, split_k, s);               \
        break;
    switch (variant) {
        AWQ_GEMV_CASE(0, 1, 4)
        AWQ_GEMV_CASE(1, 1, 8)
        AWQ_GEMV_CASE(2, 1, 16)
        AWQ_GEMV_CASE(3, 2, 4)
        AWQ_GEMV_CASE(4, 2, 8)
        AWQ_GEMV_CASE(5, 4, 4)
        AWQ_GEMV_CASE(6, 1, 1)
        AWQ_GEMV_CASE(7, 2, 1)
    }
#undef AWQ_GEMV_CASE
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

}  // namespace awq

extern "C" int awq_gemv_variant_count(void) { return awq::kNumGemvVariants; }

extern "C" const char* awq_gemv_variant_name(int variant) {
    return (variant >= 0 && variant < awq::kNumGemvVariants) ? awq::kGemvVariants[variant].name : "";
}

extern "C" size_t awq_gemv_ex_workspace_bytes(int64_t M, int64_t N, int64_t K, int variant,
                                              int split_k) {
    if (variant < 0 || variant >= awq::kNumGemvVariants || split_k < 1 || K < 32 || N < 8 || M < 1) return 0;
    return awq::gemv_ws_bytes(M, N, K, variant, split_k);
}

extern "C" size_t awq_gemv_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (K < 32 || N < 8 || M < 1) return 0;
    int v, s;
    awq::pick_gemv(M, N, K, &v, &s);
    return awq::gemv_ws_bytes(M, N, K, v, s);
}

extern "C" int awq_gemv_ex(const void* x, const int32_t* qweight, const void* qscales,
                           const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                           int64_t K, int64_t group_size, int dtype, void* workspace,
                           size_t workspace_bytes, void* stream, int variant, int split_k) {
    return awq::gemv_dispatch("awq_gemv_ex", x, qweight, qscales, qzeros, bias, y, M, N, K,
                              group_size, dtype, workspace, workspace_bytes, stream, variant,
                              split_k);
}

extern "C" int awq_gemv(const void* x, const int32_t* qweight, const void* qscales,
                        const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                        int64_t K, int64_t group_size, int dtype, void* workspace,
                        size_t workspace_bytes, void* stream) {
    int v = 0, s = 1;
    if (K >= 32 && N >= 8) awq::pick_gemv(M, N, K, &v, &s);
    return awq::gemv_dispatch("awq_gemv", x, qweight, qscales, qzeros, bias, y, M, N, K, group_size,
                              dtype, workspace, workspace_bytes, stream, v, s);
}
