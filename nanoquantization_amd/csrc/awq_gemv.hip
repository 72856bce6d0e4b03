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

// One chunk = CH steps of 32 rows inside one quantisation group.
template <int V, int CH>
struct Chunk {
    typename WordVec<V>::type w[CH][8];  // per step: 8 rows x V words
    u32x4 xa[CH];                        // per step: A operand x[m = j][k0 + 8kb .. +7]
    typename WordVec<V>::type zw;        // V zero words of the group
    u32x4 sv[V];                         // 8 scales per word
};

template <typename T, int V, int WAVES, int CH, bool PF>
__global__ __launch_bounds__(64 * WAVES) void gemv_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, float* __restrict__ partials,
    int* __restrict__ counters, int M, int N, int K, int chunks_per_group, int chunks_per_split,
    int splits) {
    using WV = typename WordVec<V>::type;
    constexpr int NF = 8 * V;  // column fragments per lane
    extern __shared__ float red[];  // [WAVES][NF*4][64]
    __shared__ int s_last;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, kb = lane >> 4;
    const int words = N >> 3;
    const int wstride = words / V;  // row stride in WV units (host guarantees words % V == 0)
    const int tile = blockIdx.x, split = blockIdx.y;
    const int wv_col = tile * 16 + j;        // this lane's column in WV units
    const bool col_ok = wv_col < wstride;
    // lanes past the last column (and A rows past M) read a valid neighbour instead of
    // branching; whatever they compute is never stored
    const int wv_ld = col_ok ? wv_col : wstride - 1;
    const int xrow = j < M ? j : 0;

    const int total_chunks = K / (32 * CH);
    const int c_begin = split * chunks_per_split;
    const int c_end = min(c_begin + chunks_per_split, total_chunks);
    const int per_wave = (max(c_end - c_begin, 0) + WAVES - 1) / WAVES;
    const int c0 = c_begin + wave * per_wave;
    const int c1 = min(c0 + per_wave, c_end);

    const WV* wlane = reinterpret_cast<const WV*>(qweight) + (size_t)(kb * 8) * wstride + wv_ld;
    const WV* zlane = reinterpret_cast<const WV*>(qzeros) + wv_ld;
    const u32x4* slane = reinterpret_cast<const u32x4*>(scales) + (size_t)wv_ld * V;
    const uint16_t* xlane = x + (size_t)xrow * K + kb * 8;

    f32x4 acc[NF];
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[f] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load_chunk = [&](int c, Chunk<V, CH>& d) {
        const int row0 = c * (32 * CH);  // wave-uniform
        const WV* wp = wlane + (size_t)row0 * wstride;
#pragma unroll
        for (int s = 0; s < CH; ++s)
#pragma unroll
            for (int r = 0; r < 8; ++r) d.w[s][r] = wp[(size_t)(s * 32 + r) * wstride];
#pragma unroll
        for (int s = 0; s < CH; ++s) d.xa[s] = *reinterpret_cast<const u32x4*>(xlane + row0 + s * 32);
        const int gi = chunks_per_group == 1 ? c : c / chunks_per_group;
        d.zw = zlane[(size_t)gi * wstride];
#pragma unroll
        for (int v = 0; v < V; ++v) d.sv[v] = slane[(size_t)gi * words + v];
    };

    const u32x4 ones = u32x4{T::ones2, T::ones2, T::ones2, T::ones2};
    const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
    auto compute_chunk = [&](const Chunk<V, CH>& d) {
        f32x4 dones = zero4;
#pragma unroll
        for (int s = 0; s < CH; ++s) dones = T::mfma16(d.xa[s], ones, dones);
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const uint32_t zw = vget<V>(d.zw, v);
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                f32x4 dlo = zero4, dhi = zero4;
#pragma unroll
                for (int s = 0; s < CH; ++s) {
                    u32x4 flo, fhi;
#pragma unroll
                    for (int rp = 0; rp < 4; ++rp) {
                        // byte b of row 2rp -> bits 0..7, byte b of row 2rp+1 -> bits 16..23
                        const uint32_t p = __builtin_amdgcn_perm(
                            vget<V>(d.w[s][2 * rp + 1], v), vget<V>(d.w[s][2 * rp], v),
                            0x0c000c00u | (uint32_t)b | ((4u + b) << 16));
                        flo[rp] = Embed<T>::lo(p);
                        fhi[rp] = Embed<T>::hi(p);
                    }
                    dlo = T::mfma16(d.xa[s], flo, dlo);
                    dhi = T::mfma16(d.xa[s], fhi, dhi);
                }
                // byte b holds column {0,4,1,5}[b] in its low and {2,6,3,7}[b] in its high nibble
                constexpr int kLoCol[4] = {0, 4, 1, 5}, kHiCol[4] = {2, 6, 3, 7};
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int c = h ? kHiCol[b] : kLoCol[b];
                    const f32x4 dq = h ? dhi : dlo;
                    const float zf = (float)(((zw >> nibble_shift(c)) & 0xFu) | 16u);
                    const uint32_t pair = d.sv[v][c >> 1];
                    const float sc = T::to_f32((uint16_t)((c & 1) ? (pair >> 16) : (pair & 0xFFFFu)));
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[v * 8 + c][r] += sc * (dq[r] - zf * dones[r]);
                }
            }
        }
    };

    if constexpr (PF) {
        Chunk<V, CH> a, b;
        if (c0 < c1) load_chunk(c0, a);
        for (int c = c0; c < c1; c += 2) {
            if (c + 1 < c1) load_chunk(c + 1, b);
            compute_chunk(a);
            if (c + 1 < c1) {
                if (c + 2 < c1) load_chunk(c + 2, a);
                compute_chunk(b);
            }
        }
    } else {
        Chunk<V, CH> a;
        for (int c = c0; c < c1; ++c) {
            load_chunk(c, a);
            compute_chunk(a);
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
            const size_t n0 = ((size_t)wv_col * V + v) * 8;
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
#pragma unroll
                for (int c = 0; c < 8; ++c) publish_f32(p + c, out[c]);
            }
        }
    }
    if (splits == 1) return;

    // ---- cross-workgroup: last arriver sums the partials in split order -----
    if (!arrive_last(&counters[tile], splits, &s_last)) return;
    const int tile_words = 16 * V;
    const int w_begin = tile * tile_words;
    const int w_count = min(tile_words, words - w_begin);
    for (int idx = threadIdx.x; idx < M * w_count; idx += 64 * WAVES) {
        const int m = idx / w_count, wc = idx - m * w_count;
        const size_t n0 = (size_t)(w_begin + wc) * 8;
        float out[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < splits; ++s) {
            const float* p = partials + ((size_t)s * M + m) * N + n0;
#pragma unroll
            for (int c = 0; c < 8; ++c) out[c] += fetch_f32(p + c);
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
    if (threadIdx.x == 0) __hip_atomic_store(&counters[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- host side -------------------------------------------------------------
struct GemvVariant {
    const char* name;
    int V, waves;
    bool prefetch;
};
static const GemvVariant kGemvVariants[] = {
    {"v1w4p", 1, 4, true},  {"v1w8p", 1, 8, true},  {"v2w4", 2, 4, false}, {"v2w8", 2, 8, false},
    {"v2w4p", 2, 4, true},  {"v1w16", 1, 16, false}, {"v1w1p", 1, 1, true}, {"v2w1", 2, 1, false},
    {"v1w4", 1, 4, false},  {"v1w8", 1, 8, false},
};
constexpr int kNumGemvVariants = sizeof(kGemvVariants) / sizeof(kGemvVariants[0]);

// rows per chunk: 128 when the group size allows it, else 32
static inline int chunk_steps(int64_t g) { return g % 128 == 0 ? 4 : 1; }

template <typename T, int V, int WAVES, int CH, bool PF>
static hipError_t launch_gemv(const void* x, const int32_t* qweight, const void* qscales,
                              const int32_t* qzeros, const void* bias, void* y, int M, int N, int K,
                              int g, void* workspace, int split_k, hipStream_t stream) {
    const int words = N / 8;
    const int tiles = (int)cdiv(words, 16 * V);
    const int total_chunks = K / (32 * CH);
    const int cps = (int)cdiv(total_chunks, split_k);
    const int splits = (int)cdiv(total_chunks, cps);
    int* counters = reinterpret_cast<int*>(workspace);
    float* partials = workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) +
                                                            kCounterBytes)
                                : nullptr;
    const size_t lds = WAVES > 1 ? (size_t)WAVES * 8 * V * 4 * 64 * sizeof(float) : 0;
    auto kern = gemv_kernel<T, V, WAVES, CH, PF>;
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
                       partials, counters, M, N, K, g / (32 * CH), cps, splits);
    return hipGetLastError();
}

// Upper bound that does not depend on the group size: the kernel never uses
// more K-splits than asked for.
static size_t gemv_ws_bytes(int64_t M, int64_t N, int64_t K, int variant, int split_k) {
    (void)variant;
    if (split_k <= 1 || K < 64) return 0;
    return kCounterBytes + (size_t)split_k * M * N * sizeof(float);
}

// Launch shape for the default entry point.
static void pick_gemv(int64_t M, int64_t N, int64_t K, int* variant, int* split_k) {
    (void)M;
    const int64_t chunks = K / 128 > 0 ? K / 128 : 1;
    const bool wide = (N % 16 == 0) && N >= 4096;
    const int v = wide ? 2 /* v2w4 */ : 0 /* v1w4p */;
    const GemvVariant& gv = kGemvVariants[v];
    const int64_t tiles = cdiv(N / 8, 16 * gv.V);
    // aim at ~2 workgroups of 4 waves per CU, but never less than one chunk per wave
    int64_t s = cdiv(512, tiles);
    const int64_t max_s = chunks / gv.waves > 0 ? chunks / gv.waves : 1;
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
    if (split_k > 1 && cdiv(N / 8, 16 * gv.V) > kMaxSplitTiles) {
        set_error("%s: split-K supports at most %lld column tiles (N=%lld)", fn,
                  (long long)kMaxSplitTiles, (long long)N);
        return AWQ_ERR_UNSUPPORTED;
    }
    const size_t need = gemv_ws_bytes(M, N, K, variant, split_k);
    if (need > 0 && (!workspace || workspace_bytes < need)) {
        set_error("%s: workspace of %zu bytes needed, %zu given", fn, need, workspace ? workspace_bytes : (size_t)0);
        return AWQ_ERR_WORKSPACE;
    }
    if (need == 0) split_k = 1;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    hipError_t e = hipErrorInvalidValue;
    const bool big_chunk = chunk_steps(g) == 4;
#define AWQ_GEMV_LAUNCH(TT, VV, WW, CC, PP)                                                        \
    launch_gemv<TT, VV, WW, CC, PP>(x, qweight, qscales, qzeros, bias, y, (int)M, (int)N, (int)K, \
                                    (int)g, workspace, split_k, s)
#define AWQ_GEMV_CASE(IDX, VV, WW, PP)                                                     \
    case IDX:                                                                              \
        if (big_chunk)                                                                     \
            e = dtype == AWQ_F16 ? AWQ_GEMV_LAUNCH(F16, VV, WW, 4, PP)                     \
                                 : AWQ_GEMV_LAUNCH(BF16, VV, WW, 4, PP);                   \
        else /* group sizes 32/64/96...: one 32-row step per chunk, no prefetch variant */ \
            e = dtype == AWQ_F16 ? AWQ_GEMV_LAUNCH(F16, VV, WW, 1, true)                   \
                                 : AWQ_GEMV_LAUNCH(BF16, VV, WW, 1, true);                 \
        break;
    switch (variant) {
        AWQ_GEMV_CASE(0, 1, 4, true)
        AWQ_GEMV_CASE(1, 1, 8, true)
        AWQ_GEMV_CASE(2, 2, 4, false)
        AWQ_GEMV_CASE(3, 2, 8, false)
        AWQ_GEMV_CASE(4, 2, 4, true)
        AWQ_GEMV_CASE(5, 1, 16, false)
        AWQ_GEMV_CASE(6, 1, 1, true)
        AWQ_GEMV_CASE(7, 2, 1, false)
        AWQ_GEMV_CASE(8, 1, 4, false)
        AWQ_GEMV_CASE(9, 1, 8, false)
    }
#undef AWQ_GEMV_CASE
#undef AWQ_GEMV_LAUNCH
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
