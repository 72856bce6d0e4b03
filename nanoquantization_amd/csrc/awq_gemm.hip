// Kernel (c): prefill-regime fused dequant + GEMM on the 32x32x16 MFMA.
//
// A workgroup of 4 wavefronts owns a BM x BN output tile and walks K in steps
// of BK = 64.  Per step it stages in LDS
//   A: x[m0.., k0..k0+63]            copied as 16-byte chunks,
//   B: W[k0..k0+63, n0..]^T          unpacked from the int4 words in registers,
//                                    multiplied out to RN_dtype((q - z) * s) --
//                                    the very values the reference's dequantise
//                                    kernel produces -- and written k-contiguous,
// both in [k-block of 8][row][8 x 16-bit] order so that one ds_read_b128 per
// lane is one MFMA operand.  Slots are XOR-swizzled so neither the writers
// (which hold 8 adjacent columns / 8 k-chunks of one row) nor the readers
// (32 adjacent rows) pile onto one LDS bank.  Global loads for step i+1 are
// issued before the MFMAs of step i and land in the other LDS buffer.
//
// The packed words are transposed in registers: a lane holds one word column
// for UR consecutive k rows and emits, per output column, UR k-consecutive
// values.  fp16 uses the packed-half magic (1024 + q) - (1024 + z), exact, then
// one packed multiply by the scale; bf16 converts q to fp32 and uses one fma
// q*s - z*s whose exact result needs no more than fp32's significand, then
// packs two rows with a single round-to-nearest-even conversion.
//
// Split-K: every split stores fp32 partials with plain stores; a second kernel
// adds them in split order (bit-stable) and applies the bias.
#include "awq_common.hpp"
#include "awq_gemm_parts.hpp"

namespace awq {

constexpr int kBK = 64;

// LDS slot (16-byte unit) of A row `row`, k-chunk `kc` (8 k's) inside a [8][BM] buffer
template <int BM>
__device__ __forceinline__ int a_slot(int row, int kc) { return kc * BM + (row ^ (2 * kc)); }

// LDS slot of B column n = 8*wc + c, k-block kblk inside a [8][BN] buffer
template <int BN>
__device__ __forceinline__ int b_slot(int wc, int c, int kblk) {
    return kblk * BN + ((wc >> 4) << 7) + (c << 4) + ((wc & 15) ^ (2 * c));
}

template <typename T, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, float* __restrict__ partials,
    int M, int N, int K, int g, int iters_per_split, int splits) {
    constexpr int NW = WM * WN, NT = 64 * NW;
    static_assert(NW == 4 || NW == 8, "4 or 8 wavefronts per workgroup");
    static_assert(BN == 256 || BN == 128, "BN is 128 or 256");
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    static_assert(TM >= 1 && TN >= 1, "wave tile at least 32x32");
    constexpr int WCOLS = BN / 8;                  // packed word columns per tile
    constexpr int UR = kBK * WCOLS / NT;           // k rows per lane per step
    static_assert(UR == 8 || UR == 4 || UR == 2, "a lane unpacks 2, 4 or 8 rows of one word column");
    constexpr int ACH = BM * 8 / NT;               // 16-byte A chunks per thread per step
    static_assert(ACH >= 1, "at least one A chunk per thread");
    constexpr int A_SLOTS = 8 * BM, B_SLOTS = 8 * BN;

    extern __shared__ u32x4 lds[];  // [2][A_SLOTS + B_SLOTS]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int split = blockIdx.z;
    const int words = N >> 3;
    const int total_iters = K / kBK;
    const int it_begin = split * iters_per_split;
    const int it_end = min(it_begin + iters_per_split, total_iters);

    // ---- loader coordinates (rows / columns past the edge read a valid neighbour; their
    //      results are never stored) -------------------------------------------------------------
    const uint16_t* a_src[ACH];
    int a_dst[ACH];
#pragma unroll
    for (int i = 0; i < ACH; ++i) {
        const int id = tid + NT * i;
        const int row = id >> 3, kc = id & 7;
        a_src[i] = x + (size_t)min(m0 + row, M - 1) * K + kc * 8;
        a_dst[i] = a_slot<BM>(row, kc);
    }
    const int wc = tid % WCOLS, rb = tid / WCOLS;  // word column, row block (UR rows)
    const int gwc = min((n0 >> 3) + wc, words - 1);
    const uint32_t w_off = (uint32_t)(rb * UR) * (uint32_t)words + (uint32_t)gwc;
    // group of row k0 + rb*UR: k0/g + (rb*UR)/g (host guarantees g % 64 == 0 or 64 % g == 0)
    const int g_lane = (rb * UR) / g;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    u32x4 areg[ACH];
    uint32_t wreg[UR];
    uint32_t zreg;
    u32x4 sreg;

    auto load_global = [&](int it) {
        const int k0 = it * kBK;
#pragma unroll
        for (int i = 0; i < ACH; ++i) areg[i] = *reinterpret_cast<const u32x4*>(a_src[i] + k0);
        const uint32_t* wp = qweight + (size_t)k0 * words;  // uniform
#pragma unroll
        for (int r = 0; r < UR; ++r) wreg[r] = (wp + (size_t)r * words)[w_off];
        const int gi = k0 / g + g_lane;
        zreg = qzeros[(size_t)gi * words + gwc];
        sreg = *reinterpret_cast<const u32x4*>(scales + ((size_t)gi * words + gwc) * 8);
    };

    auto store_lds = [&](int buf) {
        u32x4* abase = lds + buf * (A_SLOTS + B_SLOTS);
        u32x4* bbase = abase + A_SLOTS;
#pragma unroll
        for (int i = 0; i < ACH; ++i) abase[a_dst[i]] = areg[i];
        UnpackRows<T> up;
        up.set_group(zreg, sreg);
        uint32_t cols[8][UR / 2];
#pragma unroll
        for (int rp = 0; rp < UR / 2; ++rp) {
            uint32_t o[8];
            up.pair(wreg[2 * rp], wreg[2 * rp + 1], o);
#pragma unroll
            for (int c = 0; c < 8; ++c) cols[c][rp] = o[c];
        }
        constexpr int PER_BLK = 8 / UR;  // lanes sharing one 16-byte slot
        const int kblk = rb / PER_BLK, sub = rb % PER_BLK;
        if constexpr (UR == 8) {
#pragma unroll
            for (int c = 0; c < 8; ++c)
                bbase[b_slot<BN>(wc, c, kblk)] = u32x4{cols[c][0], cols[c][1], cols[c][2], cols[c][3]};
        } else if constexpr (UR == 4) {
            u32x2* b2 = reinterpret_cast<u32x2*>(bbase);
#pragma unroll
            for (int c = 0; c < 8; ++c) b2[b_slot<BN>(wc, c, kblk) * 2 + sub] = u32x2{cols[c][0], cols[c][1]};
        } else {
            uint32_t* b1 = reinterpret_cast<uint32_t*>(bbase);
#pragma unroll
            for (int c = 0; c < 8; ++c) b1[b_slot<BN>(wc, c, kblk) * 4 + sub] = cols[c][0];
        }
    };

    // ---- MFMA operand addresses, hoisted: only the k-step changes inside the loop -------------------
    const int li = lane & 31, kb2 = lane >> 5;
    int a_rd[kBK / 16];  // slot of A row wm0 + li at k-block 2*ks + kb2; + a*32 for the other tiles
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) a_rd[ks] = a_slot<BM>(wm0 + li, ks * 2 + kb2);
    int b_rd[TN];        // slot of B column wn0 + b*32 + li at k-block kb2; + ks*2*BN
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        const int n = wn0 + b * 32 + li;
        b_rd[b] = b_slot<BN>(n >> 3, n & 7, kb2);
    }
    auto compute = [&](int buf) {
        const u32x4* abase = lds + buf * (A_SLOTS + B_SLOTS);
        const u32x4* bbase = abase + A_SLOTS;
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            u32x4 af[TM], bf[TN];
#pragma unroll
            for (int a = 0; a < TM; ++a) af[a] = abase[a_rd[ks] + a * 32];
#pragma unroll
            for (int b = 0; b < TN; ++b) bf[b] = bbase[b_rd[b] + ks * 2 * BN];
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b) acc[a][b] = T::mfma32(af[a], bf[b], acc[a][b]);
        }
    };

    // With 8 waves, waves w and w+4 share a SIMD: one of them unpacks the next tile (vector ALU)
    // while the other multiplies the current one (matrix core), then they swap.
    const bool unpack_first = NW == 8 && (wave & 4);
    if (it_begin < it_end) {
        load_global(it_begin);
        store_lds(0);
        __syncthreads();
        for (int it = it_begin; it < it_end; ++it) {
            const int buf = (it - it_begin) & 1;
            const bool more = it + 1 < it_end;
            if (more) load_global(it + 1);
            if (unpack_first) {
                if (more) store_lds(buf ^ 1);
                compute(buf);
            } else {
                compute(buf);
                if (more) store_lds(buf ^ 1);
            }
            __syncthreads();
        }
    }

    gemm_epilogue<T, BM, BN, TM, TN, NT>(acc, bias, y, partials, M, N, m0, n0, wm0, wn0, split, splits);
}

// ---- host side -------------------------------------------------------------
struct GemmVariant {
    const char* name;
    int BM, BN, waves;
};
static const GemmVariant kGemmVariants[] = {
    // narrow tiles of gemm_kernel for up to 128 rows (wider and 8-wave forms of it were measured and removed)
    {"128x128", 128, 128, 4},
    {"64x256", 64, 256, 4},
    {"32x256", 32, 256, 4},
    {"256x256p", 256, 256, 8},   // the software-pipelined kernel of awq_gemm_pipe.hip, every tile cut split_k ways
    {"256x256pt", 256, 256, 8},  // the same kernel; split_k cuts only the tiles beyond the last full round of CUs
    // awq_gemm_regb.hip: B operands built in registers; the default entry points take it in place of the pipelined
    // kernel where the work items outnumber the CUs (see substitute_regb); group sizes that are not multiples of 64 run the
    // pipelined kernel under these names too
    {"256x256r", 256, 256, 4},   // every tile cut split_k ways
    {"256x256rt", 256, 256, 4},  // split_k cuts only the tiles beyond the last full round of CUs
};
enum { k128x128 = 0, k64x256 = 1, k32x256 = 2 };
constexpr int kPipeVariant = 3, kPipeTailVariant = 4, kRegbVariant = 5, kRegbTailVariant = 6;
static bool is_tile256(int v) { return v >= kPipeVariant && v <= kRegbTailVariant; }
static bool is_tail_variant(int v) { return v == kPipeTailVariant || v == kRegbTailVariant; }
constexpr int kNumGemmVariants = sizeof(kGemmVariants) / sizeof(kGemmVariants[0]);

template <typename T, int BM, int BN, int WM, int WN>
static hipError_t launch_gemm(const void* x, const int32_t* qweight, const void* qscales,
                              const int32_t* qzeros, const void* bias, void* y, int M, int N, int K,
                              int g, void* workspace, int split_k, hipStream_t stream) {
    const int tiles_m = (int)cdiv(M, BM), tiles_n = (int)cdiv(N, BN);
    const int total_iters = K / kBK;
    const int ips = (int)cdiv(total_iters, split_k);
    const int splits = (int)cdiv(total_iters, ips);
    float* partials = workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) +
                                                            kCounterBytes)
                                : nullptr;
    const size_t lds = (size_t)2 * 8 * (BM + BN) * 16;
    auto kern = gemm_kernel<T, BM, BN, WM, WN>;
    if (lds > 64 * 1024) {
        static bool raised = false;  // once per process and instantiation
        if (!raised) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
    (void)hipGetLastError();  // do not report an earlier, unrelated failure as this launch's
    hipLaunchKernelGGL(kern, dim3(tiles_n, tiles_m, splits), dim3(64 * WM * WN), lds, stream,
                       reinterpret_cast<const uint16_t*>(x),
                       reinterpret_cast<const uint32_t*>(qweight),
                       reinterpret_cast<const uint16_t*>(qscales),
                       reinterpret_cast<const uint32_t*>(qzeros),
                       reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y),
                       partials, M, N, K, g, ips, splits);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || splits == 1) return e;
    return launch_splitk_reduce(T::id, partials, bias, y, M, N, splits, stream);
}

static int gemm_effective_splits(int64_t K, int split_k) {
    const int total = (int)(K / kBK);
    const int ips = (int)cdiv(total, split_k);
    return (int)cdiv(total, ips);
}

static size_t gemm_ws_bytes(int64_t M, int64_t N, int64_t K, int variant, int split_k) {
    if (is_tile256(variant)) return pipe_ws_bytes(make_pipe_plan(M, N, K, split_k, is_tail_variant(variant)));
    const int splits = gemm_effective_splits(K, split_k);
    if (splits <= 1) return 0;
    return kCounterBytes + (size_t)splits * M * N * sizeof(float);
}

// Tile shape and split for the default entry point.  Large M: the pipelined 256 x 256 kernel with two
// wavefronts per SIMD, K split so that the tiles cover the CUs once (a split costs one more pass over
// the fp32 partials, which is cheap next to an idle CU).  Small M: narrower tiles of the plain kernel.
static void pick_gemm(int64_t M, int64_t N, int64_t K, int* variant, int* split_k) {
    const int kCUs = 256;
    // indices into kGemmVariants
    constexpr int kPipe8 = kPipeVariant;
    int v;
    if (M <= 32) v = k32x256;
    else if (M <= 64) v = k64x256;
    else if (M <= 128) v = k128x128;
    else v = kPipe8;
    const GemmVariant& gv = kGemmVariants[v];
    const int64_t tiles = cdiv(M, gv.BM) * cdiv(N, gv.BN);
    int64_t s = 1;
    if (tiles < kCUs) s = kCUs / tiles;
    const int64_t max_s = K / kBK / 8 > 0 ? K / kBK / 8 : 1;  // at least 8 K-steps per split
    if (v == kPipe8 && tiles > kCUs && tiles % kCUs != 0) {
        // The last round would leave CUs idle: cut only its R tiles into s pieces each.  The pieces take
        // ceil(R*s / CUs) rounds of (steps/s + a fixed cost of about 5 steps for prologue and partial store);
        // take the s that minimises it, if that saves a tenth of a round at least.
        const int64_t R = tiles % kCUs, steps = K / kBK;
        int64_t best_s = 1, best_t = steps;
        for (int64_t c = 2; c <= 16 && c <= max_s; ++c) {
            const int64_t t = cdiv(R * c, kCUs) * (cdiv(steps, c) + 5);
            if (t < best_t) best_t = t, best_s = c;
        }
        if (best_s > 1 && best_t * 10 <= steps * 9) v = kPipeTailVariant, s = best_s;
    }
    if (!is_tile256(v)) {
        // Narrow tiles (up to 128 rows): two workgroups of the 128x128 and 32x256 forms share a CU, one of the 64x256
        // form.  Workgroups run in rounds of that many; a round lasts one split's K steps plus about six steps of
        // prologue and partial store.  Take the split count with the least rounds x length (5120 x 25600 at 128
        // rows: 200 tiles unsplit 102 us, two splits 74 us, three -- 600 workgroups, a second, short round -- 93 us).
        const int64_t slots = v == k64x256 ? kCUs : 2 * kCUs, steps = K / kBK;
        const int64_t hi = max_s < 16 ? max_s : 16;
        int64_t best_t = -1;
        for (int64_t c = 1; c <= hi; ++c) {
            const int64_t t = cdiv(tiles * c, slots) * (cdiv(steps, c) + 6);
            if (best_t < 0 || t < best_t) best_t = t, s = c;
        }
    }
    if (s > max_s) s = max_s;
    if (s > 16) s = 16;
    if (s < 1) s = 1;
    *variant = v;
    *split_k = (int)s;
}

// The register-operand kernel addresses a launch through 32-bit buffer offsets: the packed weight and the 256 rows of
// x a tile reads must each stay below 2 GiB.
static bool regb_takes(int64_t N, int64_t K, int64_t g) {
    return g % 64 == 0 && N % 128 == 0 && K * (N / 8) * 4 < (1ll << 31) && 256 * K * 2 < (1ll << 31);
}

// What the default entry points run: pick_gemm's choice, with the pipelined 256 x 256 kernel replaced by the
// register-operand one where the work items -- whole tiles plus K slices of the tail tiles -- outnumber the CUs (that
// kernel walks a workgroup's items as one run of K steps: no prologue, no dispatch between tiles).  M = 8192 x 4096 x
// 12288: 729 against 822 us in fp16, 774 against 800 in bf16; 16384 x 1024 x 6144: 227 / 234 against 256 / 261.  With
// one item per workgroup its heavier start costs 3-11 % in bf16 on short items (fp16: level from 256 items on, its
// unpack being the cheaper one), so at exactly one item per CU: fp16 always; bf16 from 64 K steps per item on
// (2048 x 12288 x 4096 cut in two, 96 steps: 216 against 220 us; 16384 x 2048 x 1024, 32 steps: 79 against 74).
static void substitute_regb(int64_t M, int64_t N, int64_t K, int64_t g, int dtype, int* variant, int split_k) {
    if ((*variant != kPipeVariant && *variant != kPipeTailVariant) || !regb_takes(N, K, g)) return;
    const PipePlan pp = make_pipe_plan(M, N, K, split_k, *variant == kPipeTailVariant);
    const int64_t items = (int64_t)pp.full_tiles + (int64_t)pp.tail_tiles * pp.splits;
    const int64_t steps = pp.tail_tiles > 0 && pp.full_tiles == 0 ? pp.iters_per_split : K / 64;
    if (items > 256 || (items == 256 && (dtype == AWQ_F16 || steps >= 64)))
        *variant = *variant == kPipeVariant ? kRegbVariant : kRegbTailVariant;
}

static void plan_gemm(int64_t M, int64_t N, int64_t K, int64_t g, int dtype, int* variant, int* split_k) {
    pick_gemm(M, N, K, variant, split_k);
    substitute_regb(M, N, K, g, dtype, variant, *split_k);
}

// The same on the 256 x 256 kernels at any M (the gated epilogue exists there only).
static void plan_gemm_tile256(int64_t M, int64_t N, int64_t K, int64_t g, int dtype, int* variant, int* split_k) {
    pick_gemm(M > 128 ? M : 129, N, K, variant, split_k);   // tile counts depend on ceil(M / 256) only
    substitute_regb(M, N, K, g, dtype, variant, *split_k);
}

static int gemm_dispatch(const char* fn, const void* x, const int32_t* qweight, const void* qscales,
                         const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                         int64_t K, int64_t g, int dtype, void* workspace, size_t workspace_bytes,
                         void* stream, int variant, int split_k, int act = 0) {
    // prefetch hints pending on this thread were meant for this call; the GEMM fills the chip, so they are dropped
    // (before any check: an error return must not leave them for an unrelated later launch)
    PrefetchRegions dropped;
    take_prefetch_hint(&dropped);
    int rc = check_linear_args(fn, x, qweight, qscales, qzeros, y, M, N, K, g, dtype);
    if (rc != AWQ_OK) return rc;
    if (K % kBK != 0 || !(g % 64 == 0 || (64 % g == 0 && g % 8 == 0))) {
        set_error("%s: needs K %% 64 == 0 and a group size of 8, 16, 32 or a multiple of 64 (K=%lld, g=%lld)",
                  fn, (long long)K, (long long)g);
        return AWQ_ERR_UNSUPPORTED;
    }
    if (bias && (reinterpret_cast<uintptr_t>(bias) & 15u)) {
        set_error("%s: bias must be 16-byte aligned", fn);
        return AWQ_ERR_INVALID_ARG;
    }
    if (variant < 0 || variant >= kNumGemmVariants || split_k < 1) {
        set_error("%s: bad variant %d / split_k %d", fn, variant, split_k);
        return AWQ_ERR_INVALID_ARG;
    }
    if (act && (bias || N % 16 != 0 || !is_tile256(variant))) {
        set_error("%s: the gated epilogue takes no bias, needs N %% 16 == 0 and runs on the pipelined kernel", fn);
        return AWQ_ERR_UNSUPPORTED;
    }
    const GemmVariant& gv = kGemmVariants[variant];
    if (cdiv(M, gv.BM) > 65535) {
        set_error("%s: M=%lld exceeds the launch grid for tile %s", fn, (long long)M, gv.name);
        return AWQ_ERR_UNSUPPORTED;
    }
    const size_t need = gemm_ws_bytes(M, N, K, variant, split_k);
    if (need > 0 && (!workspace || workspace_bytes < need)) {
        set_error("%s: workspace of %zu bytes needed, %zu given", fn, need, workspace ? workspace_bytes : (size_t)0);
        return AWQ_ERR_WORKSPACE;
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    hipError_t e = hipErrorInvalidValue;
#define AWQ_GEMM_CASE(IDX, BM_, BN_, WM_, WN_)                                                    \
    case IDX:                                                                                     \
        e = dtype == AWQ_F16                                                                      \
                ? launch_gemm<F16, BM_, BN_, WM_, WN_>(x, qweight, qscales, qzeros, bias, y,      \
                                                       (int)M, (int)N, (int)K, (int)g, workspace, \
                                                       split_k, s)                                \
                : launch_gemm<BF16, BM_, BN_, WM_, WN_>(x, qweight, qscales, qzeros, bias, y,     \
                                                        (int)M, (int)N, (int)K, (int)g,           \
                                                        workspace, split_k, s);                   \
        break;
    switch (variant) {
        AWQ_GEMM_CASE(k128x128, 128, 128, 2, 2)
        AWQ_GEMM_CASE(k64x256, 64, 256, 1, 4)
        AWQ_GEMM_CASE(k32x256, 32, 256, 1, 4)
        case kPipeVariant:
        case kPipeTailVariant:
            e = launch_gemm_pipe(dtype, x, qweight, qscales, qzeros, bias, y, (int)M, (int)N, (int)K, (int)g,
                                 workspace, split_k, variant == kPipeTailVariant, s, act);
            break;
        case kRegbVariant:
        case kRegbTailVariant:
            // (group sizes below 64, widths that cut a wave's 16 word columns and tensors of 2 GiB or more run the
            // pipelined kernel)
            e = regb_takes(N, K, g) ? launch_gemm_regb(dtype, x, qweight, qscales, qzeros, bias, y, (int)M, (int)N, (int)K, (int)g,
                                               workspace, split_k, variant == kRegbTailVariant, s, act)
                            : launch_gemm_pipe(dtype, x, qweight, qscales, qzeros, bias, y, (int)M, (int)N, (int)K, (int)g,
                                               workspace, split_k, variant == kRegbTailVariant, s, act);
            break;
    }
#undef AWQ_GEMM_CASE
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

}  // namespace awq

extern "C" int awq_dequantize_transposed(const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                                         void* out, int64_t K, int64_t N, int64_t group_size, int dtype,
                                         void* stream) {
    const char* fn = "awq_dequantize_transposed";
    int rc = awq::check_linear_args(fn, out, qweight, qscales, qzeros, out, 1, N, K, group_size, dtype);
    if (rc != AWQ_OK) return rc;
    if (K % awq::kBK != 0 || !(group_size % 64 == 0 || (64 % group_size == 0 && group_size % 8 == 0)) ||
        N > 0x7fffffff || K > 0x7fffffff) {
        awq::set_error("%s: needs K %% 64 == 0 and a group size of 8, 16, 32 or a multiple of 64 (K=%lld, g=%lld)", fn,
                       (long long)K, (long long)group_size);
        return AWQ_ERR_UNSUPPORTED;
    }
    const hipError_t e = awq::launch_dequant_transpose(dtype, qweight, qscales, qzeros, out, (int)N, (int)K,
                                                       (int)group_size, reinterpret_cast<hipStream_t>(stream));
    return e == hipSuccess ? AWQ_OK : awq::hip_fail(fn, e);
}

extern "C" int awq_gemm_variant_count(void) { return awq::kNumGemmVariants; }

extern "C" const char* awq_gemm_variant_name(int variant) {
    return (variant >= 0 && variant < awq::kNumGemmVariants) ? awq::kGemmVariants[variant].name : "";
}

extern "C" int awq_gemm_plan(int64_t M, int64_t N, int64_t K, int64_t group_size, int dtype, int* variant,
                             int* split_k) {
    if (!variant || !split_k || M < 1 || N < 8 || N % 8 != 0 || K < awq::kBK || K % awq::kBK != 0 || group_size < 1 ||
        K % group_size != 0 || (dtype != AWQ_F16 && dtype != AWQ_BF16)) {
        awq::set_error("awq_gemm_plan: not a problem awq_gemm takes (M=%lld N=%lld K=%lld g=%lld dtype=%d)", (long long)M,
                       (long long)N, (long long)K, (long long)group_size, dtype);
        return AWQ_ERR_UNSUPPORTED;
    }
    awq::plan_gemm(M, N, K, group_size, dtype, variant, split_k);
    return AWQ_OK;
}

extern "C" size_t awq_gemm_ex_workspace_bytes(int64_t M, int64_t N, int64_t K, int variant,
                                              int split_k) {
    if (variant < 0 || variant >= awq::kNumGemmVariants || split_k < 1 || K < awq::kBK || N < 8 || M < 1)
        return 0;
    return awq::gemm_ws_bytes(M, N, K, variant, split_k);
}

extern "C" size_t awq_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (K < awq::kBK || N < 8 || M < 1) return 0;
    int v, s;
    awq::pick_gemm(M, N, K, &v, &s);
    return awq::gemm_ws_bytes(M, N, K, v, s);
}

extern "C" int awq_gemm_ex(const void* x, const int32_t* qweight, const void* qscales,
                           const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                           int64_t K, int64_t group_size, int dtype, void* workspace,
                           size_t workspace_bytes, void* stream, int variant, int split_k) {
    return awq::gemm_dispatch("awq_gemm_ex", x, qweight, qscales, qzeros, bias, y, M, N, K,
                              group_size, dtype, workspace, workspace_bytes, stream, variant,
                              split_k);
}

extern "C" int awq_gemm(const void* x, const int32_t* qweight, const void* qscales,
                        const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                        int64_t K, int64_t group_size, int dtype, void* workspace,
                        size_t workspace_bytes, void* stream) {
    int v = 0, s = 1;
    if (K >= awq::kBK && N >= 8 && M >= 1 && group_size > 0) awq::plan_gemm(M, N, K, group_size, dtype, &v, &s);
    return awq::gemm_dispatch("awq_gemm", x, qweight, qscales, qzeros, bias, y, M, N, K, group_size,
                              dtype, workspace, workspace_bytes, stream, v, s);
}

// 65..128 rows go to the GEMV (blocks of 16 rows) on weights up to this size, see kGemvMaxRows in awq_gemv.hip
static bool gemv_rows_ok(int64_t M, int64_t N, int64_t K) {
    return M <= 64 || (M <= 128 && K * N <= (20ll << 20));
}

extern "C" size_t awq_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    // the regime depends on the group size, which this query does not get: cover both
    size_t a = gemv_rows_ok(M, N, K) ? awq_gemv_workspace_bytes(M, N, K) : 0;
    const size_t b = M > 16 ? awq_gemm_workspace_bytes(M, N, K) : 0;
    if (M > 16 && K % awq::kBK != 0) {   // served by the GEMV in blocks of 16 rows
        const size_t c = awq_gemv_workspace_bytes(16, N, K);
        a = a > c ? a : c;
    }
    return a > b ? a : b;
}

extern "C" size_t awq_linear_swiglu_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (K < awq::kBK || N < 16 || M < 1) return 0;
    const size_t a = M <= 64 ? awq_gemv_workspace_bytes(M, N, K) : 0;
    int v, s;
    awq::plan_gemm_tile256(M, N, K, 128, AWQ_F16, &v, &s);   // the workspace is the same for both 256 x 256 kernels
    const size_t b = awq::gemm_ws_bytes(M, N, K, v, s);
    return a > b ? a : b;
}

extern "C" int awq_linear_swiglu(const void* x, const int32_t* qweight, const void* qscales,
                                 const int32_t* qzeros, void* y, int64_t M, int64_t N, int64_t K,
                                 int64_t group_size, int dtype, void* workspace, size_t workspace_bytes,
                                 void* stream) {
    const bool staged = N % 128 == 0 && group_size > 0 && group_size % 128 == 0;
    if (M >= 1 && M <= 64 && staged)
        return awq_gemv_swiglu(x, qweight, qscales, qzeros, y, M, N, K, group_size, dtype, workspace,
                               workspace_bytes, stream);
    int v = awq::kPipeVariant, s = 1;
    if (K >= awq::kBK && N >= 16 && M >= 1 && group_size > 0)
        awq::plan_gemm_tile256(M, N, K, group_size, dtype, &v, &s);
    return awq::gemm_dispatch("awq_linear_swiglu", x, qweight, qscales, qzeros, nullptr, y, M, N, K, group_size,
                              dtype, workspace, workspace_bytes, stream, v, s, 1);
}

extern "C" int awq_linear(const void* x, const int32_t* qweight, const void* qscales,
                          const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                          int64_t K, int64_t group_size, int dtype, void* workspace,
                          size_t workspace_bytes, void* stream) {
    // decode regime: up to 16 rows on any GEMV path, up to 64 on the staged one (128 on small weights)
    const bool staged = N % 128 == 0 && group_size > 0 && group_size % 128 == 0;
    if (M >= 1 && ((M <= 16 && group_size % 32 == 0) || (gemv_rows_ok(M, N, K) && staged)))
        return awq_gemv(x, qweight, qscales, qzeros, bias, y, M, N, K, group_size, dtype, workspace,
                        workspace_bytes, stream);
    if (M > 16 && K % awq::kBK != 0 && K % 32 == 0 && group_size > 0 && group_size % 32 == 0 && K % group_size == 0 &&
        N > 0 && x && y) {
        // a K the MFMA GEMM's 64-row steps do not divide (the reference takes any multiple of 32,
        // layers/gemm.py:268): the GEMV, 16 rows at a time -- no real model has such a width, so only
        // the result matters here
        const size_t esz = 2;
        for (int64_t m0 = 0; m0 < M; m0 += 16) {
            const int64_t rows = M - m0 < 16 ? M - m0 : 16;
            const int rc = awq_gemv(static_cast<const char*>(x) + (size_t)m0 * K * esz, qweight, qscales, qzeros, bias,
                                    static_cast<char*>(y) + (size_t)m0 * N * esz, rows, N, K, group_size, dtype,
                                    workspace, workspace_bytes, stream);
            if (rc != AWQ_OK) return rc;
        }
        return AWQ_OK;
    }
    return awq_gemm(x, qweight, qscales, qzeros, bias, y, M, N, K, group_size, dtype, workspace,
                    workspace_bytes, stream);
}
