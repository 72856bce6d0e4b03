// Kernel (c), large-M form: fused dequant + GEMM on the 32x32x16 MFMA with the unpack hidden
// behind the matrix cores.
//
// A workgroup of 8 wavefronts (2 x 4, a 128 x 64 sub-tile and 128 accumulator registers each) owns a
// 256 x 256 output tile and walks K in steps of 64.  Two wavefronts share a SIMD on purpose: a SIMD
// issues one instruction per wavefront every four cycles, and the unpack adds some 240 vector-ALU
// instructions to the 64 MFMAs of a step, so with a single wavefront per SIMD the issue slots, not
// the matrix core, set the pace (measured: 0.98 vs 1.10 PFLOP/s at M = 8192); with two, one
// wavefront's MFMAs issue beside the other's unpack and LDS traffic.
//
// LDS holds two buffers of { A tile, dequantised B tile }:
//   A: x[m0.., k0..k0+63] lands straight from global memory (global_load_lds, no registers, no
//      vector ALU), row-major, the eight 16-byte chunks of a row XOR-swizzled by the row number;
//   B: packed words go global -> registers one step ahead; while the MFMAs of step i run, the
//      same wave turns the words of step i+1 into RN_dtype((q - z) * s), two k rows at a time, and
//      stores them k-contiguous for step i+1.
//
// bf16 unpack: a nibble is masked in place at mantissa bit 8, 12 or 16 of the fp32 pattern
// 0x4B000000 (value 2^23 + q * 2^e), so  fma(f, s * 2^-e, -(2^(23-e) + z) * s) = (q - z) * s
// exactly: the product and the constant have at most 24 significant bits each, and the sum has at
// most 13.  Nibbles 0-1 and 5-7 are brought to those positions by one shift of the word each.
#include <type_traits>

#include "awq_common.hpp"
#include "awq_gemm_parts.hpp"

namespace awq {
namespace {

constexpr int kPBK = 64;

#define AWQ_GPTR(p) ((__attribute__((address_space(1))) const void*)(p))
#define AWQ_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

// ---- LDS layouts (16-byte slots) ----------------------------------------------------------------
// A [256 rows][8 chunks]: chunk kc of `row` sits at row*8 + (kc ^ swz(row)).  32 consecutive rows
// at one kc (an MFMA operand read) touch every 16-byte bank group once, whether the LDS serves 8
// or 16 lanes per cycle.
__device__ __forceinline__ int row_swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }
// B [8 k-blocks][2][8 columns c][16 word columns]: conflict-free for the writer (32 word columns
// at one c) and the reader (32 consecutive columns at one k-block).
__device__ __forceinline__ int b_slot_p(int wc, int c, int kblk) {
    return kblk * 256 + ((wc >> 4) << 7) + (c << 4) + ((wc & 15) ^ c ^ ((c & 1) << 3));
}

// ---- unpack of two k rows of one word column ----------------------------------------------------
template <typename T>
struct PipeUnpack : UnpackRows<T> {
    __device__ __forceinline__ void init() {}
};

template <>
struct PipeUnpack<BF16> {
    float sc[8], off[8];
    uint32_t mask8, mask12, mask16, magic;
    // column c lives in nibble 4*(c&1) + (c>>1); where it is picked up after the shifts:
    static __device__ __forceinline__ constexpr int src_of(int c) {   // 0: w << 8, 1: w, 2: w >> 12
        const int jn = 4 * (c & 1) + (c >> 1);
        return jn < 2 ? 0 : (jn < 5 ? 1 : 2);
    }
    static __device__ __forceinline__ constexpr int bit_of(int c) {   // 8, 12 or 16
        const int jn = 4 * (c & 1) + (c >> 1);
        return jn < 2 ? 4 * jn + 8 : (jn < 5 ? 4 * jn : 4 * jn - 12);
    }
    __device__ __forceinline__ void init() {
        mask8 = 0xF00u; mask12 = 0xF000u; mask16 = 0xF0000u; magic = 0x4B000000u;
        asm volatile("" : "+s"(mask8), "+s"(mask12), "+s"(mask16));
        asm volatile("" : "+v"(magic));
    }
    __device__ __forceinline__ float embed(uint32_t w, uint32_t wl, uint32_t wh, int c) const {
        const uint32_t src = src_of(c) == 0 ? wl : (src_of(c) == 1 ? w : wh);
        const uint32_t m = bit_of(c) == 8 ? mask8 : (bit_of(c) == 12 ? mask12 : mask16);
        return __builtin_bit_cast(float, (src & m) | magic);
    }
    __device__ __forceinline__ void set_group(uint32_t zw, u32x4 sv) {
        uint32_t zl = zw << 8, zh = zw >> 12;
        asm("" : "+v"(zl), "+v"(zh));
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint32_t pr = sv[c >> 1];
            const float s = __builtin_bit_cast(float, (c & 1) ? (pr & 0xFFFF0000u) : (pr << 16));
            const float down = bit_of(c) == 8 ? 0x1p-8f : (bit_of(c) == 12 ? 0x1p-12f : 0x1p-16f);
            sc[c] = s * down;                               // exact: a power of two
            off[c] = -(embed(zw, zl, zh, c) * sc[c]);       // (2^(23-e) + z) * s, <= 24 significant bits
        }
    }
    __device__ __forceinline__ void pair(uint32_t w0, uint32_t w1, uint32_t out[8]) const {
        uint32_t l0 = w0 << 8, h0 = w0 >> 12, l1 = w1 << 8, h1 = w1 >> 12;
        asm("" : "+v"(l0), "+v"(h0), "+v"(l1), "+v"(h1));  // keep the shifts: one per three nibbles
#pragma unroll
        for (int c = 0; c < 8; ++c)
            out[c] = BF16::pack2(__builtin_fmaf(embed(w0, l0, h0, c), sc[c], off[c]),
                                 __builtin_fmaf(embed(w1, l1, h1, c), sc[c], off[c]));
    }
};

template <int UR>
struct Raw {
    uint32_t w[UR];
    uint32_t z;
    u32x4 s;
};

template <typename T, int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN) void gemm_pipe_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight, const uint16_t* __restrict__ scales,
    const uint32_t* __restrict__ qzeros, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    float* __restrict__ partials, int M, int N, int K, int g, PipePlan plan) {
    constexpr int BM = 256, BN = 256, NW = WM * WN, NT = 64 * NW;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int UR = kPBK * 32 / NT;   // k rows of one word column per lane and step: 8 or 4
    constexpr int NP = UR / 2;           // row pairs per lane and step
    constexpr int NDMA = 32 / NW;        // direct-to-LDS loads per wave and step
    static_assert(NW == 4 || NW == 8, "4 or 8 wavefronts");
    constexpr int A_SLOTS = 8 * BM, B_SLOTS = 8 * BN, BUF = A_SLOTS + B_SLOTS;
    extern __shared__ u32x4 lds[];  // [2][BUF]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);
    // Workgroups [0, full_tiles) own a whole output tile each; the rest share the tail tiles, `splits`
    // K slices per tile, slice-major.  The hardware hands workgroups out in index order, so the short
    // tail pieces fill the CUs that the last full round would leave idle.
    int tile = blockIdx.x, split = 0;
    const bool whole = (int)blockIdx.x < plan.full_tiles;
    if (!whole) {
        const int r = blockIdx.x - plan.full_tiles;
        split = r / plan.tail_tiles;
        tile = plan.full_tiles + (r - split * plan.tail_tiles);
    }
    const int m0 = (tile / plan.tiles_n) * BM, n0 = (tile % plan.tiles_n) * BN;
    const int words = N >> 3;
    const int total_iters = K / kPBK;
    const int it_begin = whole ? 0 : split * plan.iters_per_split;
    const int it_end = whole ? total_iters : min(it_begin + plan.iters_per_split, total_iters);

    // ---- A: NDMA direct-to-LDS loads per wave and step; load i of wave w fills slots
    //      (NDMA*w + i)*64 + lane, i.e. rows 8*(NDMA*w + i) + lane/8, whose chunk at position lane%8
    //      is kc = lane%8 ^ swz(row).  Rows past M read the last row; their results are never
    //      stored.  Addresses are a wave-uniform base plus a 32-bit byte offset per lane.
    const char* a_base = reinterpret_cast<const char*>(x + (size_t)m0 * K);
    uint32_t a_off[NDMA];
#pragma unroll
    for (int i = 0; i < NDMA; ++i) {
        const int row = (wave * NDMA + i) * 8 + (lane >> 3);
        const int kc = (lane & 7) ^ row_swz(row);
        a_off[i] = ((uint32_t)min(row, M - 1 - m0) * (uint32_t)K + (uint32_t)kc * 8u) * 2u;
    }
    auto dma_a = [&](int it, int buf) {
        const char* base = a_base + (size_t)it * (kPBK * 2);  // uniform
#pragma unroll
        for (int i = 0; i < NDMA; ++i)
            __builtin_amdgcn_global_load_lds(AWQ_GPTR(base + a_off[i]),
                                             AWQ_LPTR(lds + buf * BUF + (wave * NDMA + i) * 64), 16, 0, 0);
    };

    // ---- B: a lane owns word column wc for the UR k rows of row block rb ----------------------------
    const int wc = tid & 31, rb = tid >> 5;
    const int gwc = min((n0 >> 3) + wc, words - 1);
    const uint32_t w_off = ((uint32_t)(rb * UR) * (uint32_t)words + (uint32_t)gwc) * 4u;  // bytes
    const int g_lane = (rb * UR) / g;  // host guarantees g % 64 == 0 or 64 % g == 0
    const uint32_t z_off = ((uint32_t)g_lane * (uint32_t)words + (uint32_t)gwc) * 4u;   // bytes into qzeros
    const uint32_t s_off = z_off * 4u;                                                    // bytes into scales
    auto load_raw = [&](int it, Raw<UR>& r) {
        const int k0 = it * kPBK;
        const char* wp = reinterpret_cast<const char*>(qweight + (size_t)k0 * words);  // uniform
#pragma unroll
        for (int i = 0; i < UR; ++i)
            r.w[i] = *reinterpret_cast<const uint32_t*>(wp + (size_t)i * words * 4 + w_off);
        const size_t grow = (size_t)(k0 / g) * words;  // uniform
        r.z = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const char*>(qzeros + grow) + z_off);
        r.s = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(scales + grow * 8) + s_off);
    };
    // a lane's UR rows are the part `sub` of k-block `kblk`: it writes 2*UR bytes of each 16-byte slot
    constexpr int PER_BLK = 8 / UR;
    const int kblk = rb / PER_BLK, sub = rb % PER_BLK;
    int b_wr[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) b_wr[c] = b_slot_p(wc, c, kblk) * PER_BLK + sub;
    auto store_b = [&](int buf, const uint32_t (&cols)[8][NP]) {
        u32x4* wbase = lds + buf * BUF + A_SLOTS;
        if constexpr (UR == 8) {
#pragma unroll
            for (int c = 0; c < 8; ++c) wbase[b_wr[c]] = u32x4{cols[c][0], cols[c][1], cols[c][2], cols[c][3]};
        } else {
            u32x2* w2 = reinterpret_cast<u32x2*>(wbase);
#pragma unroll
            for (int c = 0; c < 8; ++c) w2[b_wr[c]] = u32x2{cols[c][0], cols[c][1]};
        }
    };

    // ---- MFMA operand addresses ------------------------------------------------------------------
    const int li = lane & 31, kb2 = lane >> 5;
    int a_rd[4];  // row wm0 + li at k-step ks; + 256 slots per further 32 rows
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) a_rd[ks] = (wm0 + li) * 8 + ((2 * ks + kb2) ^ row_swz(wm0 + li));
    int b_rd[TN];  // column wn0 + 32b + li at k-block kb2; + 512 slots per k-step
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        const int n = wn0 + b * 32 + li;
        b_rd[b] = b_slot_p(n >> 3, n & 7, kb2);
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    PipeUnpack<T> up;
    up.init();

    // one K step: MFMAs of tile `it` (LDS buffer `buf`) interleaved with the unpack of tile it+1 (`cur`,
    // stored to the other buffer), while the packed words of tile it+2 travel to `nxt`
    auto step = [&](int it, int buf, Raw<UR>& cur, Raw<UR>& nxt) {
        load_raw(min(it + 2, it_end - 1), nxt);
        const u32x4* abase = lds + buf * BUF;
        const u32x4* bbase = abase + A_SLOTS;
        up.set_group(cur.z, cur.s);
        uint32_t cols[8][NP];
        u32x4 af[2][TM], bf[2][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a) af[0][a] = abase[a_rd[0] + a * 256];
#pragma unroll
        for (int b = 0; b < TN; ++b) bf[0][b] = bbase[b_rd[b]];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int p = ks & 1;
            if (ks < 3) {
#pragma unroll
                for (int a = 0; a < TM; ++a) af[p ^ 1][a] = abase[a_rd[ks + 1] + a * 256];
#pragma unroll
                for (int b = 0; b < TN; ++b) bf[p ^ 1][b] = bbase[b_rd[b] + (ks + 1) * 512];
            }
            if (ks % (4 / NP) == 0) {   // one pair of rows per k-step (8 rows) or per two (4 rows)
                constexpr int STRIDE = 4 / NP;
                uint32_t o[8];
                up.pair(cur.w[2 * (ks / STRIDE)], cur.w[2 * (ks / STRIDE) + 1], o);
#pragma unroll
                for (int c = 0; c < 8; ++c) cols[c][ks / STRIDE] = o[c];
            }
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b) acc[a][b] = T::mfma32(af[p][a], bf[p][b], acc[a][b]);
        }
        store_b(buf ^ 1, cols);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the A tile of step it+1 has landed
        asm volatile("" ::: "memory");
        __syncthreads();
        if (it + 2 < it_end) dma_a(it + 2, buf);
    };

    if (it_begin < it_end) {
        Raw<UR> r0, r1;
        dma_a(it_begin, 0);
        load_raw(it_begin, r0);
        load_raw(min(it_begin + 1, it_end - 1), r1);
        {
            up.set_group(r0.z, r0.s);
            uint32_t cols[8][NP];
#pragma unroll
            for (int rp = 0; rp < NP; ++rp) {
                uint32_t o[8];
                up.pair(r0.w[2 * rp], r0.w[2 * rp + 1], o);
#pragma unroll
                for (int c = 0; c < 8; ++c) cols[c][rp] = o[c];
            }
            store_b(0, cols);
        }
        if (it_begin + 1 < it_end) dma_a(it_begin + 1, 1);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" ::: "memory");
        __syncthreads();
        for (int it = it_begin; it < it_end; it += 2) {
            step(it, 0, r1, r0);
            if (it + 1 < it_end) step(it + 1, 1, r0, r1);
        }
    }
    if (whole) {
        // Direct store through LDS: the MFMA layout gives a lane one column of a 32 x 32 tile, i.e.
        // 2-byte stores; staged per wave as [32 rows][32*TN columns] the same data leaves as 16-byte
        // stores, 4*TN lanes to a row segment.  The staging area is private to the wave and LDS
        // operations of a wave execute in order, so no barrier is needed (the main loop ended with
        // one, and no direct-to-LDS load is in flight).
        constexpr int COLS = 32 * TN, PITCH = COLS + 8;  // halves per staged row, padded (bank spread)
        constexpr int LPR = COLS / 8, RPP = 64 / LPR;    // lanes per row, rows per pass
        uint16_t* stage = reinterpret_cast<uint16_t*>(lds) + wave * (32 * PITCH);
        float bv[TN];
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int n = n0 + wn0 + b * 32 + li;
            bv[b] = (bias && n < N) ? T::to_f32(bias[n]) : 0.f;
        }
        // one code path per epilogue, chosen once (merged by selects, every value pays for the bias rounding and the
        // gate product whether wanted or not: three times the instructions)
        auto rows = [&](auto mode) {
            constexpr int MODE = decltype(mode)::value;   // 0: plain, 1: + bias, 2: gated
#pragma unroll
            for (int a = 0; a < TM; ++a) {
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        stage[((v >> 2) * 8 + kb2 * 4 + (v & 3)) * PITCH + b * 32 + li] =
                            T::from_f32(MODE == 1 ? add_bias<T>(acc[a][b][v], bv[b]) : acc[a][b][v]);
#pragma unroll
                for (int j = 0; j < 32 / RPP; ++j) {
                    const int row = RPP * j + lane / LPR, chunk = lane % LPR;
                    const u32x4 val = *reinterpret_cast<const u32x4*>(stage + row * PITCH + chunk * 8);
                    const int m = m0 + wm0 + a * 32 + row, n = n0 + wn0 + chunk * 8;
                    if constexpr (MODE == 2) {
                        // a lane holds one word of 8 columns; even words are gate columns, the next word the up
                        // columns of the same outputs (N % 16 == 0, so a pair is in range or out of range together)
                        u32x4 other;
#pragma unroll
                        for (int i = 0; i < 4; ++i) other[i] = __shfl_xor(val[i], 1);
                        if (m < M && n < N)
                            swiglu_pair_store<T>(val, other, chunk & 1, y + (size_t)m * (N >> 1) + ((n & ~15) >> 1));
                    } else if (m < M && n < N) {
                        *reinterpret_cast<u32x4*>(y + (size_t)m * N + n) = val;
                    }
                }
            }
        };
        if (plan.act) rows(std::integral_constant<int, 2>{});
        else if (bias) rows(std::integral_constant<int, 1>{});
        else rows(std::integral_constant<int, 0>{});
    } else {
        // fp32 partial of this K slice, tile-compact: [slice][tail tile][256][256].  Rows and columns past
        // M and N are stored too (they stay inside the tile's slot); the reduction pass masks them.
        float* slot = partials + ((size_t)(split * plan.tail_tiles + (tile - plan.full_tiles)) << 16);
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = wm0 + a * 32 + (v >> 2) * 8 + kb2 * 4 + (v & 3);
                    slot[row * BN + wn0 + b * 32 + li] = acc[a][b][v];   // 32 lanes = one 128-byte line
                }
    }
}

// wt[n][k] = RN_T((q - z) * s): the weight dequantised exactly as the fused kernel does, transposed to k-contiguous
// rows -- the B layout a dense library GEMM runs fastest on (x @ wt^T).  A workgroup turns a 64 (k) x 256 (n) block:
// a lane owns word column wc for 8 k rows (reads of 128 B per k row), writes its 8 x 8 values as eight 16-byte
// chunks into an LDS tile [256 n][64 k], and the block leaves as full 128-byte rows.
// HBM-bound: 0.52 B read + 2 B written per weight.
template <typename T>
__global__ __launch_bounds__(256) void dequant_transpose_kernel(const uint32_t* __restrict__ qweight,
                                                                const uint16_t* __restrict__ scales,
                                                                const uint32_t* __restrict__ qzeros,
                                                                uint16_t* __restrict__ wt, int N, int K, int g) {
    __shared__ u32x4 tile[256 * 8];   // [n][8 chunks of 8 k], chunk kc of row n at n*8 + (kc ^ ((n >> 3) & 7))
    const int tid = threadIdx.x, wc = tid & 31, rb = tid >> 5;
    const int words = N >> 3;
    const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 256;
    const int gwc = min((n0 >> 3) + wc, words - 1);
    const int krow = k0 + rb * 8;
    uint32_t w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = qweight[(size_t)(krow + i) * words + gwc];
    const size_t grow = (size_t)(krow / g) * words + gwc;
    const uint32_t zw = qzeros[grow];
    const u32x4 sv = *reinterpret_cast<const u32x4*>(scales + grow * 8);
    PipeUnpack<T> up;
    up.init();
    up.set_group(zw, sv);
    uint32_t cols[8][4];
#pragma unroll
    for (int rp = 0; rp < 4; ++rp) {
        uint32_t o[8];
        up.pair(w[2 * rp], w[2 * rp + 1], o);
#pragma unroll
        for (int c = 0; c < 8; ++c) cols[c][rp] = o[c];
    }
#pragma unroll
    for (int c = 0; c < 8; ++c)
        tile[(wc * 8 + c) * 8 + (rb ^ (wc & 7))] = u32x4{cols[c][0], cols[c][1], cols[c][2], cols[c][3]};
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int n = j * 32 + (tid >> 3), kc = tid & 7;
        if (n0 + n < N)
            *reinterpret_cast<u32x4*>(wt + (size_t)(n0 + n) * K + k0 + kc * 8) = tile[n * 8 + (kc ^ ((n >> 3) & 7))];
    }
}

// Second pass over the tail tiles: y = dtype(sum over K slices, in slice order, of the fp32 partials (+ bias)).
// 32 workgroups per tile; a thread owns 8 consecutive columns of one row.
template <typename T>
__global__ __launch_bounds__(256) void gemm_tail_reduce_kernel(const float* __restrict__ partials,
                                                               const uint16_t* __restrict__ bias,
                                                               uint16_t* __restrict__ y, int M, int N, PipePlan plan) {
    const int r = blockIdx.x >> 5;
    const int vec = ((blockIdx.x & 31) << 8) + threadIdx.x;
    const int row = vec >> 5, col = (vec & 31) << 3;
    const int tile = plan.full_tiles + r;
    const int m = (tile / plan.tiles_n) * 256 + row, n = (tile % plan.tiles_n) * 256 + col;
    if (m >= M || n >= N) return;
    const float* p = partials + ((size_t)r << 16) + row * 256 + col;
    const size_t plane = (size_t)plan.tail_tiles << 16;
    f32x4 lo = f32x4{0.f, 0.f, 0.f, 0.f}, hi = lo;
    // four slices' loads in flight at a time, added in slice order
    for (int s0 = 0; s0 < plan.splits; s0 += 4) {
        f32x4 a[4], b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t off = (size_t)min(s0 + u, plan.splits - 1) * plane;
            a[u] = *reinterpret_cast<const f32x4*>(p + off);
            b[u] = *reinterpret_cast<const f32x4*>(p + off + 4);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (s0 + u < plan.splits) {
                lo += a[u];
                hi += b[u];
            }
    }
    float out[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (plan.act) {
        u32x4 mine, other;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            mine[i] = T::pack2(out[2 * i], out[2 * i + 1]);
            other[i] = __shfl_xor(mine[i], 1);   // the neighbouring word: in range together with this one
        }
        swiglu_pair_store<T>(mine, other, (n >> 3) & 1, y + (size_t)m * (N >> 1) + ((n & ~15) >> 1));
        return;
    }
    if (bias) {
        const u32x4 bvv = *reinterpret_cast<const u32x4*>(bias + n);
#pragma unroll
        for (int c = 0; c < 8; ++c)
            out[c] = add_bias<T>(out[c], T::to_f32((uint16_t)((c & 1) ? (bvv[c >> 1] >> 16) : (bvv[c >> 1] & 0xFFFFu))));
    }
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = T::pack2(out[2 * i], out[2 * i + 1]);
    *reinterpret_cast<u32x4*>(y + (size_t)m * N + n) = o;
}

template <typename T, int WM, int WN>
hipError_t launch_pipe(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                       const void* bias, void* y, int M, int N, int K, int g, void* workspace, int split_k,
                       bool tail_only, hipStream_t stream, int act) {
    PipePlan plan = make_pipe_plan(M, N, K, split_k, tail_only);
    plan.act = act;
    float* partials =
        workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kCounterBytes) : nullptr;
    const size_t lds = (size_t)2 * (8 * 256 + 8 * 256) * 16;  // 128 KiB
    auto kern = gemm_pipe_kernel<T, WM, WN>;
    static bool raised = false;  // once per process and instantiation
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        raised = true;
    }
    (void)hipGetLastError();
    hipLaunchKernelGGL(kern, dim3(plan.full_tiles + plan.tail_tiles * plan.splits), dim3(64 * WM * WN), lds, stream,
                       reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint32_t*>(qweight),
                       reinterpret_cast<const uint16_t*>(qscales), reinterpret_cast<const uint32_t*>(qzeros),
                       reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y), partials, M, N, K, g, plan);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || plan.tail_tiles == 0) return e;
    return launch_pipe_tail_reduce(T::id, partials, bias, y, M, N, plan, stream);
}

}  // namespace

hipError_t launch_pipe_tail_reduce(int dtype, const float* partials, const void* bias, void* y, int M, int N,
                                   const PipePlan& plan, hipStream_t stream) {
    const dim3 grid(plan.tail_tiles * 32), block(256);
    if (dtype == AWQ_F16)
        hipLaunchKernelGGL(gemm_tail_reduce_kernel<F16>, grid, block, 0, stream, partials,
                           reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y), M, N, plan);
    else
        hipLaunchKernelGGL(gemm_tail_reduce_kernel<BF16>, grid, block, 0, stream, partials,
                           reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y), M, N, plan);
    return hipGetLastError();
}

hipError_t launch_gemm_pipe(int dtype, const void* x, const int32_t* qweight, const void* qscales,
                            const int32_t* qzeros, const void* bias, void* y, int M, int N, int K, int g,
                            void* workspace, int split_k, bool tail_only, hipStream_t stream, int act) {
    return dtype == AWQ_F16
               ? launch_pipe<F16, 2, 4>(x, qweight, qscales, qzeros, bias, y, M, N, K, g, workspace, split_k, tail_only,
                                        stream, act)
               : launch_pipe<BF16, 2, 4>(x, qweight, qscales, qzeros, bias, y, M, N, K, g, workspace, split_k, tail_only,
                                         stream, act);
}

hipError_t launch_dequant_transpose(int dtype, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                                    void* wt, int N, int K, int g, hipStream_t stream) {
    (void)hipGetLastError();
    const dim3 grid((N + 255) / 256, K / 64), block(256);
    if (dtype == AWQ_F16)
        hipLaunchKernelGGL(dequant_transpose_kernel<F16>, grid, block, 0, stream,
                           reinterpret_cast<const uint32_t*>(qweight), reinterpret_cast<const uint16_t*>(qscales),
                           reinterpret_cast<const uint32_t*>(qzeros), reinterpret_cast<uint16_t*>(wt), N, K, g);
    else
        hipLaunchKernelGGL(dequant_transpose_kernel<BF16>, grid, block, 0, stream,
                           reinterpret_cast<const uint32_t*>(qweight), reinterpret_cast<const uint16_t*>(qscales),
                           reinterpret_cast<const uint32_t*>(qzeros), reinterpret_cast<uint16_t*>(wt), N, K, g);
    return hipGetLastError();
}

}  // namespace awq
