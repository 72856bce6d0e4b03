// Kernel (c), large-M form with the B operand built in registers: fused dequant + GEMM on the
// 16x16x32 MFMA, no dequantised weight ever in LDS.
//
// A workgroup of 4 wavefronts (2 x 2, one per SIMD, a 128 x 128 sub-tile and 256 accumulator
// registers each) owns a 256 x 256 output tile and walks K in steps of 64.
//
// Lane roles, as in the decode GEMV: a lane is (j = lane % 16, kq = lane / 16).  Per 32 k rows it
// holds the packed words of rows 8*kq + 0..7 of word column j of the wave's 16 word columns: 8 k x
// 8 columns, which is what the MFMA wants from this lane as B operand of EIGHT column tiles -- tile
// t takes nibble position t of every word, so a lane's column in tile t is 8*j + column_of(t) and
// the 8 k values of its operand are the 8 rows it holds.  v_perm_b32 pairs byte b of two rows, a
// mask puts the nibbles into a 16-bit float each, and the values are multiplied out to
// RN_dtype((q - z) * s) in registers.  Each weight is unpacked by the two wavefronts that share its
// columns (2 x the arithmetic of unpacking once per workgroup) and in exchange the B tile needs no
// LDS store, no barrier between unpack and use and no LDS operand reads; LDS carries the A tile
// only (global_load_lds, three buffers), read as 16 operand fragments per wave and step.
//
// Epilogue: a lane's eight tiles are the eight columns of its word, so a row of its accumulators
// leaves as one 16-byte store (fp32 partials of a K slice: two), without staging.
#include "awq_common.hpp"
#include "awq_gemm_parts.hpp"

namespace awq {
namespace {

constexpr int kRBK = 64;

#define AWQ_RB_GPTR(p) ((__attribute__((address_space(1))) const void*)(p))
#define AWQ_RB_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

// A [256 rows][8 chunks of 16 bytes]: chunk kc of `row` sits at row*8 + (kc ^ swz(row)); 16 consecutive
// rows at one kc (an MFMA operand read of 16 lanes) touch 16 different 16-byte bank groups.
__device__ __forceinline__ int rb_row_swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// nibble position t of a packed word holds column column_of(t) of its 8 columns, and back
__host__ __device__ constexpr int column_of(int t) { return t < 4 ? 2 * t : 2 * (t - 4) + 1; }
__host__ __device__ constexpr int position_of(int c) { return 4 * (c & 1) + (c >> 1); }

// ---- 8 MFMAs and the unpack that hides behind them, as one assembly statement ---------------------------------
// A row tile's 8 MFMAs (one A fragment against the 8 B operands of the running half step) are issued with a piece of
// the NEXT half step's unpack behind each: at most three vector-ALU instructions between two MFMAs, none of them
// reading the result of the instruction right before it.  Written as assembly because the order is the point: left to
// the compiler, ordinary expressions are placed freely by instruction selection (they clump), accumulators wander
// between the two register files, and every value that one assembly statement hands to the next costs a wait state
// (the hazard pass assumes the worst of a statement it cannot read) -- so a statement is a whole row tile, whose
// results are first read a row tile later.
// The accumulators are pinned to the AGPR file by the operand constraint: all 256 of a wave's are accumulators, the
// 256 VGPRs stay free for operands and the unpack.  An MFMA's result is next read 64 MFMAs later, or after the wait in
// front of the epilogue.
template <typename T>
struct FragUnpack;

#define AWQ_RB_ACC_OPERANDS                                                                                          \
    [c0] "+a"(acc[0]), [c1] "+a"(acc[1]), [c2] "+a"(acc[2]), [c3] "+a"(acc[3]), [c4] "+a"(acc[4]), [c5] "+a"(acc[5]), \
        [c6] "+a"(acc[6]), [c7] "+a"(acc[7])
#define AWQ_RB_AB_OPERANDS                                                                                         \
    [a] "v"(af), [b0] "v"(bfc[0]), [b1] "v"(bfc[1]), [b2] "v"(bfc[2]), [b3] "v"(bfc[3]), [b4] "v"(bfc[4]),        \
        [b5] "v"(bfc[5]), [b6] "v"(bfc[6]), [b7] "v"(bfc[7])
#define AWQ_RB_MFMA(TY, I) "v_mfma_f32_16x16x32_" TY " %[c" #I "], %[a], %[b" #I "], %[c" #I "]\n\t"

// fp16: byte b of rows k, k+1 -> 0x00HL00HL (v_perm_b32); the low nibbles under 0x6400 are 1024 + q, the high nibbles
// under 0x5400 are 64 + q (no shift); minus the zero point embedded the same way (exact), times the scale (one
// rounding: the reference's RN_f16((q - z) * s)).  Row tile mg of a half step does bytes 2*(mg%2), +1 of row pair mg/2.
template <>
struct FragUnpack<F16> {
    uint32_t ezlo[4], ezhi[4], slo[4], shi[4];
    uint32_t sel[4];             // v_perm selectors, in VGPRs
    uint32_t mask_lo, mask_hi;   // SGPRs
    uint32_t magic_lo, magic_hi; // VGPRs (v_and_or_b32 takes one scalar operand)
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            sel[b] = 0x0C040C00u | (uint32_t)b | ((uint32_t)b << 16);
            asm volatile("" : "+v"(sel[b]));
        }
        mask_lo = 0x000F000Fu; mask_hi = 0x00F000F0u; magic_lo = 0x64006400u; magic_hi = 0x54005400u;
        asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));
        asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));
    }
    __device__ __forceinline__ void set_group(uint32_t zw, u32x4 sv) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t zb = __builtin_amdgcn_perm(zw, zw, 0x0C000C00u | (uint32_t)b | ((uint32_t)b << 16));
            ezlo[b] = (zb & mask_lo) | magic_lo;
            ezhi[b] = (zb & mask_hi) | magic_hi;
            constexpr uint32_t dup_lo = 0x01000100u, dup_hi = 0x03020302u;
            const int cl = column_of(2 * b), ch = column_of(2 * b + 1);
            slo[b] = __builtin_amdgcn_perm(sv[cl >> 1], sv[cl >> 1], (cl & 1) ? dup_hi : dup_lo);
            shi[b] = __builtin_amdgcn_perm(sv[ch >> 1], sv[ch >> 1], (ch & 1) ? dup_hi : dup_lo);
        }
    }
    // acc[t] += af x bfc[t] for the 8 column tiles; meanwhile bfn[t][r] = (W[k + 2r, col t], W[k + 2r + 1, col t]) of
    // the 8 rows w[0..7] of the next half step, for r = mg/2 and the four positions t of bytes 2*(mg%2), +1
    __device__ __forceinline__ void row_tile(int mg, f32x4 (&acc)[8], const u32x4& af, const u32x4 (&bfc)[8],
                                             const uint32_t (&w)[8], u32x4 (&bfn)[8]) {
        const int r = mg >> 1, b0 = 2 * (mg & 1), b1 = b0 + 1;
        uint32_t o0, o1, o2, o3, t0, t1, t2;
        asm volatile(
            AWQ_RB_MFMA("f16", 0) "v_perm_b32 %[t0], %[w1], %[w0], %[s0]\n\t"
            AWQ_RB_MFMA("f16", 1) "v_and_or_b32 %[t1], %[mlo], %[t0], %[glo]\n\t"
                                  "v_and_or_b32 %[t2], %[mhi], %[t0], %[ghi]\n\t"
            AWQ_RB_MFMA("f16", 2) "v_pk_add_f16 %[t1], %[t1], %[z0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
                                  "v_pk_add_f16 %[t2], %[t2], %[z1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            AWQ_RB_MFMA("f16", 3) "v_pk_mul_f16 %[o0], %[t1], %[q0]\n\t"
                                  "v_pk_mul_f16 %[o1], %[t2], %[q1]\n\t"
            AWQ_RB_MFMA("f16", 4) "v_perm_b32 %[t0], %[w1], %[w0], %[s1]\n\t"
            AWQ_RB_MFMA("f16", 5) "v_and_or_b32 %[t1], %[mlo], %[t0], %[glo]\n\t"
                                  "v_and_or_b32 %[t2], %[mhi], %[t0], %[ghi]\n\t"
            AWQ_RB_MFMA("f16", 6) "v_pk_add_f16 %[t1], %[t1], %[z2] neg_lo:[0,1] neg_hi:[0,1]\n\t"
                                  "v_pk_add_f16 %[t2], %[t2], %[z3] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            AWQ_RB_MFMA("f16", 7) "v_pk_mul_f16 %[o2], %[t1], %[q2]\n\t"
                                  "v_pk_mul_f16 %[o3], %[t2], %[q3]\n\t"
            : AWQ_RB_ACC_OPERANDS, [o0] "=&v"(o0), [o1] "=&v"(o1), [o2] "=&v"(o2), [o3] "=&v"(o3), [t0] "=&v"(t0),
              [t1] "=&v"(t1), [t2] "=&v"(t2)
            : AWQ_RB_AB_OPERANDS, [w0] "v"(w[2 * r]), [w1] "v"(w[2 * r + 1]), [s0] "v"(sel[b0]), [s1] "v"(sel[b1]),
              [mlo] "s"(mask_lo), [mhi] "s"(mask_hi), [glo] "v"(magic_lo), [ghi] "v"(magic_hi), [z0] "v"(ezlo[b0]),
              [z1] "v"(ezhi[b0]), [z2] "v"(ezlo[b1]), [z3] "v"(ezhi[b1]), [q0] "v"(slo[b0]), [q1] "v"(shi[b0]),
              [q2] "v"(slo[b1]), [q3] "v"(shi[b1])
            : "memory");
        bfn[2 * b0][r] = o0;
        bfn[2 * b0 + 1][r] = o1;
        bfn[2 * b1][r] = o2;
        bfn[2 * b1 + 1][r] = o3;
    }
    // the same unpack without MFMAs (the first half step of a workgroup)
    __device__ __forceinline__ void unpack_only(const uint32_t (&w)[8], u32x4 (&bfn)[8]) const {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const uint32_t p = __builtin_amdgcn_perm(w[2 * r + 1], w[2 * r], 0x0C040C00u | (uint32_t)b | ((uint32_t)b << 16));
                const uint32_t lo = (p & mask_lo) | magic_lo, hi = (p & mask_hi) | magic_hi;
                bfn[2 * b][r] = as_u32((as_f16x2(lo) - as_f16x2(ezlo[b])) * as_f16x2(slo[b]));
                bfn[2 * b + 1][r] = as_u32((as_f16x2(hi) - as_f16x2(ezhi[b])) * as_f16x2(shi[b]));
            }
    }
};

// bf16: a nibble is masked in place at mantissa bit 8, 12 or 16 of the fp32 pattern 0x4B000000 (value 2^23 + q * 2^e),
// so fma(f, s * 2^-e, -(2^(23-e) + z) * s) = (q - z) * s exactly (product and constant have at most 24 significant
// bits, the sum at most 13); positions 0-1 and 5-7 are brought there by one shift of the word each (w << 8, w >> 12).
// Two rows are packed with one round-to-nearest-even conversion.  Row tile mg of a half step does row pair mg/2:
// positions 2, 3, 4, 0 (even mg; it also makes the two left shifts) or 1, 5, 6, 7 (odd mg; the right shifts).
template <>
struct FragUnpack<BF16> {
    float sc[8], off[8];   // per nibble position
    uint32_t mask8, mask12, mask16, magic;
    uint32_t l0, l1;
    static __device__ __forceinline__ constexpr int src_of(int t) { return t < 2 ? 0 : (t < 5 ? 1 : 2); }   // w<<8, w, w>>12
    static __device__ __forceinline__ constexpr int bit_of(int t) { return t < 2 ? 4 * t + 8 : (t < 5 ? 4 * t : 4 * t - 12); }
    __device__ __forceinline__ void init() {
        mask8 = 0xF00u; mask12 = 0xF000u; mask16 = 0xF0000u; magic = 0x4B000000u;
        asm volatile("" : "+s"(mask8), "+s"(mask12), "+s"(mask16));
        asm volatile("" : "+v"(magic));
    }
    __device__ __forceinline__ uint32_t mask_of(int t) const {
        return bit_of(t) == 8 ? mask8 : (bit_of(t) == 12 ? mask12 : mask16);
    }
    __device__ __forceinline__ void set_group(uint32_t zw, u32x4 sv) {
        const uint32_t zl = zw << 8, zh = zw >> 12;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int c = column_of(t);
            const uint32_t pr = sv[c >> 1];
            const float s = __builtin_bit_cast(float, (c & 1) ? (pr & 0xFFFF0000u) : (pr << 16));
            const float down = bit_of(t) == 8 ? 0x1p-8f : (bit_of(t) == 12 ? 0x1p-12f : 0x1p-16f);
            const uint32_t src = src_of(t) == 0 ? zl : (src_of(t) == 1 ? zw : zh);
            sc[t] = s * down;                                                                  // exact: a power of two
            off[t] = -(__builtin_bit_cast(float, (src & mask_of(t)) | magic) * sc[t]);   // (2^(23-e) + z) * s: <= 24 bits
        }
    }
#define AWQ_RB_BF16_POS(P, SRC0, SRC1)                                     \
    "v_and_or_b32 %[e0], %[m" #P "], %[" SRC0 "], %[g]\n\t"                \
    "v_and_or_b32 %[e1], %[m" #P "], %[" SRC1 "], %[g]\n\t"
#define AWQ_RB_BF16_FMA(P)                                                 \
    "v_fma_f32 %[f0], %[e0], %[s" #P "], %[k" #P "]\n\t"                   \
    "v_fma_f32 %[f1], %[e1], %[s" #P "], %[k" #P "]\n\t"
    __device__ __forceinline__ void row_tile(int mg, f32x4 (&acc)[8], const u32x4& af, const u32x4 (&bfc)[8],
                                             const uint32_t (&w)[8], u32x4 (&bfn)[8]) {
        const int r = mg >> 1;
        uint32_t o0, o1, o2, o3, e0, e1, x0, x1;
        float f0, f1;
        if ((mg & 1) == 0) {
            // positions 2, 3, 4 from the word itself, 0 from the left-shifted copy made on the way
            asm volatile(
                AWQ_RB_MFMA("bf16", 0) AWQ_RB_BF16_POS(A, "w0", "w1") "v_lshlrev_b32 %[x0], 8, %[w0]\n\t"
                AWQ_RB_MFMA("bf16", 1) AWQ_RB_BF16_FMA(A) "v_lshlrev_b32 %[x1], 8, %[w1]\n\t"
                AWQ_RB_MFMA("bf16", 2) "v_cvt_pk_bf16_f32 %[o0], %[f0], %[f1]\n\t" AWQ_RB_BF16_POS(B, "w0", "w1")
                AWQ_RB_MFMA("bf16", 3) AWQ_RB_BF16_FMA(B)
                AWQ_RB_MFMA("bf16", 4) "v_cvt_pk_bf16_f32 %[o1], %[f0], %[f1]\n\t" AWQ_RB_BF16_POS(C, "w0", "w1")
                AWQ_RB_MFMA("bf16", 5) AWQ_RB_BF16_FMA(C)
                AWQ_RB_MFMA("bf16", 6) "v_cvt_pk_bf16_f32 %[o2], %[f0], %[f1]\n\t" AWQ_RB_BF16_POS(D, "x0", "x1")
                AWQ_RB_MFMA("bf16", 7) AWQ_RB_BF16_FMA(D)
                "s_nop 0\n\t"
                "v_cvt_pk_bf16_f32 %[o3], %[f0], %[f1]\n\t"
                : AWQ_RB_ACC_OPERANDS, [o0] "=&v"(o0), [o1] "=&v"(o1), [o2] "=&v"(o2), [o3] "=&v"(o3), [e0] "=&v"(e0),
                  [e1] "=&v"(e1), [f0] "=&v"(f0), [f1] "=&v"(f1), [x0] "=&v"(x0), [x1] "=&v"(x1)
                : AWQ_RB_AB_OPERANDS, [w0] "v"(w[2 * r]), [w1] "v"(w[2 * r + 1]), [g] "v"(magic), [mA] "s"(mask_of(2)),
                  [mB] "s"(mask_of(3)), [mC] "s"(mask_of(4)), [mD] "s"(mask_of(0)), [sA] "v"(sc[2]), [sB] "v"(sc[3]),
                  [sC] "v"(sc[4]), [sD] "v"(sc[0]), [kA] "v"(off[2]), [kB] "v"(off[3]), [kC] "v"(off[4]),
                  [kD] "v"(off[0])
                : "memory");
            l0 = x0, l1 = x1;
            bfn[2][r] = o0, bfn[3][r] = o1, bfn[4][r] = o2, bfn[0][r] = o3;
        } else {
            // position 1 from the left-shifted copies of the even row tile, 5, 6, 7 from right-shifted ones
            asm volatile(
                AWQ_RB_MFMA("bf16", 0) AWQ_RB_BF16_POS(A, "l0", "l1") "v_lshrrev_b32 %[x0], 12, %[w0]\n\t"
                AWQ_RB_MFMA("bf16", 1) AWQ_RB_BF16_FMA(A) "v_lshrrev_b32 %[x1], 12, %[w1]\n\t"
                AWQ_RB_MFMA("bf16", 2) "v_cvt_pk_bf16_f32 %[o0], %[f0], %[f1]\n\t" AWQ_RB_BF16_POS(B, "x0", "x1")
                AWQ_RB_MFMA("bf16", 3) AWQ_RB_BF16_FMA(B)
                AWQ_RB_MFMA("bf16", 4) "v_cvt_pk_bf16_f32 %[o1], %[f0], %[f1]\n\t" AWQ_RB_BF16_POS(C, "x0", "x1")
                AWQ_RB_MFMA("bf16", 5) AWQ_RB_BF16_FMA(C)
                AWQ_RB_MFMA("bf16", 6) "v_cvt_pk_bf16_f32 %[o2], %[f0], %[f1]\n\t" AWQ_RB_BF16_POS(D, "x0", "x1")
                AWQ_RB_MFMA("bf16", 7) AWQ_RB_BF16_FMA(D)
                "s_nop 0\n\t"
                "v_cvt_pk_bf16_f32 %[o3], %[f0], %[f1]\n\t"
                : AWQ_RB_ACC_OPERANDS, [o0] "=&v"(o0), [o1] "=&v"(o1), [o2] "=&v"(o2), [o3] "=&v"(o3), [e0] "=&v"(e0),
                  [e1] "=&v"(e1), [f0] "=&v"(f0), [f1] "=&v"(f1), [x0] "=&v"(x0), [x1] "=&v"(x1)
                : AWQ_RB_AB_OPERANDS, [w0] "v"(w[2 * r]), [w1] "v"(w[2 * r + 1]), [l0] "v"(l0), [l1] "v"(l1),
                  [g] "v"(magic), [mA] "s"(mask_of(1)), [mB] "s"(mask_of(5)), [mC] "s"(mask_of(6)), [mD] "s"(mask_of(7)),
                  [sA] "v"(sc[1]), [sB] "v"(sc[5]), [sC] "v"(sc[6]), [sD] "v"(sc[7]), [kA] "v"(off[1]),
                  [kB] "v"(off[5]), [kC] "v"(off[6]), [kD] "v"(off[7])
                : "memory");
            bfn[1][r] = o0, bfn[5][r] = o1, bfn[6][r] = o2, bfn[7][r] = o3;
        }
    }
    __device__ __forceinline__ void unpack_only(const uint32_t (&w)[8], u32x4 (&bfn)[8]) const {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t w0 = w[2 * r], w1 = w[2 * r + 1];
            const uint32_t s0[3] = {w0 << 8, w0, w0 >> 12}, s1[3] = {w1 << 8, w1, w1 >> 12};
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const float e0 = __builtin_bit_cast(float, (s0[src_of(t)] & mask_of(t)) | magic);
                const float e1 = __builtin_bit_cast(float, (s1[src_of(t)] & mask_of(t)) | magic);
                bfn[t][r] = BF16::pack2(__builtin_fmaf(e0, sc[t], off[t]), __builtin_fmaf(e1, sc[t], off[t]));
            }
        }
    }
};

template <typename T>
__global__ __launch_bounds__(256) void gemm_regb_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight, const uint16_t* __restrict__ scales,
    const uint32_t* __restrict__ qzeros, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    float* __restrict__ partials, int M, int N, int K, int g, PipePlan plan) {
    constexpr int BM = 256, BN = 256;
    constexpr int NDMA = 8;              // direct-to-LDS loads per wave and step (4 waves x 8 x 1 KiB = the A tile)
    constexpr int A_SLOTS = 8 * BM;      // 16-byte slots per A buffer
    constexpr int NBUF = 4;
    extern __shared__ __attribute__((aligned(16))) u32x4 lds[];   // [NBUF][A_SLOTS]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;
    const int j = lane & 15, kq = lane >> 4;
    // Workgroups [0, full_tiles) own a whole output tile each; the rest share the tail tiles, `splits`
    // K slices per tile, slice-major.
    int tile = blockIdx.x, split = 0;
    const bool whole = (int)blockIdx.x < plan.full_tiles;
    if (!whole) {
        const int r = blockIdx.x - plan.full_tiles;
        split = r / plan.tail_tiles;
        tile = plan.full_tiles + (r - split * plan.tail_tiles);
    }
    const int m0 = (tile / plan.tiles_n) * BM, n0 = (tile % plan.tiles_n) * BN;
    const int words = N >> 3;
    const int total_iters = K / kRBK;
    const int it_begin = whole ? 0 : split * plan.iters_per_split;
    const int it_end = whole ? total_iters : min(it_begin + plan.iters_per_split, total_iters);

    // Global reads go through buffer descriptors: a 32-bit per-lane offset (loop-invariant) plus a scalar offset per
    // step, no 64-bit address arithmetic in the loop, and reads past the end of a tensor return zero.
    auto rsrc = [](const void* base, size_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0,
                                                 (int)(bytes < 0x7fffffffu ? bytes : 0x7fffffffu), 0x00020000);
    };
    const int groups = K / g;
    const __amdgpu_buffer_rsrc_t rs_a = rsrc(x + (size_t)m0 * K, (size_t)(M - m0) * K * 2);
    const __amdgpu_buffer_rsrc_t rs_w = rsrc(qweight, (size_t)K * words * 4);
    const __amdgpu_buffer_rsrc_t rs_z = rsrc(qzeros, (size_t)groups * words * 4);
    const __amdgpu_buffer_rsrc_t rs_s = rsrc(scales, (size_t)groups * words * 16);

    // ---- A: load i of wave w fills slots (NDMA*w + i)*64 + lane, i.e. rows 8*(NDMA*w + i) + lane/8, whose chunk
    //      at position lane%8 is kc = lane%8 ^ swz(row).  Rows past M read the last row; their results are never
    //      stored.
    int a_off[NDMA];
#pragma unroll
    for (int i = 0; i < NDMA; ++i) {
        const int row = (wave * NDMA + i) * 8 + (lane >> 3);
        const int kc = (lane & 7) ^ rb_row_swz(row);
        a_off[i] = (min(row, M - 1 - m0) * K + kc * 8) * 2;
    }
    auto dma_a = [&](int it, int buf) {
#pragma unroll
        for (int i = 0; i < NDMA; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, AWQ_RB_LPTR(lds + buf * A_SLOTS + (wave * NDMA + i) * 64), 16,
                                                     a_off[i], it * (kRBK * 2), 0, 0);
    };

    // ---- B: word column j of the wave's 16, rows 8*kq + i of each 32-row half step ---------------------------
    const int gwc = min(((n0 + wn0) >> 3) + j, words - 1);
    int w_off[8];   // byte offsets of the lane's 8 rows inside a half step
#pragma unroll
    for (int i = 0; i < 8; ++i) w_off[i] = ((kq * 8 + i) * words + gwc) * 4;
    auto load_half = [&](int it, int ks, uint32_t (&w)[8]) {
        const int so = (it * kRBK + ks * 32) * words * 4;   // uniform
#pragma unroll
        for (int i = 0; i < 8; ++i) w[i] = __builtin_amdgcn_raw_buffer_load_b32(rs_w, w_off[i], so, 0);
    };
    const int steps_per_group = g / kRBK;   // g % 64 == 0
    auto load_group = [&](int grp, uint32_t& z, u32x4& sv) {
        z = __builtin_amdgcn_raw_buffer_load_b32(rs_z, gwc * 4, grp * words * 4, 0);
        sv = __builtin_amdgcn_raw_buffer_load_b128(rs_s, gwc * 16, grp * words * 16, 0);
    };

    // ---- A operand reads: fragment f = 8*ks + m of a step is row wm0 + 16*m + j, chunk 4*ks + kq ----------------
    int a_rd[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) a_rd[ks] = (wm0 + j) * 8 + ((4 * ks + kq) ^ rb_row_swz(j));

    f32x4 acc[8][8];   // [row tile][nibble position]
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    FragUnpack<T> up;
    up.init();

    // One K step per pass, two half steps of 64 MFMAs each (row-tile-major: an A fragment serves 8 MFMAs in a row and
    // is read from LDS two fragments ahead, into a ring of four).  While half step h runs, the B operands of half step
    // h+1 are built behind its MFMAs.  Global loads are dealt out over the row tiles, one or two after each (a wave
    // that issues its 26 loads of a step back to back stalls on the memory pipeline's queue with its MFMAs waiting
    // behind): the two words a row tile has just consumed are re-loaded for the same half of the next step (a full
    // step ahead), and one eighth of this wave's share of the A tile of step it+2 goes out.  Four LDS buffers: the
    // barrier sits in the middle of a step, so a wave can be filling step i+2's buffer while another still reads step
    // i-1's -- never step i-2's, which is the same buffer.  Loads past the end of K are not guarded: the buffer
    // descriptors return zero (or another row's x, in bounds) and nothing uses them.
    if (it_begin < it_end) {
        uint32_t hi[8], lo_n[8], z_n;   // second-half words of this step, first-half words and group of the next
        u32x4 s_n;
        u32x4 bf[2][8], af[4];
        dma_a(it_begin, 0);
        dma_a(it_begin + 1, 1);
        {
            uint32_t lo[8], z;
            u32x4 sv;
            load_half(it_begin, 0, lo);
            load_half(it_begin, 1, hi);
            load_group(it_begin / steps_per_group, z, sv);
            load_half(it_begin + 1, 0, lo_n);
            up.set_group(z, sv);
            up.unpack_only(lo, bf[0]);
        }
        // group of step it+2 (loaded in the middle of step it), without a division per step
        int grp_nn = (it_begin + 2) / steps_per_group, cnt_nn = (it_begin + 2) % steps_per_group;
        load_group((it_begin + 1) / steps_per_group, z_n, s_n);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" ::: "memory");
        __syncthreads();
        int buf = 0;
        af[0] = lds[a_rd[0]];
        af[1] = lds[a_rd[0] + 128];
        for (int it = it_begin; it < it_end; ++it) {
            const int nb = (buf + 1) & 3;
            const u32x4* abase = lds + buf * A_SLOTS;
            const u32x4* anext = lds + nb * A_SLOTS;
            const int so_hi = ((it + 1) * kRBK + 32) * words * 4, so_lo = (it + 2) * kRBK * words * 4;   // uniform
            const int so_a = (it + 2) * (kRBK * 2);
            u32x4* a_dst = lds + ((buf + 2) & 3) * A_SLOTS + wave * NDMA * 64;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                if (ks == 1) {
                    // The A tile of step it+1 has landed in every wave: its last part went out behind the last row
                    // tile of the first half of step it-1, and 2 + 8 + 8 + NDMA loads have been issued since.
                    // (A bare barrier: __syncthreads() would also wait for those.)
                    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(18 + NDMA) : "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" : "+v"(z_n), "+v"(s_n));   // not before the barrier
                    up.set_group(z_n, s_n);
                    load_group(grp_nn, z_n, s_n);
                    if (++cnt_nn == steps_per_group) cnt_nn = 0, ++grp_nn;
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int m = 0; m < 8; ++m) {
                    const int f = ks * 8 + m;
                    // fragment f + 2, of the next step's buffer from f = 14 on
                    if (f + 2 < 16)
                        af[(f + 2) & 3] = abase[a_rd[(f + 2) >> 3] + ((f + 2) & 7) * 128];
                    else
                        af[(f + 2) & 3] = anext[a_rd[0] + (f + 2 - 16) * 128];
                    if (ks == 0) up.row_tile(m, acc[m], af[f & 3], bf[0], hi, bf[1]);
                    else up.row_tile(m, acc[m], af[f & 3], bf[1], lo_n, bf[0]);
                    if (m & 1) {
                        uint32_t(&w)[8] = ks == 0 ? hi : lo_n;
                        w[m - 1] = __builtin_amdgcn_raw_buffer_load_b32(rs_w, w_off[m - 1], ks == 0 ? so_hi : so_lo, 0);
                        w[m] = __builtin_amdgcn_raw_buffer_load_b32(rs_w, w_off[m], ks == 0 ? so_hi : so_lo, 0);
                    }
                    if (ks == 0)
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, AWQ_RB_LPTR(a_dst + m * 64), 16, a_off[m], so_a, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            buf = nb;
        }
        // the last MFMAs' results: 4 passes to write, read by the epilogue below
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }

    // acc[m][t][i]: row wm0 + 16*m + 4*kq + i, column wn0 + 8*j + column_of(t)
    const int n = n0 + wn0 + 8 * j;
    if (whole) {
        float bv[8];
        if (bias && n < N) {
            const u32x4 bvv = *reinterpret_cast<const u32x4*>(bias + n);
#pragma unroll
            for (int c = 0; c < 8; ++c)
                bv[c] = T::to_f32((uint16_t)((c & 1) ? (bvv[c >> 1] >> 16) : (bvv[c >> 1] & 0xFFFFu)));
        }
#pragma unroll
        for (int m = 0; m < 8; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = m0 + wm0 + m * 16 + 4 * kq + i;
                u32x4 val;
#pragma unroll
                for (int h = 0; h < 4; ++h) {
                    float lo = acc[m][position_of(2 * h)][i], hi = acc[m][position_of(2 * h + 1)][i];
                    if (bias) lo = add_bias<T>(lo, bv[2 * h]), hi = add_bias<T>(hi, bv[2 * h + 1]);
                    val[h] = T::pack2(lo, hi);
                }
                if (plan.act) {
                    // a lane holds one word of 8 columns; even words are gate columns, the next word the up
                    // columns of the same outputs (N % 16 == 0, so a pair is in range or out of range together)
                    u32x4 other;
#pragma unroll
                    for (int q = 0; q < 4; ++q) other[q] = __shfl_xor(val[q], 1);
                    if (row < M && n < N)
                        swiglu_pair_store<T>(val, other, j & 1, y + (size_t)row * (N >> 1) + ((n & ~15) >> 1));
                } else if (row < M && n < N) {
                    *reinterpret_cast<u32x4*>(y + (size_t)row * N + n) = val;
                }
            }
    } else {
        // fp32 partial of this K slice, tile-compact: [slice][tail tile][256][256].  Rows and columns past
        // M and N are stored too (they stay inside the tile's slot); the reduction pass masks them.
        float* slot = partials + ((size_t)(split * plan.tail_tiles + (tile - plan.full_tiles)) << 16);
#pragma unroll
        for (int m = 0; m < 8; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float* dst = slot + (wm0 + m * 16 + 4 * kq + i) * BN + wn0 + 8 * j;
                *reinterpret_cast<f32x4*>(dst) =
                    f32x4{acc[m][position_of(0)][i], acc[m][position_of(1)][i], acc[m][position_of(2)][i],
                          acc[m][position_of(3)][i]};
                *reinterpret_cast<f32x4*>(dst + 4) =
                    f32x4{acc[m][position_of(4)][i], acc[m][position_of(5)][i], acc[m][position_of(6)][i],
                          acc[m][position_of(7)][i]};
            }
    }
}

template <typename T>
hipError_t launch_regb(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                       const void* bias, void* y, int M, int N, int K, int g, void* workspace, int split_k,
                       bool tail_only, hipStream_t stream, int act) {
    PipePlan plan = make_pipe_plan(M, N, K, split_k, tail_only);
    plan.act = act;
    float* partials =
        workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kCounterBytes) : nullptr;
    const size_t lds = (size_t)4 * 8 * 256 * 16;  // 128 KiB
    auto kern = gemm_regb_kernel<T>;
    static bool raised = false;  // once per process and instantiation
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        raised = true;
    }
    (void)hipGetLastError();
    hipLaunchKernelGGL(kern, dim3(plan.full_tiles + plan.tail_tiles * plan.splits), dim3(256), lds, stream,
                       reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint32_t*>(qweight),
                       reinterpret_cast<const uint16_t*>(qscales), reinterpret_cast<const uint32_t*>(qzeros),
                       reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y), partials, M, N, K, g, plan);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || plan.tail_tiles == 0) return e;
    return launch_pipe_tail_reduce(T::id, partials, bias, y, M, N, plan, stream);
}

}  // namespace

hipError_t launch_gemm_regb(int dtype, const void* x, const int32_t* qweight, const void* qscales,
                            const int32_t* qzeros, const void* bias, void* y, int M, int N, int K, int g,
                            void* workspace, int split_k, bool tail_only, hipStream_t stream, int act) {
    return dtype == AWQ_F16 ? launch_regb<F16>(x, qweight, qscales, qzeros, bias, y, M, N, K, g, workspace, split_k,
                                               tail_only, stream, act)
                            : launch_regb<BF16>(x, qweight, qscales, qzeros, bias, y, M, N, K, g, workspace, split_k,
                                                tail_only, stream, act);
}

}  // namespace awq
