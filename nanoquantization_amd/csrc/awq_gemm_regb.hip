// Kernel (c), large-M form with the B operand built in registers: fused dequant + GEMM on the
// 16x16x32 MFMA; the dequantised weight exists only as MFMA operands.
//
// A workgroup of 4 wavefronts (2 x 2, one per SIMD, a 128 x 128 sub-tile and 256 accumulator
// registers each) owns a 256 x 256 output tile and walks K in steps of 64, two half steps of 32.
//
// Lane roles, as in the decode GEMV: a lane is (j = lane % 16, kq = lane / 16).  Per half step it
// holds the packed words of rows 8*kq + 0..7 of word column j of the wave's 16 word columns: 8 k x
// 8 columns, which is what the MFMA wants from this lane as B operand of EIGHT column tiles -- tile
// t takes nibble position t of every word, so a lane's column in tile t is 8*j + column_of(t) and
// the 8 k values of its operand are the 8 rows it holds.  v_perm_b32 pairs byte b of two rows (fp16)
// or a mask puts a nibble into an fp32 mantissa (bf16), and the values are multiplied out to
// RN_dtype((q - z) * s) in registers.
//
// The two wavefronts that share a column range (the upper and the lower 128 rows) split that work:
// each builds the operands of four of the eight nibble positions, two half steps ahead, and leaves
// them in LDS in operand layout (16 bytes per lane, lane-linear: no bank conflicts, no transpose);
// one half step later both read all eight back.  So every weight is unpacked once per workgroup,
// LDS carries 16 KiB of B operands per half step next to the A tile (global_load_lds, three
// buffers), and the unpack is a dozen vector-ALU instructions per 8 MFMAs.
//
// Epilogue: a lane's eight tiles are the eight columns of its word, so a row of its accumulators
// leaves as one 16-byte store (fp32 partials of a K slice: two), without staging.
//
// The workgroups are resident: the grid is at most one workgroup per CU, and a workgroup walks its
// work items (whole tiles, K slices of tail tiles) as one run of K steps -- the loads of a step are
// those of the step two ahead, across item boundaries, so only the first item of a workgroup pays
// for an unaided start, and between two items only the accumulators are stored and cleared.
//
// What the instructions cost (measured on one wave per SIMD, MFMAs back to back with one other
// instruction mixed in per 8): a 16x16x32 MFMA occupies the matrix core for 18.5 cycles and the
// SIMD's issue port for 12 of them, any other instruction for 4; LDS reads and global loads to
// registers are such 4-cycle instructions, but an LDS write of 1 KiB holds the port 32 cycles, a
// load-to-LDS of 1 KiB 44 and a barrier 12, and with one wave per SIMD nobody issues meanwhile.
// Per step that adds up to more than the matrix core's 128 x 18.5 cycles, so every instruction
// saved shows: the shared unpack (half the vector-ALU work, 8 more LDS writes per wave and step)
// is worth 3 % in bf16 and nothing in fp16 against unpacking everything in both waves of a pair.
// Forms of this kernel on the 32x32x16 MFMA (a quarter of the issue cost per flop; a 64 x 256
// sub-tile per wave with a four-way split of the unpack, or 128 x 128 with the lanes of a 32-wide
// column tile taking the low and the high nibble of 16 words) gave bit-identical results 10-15 %
// slower, and so did loading the A operands straight from global memory (no LDS at all).
#include <type_traits>

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
// A row tile's 8 MFMAs (one A fragment against the 8 B operands of the running half step) are issued with one eighth
// of the wave's unpack work behind them: one or two vector-ALU instructions between two MFMAs, none of them reading the
// result of the instruction right before it.  (Measured on one wave per SIMD: a 16x16x32 MFMA takes 12 of its 18.5
// cycles to issue, every other instruction 4, so more than one and a half of them per MFMA and the matrix core
// waits.)  Written as assembly because the order is the point: left to the compiler, ordinary expressions are placed
// freely by instruction selection (they clump), accumulators wander between the two register files, and every value
// that one assembly statement hands to the next costs a wait state (the hazard pass assumes the worst of a statement it
// cannot read) -- so a statement is a whole row tile, whose results are first read a row tile later.
// The accumulators are pinned to the AGPR file by the operand constraint: all 256 of a wave's are accumulators, the
// 256 VGPRs stay free for operands and the unpack.  An MFMA's result is next read 64 MFMAs later, or after the wait in
// front of the epilogue.  The "memory" clobber keeps the loads and LDS traffic that the loop places between two
// statements where they are.
template <typename T, int ROLE>
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
// rounding: the reference's RN_f16((q - z) * s)).  Wave ROLE of a pair owns bytes 2*ROLE, 2*ROLE + 1 of every word,
// i.e. nibble positions 4*ROLE .. 4*ROLE + 3; row tile m of a half step does byte 2*ROLE + m%2 of row pair m/2.
template <int ROLE>
struct FragUnpack<F16, ROLE> {
    static __device__ __forceinline__ constexpr int own(int i) { return 4 * ROLE + i; }   // nibble position of own[i]
    uint32_t ezlo[2], ezhi[2], slo[2], shi[2];   // of the two own bytes
    uint32_t sel[2];             // v_perm selectors, in VGPRs
    uint32_t mask_lo, mask_hi;   // SGPRs
    uint32_t magic_lo, magic_hi; // VGPRs (v_and_or_b32 takes one scalar operand)
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t b = 2 * ROLE + i;
            sel[i] = 0x0C040C00u | b | (b << 16);
            asm volatile("" : "+v"(sel[i]));
        }
        mask_lo = 0x000F000Fu; mask_hi = 0x00F000F0u; magic_lo = 0x64006400u; magic_hi = 0x54005400u;
        asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));
        asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));
    }
    __device__ __forceinline__ void set_group(uint32_t zw, u32x4 sv) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t b = 2 * ROLE + i;
            const uint32_t zb = __builtin_amdgcn_perm(zw, zw, 0x0C000C00u | b | (b << 16));
            ezlo[i] = (zb & mask_lo) | magic_lo;
            ezhi[i] = (zb & mask_hi) | magic_hi;
            constexpr uint32_t dup_lo = 0x01000100u, dup_hi = 0x03020302u;
            const int cl = column_of(2 * b), ch = column_of(2 * b + 1);
            slo[i] = __builtin_amdgcn_perm(sv[cl >> 1], sv[cl >> 1], (cl & 1) ? dup_hi : dup_lo);
            shi[i] = __builtin_amdgcn_perm(sv[ch >> 1], sv[ch >> 1], (ch & 1) ? dup_hi : dup_lo);
        }
    }
    // acc[t] += af x bfc[t] for the 8 column tiles; meanwhile out[i][r] = (W[k + 2r, own(i)], W[k + 2r + 1, own(i)])
    // of the 8 rows w[0..7] of a later half step, for r = m/2 and i = 2*(m%2), +1
    __device__ __forceinline__ void row_tile(int m, f32x4 (&acc)[8], const u32x4& af, const u32x4 (&bfc)[8],
                                             const uint32_t (&w)[8], u32x4 (&out)[4]) {
        const int r = m >> 1, i = m & 1;
        uint32_t o0, o1, t0, t1, t2;
        asm volatile(
            AWQ_RB_MFMA("f16", 0) "v_perm_b32 %[t0], %[w1], %[w0], %[s0]\n\t"
            AWQ_RB_MFMA("f16", 1) "v_and_or_b32 %[t1], %[mlo], %[t0], %[glo]\n\t"
            AWQ_RB_MFMA("f16", 2) "v_and_or_b32 %[t2], %[mhi], %[t0], %[ghi]\n\t"
            AWQ_RB_MFMA("f16", 3) "v_pk_add_f16 %[t1], %[t1], %[z0] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            AWQ_RB_MFMA("f16", 4) "v_pk_add_f16 %[t2], %[t2], %[z1] neg_lo:[0,1] neg_hi:[0,1]\n\t"
            AWQ_RB_MFMA("f16", 5) "v_pk_mul_f16 %[o0], %[t1], %[q0]\n\t"
            AWQ_RB_MFMA("f16", 6) "v_pk_mul_f16 %[o1], %[t2], %[q1]\n\t"
            AWQ_RB_MFMA("f16", 7)
            : AWQ_RB_ACC_OPERANDS, [o0] "=&v"(o0), [o1] "=&v"(o1), [t0] "=&v"(t0), [t1] "=&v"(t1), [t2] "=&v"(t2)
            : AWQ_RB_AB_OPERANDS, [w0] "v"(w[2 * r]), [w1] "v"(w[2 * r + 1]), [s0] "v"(sel[i]), [mlo] "s"(mask_lo),
              [mhi] "s"(mask_hi), [glo] "v"(magic_lo), [ghi] "v"(magic_hi), [z0] "v"(ezlo[i]), [z1] "v"(ezhi[i]),
              [q0] "v"(slo[i]), [q1] "v"(shi[i])
            : "memory");
        out[2 * i][r] = o0;
        out[2 * i + 1][r] = o1;
    }
};

// bf16: a nibble is masked in place at mantissa bit 8, 12 or 16 of the fp32 pattern 0x4B000000 (value 2^23 + q * 2^e),
// so fma(f, s * 2^-e, -(2^(23-e) + z) * s) = (q - z) * s exactly (product and constant have at most 24 significant
// bits, the sum at most 13); positions 0-1 and 5-7 are brought there by one shift of the word each (w << 8, w >> 12).
// Two rows are packed with one round-to-nearest-even conversion.  Wave 0 of a pair owns positions 2, 3, 4, 0 (the
// word itself and its left-shifted copy), wave 1 positions 1, 5, 6, 7 (the left- and the right-shifted copy); row
// tiles 2r and 2r + 1 of a half step do two of them each for row pair r.
#define AWQ_RB_E(D, SRC, MSK) "v_and_or_b32 %[" D "], %[" MSK "], %[" SRC "], %[g]\n\t"
#define AWQ_RB_F(D, E, P) "v_fma_f32 %[" D "], %[" E "], %[s" P "], %[k" P "]\n\t"
#define AWQ_RB_C(O) "v_cvt_pk_bf16_f32 %[" O "], %[f0], %[f1]\n\t"
template <int ROLE>
struct FragUnpack<BF16, ROLE> {
    static __device__ __forceinline__ constexpr int own(int i) { return ROLE == 0 ? (i < 3 ? i + 2 : 0) : (i == 0 ? 1 : i + 4); }
    static __device__ __forceinline__ constexpr int bit_of(int t) { return t < 2 ? 4 * t + 8 : (t < 5 ? 4 * t : 4 * t - 12); }
    static __device__ __forceinline__ constexpr int src_of(int t) { return t < 2 ? 0 : (t < 5 ? 1 : 2); }   // w<<8, w, w>>12
    float sc[4], off[4];   // of the four own positions
    uint32_t mask8, mask12, mask16, magic;
    uint32_t x0, x1, x2, x3;   // shifted copies handed from the even to the odd row tile of a row pair
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
        for (int i = 0; i < 4; ++i) {
            const int t = own(i), c = column_of(t);
            const uint32_t pr = sv[c >> 1];
            const float s = __builtin_bit_cast(float, (c & 1) ? (pr & 0xFFFF0000u) : (pr << 16));
            const float down = bit_of(t) == 8 ? 0x1p-8f : (bit_of(t) == 12 ? 0x1p-12f : 0x1p-16f);
            const uint32_t src = src_of(t) == 0 ? zl : (src_of(t) == 1 ? zw : zh);
            sc[i] = s * down;                                                                  // exact: a power of two
            off[i] = -(__builtin_bit_cast(float, (src & mask_of(t)) | magic) * sc[i]);   // (2^(23-e) + z) * s: <= 24 bits
        }
    }
    __device__ __forceinline__ void row_tile(int m, f32x4 (&acc)[8], const u32x4& af, const u32x4 (&bfc)[8],
                                             const uint32_t (&w)[8], u32x4 (&out)[4]) {
        const int r = m >> 1;
        uint32_t o0, o1, e0, e1, e2, e3;
        float f0, f1;
        if (ROLE == 0 && (m & 1) == 0) {
            // positions 2, 3 from the word itself; the left-shifted copies for the odd row tile
            asm volatile(
                AWQ_RB_MFMA("bf16", 0) AWQ_RB_E("e0", "w0", "mA") AWQ_RB_E("e1", "w1", "mA")
                AWQ_RB_MFMA("bf16", 1) AWQ_RB_F("f0", "e0", "A") AWQ_RB_F("f1", "e1", "A")
                AWQ_RB_MFMA("bf16", 2) AWQ_RB_E("e2", "w0", "mB") AWQ_RB_E("e3", "w1", "mB")
                AWQ_RB_MFMA("bf16", 3) AWQ_RB_C("o0") "v_lshlrev_b32 %[x0], 8, %[w0]\n\t"
                AWQ_RB_MFMA("bf16", 4) AWQ_RB_F("f0", "e2", "B") AWQ_RB_F("f1", "e3", "B")
                AWQ_RB_MFMA("bf16", 5) "v_lshlrev_b32 %[x1], 8, %[w1]\n\t"
                AWQ_RB_MFMA("bf16", 6) AWQ_RB_C("o1")
                AWQ_RB_MFMA("bf16", 7)
                : AWQ_RB_ACC_OPERANDS, [o0] "=&v"(o0), [o1] "=&v"(o1), [e0] "=&v"(e0), [e1] "=&v"(e1), [e2] "=&v"(e2),
                  [e3] "=&v"(e3), [f0] "=&v"(f0), [f1] "=&v"(f1), [x0] "=&v"(x0), [x1] "=&v"(x1)
                : AWQ_RB_AB_OPERANDS, [w0] "v"(w[2 * r]), [w1] "v"(w[2 * r + 1]), [g] "v"(magic), [mA] "s"(mask_of(2)),
                  [mB] "s"(mask_of(3)), [sA] "v"(sc[0]), [sB] "v"(sc[1]), [kA] "v"(off[0]), [kB] "v"(off[1])
                : "memory");
            out[0][r] = o0, out[1][r] = o1;
        } else if (ROLE == 0) {
            // position 4 from the word itself, position 0 from the left-shifted copies
            asm volatile(
                AWQ_RB_MFMA("bf16", 0) AWQ_RB_E("e0", "w0", "mA") AWQ_RB_E("e1", "w1", "mA")
                AWQ_RB_MFMA("bf16", 1) AWQ_RB_F("f0", "e0", "A") AWQ_RB_F("f1", "e1", "A")
                AWQ_RB_MFMA("bf16", 2) AWQ_RB_E("e2", "x0", "mB") AWQ_RB_E("e3", "x1", "mB")
                AWQ_RB_MFMA("bf16", 3) AWQ_RB_C("o0")
                AWQ_RB_MFMA("bf16", 4) AWQ_RB_F("f0", "e2", "B") AWQ_RB_F("f1", "e3", "B")
                AWQ_RB_MFMA("bf16", 5)
                AWQ_RB_MFMA("bf16", 6) AWQ_RB_C("o1")
                AWQ_RB_MFMA("bf16", 7)
                : AWQ_RB_ACC_OPERANDS, [o0] "=&v"(o0), [o1] "=&v"(o1), [e0] "=&v"(e0), [e1] "=&v"(e1), [e2] "=&v"(e2),
                  [e3] "=&v"(e3), [f0] "=&v"(f0), [f1] "=&v"(f1)
                : AWQ_RB_AB_OPERANDS, [w0] "v"(w[2 * r]), [w1] "v"(w[2 * r + 1]), [x0] "v"(x0), [x1] "v"(x1),
                  [g] "v"(magic), [mA] "s"(mask_of(4)), [mB] "s"(mask_of(0)), [sA] "v"(sc[2]), [sB] "v"(sc[3]),
                  [kA] "v"(off[2]), [kB] "v"(off[3])
                : "memory");
            out[2][r] = o0, out[3][r] = o1;
        } else if ((m & 1) == 0) {
            // position 1 from left-shifted copies, position 5 from right-shifted ones (kept for the odd row tile)
            asm volatile(
                AWQ_RB_MFMA("bf16", 0) "v_lshlrev_b32 %[x0], 8, %[w0]\n\t" "v_lshlrev_b32 %[x1], 8, %[w1]\n\t"
                AWQ_RB_MFMA("bf16", 1) "v_lshrrev_b32 %[x2], 12, %[w0]\n\t" AWQ_RB_E("e0", "x0", "mA")
                AWQ_RB_MFMA("bf16", 2) AWQ_RB_E("e1", "x1", "mA") "v_lshrrev_b32 %[x3], 12, %[w1]\n\t"
                AWQ_RB_MFMA("bf16", 3) AWQ_RB_F("f0", "e0", "A") AWQ_RB_F("f1", "e1", "A")
                AWQ_RB_MFMA("bf16", 4) AWQ_RB_E("e2", "x2", "mB") AWQ_RB_E("e3", "x3", "mB")
                AWQ_RB_MFMA("bf16", 5) AWQ_RB_C("o0")
                AWQ_RB_MFMA("bf16", 6) AWQ_RB_F("f0", "e2", "B") AWQ_RB_F("f1", "e3", "B")
                AWQ_RB_MFMA("bf16", 7) AWQ_RB_C("o1")
                : AWQ_RB_ACC_OPERANDS, [o0] "=&v"(o0), [o1] "=&v"(o1), [e0] "=&v"(e0), [e1] "=&v"(e1), [e2] "=&v"(e2),
                  [e3] "=&v"(e3), [f0] "=&v"(f0), [f1] "=&v"(f1), [x0] "=&v"(x0), [x1] "=&v"(x1), [x2] "=&v"(x2),
                  [x3] "=&v"(x3)
                : AWQ_RB_AB_OPERANDS, [w0] "v"(w[2 * r]), [w1] "v"(w[2 * r + 1]), [g] "v"(magic), [mA] "s"(mask_of(1)),
                  [mB] "s"(mask_of(5)), [sA] "v"(sc[0]), [sB] "v"(sc[1]), [kA] "v"(off[0]), [kB] "v"(off[1])
                : "memory");
            out[0][r] = o0, out[1][r] = o1;
        } else {
            // positions 6, 7 from the right-shifted copies
            asm volatile(
                AWQ_RB_MFMA("bf16", 0) AWQ_RB_E("e0", "x2", "mA") AWQ_RB_E("e1", "x3", "mA")
                AWQ_RB_MFMA("bf16", 1) AWQ_RB_F("f0", "e0", "A") AWQ_RB_F("f1", "e1", "A")
                AWQ_RB_MFMA("bf16", 2) AWQ_RB_E("e2", "x2", "mB") AWQ_RB_E("e3", "x3", "mB")
                AWQ_RB_MFMA("bf16", 3) AWQ_RB_C("o0")
                AWQ_RB_MFMA("bf16", 4) AWQ_RB_F("f0", "e2", "B") AWQ_RB_F("f1", "e3", "B")
                AWQ_RB_MFMA("bf16", 5)
                AWQ_RB_MFMA("bf16", 6) AWQ_RB_C("o1")
                AWQ_RB_MFMA("bf16", 7)
                : AWQ_RB_ACC_OPERANDS, [o0] "=&v"(o0), [o1] "=&v"(o1), [e0] "=&v"(e0), [e1] "=&v"(e1), [e2] "=&v"(e2),
                  [e3] "=&v"(e3), [f0] "=&v"(f0), [f1] "=&v"(f1)
                : AWQ_RB_AB_OPERANDS, [x2] "v"(x2), [x3] "v"(x3), [g] "v"(magic), [mA] "s"(mask_of(6)),
                  [mB] "s"(mask_of(7)), [sA] "v"(sc[2]), [sB] "v"(sc[3]), [kA] "v"(off[2]), [kB] "v"(off[3])
                : "memory");
            out[2][r] = o0, out[3][r] = o1;
        }
    }
};

// The whole unpack of 8 rows of a word column in plain code: the B operands of all eight positions, for the first two
// half steps of a workgroup (nothing to hide behind yet).
template <typename T>
__device__ __forceinline__ void unpack_all(const uint32_t (&w)[8], uint32_t zw, u32x4 sv, u32x4 (&bf)[8]) {
    UnpackRows<T> u;
    u.set_group(zw, sv);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        uint32_t o[8];   // by column
        u.pair(w[2 * r], w[2 * r + 1], o);
#pragma unroll
        for (int c = 0; c < 8; ++c) bf[position_of(c)][r] = o[c];
    }
}

// Which row tiles of a half step (ks = 0, 1; m = 0..7) have global loads issued behind them, and how many loads a wave
// has issued between the last part of an A tile and the barrier that needs the tile complete.
constexpr int kRegbGroupLoads = 2;   // load_group at the top of a step: the zero word and the scales
constexpr bool regb_issues_words(int m) { return (m & 1) != 0; }                      // two packed words
constexpr bool regb_issues_a_part(int ks, int m) { return m >= 1 && (ks == 0 || m == 1); }   // one part of the A tile
constexpr int regb_a_parts_per_step() {
    int n = 0;
    for (int ks = 0; ks < 2; ++ks)
        for (int m = 0; m < 8; ++m) n += regb_issues_a_part(ks, m) ? 1 : 0;
    return n;
}
// The last part goes out behind row tile 1 of the second half, after that row tile's words; the barrier that needs
// the tile sits in row tile 0 of the next step's second half, before that row tile issues anything.
constexpr int regb_loads_after_last_a_part() {
    int n = 0;
    for (int m = 2; m < 8; ++m) n += (regb_issues_words(m) ? 2 : 0) + (regb_issues_a_part(1, m) ? 1 : 0);
    n += kRegbGroupLoads;
    for (int m = 0; m < 8; ++m) n += (regb_issues_words(m) ? 2 : 0) + (regb_issues_a_part(0, m) ? 1 : 0);
    return n;
}

template <typename T>
__global__ __launch_bounds__(256) void gemm_regb_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight, const uint16_t* __restrict__ scales,
    const uint32_t* __restrict__ qzeros, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    float* __restrict__ partials, int M, int N, int K, int g, PipePlan plan) {
    constexpr int BM = 256, BN = 256;
    constexpr int NDMA = 8;              // direct-to-LDS loads per wave and step (4 waves x 8 x 1 KiB = the A tile)
    constexpr int A_SLOTS = 8 * BM;      // 16-byte slots per A buffer
    constexpr int NBUF = 3;
    constexpr int X_SLOTS = 4 * 4 * 64;  // 16-byte slots per B operand buffer: [wave][own position][lane]
    extern __shared__ __attribute__((aligned(16))) u32x4 lds[];   // [NBUF][A_SLOTS] A tiles, [2][X_SLOTS] B operands
    u32x4* const xlds = lds + NBUF * A_SLOTS;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;
    const int j = lane & 15, kq = lane >> 4;
    const int words = N >> 3;
    const int total_iters = K / kRBK;
    const int groups = K / g;
    const int steps_per_group = g / kRBK;   // g % 64 == 0

    // Work items [0, full_tiles) are whole output tiles; the rest are the tail tiles, `splits` K slices per tile,
    // slice-major.  A workgroup stays resident (one per CU) and takes items blockIdx.x, blockIdx.x + gridDim.x, ...
    // as ONE run of K steps: the loads of a step are always those of the step two ahead, which near the end of an
    // item is a step of the next one, so an item starts with its operands in place -- no prologue, no load latency,
    // no dispatch between tiles; only the accumulators are stored and cleared in between.
    const int items = plan.full_tiles + plan.tail_tiles * plan.splits;
    struct Item {
        int tile, split, m0, n0, it_begin, it_end;
        bool whole;
    };
    auto decode = [&](int item) {
        Item d;
        d.tile = item, d.split = 0;
        d.whole = item < plan.full_tiles;
        if (!d.whole) {
            const int r = item - plan.full_tiles;
            d.split = r / plan.tail_tiles;
            d.tile = plan.full_tiles + (r - d.split * plan.tail_tiles);
        }
        d.m0 = (d.tile / plan.tiles_n) * BM, d.n0 = (d.tile % plan.tiles_n) * BN;
        d.it_begin = d.whole ? 0 : d.split * plan.iters_per_split;
        d.it_end = d.whole ? total_iters : min(d.it_begin + plan.iters_per_split, total_iters);
        return d;
    };

    // Global reads go through buffer descriptors: a 32-bit per-lane offset (the same for every item) plus a scalar
    // offset per step, no 64-bit address arithmetic in the loop.  What depends on the item -- the tile's first row of
    // x, the wave's first word column -- is in the descriptor's base, and its size ends the tensor: rows past M read
    // zero.  (N % 128 == 0, so a wave's 16 word columns are inside the row or all outside; a window outside is moved
    // onto the row's last 16 words, whose results nobody stores.)
    auto rsrc = [](const void* base, size_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0,
                                                 (int)(bytes < 0x7fffffffu ? bytes : 0x7fffffffu), 0x00020000);
    };
    // the cursor: the step whose operands are being loaded (two ahead of the one that computes)
    __amdgpu_buffer_rsrc_t pf_a = rsrc(x, 0), pf_w = pf_a, pf_z = pf_a, pf_s = pf_a;
    int pf_item = 0, pf_it = 0, pf_end = 0, pf_grp = 0, pf_cnt = 0;
    auto open_cursor = [&](int item) {
        pf_item = item;
        if (item >= items) {   // past the workgroup's last item: nothing is fetched, the load counts stay the same
            pf_a = pf_w = pf_z = pf_s = rsrc(x, 0);
            pf_it = 0, pf_end = 0x7fffffff, pf_grp = 0, pf_cnt = 0;
            return;
        }
        const Item d = decode(item);
        const int wc0 = min((d.n0 + wn0) >> 3, words - 16);
        pf_a = rsrc(x + (size_t)d.m0 * K, (size_t)(M - d.m0) * K * 2);
        pf_w = rsrc(qweight + wc0, ((size_t)K * words - wc0) * 4);
        pf_z = rsrc(qzeros + wc0, ((size_t)groups * words - wc0) * 4);
        pf_s = rsrc(scales + (size_t)wc0 * 8, ((size_t)groups * words - wc0) * 16);
        pf_it = d.it_begin, pf_end = d.it_end;
        pf_grp = d.it_begin / steps_per_group, pf_cnt = d.it_begin % steps_per_group;
    };
    auto advance = [&]() {
        ++pf_it;
        if (++pf_cnt == steps_per_group) pf_cnt = 0, ++pf_grp;
        if (pf_it == pf_end) open_cursor(pf_item + (int)gridDim.x);
    };

    // ---- A: load i of wave w fills slots (NDMA*w + i)*64 + lane, i.e. rows 8*(NDMA*w + i) + lane/8 of the tile, whose
    //      chunk at position lane%8 is kc = lane%8 ^ swz(row).
    int a_off[NDMA];
#pragma unroll
    for (int i = 0; i < NDMA; ++i) {
        const int row = (wave * NDMA + i) * 8 + (lane >> 3);
        const int kc = (lane & 7) ^ rb_row_swz(row);
        a_off[i] = (row * K + kc * 8) * 2;
    }
    auto dma_a_part = [&](int step, int buf, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(pf_a, AWQ_RB_LPTR(lds + buf * A_SLOTS + (wave * NDMA + i) * 64), 16,
                                                 a_off[i], step * (kRBK * 2), 0, 0);
    };

    // ---- B: word column j of the wave's 16, rows 8*kq + i of each 32-row half step ---------------------------
    int w_off[8];   // byte offsets of the lane's 8 rows inside a half step
#pragma unroll
    for (int i = 0; i < 8; ++i) w_off[i] = ((kq * 8 + i) * words + j) * 4;
    auto load_word = [&](int half_step, int i) {   // half step = 2 * step + half
        return __builtin_amdgcn_raw_buffer_load_b32(pf_w, w_off[i], half_step * 32 * words * 4, 0);
    };
    auto load_group = [&](int grp, uint32_t& z, u32x4& sv) {
        z = __builtin_amdgcn_raw_buffer_load_b32(pf_z, j * 4, grp * words * 4, 0);
        sv = __builtin_amdgcn_raw_buffer_load_b128(pf_s, j * 16, grp * words * 16, 0);
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

    // The accumulators stay in the AGPR file until the store reads them, a row tile at a time (copied out all at once
    // they would push the next item's operands, which are live across the store, into scratch).
    auto pin_acc = [](f32x4 (&a)[8]) {
        asm volatile("" : "+a"(a[0]), "+a"(a[1]), "+a"(a[2]), "+a"(a[3]), "+a"(a[4]), "+a"(a[5]), "+a"(a[6]), "+a"(a[7]));
    };
    // An item's result: acc[m][t][i] is row m0 + wm0 + 16*m + 4*kq + i, column n0 + wn0 + 8*j + column_of(t).
    auto store_item = [&](const Item& d) {
        const int n = d.n0 + wn0 + 8 * j;
        if (d.whole) {
            // one code path per epilogue (chosen once per item: merged by selects, every value pays for the bias
            // rounding and the gate product whether wanted or not -- three times the instructions, 7 us per tile)
            auto rows = [&](auto mode) {
                constexpr int MODE = decltype(mode)::value;   // 0: plain, 1: + bias, 2: gated
                float bv[8];
                if constexpr (MODE == 1) {
                    if (n < N) {
                        const u32x4 bvv = *reinterpret_cast<const u32x4*>(bias + n);
#pragma unroll
                        for (int c = 0; c < 8; ++c)
                            bv[c] = T::to_f32((uint16_t)((c & 1) ? (bvv[c >> 1] >> 16) : (bvv[c >> 1] & 0xFFFFu)));
                    }
                }
#pragma unroll
                for (int m = 0; m < 8; ++m) {
                    pin_acc(acc[m]);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = d.m0 + wm0 + m * 16 + 4 * kq + i;
                        u32x4 val;
#pragma unroll
                        for (int h = 0; h < 4; ++h) {
                            float lo = acc[m][position_of(2 * h)][i], hi = acc[m][position_of(2 * h + 1)][i];
                            if constexpr (MODE == 1) lo = add_bias<T>(lo, bv[2 * h]), hi = add_bias<T>(hi, bv[2 * h + 1]);
                            val[h] = T::pack2(lo, hi);
                        }
                        if constexpr (MODE == 2) {
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
                        // one row at a time: the operands of the next item stay in their registers meanwhile
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            };
            if (plan.act) rows(std::integral_constant<int, 2>{});
            else if (bias) rows(std::integral_constant<int, 1>{});
            else rows(std::integral_constant<int, 0>{});
        } else {
            // fp32 partial of this K slice, tile-compact: [slice][tail tile][256][256].  Rows and columns past
            // M and N are stored too (they stay inside the tile's slot); the reduction pass masks them.
            float* slot = partials + ((size_t)(d.split * plan.tail_tiles + (d.tile - plan.full_tiles)) << 16);
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                pin_acc(acc[m]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float* dst = slot + (wm0 + m * 16 + 4 * kq + i) * BN + wn0 + 8 * j;
                    *reinterpret_cast<f32x4*>(dst) =
                        f32x4{acc[m][position_of(0)][i], acc[m][position_of(1)][i], acc[m][position_of(2)][i],
                              acc[m][position_of(3)][i]};
                    *reinterpret_cast<f32x4*>(dst + 4) =
                        f32x4{acc[m][position_of(4)][i], acc[m][position_of(5)][i], acc[m][position_of(6)][i],
                              acc[m][position_of(7)][i]};
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };

    // Half step h = 2 * step + half runs 8 row tiles of 8 MFMAs on the B operands bf[h % 2] (row-tile-major: an A
    // fragment serves 8 MFMAs in a row and is read from LDS two fragments ahead, into a ring of four).  Behind its
    // MFMAs the wave builds its four positions' operands for half step h + 2 from the words ws[h % 2], stores them to
    // the B operand buffer xlds[h % 2] after the last row tile, and -- once every wave has done so: the barrier after
    // row tile 0 of half step h + 1 -- both waves of a pair read all eight back into bf[h % 2], which half step h has
    // just released.
    // Global loads are dealt out over the row tiles, one to three after each (a wave that issues its 26 loads of a
    // step back to back stalls on the memory pipeline's queue with its MFMAs waiting behind): the two words a row
    // tile has just consumed are re-loaded for half step h + 4 (a full step until they are used), and one eighth of
    // this wave's share of the A tile of step + 2 goes out behind row tiles 1..7 of the first half and row tile 1
    // of the second -- after the step's first barrier, which every wave reaches only when it is done with step - 1,
    // whose LDS buffer (three in rotation) this fills.  The A tile of step + 1 is complete at the second barrier of a
    // step: 23 loads have been issued since its last part (25 if the compiler puts that part in front of the two words
    // that go out behind the same row tile).  "Step + 2" is the cursor `pf`: it walks the workgroup's items end to end.
    // The wait in front of a step's second barrier is counted by hand; the count comes from the same predicates the
    // issue sites below use, so an edit that adds, drops or moves a load changes the wait with it.
    constexpr int kWaitATile = regb_loads_after_last_a_part();
    static_assert(kWaitATile == 23, "loads in flight allowed at the second barrier of a step");
    static_assert(regb_a_parts_per_step() == NDMA, "every part of the A tile is issued once per step");
    auto main_loop = [&](auto role) {
        constexpr int ROLE = decltype(role)::value;
        FragUnpack<T, ROLE> up;
        FragUnpack<T, 1 - ROLE> other;   // for the partner's position list only
        (void)other;
        up.init();
        uint32_t ws[2][8], z_n;   // words of half steps h + 2 (parity h % 2), group of the next step
        u32x4 s_n;
        u32x4 bf[2][8], af[4], own[4];
        int item = blockIdx.x;
        Item cur = decode(item);
        open_cursor(item);
        // ---- the first two steps of the run, unaided (the second may already belong to the next item) ----
        {
            uint32_t w0[8], w1[8], z;
            u32x4 sv;
#pragma unroll
            for (int i = 0; i < NDMA; ++i) dma_a_part(pf_it, 0, i);
#pragma unroll
            for (int i = 0; i < 8; ++i) w0[i] = load_word(2 * pf_it, i), w1[i] = load_word(2 * pf_it + 1, i);
            load_group(pf_grp, z, sv);
            advance();
#pragma unroll
            for (int i = 0; i < NDMA; ++i) dma_a_part(pf_it, 1, i);
#pragma unroll
            for (int i = 0; i < 8; ++i) ws[0][i] = load_word(2 * pf_it, i), ws[1][i] = load_word(2 * pf_it + 1, i);
            load_group(pf_grp, z_n, s_n);
            advance();
            unpack_all<T>(w0, z, sv, bf[0]);
            unpack_all<T>(w1, z, sv, bf[1]);
        }
        const int x_own = wave * 256 + lane, x_partner = (wave ^ 2) * 256 + lane;
        // the first half step reads the operands of the second back like any other: leave this wave's four there
#pragma unroll
        for (int i = 0; i < 4; ++i) xlds[X_SLOTS + x_own + i * 64] = bf[1][FragUnpack<T, ROLE>::own(i)];
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" ::: "memory");
        __syncthreads();
        int buf = 0;
        af[0] = lds[a_rd[0]];
        af[1] = lds[a_rd[0] + 128];
        for (;;) {
            for (int it = cur.it_begin; it < cur.it_end; ++it) {
                const int nb = buf == NBUF - 1 ? 0 : buf + 1, nnb = nb == NBUF - 1 ? 0 : nb + 1;
                const u32x4* abase = lds + buf * A_SLOTS;
                const u32x4* anext = lds + nb * A_SLOTS;
                // the operands built during this step belong to step + 1
                up.set_group(z_n, s_n);
                load_group(pf_grp, z_n, s_n);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    u32x4* xbuf = xlds + ks * X_SLOTS;
#pragma unroll
                    for (int m = 0; m < 8; ++m) {
                        const int f = ks * 8 + m;
                        // fragment f + 2, of the next step's buffer from f = 14 on
                        if (f + 2 < 16)
                            af[(f + 2) & 3] = abase[a_rd[(f + 2) >> 3] + ((f + 2) & 7) * 128];
                        else
                            af[(f + 2) & 3] = anext[a_rd[0] + (f + 2 - 16) * 128];
                        up.row_tile(m, acc[m], af[f & 3], bf[ks], ws[ks], own);
                        if (m == 0) {
                            // Every wave has stored its operands of half step h + 1 (at the end of half step h - 1; the
                            // stores completed behind row tile 0) -- and, in the second half, its part of the A tile of
                            // step + 1.  A bare barrier: __syncthreads() would also wait for this step's own loads.
                            if (ks == 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                            else asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kWaitATile) : "memory");
                            __builtin_amdgcn_s_barrier();
                            asm volatile("" ::: "memory");
                        } else if (m <= 4) {
                            // operands of half step h + 1, written at the end of half step h - 1 into the other buffer
                            const u32x4* xprev = xlds + (1 - ks) * X_SLOTS;
                            const int i = m - 1;
                            bf[1 - ks][FragUnpack<T, ROLE>::own(i)] = xprev[x_own + i * 64];
                            bf[1 - ks][FragUnpack<T, 1 - ROLE>::own(i)] = xprev[x_partner + i * 64];
                        }
                        if (regb_issues_words(m)) {
                            ws[ks][m - 1] = load_word(2 * pf_it + ks, m - 1);
                            ws[ks][m] = load_word(2 * pf_it + ks, m);
                        }
                        if (regb_issues_a_part(ks, m)) dma_a_part(pf_it, nnb, ks == 0 ? m - 1 : 7);
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) xbuf[x_own + i * 64] = own[i];
                }
                buf = nb;
                advance();
            }
            // the last MFMAs' results: 4 passes to write
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            store_item(cur);
            item += gridDim.x;
            if (item >= items) break;
            cur = decode(item);
#pragma unroll
            for (int m = 0; m < 8; ++m)
#pragma unroll
                for (int t = 0; t < 8; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if ((wave >> 1) == 0) main_loop(std::integral_constant<int, 0>{});
    else main_loop(std::integral_constant<int, 1>{});
}

template <typename T>
hipError_t launch_regb(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                       const void* bias, void* y, int M, int N, int K, int g, void* workspace, int split_k,
                       bool tail_only, hipStream_t stream, int act) {
    PipePlan plan = make_pipe_plan(M, N, K, split_k, tail_only);
    plan.act = act;
    float* partials =
        workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kCounterBytes) : nullptr;
    const size_t lds = (size_t)(3 * 8 * 256 + 2 * 4 * 4 * 64) * 16;  // 96 KiB of A tiles + 32 KiB of B operands
    auto kern = gemm_regb_kernel<T>;
    static bool raised = false;  // once per process and instantiation
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        raised = true;
    }
    (void)hipGetLastError();
    // one resident workgroup per CU (128 KiB of LDS each); the CU count is asked for once per process, of the device
    // that is current at the first launch (a larger grid on another device is still correct: the kernel strides by
    // its grid size, and workgroups beyond a device's CUs wait their turn)
    static int resident = 0;
    if (resident <= 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        resident = cus;
    }
    const int items = plan.full_tiles + plan.tail_tiles * plan.splits;
    hipLaunchKernelGGL(kern, dim3(items < resident ? items : resident), dim3(256), lds, stream,
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
