// Kernel (b): decode-regime AWQ GEMV, 1 <= M <= 16, split-K.
//
// HBM-bound: the job is to stream 0.52 B per weight and keep everything else
// off the critical path.  The contraction runs on the 16x16x32 MFMA (A = the
// <=16 activation rows, B = 16 output columns x 32 k), because even M = 2
// would saturate the vector ALUs at HBM speed.
//
// Lane roles.  A lane is (j = lane % 16, kb = lane / 16).  Per 32-row step it
// owns V packed words from each of rows k0 + 8*kb + 0..7, word columns
// (tile*16 + j)*V .. +V-1.  Those 8 rows x V words are 8V columns x 8
// consecutive k: exactly the 8 k-slots the MFMA B operand wants per lane, once
// the nibbles of two rows are paired.
//
// In-register transposition.  v_perm_b32 puts byte b of row k into the low
// half and byte b of row k+1 into the high half of one register; one
// v_and_or_b32 (after a shift for half of the nibbles) turns a nibble pair into
// two 16-bit floats whose value is c0 + c1*q, the nibble sitting in mantissa
// bits under a fixed exponent -- no int->float conversion, no LDS transpose.
//
// Scale and zero point are applied per quantisation group, in fp32, on the
// accumulator instead of per weight:
//   y += (s[g,n]/c1) * ( sum_k x[k]*(c0+c1*q[k,n])  -  (c0+c1*z[g,n]) * sum_k x[k] )
// where sum_k x[k] comes from one extra MFMA per step against a B operand of
// ones.  The products x*(c0+c1*q) are exact in the MFMA, so this differs from
// the reference's "round W to 16 bits, then multiply" only by not rounding W.
//
// Work is cut in chunks of CH steps (128 rows when the group size allows) that
// never straddle a group.  Per chunk and column pair the MFMAs of all CH steps
// chain on one accumulator, which is folded into the running fp32 result at
// once, so only 8V x 4 accumulators stay live.
//
// Two data paths feed the same arithmetic:
//   * gemv_kernel      global -> registers (optionally one chunk ahead);
//   * gemv_dma_kernel  global -> LDS by the load-to-LDS DMA (no registers held
//                      while the data is in flight), LDS -> registers just
//                      before use: one chunk per wave always in flight at a
//                      register cost that allows 4 waves per SIMD.
//
// Reduction.  Waves of a workgroup own consecutive K sub-slices and are summed
// through LDS in a fixed order; workgroups of different K-splits publish fp32
// partials and the last one to arrive (an arrival counter per tile) adds them
// in split order, so results are bit-stable run to run.
#include <cstring>
#include <type_traits>

#include <mutex>

#include "awq_common.hpp"

namespace awq {

// Nibble -> 16-bit float embeddings.  lo()/hi() take the v_perm result
// 0x00HL00HL (two rows of one byte) and return the pair of floats for the low /
// high nibble; the value is off + mul*q with the constants below.
template <typename T>
struct Embed;
template <>
struct Embed<F16> {
    // low nibble: 0x6400 | q = 1024 + q; high nibble: 0x6400 | q<<4 = 1024 + 16 q.  No shifts.
    // The 1024 offset costs ~8 of fp32's 24 bits when it is subtracted again per group
    // (|sum x*(q-z)| is ~2^-8 of |1024*sum x|), leaving ~2^-16 relative error on a group sum.
    static constexpr uint32_t kMaskLo = 0x000F000Fu, kMagicLo = 0x64006400u;
    static constexpr uint32_t kMaskHi = 0x00F000F0u, kMagicHi = 0x64006400u;
    static constexpr float kOffLo = 1024.f, kOffHi = 1024.f;
    static __device__ __forceinline__ uint32_t pre_lo(uint32_t p) { return p; }
    static __device__ __forceinline__ uint32_t pre_hi(uint32_t p) { return p; }
    static constexpr float kMulLo = 1.f, kMulHi = 16.f;
};
template <>
struct Embed<BF16> {
    // low nibble: 0x4300 | q = 128 + q; high nibble: 0x4180 | q<<3 = 16 + q
    static constexpr uint32_t kMaskLo = 0x000F000Fu, kMagicLo = 0x43004300u;
    static constexpr uint32_t kMaskHi = 0x00780078u, kMagicHi = 0x41804180u;
    static constexpr float kOffLo = 128.f, kOffHi = 16.f;
    static __device__ __forceinline__ uint32_t pre_lo(uint32_t p) { return p; }
    static __device__ __forceinline__ uint32_t pre_hi(uint32_t p) { return p >> 1; }
    static constexpr float kMulLo = 1.f, kMulHi = 1.f;
};

// (a & mask) | magic as one v_and_or_b32: gfx950's VOP3 takes no literals and a
// single scalar operand, so the mask is pinned in an SGPR and the magic in a VGPR.
struct AndOr {
    uint32_t mask, magic;
    __device__ __forceinline__ AndOr(uint32_t m, uint32_t g) : mask(m), magic(g) {
        asm volatile("" : "+s"(mask));
        asm volatile("" : "+v"(magic));
    }
    __device__ __forceinline__ uint32_t operator()(uint32_t a) const { return (a & mask) | magic; }
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

// One chunk = CH steps of 32 rows inside one quantisation group; MT tiles of 16 activation rows.
template <int V, int CH, int MT = 1>
struct Chunk {
    typename WordVec<V>::type w[CH][8];  // per step: 8 rows x V words
    u32x4 xa[CH][MT];                    // per step and m-tile: A operand x[16*mt + j][k0 + 8kb .. +7]
    typename WordVec<V>::type zw;        // V zero words of the group
    u32x4 sv[V];                         // 8 scales per word
};

// acc[mt][8V] += one chunk.  acc[mt][v*8 + c][r] is output row 16*mt + 4*kb + r, column 8*(word v) + c.
// The unpacked B fragments are built once and multiplied against every m-tile.
template <typename T, int V, int CH, int MT = 1>
__device__ __forceinline__ void compute_chunk(const Chunk<V, CH, MT>& d, f32x4 (&acc)[MT][8 * V]) {
    const u32x4 ones = u32x4{T::ones2, T::ones2, T::ones2, T::ones2};
    const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
    const AndOr emb_lo(Embed<T>::kMaskLo, Embed<T>::kMagicLo), emb_hi(Embed<T>::kMaskHi, Embed<T>::kMagicHi);
    f32x4 dones[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        dones[mt] = zero4;
#pragma unroll
        for (int s = 0; s < CH; ++s) dones[mt] = T::mfma16(d.xa[s][mt], ones, dones[mt]);
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const uint32_t zw = vget<V>(d.zw, v);
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            f32x4 dlo[MT], dhi[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) dlo[mt] = dhi[mt] = zero4;
#pragma unroll
            for (int s = 0; s < CH; ++s) {
                u32x4 flo, fhi;
#pragma unroll
                for (int rp = 0; rp < 4; ++rp) {
                    // byte b of row 2rp -> bits 0..7, byte b of row 2rp+1 -> bits 16..23
                    const uint32_t p = __builtin_amdgcn_perm(
                        vget<V>(d.w[s][2 * rp + 1], v), vget<V>(d.w[s][2 * rp], v),
                        0x0c000c00u | (uint32_t)b | ((4u + b) << 16));
                    flo[rp] = emb_lo(Embed<T>::pre_lo(p));
                    fhi[rp] = emb_hi(Embed<T>::pre_hi(p));
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    dlo[mt] = T::mfma16(d.xa[s][mt], flo, dlo[mt]);
                    dhi[mt] = T::mfma16(d.xa[s][mt], fhi, dhi[mt]);
                }
            }
            // byte b holds column {0,4,1,5}[b] in its low and {2,6,3,7}[b] in its high nibble
            constexpr int kLoCol[4] = {0, 4, 1, 5}, kHiCol[4] = {2, 6, 3, 7};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int c = h ? kHiCol[b] : kLoCol[b];
                const float mul = h ? Embed<T>::kMulHi : Embed<T>::kMulLo;
                const float off = h ? Embed<T>::kOffHi : Embed<T>::kOffLo;
                // value of the embedded zero point, off + mul*z, and the scale / mul
                const float zf = (float)((zw >> nibble_shift(c)) & 0xFu) * mul + off;
                const uint32_t pair = d.sv[v][c >> 1];
                const float sc = T::to_f32((uint16_t)((c & 1) ? (pair >> 16) : (pair & 0xFFFFu))) * (1.f / mul);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const f32x4 dq = h ? dhi[mt] : dlo[mt];
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[mt][v * 8 + c][r] += sc * (dq[r] - zf * dones[mt][r]);
                }
            }
        }
    }
}

// The same for two of the four bytes of every word (bytes 2*BH and 2*BH + 1, i.e. the even output columns of
// a word for BH = 0 and the odd ones for BH = 1): acc[mt][2*bi + h][r] is output row 16*mt + 4*kb + r,
// column {0,2,4,6}[2*bi + h] + BH of the lane's word.  Two waves, one per half, split a column tile without
// unpacking anything twice.
template <typename T, int CH, int MT, int BH>
__device__ __forceinline__ void compute_chunk_bytes(const Chunk<1, CH, MT>& d, f32x4 (&acc)[MT][4]) {
    const u32x4 ones = u32x4{T::ones2, T::ones2, T::ones2, T::ones2};
    const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
    const AndOr emb_lo(Embed<T>::kMaskLo, Embed<T>::kMagicLo), emb_hi(Embed<T>::kMaskHi, Embed<T>::kMagicHi);
    f32x4 dones[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        dones[mt] = zero4;
#pragma unroll
        for (int s = 0; s < CH; ++s) dones[mt] = T::mfma16(d.xa[s][mt], ones, dones[mt]);
    }
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) {
        constexpr int kLoCol[4] = {0, 4, 1, 5}, kHiCol[4] = {2, 6, 3, 7};
        const int b = 2 * BH + bi;
        f32x4 dlo[MT], dhi[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) dlo[mt] = dhi[mt] = zero4;
#pragma unroll
        for (int s = 0; s < CH; ++s) {
            u32x4 flo, fhi;
#pragma unroll
            for (int rp = 0; rp < 4; ++rp) {
                const uint32_t p = __builtin_amdgcn_perm(d.w[s][2 * rp + 1], d.w[s][2 * rp],
                                                         0x0c000c00u | (uint32_t)b | ((4u + b) << 16));
                flo[rp] = emb_lo(Embed<T>::pre_lo(p));
                fhi[rp] = emb_hi(Embed<T>::pre_hi(p));
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                dlo[mt] = T::mfma16(d.xa[s][mt], flo, dlo[mt]);
                dhi[mt] = T::mfma16(d.xa[s][mt], fhi, dhi[mt]);
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int c = h ? kHiCol[b] : kLoCol[b];
            const float mul = h ? Embed<T>::kMulHi : Embed<T>::kMulLo;
            const float off = h ? Embed<T>::kOffHi : Embed<T>::kOffLo;
            const float zf = (float)((d.zw >> nibble_shift(c)) & 0xFu) * mul + off;
            const uint32_t pair = d.sv[0][c >> 1];
            const float sc = T::to_f32((uint16_t)((c & 1) ? (pair >> 16) : (pair & 0xFFFFu))) * (1.f / mul);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const f32x4 dq = h ? dhi[mt] : dlo[mt];
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[mt][2 * bi + h][r] += sc * (dq[r] - zf * dones[mt][r]);
            }
        }
    }
}

// compute_chunk for one word column and one m-tile, one 32-row step at a time: the same MFMA chains and the same
// fold, so the same bits, but a caller can start on step 0 while the rows of steps 1..3 are still on their way.
// d[2*b + h] is the running product of byte b's low (h = 0) / high (h = 1) nibble column, dones the row sums.
struct StepAcc {
    f32x4 d[8];
    f32x4 dones;
};
// kFirst: the first step of a chunk; the MFMAs start from a literal zero, so `a` need not be cleared
template <typename T, bool kFirst = false>
__device__ __forceinline__ void compute_step(const uint32_t (&w)[8], u32x4 xa, StepAcc& a, const AndOr& emb_lo,
                                             const AndOr& emb_hi) {
    const u32x4 ones = u32x4{T::ones2, T::ones2, T::ones2, T::ones2};
    const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
    a.dones = T::mfma16(xa, ones, kFirst ? zero4 : a.dones);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        u32x4 flo, fhi;
#pragma unroll
        for (int rp = 0; rp < 4; ++rp) {
            const uint32_t p = __builtin_amdgcn_perm(w[2 * rp + 1], w[2 * rp],
                                                     0x0c000c00u | (uint32_t)b | ((4u + b) << 16));
            flo[rp] = emb_lo(Embed<T>::pre_lo(p));
            fhi[rp] = emb_hi(Embed<T>::pre_hi(p));
        }
        a.d[2 * b] = T::mfma16(xa, flo, kFirst ? zero4 : a.d[2 * b]);
        a.d[2 * b + 1] = T::mfma16(xa, fhi, kFirst ? zero4 : a.d[2 * b + 1]);
    }
}
// kFirst: acc is known to be zero (nothing was folded into it yet) and need not be live before this call
template <typename T, bool kFirst = false>
__device__ __forceinline__ void fold_steps(const StepAcc& a, uint32_t zw, u32x4 sv, f32x4 (&acc)[8]) {
    constexpr int kLoCol[4] = {0, 4, 1, 5}, kHiCol[4] = {2, 6, 3, 7};
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int c = h ? kHiCol[b] : kLoCol[b];
            const float mul = h ? Embed<T>::kMulHi : Embed<T>::kMulLo;
            const float off = h ? Embed<T>::kOffHi : Embed<T>::kOffLo;
            const float zf = (float)((zw >> nibble_shift(c)) & 0xFu) * mul + off;
            const uint32_t pair = sv[c >> 1];
            const float sc = T::to_f32((uint16_t)((c & 1) ? (pair >> 16) : (pair & 0xFFFFu))) * (1.f / mul);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float t = sc * (a.d[2 * b + h][r] - zf * a.dones[r]);
                acc[c][r] = kFirst ? 0.f + t : acc[c][r] + t;   // 0 + t: the bits of the running sum (a -0 becomes +0)
            }
        }
}

// A workgroup is WN x WK waves: wave w works on column tile (group*WN + w % WN)
// and K sub-slice w / WN.  Sum the WK waves of each column tile through LDS
// (fixed order), then either store y (splits == 1) or publish this split's
// partial and let the last workgroup of the tile group add the partials in
// split order.  `group` is the workgroup's index along N.
// Gated epilogue: the N columns are word-interleaved (word 2t = 8 gate columns, word 2t+1 = the 8 up
// columns of the same outputs), a lane holds one word of a row, its neighbour (lane ^ 1) the partner
// word.  out = dtype(SiLU(dtype(gate))) * dtype(up), written to y [M, N/2] by the gate lanes.  Every lane
// of a pair must call this (the exchange is a cross-lane read).
// Epilogue of the fused q|k|v projection of a decode step (act == 2): the 128 columns of a column tile are one
// head (head_dim 128).  q and k heads: RMSNorm over the head, half-split rotary at the row's position; q goes
// to q_out, k to its paged-cache slot; v heads are written to their cache slot as they are.  The arithmetic per
// element is that of the stand-alone kernel behind nq_qk_norm_rope_store (the GEMV's fp32 sum is rounded to T first,
// as a separate projection would round it).  Cache layout [blocks][kv heads][block_size][128].
struct QkvEpilogue {
    const uint16_t* q_weight;
    const uint16_t* k_weight;
    const float* cos_sin;        // [max_positions][128]: 64 cosines, then 64 sines
    const int64_t* positions;    // [M]
    const int64_t* slots;        // [M], negative = the row owns no cache slot
    uint16_t* q_out;             // [M][nh][128]
    uint16_t* k_cache;
    uint16_t* v_cache;
    int nh, nkv, max_positions, block_size;
    int64_t num_slots;
    float eps;
};

// The 16 lanes that hold the 16 words of (row m, head n0 / 128) call this together; `valid` masks the stores.
template <typename T>
__device__ __forceinline__ void qkv_rope_store(const float (&out)[8], int m, size_t n0, bool valid,
                                               const QkvEpilogue& qe) {
    const int head = (int)(n0 >> 7), dc = (int)((n0 & 127) >> 3);
    const int row = valid ? m : 0;
    float a[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = T::to_f32(T::from_f32(out[e]));
    const int64_t slot = qe.slots[row];
    const bool slot_ok = slot >= 0 && slot < qe.num_slots;
    const bool is_q = head < qe.nh, is_k = !is_q && head < qe.nh + qe.nkv;
    if (!is_q && !is_k) {   // v (uniform over the 16 lanes: no shuffle below is reached by a partial group)
        if (valid && slot_ok) {
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = T::pack2(a[2 * i], a[2 * i + 1]);
            *reinterpret_cast<u32x4*>(qe.v_cache + (((slot / qe.block_size) * qe.nkv + (head - qe.nh - qe.nkv)) *
                                                        qe.block_size + slot % qe.block_size) * 128 + dc * 8) = o;
        }
        return;
    }
    const uint16_t* w = is_q ? qe.q_weight : qe.k_weight;
    const u32x4 wraw = *reinterpret_cast<const u32x4*>(w + dc * 8);
    int64_t pos = qe.positions[row];
    pos = pos < 0 ? 0 : (pos >= qe.max_positions ? qe.max_positions - 1 : pos);
    const int i0 = (dc & 7) * 8;
    const float* cs = qe.cos_sin + pos * 128;
    const f32x4 c0 = *reinterpret_cast<const f32x4*>(cs + i0), c1 = *reinterpret_cast<const f32x4*>(cs + i0 + 4);
    const f32x4 s0 = *reinterpret_cast<const f32x4*>(cs + 64 + i0), s1 = *reinterpret_cast<const f32x4*>(cs + 64 + i0 + 4);
    const float ss = tile_ssq(a);
    const float r = rsqrtf(ss / 128.f + qe.eps);
    const bool first = dc < 8;
    uint32_t packed[4];
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float wf = T::to_f32((uint16_t)((e & 1) ? wraw[e >> 1] >> 16 : wraw[e >> 1] & 0xFFFFu));
        const float xn = T::to_f32(T::from_f32(mul_round<T>(a[e], r) * wf));
        const float other = __shfl_xor(xn, 8);
        const float cc = e < 4 ? c0[e] : c1[e - 4], sn = e < 4 ? s0[e] : s1[e - 4];
        const float x1 = first ? xn : other, x2 = first ? other : xn;
        y[e] = as_f32_result(first ? __fsub_rn(__fmul_rn(x1, cc), __fmul_rn(x2, sn))
                                   : __fadd_rn(__fmul_rn(x1, sn), __fmul_rn(x2, cc)));
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) packed[i] = T::pack2(y[2 * i], y[2 * i + 1]);
    const u32x4 o = u32x4{packed[0], packed[1], packed[2], packed[3]};
    if (!valid) return;
    if (is_q) {
        *reinterpret_cast<u32x4*>(qe.q_out + ((int64_t)m * qe.nh + head) * 128 + dc * 8) = o;
    } else if (slot_ok) {
        *reinterpret_cast<u32x4*>(qe.k_cache + (((slot / qe.block_size) * qe.nkv + (head - qe.nh)) * qe.block_size +
                                                slot % qe.block_size) * 128 + dc * 8) = o;
    }
}

template <typename T>
__device__ __forceinline__ void swiglu_store(const float (&out)[8], uint16_t* __restrict__ y, int m, int N,
                                             size_t n0) {
    float other[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) other[c] = __shfl_xor(out[c], 1);
    if (((n0 >> 3) & 1) == 0) {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float r[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float g = T::to_f32(T::from_f32(out[2 * i + h]));
                const float u = T::to_f32(T::from_f32(other[2 * i + h]));
                r[h] = T::to_f32(T::from_f32(g / (1.f + __expf(-g)))) * u;
            }
            o[i] = T::pack2(r[0], r[1]);
        }
        *reinterpret_cast<u32x4*>(y + (size_t)m * (N >> 1) + (n0 >> 1)) = o;
    }
}

// Residual epilogue (the o_proj / down_proj of a decode step): the product is added to the residual stream in
// place, residual = T(residual + T(product)) -- the two roundings of a separate linear followed by an addition --
// and the sum of squares of the new residual over the workgroup's 128 columns goes to ssq[tile][row], so that the
// next GEMV can apply the RMSNorm of its input without a pass over the row.  The order of that sum is fixed: a
// lane adds its 8 squares in column order (fused multiply-add), the 16 lanes of a tile combine by xor 8, 4, 2, 1.
struct ResidEpilogue {
    float* ssq;      // [N / 128][m_stride]
    int m_stride;    // rows of the whole launch
};

// RMSNorm of the GEMV's input applied on the way into the MFMA operand: h = T(T(x * r) * weight), with
// r = rsqrt(sum over tiles of ssq[tile][row] / K + eps), the tiles added in index order.
struct NormPrologue {
    const uint16_t* weight;   // [K]
    const float* ssq;         // [K / 128][m_stride]
    int m_stride;
    float eps;
};

// The 16 lanes that hold the 16 words of (row m, column tile n0 / 128) call this together; `valid` masks the stores.
// `rv` = the 8 residual values at (m, n0), loaded by the caller ahead of time (residual_load) so that their latency
// hides behind the reduction.
__device__ __forceinline__ u32x4 residual_load(const uint16_t* __restrict__ y, int m, int N, size_t n0, bool valid) {
    return *reinterpret_cast<const u32x4*>(y + (size_t)(valid ? m : 0) * N + (valid ? n0 : 0));
}
template <typename T>
__device__ __forceinline__ void residual_store(const float (&out)[8], u32x4 rv, uint16_t* __restrict__ y, int m, int N,
                                               size_t n0, bool valid, const ResidEpilogue& re) {
    float xn[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float xr = T::to_f32((uint16_t)((e & 1) ? rv[e >> 1] >> 16 : rv[e >> 1] & 0xFFFFu));
        xn[e] = T::to_f32(T::from_f32(xr + T::to_f32(T::from_f32(out[e]))));
    }
    const float ss = tile_ssq(xn);
    if (!valid) return;
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = T::pack2(xn[2 * i], xn[2 * i + 1]);
    *reinterpret_cast<u32x4*>(y + (size_t)m * N + n0) = o;
    if (((n0 >> 3) & 15) == 0) re.ssq[(n0 >> 7) * re.m_stride + m] = ss;
}

// What a kernel's epilogue may need beyond y: kEpi 0 nothing, 1 the q|k|v epilogue, 2 the residual epilogue.
struct EpiArgs {
    const QkvEpilogue* qe = nullptr;
    const ResidEpilogue* re = nullptr;
};

// Host side: the optional parts of a launch of the staged kernel (at most one epilogue; the prologue combines
// with none or with the q|k|v epilogue).
// The second pass of a K-split shared-chunk GEMV as residual add + RMSNorm: y of the GEMV is the residual stream
// (updated in place), `normed` receives RMSNorm(residual) * weight.
struct AddNorm {
    const uint16_t* weight;
    uint16_t* normed;
    float eps;
};
struct GemvFusion {
    const QkvEpilogue* qe = nullptr;
    const NormPrologue* np = nullptr;
    const ResidEpilogue* re = nullptr;
    const AddNorm* an = nullptr;
    bool any() const { return qe || np || re; }
};

// kPlain: the partials are read by a later kernel, not by a concurrent workgroup: ordinary stores do.
template <typename T, int V, int WN, int WK, bool kPlain = false, int kEpi = 0>
__device__ __forceinline__ void gemv_reduce_store(f32x4 (&acc)[8 * V], int m_base, float* red, int lane,
                                                  int wave, int group, int split, int splits,
                                                  const uint16_t* __restrict__ bias,
                                                  uint16_t* __restrict__ y, float* __restrict__ partials,
                                                  int M, int N, int act, EpiArgs ea = EpiArgs{}) {
    constexpr int NF = 8 * V, NQ = 4 * V;
    const int j = lane & 15, kb = lane >> 4;
    const int words = N >> 3;
    const int wn = wave % WN, wk = wave / WN;
    const int wv_col = (group * WN + wn) * 16 + j;  // this lane's column, in units of V words
    const bool col_ok = wv_col * V < words;
    // slot q = v*4 + r holds 8 consecutive output columns of row m_base + 4*kb + r
    u32x4 rv_pre = u32x4{0u, 0u, 0u, 0u};
    if constexpr (kEpi == 2) {   // a wave stores at most one slot (q = wk): fetch its residual before the reduction
        static_assert(V == 1 && WK >= 4, "residual epilogue: one slot per wave");
        if (splits == 1 && wk < NQ)
            rv_pre = residual_load(y, m_base + 4 * kb + wk, N, (size_t)wv_col * 8, m_base + 4 * kb + wk < M && col_ok);
    }
    // rows m_base + 4*kb + r with r >= r_lim exist for no kb: with fewer than 4 rows their slots are neither
    // written nor summed (a quarter of the LDS traffic at one row)
    const int r_lim = M - m_base < 4 ? M - m_base : 4;
    if constexpr (WK > 1) {
        float* mine = red + (size_t)wave * (NF * 4 * 64);
#pragma unroll
        for (int v = 0; v < V; ++v)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (r < r_lim) {
#pragma unroll
                    for (int c = 0; c < 8; ++c) mine[((v * 4 + r) * 8 + c) * 64 + lane] = acc[v * 8 + c][r];
                }
        __syncthreads();
    }
    for (int q = wk; q < NQ; q += WK) {
        const int v = q >> 2, r = q & 3;
        if (r >= r_lim) continue;   // uniform
        const int m = m_base + 4 * kb + r;
        float out[8];
        if constexpr (WK > 1) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < WK; ++w)
                    s += red[(size_t)(w * WN + wn) * (NF * 4 * 64) + (q * 8 + c) * 64 + lane];
                out[c] = s;
            }
        } else {
            // one wave per column tile: q runs over every slot; pick from registers
#pragma unroll
            for (int vv = 0; vv < V; ++vv)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr)
                    if (vv == v && rr == r)
#pragma unroll
                        for (int c = 0; c < 8; ++c) out[c] = acc[vv * 8 + c][rr];
        }
        if constexpr (kEpi != 0) {
            if (splits == 1) {   // every lane takes part (cross-lane sums); the stores are masked
                if constexpr (kEpi == 1)
                    qkv_rope_store<T>(out, m, ((size_t)wv_col * V + v) * 8, m < M && col_ok, *ea.qe);
                else
                    residual_store<T>(out, rv_pre, y, m, N, ((size_t)wv_col * V + v) * 8, m < M && col_ok, *ea.re);
                continue;
            }
        }
        if (m < M && col_ok) {
            const size_t n0 = ((size_t)wv_col * V + v) * 8;
            if (splits == 1 && act) {
                swiglu_store<T>(out, y, m, N, n0);
            } else if (splits == 1) {
                if (bias) {
                    const u32x4 bv = *reinterpret_cast<const u32x4*>(bias + n0);
#pragma unroll
                    for (int c = 0; c < 8; ++c)
                        out[c] = add_bias<T>(out[c], T::to_f32((uint16_t)((c & 1) ? (bv[c >> 1] >> 16) : (bv[c >> 1] & 0xFFFFu))));
                }
                u32x4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = T::pack2(out[2 * i], out[2 * i + 1]);
                *reinterpret_cast<u32x4*>(y + (size_t)m * N + n0) = o;
            } else {
                float* p = partials + ((size_t)split * M + m) * N + n0;
                if constexpr (kPlain) {
                    *reinterpret_cast<f32x4*>(p) = f32x4{out[0], out[1], out[2], out[3]};
                    *reinterpret_cast<f32x4*>(p + 4) = f32x4{out[4], out[5], out[6], out[7]};
                } else {
                    publish_f32x4(p, f32x4{out[0], out[1], out[2], out[3]});
                    publish_f32x4(p + 4, f32x4{out[4], out[5], out[6], out[7]});
                }
            }
        }
    }
}

// out += partials of splits first .. splits - 1 at (row m, columns n0 .. n0 + 7), in split order; eight splits (two
// 16-byte loads each) in flight at a time.
__device__ __forceinline__ void add_split_partials(float (&out)[8], const float* __restrict__ partials, int first,
                                                   int splits, int M, int m, int N, size_t n0) {
    for (int s0 = first; s0 < splits; s0 += 8) {
        f32x4 lo[8], hi[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int s = min(s0 + u, splits - 1);
            const float* p = partials + ((size_t)s * M + m) * N + n0;
            lo[u] = fetch_f32x4_nowait(p);
            hi[u] = fetch_f32x4_nowait(p + 4);
        }
        fetch_wait(lo, hi);
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (s0 + u < splits) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    out[c] += lo[u][c];
                    out[4 + c] += hi[u][c];
                }
            }
    }
}

__device__ __forceinline__ void fetch_wait4(f32x4 (&a)[4], f32x4 (&b)[4]) {
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3])
                 :
                 : "memory");
}

// The last workgroup to arrive at a tile adds the partials of all splits, in split order, and stores y.
// An item is one word (8 columns) of one row.  With at least half as many items as threads, a thread owns an item
// and walks the splits itself, eight in flight.  With fewer (up to 8 rows of a 128-column tile in a workgroup of four
// waves) that would leave most threads idle behind one memory round trip per eight splits -- 32 splits at one row:
// four round trips in a row, 13.7 us for a launch that takes 10.3 with 8 splits --, so there the threads share the
// fetch: thread (g, item) brings splits g, g + G, ... (up to four per round, G = threads / items), stages them in LDS
// (`red`: 128 bytes per thread at least, free by now), and the item's thread adds them from there in split order:
// one round trip for up to 4 * G splits, and the same bits, since the order of the additions is the same.
template <typename T, int V, int WN, int WK, int kEpi = 0>
__device__ __forceinline__ void gemv_split_tail(float* red, int* s_last, int group, int splits,
                                                const uint16_t* __restrict__ bias,
                                                uint16_t* __restrict__ y, float* __restrict__ partials,
                                                int* __restrict__ counters, int M, int N, int act,
                                                EpiArgs ea = EpiArgs{}) {
    constexpr int WAVES = WN * WK, NT = 64 * WAVES;
    const int words = N >> 3;
    if (!arrive_last(&counters[group], splits, s_last)) return;
    const int group_words = 16 * V * WN;
    const int w_begin = group * group_words;
    const int w_count = min(group_words, words - w_begin);
    const int items = M * w_count;
    const bool shared_fetch = WAVES > 1 && items * 2 <= NT && splits > 1;   // uniform
    const int G = shared_fetch ? NT / items : 1;
    for (int i0 = 0; i0 < items; i0 += NT) {
        const int idx = i0 + (int)threadIdx.x;
        const bool owner = idx < items;
        const int m = owner ? idx / w_count : 0, wc = owner ? idx - m * w_count : 0;
        const size_t n0 = (size_t)(w_begin + wc) * 8;
        float out[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        u32x4 rv = u32x4{0u, 0u, 0u, 0u};
        if constexpr (kEpi == 2) {
            if (owner) rv = residual_load(y, m, N, n0, true);   // in flight beside the partials
        }
        if (shared_fetch) {
            // (items <= NT / 2: a single pass of the outer loop)
            const int g = (int)threadIdx.x / items, it = (int)threadIdx.x - g * items;
            const int fm = it / w_count;
            const size_t fn0 = (size_t)(w_begin + (it - fm * w_count)) * 8;
            const bool fetcher = g < G;
            f32x4* stage = reinterpret_cast<f32x4*>(red);   // [split of the round][item][2]
            for (int s0 = 0; s0 < splits; s0 += 4 * G) {
                const int ns = min(4 * G, splits - s0);
                f32x4 lo[4], hi[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    lo[u] = hi[u] = f32x4{0.f, 0.f, 0.f, 0.f};
                    const int sr = g + u * G;   // split of this round
                    if (fetcher && sr < ns) {
                        const float* p = partials + ((size_t)(s0 + sr) * M + fm) * N + fn0;
                        lo[u] = fetch_f32x4_nowait(p);
                        hi[u] = fetch_f32x4_nowait(p + 4);
                    }
                }
                fetch_wait4(lo, hi);
                if (s0 > 0) __syncthreads();   // the previous round has been added
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int sr = g + u * G;
                    if (fetcher && sr < ns) {
                        stage[(sr * items + it) * 2] = lo[u];
                        stage[(sr * items + it) * 2 + 1] = hi[u];
                    }
                }
                __syncthreads();
                if (owner) {
                    for (int sr = 0; sr < ns; ++sr) {
                        const f32x4 a = stage[(sr * items + idx) * 2], b = stage[(sr * items + idx) * 2 + 1];
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            out[c] += a[c];
                            out[4 + c] += b[c];
                        }
                    }
                }
            }
        } else if (owner) {
            add_split_partials(out, partials, 0, splits, M, m, N, n0);
        }
        if (!owner) continue;   // whole groups of 16 lanes (an item count is a multiple of 16 wherever lanes exchange)
        if constexpr (kEpi == 1) {   // w_count == 16 here: the 16 lanes of a head run the same iterations
            qkv_rope_store<T>(out, m, n0, true, *ea.qe);
            continue;
        }
        if constexpr (kEpi == 2) {   // likewise: 16 lanes per row and column tile
            residual_store<T>(out, rv, y, m, N, n0, true, *ea.re);
            continue;
        }
        if (act) {   // w_count is even here: a gate word and its up word sit in neighbouring lanes
            swiglu_store<T>(out, y, m, N, n0);
            continue;
        }
        if (bias) {
            const u32x4 bv = *reinterpret_cast<const u32x4*>(bias + n0);
#pragma unroll
            for (int c = 0; c < 8; ++c)
                out[c] = add_bias<T>(out[c], T::to_f32((uint16_t)((c & 1) ? (bv[c >> 1] >> 16) : (bv[c >> 1] & 0xFFFFu))));
        }
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = T::pack2(out[2 * i], out[2 * i + 1]);
        *reinterpret_cast<u32x4*>(y + (size_t)m * N + n0) = o;
    }
    if (threadIdx.x == 0) __hip_atomic_store(&counters[group], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A workgroup is WN x WK waves: wave w works on column tile (group*WN + w % WN)
// and K sub-slice w / WN.  Sum the WK waves of each column tile through LDS
// (fixed order), then either store y (splits == 1) or publish this split's
// partial and let the last workgroup of the tile group add the partials in
// split order.  `group` is the workgroup's index along N.
template <typename T, int V, int WN, int WK, int MT = 1, int kEpi = 0>
__device__ __forceinline__ void gemv_epilogue(f32x4 (&acc)[MT][8 * V], float* red, int* s_last, int lane,
                                              int wave, int group, int split, int splits,
                                              const uint16_t* __restrict__ bias,
                                              uint16_t* __restrict__ y, float* __restrict__ partials,
                                              int* __restrict__ counters, int M, int N, int act = 0,
                                              EpiArgs ea = EpiArgs{}) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (mt > 0) {
            if (16 * mt >= M) break;  // uniform
            __syncthreads();          // the reduction buffer is reused per m-tile
        }
        gemv_reduce_store<T, V, WN, WK, false, kEpi>(acc[mt], 16 * mt, red, lane, wave, group, split, splits, bias,
                                                     y, partials, M, N, act, ea);
    }
    if (splits == 1) return;
    gemv_split_tail<T, V, WN, WK, kEpi>(red, s_last, group, splits, bias, y, partials, counters, M, N, act, ea);
}

// Workgroups are dealt to the 8 XCDs round-robin; give each XCD a contiguous run
// of column groups so that neighbouring groups share an L2.
__device__ __forceinline__ int xcd_aware_group(int bid, int ngroups) {
    if ((ngroups & 7) != 0) return bid;
    return (bid & 7) * (ngroups >> 3) + (bid >> 3);
}

// ---- data path 1: global -> registers ------------------------------------------
template <typename T, int V, int WAVES, int CH, bool PF>
__global__ __launch_bounds__(64 * WAVES) void gemv_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, float* __restrict__ partials,
    int* __restrict__ counters, int M, int N, int K, int chunks_per_group, int chunks_per_split,
    int splits) {
    using WV = typename WordVec<V>::type;
    constexpr int NF = 8 * V;  // column fragments per lane
    extern __shared__ __attribute__((aligned(16))) float red[];  // [WAVES][NF*4][64]
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

    const WV* wbase = reinterpret_cast<const WV*>(qweight);
    const WV* zbase = reinterpret_cast<const WV*>(qzeros);
    const u32x4* sbase = reinterpret_cast<const u32x4*>(scales);
    // per-lane element offsets, 32-bit so that loads can use scalar base + vector offset
    uint32_t woff[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) woff[r] = (uint32_t)(kb * 8 + r) * (uint32_t)wstride + (uint32_t)wv_ld;
    const uint32_t xoff = (uint32_t)xrow * (uint32_t)K + (uint32_t)kb * 8u;

    f32x4 acc[1][NF];
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[0][f] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load_chunk = [&](int c, Chunk<V, CH>& d) {
        const int row0 = c * (32 * CH);  // wave-uniform
#pragma unroll
        for (int s = 0; s < CH; ++s) {
            const WV* wp = wbase + (size_t)(row0 + s * 32) * wstride;  // uniform
#pragma unroll
            for (int r = 0; r < 8; ++r) d.w[s][r] = wp[woff[r]];
        }
#pragma unroll
        for (int s = 0; s < CH; ++s) d.xa[s][0] = *reinterpret_cast<const u32x4*>(x + (row0 + s * 32) + xoff);
        const int gi = chunks_per_group == 1 ? c : c / chunks_per_group;
        d.zw = (zbase + (size_t)gi * wstride)[wv_ld];
#pragma unroll
        for (int v = 0; v < V; ++v) d.sv[v] = (sbase + (size_t)gi * words)[wv_ld * V + v];
    };

    if constexpr (PF) {
        Chunk<V, CH> a, b;
        if (c0 < c1) load_chunk(c0, a);
        for (int c = c0; c < c1; c += 2) {
            if (c + 1 < c1) load_chunk(c + 1, b);
            compute_chunk<T, V, CH>(a, acc);
            if (c + 1 < c1) {
                if (c + 2 < c1) load_chunk(c + 2, a);
                compute_chunk<T, V, CH>(b, acc);
            }
        }
    } else {
        Chunk<V, CH> a;
        for (int c = c0; c < c1; ++c) {
            load_chunk(c, a);
            compute_chunk<T, V, CH>(a, acc);
        }
    }
    gemv_epilogue<T, V, 1, WAVES>(acc, red, &s_last, lane, wave, tile, split, splits, bias, y, partials,
                                  counters, M, N);
}

// ---- data path 2: global -> LDS (DMA) -> registers -----------------------------
// V = 1, CH = 4.  Needs N % 128 == 0 and a group size that is a multiple of 128.
//
// Per wave and chunk the LDS holds
//   W  4 steps x 32 slots x 64 B   slot r*4 + kb' = row 8*kb' + r of the step, 16 words wide;
//                                  the DMA lane (slot%16 = lane/4, quarter = lane%4) brings 16 B;
//                                  the compute lane (j, kb) reads word j of slots r*4 + kb:
//                                  64 lanes hit 64 different banks
//   X  4 steps x M x 64 B          A operand, row m, 4 k-blocks of 16 B
//   ZS 16 zero words + 16 x 8 scales
#define AWQ_GPTR(p) ((__attribute__((address_space(1))) const void*)(p))
#define AWQ_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

__host__ __device__ constexpr int dma_wave_bytes(int M) { return 8192 + 256 * M + 512; }

// Forms of the staged kernel (MODE): bit 0 the q|k|v epilogue, bit 1 the RMSNorm prologue, bit 2 the residual
// epilogue.  The extra arguments of a form stay out of the plain kernel's argument block (the launch-bound decode
// GEMVs measured 0.2-0.5 us slower with them).
constexpr int kModeQkv = 1, kModeNorm = 2, kModeResid = 4;
// the step-by-step form takes the RMSNorm prologue for inputs of up to this many 128-column tiles (K <= 2048)
constexpr int kNormStreamChunks = 16;
template <int MODE>
struct GemvExtra {};
template <>
struct GemvExtra<kModeQkv> { QkvEpilogue qe; };
template <>
struct GemvExtra<kModeNorm> { NormPrologue np; };
template <>
struct GemvExtra<kModeQkv | kModeNorm> { QkvEpilogue qe; NormPrologue np; };
template <>
struct GemvExtra<kModeResid> { ResidEpilogue re; };

// STREAM: every wave has at most one chunk (decode-size launches) and takes it step by step as it lands; a form of
// its own because it needs a dozen registers more than the 128 that let four waves of the other form share a SIMD.
template <typename T, int WK, int MODE = 0, bool STREAM = false>
__global__ __launch_bounds__(64 * WK) void gemv_dma_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, float* __restrict__ partials,
    int* __restrict__ counters, int M, int N, int K, int chunks_per_group, int chunks_per_split,
    int splits, int act, int groups, int pair_map, PrefetchRegions pf, GemvExtra<MODE> ex) {
    constexpr bool QKV = (MODE & kModeQkv) != 0, NORM = (MODE & kModeNorm) != 0, RESID = (MODE & kModeResid) != 0;
    constexpr int CH = 4;
    // 16-byte aligned: the dynamic segment starts behind the static one (s_last, 4 bytes), and at the array's
    // natural 4-byte alignment every 16-byte LDS read and DMA destination below would straddle (measured: 8-10 % of a
    // decode-size launch, 2.8 x on a kernel that lives on 16-byte LDS reads)
    extern __shared__ __attribute__((aligned(16))) float red[];  // staging while streaming, [WK][32][64] floats afterwards
    __shared__ int s_last;
    // Every argument the compute path needs, fetched now in one batch of scalar loads: left alone the compiler
    // fetches them where they are first used, three round trips to the kernel-argument segment one behind the other
    // in front of the first weight load.
    asm volatile("" ::"s"(x), "s"(qweight), "s"(scales), "s"(qzeros), "s"(y), "s"(partials), "s"(counters), "s"(M),
                 "s"(N), "s"(K), "s"(chunks_per_group), "s"(chunks_per_split), "s"(splits), "s"(groups));
    // Which column tile this workgroup owns.  Workgroups go to the 8 XCDs by linear index mod 8, and two neighbouring
    // tiles share every 128-byte line of the weights (a tile's row piece is 64 bytes): the two must sit behind the
    // same L2, or each line is fetched from the fabric twice.  With a multiple of 16 tiles every XCD gets a run of
    // consecutive tiles.  Otherwise (8 or 24 tiles on the decode shapes) the grid is padded to a multiple of 16 and
    // dealt in pairs: workgroups x and x + 8 (same XCD) own tiles 2p and 2p + 1 of pair p = 8 * (slot / 2) + x % 8;
    // the indices past the last tile are the spare workgroups.
    int tile_of_wg;
    if (pair_map) {
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        tile_of_wg = 2 * ((slot >> 1) * 8 + xcd) + (slot & 1);
    } else {
        tile_of_wg = (int)blockIdx.x < groups ? xcd_aware_group(blockIdx.x, groups) : (int)blockIdx.x;
    }
    if (tile_of_wg >= groups) {
        if (blockIdx.y != 0 || blockIdx.z != 0) return;   // the extra workgroups exist once per split and row block; one set works
        // Prefetch workgroups (launched beside the compute grid on CUs a small GEMV leaves idle): touch one
        // dword of every 128-byte line of the hinted regions -- the packed weights, scales and zeros of the
        // NEXT launch -- so that it finds them in the Infinity Cache instead of HBM.
        if (pf.count == 0) return;
        const long long nthreads = (long long)(gridDim.x - groups) * blockDim.x;
        const long long tid = (long long)(tile_of_wg - groups) * blockDim.x + threadIdx.x;
        uint32_t sink = 0;
        for (int r = 0; r < pf.count; ++r) {
            const long long lines = pf.bytes[r] >> 7;
            // four independent loads in flight per thread and round: issued as assembly and waited for once (as
            // volatile accesses the compiler waits after each of them: four memory round trips in a row, which made
            // the prefetch workgroups the last to finish)
            for (long long l = tid; l < lines; l += 4 * nthreads) {
                uint32_t v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const long long lu = l + u * nthreads;
                    const char* addr = pf.ptr[r] + ((lu < lines ? lu : l) << 7);
                    asm volatile("global_load_dword %0, %1, off" : "=v"(v[u]) : "v"(addr) : "memory");
                }
                asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : : "memory");
                sink ^= v[0] ^ v[1] ^ v[2] ^ v[3];
            }
        }
        if (sink == 0x9e3779b9u && pf.count < 0) counters[0] = 0;   // never true: keeps the loads alive
        return;
    }

    {
        // More than 16 rows: blockIdx.z picks a block of 16 rows, an independent product with its own slice of
        // x, y, the partials and the arrival counters.  The weights are then read once per row block, the
        // later ones mostly from cache: worthwhile where a launch is latency-bound, not on large weights.
        const int rb = blockIdx.z;
        x += (size_t)rb * 16 * K;
        y += (size_t)rb * 16 * (act == 1 ? N >> 1 : N);
        partials += (size_t)rb * splits * 16 * N;
        counters += rb * groups;
        M = min(16, M - 16 * rb);
        if constexpr (QKV) {
            ex.qe.positions += rb * 16;
            ex.qe.slots += rb * 16;
            ex.qe.q_out += (size_t)rb * 16 * ex.qe.nh * 128;
        }
        if constexpr (NORM) ex.np.ssq += rb * 16;
        if constexpr (RESID) ex.re.ssq += rb * 16;
    }
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, kb = lane >> 4;
    const int words = N >> 3;
    const int tile = tile_of_wg, split = blockIdx.y;   // host guarantees N % 128 == 0

    const int total_chunks = K / 128;
    const int c_begin = split * chunks_per_split;
    const int c_end = min(c_begin + chunks_per_split, total_chunks);
    const int per_wave = (max(c_end - c_begin, 0) + WK - 1) / WK;
    const int c0 = c_begin + wave * per_wave;
    const int c1 = min(c0 + per_wave, c_end);

    // one staging buffer per wave
    char* stage = reinterpret_cast<char*>(red) + (size_t)wave * dma_wave_bytes(M);
    const int x_off = 8192, zs_off = 8192 + 256 * M;

    // DMA lane roles
    const int dq = lane & 3, dsl = lane >> 2;  // 16-byte quarter of the 64-byte row piece, slot % 16
    uint32_t wsrc[2];                          // word offset inside a step, for slots 0..15 / 16..31
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int slot = h * 16 + dsl;
        wsrc[h] = (uint32_t)((slot & 3) * 8 + (slot >> 2)) * (uint32_t)words + (uint32_t)(tile * 16 + dq * 4);
    }
    // x: up to 4 rows in one DMA instruction per chunk, lane = m * 16 + (step * 4 + k-block), LDS layout
    // [m][step][k-block]; more rows in one instruction per step, lane = m * 4 + k-block, layout [step][m][k-block]
    const bool x_few = M <= 4;
    const bool x_lane = x_few ? (lane >> 4) < M : (lane >> 2) < M;
    const uint32_t xsrc = x_few ? (uint32_t)(x_lane ? lane >> 4 : 0) * (uint32_t)K + (uint32_t)(lane & 15) * 8u
                                : (uint32_t)(x_lane ? lane >> 2 : 0) * (uint32_t)K + (uint32_t)(lane & 3) * 8u;
    const bool zs_lane = lane < 16;
    const uint32_t zsrc = (uint32_t)(tile * 16 + (lane & 15));

    // Order of the loads of a chunk: the weights of steps 0..3 (two loads each), x, the zero words and the scales;
    // the step-by-step form consumes them as they land and wants x first (on multi-chunk launches that order measured
    // 7 % slower at 16 rows).  x is one load for all four steps with at most 4 rows, else one per step.
    // The x loads and the zero/scale loads run under a lane mask, and the step-by-step form counts loads by hand:
    // each masked group is ONE block, fenced off from the unmasked weight loads.  (With an x load in front of every
    // step's weights the compiler threaded the four equal conditions into one divergent branch and issued the weight
    // loads in between once per side of it -- two more loads in the wave's queue than the waits below count.)
    auto issue_x = [&](int row0) {
        if (x_lane) {
            if (x_few) {
                __builtin_amdgcn_global_load_lds(AWQ_GPTR(x + row0 + xsrc), AWQ_LPTR(stage + x_off), 16, 0, 0);
            } else {
#pragma unroll
                for (int s = 0; s < CH; ++s)
                    __builtin_amdgcn_global_load_lds(AWQ_GPTR(x + (row0 + s * 32) + xsrc),
                                                     AWQ_LPTR(stage + x_off + s * 64 * M), 16, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();
    };
    auto issue_dma = [&](int c) {
        const int row0 = c * 128;
        uint32_t* w_lds = reinterpret_cast<uint32_t*>(stage);
        if constexpr (STREAM) issue_x(row0);
#pragma unroll
        for (int s = 0; s < CH; ++s) {
            const uint32_t* wp = qweight + (size_t)(row0 + s * 32) * words;
#pragma unroll
            for (int h = 0; h < 2; ++h)
                __builtin_amdgcn_global_load_lds(AWQ_GPTR(wp + wsrc[h]), AWQ_LPTR(w_lds + s * 512 + h * 256),
                                                 16, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();
        if constexpr (!STREAM) issue_x(row0);
        if (zs_lane) {
            const int gi = chunks_per_group == 1 ? c : c / chunks_per_group;
            __builtin_amdgcn_global_load_lds(AWQ_GPTR(qzeros + (size_t)gi * words + zsrc), AWQ_LPTR(stage + zs_off),
                                             4, 0, 0);
            __builtin_amdgcn_global_load_lds(AWQ_GPTR(scales + ((size_t)gi * words + zsrc) * 8),
                                             AWQ_LPTR(stage + zs_off + 64), 16, 0, 0);
        }
    };

    // compute-lane read offsets inside the staging buffer (bytes)
    const uint32_t* w_rd = reinterpret_cast<const uint32_t*>(stage + (kb * 16 + j) * 4);   // + (s*512 + r*64) words
    const int x_rd_off = x_off + (x_few ? min(j, M - 1) * 16 + kb : min(j, M - 1) * 4 + kb) * 16;   // + s * x_rd_step
    const int x_rd_step = x_few ? 64 : 64 * M;
    const int z_rd_off = zs_off + j * 4;
    const int s_rd_off = zs_off + 64 + j * 16;

    f32x4 acc[1][8];

    float rstd = 0.f;
    u32x4 nw0[CH];   // step-by-step form with the prologue: the norm weights of the wave's one chunk
    if constexpr (NORM) {   // the lane's row: 1 / rms from the tile sums, added in tile order (eight loads in flight)
        const float* sp = ex.np.ssq + min(j, M - 1);
        float tot = 0.f;
        if constexpr (STREAM) {
            // (launched with up to kNormStreamChunks tiles only.)  Every statistic and the chunk's norm weights are
            // asked for BEFORE the chunk's loads: loads return in issue order, and anything issued behind the weights
            // would keep the normalisation below waiting for the whole chunk.
            float v[kNormStreamChunks];
#pragma unroll
            for (int u = 0; u < kNormStreamChunks; ++u) v[u] = sp[(size_t)min(u, total_chunks - 1) * ex.np.m_stride];
            if (c0 < c1) {
#pragma unroll
                for (int s = 0; s < CH; ++s)
                    nw0[s] = *reinterpret_cast<const u32x4*>(ex.np.weight + c0 * 128 + s * 32 + kb * 8);
                issue_dma(c0);
            }
#pragma unroll
            for (int u = 0; u < kNormStreamChunks; ++u) tot += u < total_chunks ? v[u] : 0.f;
        } else {
            for (int t0 = 0; t0 < total_chunks; t0 += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = sp[(size_t)min(t0 + u, total_chunks - 1) * ex.np.m_stride];
                if (t0 == 0 && c0 < c1) issue_dma(c0);   // behind the first statistics loads, ahead of their use
#pragma unroll
                for (int u = 0; u < 8; ++u) tot += t0 + u < total_chunks ? v[u] : 0.f;
            }
        }
        rstd = rsqrtf(tot / (float)K + ex.np.eps);
    } else {
        if (c0 < c1) issue_dma(c0);
    }
    // h = T(T(x * r) * w) for the 8 activations of one operand register quadruple
    auto normalise = [&](u32x4& xa, const u32x4& nwv) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t xv = xa[i], wv = nwv[i];
            const float lo = mul_round<T>(T::to_f32((uint16_t)(xv & 0xFFFFu)), rstd) * T::to_f32((uint16_t)(wv & 0xFFFFu));
            const float hi = mul_round<T>(T::to_f32((uint16_t)(xv >> 16)), rstd) * T::to_f32((uint16_t)(wv >> 16));
            xa[i] = T::pack2(lo, hi);
        }
    };
    int c_first = c0;
    if constexpr (STREAM) {
        // A wave with a single chunk (a decode-size launch: the chunk is all there is, and the loads of the eight
        // waves of a workgroup queue up behind each other) takes it step by step as its rows land: wait for the
        // loads of step s only -- outstanding loads are counted in issue order --, read its operands, multiply.
        // With more chunks the next one is fetched while a whole chunk is multiplied, below.
        if (c0 < c1) {   // the host launches this form only where a wave has one chunk at most
            const AndOr emb_lo(Embed<T>::kMaskLo, Embed<T>::kMagicLo), emb_hi(Embed<T>::kMaskHi, Embed<T>::kMagicHi);
            StepAcc sa;
            uint32_t zw = 0;
            u32x4 sv = u32x4{0u, 0u, 0u, 0u};
            constexpr int kWLoads = 2, kZsLoads = 2;
            static_assert(4 * kWLoads + kZsLoads <= 15, "the wait count is four bits wide here");
            static_assert(CH == 4, "one wait per step below");
            u32x4 xn[CH];
            if constexpr (NORM) {
                // x went out first: once it is there (the weights and the zeros/scales may all be on their way still)
                // the four operand quadruples are normalised while the weights land
                __builtin_amdgcn_s_waitcnt(0x0F70 | (4 * kWLoads + kZsLoads));
                asm volatile("" ::: "memory");
#pragma unroll
                for (int s = 0; s < CH; ++s) xn[s] = *reinterpret_cast<const u32x4*>(stage + x_rd_off + s * x_rd_step);
#pragma unroll
                for (int s = 0; s < CH; ++s) normalise(xn[s], nw0[s]);
            }
#pragma unroll
            for (int s = 0; s < CH; ++s) {
                // Loads still allowed in flight while step s is read: those issue_dma issues behind step s's weights --
                // the later steps' weights (kWLoads each) and the zero words and scales (x went out first).
                if (s == 0) __builtin_amdgcn_s_waitcnt(0x0F70 | (3 * kWLoads + kZsLoads));
                if (s == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * kWLoads + kZsLoads));
                if (s == 2) __builtin_amdgcn_s_waitcnt(0x0F70 | (1 * kWLoads + kZsLoads));
                if (s == 3) __builtin_amdgcn_s_waitcnt(0x0F70);
                asm volatile("" ::: "memory");
                uint32_t w[8];
#pragma unroll
                for (int r = 0; r < 8; ++r) w[r] = w_rd[s * 512 + r * 64];
                u32x4 xa;
                if constexpr (NORM) xa = xn[s];
                else xa = *reinterpret_cast<const u32x4*>(stage + x_rd_off + s * x_rd_step);
                if (s == 3) {
                    zw = *reinterpret_cast<const uint32_t*>(stage + z_rd_off);
                    sv = *reinterpret_cast<const u32x4*>(stage + s_rd_off);
                }
                if (s == 0) compute_step<T, true>(w, xa, sa, emb_lo, emb_hi);
                else compute_step<T>(w, xa, sa, emb_lo, emb_hi);
            }
            fold_steps<T, true>(sa, zw, sv, acc[0]);
            c_first = c1;
        } else {
#pragma unroll
            for (int f = 0; f < 8; ++f) acc[0][f] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    } else {
#pragma unroll
        for (int f = 0; f < 8; ++f) acc[0][f] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int c = STREAM ? c1 : c_first; c < c1; ++c) {
        u32x4 nw[CH];
        if constexpr (NORM) {
#pragma unroll
            for (int s = 0; s < CH; ++s)
                nw[s] = *reinterpret_cast<const u32x4*>(ex.np.weight + c * 128 + s * 32 + kb * 8);
        }
        // The compiler does not order LDS reads after the DMA by itself.
        __builtin_amdgcn_s_waitcnt(0x0F70);                                      // vmcnt(0): chunk c has landed
        asm volatile("" ::: "memory");
        Chunk<1, CH, 1> d;
#pragma unroll
        for (int s = 0; s < CH; ++s) {
#pragma unroll
            for (int r = 0; r < 8; ++r) d.w[s][r] = w_rd[s * 512 + r * 64];
            d.xa[s][0] = *reinterpret_cast<const u32x4*>(stage + x_rd_off + s * x_rd_step);
        }
        d.zw = *reinterpret_cast<const uint32_t*>(stage + z_rd_off);
        d.sv[0] = *reinterpret_cast<const u32x4*>(stage + s_rd_off);
        // every LDS read has returned before the next chunk's DMA may overwrite the buffer
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);                                      // lgkmcnt(0)
        asm volatile("" ::: "memory");
        if (c + 1 < c1) issue_dma(c + 1);
        if constexpr (NORM) {
#pragma unroll
            for (int s = 0; s < CH; ++s) normalise(d.xa[s][0], nw[s]);
        }
        compute_chunk<T, 1, CH, 1>(d, acc);
    }
    __syncthreads();  // staging area becomes the reduction buffer
    EpiArgs ea;
    if constexpr (QKV) ea.qe = &ex.qe;
    if constexpr (RESID) ea.re = &ex.re;
    gemv_epilogue<T, 1, 1, WK, 1, QKV ? 1 : (RESID ? 2 : 0)>(acc, red, &s_last, lane, wave, tile, split, splits, bias,
                                                            y, partials, counters, M, N, act, ea);
}

// ---- data path 3: a workgroup of eight waves shares one staged chunk --------------------------
// For 17..64 rows the activation chunk (MT*16 rows x 128 k = 4*MT KiB) is as large as the weights of a
// column tile; staged once per workgroup instead of once per wave it leaves room for DEPTH buffers, i.e.
// DEPTH-1 chunks (4 x 8 KiB of weights each) in flight while one is multiplied.  A workgroup owns 512
// columns (four column tiles) and a K range; nothing is reduced inside it.
//   buffer = [x: 4 steps x (MT*16 rows x 64 B)] [tile 0..3: 8 KiB weights + 512 B zeros/scales]
// Waves wn and wn + 4 work on the same column tile and the same rows, one on bytes 0-1 of every word
// (even output columns), the other on bytes 2-3 (odd columns).  Nothing is unpacked or scaled twice, each
// wave holds half the accumulators, and every SIMD has two waves.  What bounds this regime is the vector
// ALU port (one instruction per SIMD every four cycles: about 270 unpack, 140 scale/zero and 2 x 144 MFMA
// issue slots per 128 x 128 weights at 64 rows), not the memory.
// At the end the two halves exchange fragments through LDS so that each stores whole words of half the rows.
// A K split leaves fp32 partials that a second kernel adds in split order -- or, TAIL (one m-tile, a few rows), the
// last workgroup of the 512 columns to arrive, as in the one-tile kernel.
__host__ __device__ constexpr int wide_buf_bytes(int MT, int WN = 4) { return 4096 * MT + WN * 8704; }

template <typename T, int DEPTH, int MT, bool TAIL = false, int WN = 4>
__global__ __launch_bounds__(128 * WN) void gemv_wide_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint16_t* __restrict__ scales, const uint32_t* __restrict__ qzeros,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, float* __restrict__ partials,
    int* __restrict__ counters, int M, int N, int K, int chunks_per_group, int chunks_per_split, int splits, int act) {
    // XP: pieces of x a wave brings per chunk (with one m-tile the four pieces go to waves 0..3, one each);
    // HMT: m-tiles each of the two byte-half waves of a column tile stores at the end
    constexpr int CH = 4, XP = MT >= 2 ? 4 * MT / (2 * WN) : 1, HMT = MT >= 2 ? MT / 2 : 1;
    // Four m-tiles on 256 columns take a chunk one 32-row step at a time (below): two such workgroups share a CU, one
    // wave each per SIMD, and a wave that first brings all its loads and then reads the whole chunk from LDS leaves its
    // SIMD to the other workgroup's wave alone.  (Measured on the other forms too: no gain with eight waves per
    // workgroup, which pass a barrier per chunk together, nor with two m-tiles, where three waves share a SIMD.)
    constexpr bool STEP = WN == 2 && MT == 4;
    static_assert(WN == 4 || WN == 2, "512 or 256 columns per workgroup");
    static_assert(DEPTH >= 2 && DEPTH <= 3, "two or three staging buffers");
    static_assert(MT == 1 || MT == 2 || MT == 4, "m-tiles per workgroup");
    static_assert(!TAIL || MT == 1, "the in-kernel tail of a K split: one m-tile only");
    extern __shared__ __attribute__((aligned(16))) float red[];
    __shared__ int s_last;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave % WN, bh = wave / WN;
    const int j = lane & 15, kb = lane >> 4;
    const int words = N >> 3;
    const int group = blockIdx.x, split = blockIdx.y;
    const int tile = group * WN + wn;   // host guarantees N % 512 == 0

    const int total_chunks = K / 128;
    const int c0 = split * chunks_per_split;
    const int c1 = min(c0 + chunks_per_split, total_chunks);

    constexpr int buf_bytes = wide_buf_bytes(MT, WN);
    constexpr int x_step = 1024 * MT;
    char* stage = reinterpret_cast<char*>(red);
    const int w_off = 4096 * MT + wn * 8704, zs_off = w_off + 8192;

    const int dq = lane & 3, dsl = lane >> 2;
    uint32_t wsrc[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int slot = h * 16 + dsl;
        wsrc[h] = (uint32_t)((slot & 3) * 8 + (slot >> 2)) * (uint32_t)words + (uint32_t)(tile * 16 + dq * 4);
    }
    // x: the 4*MT (step, m-tile) pieces of 16 rows x 64 B are dealt to the 2*WN waves, XP each
    int x_s[XP], x_mt[XP];
    uint32_t xsrc[XP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int o = MT >= 2 ? wave * XP + i : (wave & 3);
        x_s[i] = o / MT;
        x_mt[i] = o % MT;
        xsrc[i] = (uint32_t)min(16 * x_mt[i] + (lane >> 2), M - 1) * (uint32_t)K + (uint32_t)(lane & 3) * 8u;
    }
    const bool x_wave = MT >= 2 || wave < 4;   // uniform
    const uint32_t zsrc = (uint32_t)(tile * 16 + (lane & 15));
    const bool zs_lane = lane < 16;

    // per wave and chunk (an upper bound where a wave brings no x; only a third buffer waits by this count)
    constexpr int kDmaOps = CH + XP + 1;
    // one m-tile: waves 4..7 bring no x, one load fewer per chunk
    const bool full_count = MT >= 2 || wave < 4;   // uniform
    auto wait_chunks_in_flight = [&](int n) {   // all but the loads of the n newest chunks have landed
#define AWQ_WIDE_WAIT(K) __builtin_amdgcn_s_waitcnt(0x0F70 | ((K) & 15) | (((K) >> 4) << 14))
        if (n == 0) AWQ_WIDE_WAIT(0);
        else if (full_count) AWQ_WIDE_WAIT(kDmaOps);
        else AWQ_WIDE_WAIT(kDmaOps - 1);
#undef AWQ_WIDE_WAIT
    };
    auto issue_dma = [&](int c, int buf) {
        const int row0 = c * 128;
        char* base = stage + buf * buf_bytes;
        uint32_t* w_lds = reinterpret_cast<uint32_t*>(base + w_off);
#pragma unroll
        for (int i = 0; i < CH / 2; ++i) {
            const int s = bh * (CH / 2) + i;
            const uint32_t* wp = qweight + (size_t)(row0 + s * 32) * words;
#pragma unroll
            for (int h = 0; h < 2; ++h)
                __builtin_amdgcn_global_load_lds(AWQ_GPTR(wp + wsrc[h]), AWQ_LPTR(w_lds + s * 512 + h * 256),
                                                 16, 0, 0);
        }
        // the three-buffer form counts its loads (wait_chunks_in_flight): every block below is issued once per wave,
        // fenced off from its neighbours so that no branch is threaded through another block's loads
        __builtin_amdgcn_wave_barrier();
        if (x_wave) {
#pragma unroll
            for (int i = 0; i < XP; ++i)
                __builtin_amdgcn_global_load_lds(AWQ_GPTR(x + (row0 + x_s[i] * 32) + xsrc[i]),
                                                 AWQ_LPTR(base + x_s[i] * x_step + x_mt[i] * 1024), 16, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();
        if (zs_lane) {
            const int gi = chunks_per_group == 1 ? c : c / chunks_per_group;
            if (bh == 0)
                __builtin_amdgcn_global_load_lds(AWQ_GPTR(qzeros + (size_t)gi * words + zsrc),
                                                 AWQ_LPTR(base + zs_off), 4, 0, 0);
            else
                __builtin_amdgcn_global_load_lds(AWQ_GPTR(scales + ((size_t)gi * words + zsrc) * 8),
                                                 AWQ_LPTR(base + zs_off + 64), 16, 0, 0);
        }
    };

    // STEP: the same loads in four parts, one per 32-row step of the chunk being multiplied (zeros/scales and half the
    // weights, the other half, then x)
    auto issue_dma_part = [&](int c, int buf, int part) {
        const int row0 = c * 128;
        char* base = stage + buf * buf_bytes;
        if (part < 2) {
            uint32_t* w_lds = reinterpret_cast<uint32_t*>(base + w_off);
            const int s = bh * (CH / 2) + part;
            const uint32_t* wp = qweight + (size_t)(row0 + s * 32) * words;
#pragma unroll
            for (int h = 0; h < 2; ++h)
                __builtin_amdgcn_global_load_lds(AWQ_GPTR(wp + wsrc[h]), AWQ_LPTR(w_lds + s * 512 + h * 256), 16, 0, 0);
            if (part == 0 && zs_lane) {
                const int gi = chunks_per_group == 1 ? c : c / chunks_per_group;
                if (bh == 0)
                    __builtin_amdgcn_global_load_lds(AWQ_GPTR(qzeros + (size_t)gi * words + zsrc),
                                                     AWQ_LPTR(base + zs_off), 4, 0, 0);
                else
                    __builtin_amdgcn_global_load_lds(AWQ_GPTR(scales + ((size_t)gi * words + zsrc) * 8),
                                                     AWQ_LPTR(base + zs_off + 64), 16, 0, 0);
            }
        } else if (x_wave) {
#pragma unroll
            for (int i = 0; i < XP; ++i)
                if ((XP == 1 ? 2 : 2 + (i & 1)) == part)
                    __builtin_amdgcn_global_load_lds(AWQ_GPTR(x + (row0 + x_s[i] * 32) + xsrc[i]),
                                                     AWQ_LPTR(base + x_s[i] * x_step + x_mt[i] * 1024), 16, 0, 0);
        }
    };

    const int w_rd_off = w_off + (kb * 16 + j) * 4;
    int x_rd_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) x_rd_off[mt] = ((16 * mt + j) * 4 + kb) * 16;
    const int z_rd_off = zs_off + j * 4;
    const int s_rd_off = zs_off + 64 + j * 16;

    auto run = [&](auto half) {
        constexpr int BH = decltype(half)::value;
        f32x4 acc[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int f = 0; f < 4; ++f) acc[mt][f] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (c0 + d < c1) issue_dma(c0 + d, d);
        int buf = 0;
        for (int c = c0; c < c1; ++c) {
            const int newer = min(c1 - 1 - c, DEPTH - 2);
            wait_chunks_in_flight(newer);
            asm volatile("" ::: "memory");
            // every wave's share of the chunk is in LDS, and every wave is done reading the buffer of chunk c-1.
            // A bare barrier: __syncthreads() would first wait for every outstanding load, i.e. for the chunks
            // in flight too; the LDS itself needs no fence (DMA data is there once vmcnt has counted it).
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const char* base = stage + buf * buf_bytes;
            const uint32_t* w_rd = reinterpret_cast<const uint32_t*>(base + w_rd_off);
            if constexpr (STEP) {
                // One 32-row step at a time: the LDS reads of step s + 1 and a part of the next chunk's loads go out
                // before step s is multiplied.  The MFMA chains and the fold are those of compute_chunk_bytes.
                const bool more = c + DEPTH - 1 < c1;
                const int nbuf = buf == 0 ? DEPTH - 1 : buf - 1;
                const u32x4 ones = u32x4{T::ones2, T::ones2, T::ones2, T::ones2};
                const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
                const AndOr emb_lo(Embed<T>::kMaskLo, Embed<T>::kMagicLo), emb_hi(Embed<T>::kMaskHi, Embed<T>::kMagicHi);
                uint32_t w[2][8];
                u32x4 xa[2][MT];
                f32x4 dones[MT], dq[2][2][MT];
                auto lds_step = [&](int s, int slot) {
#pragma unroll
                    for (int r = 0; r < 8; ++r) w[slot][r] = w_rd[s * 512 + r * 64];
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        xa[slot][mt] = *reinterpret_cast<const u32x4*>(base + x_rd_off[mt] + s * x_step);
                };
                lds_step(0, 0);
                const uint32_t zw = *reinterpret_cast<const uint32_t*>(base + z_rd_off);
                const u32x4 sv = *reinterpret_cast<const u32x4*>(base + s_rd_off);
#pragma unroll
                for (int s = 0; s < CH; ++s) {
                    if (s + 1 < CH) lds_step(s + 1, (s + 1) & 1);
                    if (more) issue_dma_part(c + DEPTH - 1, nbuf, s);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) dones[mt] = T::mfma16(xa[s & 1][mt], ones, s ? dones[mt] : zero4);
#pragma unroll
                    for (int bi = 0; bi < 2; ++bi) {
                        const int b = 2 * BH + bi;
                        u32x4 flo, fhi;
#pragma unroll
                        for (int rp = 0; rp < 4; ++rp) {
                            const uint32_t p = __builtin_amdgcn_perm(w[s & 1][2 * rp + 1], w[s & 1][2 * rp],
                                                                     0x0c000c00u | (uint32_t)b | ((4u + b) << 16));
                            flo[rp] = emb_lo(Embed<T>::pre_lo(p));
                            fhi[rp] = emb_hi(Embed<T>::pre_hi(p));
                        }
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) {
                            dq[bi][0][mt] = T::mfma16(xa[s & 1][mt], flo, s ? dq[bi][0][mt] : zero4);
                            dq[bi][1][mt] = T::mfma16(xa[s & 1][mt], fhi, s ? dq[bi][1][mt] : zero4);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int bi = 0; bi < 2; ++bi) {
                    constexpr int kLoCol[4] = {0, 4, 1, 5}, kHiCol[4] = {2, 6, 3, 7};
                    const int b = 2 * BH + bi;
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int col = h ? kHiCol[b] : kLoCol[b];
                        const float mul = h ? Embed<T>::kMulHi : Embed<T>::kMulLo;
                        const float off = h ? Embed<T>::kOffHi : Embed<T>::kOffLo;
                        const float zf = (float)((zw >> nibble_shift(col)) & 0xFu) * mul + off;
                        const uint32_t pair = sv[col >> 1];
                        const float sc = T::to_f32((uint16_t)((col & 1) ? (pair >> 16) : (pair & 0xFFFFu))) * (1.f / mul);
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                acc[mt][2 * bi + h][r] += sc * (dq[bi][h][mt][r] - zf * dones[mt][r]);
                    }
                }
                buf = (buf + 1 == DEPTH) ? 0 : buf + 1;
                continue;
            }
            if (c + DEPTH - 1 < c1) issue_dma(c + DEPTH - 1, buf == 0 ? DEPTH - 1 : buf - 1);
            Chunk<1, CH, MT> d;
#pragma unroll
            for (int s = 0; s < CH; ++s) {
#pragma unroll
                for (int r = 0; r < 8; ++r) d.w[s][r] = w_rd[s * 512 + r * 64];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    d.xa[s][mt] = *reinterpret_cast<const u32x4*>(base + x_rd_off[mt] + s * x_step);
            }
            d.zw = *reinterpret_cast<const uint32_t*>(base + z_rd_off);
            d.sv[0] = *reinterpret_cast<const u32x4*>(base + s_rd_off);
            // no wait here: this buffer is overwritten only after the next barrier, which a wave reaches
            // with every read consumed
            buf = (buf + 1 == DEPTH) ? 0 : buf + 1;
            compute_chunk_bytes<T, CH, MT, BH>(d, acc);
        }
        if constexpr (MT == 1) {
            // One m-tile: the odd half hands its four fragments to its partner, which stores whole words.
            __syncthreads();   // staging is free
            float* xch1 = red + (size_t)wn * (16 * 64);
            if (BH == 1) {
#pragma unroll
                for (int f = 0; f < 4; ++f)
#pragma unroll
                    for (int r = 0; r < 4; ++r) xch1[(f * 4 + r) * 64 + lane] = acc[0][f][r];
            }
            __syncthreads();
            if (BH == 0) {
                f32x4 acc8[8];
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    acc8[2 * f] = acc[0][f];
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc8[2 * f + 1][r] = xch1[(f * 4 + r) * 64 + lane];
                }
                gemv_reduce_store<T, 1, WN, 1, !TAIL>(acc8, 0, red, lane, wn, group, split, splits, bias, y, partials, M,
                                                      N, act);
            }
            if constexpr (TAIL) {   // the last workgroup of the 512 columns to arrive adds the splits
                if (splits > 1)
                    gemv_split_tail<T, 1, WN, 2>(red, &s_last, group, splits, bias, y, partials, counters, M, N, act);
            }
            return;
        }
        // Exchange: this wave stores m-tiles BH*HMT .. and sends its fragments of the other m-tiles to its
        // partner (wave ^ WN).  xch[wave][(ml*4 + f)*4 + r][lane]
        __syncthreads();   // staging is free
        float* xch = red;
        constexpr int PER_WAVE = HMT * 16 * 64;
#pragma unroll
        for (int ml = 0; ml < HMT; ++ml)
#pragma unroll
            for (int f = 0; f < 4; ++f)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    xch[wave * PER_WAVE + ((ml * 4 + f) * 4 + r) * 64 + lane] = acc[(1 - BH) * HMT + ml][f][r];
        __syncthreads();
#pragma unroll
        for (int ml = 0; ml < HMT; ++ml) {
            const int mt = BH * HMT + ml;
            f32x4 acc8[8];
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                acc8[2 * f + BH] = acc[mt][f];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc8[2 * f + 1 - BH][r] = xch[(wave ^ WN) * PER_WAVE + ((ml * 4 + f) * 4 + r) * 64 + lane];
            }
            if (16 * mt < M)
                gemv_reduce_store<T, 1, WN, 1, true>(acc8, 16 * mt, red, lane, wn, group, split, splits, bias, y,
                                                     partials, M, N, act);
        }
    };
    if (bh == 0) run(std::integral_constant<int, 0>{});
    else run(std::integral_constant<int, 1>{});
}

// Second pass of a K-split wide GEMV: y = epilogue(sum over splits, in split order, of partials [splits][M][N]).
// A thread owns one word (8 columns) of one row; with the gated epilogue neighbouring threads hold a gate word
// and its up word.
template <typename T>
__global__ __launch_bounds__(256) void gemv_wide_reduce_kernel(const float* __restrict__ partials,
                                                               const uint16_t* __restrict__ bias,
                                                               uint16_t* __restrict__ y, int M, int N, int splits,
                                                               int act) {
    const int words = N >> 3;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= M * words) return;   // words is even: a gate word and its up word leave together
    const int m = idx / words, wc = idx - m * words;
    const size_t n0 = (size_t)wc * 8;
    const size_t plane = (size_t)M * N;
    const float* p = partials + (size_t)m * N + n0;
    f32x4 lo = f32x4{0.f, 0.f, 0.f, 0.f}, hi = lo;
    // eight splits' loads in flight at a time (a loop of load, add, load, add is one memory round trip per split:
    // 4.7 us for five splits of 16 rows x 25600 columns), added in split order all the same
    for (int s0 = 0; s0 < splits; s0 += 8) {
        f32x4 a[8], b[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t off = (size_t)min(s0 + u, splits - 1) * plane;
            a[u] = *reinterpret_cast<const f32x4*>(p + off);
            b[u] = *reinterpret_cast<const f32x4*>(p + off + 4);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (s0 + u < splits) {
                lo += a[u];
                hi += b[u];
            }
    }
    float out[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (act) {
        swiglu_store<T>(out, y, m, N, n0);
        return;
    }
    if (bias) {
        const u32x4 bv = *reinterpret_cast<const u32x4*>(bias + n0);
#pragma unroll
        for (int c = 0; c < 8; ++c)
            out[c] = add_bias<T>(out[c], T::to_f32((uint16_t)((c & 1) ? (bv[c >> 1] >> 16) : (bv[c >> 1] & 0xFFFFu))));
    }
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = T::pack2(out[2 * i], out[2 * i + 1]);
    *reinterpret_cast<u32x4*>(y + (size_t)m * N + n0) = o;
}

// The second pass and the residual add + RMSNorm that follows an o_proj or down_proj in one: a workgroup per row
// (N <= 8192: a thread per word), residual[m, :] = T(residual + T(sum of the splits)) in place, normed[m, :] =
// T(T(residual * rsqrt(mean square + eps)) * weight).  The splits are added as in gemv_wide_reduce_kernel, the
// sum of squares per 128-column tile and the tiles in index order as in the stand-alone norm kernel: the same bits as
// the two launches, one of which (with the gap before it) is saved -- at 64 rows x 5120 columns 6.5 + 4.4 us.
template <typename T>
__global__ __launch_bounds__(1024) void gemv_wide_reduce_add_rmsnorm_kernel(const float* __restrict__ partials,
                                                                           uint16_t* __restrict__ residual,
                                                                           const uint16_t* __restrict__ weight,
                                                                           uint16_t* __restrict__ normed, int M, int N,
                                                                           int splits, float eps) {
    __shared__ float s_tile[64];
    const int words = N >> 3, tiles = (N + 127) >> 7;
    const int m = blockIdx.x, wc = threadIdx.x;
    const bool own = wc < words;
    const size_t n0 = (size_t)wc * 8;
    const size_t plane = (size_t)M * N;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    u32x4 wraw = u32x4{0u, 0u, 0u, 0u};
    if (own) {
        const u32x4 xraw = *reinterpret_cast<const u32x4*>(residual + (size_t)m * N + n0);
        wraw = *reinterpret_cast<const u32x4*>(weight + n0);
        const float* p = partials + (size_t)m * N + n0;
        f32x4 lo = f32x4{0.f, 0.f, 0.f, 0.f}, hi = lo;
        for (int s0 = 0; s0 < splits; s0 += 8) {
            f32x4 a[8], b[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const size_t off = (size_t)min(s0 + u, splits - 1) * plane;
                a[u] = *reinterpret_cast<const f32x4*>(p + off);
                b[u] = *reinterpret_cast<const f32x4*>(p + off + 4);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (s0 + u < splits) {
                    lo += a[u];
                    hi += b[u];
                }
        }
        const float sum[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int c = 2 * i + h;
                const float x = T::to_f32((uint16_t)(h ? (xraw[i] >> 16) : (xraw[i] & 0xFFFFu)));
                const float d = T::to_f32(T::from_f32(as_f32_result(sum[c])));        // the GEMV's output, rounded
                v[c] = T::to_f32(T::from_f32(as_f32_result(x + d)));                  // the residual add, rounded
            }
            o[i] = (uint32_t)T::from_f32(v[2 * i]) | ((uint32_t)T::from_f32(v[2 * i + 1]) << 16);
        }
        *reinterpret_cast<u32x4*>(residual + (size_t)m * N + n0) = o;
    }
    const float ts = tile_ssq(v);   // every lane takes part; threads past the row add zeros
    if ((threadIdx.x & 15) == 0 && (int)(threadIdx.x >> 4) < 64) s_tile[threadIdx.x >> 4] = ts;
    __syncthreads();
    float tot = 0.f;
    for (int t = 0; t < tiles; ++t) tot += s_tile[t];
    const float r = rsqrtf(tot / (float)N + eps);
    if (own) {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float w0 = T::to_f32((uint16_t)(wraw[i] & 0xFFFFu)), w1 = T::to_f32((uint16_t)(wraw[i] >> 16));
            o[i] = (uint32_t)T::from_f32(mul_round<T>(v[2 * i], r) * w0) |
                   ((uint32_t)T::from_f32(mul_round<T>(v[2 * i + 1], r) * w1) << 16);
        }
        *reinterpret_cast<u32x4*>(normed + (size_t)m * N + n0) = o;
    }
}

// The second pass with the q|k|v epilogue of awq_gemv_qkv_rope_store: a thread owns one word of one row as in
// gemv_wide_reduce_kernel, the 16 threads of a head call qkv_rope_store together (N % 128 == 0: a head never
// straddles a row, M * N / 8 is a multiple of 16).
template <typename T>
__global__ __launch_bounds__(256) void gemv_wide_reduce_qkv_kernel(const float* __restrict__ partials, int M, int N,
                                                                   int splits, QkvEpilogue qe) {
    const int words = N >> 3;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= M * words) return;   // whole groups of 16 threads
    const int m = idx / words, wc = idx - m * words;
    const size_t n0 = (size_t)wc * 8;
    const size_t plane = (size_t)M * N;
    const float* p = partials + (size_t)m * N + n0;
    f32x4 lo = f32x4{0.f, 0.f, 0.f, 0.f}, hi = lo;
    for (int s0 = 0; s0 < splits; s0 += 8) {
        f32x4 a[8], b[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t off = (size_t)min(s0 + u, splits - 1) * plane;
            a[u] = *reinterpret_cast<const f32x4*>(p + off);
            b[u] = *reinterpret_cast<const f32x4*>(p + off + 4);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (s0 + u < splits) {
                lo += a[u];
                hi += b[u];
            }
    }
    const float out[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    qkv_rope_store<T>(out, m, n0, true, qe);
}

// ---- host side -------------------------------------------------------------
struct GemvVariant {
    const char* name;
    int V, waves;
    bool prefetch;
    int wn;     // waves side by side along N (DMA variants), 1 otherwise
    int depth;  // DMA staging buffers per wave (DMA variants), 0 otherwise
    int mt;     // tiles of 16 activation rows: M <= 16 * mt
    bool wide;  // a workgroup of eight waves shares one staged chunk (gemv_wide_kernel)
};
static const GemvVariant kGemvVariants[] = {
    // register path, named v<V>w<waves>[p = next chunk prefetched]
    {"v1w4p", 1, 4, true, 1, 0, 1},
    {"v2w4", 2, 4, false, 1, 0, 1},
    // staged (DMA) path, one column tile per workgroup, named dma1x<WK>; 17..64 rows run as blocks of 16 (grid z)
    {"dma1x4", 1, 4, false, 1, 1, 1},
    {"dma1x8", 1, 8, false, 1, 1, 1},
    // shared staged chunk, eight waves as 4 column tiles x 2 byte halves: wide d<DEPTH> m<MT>
    {"wided2m4", 1, 8, false, 4, 2, 4, true},
    {"wided2m2", 1, 8, false, 4, 2, 2, true},
    {"wided2m1", 1, 8, false, 4, 2, 1, true},
    // the same with the K splits added by the last workgroup to arrive instead of a second kernel: ...t
    {"wided2m1t", 1, 8, false, 4, 2, 1, true},
    // one m-tile with three staging buffers (two chunks in flight): for launches of one workgroup per CU at most
    {"wided3m1", 1, 8, false, 4, 3, 1, true},
    {"wided3m1t", 1, 8, false, 4, 3, 1, true},
    // the one-m-tile forms on 256 columns per workgroup (four waves: 2 column tiles x 2 byte halves): wide2d...
    {"wide2d2m1", 1, 4, false, 2, 2, 1, true},
    {"wide2d2m1t", 1, 4, false, 2, 2, 1, true},
    {"wide2d3m1", 1, 4, false, 2, 3, 1, true},
    {"wide2d3m1t", 1, 4, false, 2, 3, 1, true},
    // 256 columns, two m-tiles (17..32 rows)
    {"wide2d2m2", 1, 4, false, 2, 2, 2, true},
    {"wide2d3m2", 1, 4, false, 2, 3, 2, true},
    // 256 columns, four m-tiles (33..64 rows), a chunk taken one 32-row step at a time
    {"wide2d2m4", 1, 4, false, 2, 2, 4, true},
};
enum { kV1W4P = 0, kV2W4 = 1, kDma1x4 = 2, kDma1x8 = 3, kWideM4 = 4, kWideM2 = 5, kWideM1 = 6, kWideM1T = 7,
       kWideD3M1 = 8, kWideD3M1T = 9, kWide2D2M1 = 10, kWide2D2M1T = 11, kWide2D3M1 = 12, kWide2D3M1T = 13, kWide2D2M2 = 14, kWide2D3M2 = 15,
       kWide2D2M4 = 16 };
constexpr int kNumGemvVariants = sizeof(kGemvVariants) / sizeof(kGemvVariants[0]);
constexpr int kFirstDmaVariant = kDma1x4;

// Rows the staged kernels take as blocks of 16 (grid z).  awq_linear sends 65..128 rows here only on small weights
// (kGemvWideRowsMaxWeights), where eight blocks re-reading the weights from cache beat the narrow-tile MFMA GEMM by 2 x
// (1024 x 3072 at 128 rows: 8.2 against 17.5 us; 4096 x 4096: 14.8 against 23.0; equal from about 25 M weights on).
constexpr int kGemvMaxRows = 128;

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
    (void)hipGetLastError();  // do not report an earlier, unrelated failure as this launch's
    hipLaunchKernelGGL(kern, dim3(tiles, splits), dim3(64 * WAVES), lds, stream,
                       reinterpret_cast<const uint16_t*>(x),
                       reinterpret_cast<const uint32_t*>(qweight),
                       reinterpret_cast<const uint16_t*>(qscales),
                       reinterpret_cast<const uint32_t*>(qzeros),
                       reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y),
                       partials, counters, M, N, K, g / (32 * CH), cps, splits);
    return hipGetLastError();
}

template <typename T, int WK>
static hipError_t launch_gemv_dma(const void* x, const int32_t* qweight, const void* qscales,
                                  const int32_t* qzeros, const void* bias, void* y, int M, int N, int K,
                                  int g, void* workspace, int split_k, hipStream_t stream, int act,
                                  PrefetchRegions pf, const GemvFusion& fu = GemvFusion{}) {
    const int groups = N / 128;
    const int total_chunks = K / 128;
    const int cps = (int)cdiv(total_chunks, split_k);
    const int splits = (int)cdiv(total_chunks, cps);
    int* counters = reinterpret_cast<int*>(workspace);
    float* partials = workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) +
                                                            kCounterBytes)
                                : nullptr;
    const int row_blocks = (int)cdiv(M, 16);   // 17..64 rows: independent blocks of 16 rows along grid z
    size_t lds = (size_t)WK * dma_wave_bytes(M > 16 ? 16 : M);
    const size_t red_bytes = (size_t)WK * 32 * 64 * sizeof(float);
    if (lds < red_bytes) lds = red_bytes;
    constexpr size_t kMaxLds = (size_t)WK * dma_wave_bytes(16);
    if (kMaxLds > 64 * 1024) {
        static bool raised = false;  // once per process and instantiation (every form of the kernel)
        if (!raised) {
            const void* forms[] = {reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, 0>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, kModeQkv>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, kModeNorm>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, kModeQkv | kModeNorm>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, kModeResid>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, 0, true>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, kModeQkv, true>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, kModeResid, true>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, kModeNorm, true>),
                                   reinterpret_cast<const void*>(gemv_dma_kernel<T, WK, kModeQkv | kModeNorm, true>)};
            for (const void* f : forms) {
                hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds);
                if (e != hipSuccess) return e;
            }
            raised = true;
        }
    }
    (void)hipGetLastError();  // do not report an earlier, unrelated failure as this launch's
    // the caller's pending prefetch hints ride on this launch when the compute grid leaves CUs idle
    long long pf_bytes = 0;
    for (int r = 0; r < pf.count; ++r) pf_bytes += pf.bytes[r];
    int pf_wgs = 0;
    const long long compute_wgs = (long long)groups * splits * row_blocks;
    if (pf_bytes >= 128 && compute_wgs < 192) {
        const long long want = cdiv(pf_bytes >> 7, 64 * WK * 2);   // about 2 lines per thread
        const long long room = (256 - compute_wgs) / ((long long)splits * row_blocks);   // stay within one wave of workgroups
        pf_wgs = (int)(want < room ? want : room);
        if (pf_wgs < 1) pf_wgs = 1;
    } else {
        pf.count = 0;
    }
    // tiles in pairs per XCD on the narrow weights of decode-size launches, where the other mapping leaves the two
    // halves of every line to two XCDs (8 or 24 tiles; fetch from the fabric per launch of the Qwen3-0.6B sweep
    // 3.1 -> 2.3 MB, 6.0 -> 5.7 us).  Wide weights keep runs of consecutive tiles per XCD: pairs dealt round-robin
    // measured slower there (40 tiles x 200 chunks at 16 rows 26.5 -> 39.4 us).
    const int pair_map = (groups % 16 != 0 && groups >= 2 && groups <= 24) ? 1 : 0;
    int grid_x = groups + pf_wgs;
    if (pair_map) grid_x = (int)cdiv(grid_x, 16) * 16;
    const dim3 grid(grid_x, splits, row_blocks), block(64 * WK);
    const bool stream_form = cps <= WK;   // one chunk per wave at most
#define AWQ_DMA_LAUNCH(MODE, EXTRA)                                                                                \
    AWQ_DMA_LAUNCH_FORM(MODE, false, EXTRA)
#define AWQ_DMA_LAUNCH_S(MODE, EXTRA)                                                                              \
    do {                                                                                                           \
        if (stream_form) AWQ_DMA_LAUNCH_FORM(MODE, true, EXTRA);                                                   \
        else AWQ_DMA_LAUNCH_FORM(MODE, false, EXTRA);                                                              \
    } while (0)
#define AWQ_DMA_LAUNCH_FORM(MODE, STREAMED, EXTRA)                                                                 \
    hipLaunchKernelGGL((gemv_dma_kernel<T, WK, MODE, STREAMED>), grid, block, lds, stream,                        \
                       reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint32_t*>(qweight),          \
                       reinterpret_cast<const uint16_t*>(qscales), reinterpret_cast<const uint32_t*>(qzeros),     \
                       reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y), partials, counters, \
                       M, N, K, g / 128, cps, splits, act, groups, pair_map, pf, EXTRA)
    const bool norm_stream = stream_form && total_chunks <= kNormStreamChunks;
    if (fu.qe && fu.np) {
        if (norm_stream) AWQ_DMA_LAUNCH_FORM(kModeQkv | kModeNorm, true, (GemvExtra<kModeQkv | kModeNorm>{*fu.qe, *fu.np}));
        else AWQ_DMA_LAUNCH(kModeQkv | kModeNorm, (GemvExtra<kModeQkv | kModeNorm>{*fu.qe, *fu.np}));
    } else if (fu.qe)
        AWQ_DMA_LAUNCH_S(kModeQkv, (GemvExtra<kModeQkv>{*fu.qe}));
    else if (fu.np) {
        if (norm_stream) AWQ_DMA_LAUNCH_FORM(kModeNorm, true, (GemvExtra<kModeNorm>{*fu.np}));
        else AWQ_DMA_LAUNCH(kModeNorm, (GemvExtra<kModeNorm>{*fu.np}));
    }
    else if (fu.re)
        AWQ_DMA_LAUNCH_S(kModeResid, (GemvExtra<kModeResid>{*fu.re}));
    else
        AWQ_DMA_LAUNCH_S(0, (GemvExtra<0>{}));
#undef AWQ_DMA_LAUNCH
#undef AWQ_DMA_LAUNCH_S
#undef AWQ_DMA_LAUNCH_FORM
    return hipGetLastError();
}

// The one-m-tile form comes with either way of adding its K splits (variants wided2m1 / wided2m1t): the last
// workgroup's serial tail grows with rows x splits -- 5120 x 25600 in five splits: 19.6 us with the tail against 20.4
// with the second pass at one row, 20.9 / 21.3 at four, 22.0 / 21.3 at eight, 25.3 / 22.1 at sixteen.
constexpr int kWideTailRows = 4;   // the default dispatch takes the tail up to here

template <typename T, int DEPTH, int MT, bool TAIL = false, int WN = 4>
static hipError_t launch_gemv_wide(const void* x, const int32_t* qweight, const void* qscales,
                                   const int32_t* qzeros, const void* bias, void* y, int M, int N, int K,
                                   int g, void* workspace, int split_k, hipStream_t stream, int act,
                                   const AddNorm* an = nullptr, const QkvEpilogue* qe = nullptr) {
    const int groups = N / (128 * WN);
    const int total_chunks = K / 128;
    const int cps = (int)cdiv(total_chunks, split_k);
    const int splits = (int)cdiv(total_chunks, cps);
    float* partials = workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kCounterBytes)
                                : nullptr;
    int* counters = reinterpret_cast<int*>(workspace);
    constexpr size_t lds = (size_t)DEPTH * wide_buf_bytes(MT, WN);
    static_assert(lds <= 160 * 1024 - 1024, "staging buffers exceed the LDS");
    static_assert(!TAIL || lds >= 128 * WN * 128, "the tail stages 128 bytes per thread");
    if ((an || qe) && (splits == 1 || TAIL)) return hipErrorInvalidValue;   // their work is the second pass's
    auto kern = gemv_wide_kernel<T, DEPTH, MT, TAIL, WN>;
    static bool raised = false;  // once per process and instantiation
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        raised = true;
    }
    (void)hipGetLastError();
    hipLaunchKernelGGL(kern, dim3(groups, splits), dim3(128 * WN), lds, stream,
                       reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint32_t*>(qweight),
                       reinterpret_cast<const uint16_t*>(qscales), reinterpret_cast<const uint32_t*>(qzeros),
                       reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y), partials, counters,
                       M, N, K, g / 128, cps, splits, act);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || splits == 1 || TAIL) return e;
    if (qe) {
        hipLaunchKernelGGL(gemv_wide_reduce_qkv_kernel<T>, dim3((unsigned)cdiv((int64_t)M * (N / 8), 256)), dim3(256), 0,
                           stream, partials, M, N, splits, *qe);
        return hipGetLastError();
    }
    if (an) {   // (checked by the caller: splits > 1, no tail, no bias, no gate, N <= 8192)
        hipLaunchKernelGGL(gemv_wide_reduce_add_rmsnorm_kernel<T>, dim3((unsigned)M), dim3(1024), 0, stream, partials,
                           reinterpret_cast<uint16_t*>(y), an->weight, an->normed, M, N, splits, an->eps);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(gemv_wide_reduce_kernel<T>, dim3((unsigned)cdiv((int64_t)M * (N / 8), 256)), dim3(256), 0, stream, partials,
                       reinterpret_cast<const uint16_t*>(bias), reinterpret_cast<uint16_t*>(y), M, N, splits, act);
    return hipGetLastError();
}

// Upper bound that does not depend on the group size: the kernel never uses
// more K-splits than asked for.
static size_t gemv_ws_bytes(int64_t M, int64_t N, int64_t K, int variant, int split_k) {
    (void)variant;
    if (split_k <= 1 || K < 64) return 0;
    return kCounterBytes + (size_t)split_k * (M > 16 ? cdiv(M, 16) * 16 : M) * N * sizeof(float);   // row blocks of 16
}

// Launch shape for the default entry point.
//
// The DMA path (N % 128 == 0, group size % 128 == 0) runs one column tile per
// workgroup with WK waves over K.  Splitting K across workgroups costs a
// serial tail (publish, arrival counter, fetch: a few microseconds), so it is
// used only while one workgroup per column tile leaves most SIMDs empty.
// A workgroup gives each of its `wk` waves ceil(chunks_per_split / wk) chunks and lasts as long as the
// busiest one (40 chunks in 4 splits over 4 waves: 3, 3, 3, 1 -- a quarter of the time wasted).  Among the
// split counts from `s` to twice that (capped), take the one that wastes the fewest wave slots.
static int64_t balance_splits(int64_t chunks, int64_t s, int64_t wk, int64_t cap) {
    if (s <= 1) return 1;
    int64_t best = s;
    double best_eff = 0.0;
    const int64_t hi = 2 * s < cap ? 2 * s : cap;
    for (int64_t c = s; c <= hi; ++c) {
        const int64_t cps = cdiv(chunks, c), splits = cdiv(chunks, cps);
        const double eff = (double)chunks / (double)(splits * wk * cdiv(cps, wk));
        if (eff > best_eff + 1e-9) {
            best_eff = eff;
            best = c;
        }
    }
    return best;
}

// The one-m-tile forms of the shared-chunk kernel for up to 16 rows on large weights: which one, and its K split
// (0 = the one-tile staged kernel runs).  The one-tile kernel's waves each bring their own x (4 KiB per chunk beside
// 8 KiB of weights at 16 rows) and fetch 64-byte row pieces; in a shared-chunk workgroup x is staged once and the row
// pieces are 128 or 256 bytes wide.  From sweeps of every form x split on 17 weights of 50..260 M elements:
//  * N >= 28672 (the fused gate|up of Qwen3-14B/32B, 8192 x 28672): 512 columns per workgroup.  Few splits fill the
//    chip there, and every split costs a tail (per row) or partial traffic.  Up to four rows with the in-kernel tail,
//    the split count from a cost in chunk times -- rounds of 256 workgroups x chunks per split + 0.06 per row and
//    split, 5 % off where one workgroup per CU lets the three-buffer form run -- (5120 x 51200 at one row 35.5 -> 32.2
//    us in five splits, 8192 x 28672 33.4 -> 28.6 in four, 5120 x 34816 26.0 -> 24.4 in seven); at three and four rows
//    only where five splits or fewer do (5120 x 34816 in ten: 27.3 -> 29.9).  5..16 rows: second pass, about one
//    workgroup per CU (5120 x 51200 at 16 rows 46.2 -> 36.6 us, 5120 x 34816 34.7 -> 28.3, 8192 x 28672 -> 32.2).
//  * 8192 <= N < 28672 and 64 Mi weights or more (52 M from five rows, 50 M from nine rows on: 5120 x 10240 at 8 / 16
//    rows 15.2 / 16.2 -> 13.9 / 14.3 us, 6144 x 10240 at 8 rows 16.5 -> 14.4, while at up to four rows these lose 0.5 us
//    and 4096 x 12288 at 8 rows 12.4 -> 13.7): 256 columns per workgroup (four waves).  Plan A: two buffers,
//    about 500 workgroups (two or three share a CU); plan B: about one workgroup per CU (at least 85 % of them),
//    three buffers if a split has six chunks or more.  Up to eight rows with the tail while rows x splits <= 64 -- A,
//    or B where A needs eleven splits or more -- (one row: 5120 x 25600 19.9 -> 17.6 us, 5120 x 17408 15.8 -> 14.1,
//    12288 x 8192 19.5 -> 16.0, 8192 x 8192 15.5 -> 12.9, 4096 x 22016 19.3 -> 15.4, 3584 x 18944 15.4 -> 12.8; four
//    rows: 8192 x 10240 18.2 -> 16.4, 12288 x 8192 20.3 -> 18.1, 5120 x 25600 20.6 -> 18.3; eight: 22.7 -> 19.1),
//    beyond that B with the second pass (12288 x 8192 at 16 rows 21.6 -> 18.9 us, 8192 x 8192 17.2 -> 15.8,
//    8192 x 10240 19.7 -> 18.3, 6144 x 16384 21.8 -> 18.6), else the 512-column form if that fills the CUs
//    (4096 x 24576: 19.4), else A (5120 x 25600 21.2 -> 20.7, 5120 x 17408 18.4 -> 17.7).  Smaller weights (4096 x
//    12288, 12288 x 4096, 8192 x 5120, 5120 x 12288) and narrower ones (16384 x 4096, 25600 x 5120, 8192 x 7168:
//    28..56 column tiles) lose up to 2 us to the one-tile kernel.
static int64_t pick_one_m_tile(int64_t M, int64_t N, int64_t K, int64_t chunks, int* variant) {
    if (chunks < 8) return 0;
    auto normalised = [&](int64_t c) { return cdiv(chunks, cdiv(chunks, c)); };   // the split count a launch ends up with
    // 512 columns per workgroup, second pass: about one workgroup per CU
    auto wide512_pass = [&]() -> int64_t {
        int64_t c = 256 / (N / 512);
        if (c < 2) c = 2;
        if (c > chunks / 4) c = chunks / 4;
        const int64_t cps = cdiv(chunks, c);
        *variant = (N / 512 * normalised(c) <= 256 && cps >= 8) ? kWideD3M1 : kWideM1;
        return c;
    };
    if (N >= 28672) {
        if (N % 512 != 0 || K * N < 80000000ll) return 0;
        if (M > kWideTailRows) return wide512_pass();
        double best = 1e30;
        int64_t best_c = 0;
        bool best_d3 = false;
        const int64_t hi = chunks / 4 < 16 ? chunks / 4 : 16;
        for (int64_t c = 2; c <= hi; ++c) {
            const int64_t cps = cdiv(chunks, c), splits = cdiv(chunks, cps);
            if (splits != c) continue;
            const int64_t wgs = N / 512 * splits;
            const bool d3 = wgs <= 256 && cps >= 6;
            const double cost = ((double)(cdiv(wgs, 256) * cps) + 0.06 * (double)(M * splits)) * (d3 ? 0.95 : 1.0);
            if (cost < best - 1e-9) {
                best = cost;
                best_c = c;
                best_d3 = d3;
            }
        }
        if (best_c == 0 || (M > 2 && best_c > 5)) return 0;
        *variant = best_d3 ? kWideD3M1T : kWideM1T;
        return best_c;
    }
    if (N % 256 != 0 || K * N < (M <= 4 ? (64ll << 20) : (M <= 8 ? 52000000ll : 50000000ll))) return 0;
    // (40 to 63 column tiles: at one and two rows from 80 M weights on -- 25600 x 5120 22.0 -> 20.3 us, 17408 x 5120
    // 17.5 -> 16.4 in 20 splits --, from five rows on from 120 M -- 25600 x 5120 at 16 rows 26.2 -> 24.8 us; otherwise, and
    // on 16384 x 4096 at any row count, the one-tile kernel is as fast or faster)
    if (N < 8192 && (N < 5120 || (M <= 2 ? K * N < 80000000ll : (M < 5 || K * N < 120000000ll)))) return 0;
    const int64_t groups = N / 256;
    int64_t sa = 512 / groups;
    if (sa > 20) sa = 20;
    if (sa > chunks / 4) sa = chunks / 4;
    if (sa < 2) return 0;
    sa = normalised(sa);
    int64_t sb = 256 / groups;
    if (sb > chunks / 4) sb = chunks / 4;
    const bool b_valid = sb >= 2 && normalised(sb) * groups >= 218;
    if (b_valid) sb = normalised(sb);
    const bool b_d3 = b_valid && cdiv(chunks, sb) >= 6;
    if (M <= 8) {
        const bool use_b = b_valid && sa >= 11 && N >= 8192;
        const int64_t c = use_b ? sb : sa;
        if (M * c <= 64) {
            *variant = use_b ? (b_d3 ? kWide2D3M1T : kWide2D2M1T) : kWide2D2M1T;
            return c;
        }
    }
    if (b_valid) {
        *variant = b_d3 ? kWide2D3M1 : kWide2D2M1;
        return sb;
    }
    if (N % 512 == 0 && (256 / (N / 512)) * (N / 512) >= 230 && K * N >= 80000000ll) return wide512_pass();
    *variant = kWide2D2M1;
    return sa;
}

// 17..32 rows: the shared-chunk kernel on 256 columns per workgroup with two m-tiles (four waves: two or three of
// these smaller workgroups share a CU and run out of step, where the eight waves of a 512-column workgroup pass one
// barrier per chunk together), second pass for the K splits.  Split as for up to 16 rows: about one workgroup per CU
// if that fills 85 % of them (plan B; three buffers where a split has six chunks or more), else about 500 (plan A).
// For N < 28672 and 48 M weights or more -- against the row blocks of the one-tile kernel or the 512-column form at
// 24 / 32 rows: 5120 x 17408 27.6 / 28.9 -> 20.3 / 21.8 us, 17408 x 5120 26.5 / 27.0 -> 21.4 / 22.4, 8192 x 8192
// 22.3 / 22.8 -> 17.0 / 17.8, 5120 x 10240 19.6 / 20.2 -> 16.4 / 16.6, 12288 x 4096 18.5 -> 16.1 / 16.7, 6144 x 8192
// 17.8 / 18.3 -> 15.6 / 16.4, 5120 x 25600 26.6 / 26.8 -> 25.1; 5120 x 51200 stays with 512 columns (44.6 against
// 46.6).
// 33..64 rows: the same with four m-tiles, 244 registers a wave, so two workgroups a CU and one wave of each per SIMD;
// the kernel then takes a chunk step by step.  From 45 M weights (40 M above 48 rows, where the row blocks are four:
// 8192 x 5120 at 64 rows 23.5 -> 22.3 us, at 48 rows 19.2 against 21.7), 3584 columns and K = 3584 on (2560 x 19456 at
// 40 rows 23.4 us against 19.1 in row blocks), any N; plan B with up to 11 chunks a split (with 16, 4096 x 28672
// runs 38.6 us in 224 workgroups and 36.9 in 448 of 8 chunks; 25600 x 5120 at 40 rows 37.6 us in 12 splits of 17
// chunks, 33.7 in 25 of 8; 17408 x 5120 at 40 rows 29.8 us in 12 splits of 12, 27.7 in 23 of 6).  Against the
// 512-column form or the one-tile kernel's row blocks at 64 rows: 8192 x 8192 30.4 -> 26.1 us, 5120 x 10240 27.8 ->
// 23.7, 13824 x 5120 31.4 -> 27.2, 18944 x 3584 31.6 -> 27.7, 8192 x 10240 33.8 -> 29.9, 4096 x 12288 25.9 -> 23.5,
// 5120 x 17408 34.1 -> 32.5, 4096 x 28672 39.6 -> 36.9, 5120 x 25600 40.8 -> 39.1, 5120 x 51200 70.7 -> 65.6; at 40
// and 48 rows equal to 10 % faster (12288 x 4096 at 48 rows 25.0 -> 21.5); 4096 x 8192 and 5120 x 8192 keep the row
// blocks (17.2 and 19.9 against 22.5 and 21.8).
static int64_t pick_shared_256(int64_t M, int64_t N, int64_t K, int64_t chunks, int* variant) {
    if (M > 64 || N % 256 != 0 || chunks < 8) return 0;
    const bool four = M > 32;   // m-tiles: four, else two
    if (four ? (N < 3584 || chunks < 28 || K * N < (M > 48 ? 40000000ll : 45000000ll))
             : (N < 4096 || N >= 28672 || K * N < 48000000ll))
        return 0;
    auto normalised = [&](int64_t c) { return cdiv(chunks, cdiv(chunks, c)); };
    const int64_t groups = N / 256;
    int64_t sb = 256 / groups;
    if (sb > chunks / 4) sb = chunks / 4;
    if (sb >= 2 && normalised(sb) * groups >= (four ? 216 : 218) && (!four || cdiv(chunks, sb) <= 11)) {
        sb = normalised(sb);
        *variant = four ? kWide2D2M4 : (cdiv(chunks, sb) >= 6 ? kWide2D3M2 : kWide2D2M2);
        return sb;
    }
    int64_t sa = 512 / groups;
    if (sa > 25) sa = 25;
    if (sa > chunks / 4) sa = chunks / 4;
    if (sa < 1) return 0;
    *variant = four ? kWide2D2M4 : kWide2D2M2;
    return normalised(sa);
}

static void pick_gemv(int64_t M, int64_t N, int64_t K, int64_t g, int* variant, int* split_k,
                      bool allow_shared_chunk = true) {
    const int64_t chunks = K / 128 > 0 ? K / 128 : 1;
    if (N % 128 == 0 && g % 128 == 0) {
        // From sweeps on MI355X (HBM-streaming): short K runs best as one workgroup of 8 waves per
        // column tile; otherwise 4-wave workgroups, split over K for M <= 4 until ~3000 waves exist
        // (the split's tail grows with M, so larger M splits only to cover the CUs).
        const int64_t tiles = N / 128;
        int v = kDma1x4;
        int64_t s = 1;
        const int64_t row_blocks = cdiv(M, 16);   // above 16 rows the one-m-tile kernels run one block of 16 per z
        // Up to 16 rows on large weights: the one-m-tile forms of the shared-chunk kernel (pick_one_m_tile), 0 = none.
        int64_t m1_splits = 0;
        int m1_variant = 0;
        if (allow_shared_chunk && M <= 16) m1_splits = pick_one_m_tile(M, N, K, chunks, &m1_variant);
        if (allow_shared_chunk && M > 16 && M <= 64) m1_splits = pick_shared_256(M, N, K, chunks, &m1_variant);
        if (m1_splits == 0 && allow_shared_chunk && M > 16 && M <= 64 && N % 512 == 0 && N >= 5120 &&
            K * N >= (M > 48 ? (50ll << 20) : (M > 32 ? 64000000ll : 95000000ll))) {
            // 17..64 rows on the largest weights (from sweeps: the fused gate|up of Qwen3-8B and the MLP of
            // Qwen3-14B/32B and, above 32 rows, the 32B fused q/k/v): eight-wave workgroups of 512 columns sharing the staged chunk, K split so that about
            // one workgroup per CU exists, four chunks per split at least.  Below these sizes re-reading the
            // weights once per block of 16 rows (mostly from cache) is faster than the shared chunk's second pass.
            v = M > 32 ? kWideM4 : kWideM2;
            s = 256 / (N / 512);
            if (s > chunks / 4) s = chunks / 4;
        } else if (m1_splits > 0) {
            v = m1_variant;
            s = m1_splits;
        } else if (chunks <= 8) {
            v = kDma1x8;
        } else if (M <= 4) {
            // About 2048 waves in four-wave workgroups and no more than 16 splits: every split of a tile bumps the
            // same arrival counter, and those updates are served one after the other -- 9728 x 2560 at one row 13.7 us
            // in 26 splits, 10.5 in 14; 17408 x 5120 17.5 us in 20, 16.3 in 13; 12288 x 4096 13.1 us in 24, 12.5 in 16.
            // Eight-wave workgroups, i.e. half the splits for the same waves, on the longest K with few column tiles
            // (25600 x 5120: 22.3 us in 25 splits of four waves, 20.4 in 13 of eight; on shorter K they lose:
            // 4096 x 2048 8.3 us in 4 splits of eight waves against 7.4 in 8 of four).
            // short K: one chunk per wave (the step-by-step form), at most 10 splits (the tail is a larger share of
            // a 6 us launch: 2048 x 1024 at one row 5.55 us in 8 splits, 5.23 in 4)
            // (that limit is for launches of a few microseconds; from 32 Mi weights on up to 16 again: 6144 x 10240
            // at one row 15.4 us in 7 splits, two chunks per wave, 12.9 in 12)
            const int64_t short_cap = K * N >= (32ll << 20) ? 16 : 10;
            const int64_t cap = chunks < 64 ? (chunks / 4 < short_cap ? chunks / 4 : short_cap) : 16;
            int64_t wk = 4;
            s = cdiv(2048, tiles * 4);
            // and no more than two chunks per wave: a wave takes its chunks one after the other, each a round trip
            // of its own (5120 x 51200 at one row 41.5 us in 2 splits -- five chunks per wave --, 32.5 in 5 or 6;
            // 5120 x 34816 32.9 -> 24.9 us)
            if (s < cdiv(chunks, 8) && cdiv(chunks, 8) <= cap) s = cdiv(chunks, 8);
            if (s > cap) s = cap;
            s = balance_splits(chunks, s, wk, cap);
            if (tiles <= 56 && chunks > 64) {
                // (long K, few column tiles: eight-wave workgroups where their split wastes no more wave slots than the
                // four-wave one -- 16384 x 4096 17.6 -> 14.1 us in 16 splits, 14336 x 4096 14.2 -> 13.3, 8192 x 7168
                // 13.1 -> 12.2, 12288 x 4096 12.55 -> 12.2; 17408 x 5120 keeps four waves: 13 splits of 11 chunks are
                // 3, 3, 3, 2 per wave there and 2, 2, 2, 1, 1, 1, 1, 1 on eight: 16.3 against 16.9 us)
                auto wasted = [&](int64_t c, int64_t waves) {
                    const int64_t cps = cdiv(chunks, c), splits = cdiv(chunks, cps);
                    return 1.0 - (double)chunks / (double)(splits * waves * cdiv(cps, waves));
                };
                // (two eight-wave workgroups fit a CU: beyond about 512 of them a third round starts -- 13824 x 5120 in
                // 14 splits, 560 workgroups, 14.9 us against 13.7 in 12 splits of four waves)
                int64_t cap8 = 540 / tiles < cap ? 540 / tiles : cap;
                int64_t s8 = cdiv(4096, tiles * 8);
                if (s8 > cap8) s8 = cap8;
                s8 = balance_splits(chunks, s8, 8, cap8);
                if (wasted(s8, 8) <= wasted(s, 4) + 1e-9) {
                    wk = 8;
                    s = s8;
                    v = kDma1x8;
                }
            } else if (tiles <= 64 && chunks >= 48 && chunks <= 64 &&
                       (tiles * 8 <= 256 || tiles * 8 * 20 >= 256 * cdiv(tiles * 8, 256) * 17)) {
                // 6144 <= K <= 8192 on up to 64 column tiles: eight splits of eight waves, one chunk per wave at most
                // (the step-by-step form) -- 6144 x 4096 10.4 -> 8.8 us, 8192 x 4096 10.0 -> 9.4, 8192 x 2048 9.6 -> 9.0,
                // 7168 x 8192 14.4 -> 13.0 --, where those workgroups come in whole rounds of the CUs (40 or 48 tiles
                // make 1.25 / 1.5 rounds: 8192 x 5120 11.1 -> 11.7, 6144 x 6144 10.5 -> 11.0)
                wk = 8;
                s = 8;
                v = kDma1x8;
            }
        } else {
            // 5..64 rows.  A CU streams at a fixed rate whatever the number of workgroups on it, so the launch lasts
            // as long as the CU with the most bytes: at least about 200 workgroups, and a count that fills whole
            // rounds of the 256 CUs (272 column tiles unsplit = two rounds, the second almost empty: 48.9 us
            // against 34.9 us cut four ways, 5120 x 34816 at 16 rows).  Each further split costs a tail
            // (publish, fetch, add) that grows with the rows of a block, hence the penalty: at 5120 x 25600 five
            // splits win at 8 rows (22.9 against 24.4 us) and lose at 16 (27.4 against 24.7).
            const int64_t wgs = tiles * row_blocks;
            // 65..128 rows (five to eight blocks of 16, small weights only): the blocks fill the chip, a split only
            // adds its tail (2048 x 2048 at 128 rows: 8.6 us unsplit, 9.4 in two)
            const int64_t cap = M > 64 && wgs >= 64 ? 1 : (chunks / 4 > 1 ? chunks / 4 : 1);
            // From 17 rows on, weights under 32 Mi elements (16 MB packed: the linears of Qwen3-1.7B / 4B) are not
            // streaming-bound, and with 144 workgroups or more any split only adds its tail -- 2560 x 9728 at 64 rows
            // 27.2 us in five splits, 16.8 unsplit (304 workgroups); at 32 rows 16.2 -> 13.1; 2048 x 6144 at 64 rows
            // 12.3 -> 9.7, at 48 rows (144 workgroups) 11.9 -> 10.2; likewise four row blocks of 128 tiles or more:
            // 2560 x 19456 at 64 rows 33.4 -> 23.4.
            const bool unsplit = row_blocks >= 2 && wgs >= 144 &&
                                 (K * N < (32ll << 20) || (row_blocks >= 4 && wgs >= 512));
            int64_t s0 = wgs < 200 ? cdiv(200, wgs) : 1;
            if (s0 > cap) s0 = cap;
            const int64_t hi = s0 + 5 < cap ? s0 + 5 : cap;
            double best_score = -1.0;
            for (int64_t c = s0; c <= hi; ++c) {
                const int64_t cps = cdiv(chunks, c), splits = cdiv(chunks, cps);
                const double eff_wave = (double)chunks / (double)(splits * 4 * cdiv(cps, 4));
                const double eff_cu = (double)(wgs * splits) / (double)(256 * cdiv(wgs * splits, 256));
                // (the tail is a cost per launch, the imbalance a share of it: on weights beyond 32 Mi elements the
                // penalty shrinks in proportion -- 5120 x 51200 at 16 rows ran 50.9 us unsplit, 400 workgroups on 256
                // CUs, against 40.3 us at 8 rows in five splits)
                const double big = (double)(K * N) / (double)(32ll << 20);
                const double score = eff_wave * eff_cu -
                                     0.05 * (double)(M < 16 ? M : 16) / 16.0 * (double)(c - s0) / (big > 1.0 ? big : 1.0);
                if (score > best_score + 1e-9) {
                    best_score = score;
                    s = c;
                }
            }
            if (unsplit) s = 1;
            // K of 4096..8192: eight-wave workgroups with one chunk per wave (the step-by-step form) where they make
            // 150..256 workgroups, at most one per CU -- 4096 x 2560 at 32 rows 12.7 -> 9.9 us, 4096 x 8192 at 16 rows
            // 11.6 -> 10.9, 8192 x 4096 at 8 rows 11.9 -> 10.5, 5120 x 5120 at 8 rows 10.8 -> 10.0; with more
            // workgroups than that the four-wave split is faster (4096 x 8192 at 32 rows 14.6 against 17.3 us).
            if (chunks >= 32 && chunks <= 64 && row_blocks <= 2) {
                const int64_t s8 = cdiv(chunks, 8);
                if (wgs * s8 >= 150 && wgs * s8 <= 256) {
                    v = kDma1x8;
                    s = s8;
                }
            }
        }
        if (s < 1) s = 1;
        *variant = v;
        *split_k = (int)s;
        return;
    }
    const bool wide = (N % 16 == 0) && N >= 4096;
    const int v = wide ? kV2W4 : kV1W4P;
    const GemvVariant& gv = kGemvVariants[v];
    const int64_t tiles = cdiv(N / 8, 16 * gv.V);
    int64_t s = cdiv(512, tiles);
    const int64_t max_s = chunks / gv.waves > 0 ? chunks / gv.waves : 1;
    if (s > max_s) s = max_s;
    if (s < 1) s = 1;
    if (s > 32) s = 32;
    *variant = v;
    *split_k = (int)s;
}

static int gemv_dispatch(const char* fn, const void* x, const int32_t* qweight, const void* qscales,
                         const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                         int64_t K, int64_t g, int dtype, void* workspace, size_t workspace_bytes,
                         void* stream, int variant, int split_k, int act = 0,
                         const GemvFusion& fu = GemvFusion{}) {
    // Pending prefetch hints belong to this call whatever becomes of it: they are taken before any check, ride on
    // the one-tile staged launch, and are dropped by every other kernel and by every error return.
    PrefetchRegions pf;
    take_prefetch_hint(&pf);
    int rc = check_linear_args(fn, x, qweight, qscales, qzeros, y, M, N, K, g, dtype);
    if (rc != AWQ_OK) return rc;
    if (act && (variant < kFirstDmaVariant || bias)) {
        set_error("%s: the gated epilogue runs on the staged path only (N %% 128 == 0, group_size %% 128 == 0) "
                  "and takes no bias", fn);
        return AWQ_ERR_UNSUPPORTED;
    }
    if ((act == 2) != (fu.qe != nullptr) || (fu.re && (act || fu.np || bias))) {
        set_error("%s: inconsistent epilogue arguments", fn);
        return AWQ_ERR_INVALID_ARG;
    }
    // the q|k|v epilogue also runs in the second pass of a K-split shared-chunk plan (no norm prologue there)
    const bool wide_second_pass = variant >= 0 && variant < kNumGemvVariants && kGemvVariants[variant].wide &&
                                  kGemvVariants[variant].name[strlen(kGemvVariants[variant].name) - 1] != 't' &&
                                  split_k >= 2;
    const bool qkv_second_pass = fu.qe && !fu.np && !fu.re && wide_second_pass && N % 128 == 0;
    const int wide_act = qkv_second_pass ? 0 : act;   // the main kernel of such a launch only writes partials
    if (fu.any() && !qkv_second_pass &&
        (variant < kFirstDmaVariant || variant >= kNumGemvVariants || kGemvVariants[variant].wide ||
         kGemvVariants[variant].wn != 1)) {
        set_error("%s: the q|k|v / residual epilogues and the RMSNorm prologue run on the one-tile-per-workgroup "
                  "staged kernels only (N %% 128 == 0, group_size %% 128 == 0)", fn);
        return AWQ_ERR_UNSUPPORTED;
    }
    if (fu.an) {
        if (!wide_second_pass || bias || act || fu.any() || N > 8192 || N % 8 != 0) {
            set_error("%s: the residual add + RMSNorm second pass needs a K-split shared-chunk plan (see awq_gemv_plan), "
                      "no bias and N <= 8192", fn);
            return AWQ_ERR_UNSUPPORTED;
        }
    }
    if (M > kGemvMaxRows) {
        set_error("%s: M=%lld is outside the decode regime (1..%d); use awq_gemm", fn, (long long)M, kGemvMaxRows);
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
    const bool staged = variant >= kFirstDmaVariant;
    // 17..64 rows: blocks of 16 on the one-tile staged kernels, up to 16 * mt on the shared-chunk kernel
    const bool row_blocked = staged && !gv.wide;
    if (M > 16 * gv.mt && !row_blocked) {
        set_error("%s: variant %s takes at most %d rows (M=%lld); rows 17..64 need the staged path "
                  "(N %% 128 == 0, group_size %% 128 == 0)", fn, gv.name, 16 * gv.mt, (long long)M);
        return AWQ_ERR_UNSUPPORTED;
    }
    if ((N / 8) % gv.V != 0) {
        set_error("%s: variant %s needs N %% %d == 0 (N=%lld)", fn, gv.name, 8 * gv.V, (long long)N);
        return AWQ_ERR_UNSUPPORTED;
    }
    if (staged && (N % (128 * gv.wn) != 0 || g % 128 != 0)) {
        set_error("%s: variant %s needs N %% %d == 0 and group_size %% 128 == 0", fn, gv.name, 128 * gv.wn);
        return AWQ_ERR_UNSUPPORTED;
    }
    if (split_k > 1 && cdiv(N / 8, 16 * gv.V) * (row_blocked ? cdiv(M, 16) : 1) > kMaxSplitTiles) {
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
    const int Mi = (int)M, Ni = (int)N, Ki = (int)K, gi = (int)g;
    const bool f16 = dtype == AWQ_F16;
    switch (variant) {
        case kWideM4:
            e = f16 ? launch_gemv_wide<F16, 2, 4>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe)
                    : launch_gemv_wide<BF16, 2, 4>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe);
            break;
        case kWideM1:
            e = f16 ? launch_gemv_wide<F16, 2, 1>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe)
                    : launch_gemv_wide<BF16, 2, 1>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe);
            break;
        case kWideM1T:
            e = f16 ? launch_gemv_wide<F16, 2, 1, true>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe)
                    : launch_gemv_wide<BF16, 2, 1, true>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe);
            break;
#define AWQ_WIDE2_CASE(ID, DD, TT)                                                                                      \
        case ID:                                                                                                        \
            e = f16 ? launch_gemv_wide<F16, DD, 1, TT, 2>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe) \
                    : launch_gemv_wide<BF16, DD, 1, TT, 2>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe); \
            break;
        AWQ_WIDE2_CASE(kWide2D2M1, 2, false)
        AWQ_WIDE2_CASE(kWide2D2M1T, 2, true)
        AWQ_WIDE2_CASE(kWide2D3M1, 3, false)
        AWQ_WIDE2_CASE(kWide2D3M1T, 3, true)
#undef AWQ_WIDE2_CASE
#define AWQ_WIDE2M_CASE(ID, DD, MM)                                                                                     \
        case ID:                                                                                                        \
            e = f16 ? launch_gemv_wide<F16, DD, MM, false, 2>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe) \
                    : launch_gemv_wide<BF16, DD, MM, false, 2>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe); \
            break;
        AWQ_WIDE2M_CASE(kWide2D2M2, 2, 2)
        AWQ_WIDE2M_CASE(kWide2D3M2, 3, 2)
        AWQ_WIDE2M_CASE(kWide2D2M4, 2, 4)
#undef AWQ_WIDE2M_CASE
        case kWideD3M1T:
            e = f16 ? launch_gemv_wide<F16, 3, 1, true>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe)
                    : launch_gemv_wide<BF16, 3, 1, true>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe);
            break;
        case kWideD3M1:
            e = f16 ? launch_gemv_wide<F16, 3, 1, false>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe)
                    : launch_gemv_wide<BF16, 3, 1, false>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe);
            break;
        case kWideM2:
            e = f16 ? launch_gemv_wide<F16, 2, 2>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe)
                    : launch_gemv_wide<BF16, 2, 2>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, wide_act, fu.an, fu.qe);
            break;
        case kDma1x4:
            e = f16 ? launch_gemv_dma<F16, 4>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, act, pf, fu)
                    : launch_gemv_dma<BF16, 4>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, act, pf, fu);
            break;
        case kDma1x8:
            e = f16 ? launch_gemv_dma<F16, 8>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, act, pf, fu)
                    : launch_gemv_dma<BF16, 8>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s, act, pf, fu);
            break;
        default: {
            // register path; group sizes 32/64/96...: one 32-row step per chunk, always with the next chunk prefetched
            const bool big_chunk = chunk_steps(g) == 4;
#define AWQ_GEMV_LAUNCH(TT, VV, CC, PP) \
    launch_gemv<TT, VV, 4, CC, PP>(x, qweight, qscales, qzeros, bias, y, Mi, Ni, Ki, gi, workspace, split_k, s)
            if (variant == kV1W4P)
                e = big_chunk ? (f16 ? AWQ_GEMV_LAUNCH(F16, 1, 4, true) : AWQ_GEMV_LAUNCH(BF16, 1, 4, true))
                              : (f16 ? AWQ_GEMV_LAUNCH(F16, 1, 1, true) : AWQ_GEMV_LAUNCH(BF16, 1, 1, true));
            else
                e = big_chunk ? (f16 ? AWQ_GEMV_LAUNCH(F16, 2, 4, false) : AWQ_GEMV_LAUNCH(BF16, 2, 4, false))
                              : (f16 ? AWQ_GEMV_LAUNCH(F16, 2, 1, true) : AWQ_GEMV_LAUNCH(BF16, 2, 1, true));
#undef AWQ_GEMV_LAUNCH
        }
    }
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

}  // namespace awq

extern "C" int awq_gemv_variant_count(void) { return awq::kNumGemvVariants; }

extern "C" const char* awq_gemv_variant_name(int variant) {
    return (variant >= 0 && variant < awq::kNumGemvVariants) ? awq::kGemvVariants[variant].name : "";
}

extern "C" int awq_gemv_plan(int64_t M, int64_t N, int64_t K, int64_t group_size, int* variant, int* split_k) {
    if (!variant || !split_k || M < 1 || M > awq::kGemvMaxRows || N < 8 || N % 8 != 0 || K < 32 || group_size < 32 ||
        group_size % 32 != 0 || K % group_size != 0) {
        awq::set_error("awq_gemv_plan: not a shape awq_gemv takes (M=%lld N=%lld K=%lld g=%lld)", (long long)M,
                       (long long)N, (long long)K, (long long)group_size);
        return AWQ_ERR_UNSUPPORTED;
    }
    awq::pick_gemv(M, N, K, group_size, variant, split_k);
    if (M > 16 && *variant < awq::kFirstDmaVariant) {
        awq::set_error("awq_gemv_plan: rows 17..64 need the staged path (N %% 128 == 0, group_size %% 128 == 0)");
        return AWQ_ERR_UNSUPPORTED;
    }
    return AWQ_OK;
}

extern "C" size_t awq_gemv_ex_workspace_bytes(int64_t M, int64_t N, int64_t K, int variant,
                                              int split_k) {
    if (variant < 0 || variant >= awq::kNumGemvVariants || split_k < 1 || K < 32 || N < 8 || M < 1) return 0;
    return awq::gemv_ws_bytes(M, N, K, variant, split_k);
}

extern "C" size_t awq_gemv_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (K < 32 || N < 8 || M < 1) return 0;
    int v, s;
    // the caller passes neither the group size nor the entry point: cover both data paths, and the staged path
    // with and without the shared-chunk kernel (the fused forms never take it)
    size_t need = 0;
    for (int form = 0; form < 3; ++form) {
        awq::pick_gemv(M, N, K, form == 2 ? 32 : 128, &v, &s, form != 1);
        const size_t b = awq::gemv_ws_bytes(M, N, K, v, s);
        if (b > need) need = b;
    }
    return need;
}

extern "C" int awq_gemv_swiglu(const void* x, const int32_t* qweight, const void* qscales,
                               const int32_t* qzeros, void* y, int64_t M, int64_t N, int64_t K,
                               int64_t group_size, int dtype, void* workspace, size_t workspace_bytes,
                               void* stream) {
    int v = 0, s = 1;
    if (K >= 32 && N >= 8 && group_size > 0) awq::pick_gemv(M, N, K, group_size, &v, &s);
    return awq::gemv_dispatch("awq_gemv_swiglu", x, qweight, qscales, qzeros, nullptr, y, M, N, K, group_size,
                              dtype, workspace, workspace_bytes, stream, v, s, 1);
}

namespace awq {
// error return of an entry point that has not reached gemv_dispatch: pending prefetch hints go with it
static int fail_drop(int rc) {
    PrefetchRegions dropped;
    take_prefetch_hint(&dropped);
    return rc;
}

static int make_norm_prologue(const char* fn, const float* ssq, const void* norm_weight, float norm_eps, int64_t M,
                              NormPrologue* np) {
    if (!ssq || !norm_weight) {
        set_error("%s: null pointer argument", fn);
        return fail_drop(AWQ_ERR_INVALID_ARG);
    }
    if ((reinterpret_cast<uintptr_t>(norm_weight) & 15u) || (reinterpret_cast<uintptr_t>(ssq) & 3u)) {
        set_error("%s: the norm weight must be 16-byte aligned, the sums of squares 4-byte aligned", fn);
        return fail_drop(AWQ_ERR_INVALID_ARG);
    }
    np->weight = reinterpret_cast<const uint16_t*>(norm_weight);
    np->ssq = ssq;
    np->m_stride = (int)M;
    np->eps = norm_eps;
    return AWQ_OK;
}

static int qkv_rope_store_entry(const char* fn, const void* x, const NormPrologue* np, const int32_t* qweight,
                                const void* qscales, const int32_t* qzeros, const void* q_weight, const void* k_weight,
                                const float* cos_sin, const int64_t* positions, const int64_t* slots, void* q_out,
                                void* k_cache, void* v_cache, int64_t M, int64_t N, int64_t K, int64_t group_size,
                                int64_t num_heads, int64_t num_kv_heads, int64_t max_positions, int64_t num_slots,
                                int64_t block_size, float eps, int dtype, void* workspace, size_t workspace_bytes,
                                void* stream) {
    if (!q_weight || !k_weight || !cos_sin || !positions || !slots || !q_out || !k_cache || !v_cache) {
        set_error("%s: null pointer argument", fn);
        return fail_drop(AWQ_ERR_INVALID_ARG);
    }
    if ((reinterpret_cast<uintptr_t>(q_weight) | reinterpret_cast<uintptr_t>(k_weight) |
         reinterpret_cast<uintptr_t>(cos_sin) | reinterpret_cast<uintptr_t>(q_out) |
         reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache)) & 15u) {
        set_error("%s: every tensor must be 16-byte aligned", fn);
        return fail_drop(AWQ_ERR_INVALID_ARG);
    }
    if (num_heads <= 0 || num_kv_heads <= 0 || N != (num_heads + 2 * num_kv_heads) * 128 || max_positions <= 0 ||
        max_positions > 0x7fffffff || block_size <= 0 || block_size > 0x7fffffff || num_slots <= 0 ||
        num_slots % block_size != 0) {
        set_error("%s: needs head_dim 128 (N == (num_heads + 2 * num_kv_heads) * 128), positive max_positions and "
                  "block_size, and num_slots a multiple of block_size", fn);
        return fail_drop(AWQ_ERR_INVALID_ARG);
    }
    QkvEpilogue qe;
    qe.q_weight = reinterpret_cast<const uint16_t*>(q_weight);
    qe.k_weight = reinterpret_cast<const uint16_t*>(k_weight);
    qe.cos_sin = cos_sin;
    qe.positions = positions;
    qe.slots = slots;
    qe.q_out = reinterpret_cast<uint16_t*>(q_out);
    qe.k_cache = reinterpret_cast<uint16_t*>(k_cache);
    qe.v_cache = reinterpret_cast<uint16_t*>(v_cache);
    qe.nh = (int)num_heads;
    qe.nkv = (int)num_kv_heads;
    qe.max_positions = (int)max_positions;
    qe.block_size = (int)block_size;
    qe.num_slots = num_slots;
    qe.eps = eps;
    int v = 0, s = 1;
    if (K >= 32 && N >= 8 && group_size > 0) {
        // From 17 rows on, where the plain GEMV of this weight is a K-split shared-chunk launch, the epilogue runs in
        // its second pass (Qwen3-32B q|k|v, 5120 x 10240, at 64 rows: 32.4 us in four blocks of 16 rows on the
        // one-tile kernel); with the norm prologue and below, the one-tile kernels.
        bool second_pass = false;
        if (!np && M > 16) {
            pick_gemv(M, N, K, group_size, &v, &s, true);
            const char* name = kGemvVariants[v].name;
            second_pass = kGemvVariants[v].wide && name[strlen(name) - 1] != 't' && s >= 2;
        }
        if (!second_pass) pick_gemv(M, N, K, group_size, &v, &s, false);
    }
    GemvFusion fu;
    fu.qe = &qe;
    fu.np = np;
    return gemv_dispatch(fn, x, qweight, qscales, qzeros, nullptr, q_out, M, N, K, group_size, dtype, workspace,
                         workspace_bytes, stream, v, s, 2, fu);
}
}  // namespace awq

extern "C" int awq_gemv_qkv_rope_store(const void* x, const int32_t* qweight, const void* qscales,
                                       const int32_t* qzeros, const void* q_weight, const void* k_weight,
                                       const float* cos_sin, const int64_t* positions, const int64_t* slots,
                                       void* q_out, void* k_cache, void* v_cache, int64_t M, int64_t N, int64_t K,
                                       int64_t group_size, int64_t num_heads, int64_t num_kv_heads,
                                       int64_t max_positions, int64_t num_slots, int64_t block_size, float eps,
                                       int dtype, void* workspace, size_t workspace_bytes, void* stream) {
    return awq::qkv_rope_store_entry("awq_gemv_qkv_rope_store", x, nullptr, qweight, qscales, qzeros, q_weight,
                                     k_weight, cos_sin, positions, slots, q_out, k_cache, v_cache, M, N, K, group_size,
                                     num_heads, num_kv_heads, max_positions, num_slots, block_size, eps, dtype,
                                     workspace, workspace_bytes, stream);
}

extern "C" int awq_gemv_rmsnorm_qkv_rope_store(const void* x, const float* ssq, const void* norm_weight,
                                               float norm_eps, const int32_t* qweight, const void* qscales,
                                               const int32_t* qzeros, const void* q_weight, const void* k_weight,
                                               const float* cos_sin, const int64_t* positions, const int64_t* slots,
                                               void* q_out, void* k_cache, void* v_cache, int64_t M, int64_t N,
                                               int64_t K, int64_t group_size, int64_t num_heads, int64_t num_kv_heads,
                                               int64_t max_positions, int64_t num_slots, int64_t block_size, float eps,
                                               int dtype, void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "awq_gemv_rmsnorm_qkv_rope_store";
    awq::NormPrologue np;
    const int rc = awq::make_norm_prologue(fn, ssq, norm_weight, norm_eps, M, &np);
    if (rc != AWQ_OK) return rc;
    return awq::qkv_rope_store_entry(fn, x, &np, qweight, qscales, qzeros, q_weight, k_weight, cos_sin, positions,
                                     slots, q_out, k_cache, v_cache, M, N, K, group_size, num_heads, num_kv_heads,
                                     max_positions, num_slots, block_size, eps, dtype, workspace, workspace_bytes,
                                     stream);
}

extern "C" int awq_gemv_rmsnorm(const void* x, const float* ssq, const void* norm_weight, float norm_eps,
                                const int32_t* qweight, const void* qscales, const int32_t* qzeros, void* y,
                                int64_t M, int64_t N, int64_t K, int64_t group_size, int gated, int dtype,
                                void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "awq_gemv_rmsnorm";
    awq::NormPrologue np;
    const int rc = awq::make_norm_prologue(fn, ssq, norm_weight, norm_eps, M, &np);
    if (rc != AWQ_OK) return rc;
    int v = 0, s = 1;
    if (K >= 32 && N >= 8 && group_size > 0) awq::pick_gemv(M, N, K, group_size, &v, &s, false);
    awq::GemvFusion fu;
    fu.np = &np;
    return awq::gemv_dispatch(fn, x, qweight, qscales, qzeros, nullptr, y, M, N, K, group_size, dtype, workspace,
                              workspace_bytes, stream, v, s, gated ? 1 : 0, fu);
}

extern "C" int awq_gemv_add_residual(const void* x, const int32_t* qweight, const void* qscales,
                                     const int32_t* qzeros, void* residual, float* ssq, int64_t M, int64_t N,
                                     int64_t K, int64_t group_size, int dtype, void* workspace,
                                     size_t workspace_bytes, void* stream) {
    const char* fn = "awq_gemv_add_residual";
    if (!ssq || (reinterpret_cast<uintptr_t>(ssq) & 3u)) {
        awq::set_error("%s: ssq must be a 4-byte aligned device pointer", fn);
        return awq::fail_drop(AWQ_ERR_INVALID_ARG);
    }
    awq::ResidEpilogue re;
    re.ssq = ssq;
    re.m_stride = (int)M;
    int v = 0, s = 1;
    if (K >= 32 && N >= 8 && group_size > 0) awq::pick_gemv(M, N, K, group_size, &v, &s, false);
    awq::GemvFusion fu;
    fu.re = &re;
    return awq::gemv_dispatch(fn, x, qweight, qscales, qzeros, nullptr, residual, M, N, K, group_size, dtype,
                              workspace, workspace_bytes, stream, v, s, 0, fu);
}

extern "C" int awq_gemv_add_rmsnorm(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                                    void* residual, const void* norm_weight, float norm_eps, void* normed, int64_t M,
                                    int64_t N, int64_t K, int64_t group_size, int dtype, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    const char* fn = "awq_gemv_add_rmsnorm";
    if (!norm_weight || !normed || ((reinterpret_cast<uintptr_t>(norm_weight) | reinterpret_cast<uintptr_t>(normed)) & 15u)) {
        awq::set_error("%s: norm_weight and normed must be 16-byte aligned device pointers", fn);
        return awq::fail_drop(AWQ_ERR_INVALID_ARG);
    }
    int v = 0, s = 1;
    if (K >= 32 && N >= 8 && group_size > 0 && M >= 1) awq::pick_gemv(M, N, K, group_size, &v, &s);
    awq::AddNorm an{reinterpret_cast<const uint16_t*>(norm_weight), reinterpret_cast<uint16_t*>(normed), norm_eps};
    awq::GemvFusion fu;
    fu.an = &an;
    return awq::gemv_dispatch(fn, x, qweight, qscales, qzeros, nullptr, residual, M, N, K, group_size, dtype,
                              workspace, workspace_bytes, stream, v, s, 0, fu);
}

extern "C" int awq_gemv_ex(const void* x, const int32_t* qweight, const void* qscales,
                           const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                           int64_t K, int64_t group_size, int dtype, void* workspace,
                           size_t workspace_bytes, void* stream, int variant, int split_k) {
    return awq::gemv_dispatch("awq_gemv_ex", x, qweight, qscales, qzeros, bias, y, M, N, K,
                              group_size, dtype, workspace, workspace_bytes, stream, variant,
                              split_k);
}

// ---- awq_gemv without any allocation: the split-K scratch is a static device array ----------------------------
// Zero at load, and every launch leaves its arrival counters at zero again (the last workgroup of a tile resets its
// counter), so the counters need no clearing between calls; the partials are written before they are read.
namespace awq {
constexpr size_t kStaticScratchBytes = kCounterBytes + ((size_t)16 << 20);
constexpr int kMaxScratchDevices = 64;
}  // namespace awq
static __device__ __align__(256) unsigned char scratch[awq::kStaticScratchBytes];

namespace awq {
// Device address of `scratch` on the current device, looked up once per device (every device has its own copy of
// the array at its own address); nullptr with the error text set on failure.
static void* static_scratch_ptr(const char* fn) {
    static void* ptrs[kMaxScratchDevices] = {};
    static std::mutex mu;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        hip_fail(fn, e);
        return nullptr;
    }
    if (dev < 0 || dev >= kMaxScratchDevices) {
        set_error("%s: device index %d outside 0..%d", fn, dev, kMaxScratchDevices - 1);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            hip_fail(fn, e != hipSuccess ? e : hipErrorInvalidSymbol);
            return nullptr;
        }
        ptrs[dev] = p;
    }
    return ptrs[dev];
}
}  // namespace awq

extern "C" size_t awq_gemv_static_scratch_bytes(void) { return awq::kStaticScratchBytes; }

extern "C" int awq_gemv_static(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                               const void* bias, void* y, int64_t M, int64_t N, int64_t K, int64_t group_size,
                               int dtype, void* stream) {
    const char* fn = "awq_gemv_static";
    int v = 0, s = 1;
    if (K >= 32 && N >= 8 && group_size > 0 && M >= 1) awq::pick_gemv(M, N, K, group_size, &v, &s);
    const size_t need = (K >= 32 && N >= 8 && M >= 1) ? awq::gemv_ws_bytes(M, N, K, v, s) : 0;
    if (need > awq::kStaticScratchBytes) {
        awq::set_error("%s: M=%lld N=%lld K=%lld needs %zu bytes of split-K scratch, the static buffer holds %zu; "
                       "use awq_gemv with a caller-provided workspace", fn, (long long)M, (long long)N, (long long)K,
                       need, awq::kStaticScratchBytes);
        return awq::fail_drop(AWQ_ERR_UNSUPPORTED);
    }
    void* ws = nullptr;
    if (need > 0) {
        ws = awq::static_scratch_ptr(fn);
        if (!ws) return awq::fail_drop(AWQ_ERR_HIP);
    }
    return awq::gemv_dispatch(fn, x, qweight, qscales, qzeros, bias, y, M, N, K, group_size, dtype, ws,
                              need > 0 ? awq::kStaticScratchBytes : 0, stream, v, s);
}

extern "C" int awq_gemv(const void* x, const int32_t* qweight, const void* qscales,
                        const int32_t* qzeros, const void* bias, void* y, int64_t M, int64_t N,
                        int64_t K, int64_t group_size, int dtype, void* workspace,
                        size_t workspace_bytes, void* stream) {
    int v = 0, s = 1;
    if (K >= 32 && N >= 8 && group_size > 0) awq::pick_gemv(M, N, K, group_size, &v, &s);
    return awq::gemv_dispatch("awq_gemv", x, qweight, qscales, qzeros, bias, y, M, N, K, group_size,
                              dtype, workspace, workspace_bytes, stream, v, s);
}
