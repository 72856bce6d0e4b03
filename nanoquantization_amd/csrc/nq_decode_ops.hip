// Kernels of the decode step that sit between the AWQ linears of a Qwen3 block:
// residual-add + RMSNorm, per-head q/k RMSNorm + rotary + KV-cache write, attention over
// the paged KV cache, and SiLU(gate)*up.  All of them are HBM/latency bound byte movers;
// arithmetic is fp32 with the rounding points of the torch modules they stand in for.
#include "awq_common.hpp"
#include "../../include/nq_engine_ops.h"

namespace awq {
namespace {

constexpr float kLog2e = 1.4426950408889634f;

template <typename T>
__device__ __forceinline__ void unpack8(u32x4 v, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w = v[i];
        f[2 * i] = T::to_f32((uint16_t)(w & 0xFFFFu));
        f[2 * i + 1] = T::to_f32((uint16_t)(w >> 16));
    }
}
template <typename T>
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (uint32_t)T::from_f32(f[2 * i]) | ((uint32_t)T::from_f32(f[2 * i + 1]) << 16);
    return v;
}
template <typename T>
__device__ __forceinline__ float round_to(float f) { return T::to_f32(T::from_f32(f)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// ---------------------------------------------------------------------------------------------
// residual (+= delta); y = RMSNorm(residual) * weight.  One workgroup per row, 8 values per lane
// and pass, at most 4 passes (hidden <= 8192).  The sum of squares is built per 128-column tile
// (tile_ssq) and the tiles are added in index order: the order the AWQ GEMVs with a residual epilogue
// and an RMSNorm prologue use, so both routes give the same bits.
constexpr int kNormThreads = 256;
constexpr int kNormPasses = 4;
constexpr int kNormTiles = kNormPasses * kNormThreads / 16;

// Loads the row (adding and storing delta if given), leaves the tile sums in s_tile and returns their total.
template <typename T>
__device__ __forceinline__ float row_load_ssq(uint16_t* __restrict__ residual, const uint16_t* __restrict__ delta,
                                              int64_t base, int hidden, float (&v)[kNormPasses][8], float* s_tile) {
#pragma unroll
    for (int p = 0; p < kNormPasses; ++p) {
        const int i = (p * kNormThreads + threadIdx.x) * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[p][e] = 0.f;
        if (i < hidden) {
            unpack8<T>(*reinterpret_cast<const u32x4*>(residual + base + i), v[p]);
            if (delta) {
                float d[8];
                unpack8<T>(*reinterpret_cast<const u32x4*>(delta + base + i), d);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[p][e] = round_to<T>(v[p][e] + d[e]);
                *reinterpret_cast<u32x4*>(residual + base + i) = pack8<T>(v[p]);
            }
        }
        const float ts = tile_ssq(v[p]);   // every lane takes part; lanes past the row add zeros
        if ((threadIdx.x & 15) == 0) s_tile[p * (kNormThreads / 16) + (threadIdx.x >> 4)] = ts;
    }
    __syncthreads();
    const int tiles = (hidden + 127) >> 7;
    float tot = 0.f;
    for (int t = 0; t < tiles; ++t) tot += s_tile[t];
    return tot;
}

template <typename T>
__global__ __launch_bounds__(kNormThreads) void add_rmsnorm_kernel(uint16_t* __restrict__ residual,
                                                                  const uint16_t* __restrict__ delta,
                                                                  const uint16_t* __restrict__ weight,
                                                                  uint16_t* __restrict__ y, int hidden, float eps) {
    __shared__ float s_tile[kNormTiles];
    const int64_t base = (int64_t)blockIdx.x * hidden;
    float v[kNormPasses][8];
    u32x4 wraw[kNormPasses];   // the weight does not depend on the reduction: fetched up front
#pragma unroll
    for (int p = 0; p < kNormPasses; ++p) {
        const int i = (p * kNormThreads + threadIdx.x) * 8;
        if (i < hidden) wraw[p] = *reinterpret_cast<const u32x4*>(weight + i);
    }
    const float tot = row_load_ssq<T>(residual, delta, base, hidden, v, s_tile);
    const float r = rsqrtf(tot / (float)hidden + eps);
#pragma unroll
    for (int p = 0; p < kNormPasses; ++p) {
        const int i = (p * kNormThreads + threadIdx.x) * 8;
        if (i < hidden) {
            float w[8], o[8];
            unpack8<T>(wraw[p], w);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = mul_round<T>(v[p][e], r) * w[e];
            *reinterpret_cast<u32x4*>(y + base + i) = pack8<T>(o);
        }
    }
}

// ssq[tile][row] = sum of squares of x[row, 128 tile .. 128 tile + 127]: the statistics an AWQ GEMV with an
// RMSNorm prologue reads, for a residual stream that no GEMV with a residual epilogue has produced yet.
// With `ids` the row is gathered from a table first (row ids[r] of `x`, clamped to the table) and copied to x_out:
// the embedding lookup of a decode step and its statistics in one launch.
template <typename T>
__global__ __launch_bounds__(kNormThreads) void row_ssq_kernel(const uint16_t* __restrict__ x, float* __restrict__ ssq,
                                                              int rows, int hidden, const int64_t* __restrict__ ids,
                                                              int64_t table_rows, uint16_t* __restrict__ x_out) {
    __shared__ float s_tile[kNormTiles];
    float v[kNormPasses][8];
    int64_t src = blockIdx.x;
    if (ids) {
        src = ids[blockIdx.x];
        src = src < 0 ? 0 : (src >= table_rows ? table_rows - 1 : src);
    }
    row_load_ssq<T>(const_cast<uint16_t*>(x), nullptr, src * hidden, hidden, v, s_tile);
    const int tiles = (hidden + 127) >> 7;
    if ((int)threadIdx.x < tiles) ssq[(size_t)threadIdx.x * rows + blockIdx.x] = s_tile[threadIdx.x];
    if (x_out) {
#pragma unroll
        for (int p = 0; p < kNormPasses; ++p) {
            const int i = (p * kNormThreads + threadIdx.x) * 8;
            if (i < hidden) *reinterpret_cast<u32x4*>(x_out + (int64_t)blockIdx.x * hidden + i) = pack8<T>(v[p]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// One wave per (token row, head) of the fused q|k|v projection output.  q and k heads: RMSNorm over
// the head, then the half-split rotary at the row's position; q goes to q_out, k to its cache
// slot; v heads are copied to their cache slot.  A lane owns the rotary pairs (i, i + hd/2).
// Cache layout [blocks][kv heads][block_size][head_dim]: slot s is token s % block_size of block s / block_size.
constexpr int kMaxPairs = 2;  // head_dim <= 256

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_store_kernel(
    const uint16_t* __restrict__ qkv, const uint16_t* __restrict__ q_weight, const uint16_t* __restrict__ k_weight,
    const float* __restrict__ cos_sin, const int64_t* __restrict__ positions, const int64_t* __restrict__ slots,
    uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_out, uint16_t* __restrict__ k_cache,
    uint16_t* __restrict__ v_cache, int rows, int nh, int nkv, int hd, int max_positions, int64_t num_slots,
    int block_size, float eps) {
    const int heads = nh + 2 * nkv;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (int64_t)rows * heads) return;
    const int row = (int)(item / heads), h = (int)(item % heads), lane = threadIdx.x & 63, half = hd >> 1;
    const uint16_t* src = qkv + ((int64_t)row * heads + h) * hd;
    const int64_t slot = slots[row];
    const bool slot_ok = slot >= 0 && slot < num_slots;
    uint16_t* dst;
    uint16_t* dst2 = nullptr;   // dense copy of a normalised, rotated k head (prefill attention reads it)
    if (h < nh) {
        dst = q_out + ((int64_t)row * nh + h) * hd;
    } else if (h < nh + nkv) {
        if (k_out) dst2 = k_out + ((int64_t)row * nkv + (h - nh)) * hd;
        if (!slot_ok) {
            if (!dst2) return;
            dst = dst2;
            dst2 = nullptr;
        } else {
            dst = k_cache + (((slot / block_size) * nkv + (h - nh)) * block_size + slot % block_size) * hd;
        }
    } else {
        if (!slot_ok) return;
        dst = v_cache + (((slot / block_size) * nkv + (h - nh - nkv)) * block_size + slot % block_size) * hd;
    }
    float a[kMaxPairs], b[kMaxPairs];
    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < kMaxPairs; ++p) {
        const int i = p * 64 + lane;
        a[p] = b[p] = 0.f;
        if (i < half) {
            a[p] = T::to_f32(src[i]);
            b[p] = T::to_f32(src[i + half]);
            ss += a[p] * a[p] + b[p] * b[p];
        }
    }
    if (h >= nh + nkv) {  // v: plain copy
#pragma unroll
        for (int p = 0; p < kMaxPairs; ++p) {
            const int i = p * 64 + lane;
            if (i < half) {
                dst[i] = src[i];
                dst[i + half] = src[i + half];
            }
        }
        return;
    }
    // norm weight and angles do not depend on the reduction: fetched before it
    const uint16_t* w = h < nh ? q_weight : k_weight;
    int64_t pos = positions[row];
    pos = pos < 0 ? 0 : (pos >= max_positions ? max_positions - 1 : pos);
    const float* cs = cos_sin + pos * hd;
    float w1[kMaxPairs], w2[kMaxPairs], cc[kMaxPairs], sn[kMaxPairs];
#pragma unroll
    for (int p = 0; p < kMaxPairs; ++p) {
        const int i = p * 64 + lane;
        w1[p] = w2[p] = cc[p] = sn[p] = 0.f;
        if (i < half) {
            w1[p] = T::to_f32(w[i]);
            w2[p] = T::to_f32(w[i + half]);
            cc[p] = cs[i];
            sn[p] = cs[i + half];
        }
    }
    const float r = rsqrtf(wave_sum(ss) / (float)hd + eps);
#pragma unroll
    for (int p = 0; p < kMaxPairs; ++p) {
        const int i = p * 64 + lane;
        if (i < half) {
            const float x1 = round_to<T>(round_to<T>(a[p] * r) * w1[p]);
            const float x2 = round_to<T>(round_to<T>(b[p] * r) * w2[p]);
            const uint16_t y1 = T::from_f32(as_f32_result(__fsub_rn(__fmul_rn(x1, cc[p]), __fmul_rn(x2, sn[p]))));
            const uint16_t y2 = T::from_f32(as_f32_result(__fadd_rn(__fmul_rn(x1, sn[p]), __fmul_rn(x2, cc[p]))));
            dst[i] = y1;
            dst[i + half] = y2;
            if (dst2) {
                dst2[i] = y1;
                dst2[i + half] = y2;
            }
        }
    }
}

// The same with 16-byte accesses, for head dims of 64, 128 or 256 and 16-byte aligned tensors (the scalar kernel
// above moves 2 bytes per lane and instruction: 260 us per layer for a 16,384-token prefill of Qwen3-0.6B).
// A lane owns 8 consecutive dims of a head, HD/8 lanes a head, a wave 64/(HD/8) heads; the rotary partner
// (dims i and i + HD/2) sits HD/16 lanes away.  The arithmetic per element is that of the scalar kernel.
template <typename T, int HD>
__global__ __launch_bounds__(256) void qk_norm_rope_store_vec_kernel(
    const uint16_t* __restrict__ qkv, const uint16_t* __restrict__ q_weight, const uint16_t* __restrict__ k_weight,
    const float* __restrict__ cos_sin, const int64_t* __restrict__ positions, const int64_t* __restrict__ slots,
    uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_out, uint16_t* __restrict__ k_cache,
    uint16_t* __restrict__ v_cache, int rows, int nh, int nkv, int max_positions, int64_t num_slots, int block_size,
    float eps) {
    constexpr int LPH = HD / 8, HPW = 64 / LPH, HALF = HD / 2;
    const int heads = nh + 2 * nkv;
    const int lane = threadIdx.x & 63, sub = lane / LPH, dc = lane % LPH;
    const int64_t items = (int64_t)rows * heads;
    int64_t item = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * HPW + sub;
    const bool live = item < items;   // lanes past the end follow the last item (the shuffles need them) and store nothing
    item = live ? item : items - 1;
    const int row = (int)(item / heads), h = (int)(item % heads);
    const uint16_t* src = qkv + ((int64_t)row * heads + h) * HD + dc * 8;
    const int64_t slot = slots[row];
    const bool slot_ok = slot >= 0 && slot < num_slots;
    float a[8];
    const u32x4 raw = *reinterpret_cast<const u32x4*>(src);
    unpack8<T>(raw, a);
    if (h >= nh + nkv) {   // v: plain copy
        if (live && slot_ok)
            *reinterpret_cast<u32x4*>(v_cache + (((slot / block_size) * nkv + (h - nh - nkv)) * block_size +
                                                  slot % block_size) * HD + dc * 8) = raw;
        // no return: heads of one wave differ in kind, and the shuffles below need every lane
    }
    const bool is_q = h < nh, is_k = !is_q && h < nh + nkv;
    const uint16_t* w = is_q ? q_weight : k_weight;
    float wf[8];
    unpack8<T>(*reinterpret_cast<const u32x4*>(w + dc * 8), wf);
    int64_t pos = positions[row];
    pos = pos < 0 ? 0 : (pos >= max_positions ? max_positions - 1 : pos);
    const int i0 = (dc % (LPH / 2)) * 8;   // index of this lane's first dim inside its half
    const float* cs = cos_sin + pos * HD;
    const f32x4 c0 = *reinterpret_cast<const f32x4*>(cs + i0), c1 = *reinterpret_cast<const f32x4*>(cs + i0 + 4);
    const f32x4 s0 = *reinterpret_cast<const f32x4*>(cs + HALF + i0), s1 = *reinterpret_cast<const f32x4*>(cs + HALF + i0 + 4);
    // the summation order and rounding points of the q|k|v GEMV's fused epilogue (head_dim 128: tile_ssq), so that
    // both routes give the same bits
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = __builtin_fmaf(a[e], a[e], ss);
#pragma unroll
    for (int o = LPH / 2; o >= 1; o >>= 1) ss += __shfl_xor(ss, o);
    const float r = rsqrtf(ss / (float)HD + eps);
    float xn[8], y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) xn[e] = round_to<T>(mul_round<T>(a[e], r) * wf[e]);
    const bool first = dc < LPH / 2;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float other = __shfl_xor(xn[e], LPH / 2);
        const float cc = e < 4 ? c0[e] : c1[e - 4], sn = e < 4 ? s0[e] : s1[e - 4];
        const float x1 = first ? xn[e] : other, x2 = first ? other : xn[e];
        y[e] = as_f32_result(first ? __fsub_rn(__fmul_rn(x1, cc), __fmul_rn(x2, sn))
                                   : __fadd_rn(__fmul_rn(x1, sn), __fmul_rn(x2, cc)));
    }
    if (!live || !(is_q || is_k)) return;
    const u32x4 packed = pack8<T>(y);
    if (is_q) {
        *reinterpret_cast<u32x4*>(q_out + ((int64_t)row * nh + h) * HD + dc * 8) = packed;
        return;
    }
    if (k_out) *reinterpret_cast<u32x4*>(k_out + ((int64_t)row * nkv + (h - nh)) * HD + dc * 8) = packed;
    if (slot_ok)
        *reinterpret_cast<u32x4*>(k_cache + (((slot / block_size) * nkv + (h - nh)) * block_size + slot % block_size) * HD +
                                  dc * 8) = packed;
}

// ---------------------------------------------------------------------------------------------
// Attention of one new token per sequence over its paged KV cache (flash-decoding).
// Workgroup = (sequence, kv head, context split), WAVES waves (16 for up to 2 query heads per kv head, 8 for
// 4, 4 for 8: the wave merge buffer grows with G); with enough waves per workgroup a batch of sequences
// needs no context split and no second kernel.  A wave covers TPW = 64 / (HD/8) tokens
// per step: a lane holds 8 head dims of one token's K and V rows (one 16-byte load each), the G
// query heads of the kv group share those loads.  Every lane group keeps its own online-softmax
// state (running max, sum, 8 accumulators per query head); the states are merged across lane
// groups, then waves (LDS), then splits (fp32 partials + a second kernel).
constexpr float kNegBig = -3.0e38f;

template <typename T, int G, int HD, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void paged_attn_decode_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, const int32_t* __restrict__ context_lens, uint16_t* __restrict__ out,
    float* __restrict__ partial, int nkv, int block_size, int max_blocks, int num_blocks, int nsplit, float scale) {
    constexpr int LPT = HD / 8;    // lanes per token
    constexpr int TPW = 64 / LPT;  // tokens per wave step
    constexpr int U = 2;           // token steps in flight
    const int sp = blockIdx.x % nsplit;
    const int kvh = (blockIdx.x / nsplit) % nkv;
    const int b = blockIdx.x / (nsplit * nkv);
    const int nh = nkv * G;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int dc = lane % LPT, ts = lane / LPT;

    int ctx = context_lens[b];
    ctx = ctx < 0 ? 0 : (ctx > max_blocks * block_size ? max_blocks * block_size : ctx);
    const int per = (ctx + nsplit - 1) / nsplit;
    const int t0 = sp * per, t1 = min(ctx, t0 + per);

    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        unpack8<T>(*reinterpret_cast<const u32x4*>(q + ((int64_t)b * nh + kvh * G + g) * HD + dc * 8), qf[g]);
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[g][e] *= scale * kLog2e;
    }
    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = kNegBig;
        l[g] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    }

    const int32_t* table = block_table + (int64_t)b * max_blocks;
    for (int t = t0 + wave * TPW + ts; t - ts < t1; t += WAVES * TPW * U) {
        u32x4 kr[U], vr[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int tt = t + u * WAVES * TPW;
            ok[u] = tt < t1;
            const int tc = ok[u] ? tt : t0;
            int blk = table[tc / block_size];
            blk = blk < 0 ? 0 : (blk >= num_blocks ? num_blocks - 1 : blk);
            const int64_t off = (((int64_t)blk * nkv + kvh) * block_size + tc % block_size) * HD + dc * 8;
            kr[u] = *reinterpret_cast<const u32x4*>(k_cache + off);
            vr[u] = *reinterpret_cast<const u32x4*>(v_cache + off);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float kf[8], vf[8];
            unpack8<T>(kr[u], kf);
            unpack8<T>(vr[u], vf);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float s = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) s += qf[g][e] * kf[e];
#pragma unroll
                for (int o = LPT / 2; o >= 1; o >>= 1) s += __shfl_xor(s, o);
                s = ok[u] ? s : kNegBig;
                const float mn = fmaxf(m[g], s);
                const float c = exp2f(m[g] - mn);
                const float p = ok[u] ? exp2f(s - mn) : 0.f;
                m[g] = mn;
                l[g] = l[g] * c + p;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[g][e] = acc[g][e] * c + p * vf[e];
            }
        }
    }

    // merge the TPW lane groups of this wave
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int o = LPT; o < 64; o <<= 1) {
            const float mo = __shfl_xor(m[g], o), lo = __shfl_xor(l[g], o);
            const float mn = fmaxf(m[g], mo);
            const float ca = exp2f(m[g] - mn), cb = exp2f(mo - mn);
            l[g] = l[g] * ca + lo * cb;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[g][e] = acc[g][e] * ca + __shfl_xor(acc[g][e], o) * cb;
            m[g] = mn;
        }
    }
    // merge the waves through LDS: [wave][g][HD + 2]
    __shared__ float s_acc[WAVES][G][HD + 2];
    if (ts == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int e = 0; e < 8; ++e) s_acc[wave][g][dc * 8 + e] = acc[g][e];
            if (dc == 0) {
                s_acc[wave][g][HD] = m[g];
                s_acc[wave][g][HD + 1] = l[g];
            }
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * HD; idx += 64 * WAVES) {
        const int g = idx / HD, d = idx % HD;
        float mn = kNegBig;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) mn = fmaxf(mn, s_acc[w][g][HD]);
        float lt = 0.f, at = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float c = exp2f(s_acc[w][g][HD] - mn);
            lt += s_acc[w][g][HD + 1] * c;
            at += s_acc[w][g][d] * c;
        }
        const int64_t head = (int64_t)b * nh + kvh * G + g;
        if (nsplit == 1) {
            out[head * HD + d] = T::from_f32(lt > 0.f ? at / lt : 0.f);
        } else {
            float* dst = partial + (head * nsplit + sp) * (HD + 2);
            dst[d] = at;
            if (d == 0) {
                dst[HD] = mn;
                dst[HD + 1] = lt;
            }
        }
    }
}

// The same for 4 or 8 query heads per kv head and 128 head dims, where the kernel above is bound by its
// vector-ALU dot products (8 FMAs, 4 shuffles and an online-softmax update per token, head and lane).
// A wave takes tiles of 16 tokens.  Scores: S^T = K q^T on the 16x16x32 MFMA (A = 16 token rows of K, 32 head dims
// per instruction; B = the G query heads as columns, the rest zero), so a lane ends up with 4 tokens of one head and
// the softmax bookkeeping is done once per tile and head, not per token and lane.  The probabilities cross to the
// value phase through a 16 x G array in LDS (private to the wave); there a lane holds 8 head dims of one token's V row
// as before and adds p * v for the G heads.  Tiles start at multiples of 16 tokens inside a context split and
// block_size % 16 == 0, so a tile never straddles a cache block.
template <typename T, int G, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void paged_attn_decode_mfma_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, const int32_t* __restrict__ context_lens, uint16_t* __restrict__ out,
    float* __restrict__ partial, int nkv, int block_size, int max_blocks, int num_blocks, int nsplit, float scale) {
    constexpr int HD = 128, TT = 16;
    static_assert(G == 4 || G == 8, "query heads per kv head");
    const int sp = blockIdx.x % nsplit;
    const int kvh = (blockIdx.x / nsplit) % nkv;
    const int b = blockIdx.x / (nsplit * nkv);
    const int nh = nkv * G;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lo = lane & 15, hi = lane >> 4;   // score phase: head lo, token quad hi; value phase: dims 8*lo.., token hi

    int ctx = context_lens[b];
    ctx = ctx < 0 ? 0 : (ctx > max_blocks * block_size ? max_blocks * block_size : ctx);
    const int per = ((ctx + nsplit - 1) / nsplit + TT - 1) / TT * TT;
    const int t0 = sp * per, t1 = min(ctx, t0 + per);

    __shared__ float s_p[WAVES][TT * G + G];   // per wave: p[token][head], then the rescale factor per head
    __shared__ float s_acc[WAVES][G][HD + 2];
    float* P = s_p[wave];

    u32x4 bq[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bq[i] = u32x4{0u, 0u, 0u, 0u};
        if (lo < G)
            bq[i] = *reinterpret_cast<const u32x4*>(q + ((int64_t)b * nh + kvh * G + lo) * HD + 32 * i + 8 * hi);
    }
    const float sc = scale * kLog2e;
    float m = kNegBig, lpart = 0.f;
    float acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;

    const int32_t* table = block_table + (int64_t)b * max_blocks;
    for (int tb = t0 + wave * TT; tb < t1; tb += WAVES * TT) {
        int blk = table[tb / block_size];                         // wave-uniform
        blk = blk < 0 ? 0 : (blk >= num_blocks ? num_blocks - 1 : blk);
        const int64_t base = (((int64_t)blk * nkv + kvh) * block_size + tb % block_size) * HD;
        u32x4 ka[4], va[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)   // K row of token tb + lo (rows past the context are masked below)
            ka[i] = *reinterpret_cast<const u32x4*>(k_cache + base + (int64_t)lo * HD + 32 * i + 8 * hi);
#pragma unroll
        for (int u = 0; u < 4; ++u) {   // V rows: a masked token reads the last valid row (its p is 0, the row is finite)
            const int tv = min(4 * u + hi, t1 - 1 - tb);
            va[u] = *reinterpret_cast<const u32x4*>(v_cache + base + (int64_t)tv * HD + 8 * lo);
        }
        f32x4 st = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; ++i) st = T::mfma16(ka[i], bq[i], st);
        // st[r]: head lo, token tb + 4*hi + r
        float sv[4], mx = kNegBig;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            sv[r] = (tb + 4 * hi + r < t1) ? st[r] * sc : kNegBig;
            mx = fmaxf(mx, sv[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float mn = fmaxf(m, mx);
        const float c = exp2f(m - mn);
        m = mn;
        float ps = 0.f;
        float pr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            pr[r] = (tb + 4 * hi + r < t1) ? exp2f(sv[r] - mn) : 0.f;
            ps += pr[r];
        }
        lpart = lpart * c + ps;
        if (lo < G) {
#pragma unroll
            for (int r = 0; r < 4; ++r) P[(4 * hi + r) * G + lo] = pr[r];
            if (hi == 0) P[TT * G + lo] = c;
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();   // LDS operations of a wave execute in order: the reads below see these writes
        asm volatile("" ::: "memory");
        float cg[G];
#pragma unroll
        for (int g = 0; g < G; g += 4) {
            const f32x4 v4 = *reinterpret_cast<const f32x4*>(P + TT * G + g);
            cg[g] = v4[0]; cg[g + 1] = v4[1]; cg[g + 2] = v4[2]; cg[g + 3] = v4[3];
        }
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[g][e] *= cg[g];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            float vf[8], pg[G];
            unpack8<T>(va[u], vf);
#pragma unroll
            for (int g = 0; g < G; g += 4) {
                const f32x4 v4 = *reinterpret_cast<const f32x4*>(P + (4 * u + hi) * G + g);
                pg[g] = v4[0]; pg[g + 1] = v4[1]; pg[g + 2] = v4[2]; pg[g + 3] = v4[3];
            }
#pragma unroll
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[g][e] += pg[g] * vf[e];
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();   // the next tile's writes come after these reads
        asm volatile("" ::: "memory");
    }

    // the four token groups of the wave share m: their accumulators and partial sums just add
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[g][e] += __shfl_xor(acc[g][e], 16);
            acc[g][e] += __shfl_xor(acc[g][e], 32);
        }
    lpart += __shfl_xor(lpart, 16);
    lpart += __shfl_xor(lpart, 32);
    if (hi == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) s_acc[wave][g][lo * 8 + e] = acc[g][e];
        if (lo < G) {
            s_acc[wave][lo][HD] = m;
            s_acc[wave][lo][HD + 1] = lpart;
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * HD; idx += 64 * WAVES) {
        const int g = idx / HD, d = idx % HD;
        float mn = kNegBig;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) mn = fmaxf(mn, s_acc[w][g][HD]);
        float lt = 0.f, at = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float c = exp2f(s_acc[w][g][HD] - mn);
            lt += s_acc[w][g][HD + 1] * c;
            at += s_acc[w][g][d] * c;
        }
        const int64_t head = (int64_t)b * nh + kvh * G + g;
        if (nsplit == 1) {
            out[head * HD + d] = T::from_f32(lt > 0.f ? at / lt : 0.f);
        } else {
            float* dst = partial + (head * nsplit + sp) * (HD + 2);
            dst[d] = at;
            if (d == 0) {
                dst[HD] = mn;
                dst[HD + 1] = lt;
            }
        }
    }
}

// Both products on the matrix cores, for 128 head dims and block sizes that are multiples of 16.  The query heads of
// a kv head are columns of a 16-column MFMA tile, so any count up to 16 fits: G > 0 fixes it at compile time (the
// launcher uses 8), G = 0 takes it from `heads_per_kv` -- the route of the head ratios the other kernels have no
// instantiation for (Qwen3-14B: 40 query heads on 8 kv heads).  The kernel above multiplies the probabilities with V on the vector ALU (G x 8
// FMAs per token and lane), which with 8 heads per kv head costs as much as fetching the cache: cache-resident it
// still takes 62 of the 102 us it needs from HBM at 64 sequences x 8 kv heads x 2060 tokens.  Here a wave takes
// tiles of 32 tokens:
//   scores   S^T = K q^T as above (two 16-token halves, four MFMAs each): a lane ends up with the scores of head
//            lane % 16 and tokens 4 * (lane / 16) + r of both halves -- which is where the B operand of the second
//            product wants the probabilities of that head, so they never leave their registers;
//   values   out^T[dims, heads] = V^T P^T, one MFMA per 16 head dims and tile.  Its A operand needs, per lane, eight
//            tokens of ONE head dim, but a V row has the dims side by side: the tile is brought to LDS (load-to-LDS,
//            16 lanes per row) and read back with the transposing LDS read (ds_read_b64_tr_b16: in each group of 16
//            lanes, lane 4q + c receives element c of the four 8-byte pieces that lanes q, q + 4, q + 8, q + 12 point
//            at).  Rows sit 256 bytes apart, i.e. on the same banks; each row is therefore stored rotated by its own
//            index in units of 32 bytes (the load's lanes simply fetch the rotated piece), and the 16 tokens of one
//            transposing read fall on all 64 banks twice.
// The online-softmax state (running maximum, rescale factor) is per head and lives in the lanes of that head, which
// are also the lanes that hold that head's output column: nothing crosses lanes but the maximum.
// Rows past the context may hold anything: their scores are replaced before the maximum, their probabilities are
// zero, and their V rows are fetched from the last valid token of the tile (0 x NaN would be NaN).
#define NQ_GPTR(p) ((__attribute__((address_space(1))) void*)(p))
#define NQ_LPTR(p) ((__attribute__((address_space(3))) void*)(p))
typedef short nq_s16x4 __attribute__((ext_vector_type(4)));

template <typename T, int G, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void paged_attn_decode_tr_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, const int32_t* __restrict__ context_lens, uint16_t* __restrict__ out,
    float* __restrict__ partial, int nkv, int block_size, int max_blocks, int num_blocks, int nsplit, float scale,
    int heads_per_kv) {
    constexpr int HD = 128, TT = 32, VBYTES = TT * HD * 2, WBYTES = 2 * VBYTES;   // a wave's K tile and V tile
    constexpr int GA = G ? G : 16;                                                // rows of the per-wave result
    static_assert(G >= 0 && G <= 16, "query heads per kv head");
    static_assert(GA * (HD + 2) * 4 <= WBYTES, "the per-wave results reuse the wave's tiles");
    const int Gv = G ? G : heads_per_kv;
    const int sp = blockIdx.x % nsplit;
    const int kvh = (blockIdx.x / nsplit) % nkv;
    const int b = blockIdx.x / (nsplit * nkv);
    const int nh = nkv * Gv;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lo = lane & 15, hi = lane >> 4;

    int ctx = context_lens[b];
    ctx = ctx < 0 ? 0 : (ctx > max_blocks * block_size ? max_blocks * block_size : ctx);
    const int per = ((ctx + nsplit - 1) / nsplit + TT - 1) / TT * TT;
    const int t0 = sp * per, t1 = min(ctx, t0 + per);

    __shared__ __attribute__((aligned(1024))) unsigned char s_raw[WAVES * WBYTES];
    unsigned char* kt = s_raw + wave * WBYTES;                       // this wave's K tile [32 tokens][256 B, rotated]
    unsigned char* vt = kt + VBYTES;                                 // and its V tile
    float (*s_acc)[GA][HD + 2] = reinterpret_cast<float (*)[GA][HD + 2]>(s_raw);   // after the loop

    u32x4 bq[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bq[i] = u32x4{0u, 0u, 0u, 0u};
        if (lo < Gv)
            bq[i] = *reinterpret_cast<const u32x4*>(q + ((int64_t)b * nh + kvh * Gv + lo) * HD + 32 * i + 8 * hi);
    }
    const float sc = scale * kLog2e;
    float m = kNegBig, lpart = 0.f;
    f32x4 acc[8];
#pragma unroll
    for (int cb = 0; cb < 8; ++cb) acc[cb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // load-to-LDS lane roles: instruction k fills rows 4k .. 4k + 3, 16 lanes a row (a whole 256-byte row per 16
    // lanes: 16 rows x 64 bytes per instruction, the A-operand layout of the score product, moves half as fast).
    // V: 16-byte position c' of row r holds the row's piece (window (c' / 2 - r) mod 8, half c' % 2); K: position c'
    // holds piece (c' - r) mod 16, so that the 16 token rows a b128 read of one piece index touches differ in bank.
    const int dma_row = lane >> 4, dma_piece = lane & 15;
    // transposing read: as a source, this lane points at token 4 * hi + lo / 4 (+ 16 for the second half), quad lo % 4
    const int tr_tok = 4 * hi + (lo >> 2), tr_quad = (lo & 3) * 8;

    const int32_t* table = block_table + (int64_t)b * max_blocks;
    for (int tb = t0 + wave * TT; tb < t1; tb += WAVES * TT) {
        int blk = table[tb / block_size];                         // wave-uniform
        blk = blk < 0 ? 0 : (blk >= num_blocks ? num_blocks - 1 : blk);
        const int64_t base = (((int64_t)blk * nkv + kvh) * block_size + tb % block_size) * HD;
        const int last = min(TT, t1 - tb) - 1;                    // last valid row of the tile
        // rows 16..31: in the same cache block 16 rows on, or (block sizes that are odd multiples of 16) at the start
        // of the next one; where the context ends before them, the first 16 rows stand in (their scores are replaced)
        int64_t base16 = base + 16 * HD;
        if (tb % block_size + 16 >= block_size) {                 // wave-uniform
            base16 = base;
            if (tb + 16 < t1) {
                int blk1 = table[(tb + 16) / block_size];
                blk1 = blk1 < 0 ? 0 : (blk1 >= num_blocks ? num_blocks - 1 : blk1);
                base16 = ((int64_t)blk1 * nkv + kvh) * block_size * HD;
            }
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {   // rows past the context are fetched as they are: their scores are replaced
            const int r = 4 * k + dma_row;
            const uint16_t* src = k_cache + (k < 4 ? base : base16) + (int64_t)(r & 15) * HD + 8 * ((dma_piece - r) & 15);
            __builtin_amdgcn_global_load_lds(NQ_GPTR(src), NQ_LPTR(kt + k * 1024), 16, 0, 0);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int r = 4 * k + dma_row;
            const int w = ((dma_piece >> 1) - r) & 7;
            const int rr = min(r, last);
            const uint16_t* src = v_cache + (rr < 16 ? base : base16) + (int64_t)(rr & 15) * HD + 16 * w + 8 * (dma_piece & 1);
            __builtin_amdgcn_global_load_lds(NQ_GPTR(src), NQ_LPTR(vt + k * 1024), 16, 0, 0);
        }
        // the K tile has landed: a wave's loads return in order, the eight of the V tile are the newest
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        f32x4 st[2];
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            st[a] = f32x4{0.f, 0.f, 0.f, 0.f};
            const int r = 16 * a + lo;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32x4 ka = *reinterpret_cast<const u32x4*>(kt + r * 256 + ((4 * i + hi + r) & 15) * 16);
                st[a] = T::mfma16(ka, bq[i], st[a]);
            }
        }
        // st[a][r]: head lo, token tb + 16 a + 4 hi + r
        float sv[2][4], mx = kNegBig;
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sv[a][r] = (16 * a + 4 * hi + r <= last) ? st[a][r] * sc : kNegBig;
                mx = fmaxf(mx, sv[a][r]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float mn = fmaxf(m, mx);
        const float c = exp2f(m - mn);
        m = mn;
        float pr[2][4], ps = 0.f;
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                pr[a][r] = (16 * a + 4 * hi + r <= last) ? exp2f(sv[a][r] - mn) : 0.f;
                ps += pr[a][r];
            }
        lpart = lpart * c + ps;
        const u32x4 pb = u32x4{T::pack2(pr[0][0], pr[0][1]), T::pack2(pr[0][2], pr[0][3]),
                               T::pack2(pr[1][0], pr[1][1]), T::pack2(pr[1][2], pr[1][3])};
#pragma unroll
        for (int cb = 0; cb < 8; ++cb)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[cb][r] *= c;
        // the V tile has landed
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int cb = 0; cb < 8; ++cb) {
            u32x4 vf;
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const int tok = 16 * a + tr_tok;
                const nq_s16x4 t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (nq_s16x4 __attribute__((address_space(3)))*)(vt + tok * 256 + (((cb + tok) & 7) << 5) + tr_quad));
                const u32x2 t2 = __builtin_bit_cast(u32x2, t4);
                vf[2 * a] = t2[0];
                vf[2 * a + 1] = t2[1];
            }
            acc[cb] = T::mfma16(vf, pb, acc[cb]);   // rows: dims 16 cb + 4 hi + r, column: head lo
        }
        // the next tile's loads overwrite both tiles: every read of them has returned
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }

    lpart += __shfl_xor(lpart, 16);
    lpart += __shfl_xor(lpart, 32);
    __syncthreads();   // every wave is done with its tiles: the area now holds the per-wave results
    if (lo < Gv) {
#pragma unroll
        for (int cb = 0; cb < 8; ++cb)
#pragma unroll
            for (int r = 0; r < 4; ++r) s_acc[wave][lo][16 * cb + 4 * hi + r] = acc[cb][r];
        if (hi == 0) {
            s_acc[wave][lo][HD] = m;
            s_acc[wave][lo][HD + 1] = lpart;
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < Gv * HD; idx += 64 * WAVES) {
        const int g = idx / HD, d = idx % HD;
        float mn = kNegBig;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) mn = fmaxf(mn, s_acc[w][g][HD]);
        float lt = 0.f, at = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float c = exp2f(s_acc[w][g][HD] - mn);
            lt += s_acc[w][g][HD + 1] * c;
            at += s_acc[w][g][d] * c;
        }
        const int64_t head = (int64_t)b * nh + kvh * Gv + g;
        if (nsplit == 1) {
            out[head * HD + d] = T::from_f32(lt > 0.f ? at / lt : 0.f);
        } else {
            float* dst = partial + (head * nsplit + sp) * (HD + 2);
            dst[d] = at;
            if (d == 0) {
                dst[HD] = mn;
                dst[HD + 1] = lt;
            }
        }
    }
}

// Merge of the context splits: one workgroup of HD threads per (sequence, query head).
template <typename T, int HD>
__global__ __launch_bounds__(HD) void paged_attn_merge_kernel(const float* __restrict__ partial,
                                                              uint16_t* __restrict__ out, int nsplit) {
    const float* src = partial + (int64_t)blockIdx.x * nsplit * (HD + 2);
    const int d = threadIdx.x;
    float mn = kNegBig;
    for (int s = 0; s < nsplit; ++s) mn = fmaxf(mn, src[s * (HD + 2) + HD]);
    float lt = 0.f, at = 0.f;
    for (int s = 0; s < nsplit; ++s) {
        const float c = exp2f(src[s * (HD + 2) + HD] - mn);
        lt += src[s * (HD + 2) + HD + 1] * c;
        at += src[s * (HD + 2) + d] * c;
    }
    out[(int64_t)blockIdx.x * HD + d] = T::from_f32(lt > 0.f ? at / lt : 0.f);
}

// ---------------------------------------------------------------------------------------------
// out[r, i] = SiLU(gate_up[r, i]) * gate_up[r, inter + i], SiLU rounded to the tensor type first.
// Greedy sampler: out[r] = index of the largest logits[r, :] (the lowest index among equal maxima; NaNs are never
// selected).  One workgroup of 16 waves per row, 16-byte loads.
template <typename T>
__global__ __launch_bounds__(1024) void argmax_rows_kernel(const uint16_t* __restrict__ logits,
                                                           int64_t* __restrict__ out, int vocab) {
    const uint16_t* row = logits + (size_t)blockIdx.x * vocab;
    float best = -__builtin_inff();
    int bi = 0x7fffffff;
    auto take = [&](float f, int idx) {
        if (f > best || (f == best && idx < bi)) {
            best = f;
            bi = idx;
        }
    };
    const int nvec = (vocab & 7) == 0 ? vocab >> 3 : 0;   // rows are 16-byte aligned only then
    for (int v0 = threadIdx.x; v0 < nvec; v0 += 4 * 1024) {
        u32x4 d[4];   // four loads in flight
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int v = v0 + u * 1024;
            d[u] = *reinterpret_cast<const u32x4*>(row + (size_t)(v < nvec ? v : v0) * 8);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int v = v0 + u * 1024;
            if (v < nvec) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    take(T::to_f32((uint16_t)(d[u][i] & 0xFFFFu)), v * 8 + 2 * i);
                    take(T::to_f32((uint16_t)(d[u][i] >> 16)), v * 8 + 2 * i + 1);
                }
            }
        }
    }
    for (int i = nvec * 8 + threadIdx.x; i < vocab; i += 1024) take(T::to_f32(row[i]), i);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) take(__shfl_xor(best, off), __shfl_xor(bi, off));
    __shared__ float s_best[16];
    __shared__ int s_idx[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        s_best[wave] = best;
        s_idx[wave] = bi;
    }
    __syncthreads();
    if (wave == 0) {
        best = lane < 16 ? s_best[lane] : -__builtin_inff();
        bi = lane < 16 ? s_idx[lane] : 0x7fffffff;
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) take(__shfl_xor(best, off), __shfl_xor(bi, off));
        if (lane == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    }
}

// IL: gate and up interleaved in words of 8 columns (word 2t = gate outputs 8t.., word 2t+1 = the up columns of the
// same outputs) instead of side by side.
template <typename T, bool IL>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* __restrict__ gate_up,
                                                       uint16_t* __restrict__ out, int64_t rows, int inter) {
    const int64_t vec = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int per_row = inter / 8;
    if (vec >= rows * per_row) return;
    const int64_t r = vec / per_row;
    const int i = (int)(vec % per_row) * 8;
    float g[8], u[8], o[8];
    const uint16_t* row = gate_up + r * 2 * inter;
    unpack8<T>(*reinterpret_cast<const u32x4*>(row + (IL ? 2 * i : i)), g);
    unpack8<T>(*reinterpret_cast<const u32x4*>(row + (IL ? 2 * i + 8 : inter + i)), u);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = round_to<T>(g[e] / (1.f + __expf(-g[e]))) * u[e];
    *reinterpret_cast<u32x4*>(out + r * inter + i) = pack8<T>(o);
}

int bad(const char* fn, const char* what) {
    set_error("%s: %s", fn, what);
    return AWQ_ERR_INVALID_ARG;
}
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The kernel with both products on the matrix cores takes 128 head dims and block sizes that are multiples of 16; it
// is used at 8 query heads per kv head, where the vector-ALU value product of the other kernels costs the most
// (bf16, against them: 128 sequences x 8 kv heads x 1024 tokens 120 -> 102 us, 32 x 8 x 512 23.2 -> 19.9, 1 x 8 x 8000
// 31.7 -> 24.6, 64 x 8 x 2060 the same 102 us = 5.3 TB/s; at 4 and 2 heads per kv head it measured equal or slower:
// 16 x 8 x 4000 at 4 heads 52.6 -> 55.0 us, the Qwen3-0.6B decode step 1.615 -> 1.673 ms).
// Head ratios other than 1, 2, 4 and 8 (up to 16) have no other kernel and take it as well.
bool attn_tr(int G, int64_t head_dim, int64_t block_size) {
    return (G == 8 || (G != 1 && G != 2 && G != 4 && G >= 1 && G <= 16)) && head_dim == 128 && block_size % 16 == 0;
}
int attn_waves(int G, bool tr) { return tr ? 4 : (G <= 2 ? 16 : (G <= 4 ? 8 : 4)); }

// Context splits of a (sequence, kv head) pair.  From sweeps at 1..128 sequences x 512..8000 tokens (bf16, caches
// larger than the Infinity Cache): four- and eight-wave workgroups run best at about 2048 waves on the chip, the
// 16-wave ones at about 4096, with 128 tokens or more per split -- 64 sequences x 8 kv heads x 2060 tokens at 8 heads
// per kv head 124 us in two splits + merge, 105 unsplit; 16 sequences 46 us in eight, 36 in four; 2 x 8 x 1000 at 4
// heads per kv head 16.1 us in sixteen, 12.9 in eight.
int pick_splits(int64_t batch, int64_t nkv, int64_t max_context, int G, bool tr) {
    const int64_t waves = attn_waves(G, tr);
    int64_t s = cdiv(waves >= 16 ? 4096 : 2048, batch * nkv * waves);
    const int64_t cap = max_context / 128 > 1 ? max_context / 128 : 1;
    s = s > cap ? cap : s;
    s = s > 16 ? 16 : s;
    return (int)(s < 1 ? 1 : s);
}

template <typename T, int G, int HD>
void launch_attn(const void* q, const void* kc, const void* vc, const int32_t* table, const int32_t* ctx, void* out,
                 float* partial, int64_t batch, int nkv, int bs, int max_blocks, int num_blocks, int nsplit,
                 float scale, hipStream_t st) {
    constexpr int WAVES = G <= 2 ? 16 : (G <= 4 ? 8 : 4);
    if constexpr (HD == 128 && G == 8) {
        if (attn_tr(G, HD, bs)) {
            paged_attn_decode_tr_kernel<T, G, 4><<<dim3((unsigned)(batch * nkv * nsplit)), dim3(256), 0, st>>>(
                (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, table, ctx, (uint16_t*)out, partial, nkv,
                bs, max_blocks, num_blocks, nsplit, scale, G);
            if (nsplit > 1)
                paged_attn_merge_kernel<T, HD><<<dim3((unsigned)(batch * nkv * G)), dim3(HD), 0, st>>>(
                    partial, (uint16_t*)out, nsplit);
            return;
        }
    }
    if constexpr (HD == 128 && (G == 4 || G == 8)) {
        if (bs % 16 == 0) {
            paged_attn_decode_mfma_kernel<T, G, WAVES><<<dim3((unsigned)(batch * nkv * nsplit)), dim3(64 * WAVES), 0, st>>>(
                (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, table, ctx, (uint16_t*)out, partial, nkv,
                bs, max_blocks, num_blocks, nsplit, scale);
            if (nsplit > 1)
                paged_attn_merge_kernel<T, HD><<<dim3((unsigned)(batch * nkv * G)), dim3(HD), 0, st>>>(
                    partial, (uint16_t*)out, nsplit);
            return;
        }
    }
    paged_attn_decode_kernel<T, G, HD, WAVES><<<dim3((unsigned)(batch * nkv * nsplit)), dim3(64 * WAVES), 0, st>>>(
        (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, table, ctx, (uint16_t*)out, partial, nkv, bs,
        max_blocks, num_blocks, nsplit, scale);
    if (nsplit > 1)
        paged_attn_merge_kernel<T, HD><<<dim3((unsigned)(batch * nkv * G)), dim3(HD), 0, st>>>(partial, (uint16_t*)out,
                                                                                               nsplit);
}

template <typename T, int HD>
int launch_attn_g(int G, const void* q, const void* kc, const void* vc, const int32_t* table, const int32_t* ctx,
                  void* out, float* partial, int64_t batch, int nkv, int bs, int max_blocks, int num_blocks,
                  int nsplit, float scale, hipStream_t st) {
    switch (G) {
#define NQ_CASE(g)                                                                                              \
    case g:                                                                                                     \
        launch_attn<T, g, HD>(q, kc, vc, table, ctx, out, partial, batch, nkv, bs, max_blocks, num_blocks,      \
                              nsplit, scale, st);                                                               \
        return AWQ_OK;
        NQ_CASE(1) NQ_CASE(2) NQ_CASE(4) NQ_CASE(8)
#undef NQ_CASE
    }
    if constexpr (HD == 128) {
        if (attn_tr(G, HD, bs)) {   // any other ratio up to 16: the matrix-core kernel with the count at run time
            paged_attn_decode_tr_kernel<T, 0, 4><<<dim3((unsigned)(batch * nkv * nsplit)), dim3(256), 0, st>>>(
                (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, table, ctx, (uint16_t*)out, partial, nkv,
                bs, max_blocks, num_blocks, nsplit, scale, G);
            if (nsplit > 1)
                paged_attn_merge_kernel<T, HD><<<dim3((unsigned)(batch * nkv * G)), dim3(HD), 0, st>>>(
                    partial, (uint16_t*)out, nsplit);
            return AWQ_OK;
        }
    }
    set_error("nq_paged_attention_decode: query heads per kv head must be 1, 2, 4 or 8 (or, with head_dim 128 and a "
              "block size that is a multiple of 16, any count up to 16), got %d", G);
    return AWQ_ERR_UNSUPPORTED;
}

// ---------------------------------------------------------------------------------------------
// Bookkeeping of a decode step over the paged cache, one launch each instead of a dozen elementwise ones.
// prepare: the cache slot and the context length of the token each row feeds at its position.
__global__ __launch_bounds__(256) void decode_prepare_kernel(const int64_t* __restrict__ pos,
                                                            const uint8_t* __restrict__ active,
                                                            const int32_t* __restrict__ table,
                                                            int64_t* __restrict__ slots, int32_t* __restrict__ ctx,
                                                            int rows, int max_blocks, int block_size) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    int64_t p = pos[r];
    p = p < 0 ? 0 : p;
    int64_t blk = p / block_size;
    blk = blk >= max_blocks ? max_blocks - 1 : blk;
    slots[r] = active[r] ? (int64_t)table[(int64_t)r * max_blocks + blk] * block_size + p % block_size : -1;
    ctx[r] = (int32_t)(p + 1);
}

// advance: the sampled tokens become row step[0] of the output log and the next step's input; active rows move on
// one position; the step counter goes up.  One workgroup, so that every thread has read the counter before it changes.
__global__ __launch_bounds__(1024) void decode_advance_kernel(const int64_t* __restrict__ next,
                                                             const uint8_t* __restrict__ active,
                                                             int64_t* __restrict__ out, int64_t* __restrict__ ids,
                                                             int64_t* __restrict__ pos, int64_t* __restrict__ step,
                                                             int rows, int64_t out_rows) {
    const int64_t s = step[0];
    __syncthreads();
    for (int r = threadIdx.x; r < rows; r += blockDim.x) {
        const int64_t t = next[r];
        if (s >= 0 && s < out_rows) out[s * rows + r] = t;
        ids[r] = t;
        if (active[r]) pos[r] += 1;
    }
    if (threadIdx.x == 0) step[0] = s + 1;
}

}  // namespace
}  // namespace awq

using namespace awq;

extern "C" int nq_add_rmsnorm(void* residual, const void* delta, const void* weight, void* y, int64_t rows,
                              int64_t hidden, float eps, int dtype, void* stream) {
    const char* fn = "nq_add_rmsnorm";
    if (!residual || !weight || !y) return bad(fn, "null pointer argument");
    if (!aligned16(residual) || !aligned16(weight) || !aligned16(y) || !aligned16(delta))
        return bad(fn, "every tensor must be 16-byte aligned");
    if (dtype != AWQ_F16 && dtype != AWQ_BF16) return bad(fn, "dtype must be AWQ_F16 or AWQ_BF16");
    if (rows <= 0 || hidden <= 0 || hidden % 8 != 0) return bad(fn, "rows > 0 and hidden a positive multiple of 8");
    if (hidden > kNormThreads * 8 * kNormPasses || rows > 0x7fffffff) {
        set_error("%s: hidden=%lld exceeds %d", fn, (long long)hidden, kNormThreads * 8 * kNormPasses);
        return AWQ_ERR_UNSUPPORTED;
    }
    hipStream_t st = (hipStream_t)stream;
    (void)hipGetLastError();
    if (dtype == AWQ_F16)
        add_rmsnorm_kernel<F16><<<dim3((unsigned)rows), dim3(kNormThreads), 0, st>>>(
            (uint16_t*)residual, (const uint16_t*)delta, (const uint16_t*)weight, (uint16_t*)y, (int)hidden, eps);
    else
        add_rmsnorm_kernel<BF16><<<dim3((unsigned)rows), dim3(kNormThreads), 0, st>>>(
            (uint16_t*)residual, (const uint16_t*)delta, (const uint16_t*)weight, (uint16_t*)y, (int)hidden, eps);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

static int row_ssq_entry(const char* fn, const void* x, float* ssq, int64_t rows, int64_t hidden, const int64_t* ids,
                         int64_t table_rows, void* x_out, int dtype, void* stream);

extern "C" int nq_row_ssq(const void* x, float* ssq, int64_t rows, int64_t hidden, int dtype, void* stream) {
    return row_ssq_entry("nq_row_ssq", x, ssq, rows, hidden, nullptr, 0, nullptr, dtype, stream);
}

extern "C" int nq_embed_row_ssq(const int64_t* ids, const void* table, void* x_out, float* ssq, int64_t rows,
                                int64_t hidden, int64_t table_rows, int dtype, void* stream) {
    const char* fn = "nq_embed_row_ssq";
    if (!ids || !x_out) return bad(fn, "null pointer argument");
    if (!aligned16(x_out)) return bad(fn, "x_out must be 16-byte aligned");
    if (table_rows <= 0) return bad(fn, "table_rows must be positive");
    return row_ssq_entry(fn, table, ssq, rows, hidden, ids, table_rows, x_out, dtype, stream);
}

static int row_ssq_entry(const char* fn, const void* x, float* ssq, int64_t rows, int64_t hidden, const int64_t* ids,
                         int64_t table_rows, void* x_out, int dtype, void* stream) {
    if (!x || !ssq) return bad(fn, "null pointer argument");
    if (!aligned16(x) || (reinterpret_cast<uintptr_t>(ssq) & 3u)) return bad(fn, "x must be 16-byte, ssq 4-byte aligned");
    if (dtype != AWQ_F16 && dtype != AWQ_BF16) return bad(fn, "dtype must be AWQ_F16 or AWQ_BF16");
    if (rows <= 0 || hidden <= 0 || hidden % 8 != 0) return bad(fn, "rows > 0 and hidden a positive multiple of 8");
    if (hidden > kNormThreads * 8 * kNormPasses || rows > 0x7fffffff) {
        set_error("%s: hidden=%lld exceeds %d", fn, (long long)hidden, kNormThreads * 8 * kNormPasses);
        return AWQ_ERR_UNSUPPORTED;
    }
    hipStream_t st = (hipStream_t)stream;
    (void)hipGetLastError();
    if (dtype == AWQ_F16)
        row_ssq_kernel<F16><<<dim3((unsigned)rows), dim3(kNormThreads), 0, st>>>((const uint16_t*)x, ssq, (int)rows, (int)hidden,
                                                                                ids, table_rows, (uint16_t*)x_out);
    else
        row_ssq_kernel<BF16><<<dim3((unsigned)rows), dim3(kNormThreads), 0, st>>>((const uint16_t*)x, ssq, (int)rows, (int)hidden,
                                                                                 ids, table_rows, (uint16_t*)x_out);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

extern "C" int nq_qk_norm_rope_store(const void* qkv, const void* q_weight, const void* k_weight, const float* cos_sin,
                                     const int64_t* positions, const int64_t* slots, void* q_out, void* k_out,
                                     void* k_cache, void* v_cache, int64_t rows, int64_t num_heads, int64_t num_kv_heads,
                                     int64_t head_dim, int64_t max_positions, int64_t num_slots, int64_t block_size,
                                     float eps, int dtype, void* stream) {
    const char* fn = "nq_qk_norm_rope_store";
    if (!qkv || !q_weight || !k_weight || !cos_sin || !positions || !slots || !q_out || !k_cache || !v_cache)
        return bad(fn, "null pointer argument");
    if (dtype != AWQ_F16 && dtype != AWQ_BF16) return bad(fn, "dtype must be AWQ_F16 or AWQ_BF16");
    if (rows <= 0 || num_heads <= 0 || num_kv_heads <= 0 || max_positions <= 0 || num_slots <= 0 || block_size <= 0 ||
        block_size > 0x7fffffff || num_slots % block_size != 0)
        return bad(fn, "rows, head counts, max_positions, block_size must be positive and num_slots a multiple of block_size");
    if (head_dim <= 0 || head_dim % 2 != 0 || head_dim > 128 * kMaxPairs) {
        set_error("%s: head_dim must be even and at most %d, got %lld", fn, 128 * kMaxPairs, (long long)head_dim);
        return AWQ_ERR_UNSUPPORTED;
    }
    const int64_t items = rows * (num_heads + 2 * num_kv_heads);
    if (items > ((int64_t)1 << 32)) return bad(fn, "too many rows");
    hipStream_t st = (hipStream_t)stream;
    (void)hipGetLastError();
    const bool vec = (head_dim == 64 || head_dim == 128 || head_dim == 256) && aligned16(qkv) && aligned16(q_weight) &&
                     aligned16(k_weight) && aligned16(cos_sin) && aligned16(q_out) && aligned16(k_out) &&
                     aligned16(k_cache) && aligned16(v_cache);
    if (vec) {
#define NQ_ROPE_VEC(TT, HH)                                                                                          \
    qk_norm_rope_store_vec_kernel<TT, HH><<<dim3((unsigned)cdiv(items, 4 * (64 / (HH / 8)))), dim3(256), 0, st>>>(  \
        (const uint16_t*)qkv, (const uint16_t*)q_weight, (const uint16_t*)k_weight, cos_sin, positions, slots,      \
        (uint16_t*)q_out, (uint16_t*)k_out, (uint16_t*)k_cache, (uint16_t*)v_cache, (int)rows, (int)num_heads,       \
        (int)num_kv_heads, (int)max_positions, num_slots, (int)block_size, eps)
        if (dtype == AWQ_F16) {
            if (head_dim == 64) NQ_ROPE_VEC(F16, 64);
            else if (head_dim == 128) NQ_ROPE_VEC(F16, 128);
            else NQ_ROPE_VEC(F16, 256);
        } else {
            if (head_dim == 64) NQ_ROPE_VEC(BF16, 64);
            else if (head_dim == 128) NQ_ROPE_VEC(BF16, 128);
            else NQ_ROPE_VEC(BF16, 256);
        }
#undef NQ_ROPE_VEC
        const hipError_t ev = hipGetLastError();
        return ev == hipSuccess ? AWQ_OK : hip_fail(fn, ev);
    }
    const dim3 grid((unsigned)cdiv(items, 4)), block(256);
    if (dtype == AWQ_F16)
        qk_norm_rope_store_kernel<F16><<<grid, block, 0, st>>>(
            (const uint16_t*)qkv, (const uint16_t*)q_weight, (const uint16_t*)k_weight, cos_sin, positions, slots,
            (uint16_t*)q_out, (uint16_t*)k_out, (uint16_t*)k_cache, (uint16_t*)v_cache, (int)rows, (int)num_heads,
            (int)num_kv_heads,
            (int)head_dim, (int)max_positions, num_slots, (int)block_size, eps);
    else
        qk_norm_rope_store_kernel<BF16><<<grid, block, 0, st>>>(
            (const uint16_t*)qkv, (const uint16_t*)q_weight, (const uint16_t*)k_weight, cos_sin, positions, slots,
            (uint16_t*)q_out, (uint16_t*)k_out, (uint16_t*)k_cache, (uint16_t*)v_cache, (int)rows, (int)num_heads,
            (int)num_kv_heads,
            (int)head_dim, (int)max_positions, num_slots, (int)block_size, eps);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

extern "C" size_t nq_paged_attention_workspace_bytes(int64_t batch, int64_t num_heads, int64_t num_kv_heads,
                                                     int64_t head_dim, int64_t max_context) {
    if (batch <= 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || max_context <= 0) return 0;
    // the block size decides the kernel and with it the split count: room for either
    const int G = (int)(num_heads / num_kv_heads);
    int s = pick_splits(batch, num_kv_heads, max_context, G, false);
    if (attn_tr(G, head_dim, 32)) s = std::max(s, pick_splits(batch, num_kv_heads, max_context, G, true));
    return s > 1 ? (size_t)(batch * num_heads * s * (head_dim + 2)) * sizeof(float) : 0;
}

extern "C" int nq_paged_attention_decode(const void* q, const void* k_cache, const void* v_cache,
                                         const int32_t* block_table, const int32_t* context_lens, void* out,
                                         int64_t batch, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                                         int64_t block_size, int64_t max_blocks_per_seq, int64_t num_blocks, float scale,
                                         int dtype, void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "nq_paged_attention_decode";
    if (!q || !k_cache || !v_cache || !block_table || !context_lens || !out) return bad(fn, "null pointer argument");
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out))
        return bad(fn, "q, caches and out must be 16-byte aligned");
    if (dtype != AWQ_F16 && dtype != AWQ_BF16) return bad(fn, "dtype must be AWQ_F16 or AWQ_BF16");
    if (batch <= 0 || num_heads <= 0 || num_kv_heads <= 0 || block_size <= 0 || max_blocks_per_seq <= 0 ||
        num_blocks <= 0 || num_heads % num_kv_heads != 0)
        return bad(fn, "sizes must be positive and num_heads a multiple of num_kv_heads");
    if (head_dim != 64 && head_dim != 128) {
        set_error("%s: head_dim must be 64 or 128, got %lld", fn, (long long)head_dim);
        return AWQ_ERR_UNSUPPORTED;
    }
    const int64_t max_context = block_size * max_blocks_per_seq;
    if (max_context > 0x7fffffff || num_blocks * block_size > 0x7fffffff || batch * num_kv_heads * 16 > 0x7fffffff)
        return bad(fn, "problem too large");
    const int nsplit = pick_splits(batch, num_kv_heads, max_context, (int)(num_heads / num_kv_heads),
                                   attn_tr((int)(num_heads / num_kv_heads), head_dim, block_size));
    const size_t need = nsplit > 1 ? (size_t)(batch * num_heads * nsplit * (head_dim + 2)) * sizeof(float) : 0;
    if (need && (!workspace || workspace_bytes < need || !aligned16(workspace))) {
        set_error("%s: workspace of %zu bytes needed, %zu given", fn, need, workspace ? workspace_bytes : (size_t)0);
        return AWQ_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    (void)hipGetLastError();
    const int G = (int)(num_heads / num_kv_heads);
    int rc;
    if (dtype == AWQ_F16)
        rc = head_dim == 128
                 ? launch_attn_g<F16, 128>(G, q, k_cache, v_cache, block_table, context_lens, out, (float*)workspace,
                                           batch, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq,
                                           (int)num_blocks, nsplit, scale, st)
                 : launch_attn_g<F16, 64>(G, q, k_cache, v_cache, block_table, context_lens, out, (float*)workspace,
                                          batch, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq,
                                          (int)num_blocks, nsplit, scale, st);
    else
        rc = head_dim == 128
                 ? launch_attn_g<BF16, 128>(G, q, k_cache, v_cache, block_table, context_lens, out, (float*)workspace,
                                            batch, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq,
                                            (int)num_blocks, nsplit, scale, st)
                 : launch_attn_g<BF16, 64>(G, q, k_cache, v_cache, block_table, context_lens, out, (float*)workspace,
                                           batch, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq,
                                           (int)num_blocks, nsplit, scale, st);
    if (rc != AWQ_OK) return rc;
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

extern "C" int nq_argmax_rows(const void* logits, int64_t* out, int64_t rows, int64_t vocab, int dtype,
                              void* stream) {
    const char* fn = "nq_argmax_rows";
    if (!logits || !out) return bad(fn, "null pointer argument");
    if (!aligned16(logits)) return bad(fn, "logits must be 16-byte aligned");
    if (dtype != AWQ_F16 && dtype != AWQ_BF16) return bad(fn, "dtype must be AWQ_F16 or AWQ_BF16");
    if (rows <= 0 || vocab <= 0 || rows > 0x7fffffff || vocab > 0x7ffffff0) return bad(fn, "rows and vocab must be positive 31-bit counts");
    hipStream_t st = (hipStream_t)stream;
    (void)hipGetLastError();
    if (dtype == AWQ_F16)
        argmax_rows_kernel<F16><<<dim3((unsigned)rows), dim3(1024), 0, st>>>((const uint16_t*)logits, out, (int)vocab);
    else
        argmax_rows_kernel<BF16><<<dim3((unsigned)rows), dim3(1024), 0, st>>>((const uint16_t*)logits, out, (int)vocab);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

extern "C" int nq_decode_prepare(const int64_t* positions, const uint8_t* active, const int32_t* block_table,
                                 int64_t* slots, int32_t* context_lens, int64_t rows, int64_t max_blocks,
                                 int64_t block_size, void* stream) {
    const char* fn = "nq_decode_prepare";
    if (!positions || !active || !block_table || !slots || !context_lens) return bad(fn, "null pointer argument");
    if (rows <= 0 || max_blocks <= 0 || block_size <= 0 || rows > 0x7fffffff || max_blocks > 0x7fffffff ||
        block_size > 0x7fffffff)
        return bad(fn, "rows, max_blocks and block_size must be positive 31-bit counts");
    (void)hipGetLastError();
    decode_prepare_kernel<<<dim3((unsigned)cdiv(rows, 256)), dim3(256), 0, (hipStream_t)stream>>>(
        positions, active, block_table, slots, context_lens, (int)rows, (int)max_blocks, (int)block_size);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

extern "C" int nq_decode_advance(const int64_t* next_tokens, const uint8_t* active, int64_t* out_log, int64_t* ids,
                                 int64_t* positions, int64_t* step, int64_t rows, int64_t out_rows, void* stream) {
    const char* fn = "nq_decode_advance";
    if (!next_tokens || !active || !out_log || !ids || !positions || !step) return bad(fn, "null pointer argument");
    if (rows <= 0 || rows > 0x7fffffff || out_rows <= 0) return bad(fn, "rows and out_rows must be positive");
    (void)hipGetLastError();
    decode_advance_kernel<<<dim3(1), dim3(1024), 0, (hipStream_t)stream>>>(next_tokens, active, out_log, ids, positions,
                                                                         step, (int)rows, out_rows);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

static int silu_mul_entry(const char* fn, bool interleaved, const void* gate_up, void* out, int64_t rows, int64_t inter,
                          int dtype, void* stream) {
    if (!gate_up || !out) return bad(fn, "null pointer argument");
    if (!aligned16(gate_up) || !aligned16(out)) return bad(fn, "tensors must be 16-byte aligned");
    if (dtype != AWQ_F16 && dtype != AWQ_BF16) return bad(fn, "dtype must be AWQ_F16 or AWQ_BF16");
    if (rows <= 0 || inter <= 0 || inter % 8 != 0) return bad(fn, "rows > 0 and inter a positive multiple of 8");
    const int64_t vecs = rows * (inter / 8);
    if (cdiv(vecs, 256) > 0x7fffffff || inter > 0x3fffffff) return bad(fn, "problem too large");
    hipStream_t st = (hipStream_t)stream;
    (void)hipGetLastError();
    const dim3 grid((unsigned)cdiv(vecs, 256)), block(256);
    if (dtype == AWQ_F16) {
        if (interleaved) silu_mul_kernel<F16, true><<<grid, block, 0, st>>>((const uint16_t*)gate_up, (uint16_t*)out, rows, (int)inter);
        else silu_mul_kernel<F16, false><<<grid, block, 0, st>>>((const uint16_t*)gate_up, (uint16_t*)out, rows, (int)inter);
    } else {
        if (interleaved) silu_mul_kernel<BF16, true><<<grid, block, 0, st>>>((const uint16_t*)gate_up, (uint16_t*)out, rows, (int)inter);
        else silu_mul_kernel<BF16, false><<<grid, block, 0, st>>>((const uint16_t*)gate_up, (uint16_t*)out, rows, (int)inter);
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AWQ_OK : hip_fail(fn, e);
}

extern "C" int nq_silu_mul(const void* gate_up, void* out, int64_t rows, int64_t inter, int dtype, void* stream) {
    return silu_mul_entry("nq_silu_mul", false, gate_up, out, rows, inter, dtype, stream);
}

extern "C" int nq_silu_mul_interleaved(const void* gate_up, void* out, int64_t rows, int64_t inter, int dtype,
                                       void* stream) {
    return silu_mul_entry("nq_silu_mul_interleaved", true, gate_up, out, rows, inter, dtype, stream);
}
