/* CPU oracle for the AWQ W4A16 linear path, plain-C restatement.
 *
 * TEST INFRASTRUCTURE, NOT PRODUCT: only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg may load the library built from this file.
 *
 * Scalar loops, written independently of oracle/awq_oracle.py (which is
 * vectorised numpy) so that the two check each other.  Citations are paths
 * under the reference checkout:
 *   awq_oracle_pack            nanoquantization/layers/gemm.py:501-520
 *   awq_oracle_unpack          nanoquantization/layers/gemm.py:52-69
 *   awq_oracle_quantize_f32    nanoquantization/utils/quantization.py:20-41
 *   awq_oracle_dequant         nanoquantization/layers/gemm.py:64-69,91,112
 *   awq_oracle_linear          nanoquantization/layers/gemm.py:303-311,560-561
 *                              (double accumulation of x * RN_dtype((q-z)*s))
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static const int kOrder[8] = {0, 2, 4, 6, 1, 3, 5, 7};

static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static float bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

static uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

static float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return bits_f32(sign);
        float v = (float)m * 5.9604644775390625e-08f; /* m * 2^-24 */
        return (sign ? -v : v);
    }
    if (e == 31) return bits_f32(sign | 0x7F800000u | (m << 13));
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* round-to-nearest-even, with subnormals, overflow to inf */
static uint16_t f32_to_f16(float f) {
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);          /* >= 65536 -> inf */
    if (a < 0x38800000u) {                                             /* < 2^-14: subnormal */
        /* value = a_float; result mantissa = RNE(a_float * 2^24) */
        float v = bits_f32(a) * 16777216.0f;                          /* exact scaling */
        float r = nearbyintf(v);                                      /* default mode: RNE */
        return (uint16_t)(sign | (uint16_t)r);
    }
    uint32_t mant = a & 0x7FFFFFu, exp = (a >> 23) - 112u;
    uint32_t half = (exp << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;      /* may carry into exp / inf */
    return (uint16_t)(sign | half);
}

static float load16(uint16_t b, int is_bf16) { return is_bf16 ? bf16_to_f32(b) : f16_to_f32(b); }
static uint16_t store16(float f, int is_bf16) { return is_bf16 ? f32_to_bf16(f) : f32_to_f16(f); }

void awq_oracle_f16_roundtrip(const float* in, int64_t n, uint16_t* bits, float* back) {
    for (int64_t i = 0; i < n; ++i) { bits[i] = f32_to_f16(in[i]); back[i] = f16_to_f32(bits[i]); }
}

void awq_oracle_pack(const int32_t* iw, int64_t rows, int64_t cols, int32_t* out) {
    int64_t words = cols / 8;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t i = 0; i < words; ++i) {
            uint32_t w = 0;
            for (int j = 0; j < 8; ++j)
                w |= ((uint32_t)iw[r * cols + i * 8 + kOrder[j]]) << (4 * j);
            out[r * words + i] = (int32_t)w;
        }
}

static inline int nibble(int32_t word, int c) {
    /* logical column c sits at nibble position p with kOrder[p] == c */
    int p = (c & 1) * 4 + (c >> 1);
    return (int)(((uint32_t)word >> (4 * p)) & 0xFu);
}

void awq_oracle_unpack(const int32_t* packed, int64_t rows, int64_t words, int32_t* out) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t i = 0; i < words; ++i)
            for (int c = 0; c < 8; ++c)
                out[(r * words + i) * 8 + c] = nibble(packed[r * words + i], c);
}

/* w [out_f, in_f] fp32 -> w_dq [out_f,in_f], s [out_f, in_f/g], z [out_f, in_f/g] */
void awq_oracle_quantize_f32(const float* w, int64_t out_f, int64_t in_f, int64_t g,
                             float* w_dq, float* s, float* z) {
    int64_t G = in_f / g;
    for (int64_t o = 0; o < out_f; ++o)
        for (int64_t gi = 0; gi < G; ++gi) {
            const float* p = w + o * in_f + gi * g;
            float hi = p[0], lo = p[0];
            for (int64_t i = 1; i < g; ++i) { if (p[i] > hi) hi = p[i]; if (p[i] < lo) lo = p[i]; }
            float range = hi - lo;
            if (range < 1e-5f) range = 1e-5f;
            float sc = range / 15.0f;
            float zp = -nearbyintf(lo / sc);
            if (zp < 0.0f) zp = 0.0f;
            if (zp > 15.0f) zp = 15.0f;
            for (int64_t i = 0; i < g; ++i) {
                float q = nearbyintf(p[i] / sc) + zp;
                if (q < 0.0f) q = 0.0f;
                if (q > 15.0f) q = 15.0f;
                w_dq[o * in_f + gi * g + i] = (q - zp) * sc;
            }
            s[o * G + gi] = sc;
            z[o * G + gi] = zp;
        }
}

/* W[k, n] = RN_dtype(float(q - z) * s[k/g, n]) as 16-bit patterns */
void awq_oracle_dequant(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales,
                        int64_t K, int64_t N, int64_t g, int is_bf16, uint16_t* out) {
    int64_t words = N / 8;
    for (int64_t k = 0; k < K; ++k) {
        int64_t gi = k / g;
        for (int64_t n = 0; n < N; ++n) {
            int q = nibble(qweight[k * words + n / 8], (int)(n % 8));
            int zp = nibble(qzeros[gi * words + n / 8], (int)(n % 8));
            float sc = load16(scales[gi * N + n], is_bf16);
            out[k * N + n] = store16((float)(q - zp) * sc, is_bf16);
        }
    }
}

/* y[m, n] = sum_k x[m,k] * W[k,n] (+ bias[n]) in double, W as awq_oracle_dequant */
void awq_oracle_linear(const uint16_t* x, const int32_t* qweight, const int32_t* qzeros,
                       const uint16_t* scales, const float* bias, int64_t M, int64_t K, int64_t N,
                       int64_t g, int is_bf16, float* y) {
    int64_t words = N / 8;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                int64_t gi = k / g;
                int q = nibble(qweight[k * words + n / 8], (int)(n % 8));
                int zp = nibble(qzeros[gi * words + n / 8], (int)(n % 8));
                float sc = load16(scales[gi * N + n], is_bf16);
                float wv = load16(store16((float)(q - zp) * sc, is_bf16), is_bf16);
                acc += (double)load16(x[m * K + k], is_bf16) * (double)wv;
            }
            if (bias) acc += (double)bias[n];
            y[m * N + n] = (float)acc;
        }
}
