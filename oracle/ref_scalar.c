/*
 * Scalar C restatement of the reference's reorder-quantize kernels.
 *
 * TEST INFRASTRUCTURE ONLY: used by tests/, by __graft_entry__.smoke() and by
 * the cpu_baseline leg of bench.py as the checker.  Never linked into or called
 * by the shipped library.
 *
 * Where oracle/mx_oracle.py works from closed forms and look-up tables, this
 * file follows the reference's float arithmetic step by step with libm
 * (log2f / ceilf / ldexpf / roundf) and converts to the element formats by
 * exponent/mantissa manipulation, so the two are independent derivations of the
 * same contract and each pins the other.
 *
 * Follows (paths relative to the reference tree):
 *   src/reorder.cu:94-269   reorder_bf16_mixed_kernel   -> orc_quantize_x
 *   src/reorder.cu:271-432  reorder_bf16_fp4_kernel     -> orc_quantize_w
 *   src/reorder.cu:54-63    pack_4_fp6_to_3_bytes
 *   src/reorder.cu:30-33    PackFp4 (even element = low nibble)
 *   src/reorder.cu:182-185  scale-factor coordinates; include/reorder.cuh:119-124
 * The NumericConverter calls (src/reorder.cu:138-143) resolve into NVIDIA
 * CUTLASS, which the reference does not vendor; their round-to-nearest-even,
 * saturating, sign-preserving behaviour is restated in f32_to_exmy().
 *
 * Parity unpinned: NaN/Inf inputs and blocks with absmax < MAX*2^-127 (the
 * scale exponent is clamped to >= -127 here; the reference leaves the normal
 * range of bf16/E8M0 there).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define GROUP 32

static float bf16_bits_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* float -> bf16 -> float, round to nearest even */
static float f32_round_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
    memcpy(&f, &u, 4);
    return f;
}

/* float -> ExMy code (sign in bit ebits+mbits), RNE, saturating at maxv, sign of
 * zero kept.  Caller passes finite values only. */
uint8_t orc_f32_to_exmy(float f, int ebits, int mbits, int bias, float maxv) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint8_t sign = (uint8_t)((u >> 31) << (ebits + mbits));
    float a = fabsf(f);
    if (a > maxv) a = maxv;
    float min_normal = ldexpf(1.0f, 1 - bias);
    uint32_t code;
    if (a < min_normal) {
        /* subnormal: multiples of 2^(1-bias-mbits); a carry lands on the first normal */
        code = (uint32_t)nearbyintf(ldexpf(a, -(1 - bias - mbits)));
    } else {
        int e;
        float m = frexpf(a, &e);       /* a = m * 2^e, m in [0.5,1) */
        m *= 2.0f;
        e -= 1;                        /* a = m * 2^e, m in [1,2)  */
        uint32_t q = (uint32_t)nearbyintf((m - 1.0f) * (float)(1 << mbits));
        if (q == (1u << mbits)) { q = 0; e += 1; }
        code = ((uint32_t)(e + bias) << mbits) | q;
    }
    return (uint8_t)(sign | code);
}

/* The reference's scale: 0.5 for an all-zero block, else
 * bf16(2^ceil(log2(amax/MAX))) (src/reorder.cu:179-180).  Returns the exponent. */
int orc_scale_exponent(float amax, float maxv) {
    if (amax == 0.0f) return -1;
    int e = (int)ceilf(log2f(amax / maxv));
    if (e < -127) e = -127;
    return e;
}

typedef struct { int ebits, mbits, bias; float maxv; } fmt_t;
static const fmt_t E2M1 = {2, 1, 1, 6.0f};
static const fmt_t E3M2 = {3, 2, 3, 28.0f};
static const fmt_t E4M3 = {4, 3, 7, 448.0f};

static int64_t sf_offset(int r, int kb, int kseg) {
    int katoms = (kseg + 127) / 128;
    return ((int64_t)(r / 128) * katoms + kb / 4) * 512 + (r % 32) * 16 + ((r / 32) % 4) * 4 + (kb % 4);
}

/* quantize one gathered 32-block; codes[32] gets one code per byte */
static uint8_t quant_block(const float *v, fmt_t f, uint8_t *codes) {
    float maxv = 0.0f;
    for (int i = 0; i < GROUP; ++i) {
        float a = fabsf(v[i]);
        maxv = maxv > a ? maxv : a;
    }
    int e = orc_scale_exponent(maxv, f.maxv);
    float scale = f32_round_bf16(ldexpf(1.0f, e));
    float r_scale = 1.0f / scale;
    for (int i = 0; i < GROUP; ++i) {
        float q = roundf(v[i] * r_scale);
        q = q < -f.maxv ? -f.maxv : (q > f.maxv ? f.maxv : q);
        /* -0.0 survives roundf and the clamp (both compares are false for it) */
        q = f32_round_bf16(q);
        codes[i] = orc_f32_to_exmy(q, f.ebits, f.mbits, f.bias, f.maxv);
    }
    return (uint8_t)(e + 127);
}

static void pack4(const uint8_t *c, uint8_t *out) {       /* 32 codes -> 16 bytes */
    for (int i = 0; i < 16; ++i) out[i] = (uint8_t)((c[2 * i] & 0xF) | ((c[2 * i + 1] & 0xF) << 4));
}

static void pack6(const uint8_t *c, uint8_t *out) {       /* 32 codes -> 24 bytes */
    for (int i = 0; i < 8; ++i) {
        uint8_t v0 = c[4 * i] & 0x3F, v1 = c[4 * i + 1] & 0x3F, v2 = c[4 * i + 2] & 0x3F, v3 = c[4 * i + 3] & 0x3F;
        out[3 * i + 0] = (uint8_t)(v0 | ((v1 & 0x03) << 6));
        out[3 * i + 1] = (uint8_t)((v1 >> 2) | ((v2 & 0x0F) << 4));
        out[3 * i + 2] = (uint8_t)((v2 >> 4) | (v3 << 2));
    }
}

static void quantize_rows(const uint16_t *x, const int16_t *idx, int rows, int K, int KN, int KS, int KO,
                          uint8_t *qn, uint8_t *qs, uint8_t *qo, uint8_t *sfn, uint8_t *sfs, uint8_t *sfo,
                          int weights) {
    int nbn = KN / GROUP, nbs = KS / GROUP, nbo = KO / GROUP;
    int64_t ldn = KN / 2;
    int64_t lds = weights ? KS / 2 : KS / 4 * 3;
    int64_t ldo = weights ? KO / 2 : KO;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        const uint16_t *row = x + (int64_t)r * K;
        float v[GROUP];
        uint8_t codes[GROUP];
        for (int b = 0; b < nbn + nbs + nbo; ++b) {
            for (int i = 0; i < GROUP; ++i) v[i] = bf16_bits_to_f32(row[(uint16_t)idx[b * GROUP + i]]);
            if (b < nbn) {
                sfn[sf_offset(r, b, KN)] = quant_block(v, E2M1, codes);
                pack4(codes, qn + r * ldn + b * 16);
            } else if (b < nbn + nbs) {
                int j = b - nbn;
                sfs[sf_offset(r, j, KS)] = quant_block(v, weights ? E2M1 : E3M2, codes);
                if (weights) pack4(codes, qs + r * lds + j * 16);
                else pack6(codes, qs + r * lds + j * 24);
            } else {
                int j = b - nbn - nbs;
                sfo[sf_offset(r, j, KO)] = quant_block(v, weights ? E2M1 : E4M3, codes);
                if (weights) pack4(codes, qo + r * ldo + j * 16);
                else memcpy(qo + r * ldo + j * 32, codes, 32);
            }
        }
    }
}

void orc_quantize_x(const uint16_t *x, const int16_t *idx, int M, int K, int KN, int KS, int KO,
                    uint8_t *qn, uint8_t *qs, uint8_t *qo, uint8_t *sfn, uint8_t *sfs, uint8_t *sfo) {
    quantize_rows(x, idx, M, K, KN, KS, KO, qn, qs, qo, sfn, sfs, sfo, 0);
}

void orc_quantize_w(const uint16_t *w, const int16_t *idx, int N, int K, int KN, int KS, int KO,
                    uint8_t *qn, uint8_t *qs, uint8_t *qo, uint8_t *sfn, uint8_t *sfs, uint8_t *sfo) {
    quantize_rows(w, idx, N, K, KN, KS, KO, qn, qs, qo, sfn, sfs, sfo, 1);
}
