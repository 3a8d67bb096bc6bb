/*
 * l2c.c -- CPU restatement of Llama2.jl's per-token decode path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP path is compared
 * against (tests/, the smoke check, and the "cpu_baseline" leg of bench.py).  The
 * product library never links, loads or calls it.
 *
 * Every function cites the reference file:line it restates (paths relative to the
 * Llama2.jl source tree).  Indices here are 0-based; the reference is 1-based.
 *
 * Numeric modes (bit flags, argument `mode`):
 *   0                     the reference snapshot: float activations, fp32 running sums
 *                         in index order, libm expf/sinf/cosf.  The reference marks its
 *                         sums `add_fast`/`@fastmath`/BLAS (order unspecified), so index
 *                         order is one legal reading of it.
 *   L2C_ACT_Q8K  (1)      activations entering a k-quant matvec are first quantized to
 *                         q8_K blocks and the dot product is done on integers
 *                         (llama.cpp's quantize_row_q8_K / vec_dot_*_q8_K rules; the
 *                         reference declares block_q8_K, src/kquants.jl:37-42, but holds
 *                         no quantizer and no integer dot).
 *   L2C_CANON    (2)      every reassociable sum is accumulated in fp64 from exact
 *                         products and rounded to fp32 once; exp/sin/cos are evaluated in
 *                         fp64 and rounded to fp32.  The result is independent of the
 *                         summation order up to fp64 round-off, so a parallel
 *                         implementation reproduces it (almost always bit for bit).
 *   3 = both              the specification of the GPU path.
 *   L2C_KV16     (4)      the rows appended to the KV cache are rounded to binary16 (round to
 *                         nearest even) and read back widened: the device's optional fp16 cache.
 *                         Not in the reference, whose cache is Float32 (src/inference.jl:62-65).
 *
 * What pins this file (the reference ships no tests, fixtures or golden vectors):
 *   codecs   hand-built blocks with by-hand expected values, per-field toggles of the
 *            6-bit scale packing, an independent numpy restatement diffed on random
 *            blocks, and the reference-implied identity vecdot(x,y) == dot(dequantize(x),y);
 *   q8_K     closed-form properties (extreme maps to -/+127, |q*d-x| <= |d|/2, bsums ==
 *            brute force, first-index tie rule, all-zero block);
 *   integer dots   brute-force triple loops over dequantized integers;
 *   rmsnorm / rope / softmax / attention / SwiGLU   float64 numpy closed forms.
 * PARITY UNPINNED (only a run of the Julia package could pin them): the last-ulp
 * behaviour of Julia's exp/cis/^ for Float32, OpenBLAS's sdot/sgemv summation order,
 * LLVM's reassociation of the add_fast chains, and StatsBase.wsample's draw order.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define QK_K 256 /* src/kquants.jl:1 */

#define L2C_ACT_Q8K 1
#define L2C_CANON 2
#define L2C_KV16 4

enum { L2C_F32 = 0, L2C_Q4_K = 12, L2C_Q5_K = 13, L2C_Q6_K = 14 }; /* src/load_gguf.jl:26-42 */

#pragma pack(push, 1)
typedef struct { /* src/kquants.jl:7-12, 144 bytes */
    uint16_t d, dmin;
    uint8_t scales[12];
    uint8_t qs[QK_K / 2];
} block_q4_K;
typedef struct { /* src/kquants.jl:18-24, 176 bytes */
    uint16_t d, dmin;
    uint8_t scales[12];
    uint8_t qh[QK_K / 8];
    uint8_t qs[QK_K / 2];
} block_q5_K;
typedef struct { /* src/kquants.jl:30-35, 210 bytes */
    uint8_t ql[QK_K / 2];
    uint8_t qh[QK_K / 4];
    int8_t scales[QK_K / 16];
    uint16_t d;
} block_q6_K;
typedef struct { /* src/kquants.jl:38-42, 292 bytes */
    float d;
    int8_t qs[QK_K];
    int16_t bsums[QK_K / 16];
} block_q8_K;
#pragma pack(pop)

_Static_assert(sizeof(block_q4_K) == 144, "q4_K");
_Static_assert(sizeof(block_q5_K) == 176, "q5_K");
_Static_assert(sizeof(block_q6_K) == 210, "q6_K");
_Static_assert(sizeof(block_q8_K) == 292, "q8_K");

int64_t l2c_block_bytes(int type) {
    switch (type) {
    case L2C_F32: return 4;
    case L2C_Q4_K: return 144;
    case L2C_Q5_K: return 176;
    case L2C_Q6_K: return 210;
    }
    return -1;
}

/* IEEE binary32 -> binary16, round to nearest even, overflow to infinity, subnormals kept (what
 * Julia's Float16(::Float32) and numpy's astype(float16) do). */
uint16_t l2c_fp32_to_fp16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t mag = x & 0x7FFFFFFFu;
    if (mag >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | ((mag > 0x7F800000u) ? 0x200u : 0u)); /* inf / nan */
    if (mag >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to infinity */
    if (mag < 0x33000001u) return (uint16_t)sign;               /* <= 2^-25: rounds to zero (2^-25 itself ties to even 0) */
    const int e = (int)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    int shift;                                      /* bits to drop */
    uint32_t base;
    if (e >= -14) { /* normal half: keep 11 bits */
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7FFFFFu; /* implicit bit goes into the exponent field */
    } else {          /* subnormal half: value = man * 2^(e-23), unit 2^-24 */
        shift = 13 + (-14 - e);
        base = 0;
    }
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++; /* a carry runs into the exponent field: correct */
    return (uint16_t)(sign | (base + q));
}

/* IEEE binary16 -> binary32, exact (Julia's Float32(::Float16), src/kquants.jl:74). */
float l2c_fp16_to_fp32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* 6-bit scale/min of sub-block s (0..7) from the 12 packed bytes.
 * s<4: src/kquants.jl:80-81,86-87.  s>=4: src/kquants.jl:102-103,108-109. */
static inline void scale_min_k4(int s, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (s < 4) {
        *sc = q[s] & 63;
        *m = q[s + 4] & 63;
    } else {
        *sc = (uint8_t)((q[s + 4] & 0xF) | ((q[s - 4] >> 6) << 4));
        *m = (uint8_t)((q[s + 4] >> 4) | ((q[s] >> 6) << 4));
    }
}

void l2c_scale_min_k4(const uint8_t *packed12, uint8_t *sc8, uint8_t *m8) {
    for (int s = 0; s < 8; s++) scale_min_k4(s, packed12, &sc8[s], &m8[s]);
}

/* ------------------------------------------------------------------------------------
 * dequantize!  (src/kquants.jl:70-125 q4_K, :186-251 q5_K, :322-363 q6_K)
 * ---------------------------------------------------------------------------------- */
void l2c_dequantize_q4_K(const void *vx, int64_t nb, float *y) {
    const block_q4_K *x = (const block_q4_K *)vx;
    for (int64_t i = 0; i < nb; i++) {
        const float d = l2c_fp16_to_fp32(x[i].d);
        const float dmin = l2c_fp16_to_fp32(x[i].dmin);
        const uint8_t *q = x[i].qs;
        for (int j = 0; j < 4; j++) { /* pairs of sub-blocks; :79 and :101 */
            uint8_t sc, m;
            scale_min_k4(2 * j, x[i].scales, &sc, &m);
            const float d1 = d * (float)sc, m1 = dmin * (float)m; /* :83-84 */
            scale_min_k4(2 * j + 1, x[i].scales, &sc, &m);
            const float d2 = d * (float)sc, m2 = dmin * (float)m; /* :89-90 */
            for (int l = 0; l < 32; l++) /* :92-94 */
                y[QK_K * i + 64 * j + l] = d1 * (float)(q[32 * j + l] & 0xF) - m1;
            for (int l = 0; l < 32; l++) /* :96-98 */
                y[QK_K * i + 64 * j + 32 + l] = d2 * (float)(q[32 * j + l] >> 4) - m2;
        }
    }
}

void l2c_dequantize_q5_K(const void *vx, int64_t nb, float *y) {
    const block_q5_K *x = (const block_q5_K *)vx;
    for (int64_t i = 0; i < nb; i++) {
        const float d = l2c_fp16_to_fp32(x[i].d);
        const float dmin = l2c_fp16_to_fp32(x[i].dmin);
        const uint8_t *ql = x[i].qs, *qh = x[i].qh;
        uint8_t u1 = 1, u2 = 2; /* :196-197 */
        for (int j = 0; j < 4; j++) {
            uint8_t sc, m;
            scale_min_k4(2 * j, x[i].scales, &sc, &m);
            const float d1 = d * (float)sc, m1 = dmin * (float)m;
            scale_min_k4(2 * j + 1, x[i].scales, &sc, &m);
            const float d2 = d * (float)sc, m2 = dmin * (float)m;
            for (int l = 0; l < 32; l++) /* :213 */
                y[QK_K * i + 64 * j + l] =
                    d1 * (float)(uint8_t)((ql[32 * j + l] & 0xF) + ((qh[l] & u1) ? 16 : 0)) - m1;
            for (int l = 0; l < 32; l++) /* :217 */
                y[QK_K * i + 64 * j + 32 + l] =
                    d2 * (float)(uint8_t)((ql[32 * j + l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - m2;
            u1 <<= 2; /* :220-221 */
            u2 <<= 2;
        }
    }
}

/* the four 6-bit quants that share ql/qh bytes; src/kquants.jl:333-336 */
static inline void q6_quads(const block_q6_K *b, int n, int l, int *q1, int *q2, int *q3, int *q4) {
    const uint8_t *ql = b->ql + 64 * n, *qh = b->qh + 32 * n;
    *q1 = (int)(int8_t)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
    *q2 = (int)(int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
    *q3 = (int)(int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
    *q4 = (int)(int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
}

void l2c_dequantize_q6_K(const void *vx, int64_t nb, float *y) {
    const block_q6_K *x = (const block_q6_K *)vx;
    for (int64_t i = 0; i < nb; i++) {
        const float d = l2c_fp16_to_fp32(x[i].d);
        for (int n = 0; n < QK_K / 128; n++) {
            for (int l = 0; l < 32; l++) {
                int q1, q2, q3, q4;
                q6_quads(&x[i], n, l, &q1, &q2, &q3, &q4);
                const int is = 8 * n + l / 16; /* :338, :352 */
                const int8_t *sc = x[i].scales;
                float *o = y + QK_K * i + 128 * n + l;
                o[0] = d * (float)(int16_t)(sc[is + 0] * q1); /* :340-343 */
                o[32] = d * (float)(int16_t)(sc[is + 2] * q2);
                o[64] = d * (float)(int16_t)(sc[is + 4] * q3);
                o[96] = d * (float)(int16_t)(sc[is + 6] * q4);
            }
        }
    }
}

int l2c_dequantize(int type, const void *x, int64_t nb, float *y) {
    switch (type) {
    case L2C_F32: memcpy(y, x, (size_t)nb * 4); return 0; /* src/kquants.jl:44-47; nb = element count */
    case L2C_Q4_K: l2c_dequantize_q4_K(x, nb, y); return 0;
    case L2C_Q5_K: l2c_dequantize_q5_K(x, nb, y); return 0;
    case L2C_Q6_K: l2c_dequantize_q6_K(x, nb, y); return 0;
    }
    return -1;
}

/* ------------------------------------------------------------------------------------
 * vecdot with float activations (src/kquants.jl:127-184, :253-320, :365-408).
 * The weight value is formed exactly as in dequantize! (same expression in the
 * reference), multiplied by y in fp32, then added: fp32 running sum in index order
 * (canon=0) or fp64 sum of the fp32 products' exact values... see below.
 *
 * canon=1: the fp32 weight value w (rounded as the reference rounds it) times y is
 * taken exactly (fp64 product of two fp32 numbers) and summed in fp64; one final
 * rounding to fp32.
 * ---------------------------------------------------------------------------------- */
static float dot_f32(const float *w, const float *y, int64_t n, int canon) {
    if (canon) {
        double s = 0.0;
        for (int64_t i = 0; i < n; i++) s += (double)w[i] * (double)y[i];
        return (float)s;
    }
    float s = 0.0f;
    for (int64_t i = 0; i < n; i++) s = s + y[i] * w[i];
    return s;
}

float l2c_vecdot_f32act(int type, const void *x, int64_t nb, const float *y, int canon) {
    /* Per super-block: dequantize 256 values with the reference expressions, then
     * accumulate y*w in element order -- the same sequence of roundings as the fused
     * loops at src/kquants.jl:152,156 / :282,286 / :385-388 when the q6_K inner loop
     * is read in element order.  (q6_K's reference loop interleaves four strided
     * elements per l; with add_fast the order is not part of its meaning.) */
    float w[QK_K];
    if (canon) {
        double s = 0.0;
        for (int64_t i = 0; i < nb; i++) {
            l2c_dequantize(type, (const char *)x + i * l2c_block_bytes(type), 1, w);
            for (int k = 0; k < QK_K; k++) s += (double)w[k] * (double)y[QK_K * i + k];
        }
        return (float)s;
    }
    float s = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        l2c_dequantize(type, (const char *)x + i * l2c_block_bytes(type), 1, w);
        for (int k = 0; k < QK_K; k++) s = s + y[QK_K * i + k] * w[k];
    }
    return s;
}

/* ------------------------------------------------------------------------------------
 * q8_K activation quantizer.  The reference declares the block (src/kquants.jl:37-42)
 * and nothing else; the rule below is llama.cpp's quantize_row_q8_K_ref (ggml-quants.c,
 * the project the reference's README names as the source of its quantization code):
 * scan ascending, keep the first element of largest magnitude (strict >), iscale =
 * -127/max, q = min(127, round-half-even(iscale*x)), bsums over groups of 16, d = 1/iscale.
 * ---------------------------------------------------------------------------------- */
void l2c_quantize_q8_K(const float *x, int64_t n, void *vy) {
    block_q8_K *y = (block_q8_K *)vy;
    const int64_t nb = n / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        float max = 0.0f, amax = 0.0f;
        for (int j = 0; j < QK_K; j++) {
            const float ax = fabsf(x[j]);
            if (ax > amax) {
                amax = ax;
                max = x[j];
            }
        }
        if (amax == 0.0f) {
            memset(&y[i], 0, sizeof(block_q8_K));
            x += QK_K;
            continue;
        }
        const float iscale = -127.0f / max;
        for (int j = 0; j < QK_K; j++) {
            int v = (int)rintf(iscale * x[j]); /* default rounding mode = ties-to-even */
            y[i].qs[j] = (int8_t)(v < 127 ? v : 127);
        }
        for (int g = 0; g < QK_K / 16; g++) {
            int sum = 0;
            for (int k = 0; k < 16; k++) sum += y[i].qs[16 * g + k];
            y[i].bsums[g] = (int16_t)sum;
        }
        y[i].d = 1.0f / iscale;
        x += QK_K;
    }
}

/* ------------------------------------------------------------------------------------
 * integer dot products k-quant x q8_K (llama.cpp's ggml_vec_dot_q{4,5,6}_K_q8_K generic
 * path, expressed per super-block).  For super-block b:
 *   q4_K/q5_K:  I_sc  = sum_s sc_s * sum_{e in sub-block s} q_e * q8_e
 *               I_min = sum_s m_s  * (bsums[2s] + bsums[2s+1])
 *               term  = (d*yd) * I_sc - (dmin*yd) * I_min
 *   q6_K:       I_sc  = sum_{s<16} sc_s * sum_{e in 16-group s} (q_e - 32) * q8_e,  I_min = 0
 *               term  = (d*yd) * I_sc
 * where q_e are the unsigned/offset integer quants that dequantize! multiplies by the
 * scale (same bit extraction as src/kquants.jl:93,97,213,217,333-336), d*yd and dmin*yd
 * are rounded to fp32.  canon=0: term rounded to fp32 step by step, fp32 running sum
 * over blocks.  canon=1: the two products are exact in fp64, fp64 sum over blocks, one
 * final rounding.
 * I_sc / I_min (may be NULL) receive the per-block integers.
 * ---------------------------------------------------------------------------------- */
static void block_ints_q4_K(const block_q4_K *x, const block_q8_K *y, int32_t *isc, int32_t *imin) {
    int32_t a = 0, b = 0;
    for (int s = 0; s < 8; s++) {
        uint8_t sc, m;
        scale_min_k4(s, x->scales, &sc, &m);
        const int j = s >> 1;
        int32_t dot = 0;
        for (int l = 0; l < 32; l++) {
            const int q = (s & 1) ? (x->qs[32 * j + l] >> 4) : (x->qs[32 * j + l] & 0xF);
            dot += q * (int)y->qs[32 * s + l];
        }
        a += (int32_t)sc * dot;
        b += (int32_t)m * ((int32_t)y->bsums[2 * s] + (int32_t)y->bsums[2 * s + 1]);
    }
    *isc = a;
    *imin = b;
}

static void block_ints_q5_K(const block_q5_K *x, const block_q8_K *y, int32_t *isc, int32_t *imin) {
    int32_t a = 0, b = 0;
    for (int s = 0; s < 8; s++) {
        uint8_t sc, m;
        scale_min_k4(s, x->scales, &sc, &m);
        const int j = s >> 1;
        int32_t dot = 0;
        for (int l = 0; l < 32; l++) {
            int q = (s & 1) ? (x->qs[32 * j + l] >> 4) : (x->qs[32 * j + l] & 0xF);
            if (x->qh[l] & (1u << s)) q += 16;
            dot += q * (int)y->qs[32 * s + l];
        }
        a += (int32_t)sc * dot;
        b += (int32_t)m * ((int32_t)y->bsums[2 * s] + (int32_t)y->bsums[2 * s + 1]);
    }
    *isc = a;
    *imin = b;
}

static void block_ints_q6_K(const block_q6_K *x, const block_q8_K *y, int32_t *isc, int32_t *imin) {
    int32_t a = 0;
    for (int n = 0; n < 2; n++) {
        for (int l = 0; l < 32; l++) {
            int q1, q2, q3, q4;
            q6_quads(x, n, l, &q1, &q2, &q3, &q4);
            const int is = 8 * n + l / 16;
            const int8_t *q8 = y->qs + 128 * n + l;
            a += (int32_t)x->scales[is + 0] * q1 * (int)q8[0];
            a += (int32_t)x->scales[is + 2] * q2 * (int)q8[32];
            a += (int32_t)x->scales[is + 4] * q3 * (int)q8[64];
            a += (int32_t)x->scales[is + 6] * q4 * (int)q8[96];
        }
    }
    *isc = a;
    *imin = 0;
}

float l2c_vecdot_q8k(int type, const void *vx, const void *vy, int64_t nb, int canon, int32_t *I_sc,
                     int32_t *I_min) {
    const block_q8_K *y = (const block_q8_K *)vy;
    float s32 = 0.0f;
    double s64 = 0.0;
    for (int64_t i = 0; i < nb; i++) {
        int32_t a = 0, b = 0;
        float d = 0.0f, dmin = 0.0f;
        if (type == L2C_Q4_K) {
            const block_q4_K *x = (const block_q4_K *)vx + i;
            block_ints_q4_K(x, &y[i], &a, &b);
            d = l2c_fp16_to_fp32(x->d);
            dmin = l2c_fp16_to_fp32(x->dmin);
        } else if (type == L2C_Q5_K) {
            const block_q5_K *x = (const block_q5_K *)vx + i;
            block_ints_q5_K(x, &y[i], &a, &b);
            d = l2c_fp16_to_fp32(x->d);
            dmin = l2c_fp16_to_fp32(x->dmin);
        } else {
            const block_q6_K *x = (const block_q6_K *)vx + i;
            block_ints_q6_K(x, &y[i], &a, &b);
            d = l2c_fp16_to_fp32(x->d);
        }
        if (I_sc) I_sc[i] = a;
        if (I_min) I_min[i] = b;
        const float dy = d * y[i].d, my = dmin * y[i].d;
        if (canon) {
            s64 += (double)dy * (double)a - (double)my * (double)b;
        } else {
            const float t1 = dy * (float)a;
            const float t2 = my * (float)b;
            s32 = s32 + (t1 - t2);
        }
    }
    return canon ? (float)s64 : s32;
}

/* ------------------------------------------------------------------------------------
 * matmul!(y, A, x):  y[i] = A[:, i] . x   (src/matmul.jl:3-11 fp32, :13-23 k-quant).
 * A holds ne1 output rows of ne0 input features each, row-contiguous (GGUF ne0 fastest).
 * Rows are split over threads as Threads.@threads does (src/matmul.jl:18).
 * xq8 (k-quant + L2C_ACT_Q8K only): the already-quantized x, or NULL to quantize here.
 * ---------------------------------------------------------------------------------- */
int l2c_matmul(int type, const void *A, int64_t ne0, int64_t ne1, const float *x, const void *xq8, float *y,
               int mode, int nthreads) {
    const int canon = (mode & L2C_CANON) != 0;
    if (nthreads < 1) nthreads = 1;
    if (type == L2C_F32) {
        const float *a = (const float *)A;
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t i = 0; i < ne1; i++) y[i] = dot_f32(a + i * ne0, x, ne0, canon);
        return 0;
    }
    if (ne0 % QK_K != 0) return -1; /* src/load_gguf.jl:141 */
    const int64_t nb = ne0 / QK_K, bs = l2c_block_bytes(type);
    if (bs < 0) return -1;
    if (mode & L2C_ACT_Q8K) {
        void *tmp = NULL;
        if (!xq8) {
            tmp = malloc((size_t)nb * sizeof(block_q8_K));
            l2c_quantize_q8_K(x, ne0, tmp);
            xq8 = tmp;
        }
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t i = 0; i < ne1; i++)
            y[i] = l2c_vecdot_q8k(type, (const char *)A + i * nb * bs, xq8, nb, canon, NULL, NULL);
        free(tmp);
    } else {
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t i = 0; i < ne1; i++)
            y[i] = l2c_vecdot_f32act(type, (const char *)A + i * nb * bs, nb, x, canon);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------
 * rmsnorm!(o, x, weight)  src/inference.jl:102-110.  o may alias x (:309).
 * ---------------------------------------------------------------------------------- */
void l2c_rmsnorm(float *o, const float *x, const float *weight, int64_t n, int mode) {
    float ss;
    if (mode & L2C_CANON) {
        double s = 0.0;
        for (int64_t i = 0; i < n; i++) s += (double)x[i] * (double)x[i];
        ss = (float)s;
    } else {
        ss = 0.0f;
        for (int64_t i = 0; i < n; i++) ss = ss + x[i] * x[i];
    }
    ss /= (float)n;        /* :104 */
    ss += 1e-5f;           /* :105 */
    ss = 1.0f / sqrtf(ss); /* :106 */
    for (int64_t i = 0; i < n; i++) o[i] = weight[i] * (ss * x[i]); /* :108 */
}

/* theta_scale = freq_base ^ (-1/(head_size/2)) in fp32; src/inference.jl:119,140 */
float l2c_rope_theta_scale(float freq_base, int head_size) {
    return powf(freq_base, -(1.0f / (float)(head_size / 2)));
}

/* rope!(x, pos, config)  src/inference.jl:112-131 (interleaved pairs) and :133-157
 * (neox: pairs (i, i+head_size/2)).  pos0 is 0-based (= the reference's pos-1, :122).
 * theta is advanced by repeated fp32 multiplication (:126,:152). */
void l2c_rope(float *x, int head_size, int n_heads, int pos0, float theta_scale, int neox, int mode) {
    const int half = head_size / 2;
    for (int h = 0; h < n_heads; h++) {
        float theta = 1.0f * (float)pos0; /* freq_scale = 1 (:117,:122) */
        float *xh = x + (int64_t)h * head_size;
        for (int i = 0; i < half; i++) {
            float c, s;
            if (mode & L2C_CANON) {
                c = (float)cos((double)theta);
                s = (float)sin((double)theta);
            } else {
                c = cosf(theta);
                s = sinf(theta);
            }
            float *pr = neox ? &xh[i] : &xh[2 * i];
            float *pi = neox ? &xh[half + i] : &xh[2 * i + 1];
            const float a = *pr, b = *pi;
            /* Complex{Float32} product: (a+bi)(c+si), each product rounded */
            const float ac = a * c, bs = b * s, as = a * s, bc = b * c;
            *pr = ac - bs;
            *pi = as + bc;
            theta *= theta_scale;
        }
    }
}

/* softmax!(x)  src/inference.jl:169-174 */
void l2c_softmax(float *x, int64_t n, int mode) {
    float mx = x[0];
    for (int64_t i = 1; i < n; i++)
        if (x[i] > mx) mx = x[i];
    if (mode & L2C_CANON) {
        double s = 0.0;
        for (int64_t i = 0; i < n; i++) {
            x[i] = (float)exp((double)(x[i] - mx));
            s += (double)x[i];
        }
        const float sf = (float)s;
        for (int64_t i = 0; i < n; i++) x[i] /= sf;
    } else {
        float s = 0.0f;
        for (int64_t i = 0; i < n; i++) {
            x[i] = expf(x[i] - mx);
            s = s + x[i];
        }
        for (int64_t i = 0; i < n; i++) x[i] /= s;
    }
}

/* One head-group of decode attention for position pos0 (0-based), i.e. over cache
 * entries t = 0..pos0:  attention_weights! (src/inference.jl:176-197), the scaling by
 * sqrt(head_size) (:268), softmax per head (:270-273), combine_values! (:199-220).
 * Cache layout here: kc[t*kv_dim + kvh*hs + i], vc likewise (the reference's
 * (hs,n_kv,seq) / (seq,hs,n_kv) arrays hold the same numbers).
 * att: scratch of n_heads*(pos0+1) floats, returned filled with the probabilities. */
void l2c_attention(float *out, const float *q, const float *kc, const float *vc, float *att, int head_size,
                   int n_heads, int n_kv_heads, int pos0, int mode) {
    const int n_gqa = n_heads / n_kv_heads, kv_dim = head_size * n_kv_heads, np = pos0 + 1;
    const int canon = (mode & L2C_CANON) != 0;
    const float scale = sqrtf((float)head_size);
    for (int h = 0; h < n_heads; h++) {
        const int kvh = h / n_gqa; /* :191-193 */
        const float *qh = q + (int64_t)h * head_size;
        float *a = att + (int64_t)h * np;
        for (int t = 0; t < np; t++) {
            const float *k = kc + (int64_t)t * kv_dim + (int64_t)kvh * head_size;
            if (canon) {
                double s = 0.0;
                for (int i = 0; i < head_size; i++) s += (double)qh[i] * (double)k[i];
                a[t] = (float)s;
            } else {
                float s = 0.0f;
                for (int i = 0; i < head_size; i++) s = s + qh[i] * k[i];
                a[t] = s;
            }
        }
        for (int t = 0; t < np; t++) a[t] /= scale; /* :268 */
        l2c_softmax(a, np, mode);
        for (int i = 0; i < head_size; i++) {
            if (canon) {
                double s = 0.0;
                for (int t = 0; t < np; t++)
                    s += (double)a[t] * (double)vc[(int64_t)t * kv_dim + (int64_t)kvh * head_size + i];
                out[(int64_t)h * head_size + i] = (float)s;
            } else {
                float s = 0.0f;
                for (int t = 0; t < np; t++) s = s + a[t] * vc[(int64_t)t * kv_dim + (int64_t)kvh * head_size + i];
                out[(int64_t)h * head_size + i] = s;
            }
        }
    }
}

/* hb[i] = hb[i] * (1/(1+exp(-hb[i]))); hb .*= hb2   src/inference.jl:295-299 */
void l2c_swiglu(float *hb, const float *hb2, int64_t n, int mode) {
    for (int64_t i = 0; i < n; i++) {
        float e;
        if (mode & L2C_CANON)
            e = (float)exp((double)(-hb[i]));
        else
            e = expf(-hb[i]);
        const float v = hb[i] * (1.0f / (1.0f + e));
        hb[i] = v * hb2[i];
    }
}

/* argmax(logits): first maximal index (Julia semantics), 0-based; src/inference.jl:360 */
int64_t l2c_argmax(const float *x, int64_t n) {
    int64_t best = 0;
    for (int64_t i = 1; i < n; i++)
        if (x[i] > x[best]) best = i;
    return best;
}

/* ------------------------------------------------------------------------------------
 * Model container + transformer!  (src/inference.jl:27-100, :222-315)
 * ---------------------------------------------------------------------------------- */
typedef struct {
    int32_t dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
    float rope_freq_base;
    int32_t rope_is_neox;
} l2c_config; /* ModelConfig, src/inference.jl:1-11 */

enum {
    L2C_TOK_EMB = 0, L2C_RMS_FINAL = 1, L2C_OUTPUT = 2, /* per-model */
    L2C_RMS_ATT = 3, L2C_RMS_FFN = 4, L2C_WQ = 5, L2C_WK = 6, L2C_WV = 7, L2C_WO = 8, L2C_W1 = 9, L2C_W2 = 10,
    L2C_W3 = 11, L2C_N_ROLES = 12
};

typedef struct {
    const void *p;
    int type;
    int64_t ne0, ne1;
} l2c_tensor;

typedef struct l2c_model {
    l2c_config c;
    l2c_tensor glob[3];
    l2c_tensor *layer; /* [n_layers][L2C_N_ROLES] */
    /* RunState, src/inference.jl:72-100 */
    float *x, *xb, *xb2, *hb, *hb2, *q, *k, *v, *att, *logits;
    float *kc, *vc; /* [n_layers][seq_len][kv_dim] */
    void *q8;       /* scratch for quantized activations */
    int nthreads;
} l2c_model;

l2c_model *l2c_model_create(const l2c_config *c, int nthreads) {
    l2c_model *m = (l2c_model *)calloc(1, sizeof(l2c_model));
    m->c = *c;
    m->nthreads = nthreads < 1 ? 1 : nthreads;
    const int hs = c->dim / c->n_heads, kv_dim = hs * c->n_kv_heads;
    m->layer = (l2c_tensor *)calloc((size_t)c->n_layers * L2C_N_ROLES, sizeof(l2c_tensor));
    m->x = (float *)calloc(c->dim, 4);
    m->xb = (float *)calloc(c->dim, 4);
    m->xb2 = (float *)calloc(c->dim, 4);
    m->hb = (float *)calloc(c->hidden_dim, 4);
    m->hb2 = (float *)calloc(c->hidden_dim, 4);
    m->q = (float *)calloc(c->dim, 4);
    m->k = (float *)calloc(kv_dim, 4);
    m->v = (float *)calloc(kv_dim, 4);
    m->att = (float *)calloc((size_t)c->seq_len * c->n_heads, 4);
    m->logits = (float *)calloc(c->vocab_size, 4);
    m->kc = (float *)calloc((size_t)c->n_layers * c->seq_len * kv_dim, 4);
    m->vc = (float *)calloc((size_t)c->n_layers * c->seq_len * kv_dim, 4);
    const int64_t maxk = c->dim > c->hidden_dim ? c->dim : c->hidden_dim;
    m->q8 = calloc((size_t)(maxk / QK_K + 1), sizeof(block_q8_K));
    return m;
}

void l2c_model_destroy(l2c_model *m) {
    if (!m) return;
    free(m->layer); free(m->x); free(m->xb); free(m->xb2); free(m->hb); free(m->hb2); free(m->q);
    free(m->k); free(m->v); free(m->att); free(m->logits); free(m->kc); free(m->vc); free(m->q8);
    free(m);
}

/* host pointer is borrowed: it must outlive the model */
int l2c_model_set_tensor(l2c_model *m, int role, int layer, int type, const void *p, int64_t ne0, int64_t ne1) {
    if (role < 0 || role >= L2C_N_ROLES) return -1;
    l2c_tensor t = {p, type, ne0, ne1};
    if (role < 3)
        m->glob[role] = t;
    else {
        if (layer < 0 || layer >= m->c.n_layers) return -1;
        m->layer[(size_t)layer * L2C_N_ROLES + role] = t;
    }
    return 0;
}

void l2c_state_reset(l2c_model *m) {
    const int hs = m->c.dim / m->c.n_heads, kv_dim = hs * m->c.n_kv_heads;
    memset(m->kc, 0, (size_t)m->c.n_layers * m->c.seq_len * kv_dim * 4);
    memset(m->vc, 0, (size_t)m->c.n_layers * m->c.seq_len * kv_dim * 4);
}

/* write n cache rows (post-RoPE keys, values) of one layer starting at pos0 */
int l2c_kv_write(l2c_model *m, int layer, int pos0, int n, const float *k, const float *v) {
    const int hs = m->c.dim / m->c.n_heads, kv_dim = hs * m->c.n_kv_heads;
    if (layer < 0 || layer >= m->c.n_layers || pos0 < 0 || pos0 + n > m->c.seq_len) return -1;
    const size_t off = ((size_t)layer * m->c.seq_len + pos0) * kv_dim;
    memcpy(m->kc + off, k, (size_t)n * kv_dim * 4);
    memcpy(m->vc + off, v, (size_t)n * kv_dim * 4);
    return 0;
}

int l2c_kv_read(l2c_model *m, int layer, int pos0, int n, float *k, float *v) {
    const int hs = m->c.dim / m->c.n_heads, kv_dim = hs * m->c.n_kv_heads;
    if (layer < 0 || layer >= m->c.n_layers || pos0 < 0 || pos0 + n > m->c.seq_len) return -1;
    const size_t off = ((size_t)layer * m->c.seq_len + pos0) * kv_dim;
    memcpy(k, m->kc + off, (size_t)n * kv_dim * 4);
    memcpy(v, m->vc + off, (size_t)n * kv_dim * 4);
    return 0;
}

/* matmul! on a model tensor */
static void mm(l2c_model *m, float *y, const l2c_tensor *t, const float *x, int mode) {
    const void *xq8 = NULL;
    if (t->type != L2C_F32 && (mode & L2C_ACT_Q8K)) {
        l2c_quantize_q8_K(x, t->ne0, m->q8);
        xq8 = m->q8;
    }
    l2c_matmul(t->type, t->p, t->ne0, t->ne1, x, xq8, y, mode, m->nthreads);
}

/* transformer!(token, pos, config, s, weights)  src/inference.jl:222-315.
 * token and pos0 are 0-based.  Writes m->logits; copies to logits_out if non-NULL. */
int l2c_forward(l2c_model *m, int token, int pos0, int mode, float *logits_out) {
    const l2c_config *c = &m->c;
    const int dim = c->dim, hs = dim / c->n_heads, kv_dim = hs * c->n_kv_heads;
    if (token < 0 || token >= c->vocab_size || pos0 < 0 || pos0 >= c->seq_len) return -1;
    const float theta_scale = l2c_rope_theta_scale(c->rope_freq_base, hs);

    { /* :236  dequantize!(x, token_embedding_table[:, token]) */
        const l2c_tensor *e = &m->glob[L2C_TOK_EMB];
        if (e->type == L2C_F32)
            memcpy(m->x, (const float *)e->p + (size_t)token * dim, (size_t)dim * 4);
        else
            l2c_dequantize(e->type, (const char *)e->p + (size_t)token * (dim / QK_K) * l2c_block_bytes(e->type),
                           dim / QK_K, m->x);
    }

    for (int l = 0; l < c->n_layers; l++) {
        const l2c_tensor *w = m->layer + (size_t)l * L2C_N_ROLES;
        float *kc = m->kc + (size_t)l * c->seq_len * kv_dim;
        float *vc = m->vc + (size_t)l * c->seq_len * kv_dim;

        l2c_rmsnorm(m->xb, m->x, (const float *)w[L2C_RMS_ATT].p, dim, mode); /* :244 */
        mm(m, m->q, &w[L2C_WQ], m->xb, mode);                               /* :247 */
        mm(m, m->k, &w[L2C_WK], m->xb, mode); /* :248 */
        mm(m, m->v, &w[L2C_WV], m->xb, mode);                               /* :249 */
        l2c_rope(m->q, hs, c->n_heads, pos0, theta_scale, c->rope_is_neox, mode);    /* :255 */
        l2c_rope(m->k, hs, c->n_kv_heads, pos0, theta_scale, c->rope_is_neox, mode); /* :256 */
        if (mode & L2C_KV16) {
            for (int i = 0; i < kv_dim; i++) {
                m->k[i] = l2c_fp16_to_fp32(l2c_fp32_to_fp16(m->k[i]));
                m->v[i] = l2c_fp16_to_fp32(l2c_fp32_to_fp16(m->v[i]));
            }
        }
        memcpy(kc + (size_t)pos0 * kv_dim, m->k, (size_t)kv_dim * 4); /* :259 */
        memcpy(vc + (size_t)pos0 * kv_dim, m->v, (size_t)kv_dim * 4); /* :260 */
        l2c_attention(m->xb, m->q, kc, vc, m->att, hs, c->n_heads, c->n_kv_heads, pos0, mode); /* :266-278 */
        mm(m, m->xb2, &w[L2C_WO], m->xb, mode);           /* :281 */
        for (int i = 0; i < dim; i++) m->x[i] += m->xb2[i];  /* :284 */
        l2c_rmsnorm(m->xb, m->x, (const float *)w[L2C_RMS_FFN].p, dim, mode); /* :287 */
        mm(m, m->hb, &w[L2C_W1], m->xb, mode);            /* :291 */
        mm(m, m->hb2, &w[L2C_W3], m->xb, mode);           /* :292 */
        l2c_swiglu(m->hb, m->hb2, c->hidden_dim, mode);      /* :295-299 */
        mm(m, m->xb, &w[L2C_W2], m->hb, mode);            /* :302 */
        for (int i = 0; i < dim; i++) m->x[i] += m->xb[i];   /* :305 */
    }
    l2c_rmsnorm(m->x, m->x, (const float *)m->glob[L2C_RMS_FINAL].p, dim, mode); /* :309 */
    mm(m, m->logits, &m->glob[L2C_OUTPUT], m->x, mode);                       /* :312 */
    if (logits_out) memcpy(logits_out, m->logits, (size_t)c->vocab_size * 4);
    return 0;
}

/* The token loop of sample() with temperature == 0 (src/inference.jl:349-386), on token
 * ids: feeds prompt[0..n_prompt) from position pos0, then n_new greedy tokens.
 * out receives the n_new generated ids (0-based).  last_logits (may be NULL) receives
 * the logits of the final forward call. */
int l2c_generate_greedy(l2c_model *m, const int32_t *prompt, int n_prompt, int pos0, int n_new, int mode,
                        int32_t *out, float *last_logits) {
    if (n_prompt < 1) return -1; /* :326-328 */
    int token = prompt[0];
    int produced = 0;
    const int total = n_prompt - 1 + n_new;
    for (int step = 0; step < total; step++) {
        if (pos0 + step >= m->c.seq_len) break; /* :349 */
        int rc = l2c_forward(m, token, pos0 + step, mode, NULL);
        if (rc) return rc;
        int next;
        if (step + 1 < n_prompt) {
            next = prompt[step + 1]; /* :354-355 */
        } else {
            next = (int)l2c_argmax(m->logits, m->c.vocab_size); /* :360 */
            out[produced++] = next;
        }
        token = next; /* :385 */
    }
    if (last_logits) memcpy(last_logits, m->logits, (size_t)m->c.vocab_size * 4);
    return produced;
}

const float *l2c_model_logits(l2c_model *m) { return m->logits; }
