// Host-side synthetic-weight factory: a counter-based normal generator and fp32 -> k-quant
// encoders.  The reference (Llama2.jl) only decodes k-quants (src/kquants.jl dequantize!);
// these encoders emit GGUF super-blocks in the llama.cpp block structure that those decoders
// read back.  They search no scales (min/max per sub-block only), so they are fast enough to
// quantize billions of weights on the host cores for each benchmark run.
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <thread>
#include <vector>

#include "l2h.h"

namespace {

inline uint64_t mix64(uint64_t z) {  // splitmix64 finaliser
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline void normal_pair(uint64_t seed, uint64_t stream, uint64_t pair, float &z0, float &z1) {
    const uint64_t key = mix64(seed ^ mix64(stream * 0xD1342543DE82EF95ull + 1));
    const uint64_t a = mix64(key ^ (2 * pair));
    const uint64_t b = mix64(key ^ (2 * pair + 1));
    // u1 in (0,1], u2 in [0,1)
    const double u1 = ((double)(a >> 11) + 1.0) * (1.0 / 9007199254740992.0);
    const double u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);
    const double r = sqrt(-2.0 * log(u1));
    const double th = 6.283185307179586476925 * u2;
    z0 = (float)(r * cos(th));
    z1 = (float)(r * sin(th));
}

template <class F>
void parallel_for(int64_t n, int nthreads, F f) {
    nthreads = std::max(1, nthreads);
    if (nthreads == 1 || n < 2 * nthreads) {
        f(0, n);
        return;
    }
    std::vector<std::thread> th;
    const int64_t per = (n + nthreads - 1) / nthreads;
    for (int t = 0; t < nthreads; t++) {
        const int64_t lo = t * per, hi = std::min<int64_t>(n, lo + per);
        if (lo >= hi) break;
        th.emplace_back([=] { f(lo, hi); });
    }
    for (auto &t : th) t.join();
}

uint16_t fp32_to_fp16(float f) {  // round to nearest even
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (x > 0x7F800000u ? 0x200u : 0));
    if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);  // rounds to inf
    if (x < 0x33000001u) return (uint16_t)sign;               // rounds to zero
    int exp = (int)(x >> 23) - 127;
    uint32_t man = (x & 0x7FFFFFu) | 0x800000u;
    int shift;
    if (exp < -14) {  // subnormal half
        shift = 13 + (-14 - exp);
        exp = -15;
    } else {
        shift = 13;
    }
    uint32_t half_man = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (half_man & 1))) half_man++;
    // half_man includes the implicit bit for normals; adding it to the exponent field carries correctly
    uint32_t out = (exp == -15) ? half_man : (((uint32_t)(exp + 15) << 10) + (half_man - 0x400u));
    return (uint16_t)(sign | out);
}

float fp16_to_fp32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1F, man = h & 0x3FF, bits;
    if (exp == 0) {
        if (man == 0)
            bits = sign;
        else {
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FF) << 13);
        }
    } else if (exp == 31)
        bits = sign | 0x7F800000u | (man << 13);
    else
        bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

inline int nearest_int(float v) { return (int)lrintf(v); }

// scales/mins of 8 sub-blocks -> 6-bit codes in the 12-byte packing (the inverse of the
// unpacking at reference src/kquants.jl:80-81,102-103)
void pack_scales_k4(const uint8_t ls[8], const uint8_t lm[8], uint8_t out[12]) {
    memset(out, 0, 12);
    for (int j = 0; j < 8; j++) {
        if (j < 4) {
            out[j] |= ls[j];
            out[j + 4] |= lm[j];
        } else {
            out[j + 4] = (uint8_t)((ls[j] & 0xF) | ((lm[j] & 0xF) << 4));
            out[j - 4] |= (uint8_t)((ls[j] >> 4) << 6);
            out[j] |= (uint8_t)((lm[j] >> 4) << 6);
        }
    }
}

// shared front end of q4_K / q5_K: per-sub-block affine ranges -> codes, d, dmin, integer levels
void encode_k45(const float *x, int nmax, uint16_t &d16, uint16_t &dmin16, uint8_t packed[12], uint8_t L[256]) {
    float scales[8], mins[8];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int s = 0; s < 8; s++) {
        float mn = x[32 * s], mx = x[32 * s];
        for (int l = 1; l < 32; l++) {
            mn = std::min(mn, x[32 * s + l]);
            mx = std::max(mx, x[32 * s + l]);
        }
        if (mn > 0.0f) mn = 0.0f;
        if (mx < mn) mx = mn;
        scales[s] = (mx - mn) / (float)nmax;
        mins[s] = -mn;
        max_scale = std::max(max_scale, scales[s]);
        max_min = std::max(max_min, mins[s]);
    }
    const float inv_scale = max_scale > 0 ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0 ? 63.0f / max_min : 0.0f;
    uint8_t ls[8], lm[8];
    for (int s = 0; s < 8; s++) {
        ls[s] = (uint8_t)std::min(63, std::max(0, nearest_int(inv_scale * scales[s])));
        lm[s] = (uint8_t)std::min(63, std::max(0, nearest_int(inv_min * mins[s])));
    }
    pack_scales_k4(ls, lm, packed);
    d16 = fp32_to_fp16(max_scale / 63.0f);
    dmin16 = fp32_to_fp16(max_min / 63.0f);
    const float d = fp16_to_fp32(d16), dmin = fp16_to_fp32(dmin16);
    for (int s = 0; s < 8; s++) {
        const float dd = d * (float)ls[s], dm = dmin * (float)lm[s];
        for (int l = 0; l < 32; l++) {
            int q = 0;
            if (dd != 0.0f) q = nearest_int((x[32 * s + l] + dm) / dd);
            L[32 * s + l] = (uint8_t)std::min(nmax, std::max(0, q));
        }
    }
}

void quantize_q4_K(const float *x, int64_t nb, uint8_t *out) {
    for (int64_t i = 0; i < nb; i++, x += 256, out += 144) {
        uint16_t d, dmin;
        uint8_t L[256];
        encode_k45(x, 15, d, dmin, out + 4, L);
        memcpy(out, &d, 2);
        memcpy(out + 2, &dmin, 2);
        uint8_t *qs = out + 16;
        for (int j = 0; j < 4; j++)
            for (int l = 0; l < 32; l++) qs[32 * j + l] = (uint8_t)(L[64 * j + l] | (L[64 * j + 32 + l] << 4));
    }
}

void quantize_q5_K(const float *x, int64_t nb, uint8_t *out) {
    for (int64_t i = 0; i < nb; i++, x += 256, out += 176) {
        uint16_t d, dmin;
        uint8_t L[256];
        encode_k45(x, 31, d, dmin, out + 4, L);
        memcpy(out, &d, 2);
        memcpy(out + 2, &dmin, 2);
        uint8_t *qh = out + 16, *qs = out + 48;
        memset(qh, 0, 32);
        for (int j = 0; j < 4; j++)
            for (int l = 0; l < 32; l++) {
                const int a = L[64 * j + l], b = L[64 * j + 32 + l];
                qs[32 * j + l] = (uint8_t)((a & 0xF) | ((b & 0xF) << 4));
                if (a > 15) qh[l] |= (uint8_t)(1u << (2 * j));
                if (b > 15) qh[l] |= (uint8_t)(1u << (2 * j + 1));
            }
    }
}

void quantize_q6_K(const float *x, int64_t nb, uint8_t *out) {
    for (int64_t i = 0; i < nb; i++, x += 256, out += 210) {
        float scales[16];
        float max_scale = 0.0f, max_abs_scale = 0.0f;
        for (int g = 0; g < 16; g++) {
            float amax = 0.0f, mx = 0.0f;
            for (int l = 0; l < 16; l++) {
                const float ax = fabsf(x[16 * g + l]);
                if (ax > amax) {
                    amax = ax;
                    mx = x[16 * g + l];
                }
            }
            scales[g] = amax > 0 ? mx / -32.0f : 0.0f;
            if (fabsf(scales[g]) > max_abs_scale) {
                max_abs_scale = fabsf(scales[g]);
                max_scale = scales[g];
            }
        }
        uint8_t *ql = out, *qh = out + 128;
        int8_t *sc = (int8_t *)(out + 192);
        uint16_t d16 = 0;
        if (max_abs_scale == 0.0f) {
            memset(out, 0, 210);
            // all-zero block: q = 32 decodes to 0
            memset(ql, 0, 128);
            memset(qh, 0xAA, 64);
            memcpy(out + 208, &d16, 2);
            continue;
        }
        const float iscale = -128.0f / max_scale;
        d16 = fp32_to_fp16(1.0f / iscale);
        const float d = fp16_to_fp32(d16);
        uint8_t L[256];
        for (int g = 0; g < 16; g++) {
            sc[g] = (int8_t)std::min(127, nearest_int(iscale * scales[g]));
            const float dd = d * (float)sc[g];
            for (int l = 0; l < 16; l++) {
                int q = 0;
                if (dd != 0.0f) q = nearest_int(x[16 * g + l] / dd);
                q = std::min(31, std::max(-32, q));
                L[16 * g + l] = (uint8_t)(q + 32);
            }
        }
        for (int n = 0; n < 2; n++)
            for (int l = 0; l < 32; l++) {
                const uint8_t q1 = L[128 * n + l], q2 = L[128 * n + l + 32], q3 = L[128 * n + l + 64],
                              q4 = L[128 * n + l + 96];
                ql[64 * n + l] = (uint8_t)((q1 & 0xF) | ((q3 & 0xF) << 4));
                ql[64 * n + l + 32] = (uint8_t)((q2 & 0xF) | ((q4 & 0xF) << 4));
                qh[32 * n + l] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
            }
        memcpy(out + 208, &d16, 2);
    }
}

}  // namespace

extern "C" int l2h_synth_normal(uint64_t seed, uint64_t stream, int64_t offset, int64_t n, float sigma, float *out,
                                int nthreads) {
    if (n < 0 || offset < 0 || !out) return L2H_EINVAL;
    parallel_for(n, nthreads, [=](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi;) {
            const uint64_t g = (uint64_t)(offset + i);
            float z0, z1;
            normal_pair(seed, stream, g >> 1, z0, z1);
            if (g & 1) {
                out[i++] = sigma * z1;
            } else {
                out[i++] = sigma * z0;
                if (i < hi) out[i++] = sigma * z1;
            }
        }
    });
    return L2H_OK;
}

extern "C" int l2h_quantize_weights(int ggml_type, const float *x, int64_t n, void *out_blocks, int nthreads) {
    if (n < 0 || n % 256 != 0 || !x || !out_blocks) return L2H_EINVAL;
    const int64_t nb = n / 256;
    uint8_t *out = (uint8_t *)out_blocks;
    switch (ggml_type) {
    case L2H_TYPE_Q4_K:
        parallel_for(nb, nthreads, [=](int64_t lo, int64_t hi) { quantize_q4_K(x + lo * 256, hi - lo, out + lo * 144); });
        return L2H_OK;
    case L2H_TYPE_Q5_K:
        parallel_for(nb, nthreads, [=](int64_t lo, int64_t hi) { quantize_q5_K(x + lo * 256, hi - lo, out + lo * 176); });
        return L2H_OK;
    case L2H_TYPE_Q6_K:
        parallel_for(nb, nthreads, [=](int64_t lo, int64_t hi) { quantize_q6_K(x + lo * 256, hi - lo, out + lo * 210); });
        return L2H_OK;
    }
    return L2H_ETYPE;
}
