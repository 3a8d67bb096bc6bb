// Batched prompt pass ("prefill"): the same layer sequence as transformer! (reference
// src/inference.jl:222-315) applied to M positions at once, where the matrix products are dense
// contractions and run on the matrix cores: weights are dequantized tile by tile into LDS as bf16
// (the reference's fp32 dequantization expressions, src/kquants.jl:83-98,213-217,333-343, then one
// rounding to bf16), activations are bf16, accumulation is fp32 (v_mfma_f32_32x32x16_bf16).
// The reference has no batched path; the result is defined as what its per-token loop would leave
// in the KV cache and the last position's logits, to bf16 accuracy.
#include "matvec_dev.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    bf16x2 v;
    v.x = (__bf16)a;
    v.y = (__bf16)b;
    return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// ------------------------------------------------------------------------------------------
// small per-position kernels
// ------------------------------------------------------------------------------------------
// X[m][:] = dequantized embedding row of tokens[m]  (src/inference.jl:236)
__global__ __launch_bounds__(256) void pf_embed_kernel(DevTensor emb, const int32_t *tokens, float *X, int M) {
    const int m = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= M || i >= emb.ne0) return;
    X[(int64_t)m * emb.ne0 + i] = dequant_elem(emb, tokens[m], i);
}

// cos/sin of the RoPE angles of positions pos0..pos0+M-1: theta_i = fp32(pos) advanced by i fp32
// multiplications (src/inference.jl:122-127), cos/sin in fp64, rounded.  cs[m][i][2].
__global__ __launch_bounds__(64) void pf_rope_table_kernel(float *cs, int pos0, int M, int half, float theta_scale) {
    const int m = blockIdx.x, i = threadIdx.x;
    if (m >= M) return;
    for (int p = i; p < half; p += blockDim.x) {
        float theta = 1.0f * (float)(pos0 + m);
        for (int k = 0; k < p; k++) theta *= theta_scale;
        cs[((int64_t)m * half + p) * 2] = (float)cos((double)theta);
        cs[((int64_t)m * half + p) * 2 + 1] = (float)sin((double)theta);
    }
}

// rmsnorm! of every row (src/inference.jl:102-110), fp64 sum of squares, output rounded to bf16
__global__ __launch_bounds__(256) void pf_rmsnorm_kernel(const float *X, const float *w, uint16_t *out, int64_t K) {
    __shared__ double red[16];
    const float *x = X + (int64_t)blockIdx.x * K;
    __bf16 *o = (__bf16 *)out + (int64_t)blockIdx.x * K;
    if (K % 4 == 0 && K <= 256 * 4 * 8) {  // the row stays in registers: 16 bytes per lane and load, one pass
        float4 v[8];
        double acc = 0.0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int64_t i = 4 * (threadIdx.x + 256 * j);
            v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (i < K) v[j] = *(const float4 *)(x + i);
            acc = fma((double)v[j].x, (double)v[j].x, acc);
            acc = fma((double)v[j].y, (double)v[j].y, acc);
            acc = fma((double)v[j].z, (double)v[j].z, acc);
            acc = fma((double)v[j].w, (double)v[j].w, acc);
        }
        float ss = (float)block_sum_f64(acc, red);
        ss /= (float)K;
        ss += 1e-5f;
        ss = 1.0f / sqrtf(ss);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int64_t i = 4 * (threadIdx.x + 256 * j);
            if (i < K) {
                const float4 g = *(const float4 *)(w + i);
                uint2 pk;
                pk.x = pack_bf16(g.x * (ss * v[j].x), g.y * (ss * v[j].y));
                pk.y = pack_bf16(g.z * (ss * v[j].z), g.w * (ss * v[j].w));
                *(uint2 *)(o + i) = pk;
            }
        }
        return;
    }
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < K; i += blockDim.x) acc = fma((double)x[i], (double)x[i], acc);
    float ss = (float)block_sum_f64(acc, red);
    ss /= (float)K;
    ss += 1e-5f;
    ss = 1.0f / sqrtf(ss);
    for (int64_t i = threadIdx.x; i < K; i += blockDim.x) o[i] = (__bf16)(w[i] * (ss * x[i]));
}

__global__ __launch_bounds__(256) void pf_rope_scatter_kernel(const float *raw, const float *cs, uint16_t *Qb,
                                                              float *kc, float *vc, int M, int pos0, int dim,
                                                              int kv_dim, int hs, int seq_len, int neox) {
    const int m = blockIdx.x;
    if (m >= M) return;
    const float *r = raw + (int64_t)m * (dim + 2 * kv_dim);
    const int half = hs >> 1, pos = pos0 + m;
    // a thread turns 4 consecutive pairs of one head: rotation indices i0 .. i0+3, whose 8 elements are two
    // runs of 4 (interleaved pairs: 2 i0 .. and 2 i0 + 4 ..; half-split pairs: i0 .. and i0 + half ..)
    const int qpH = half >> 2, nquads = ((dim + kv_dim) / hs) * qpH;
    for (int p = threadIdx.x; p < nquads; p += blockDim.x) {
        const int hh = p / qpH, i0 = 4 * (p % qpH);
        const bool is_q = hh < dim / hs;
        const int h = is_q ? hh : hh - dim / hs;
        const float *src = r + (is_q ? 0 : dim) + h * hs;
        const int ea = neox ? i0 : 2 * i0, eb = neox ? i0 + half : 2 * i0 + 4;
        const float4 a = *(const float4 *)(src + ea), b = *(const float4 *)(src + eb);
        const float4 c0 = *(const float4 *)(cs + ((int64_t)m * half + i0) * 2);      // cos, sin of i0, i0+1
        const float4 c1 = *(const float4 *)(cs + ((int64_t)m * half + i0 + 2) * 2);  // ... of i0+2, i0+3
        float4 oa, ob;
        if (neox) {  // pair k = (a[k], b[k])
            oa.x = (a.x * c0.x) - (b.x * c0.y), ob.x = (a.x * c0.y) + (b.x * c0.x);
            oa.y = (a.y * c0.z) - (b.y * c0.w), ob.y = (a.y * c0.w) + (b.y * c0.z);
            oa.z = (a.z * c1.x) - (b.z * c1.y), ob.z = (a.z * c1.y) + (b.z * c1.x);
            oa.w = (a.w * c1.z) - (b.w * c1.w), ob.w = (a.w * c1.w) + (b.w * c1.z);
        } else {  // pairs (a.x, a.y), (a.z, a.w), (b.x, b.y), (b.z, b.w)
            oa.x = (a.x * c0.x) - (a.y * c0.y), oa.y = (a.x * c0.y) + (a.y * c0.x);
            oa.z = (a.z * c0.z) - (a.w * c0.w), oa.w = (a.z * c0.w) + (a.w * c0.z);
            ob.x = (b.x * c1.x) - (b.y * c1.y), ob.y = (b.x * c1.y) + (b.y * c1.x);
            ob.z = (b.z * c1.z) - (b.w * c1.w), ob.w = (b.z * c1.w) + (b.w * c1.z);
        }
        if (is_q) {
            uint16_t *q = Qb + (int64_t)m * dim + h * hs;
            *(uint2 *)(q + ea) = make_uint2(pack_bf16(oa.x, oa.y), pack_bf16(oa.z, oa.w));
            *(uint2 *)(q + eb) = make_uint2(pack_bf16(ob.x, ob.y), pack_bf16(ob.z, ob.w));
        } else {  // kv.key_cache[:, :, pos] = k (src/inference.jl:259), elements in groups of 4 per timestep
            *(float4 *)(kc + (((int64_t)h * (hs >> 2) + (ea >> 2)) * seq_len + pos) * 4) = oa;
            *(float4 *)(kc + (((int64_t)h * (hs >> 2) + (eb >> 2)) * seq_len + pos) * 4) = ob;
        }
    }
    for (int e = 4 * threadIdx.x; e < kv_dim; e += 4 * blockDim.x) {  // kv.value_cache[pos, :, :] = v (:260)
        const int h = e / hs, d = e % hs;
        *(float4 *)(vc + ((int64_t)h * seq_len + pos) * hs + d) = *(const float4 *)(r + dim + kv_dim + e);
    }
}

// ------------------------------------------------------------------------------------------
// dense product  C[m][L] = sum_k act[m][k] * W[L][k]   over logical weight rows L
// ------------------------------------------------------------------------------------------
struct PfGemmArgs {
    DevTensor w[3];
    int nseg;
    int interleave;  // logical row L = (segment L & 1, row L >> 1): w1/w3 pairs for SwiGLU
    int64_t n_rows;  // logical rows
    int64_t K;
    const uint16_t *act;  // bf16 [M][K]
    int M;
    float *out;  // STORE: fp32 [M][ldo] at column out_col0 + L; RESID: out[m][L] += C
    int64_t ldo, out_col0;
    uint16_t *out_bf;  // SWIGLU: bf16 [M][ldb], column L/2
    int64_t ldb;
    const uint16_t *wbf;  // pf_gemm_bf16_kernel: the weights expanded beforehand (pf_expand_kernel's tiles)
};

struct PfRow {
    bool valid;
    int seg;
    int64_t row;
};
__device__ __forceinline__ PfRow pf_row(const PfGemmArgs &a, int64_t L) {
    PfRow r{false, 0, 0};
    if (L >= a.n_rows) return r;
    r.valid = true;
    if (a.interleave) {
        r.seg = (int)(L & 1);
        r.row = L >> 1;
        return r;
    }
    const int64_t n0 = a.w[0].ne1, n1 = a.nseg > 1 ? a.w[1].ne1 : 0;
    if (L < n0) {
        r.seg = 0;
        r.row = L;
    } else if (L < n0 + n1) {
        r.seg = 1;
        r.row = L - n0;
    } else {
        r.seg = 2;
        r.row = L - n0 - n1;
    }
    return r;
}

// raw bytes of 32 consecutive weights of one row (k0 a multiple of 32), and their conversion to bf16
struct PfRaw {
    uint4 hdr, qa, qb, ha, hb;
    uint32_t sc[2];
    uint32_t d;
};

struct PfRowPtr {  // stream pointers of the row a thread dequantizes
    const uint4 *hdr;
    const uint8_t *qs, *qh;
    const uint32_t *sc6;
    const uint16_t *d6;
    const float *f32;
    int64_t nb, ne0;
    bool valid;
};

template <int TYPE>
__device__ __forceinline__ void pf_load_raw(PfRaw &r, const PfRowPtr &p, int64_t row, int64_t k0, int64_t K) {
    if (!p.valid) return;
    const int64_t blk = row * p.nb + (k0 >> 8);
    const int rr = (int)(k0 & 255);
    if (TYPE == L2H_TYPE_Q4_K || TYPE == L2H_TYPE_Q5_K) {
        const int j = rr >> 6;
        r.hdr = p.hdr[blk];
        const uint4 *q = (const uint4 *)(p.qs + blk * 128 + 32 * j);
        r.qa = q[0];
        r.qb = q[1];
        if (TYPE == L2H_TYPE_Q5_K) {
            const uint4 *h = (const uint4 *)(p.qh + blk * 32);
            r.ha = h[0];
            r.hb = h[1];
        }
    } else if (TYPE == L2H_TYPE_Q6_K) {
        const int n = rr >> 7, g = (rr & 127) >> 5;
        const uint4 *q = (const uint4 *)(p.qs + blk * 128 + 64 * n + 32 * (g & 1));
        r.qa = q[0];
        r.qb = q[1];
        const uint4 *h = (const uint4 *)(p.qh + blk * 64 + 32 * n);
        r.ha = h[0];
        r.hb = h[1];
        r.sc[0] = p.sc6[blk * 4 + 2 * n];
        r.sc[1] = p.sc6[blk * 4 + 2 * n + 1];
        r.d = p.d6[blk];
    } else {  // F32: 32 floats kept in the five uint4 + ... (loaded in convert; nothing to stage here)
    }
}

__device__ __forceinline__ uint32_t u4_word(const uint4 &a, const uint4 &b, int w) {  // word w (0..7) of a|b
    switch (w) {
    case 0: return a.x;
    case 1: return a.y;
    case 2: return a.z;
    case 3: return a.w;
    case 4: return b.x;
    case 5: return b.y;
    case 6: return b.z;
    default: return b.w;
    }
}

// out[4] = the 32 weights as bf16 (8 per uint4), in element order
template <int TYPE>
__device__ __forceinline__ void pf_convert(const PfRaw &r, const PfRowPtr &p, int64_t row, int64_t k0, int64_t K,
                                           uint4 out[4]) {
    uint32_t pk[16];
    if (!p.valid) {
#pragma unroll
        for (int i = 0; i < 16; i++) pk[i] = 0;
    } else if (TYPE == L2H_TYPE_Q4_K || TYPE == L2H_TYPE_Q5_K) {
        const int rr = (int)(k0 & 255), s = rr >> 5, hi = s & 1;
        int sc, mn;
        kq_scale_min(r.hdr, s, sc, mn);
        const float d = half_bits_to_float((uint16_t)(r.hdr.x & 0xFFFF));
        const float dmin = half_bits_to_float((uint16_t)(r.hdr.x >> 16));
        const float d1 = d * (float)sc, m1 = dmin * (float)mn;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            uint32_t qw = u4_word(r.qa, r.qb, w);
            qw = hi ? (qw >> 4) & 0x0F0F0F0Fu : qw & 0x0F0F0F0Fu;
            if (TYPE == L2H_TYPE_Q5_K) {
                const uint32_t hw = u4_word(r.ha, r.hb, w);
                qw |= ((hw >> s) & 0x01010101u) << 4;
            }
            const float v0 = d1 * (float)(qw & 0xFF) - m1, v1 = d1 * (float)((qw >> 8) & 0xFF) - m1;
            const float v2 = d1 * (float)((qw >> 16) & 0xFF) - m1, v3 = d1 * (float)(qw >> 24) - m1;
            pk[2 * w] = pack_bf16(v0, v1);
            pk[2 * w + 1] = pack_bf16(v2, v3);
        }
    } else if (TYPE == L2H_TYPE_Q6_K) {
        const int rr = (int)(k0 & 255), g = (rr & 127) >> 5;
        const float d = half_bits_to_float((uint16_t)r.d);
#pragma unroll
        for (int w = 0; w < 8; w++) {
            uint32_t qw = u4_word(r.qa, r.qb, w);
            qw = (g & 2) ? (qw >> 4) & 0x0F0F0F0Fu : qw & 0x0F0F0F0Fu;
            const uint32_t hw = u4_word(r.ha, r.hb, w);
            qw |= ((hw >> (2 * g)) & 0x03030303u) << 4;
            const uint32_t scw = r.sc[w >> 2];  // elements 0..15 -> first scale dword, 16..31 -> second
            const int sc = (int)(int8_t)((scw >> (8 * g)) & 0xFF);
            const float v0 = d * (float)(sc * ((int)(qw & 0xFF) - 32)), v1 = d * (float)(sc * ((int)((qw >> 8) & 0xFF) - 32));
            const float v2 = d * (float)(sc * ((int)((qw >> 16) & 0xFF) - 32)), v3 = d * (float)(sc * ((int)(qw >> 24) - 32));
            pk[2 * w] = pack_bf16(v0, v1);
            pk[2 * w + 1] = pack_bf16(v2, v3);
        }
    } else {
        const float *src = p.f32 + row * p.ne0 + k0;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float v0 = (k0 + 2 * i) < K ? src[2 * i] : 0.0f;
            const float v1 = (k0 + 2 * i + 1) < K ? src[2 * i + 1] : 0.0f;
            pk[i] = pack_bf16(v0, v1);
        }
    }
#pragma unroll
    for (int c = 0; c < 4; c++) out[c] = make_uint4(pk[4 * c], pk[4 * c + 1], pk[4 * c + 2], pk[4 * c + 3]);
}

// Placement of the 16-byte chunks of a 128-byte tile row in LDS.  The LDS has 64 banks of 4 bytes and serves
// 16-byte accesses 16 lanes at a time; lanes read one chunk index of 16 consecutive rows, which the
// exclusive-or with (r >> 1) % 8 sends to the 16 different 16-byte slots of the 256-byte bank row (the row's
// parity picks the half).  With r % 8 instead, rows r and r + 8 collide: half the LDS cycles were conflicts.
__host__ __device__ __forceinline__ int pf_swz(int r) { return (r >> 1) & 7; }

// the stream pointers of logical weight row L
template <int TYPE>
__device__ __forceinline__ void pf_row_ptr(const PfGemmArgs &a, int64_t L, PfRow &lr, PfRowPtr &rp) {
    lr = pf_row(a, L);
    const int sg = lr.seg;
#define PICK(F) (sg == 0 ? a.w[0].F : (sg == 1 ? a.w[1].F : a.w[2].F))
    rp.hdr = PICK(hdr);
    rp.qs = PICK(qs);
    rp.qh = PICK(qh);
    rp.sc6 = PICK(sc6);
    rp.d6 = PICK(d6);
    rp.f32 = PICK(f32);
    rp.nb = PICK(nb);
    rp.ne0 = PICK(ne0);
#undef PICK
    rp.valid = lr.valid;
}

// One thread expands 32 consecutive weights of one logical row to bf16, with the arithmetic the fused
// product kernel uses on them.  The destination is a sequence of 32 KB tiles, tile (nt, kt) = weight
// rows 256 nt.. x inputs 64 kt.. at ((nt K/64) + kt) * 16384 elements, and inside a tile the image the
// product kernel keeps in LDS: the 16-byte chunk c of row r at chunk index 8 r + (c ^ pf_swz(r)).  Logical
// row L goes to row dst_row0 + L; rows from n_rows up to rows_end (padding of the last tile) are zero.
// plain: row R is K values in a row at dst + R K instead (the layout a library product takes).
template <int TYPE>
__global__ __launch_bounds__(256) void pf_expand_kernel(PfGemmArgs a, uint16_t *dst, int64_t dst_row0, int64_t rows_end,
                                                        int plain) {
    const int64_t groups = a.K >> 5, nk = a.K >> 6;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows_end * groups) return;
    const int64_t L = idx / groups, g = idx - L * groups, k0 = 32 * g;
    PfRow lr;
    PfRowPtr rp;
    pf_row_ptr<TYPE>(a, L, lr, rp);
    PfRaw raw;
    pf_load_raw<TYPE>(raw, rp, lr.row, k0, a.K);
    uint4 wv[4];
    pf_convert<TYPE>(raw, rp, lr.row, k0, a.K, wv);
    const int64_t R = dst_row0 + L, nt = R >> 8, kt = g >> 1;
    if (plain) {
        uint4 *row = (uint4 *)(dst + R * a.K + k0);
#pragma unroll
        for (int cc = 0; cc < 4; cc++) row[cc] = wv[cc];
        return;
    }
    const int r = (int)(R & 255);
    uint4 *tile = (uint4 *)(dst + (nt * nk + kt) * 16384);
#pragma unroll
    for (int cc = 0; cc < 4; cc++) {
        const int c = 4 * (int)(g & 1) + cc;
        tile[r * 8 + (c ^ pf_swz(r))] = wv[cc];
    }
}

// Results of one workgroup tile: a lane holds position m0 + 32 JT wm + 32 j + lane%32 and, in register r
// of tile i, logical weight row n0 + 64 wn + 32 i + 8 (r/4) + 4 (lane/32) + r%4.
template <int EPI, int JT>
__device__ __forceinline__ void pf_epilogue(const PfGemmArgs &a, f32x16 (&acc)[2][JT], int64_t n0, int m0, int wn, int wm,
                                            int lane) {
#pragma unroll
    for (int j = 0; j < JT; j++) {
        const int m = m0 + 32 * JT * wm + 32 * j + (lane & 31);
        if (m >= a.M) continue;
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int rq = 0; rq < 4; rq++) {
                const int64_t L = n0 + 64 * wn + 32 * i + 8 * rq + 4 * (lane >> 5);
                if (L >= a.n_rows) continue;
                const float v0 = acc[i][j][4 * rq], v1 = acc[i][j][4 * rq + 1], v2 = acc[i][j][4 * rq + 2],
                            v3 = acc[i][j][4 * rq + 3];
                if (EPI == PF_SWIGLU) {  // (w1 row u, w3 row u) = logical rows (2u, 2u+1), src/inference.jl:295-299
                    const float h0 = swiglu_val(v0, v1), h1 = swiglu_val(v2, v3);
                    uint16_t *o = a.out_bf + (int64_t)m * a.ldb + (L >> 1);
                    if (L + 3 < a.n_rows)
                        *(uint32_t *)o = pack_bf16(h0, h1);  // L/2 is even and ldb is even: aligned
                    else
                        ((__bf16 *)o)[0] = (__bf16)h0;
                } else {
                    float *o = a.out + (int64_t)m * a.ldo + a.out_col0 + L;
                    const float v[4] = {v0, v1, v2, v3};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (L + e >= a.n_rows) break;
                        if (EPI == PF_RESID)
                            o[e] += v[e];  // x .+= ... (src/inference.jl:284,305)
                        else
                            o[e] = v[e];
                    }
                }
            }
        }
    }
}

// Workgroup tile: 128 weight rows x 128 positions, K in steps of 64; 4 wavefronts, each 64 x 64 as
// 2 x 2 tiles of 32 x 32.  Weights are the A operand (rows), positions the B operand (columns), so
// a lane ends up holding one position and groups of 4 consecutive weight rows: neighbours such as a
// w1/w3 pair sit in one lane.  LDS rows are 64 bf16 = 8 chunks of 16 bytes, chunk c of row r kept at
// c ^ pf_swz(r).
template <int TYPE, int EPI, int JT>
__global__ __launch_bounds__(256) void pf_gemm_kernel(PfGemmArgs a) {
    constexpr int MT = 64 * JT;  // positions per workgroup: 2 wavefront columns x JT tiles of 32
    __shared__ uint4 s_w[128 * 8];
    __shared__ uint4 s_x[MT * 8];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wn = wave & 1, wm = wave >> 1;
    const int64_t n0 = (int64_t)blockIdx.y * 128;
    const int m0 = blockIdx.x * MT;
    const int64_t K = a.K;

    // the weight row this thread dequantizes: row t/2 of the tile, elements 32*(t&1).. of each K step
    const int wr = t >> 1, whh = t & 1;
    PfRow lr;
    PfRowPtr rp;
    pf_row_ptr<TYPE>(a, n0 + wr, lr, rp);
    // activations: 2 JT chunks of 16 bytes per thread and K step: position (t>>3) + 32*i, chunk t&7
    constexpr int XL = 2 * JT;
    const int xc = t & 7;
    const uint16_t *xrow[XL];
    bool xvalid[XL];
#pragma unroll
    for (int i = 0; i < XL; i++) {
        const int m = m0 + (t >> 3) + 32 * i;
        xvalid[i] = m < a.M;
        xrow[i] = a.act + (int64_t)(xvalid[i] ? m : 0) * K + 8 * xc;
    }

    f32x16 acc[2][JT];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < JT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    PfRaw raw;
    uint4 xreg[XL];
    auto gload = [&](int64_t k0) {
        if (k0 + 32 * whh < K) pf_load_raw<TYPE>(raw, rp, lr.row, k0 + 32 * whh, K);
#pragma unroll
        for (int i = 0; i < XL; i++) {
            xreg[i] = make_uint4(0, 0, 0, 0);
            if (xvalid[i] && k0 + 8 * xc < K) xreg[i] = *(const uint4 *)(xrow[i] + k0);
        }
    };
    gload(0);
    for (int64_t k0 = 0; k0 < K; k0 += 64) {
        // registers -> LDS
        {
            uint4 wv[4];
            PfRowPtr q = rp;
            q.valid = rp.valid && (k0 + 32 * whh < K);
            pf_convert<TYPE>(raw, q, lr.row, k0 + 32 * whh, K, wv);
#pragma unroll
            for (int c = 0; c < 4; c++) s_w[wr * 8 + ((4 * whh + c) ^ pf_swz(wr))] = wv[c];
#pragma unroll
            for (int i = 0; i < XL; i++) {
                const int r = (t >> 3) + 32 * i;
                s_x[r * 8 + (xc ^ pf_swz(r))] = xreg[i];
            }
        }
        __syncthreads();
        if (k0 + 64 < K) gload(k0 + 64);  // in flight during the products
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const int c = 2 * kk + (lane >> 5);
            bf16x8 A[2], B[JT];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int ra = 64 * wn + 32 * i + (lane & 31);
                A[i] = as_bf16x8(s_w[ra * 8 + (c ^ pf_swz(ra))]);
            }
#pragma unroll
            for (int j = 0; j < JT; j++) {
                const int rb = 32 * JT * wm + 32 * j + (lane & 31);
                B[j] = as_bf16x8(s_x[rb * 8 + (c ^ pf_swz(rb))]);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < JT; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[i], B[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    pf_epilogue<EPI, JT>(a, acc, n0, m0, wn, wm, lane);
}

#define PF_AS1 __attribute__((address_space(1)))
#define PF_AS3 __attribute__((address_space(3)))

// The same product from weights expanded beforehand (pf_expand_kernel): no arithmetic on the operands.
// The tile is 256 weight rows x 64 JT positions (JT = 4: 256 positions, 64 KB fetched per 64 inputs, half
// the bytes per product of a 128 x 128 tile; JT = 2: 128 positions, for matrices with too few rows to give
// every CU a 256 x 256 tile), worked on by 8 wavefronts, 4 row groups x 2 position groups, each 64 rows x
// 32 JT positions.  Both operand tiles of a K step travel from global memory
// straight into LDS (16 bytes per lane and load, a wavefront's load filling 1 KB in lane order): the weight
// tile is a linear copy of its 32 KB image, the position tile gets the c ^ pf_swz(r) placement by the choice
// of the address each lane reads.  Two LDS stages: the loads of step kt + 1 are in flight during the products
// of step kt, one barrier per step.  Workgroups are dealt to the 8 XCDs in turn, so workgroup w takes tile
// (w % 8) * per + w / 8: each XCD works through a contiguous run of tiles, positions fastest, and the
// workgroups that share a weight tile share an L2.
typedef uint32_t pf_u32x4 __attribute__((ext_vector_type(4)));

// the tile (row group nt, position block mt) of one workgroup; s_all: two stages of LDS
template <int EPI, int JT>
__device__ __forceinline__ void pf_gemm_bf16_tile(const PfGemmArgs &a, unsigned nt, unsigned mt, uint4 *s_all) {
    constexpr int MT = 64 * JT;                   // positions per workgroup
    constexpr int STAGE = 32768 + MT * 128;       // bytes: weight tile, then position tile
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), wn = wave & 3, wm = wave >> 2;
    const int64_t n0 = (int64_t)nt * 256;
    const int m0 = (int)mt * MT;
    const int64_t K = a.K, nk = K >> 6;

    // weights: this wavefront copies bytes [4096 wave, +4096) of every tile, 1 KB per load
    const unsigned char *gw = (const unsigned char *)(a.wbf + (int64_t)nt * nk * 16384) + wave * 4096 + lane * 16;
    // positions: load i of this wavefront fills chunks 64 (JT wave + i) + lane: row 8 (JT wave + i) + lane / 8,
    // placed chunk lane % 8 = the data chunk (lane % 8) ^ pf_swz(row)
    const unsigned char *gx[JT];
#pragma unroll
    for (int i = 0; i < JT; i++) {
        const int r = 8 * (JT * wave + i) + (lane >> 3);
        int m = m0 + r;
        m = m < a.M ? m : a.M - 1;  // rows past the end repeat the last one; their results are not stored
        gx[i] = (const unsigned char *)(a.act + (int64_t)m * K + 8 * ((lane & 7) ^ pf_swz(r)));
    }
    // LDS byte offsets of this lane's operands inside a stage: slice kk holds chunk 2 kk + lane / 32 of its rows
    unsigned aw[2][4], ax[JT][4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
        const int c = 2 * kk + (lane >> 5);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int ra = 64 * wn + 32 * i + (lane & 31);
            aw[i][kk] = 16u * (unsigned)(ra * 8 + (c ^ pf_swz(ra)));
        }
#pragma unroll
        for (int j = 0; j < JT; j++) {
            const int rb = 32 * JT * wm + 32 * j + (lane & 31);
            ax[j][kk] = 32768u + 16u * (unsigned)(rb * 8 + (c ^ pf_swz(rb)));
        }
    }
    const unsigned lds0 = (unsigned)(size_t)s_all;

    f32x16 acc[2][JT];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < JT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    auto issue = [&](int stage) {
        unsigned char *lw = (unsigned char *)s_all + stage * STAGE + wave * 4096;
        unsigned char *lx = (unsigned char *)s_all + stage * STAGE + 32768 + wave * (1024 * JT);
        __builtin_amdgcn_global_load_lds((const PF_AS1 void *)gw, (PF_AS3 void *)lw, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const PF_AS1 void *)gw, (PF_AS3 void *)lw, 16, 1024, 0);
        __builtin_amdgcn_global_load_lds((const PF_AS1 void *)gw, (PF_AS3 void *)lw, 16, 2048, 0);
        __builtin_amdgcn_global_load_lds((const PF_AS1 void *)gw, (PF_AS3 void *)lw, 16, 3072, 0);
#pragma unroll
        for (int i = 0; i < JT; i++) {
            __builtin_amdgcn_global_load_lds((const PF_AS1 void *)gx[i], (PF_AS3 void *)(lx + 1024 * i), 16, 0, 0);
            gx[i] += 128;
        }
        gw += 32768;
    };

    // The operands of a 16-wide slice (2 weight groups, JT position groups) are read from LDS one slice ahead
    // of the products that use them, into two register sets used in turn, so that a wavefront's LDS latency
    // lies under its own products.  Reads and waits are asm: the compiler then does not make them wait for the
    // copies in flight into the other stage.  Between a PF_READ and the PF_WAIT that retires it the registers
    // of the set hold nothing yet: the set only appears as an operand of those two statements and of the
    // products after the wait (LDS reads complete in order, so lgkmcnt(2 + JT) retires all but the newest set;
    // the build's asm check walks the generated code for any other touch of such a register).
    pf_u32x4 F0[2 + JT], F1[2 + JT];
#define PF_READ(F, KK)                                                                                            \
    do {                                                                                                          \
        if constexpr (JT == 2)                                                                                    \
            asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %5\n\tds_read_b128 %2, %6\n\tds_read_b128 %3, %7"  \
                         : "=&v"(F[0]), "=&v"(F[1]), "=&v"(F[2]), "=&v"(F[3])                                     \
                         : "v"(sb + aw[0][KK]), "v"(sb + aw[1][KK]), "v"(sb + ax[0][KK]), "v"(sb + ax[1][KK])     \
                         : "memory");                                                                             \
        else                                                                                                      \
            asm volatile("ds_read_b128 %0, %6\n\tds_read_b128 %1, %7\n\tds_read_b128 %2, %8\n\tds_read_b128 %3, %9"  \
                         "\n\tds_read_b128 %4, %10\n\tds_read_b128 %5, %11"                                       \
                         : "=&v"(F[0]), "=&v"(F[1]), "=&v"(F[2]), "=&v"(F[3]), "=&v"(F[4]), "=&v"(F[5])           \
                         : "v"(sb + aw[0][KK]), "v"(sb + aw[1][KK]), "v"(sb + ax[0][KK]), "v"(sb + ax[1][KK]),    \
                           "v"(sb + ax[JT - 2][KK]), "v"(sb + ax[JT - 1][KK])                                     \
                         : "memory");                                                                             \
    } while (0)
    // LAST: nothing newer is in flight
#define PF_WAIT(F, LAST)                                                                                          \
    do {                                                                                                          \
        if constexpr (JT == 2) {                                                                                  \
            if (LAST)                                                                                             \
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(F[0]), "+v"(F[1]), "+v"(F[2]), "+v"(F[3])::"memory");  \
            else                                                                                                  \
                asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(F[0]), "+v"(F[1]), "+v"(F[2]), "+v"(F[3])::"memory");  \
        } else {                                                                                                  \
            if (LAST)                                                                                             \
                asm volatile("s_waitcnt lgkmcnt(0)"                                                               \
                             : "+v"(F[0]), "+v"(F[1]), "+v"(F[2]), "+v"(F[3]), "+v"(F[JT]), "+v"(F[JT + 1])::"memory"); \
            else                                                                                                  \
                asm volatile("s_waitcnt lgkmcnt(6)"                                                               \
                             : "+v"(F[0]), "+v"(F[1]), "+v"(F[2]), "+v"(F[3]), "+v"(F[JT]), "+v"(F[JT + 1])::"memory"); \
        }                                                                                                         \
    } while (0)
#define PF_PRODUCTS(F)                                                                                            \
    do {                                                                                                          \
        const bf16x8 W0 = __builtin_bit_cast(bf16x8, F[0]), W1 = __builtin_bit_cast(bf16x8, F[1]);                \
        _Pragma("unroll") for (int j = 0; j < JT; j++) {                                                          \
            const bf16x8 P = __builtin_bit_cast(bf16x8, F[2 + j]);                                                \
            acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(W0, P, acc[0][j], 0, 0, 0);                       \
            acc[1][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(W1, P, acc[1][j], 0, 0, 0);                       \
        }                                                                                                         \
    } while (0)

    issue(0);
    for (int64_t kt = 0; kt < nk; kt++) {
        const int stage = (int)(kt & 1);
        // this wavefront's loads of the stage have landed; the barrier says the same of the others' and that
        // everyone is done reading the other stage (its last PF_WAIT retired every read), which the next loads
        // then overwrite
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        if (kt + 1 < nk) issue(stage ^ 1);
        const unsigned sb = lds0 + (unsigned)(stage * STAGE);
        PF_READ(F0, 0);
        PF_READ(F1, 1);
        PF_WAIT(F0, false);
        PF_PRODUCTS(F0);
        PF_READ(F0, 2);
        PF_WAIT(F1, false);
        PF_PRODUCTS(F1);
        PF_READ(F1, 3);
        PF_WAIT(F0, false);
        PF_PRODUCTS(F0);
        PF_WAIT(F1, true);
        PF_PRODUCTS(F1);
    }
#undef PF_PRODUCTS
#undef PF_WAIT
#undef PF_READ
    pf_epilogue<EPI, JT>(a, acc, n0, m0, wn, wm, lane);
}

// row groups nt0 .. in tiles of 64 JT positions
template <int EPI, int JT>
__global__ __launch_bounds__(512) void pf_gemm_bf16_kernel(PfGemmArgs a, unsigned nt0, unsigned n_mt, unsigned n_tiles,
                                                           unsigned per) {
    extern __shared__ uint4 s_all[];
    const unsigned tile = (blockIdx.x & 7u) * per + (blockIdx.x >> 3);
    if (tile >= n_tiles) return;
    pf_gemm_bf16_tile<EPI, JT>(a, nt0 + tile / n_mt, tile % n_mt, s_all);
}

// One round of the CUs over a matrix that would need between one and two rounds of 256 x 128 tiles: the
// first nt4 row groups in 256 x 256 tiles, the others in 256 x 128 tiles, sized by the caller so that every
// CU gets one workgroup (each XCD takes per4 of the large and then per2 of the small tiles, again as
// contiguous runs, positions fastest).
template <int EPI>
__global__ __launch_bounds__(512) void pf_gemm_bf16_mixed_kernel(PfGemmArgs a, unsigned nt4, unsigned n_mt4, unsigned n_mt2,
                                                                 unsigned n_tiles4, unsigned n_tiles2, unsigned per4,
                                                                 unsigned per2) {
    extern __shared__ uint4 s_all[];
    const unsigned xcd = blockIdx.x & 7u, k = blockIdx.x >> 3;
    if (k < per4) {
        const unsigned tile = xcd * per4 + k;
        if (tile >= n_tiles4) return;
        pf_gemm_bf16_tile<EPI, 4>(a, tile / n_mt4, tile % n_mt4, s_all);
    } else {
        const unsigned tile = xcd * per2 + (k - per4);
        if (tile >= n_tiles2) return;
        pf_gemm_bf16_tile<EPI, 2>(a, nt4 + tile / n_mt2, tile % n_mt2, s_all);
    }
}

// ------------------------------------------------------------------------------------------
// causal attention over a block of positions (src/inference.jl:263-278 for each of them):
// one workgroup = one head x 128 query positions (32 per wavefront), keys in tiles of 32.
//   S^T = K_tile Q^T          A = K rows (keys), B = Q columns (queries)
//   running max / sum per query (a lane holds one query: 16 of the 32 keys, the lane 32 further the rest)
//   O^T += V_tile^T P^T       A = V^T rows (head dims), B = P^T columns (queries)
// The k index of the second product is a permutation of the keys chosen so that the lane's own
// probabilities are its B operand without any exchange; V^T is kept in that key order.
//
// The fp32 cache is first rewritten, once per layer, as bf16 tiles that are the very bytes the attention
// workgroups want in LDS (pf_kv_tiles_kernel): per KV head and 32 keys, the K rows (key-major, 16 bytes of
// padding per row to spread the banks) followed by V^T (head-dim-major, keys permuted, padded rows).  The 64
// workgroups that need a tile (4 heads of the group x 16 query blocks) then only copy it.
// ------------------------------------------------------------------------------------------
template <int HS>
struct PfKvTile {
    static constexpr int KROW = HS * 2 + 16;  // bytes per key row
    static constexpr int VROW = 80;           // bytes per head-dim row of V^T: 32 keys + 16 bytes of padding
    static constexpr int K_BYTES = 32 * KROW, V_BYTES = HS * VROW;
    static constexpr int BYTES = (K_BYTES + V_BYTES + 1023) / 1024 * 1024;  // copied 1 KB at a time
};

template <int HS>
__global__ __launch_bounds__(256) void pf_kv_tiles_kernel(const float *kc, const float *vc, unsigned char *tiles,
                                                          int seq_len, int n_tiles_max) {
    typedef PfKvTile<HS> T;
    __shared__ __align__(16) unsigned char s_img[T::BYTES];
    unsigned char *s_k = s_img, *s_v = s_img + T::K_BYTES;
    const int t = threadIdx.x, kt = blockIdx.x, kvh = blockIdx.y, key0 = 32 * kt;
    for (int c = t; c < T::BYTES / 16; c += 256) ((uint4 *)s_img)[c] = make_uint4(0, 0, 0, 0);
    __syncthreads();
    for (int idx = t; idx < 32 * (HS / 4); idx += 256) {  // K tile -> bf16 rows
        const int key = idx & 31, i4 = idx >> 5;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (key0 + key < seq_len) v = *(const float4 *)(kc + (((int64_t)kvh * (HS / 4) + i4) * seq_len + key0 + key) * 4);
        uint2 w;
        w.x = pack_bf16(v.x, v.y);
        w.y = pack_bf16(v.z, v.w);
        *(uint2 *)(s_k + key * T::KROW + i4 * 8) = w;
    }
    for (int idx = t; idx < 32 * (HS / 4); idx += 256) {  // V tile -> bf16, transposed, keys permuted
        const int d4 = idx % (HS / 4), key = idx / (HS / 4);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (key0 + key < seq_len) v = *(const float4 *)(vc + ((int64_t)kvh * seq_len + key0 + key) * HS + 4 * d4);
        // key = 16 s + 8 a + 4 g + b  ->  slot 16 s + 8 g + 4 a + b
        const int rem = key & 15;
        const int slot = (key & 16) + 8 * ((rem >> 2) & 1) + 4 * (rem >> 3) + (rem & 3);
        __bf16 *dst = (__bf16 *)(s_v + (4 * d4) * T::VROW) + slot;
        dst[0] = (__bf16)v.x;
        dst[T::VROW / 2] = (__bf16)v.y;
        dst[T::VROW] = (__bf16)v.z;
        dst[3 * T::VROW / 2] = (__bf16)v.w;
    }
    __syncthreads();
    uint4 *dst = (uint4 *)(tiles + ((int64_t)kvh * n_tiles_max + kt) * T::BYTES);
    for (int c = t; c < T::BYTES / 16; c += 256) dst[c] = ((const uint4 *)s_img)[c];
}

// N 16-byte LDS reads STRIDE bytes apart, issued and not waited for: until pf_lds_retire has run for `o`
// its registers hold nothing yet and must appear nowhere else (the asm check of the build walks the generated
// code for that).  Being asm, the reads are not made to wait for the tile copies in flight into the other stage.
template <int N, int STRIDE>
__device__ __forceinline__ void pf_lds_issue(pf_u32x4 (&o)[4], unsigned addr) {
    static_assert(N >= 1 && N <= 4 && 3 * STRIDE < 65536, "");
    if constexpr (N == 1)
        asm volatile("ds_read_b128 %0, %1" : "=&v"(o[0]) : "v"(addr) : "memory");
    else if constexpr (N == 2)
        asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:%3"
                     : "=&v"(o[0]), "=&v"(o[1])
                     : "v"(addr), "n"(STRIDE)
                     : "memory");
    else if constexpr (N == 3)
        asm volatile("ds_read_b128 %0, %3\n\tds_read_b128 %1, %3 offset:%4\n\tds_read_b128 %2, %3 offset:%5"
                     : "=&v"(o[0]), "=&v"(o[1]), "=&v"(o[2])
                     : "v"(addr), "n"(STRIDE), "n"(2 * STRIDE)
                     : "memory");
    else
        asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:%5\n\tds_read_b128 %2, %4 offset:%6\n\t"
                     "ds_read_b128 %3, %4 offset:%7"
                     : "=&v"(o[0]), "=&v"(o[1]), "=&v"(o[2]), "=&v"(o[3])
                     : "v"(addr), "n"(STRIDE), "n"(2 * STRIDE), "n"(3 * STRIDE)
                     : "memory");
}
// every LDS read issued so far is complete; from here on `o` holds its values
template <int N>
__device__ __forceinline__ void pf_lds_retire(pf_u32x4 (&o)[4]) {
    if constexpr (N == 1)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(o[0])::"memory");
    else if constexpr (N == 2)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(o[0]), "+v"(o[1])::"memory");
    else if constexpr (N == 3)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2])::"memory");
    else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3])::"memory");
}

// the value of the lane 32 further on (or back): the two halves of the wavefront exchanged in one instruction
__device__ __forceinline__ float pf_other_half(float x) {
    typedef unsigned pf_u32x2 __attribute__((ext_vector_type(2)));
    const pf_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    // r[0] = {low half, low half}, r[1] = {high half, high half}
    return (threadIdx.x & 32) ? __uint_as_float(r[0]) : __uint_as_float(r[1]);
}

template <int HS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void pf_attn_kernel(const uint16_t *Qb, uint16_t *Att, const unsigned char *tiles,
                                                      int n_tiles_max, int M, int qpos0, int n_heads, int n_kv, int dim,
                                                      unsigned n_qb, unsigned n_items, unsigned per) {
    typedef PfKvTile<HS> T;
    constexpr int KSTEPS = HS / 16, DT = HS / 32, KH = KSTEPS / 2;
    // two stages: the copy of tile kt + 1 is in flight during the products of tile kt, one barrier per tile
    __shared__ __align__(16) unsigned char s_t[2 * T::BYTES];
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), g = lane >> 5, ql = lane & 31;
    // Workgroups are dealt to the 8 XCDs in turn: workgroup w takes item (w % 8) * per + w / 8 of the list
    // (head, query block), so an XCD works through a few heads (the heads of a KV group share its L2).  A
    // block's work grows with its index (causal); two workgroups share a CU, the second of them from the
    // later half of the XCD's run, so the heads that start in that half take their query blocks in reverse
    // order and a long block meets a short one.
    const unsigned item = (blockIdx.x & 7u) * per + (blockIdx.x >> 3);
    if (item >= n_items) return;
    const int h = (int)(item / n_qb), u = (int)(item % n_qb);
    const int kvh = h / (n_heads / n_kv);
    const int qb = ((unsigned)h * n_qb) % per >= (per + 1) / 2 ? (int)n_qb - 1 - u : u;
    const int q0 = qb * 128;
    const int myq = q0 + 32 * wave + ql;
    const bool qvalid = myq < M;
    bf16x8 qf[KSTEPS];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; kk++) {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (qvalid) v = *(const uint4 *)(Qb + (int64_t)myq * dim + h * HS + 16 * kk + 8 * g);
        qf[kk] = as_bf16x8(v);
    }
    f32x16 o[DT];
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[d][r] = 0.0f;
    float mrun = -INFINITY, lrun = 0.0f;
    const int wave_qmax = min(M - 1, q0 + 32 * wave + 31), wg_qmax = min(M - 1, q0 + 127);
    const int nkt = (qpos0 + wg_qmax) / 32 + 1;
    const float c_log2 = 1.44269504088896341f / sqrtf((float)HS);
    const unsigned char *src = tiles + (int64_t)kvh * n_tiles_max * T::BYTES + lane * 16;
    const unsigned lds0 = (unsigned)(size_t)s_t;
    const unsigned k_addr = lds0 + (unsigned)(ql * T::KROW + 16 * g), v_addr = lds0 + (unsigned)(T::K_BYTES + ql * T::VROW + 16 * g);
    // this wavefront copies KB wave, wave + 4, ... of a tile, a KB per load (16 bytes per lane, lane order)
    auto issue = [&](int stage, int kt) {
        const unsigned char *gp = src + (int64_t)kt * T::BYTES;
        unsigned char *lp = s_t + stage * T::BYTES;
#pragma unroll
        for (int b = 0; b < T::BYTES / 1024; b += 4)
            if (b + wave < T::BYTES / 1024)
                __builtin_amdgcn_global_load_lds((const PF_AS1 void *)(gp + (b + wave) * 1024),
                                                 (PF_AS3 void *)(lp + (b + wave) * 1024), 16, 0, 0);
    };
    issue(0, 0);
    for (int kt = 0; kt < nkt; kt++) {
        const int key0 = 32 * kt, stage = kt & 1;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's part of the tile has landed
        __syncthreads();                                  // ... and everyone's; the other stage is free
        if (kt + 1 < nkt) issue(stage ^ 1, kt + 1);
        if (key0 > qpos0 + wave_qmax) continue;  // every key of the tile lies in this wavefront's future
        const unsigned so = (unsigned)(stage * T::BYTES);
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.0f;
        {
            pf_u32x4 ka[2][4];
            pf_lds_issue<KH, 32>(ka[0], k_addr + so);
            pf_lds_issue<KH, 32>(ka[1], k_addr + so + (unsigned)(32 * KH));
            pf_lds_retire<KH>(ka[0]);
            pf_lds_retire<KH>(ka[1]);
#pragma unroll
            for (int half = 0; half < 2; half++)
#pragma unroll
                for (int i = 0; i < KH; i++)
                    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[half][i]), qf[KH * half + i], s, 0, 0, 0);
        }
        // the V^T operands of the second product are asked for now and arrive during the softmax arithmetic
        pf_u32x4 va[2][4];
        pf_lds_issue<DT, 32 * T::VROW>(va[0], v_addr + so);
        pf_lds_issue<DT, 32 * T::VROW>(va[1], v_addr + so + 32u);
        // scores in units of log2 e: softmax(s / sqrt(hs)) = 2^(c s - max) / sum with c = log2 e / sqrt(hs)
        // (att ./= sqrt(hs); softmax!, src/inference.jl:268-270); only a tile on the diagonal needs the mask
        float tmax = -INFINITY;
        // (wavefront-uniform: the tile reaches past the first query of the wavefront, or some query is past M)
        const bool diagonal = key0 + 31 > qpos0 + q0 + 32 * wave || q0 + 32 * wave + 31 >= M;
        if (diagonal) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = key0 + 8 * (r >> 2) + 4 * g + (r & 3);
                float v = s[r] * c_log2;
                if (!qvalid || key > qpos0 + myq) v = -INFINITY;
                s[r] = v;
                tmax = fmaxf(tmax, v);
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                s[r] *= c_log2;
                tmax = fmaxf(tmax, s[r]);
            }
        }
        tmax = fmaxf(tmax, pf_other_half(tmax));
        // The reference point of a query's exponents (mrun) follows its maximum only when the maximum has grown
        // by more than 8 (a factor 256) since the reference was set, or when there was none: terms stay below
        // 2^8, far inside fp32 and bf16 range, and the sums are rescaled on few tiles instead of on most (some
        // query of the 64 in a wavefront meets a new maximum in nearly every tile).  The quotient sum / total at
        // the end is the same softmax.
        const bool move = tmax > mrun + 8.0f || (mrun == -INFINITY && tmax != -INFINITY);
        if (__any(move)) {
            const float mnew = fmaxf(mrun, tmax);
            const float alpha = (mnew == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(mrun - mnew);
            lrun *= alpha;
            mrun = mnew;
#pragma unroll
            for (int d = 0; d < DT; d++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[d][r] *= alpha;
        }
        const float msub = (mrun == -INFINITY) ? 0.0f : mrun;  // a row with nothing visible yet: all terms 0
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float pv = __builtin_amdgcn_exp2f(s[r] - msub);
            s[r] = pv;
            psum += pv;
        }
        psum += pf_other_half(psum);
        lrun += psum;
        pf_lds_retire<DT>(va[0]);
        pf_lds_retire<DT>(va[1]);
#pragma unroll
        for (int st = 0; st < 2; st++) {
            const uint4 pb = make_uint4(pack_bf16(s[8 * st], s[8 * st + 1]), pack_bf16(s[8 * st + 2], s[8 * st + 3]),
                                        pack_bf16(s[8 * st + 4], s[8 * st + 5]), pack_bf16(s[8 * st + 6], s[8 * st + 7]));
            const bf16x8 B = as_bf16x8(pb);
#pragma unroll
            for (int d = 0; d < DT; d++)
                o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, va[st][d]), B, o[d], 0, 0, 0);
        }
    }
    if (!qvalid) return;
    const float inv = 1.0f / lrun;
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
            const int e = 32 * d + 8 * rq + 4 * g;
            uint2 w;
            w.x = pack_bf16(o[d][4 * rq] * inv, o[d][4 * rq + 1] * inv);
            w.y = pack_bf16(o[d][4 * rq + 2] * inv, o[d][4 * rq + 3] * inv);
            *(uint2 *)(Att + (int64_t)myq * dim + h * HS + e) = w;
        }
}

// ------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------
hipError_t k_pf_embed(hipStream_t s, const DevTensor &emb, const int32_t *tokens, float *X, int M) {
    hipLaunchKernelGGL(pf_embed_kernel, dim3((unsigned)((emb.ne0 + 255) / 256), (unsigned)M), dim3(256), 0, s, emb,
                       tokens, X, M);
    return hipGetLastError();
}
hipError_t k_pf_rope_table(hipStream_t s, float *cs, int pos0, int M, int half, float theta_scale) {
    hipLaunchKernelGGL(pf_rope_table_kernel, dim3((unsigned)M), dim3(64), 0, s, cs, pos0, M, half, theta_scale);
    return hipGetLastError();
}
hipError_t k_pf_rmsnorm(hipStream_t s, const float *X, const float *w, uint16_t *out, int M, int64_t K) {
    hipLaunchKernelGGL(pf_rmsnorm_kernel, dim3((unsigned)M), dim3(256), 0, s, X, w, out, K);
    return hipGetLastError();
}
hipError_t k_pf_rope_scatter(hipStream_t s, const float *raw, const float *cs, uint16_t *Qb, float *kc, float *vc, int M,
                             int pos0, int dim, int kv_dim, int hs, int seq_len, int neox) {
    hipLaunchKernelGGL(pf_rope_scatter_kernel, dim3((unsigned)M), dim3(256), 0, s, raw, cs, Qb, kc, vc, M, pos0, dim,
                       kv_dim, hs, seq_len, neox);
    return hipGetLastError();
}

// JT tiles of 32 positions per wavefront column: 64 JT positions per workgroup
template <int TYPE, int JT>
static hipError_t pf_gemm_type(hipStream_t s, const PfGemmArgs &a, int epi, int64_t rows) {
    const dim3 grid((unsigned)((a.M + 64 * JT - 1) / (64 * JT)), (unsigned)((rows + 127) / 128));
    switch (epi) {
    case PF_STORE: hipLaunchKernelGGL((pf_gemm_kernel<TYPE, PF_STORE, JT>), grid, dim3(256), 0, s, a); break;
    case PF_RESID: hipLaunchKernelGGL((pf_gemm_kernel<TYPE, PF_RESID, JT>), grid, dim3(256), 0, s, a); break;
    case PF_SWIGLU: hipLaunchKernelGGL((pf_gemm_kernel<TYPE, PF_SWIGLU, JT>), grid, dim3(256), 0, s, a); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

static hipError_t pf_weight_args(PfGemmArgs &a, const DevTensor *w, int nseg, int interleave, int64_t K) {
    int64_t rows = 0;
    if (nseg < 1 || nseg > 3) return hipErrorInvalidValue;
    for (int i = 0; i < nseg; i++) {
        if (w[i].type != w[0].type || w[i].ne0 != K) return hipErrorInvalidValue;
        a.w[i] = w[i];
        rows += w[i].ne1;
    }
    if (interleave && (nseg != 2 || w[0].ne1 != w[1].ne1)) return hipErrorInvalidValue;
    a.nseg = nseg;
    a.interleave = interleave;
    a.n_rows = rows;
    a.K = K;
    return hipSuccess;
}

#define PF_MAX_DEVICES 64

// w: nseg tensors of one type sharing the input, or (wbf != nullptr) n_rows_bf rows expanded by
// k_pf_expand; see PfGemmArgs for the outputs
hipError_t k_pf_gemm(hipStream_t s, const DevTensor *w, int nseg, int interleave, const uint16_t *wbf, int64_t n_rows_bf,
                     const uint16_t *act, int M, int64_t K, int epi, float *out, int64_t ldo, int64_t out_col0,
                     uint16_t *out_bf, int64_t ldb) {
    PfGemmArgs a{};
    if (wbf) {
        if (K % 64 != 0) return hipErrorInvalidValue;
        a.n_rows = n_rows_bf;
        a.K = K;
        a.wbf = wbf;
    } else {
        const hipError_t e = pf_weight_args(a, w, nseg, interleave, K);
        if (e != hipSuccess) return e;
    }
    if (K % 8 != 0 || M < 1) return hipErrorInvalidValue;
    const int64_t rows = a.n_rows;
    a.act = act;
    a.M = M;
    a.out = out;
    a.ldo = ldo;
    a.out_col0 = out_col0;
    a.out_bf = out_bf;
    a.ldb = ldb;
    if (wbf) {
        int dev = 0;
        {
            const hipError_t e = hipGetDevice(&dev);
            if (e != hipSuccess) return e;
            if (dev < 0 || dev >= PF_MAX_DEVICES) return hipErrorInvalidDevice;
        }
        // 256 x 256 tiles (JT = 4) for as many row groups as fill whole rounds of the 256 CUs; what is left, or
        // a matrix too small for one such round, goes in 256 x 128 tiles (JT = 2), which spread it over twice
        // as many workgroups
        const unsigned n_nt = (unsigned)((rows + 255) / 256), n_mt4 = (unsigned)((M + 255) / 256);
        const unsigned nt4 = (n_nt * n_mt4 / 256) * 256 / n_mt4;  // row groups in whole rounds of 256 x 256 tiles
        auto launch = [&](int jt, unsigned nt0, unsigned nnt) -> hipError_t {
            const unsigned n_mt = (unsigned)((M + 64 * jt - 1) / (64 * jt)), n_tiles = n_mt * nnt;
            const unsigned per = (n_tiles + 7) / 8;
            const dim3 grid(8 * per);
            const size_t lds = 2 * (size_t)(32768 + 64 * jt * 128);
#define GO(E, J)                                                                                              \
    do {                                                                                                      \
        static bool attr_set[PF_MAX_DEVICES] = {}; /* the attribute is kept per device */                     \
        if (!attr_set[dev]) {                                                                                 \
            const hipError_t e = hipFuncSetAttribute((const void *)pf_gemm_bf16_kernel<E, J>,                 \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);   \
            if (e != hipSuccess) return e;                                                                    \
            attr_set[dev] = true;                                                                             \
        }                                                                                                     \
        hipLaunchKernelGGL((pf_gemm_bf16_kernel<E, J>), grid, dim3(512), lds, s, a, nt0, n_mt, n_tiles, per); \
    } while (0)
            if (jt == 4) {
                switch (epi) {
                case PF_STORE: GO(PF_STORE, 4); break;
                case PF_RESID: GO(PF_RESID, 4); break;
                case PF_SWIGLU: GO(PF_SWIGLU, 4); break;
                default: return hipErrorInvalidValue;
                }
            } else {
                switch (epi) {
                case PF_STORE: GO(PF_STORE, 2); break;
                case PF_RESID: GO(PF_RESID, 2); break;
                case PF_SWIGLU: GO(PF_SWIGLU, 2); break;
                default: return hipErrorInvalidValue;
                }
            }
#undef GO
            return hipGetLastError();
        };
        const unsigned n_mt2 = (unsigned)((M + 127) / 128);
        if (nt4 == 0 && n_nt * n_mt2 > 256 && n_mt2 > n_mt4) {
            // more than one round of 256 x 128 tiles, less than one of 256 x 256: mix the two so that the work
            // fits one round, na row groups in large tiles
            const unsigned na = (n_nt * n_mt2 - 256 + (n_mt2 - n_mt4) - 1) / (n_mt2 - n_mt4);
            if (na <= n_nt) {
                const unsigned t4 = na * n_mt4, t2 = (n_nt - na) * n_mt2, per4 = (t4 + 7) / 8, per2 = (t2 + 7) / 8;
                const dim3 grid(8 * (per4 + per2));
                const size_t lds = 2 * (size_t)(32768 + 256 * 128);
#define GO(E)                                                                                                       \
    do {                                                                                                            \
        static bool attr_set[PF_MAX_DEVICES] = {};                                                                  \
        if (!attr_set[dev]) {                                                                                       \
            const hipError_t e = hipFuncSetAttribute((const void *)pf_gemm_bf16_mixed_kernel<E>,                    \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);         \
            if (e != hipSuccess) return e;                                                                          \
            attr_set[dev] = true;                                                                                   \
        }                                                                                                           \
        hipLaunchKernelGGL((pf_gemm_bf16_mixed_kernel<E>), grid, dim3(512), lds, s, a, na, n_mt4, n_mt2, t4, t2, per4, per2); \
    } while (0)
                switch (epi) {
                case PF_STORE: GO(PF_STORE); break;
                case PF_RESID: GO(PF_RESID); break;
                case PF_SWIGLU: GO(PF_SWIGLU); break;
                default: return hipErrorInvalidValue;
                }
#undef GO
                return hipGetLastError();
            }
        }
        if (nt4 > 0) {
            const hipError_t e = launch(4, 0, nt4);
            if (e != hipSuccess) return e;
        }
        return nt4 < n_nt ? launch(2, nt4, n_nt - nt4) : hipSuccess;
    }
    // (a 256-position tile, JT = 4, was measured slower: its 272 registers leave one wavefront per SIMD)
    switch (w[0].type) {
    case L2H_TYPE_Q4_K: return pf_gemm_type<L2H_TYPE_Q4_K, 2>(s, a, epi, rows);
    case L2H_TYPE_Q5_K: return pf_gemm_type<L2H_TYPE_Q5_K, 2>(s, a, epi, rows);
    case L2H_TYPE_Q6_K: return pf_gemm_type<L2H_TYPE_Q6_K, 2>(s, a, epi, rows);
    case L2H_TYPE_F32: return pf_gemm_type<L2H_TYPE_F32, 2>(s, a, epi, rows);
    }
    return hipErrorInvalidValue;
}

// Expands the rows of the nseg tensors (one after another, or w1/w3 rows in turn when interleave is set) to
// bf16 into the tiled matrix dst (see pf_expand_kernel) from row dst_row0 on; with pad the rows up to the
// next multiple of 256 are zeroed.  K a multiple of 64.
hipError_t k_pf_expand(hipStream_t s, const DevTensor *w, int nseg, int interleave, int64_t K, uint16_t *dst,
                       int64_t dst_row0, int pad, int plain) {
    PfGemmArgs a{};
    const hipError_t e = pf_weight_args(a, w, nseg, interleave, K);
    if (e != hipSuccess) return e;
    if (K % 64 != 0) return hipErrorInvalidValue;
    int64_t rows_end = a.n_rows;
    if (pad) rows_end = (dst_row0 + a.n_rows + 255) / 256 * 256 - dst_row0;
    const int64_t n = rows_end * (K >> 5);
    const dim3 grid((unsigned)((n + 255) / 256));
#define GO(T) hipLaunchKernelGGL((pf_expand_kernel<T>), grid, dim3(256), 0, s, a, dst, dst_row0, rows_end, plain)
    switch (w[0].type) {
    case L2H_TYPE_Q4_K: GO(L2H_TYPE_Q4_K); break;
    case L2H_TYPE_Q5_K: GO(L2H_TYPE_Q5_K); break;
    case L2H_TYPE_Q6_K: GO(L2H_TYPE_Q6_K); break;
    case L2H_TYPE_F32: GO(L2H_TYPE_F32); break;
    default: return hipErrorInvalidValue;
    }
#undef GO
    return hipGetLastError();
}

bool k_pf_attention_supported(int hs) { return hs == 32 || hs == 64 || hs == 96 || hs == 128; }

int64_t k_pf_kv_tile_bytes(int hs) {
    switch (hs) {
    case 32: return PfKvTile<32>::BYTES;
    case 64: return PfKvTile<64>::BYTES;
    case 96: return PfKvTile<96>::BYTES;
    case 128: return PfKvTile<128>::BYTES;
    }
    return 0;
}

// tiles: n_kv x n_tiles_max tiles of k_pf_kv_tile_bytes(hs); the first n_tiles of every KV head are rewritten
hipError_t k_pf_kv_tiles(hipStream_t s, const float *kc, const float *vc, unsigned char *tiles, int n_tiles,
                         int n_tiles_max, int hs, int n_kv, int seq_len) {
    if (n_tiles < 1 || n_tiles > n_tiles_max) return hipErrorInvalidValue;
    const dim3 grid((unsigned)n_tiles, (unsigned)n_kv);
#define GO(HS) hipLaunchKernelGGL((pf_kv_tiles_kernel<HS>), grid, dim3(256), 0, s, kc, vc, tiles, seq_len, n_tiles_max)
    switch (hs) {
    case 32: GO(32); break;
    case 64: GO(64); break;
    case 96: GO(96); break;
    case 128: GO(128); break;
    default: return hipErrorInvalidValue;
    }
#undef GO
    return hipGetLastError();
}

// tiles must hold the keys 0 .. qpos0 + M - 1 (k_pf_kv_tiles)
hipError_t k_pf_attention(hipStream_t s, const uint16_t *Qb, uint16_t *Att, const unsigned char *tiles, int n_tiles_max,
                          int M, int qpos0, int hs, int n_heads, int n_kv, int dim) {
    if ((qpos0 + M + 31) / 32 > n_tiles_max) return hipErrorInvalidValue;
    const unsigned n_qb = (unsigned)((M + 127) / 128), n_items = n_qb * (unsigned)n_heads, per = (n_items + 7) / 8;
    const dim3 grid(8 * per);
#define GO(HS) \
    hipLaunchKernelGGL((pf_attn_kernel<HS>), grid, dim3(256), 0, s, Qb, Att, tiles, n_tiles_max, M, qpos0, n_heads, n_kv, dim, n_qb, n_items, per)
    switch (hs) {
    case 32: GO(32); break;
    case 64: GO(64); break;
    case 96: GO(96); break;
    case 128: GO(128); break;
    default: return hipErrorInvalidValue;
    }
#undef GO
    return hipGetLastError();
}
