// Device code of the k-quant / fp32 matvec phases, shared by the per-phase kernels and the
// persistent decode kernel.
#pragma once
#include <hip/hip_fp16.h>

#include "dev_common.h"

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 ldg_nt(const uint4 *p) {
    const u32x4 t = __builtin_nontemporal_load((const u32x4 *)p);
    return make_uint4(t.x, t.y, t.z, t.w);
}

typedef float f32x4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ldg_nt_f4(const float4 *p) {
    const f32x4v t = __builtin_nontemporal_load((const f32x4v *)p);
    return make_float4(t.x, t.y, t.z, t.w);
}
// The KV cache holds fp32 elements (the reference's, src/inference.jl:62-65) or, as an option, fp16 ones.  In both a
// lane reads 16 bytes per load: the fp32 K cache is [n_kv][hs/4][seq_len][4], the fp16 one [n_kv][hs/8][seq_len][8]; V is
// [n_kv][seq_len][hs] in both.
struct Half8 {
    float v[8];
};
// 8 consecutive fp16 elements (group g of 16 bytes): the load, and the widening to fp32 (exact).  Separate, so that a
// caller can request several groups before it waits for the first.
typedef unsigned int h8_bits __attribute__((ext_vector_type(4)));
__device__ __forceinline__ h8_bits ldg_nt_h8_bits(const void *base, int64_t g) {
    return __builtin_nontemporal_load((const h8_bits *)base + g);
}
__device__ __forceinline__ Half8 h8_widen(const h8_bits t) {
    Half8 r;
    r.v[0] = half_bits_to_float((uint16_t)(t.x & 0xFFFF));
    r.v[1] = half_bits_to_float((uint16_t)(t.x >> 16));
    r.v[2] = half_bits_to_float((uint16_t)(t.y & 0xFFFF));
    r.v[3] = half_bits_to_float((uint16_t)(t.y >> 16));
    r.v[4] = half_bits_to_float((uint16_t)(t.z & 0xFFFF));
    r.v[5] = half_bits_to_float((uint16_t)(t.z >> 16));
    r.v[6] = half_bits_to_float((uint16_t)(t.w & 0xFFFF));
    r.v[7] = half_bits_to_float((uint16_t)(t.w >> 16));
    return r;
}
__device__ __forceinline__ Half8 ldg_nt_h8(const void *base, int64_t g) { return h8_widen(ldg_nt_h8_bits(base, g)); }
// element i of a cache <- v (fp16: rounded to nearest even)
__device__ __forceinline__ void st_kv(void *base, int64_t i, float v, bool h16) {
    if (h16)
        ((__half *)base)[i] = __float2half_rn(v);
    else
        ((float *)base)[i] = v;
}

// ------------------------------------------------------------------------------------------
// Activations exchanged between workgroups INSIDE one kernel (the persistent decode kernel) are
// written and read with device-scope relaxed atomics: such stores go through to memory and such
// loads do not hit a stale line of another XCD's L2.  COH = false (one kernel per phase) uses
// plain accesses; the kernel boundary orders them.
// ------------------------------------------------------------------------------------------
template <bool COH>
__device__ __forceinline__ float ld_f32(const float *p) {
    if (COH) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}
template <bool COH>
__device__ __forceinline__ float4 ld_f32x4(const float *p) {
    if (COH) {
        const unsigned long long lo =
            __hip_atomic_load((const unsigned long long *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long hi =
            __hip_atomic_load((const unsigned long long *)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return make_float4(__uint_as_float((uint32_t)lo), __uint_as_float((uint32_t)(lo >> 32)),
                           __uint_as_float((uint32_t)hi), __uint_as_float((uint32_t)(hi >> 32)));
    }
    return *(const float4 *)p;
}
template <bool COH>
__device__ __forceinline__ void st_f32(float *p, float v) {
    if (COH)
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *p = v;
}
template <bool COH>
__device__ __forceinline__ void st_f64(double *p, double v) {
    if (COH)
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *p = v;
}

// a*b + c on the 24-bit multiplier (v_mad_i32_i24): a and b must fit 24 bits
__device__ __forceinline__ int mad24(int a, int b, int c) { return __mul24(a, b) + c; }

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// Activations staged in LDS for one workgroup.
struct XLds {
    const int8_t *qs;
    const int16_t *bsums;
    const float *d;
    const float *xf;  // F32 weights: the fp32 input vector
};

// ---- what one lane loads for one chunk of a row ------------------------------------------------
// q4_K: chunk c (0..7) of a block = qs bytes [16c, 16c+16): low nibbles are elements 64j+16h+k of
// sub-block 2j, high nibbles elements 64j+32+16h+k of sub-block 2j+1 (j = c>>1, h = c&1;
// reference src/kquants.jl:92-98).
// q5_K: as q4_K plus bit 2j / 2j+1 of qh[16h+k] (src/kquants.jl:213,217,220-221).
// q6_K: chunk c (0..3) = ql bytes [64n+16h,+16) and [64n+32+16h,+16) with qh bytes [32n+16h,+16),
// n = c>>1, h = c&1: four groups of 16 elements at 128n+32g+16h (src/kquants.jl:333-343).
template <int TYPE>
struct Chunk;
template <>
struct Chunk<L2H_TYPE_Q4_K> {
    uint4 w, hdr;
};
template <>
struct Chunk<L2H_TYPE_Q5_K> {
    uint4 w, qh, hdr;
};
template <>
struct Chunk<L2H_TYPE_Q6_K> {
    uint4 la, lb, qh;
    uint32_t sc;
    uint32_t d;
};

__device__ __forceinline__ void zero_chunk(Chunk<L2H_TYPE_Q4_K> &c) {
    c.w = make_uint4(0, 0, 0, 0);
    c.hdr = make_uint4(0, 0, 0, 0);
}
__device__ __forceinline__ void zero_chunk(Chunk<L2H_TYPE_Q5_K> &c) {
    c.w = make_uint4(0, 0, 0, 0);
    c.qh = make_uint4(0, 0, 0, 0);
    c.hdr = make_uint4(0, 0, 0, 0);
}
__device__ __forceinline__ void zero_chunk(Chunk<L2H_TYPE_Q6_K> &c) {
    c.la = make_uint4(0, 0, 0, 0);
    c.lb = make_uint4(0, 0, 0, 0);
    c.qh = make_uint4(0, 0, 0, 0);
    c.sc = 0;
    c.d = 0;
}

template <int TYPE>
__device__ __forceinline__ int chunks_per_block() {
    return TYPE == L2H_TYPE_Q6_K ? 4 : 8;
}

// Stream pointers of the segment a row lives in, picked with selects so that the kernel
// arguments are only ever read at fixed offsets (one batch of scalar loads at kernel entry).
struct SegPtrs {
    const uint4 *hdr, *qs, *qh;
    const uint32_t *sc6;
    const uint16_t *d6;
    int64_t nb;
};
template <class T>
__device__ __forceinline__ T *at_layer(T *p, int64_t stride_bytes, int layer) {
    return (T *)((char *)p + stride_bytes * layer);
}
// `layer` selects the copy inside a per-role slab (0 when the pointers already name the layer)
__device__ __forceinline__ SegPtrs seg_ptrs(const PhaseArgs &a, int seg, int layer) {
    SegPtrs p;
#define PICK(F) (seg == 0 ? a.w[0].F : (seg == 1 ? a.w[1].F : a.w[2].F))
    const int64_t off = PICK(layer_stride) * layer;
    p.hdr = (const uint4 *)((const char *)PICK(hdr) + off);
    p.qs = (const uint4 *)((const char *)PICK(qs) + off);
    p.qh = (const uint4 *)((const char *)PICK(qh) + off);
    p.sc6 = (const uint32_t *)((const char *)PICK(sc6) + off);
    p.d6 = (const uint16_t *)((const char *)PICK(d6) + off);
#undef PICK
    p.nb = a.w[0].nb;
    return p;
}

template <int TYPE>
__device__ __forceinline__ void load_chunk(Chunk<TYPE> &c, const SegPtrs &t, int64_t row, int g);

template <>
__device__ __forceinline__ void load_chunk<L2H_TYPE_Q4_K>(Chunk<L2H_TYPE_Q4_K> &c, const SegPtrs &t, int64_t row,
                                                          int g) {
    c.w = ldg_nt(t.qs + row * t.nb * 8 + g);
    c.hdr = ldg_nt(t.hdr + row * t.nb + (g >> 3));
}
template <>
__device__ __forceinline__ void load_chunk<L2H_TYPE_Q5_K>(Chunk<L2H_TYPE_Q5_K> &c, const SegPtrs &t, int64_t row,
                                                          int g) {
    c.w = ldg_nt(t.qs + row * t.nb * 8 + g);
    c.qh = ldg_nt(t.qh + (row * t.nb + (g >> 3)) * 2 + (g & 1));
    c.hdr = ldg_nt(t.hdr + row * t.nb + (g >> 3));
}
template <>
__device__ __forceinline__ void load_chunk<L2H_TYPE_Q6_K>(Chunk<L2H_TYPE_Q6_K> &c, const SegPtrs &t, int64_t row,
                                                          int g) {
    const int64_t blk = row * t.nb + (g >> 2);
    const int n = (g >> 1) & 1, h = g & 1;
    c.la = ldg_nt(t.qs + blk * 8 + 4 * n + h);
    c.lb = ldg_nt(t.qs + blk * 8 + 4 * n + 2 + h);
    c.qh = ldg_nt(t.qh + blk * 4 + 2 * n + h);
    c.sc = __builtin_nontemporal_load(t.sc6 + blk * 4 + 2 * n + h);
    c.d = (uint32_t)__builtin_nontemporal_load(t.d6 + blk);
}

// ---- this lane's fp64 share of one chunk; DEBUG also stores the per-block integer sums ----------
// q4_K chunk given its unpacked scales: this lane's integer sums and their fp64 term
__device__ __forceinline__ double q4_term(const uint4 w, uint32_t d_dmin, int sc_a, int sc_b, int m_a, int m_b, int g,
                                          const XLds &x, int &i_sc, int &i_min) {
    const int b = g >> 3, c = g & 7, j = c >> 1, h = c & 1;
    const int8_t *xb = x.qs + b * 256 + 64 * j + 16 * h;
    const uint4 xlo = *(const uint4 *)xb;
    const uint4 xhi = *(const uint4 *)(xb + 32);
    int dot_a = 0, dot_b = 0;
    dot_a = sdot4(w.x & 0x0F0F0F0Fu, xlo.x, dot_a);
    dot_a = sdot4(w.y & 0x0F0F0F0Fu, xlo.y, dot_a);
    dot_a = sdot4(w.z & 0x0F0F0F0Fu, xlo.z, dot_a);
    dot_a = sdot4(w.w & 0x0F0F0F0Fu, xlo.w, dot_a);
    dot_b = sdot4((w.x >> 4) & 0x0F0F0F0Fu, xhi.x, dot_b);
    dot_b = sdot4((w.y >> 4) & 0x0F0F0F0Fu, xhi.y, dot_b);
    dot_b = sdot4((w.z >> 4) & 0x0F0F0F0Fu, xhi.z, dot_b);
    dot_b = sdot4((w.w >> 4) & 0x0F0F0F0Fu, xhi.w, dot_b);
    const int16_t *bs = x.bsums + b * 16 + 4 * j + h;
    // every factor fits 24 bits (scales < 64, |dot| <= 16*15*127, |bsum| <= 16*127): full-rate multiplies
    i_sc = mad24(sc_a, dot_a, __mul24(sc_b, dot_b));
    i_min = mad24(m_a, (int)bs[0], __mul24(m_b, (int)bs[2]));
    const float yd = x.d[b];
    const float dy = half_bits_to_float((uint16_t)(d_dmin & 0xFFFF)) * yd;
    const float my = half_bits_to_float((uint16_t)(d_dmin >> 16)) * yd;
    double t = (double)dy * (double)i_sc;
    t = fma(-(double)my, (double)i_min, t);
    return t;
}

template <bool DEBUG>
__device__ __forceinline__ double chunk_term(const Chunk<L2H_TYPE_Q4_K> &ch, int g, const XLds &x, int32_t *dbg_isc,
                                             int32_t *dbg_imin, int64_t dbg_base) {
    const int b = g >> 3, c = g & 7, j = c >> 1;
    int sc_a, sc_b, m_a, m_b;
    kq_scales_pair(ch.hdr, j, sc_a, sc_b, m_a, m_b);
    int i_sc, i_min;
    const double t = q4_term(ch.w, ch.hdr.x, sc_a, sc_b, m_a, m_b, g, x, i_sc, i_min);
    if (DEBUG) {
        i_sc += __shfl_xor(i_sc, 1, WAVE);
        i_min += __shfl_xor(i_min, 1, WAVE);
        i_sc += __shfl_xor(i_sc, 2, WAVE);
        i_min += __shfl_xor(i_min, 2, WAVE);
        i_sc += __shfl_xor(i_sc, 4, WAVE);
        i_min += __shfl_xor(i_min, 4, WAVE);
        if (c == 0) {
            dbg_isc[dbg_base + b] = i_sc;
            dbg_imin[dbg_base + b] = i_min;
        }
    }
    return t;
}

template <bool DEBUG>
__device__ __forceinline__ double chunk_term(const Chunk<L2H_TYPE_Q5_K> &ch, int g, const XLds &x, int32_t *dbg_isc,
                                             int32_t *dbg_imin, int64_t dbg_base) {
    const int b = g >> 3, c = g & 7, j = c >> 1, h = c & 1;
    int sc_a, sc_b, m_a, m_b;
    kq_scales_pair(ch.hdr, j, sc_a, sc_b, m_a, m_b);
    const int8_t *xb = x.qs + b * 256 + 64 * j + 16 * h;
    const uint4 xlo = *(const uint4 *)xb;
    const uint4 xhi = *(const uint4 *)(xb + 32);
    const uint4 w = ch.w, qh = ch.qh;
    const int sa = 2 * j, sb = 2 * j + 1;
    int dot_a = 0, dot_b = 0;
#define Q5LO(W, H) (((W)&0x0F0F0F0Fu) | ((((H) >> sa) & 0x01010101u) << 4))
#define Q5HI(W, H) ((((W) >> 4) & 0x0F0F0F0Fu) | ((((H) >> sb) & 0x01010101u) << 4))
    dot_a = sdot4(Q5LO(w.x, qh.x), xlo.x, dot_a);
    dot_a = sdot4(Q5LO(w.y, qh.y), xlo.y, dot_a);
    dot_a = sdot4(Q5LO(w.z, qh.z), xlo.z, dot_a);
    dot_a = sdot4(Q5LO(w.w, qh.w), xlo.w, dot_a);
    dot_b = sdot4(Q5HI(w.x, qh.x), xhi.x, dot_b);
    dot_b = sdot4(Q5HI(w.y, qh.y), xhi.y, dot_b);
    dot_b = sdot4(Q5HI(w.z, qh.z), xhi.z, dot_b);
    dot_b = sdot4(Q5HI(w.w, qh.w), xhi.w, dot_b);
#undef Q5LO
#undef Q5HI
    const int16_t *bs = x.bsums + b * 16 + 4 * j + h;
    int i_sc = mad24(sc_a, dot_a, __mul24(sc_b, dot_b));
    int i_min = mad24(m_a, (int)bs[0], __mul24(m_b, (int)bs[2]));
    const float yd = x.d[b];
    const float dy = half_bits_to_float((uint16_t)(ch.hdr.x & 0xFFFF)) * yd;
    const float my = half_bits_to_float((uint16_t)(ch.hdr.x >> 16)) * yd;
    double t = (double)dy * (double)i_sc;
    t = fma(-(double)my, (double)i_min, t);
    if (DEBUG) {
        i_sc += __shfl_xor(i_sc, 1, WAVE);
        i_min += __shfl_xor(i_min, 1, WAVE);
        i_sc += __shfl_xor(i_sc, 2, WAVE);
        i_min += __shfl_xor(i_min, 2, WAVE);
        i_sc += __shfl_xor(i_sc, 4, WAVE);
        i_min += __shfl_xor(i_min, 4, WAVE);
        if (c == 0) {
            dbg_isc[dbg_base + b] = i_sc;
            dbg_imin[dbg_base + b] = i_min;
        }
    }
    return t;
}

// q-32 is folded in through the q8_K group sums: sum (q-32)*x = sum q*x - 32*bsum.
template <bool DEBUG>
__device__ __forceinline__ double chunk_term(const Chunk<L2H_TYPE_Q6_K> &ch, int g, const XLds &x, int32_t *dbg_isc,
                                             int32_t *dbg_imin, int64_t dbg_base) {
    const int b = g >> 2, c = g & 3, n = c >> 1, h = c & 1;
    const int8_t *xb = x.qs + b * 256 + 128 * n + 16 * h;
    const uint4 x0 = *(const uint4 *)xb, x1 = *(const uint4 *)(xb + 32), x2 = *(const uint4 *)(xb + 64),
                x3 = *(const uint4 *)(xb + 96);
    const uint4 la = ch.la, lb = ch.lb, qh = ch.qh;
    int d0 = 0, d1 = 0, d2 = 0, d3 = 0;
#define Q6STEP(A, B, H, X0, X1, X2, X3)                                 \
    d0 = sdot4(((A)&0x0F0F0F0Fu) | (((H) << 4) & 0x30303030u), X0, d0); \
    d1 = sdot4(((B)&0x0F0F0F0Fu) | (((H) << 2) & 0x30303030u), X1, d1); \
    d2 = sdot4((((A) >> 4) & 0x0F0F0F0Fu) | ((H)&0x30303030u), X2, d2); \
    d3 = sdot4((((B) >> 4) & 0x0F0F0F0Fu) | (((H) >> 2) & 0x30303030u), X3, d3);
    Q6STEP(la.x, lb.x, qh.x, x0.x, x1.x, x2.x, x3.x)
    Q6STEP(la.y, lb.y, qh.y, x0.y, x1.y, x2.y, x3.y)
    Q6STEP(la.z, lb.z, qh.z, x0.z, x1.z, x2.z, x3.z)
    Q6STEP(la.w, lb.w, qh.w, x0.w, x1.w, x2.w, x3.w)
#undef Q6STEP
    const int16_t *bs = x.bsums + b * 16 + 8 * n + h;
    const uint32_t scw = ch.sc;
    const int s0 = (int)(int8_t)(scw & 0xFF), s1 = (int)(int8_t)((scw >> 8) & 0xFF),
              s2 = (int)(int8_t)((scw >> 16) & 0xFF), s3 = (int)(int8_t)(scw >> 24);
    // |d - 32 bsum| < 2^18 and |scale| < 2^7: 24-bit (full-rate) multiplies are exact
    int i_sc = mad24(s0, d0 - 32 * (int)bs[0],
                       mad24(s1, d1 - 32 * (int)bs[2], mad24(s2, d2 - 32 * (int)bs[4], __mul24(s3, d3 - 32 * (int)bs[6]))));
    const float dy = half_bits_to_float((uint16_t)ch.d) * x.d[b];
    const double t = (double)dy * (double)i_sc;
    if (DEBUG) {
        i_sc += __shfl_xor(i_sc, 1, WAVE);
        i_sc += __shfl_xor(i_sc, 2, WAVE);
        if (c == 0) {
            dbg_isc[dbg_base + b] = i_sc;
            dbg_imin[dbg_base + b] = 0;
        }
    }
    return t;
}

// ------------------------------------------------------------------------------------------
// wavefront reductions on DPP row operations (ALU latency, no LDS crossbar round trips)
// ------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ double dpp_f64(double v) {
    // (quad_perm / row mirrors read a valid lane everywhere, so the "old" operand is never used)
    const int l = __double2loint(v), h = __double2hiint(v);
    const int lo = __builtin_amdgcn_update_dpp(l, l, CTRL, 0xF, 0xF, true);
    const int hi = __builtin_amdgcn_update_dpp(h, h, CTRL, 0xF, 0xF, true);
    return __hiloint2double(hi, lo);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ double readlane_f64(double v, int lane) {
    const int lo = __builtin_amdgcn_readlane(__double2loint(v), lane);
    const int hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
    return __hiloint2double(hi, lo);
}
#define DPP_QUAD_SWAP1 0xB1     // quad_perm [1,0,3,2]
#define DPP_QUAD_SWAP2 0x4E     // quad_perm [2,3,0,1]
#define DPP_ROW_HALF_MIRROR 0x141
#define DPP_ROW_MIRROR 0x140

// Sum over the 64 lanes; the same value is returned on every lane.  Fixed order.
__device__ __forceinline__ double wave_sum_f64_dpp(double v) {
    v += dpp_f64<DPP_QUAD_SWAP1>(v);
    v += dpp_f64<DPP_QUAD_SWAP2>(v);
    v += dpp_f64<DPP_ROW_HALF_MIRROR>(v);
    v += dpp_f64<DPP_ROW_MIRROR>(v);
    return (readlane_f64(v, 0) + readlane_f64(v, 16)) + (readlane_f64(v, 32) + readlane_f64(v, 48));
}
// the first four steps of wave_sum_f64_dpp: every lane ends with the sum of its row of 16 lanes
__device__ __forceinline__ double row16_sum_f64_dpp(double v) {
    v += dpp_f64<DPP_QUAD_SWAP1>(v);
    v += dpp_f64<DPP_QUAD_SWAP2>(v);
    v += dpp_f64<DPP_ROW_HALF_MIRROR>(v);
    v += dpp_f64<DPP_ROW_MIRROR>(v);
    return v;
}
__device__ __forceinline__ float wave_max_f32_dpp(float v) {
    v = fmaxf(v, dpp_f32<DPP_QUAD_SWAP1>(v));
    v = fmaxf(v, dpp_f32<DPP_QUAD_SWAP2>(v));
    v = fmaxf(v, dpp_f32<DPP_ROW_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_f32<DPP_ROW_MIRROR>(v));
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
// sum within aligned groups of 4 lanes
__device__ __forceinline__ int quad_sum_i32(int v) {
    v += __builtin_amdgcn_update_dpp(v, v, DPP_QUAD_SWAP1, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(v, v, DPP_QUAD_SWAP2, 0xF, 0xF, true);
    return v;
}

// ------------------------------------------------------------------------------------------
// prologue: activations -> this workgroup's LDS
// ------------------------------------------------------------------------------------------
// One wavefront quantizes one q8_K block; lane l holds elements 4l..4l+3.  llama.cpp's
// quantize_row_q8_K rule: the FIRST element of largest magnitude fixes the scale (ties go to the
// lowest index), iscale = -127/max, q = min(127, round-half-even(iscale*x)), d = 1/iscale.
__device__ __forceinline__ void q8k_quantize_wave(const float v[4], uint32_t &packed, int &bsum16, float &d) {
    float amax = 0.0f, mx = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const float ax = fabsf(v[k]);
        if (ax > amax) {
            amax = ax;
            mx = v[k];
        }
    }
    const float wmax = wave_max_f32_dpp(amax);
    // lowest lane whose own extreme reaches the block's: its first such element is the block's first
    // (no lane holds it only where the block has a NaN: lane 0 then stands in, so that `first` is always a lane)
    const unsigned long long held = __ballot(amax == wmax), holders = held | (unsigned long long)(held == 0ull);
    const int first = __builtin_ctzll(holders);
    const float bmx = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mx), first));
    // an all-zero block gives q = 0, d = 0 (no branch: several blocks' code can then be interleaved)
    const bool zero = wmax == 0.0f;
    const float iscale = zero ? 0.0f : -127.0f / bmx;
    uint32_t word = 0;
    int sum = 0;
#pragma unroll
    for (int b = 0; b < 4; b++) {
        int q = (int)rintf(iscale * v[b]);
        q = q < 127 ? q : 127;
        sum += (int)(int8_t)q;
        word |= ((uint32_t)(q & 0xFF)) << (8 * b);
    }
    packed = word;
    bsum16 = quad_sum_i32(sum);
    d = zero ? 0.0f : 1.0f / iscale;
}

// The same with four blocks per wavefront: a row of 16 lanes holds a block, lane g of the row its elements 16g .. 16g+15
// (one group of 16, so the group's sum is the lane's own).  64 weights' worth of per-block work (the search for the
// extreme, two divisions) is then paid once per four blocks: a quarter of the instructions per block.
typedef unsigned int q8k_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void q8k_quantize_rows16(const float (&v)[16], q8k_u32x4 &packed, int &bsum, float &d) {
    // the lane's first element of largest magnitude, as a tree (of two candidates the later one wins only if it is larger)
    float c[8];
#pragma unroll
    for (int k = 0; k < 8; k++) c[k] = fabsf(v[2 * k + 1]) > fabsf(v[2 * k]) ? v[2 * k + 1] : v[2 * k];
#pragma unroll
    for (int k = 0; k < 4; k++) c[k] = fabsf(c[2 * k + 1]) > fabsf(c[2 * k]) ? c[2 * k + 1] : c[2 * k];
#pragma unroll
    for (int k = 0; k < 2; k++) c[k] = fabsf(c[2 * k + 1]) > fabsf(c[2 * k]) ? c[2 * k + 1] : c[2 * k];
    const float mx = fabsf(c[1]) > fabsf(c[0]) ? c[1] : c[0], amax = fabsf(mx);
    // The row's first element of largest magnitude: the sixteen lanes of a row agree on the lane with the largest |x| --
    // among equal ones the lowest, whose first such element is the block's first -- and on that lane's signed value.
    // (|x| >= 0 compares as an unsigned integer; a NaN compares above everything and then fixes the scale: unspecified
    // quants, no fault.  The four exchanges leave every lane of the row with the row's winner, as they do for a maximum.)
    unsigned kb = __float_as_uint(amax), kl = threadIdx.x & 15u;
    float bmx = mx;
#define Q8K_ROW_STEP(CTRL)                                                                                        \
    do {                                                                                                          \
        const unsigned ob = (unsigned)__builtin_amdgcn_update_dpp((int)kb, (int)kb, CTRL, 0xF, 0xF, true);        \
        const unsigned ol = (unsigned)__builtin_amdgcn_update_dpp((int)kl, (int)kl, CTRL, 0xF, 0xF, true);        \
        const float ov = dpp_f32<CTRL>(bmx);                                                                      \
        const bool take = ob > kb || (ob == kb && ol < kl);                                                       \
        kb = take ? ob : kb;                                                                                      \
        kl = take ? ol : kl;                                                                                      \
        bmx = take ? ov : bmx;                                                                                    \
    } while (0)
    Q8K_ROW_STEP(DPP_QUAD_SWAP1);
    Q8K_ROW_STEP(DPP_QUAD_SWAP2);
    Q8K_ROW_STEP(DPP_ROW_HALF_MIRROR);
    Q8K_ROW_STEP(DPP_ROW_MIRROR);
#undef Q8K_ROW_STEP
    const float rmax = __uint_as_float(kb);
    const bool zero = rmax == 0.0f;
    const float iscale = zero ? 0.0f : -127.0f / bmx;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int b = 0; b < 16; b++) {
        int q = (int)rintf(iscale * v[b]);
        q = q < 127 ? q : 127;
        w[b >> 2] |= ((uint32_t)(q & 0xFF)) << (8 * (b & 3));
    }
    packed.x = w[0];
    packed.y = w[1];
    packed.z = w[2];
    packed.w = w[3];
    // the group's sum of the quants as stored (int8): four signed byte dot products with ones
    bsum = sdot4(w[3], 0x01010101u, sdot4(w[2], 0x01010101u, sdot4(w[1], 0x01010101u, sdot4(w[0], 0x01010101u, 0))));
    d = zero ? 0.0f : 1.0f / iscale;
}

#define STAGE_MAX_ROUNDS 4  // q8_K blocks per wavefront: K <= 4 * 16 * 256

template <int PRO, bool KQ, bool COH>
__device__ __forceinline__ void stage_activations(const PhaseArgs &a, int layer, int64_t K, int8_t *s_qs, int16_t *s_bs,
                                                  float *s_d, float *s_xf, double *red) {
    const float *normw = at_layer(a.normw, a.normw_stride, layer);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    if (PRO == PRO_Q8) {
        const uint4 *g_qs = (const uint4 *)a.xq.qs;
        for (int i = tid; i < K / 16; i += blockDim.x) ((uint4 *)s_qs)[i] = g_qs[i];
        const uint4 *g_bs = (const uint4 *)a.xq.bsums;
        for (int i = tid; i < K / 128; i += blockDim.x) ((uint4 *)s_bs)[i] = g_bs[i];
        for (int i = tid; i < K / 256; i += blockDim.x) s_d[i] = a.xq.d[i];
        return;
    }
    if (!KQ) {  // F32 weights consume fp32 activations
        float ss = 1.0f;
        if (PRO == PRO_RMSNORM) {
            double acc = 0.0;
            for (int64_t i = tid; i < K; i += blockDim.x) {
                const double v = (double)ld_f32<COH>(a.xf + i);
                acc = fma(v, v, acc);
            }
            ss = (float)block_sum_f64(acc, red);
            ss /= (float)K;
            ss += 1e-5f;
            ss = 1.0f / sqrtf(ss);
        }
        for (int64_t i = tid; i < K; i += blockDim.x)
            s_xf[i] = PRO == PRO_RMSNORM ? normw[i] * (ss * ld_f32<COH>(a.xf + i)) : ld_f32<COH>(a.xf + i);
        return;
    }
    // k-quant weights: wavefront w takes q8_K blocks w, w+nwaves, ...; all loads issued first
    const int nb = (int)(K >> 8);
    float4 xv[STAGE_MAX_ROUNDS], wv[STAGE_MAX_ROUNDS];
#pragma unroll
    for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
        const int b = wave + r * nwaves;
        if (b < nb) {
            xv[r] = ld_f32x4<COH>(a.xf + 256 * b + 4 * lane);
            if (PRO == PRO_RMSNORM) wv[r] = *(const float4 *)(normw + 256 * b + 4 * lane);
        }
    }
    float ss = 1.0f;
    if (PRO == PRO_RMSNORM) {  // rmsnorm! (reference src/inference.jl:102-110)
        double acc = 0.0;
#pragma unroll
        for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
            const int b = wave + r * nwaves;
            if (b < nb) {
                acc = fma((double)xv[r].x, (double)xv[r].x, acc);
                acc = fma((double)xv[r].y, (double)xv[r].y, acc);
                acc = fma((double)xv[r].z, (double)xv[r].z, acc);
                acc = fma((double)xv[r].w, (double)xv[r].w, acc);
            }
        }
        acc = wave_sum_f64_dpp(acc);
        if (lane == 0) red[wave] = acc;
        __syncthreads();
        double t = 0.0;
        for (int w = 0; w < nwaves; w++) t += red[w];
        ss = (float)t;
        ss /= (float)K;
        ss += 1e-5f;
        ss = 1.0f / sqrtf(ss);
    }
#pragma unroll
    for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
        const int b = wave + r * nwaves;
        if (b < nb) {
            float v[4] = {xv[r].x, xv[r].y, xv[r].z, xv[r].w};
            if (PRO == PRO_RMSNORM) {
                v[0] = wv[r].x * (ss * v[0]);
                v[1] = wv[r].y * (ss * v[1]);
                v[2] = wv[r].z * (ss * v[2]);
                v[3] = wv[r].w * (ss * v[3]);
            }
            uint32_t packed;
            int bsum;
            float d;
            q8k_quantize_wave(v, packed, bsum, d);
            ((uint32_t *)s_qs)[64 * b + lane] = packed;
            if ((lane & 3) == 0) s_bs[16 * b + (lane >> 2)] = (int16_t)bsum;
            if (lane == 0) s_d[b] = d;
        }
    }
}

// ------------------------------------------------------------------------------------------
// logical rows.  Rows are numbered so that the two rows an epilogue combines are neighbours
// (2i, 2i+1): a w1/w3 pair, a RoPE pair; otherwise the concatenation of the segments' rows.
// ------------------------------------------------------------------------------------------
struct RowRef {
    int seg;      // segment index, -1 = no such row
    int64_t row;  // row inside the segment
};

// the row of a tile is the same on every lane: say so, and the address arithmetic and the
// selection of the segment's pointers run on the scalar unit
__device__ __forceinline__ RowRef uniform_row(RowRef r) {
    RowRef u;
    u.seg = __builtin_amdgcn_readfirstlane(r.seg);
    const int lo = __builtin_amdgcn_readfirstlane((int)(r.row & 0xFFFFFFFFll));
    const int hi = __builtin_amdgcn_readfirstlane((int)(r.row >> 32));
    u.row = ((int64_t)hi << 32) | (uint32_t)lo;
    return u;
}

template <int EPI>
__device__ __forceinline__ RowRef logical_row(const PhaseArgs &a, int64_t L) {
    RowRef rr;
    if (EPI == EPI_SWIGLU) {  // (w1 row g, w3 row g)
        rr.seg = (int)(L & 1);
        rr.row = L >> 1;
        return rr;
    }
    const int64_t n0 = a.w[0].ne1, n1 = a.nseg > 1 ? a.w[1].ne1 : 0, n2 = a.nseg > 2 ? a.w[2].ne1 : 0;
    if (L < n0) {
        rr.seg = 0;
    } else if (L < n0 + n1) {
        rr.seg = 1;
        L -= n0;
    } else if (L < n0 + n1 + n2) {
        rr.seg = 2;
        L -= n0 + n1;
    } else {
        rr.seg = -1;
    }
    rr.row = L;
    if (EPI == EPI_ROPE_KV && rr.seg >= 0 && a.neox) {
        const int role = (a.seg_roles >> (2 * rr.seg)) & 3;
        if (role != SEG_V) {  // neox pairs element i with i + hs/2 (reference src/inference.jl:146)
            const int half = a.hs >> 1;
            const int64_t h = L / a.hs;
            const int e = (int)(L % a.hs);
            rr.row = h * a.hs + (e >> 1) + ((e & 1) ? half : 0);
        }
    }
    return rr;
}

// exp evaluated in fp64 and rounded to fp32 (reference src/inference.jl:296)
__device__ __forceinline__ float swiglu_val(float h1, float h3) {
    const float e = (float)exp((double)(-h1));
    const float v = h1 * (1.0f / (1.0f + e));
    return v * h3;
}

// One thread finishes logical row L; `other` is the value of its neighbour row L^1.
template <int EPI, bool COH>
__device__ __forceinline__ void finish_row(const PhaseArgs &a, int layer, int64_t L, float val, float other) {
    const RowRef rr = logical_row<EPI>(a, L);
    if (rr.seg < 0) return;
    const int r = (int)(L & 1);
    if (EPI == EPI_STORE) {
        float *y = rr.seg == 0 ? a.y[0] : (rr.seg == 1 ? a.y[1] : a.y[2]);
        st_f32<COH>(y + rr.row, val);
    } else if (EPI == EPI_RESID) {  // x .+= ... (src/inference.jl:284,305)
        st_f32<COH>(a.y[0] + rr.row, ld_f32<COH>(a.resid + rr.row) + val);
    } else if (EPI == EPI_SWIGLU) {  // src/inference.jl:295-299
        if (r == 0) st_f32<COH>(a.y[0] + rr.row, swiglu_val(val, other));
    } else {  // EPI_ROPE_KV: rope! (src/inference.jl:112-157) and cache append (:259-260)
        const int role = (a.seg_roles >> (2 * rr.seg)) & 3;
        const int pos = a.ctl->pos;
        const int h = (int)(rr.row / a.hs), e = (int)(rr.row % a.hs);
        if (role == SEG_V) {
            if (a.kv16)
                st_kv(at_layer(a.vc, a.cache_stride, layer), ((int64_t)h * a.seq_len + pos) * a.hs + e, val, true);
            else
                st_f32<COH>(at_layer(a.vc, a.cache_stride, layer) + ((int64_t)h * a.seq_len + pos) * a.hs + e, val);
            return;
        }
        const int half = a.hs >> 1;
        const int i = a.neox ? (e % half) : (e >> 1);
        const float c = ld_f32<COH>(a.rope_cs + 2 * i), s = ld_f32<COH>(a.rope_cs + 2 * i + 1);
        // complex product (re + i im)(c + i s), each of the four products rounded
        const float re = r == 0 ? val : other, im = r == 0 ? other : val;
        const float out = r == 0 ? (re * c) - (im * s) : (re * s) + (im * c);
        if (role == SEG_Q) {
            st_f32<COH>(a.y[0] + rr.row, out);  // q is always the first segment of its launch
            st_f64<COH>(a.qd + rr.row, (double)out);
        } else {
            if (a.kv16)
                st_kv(at_layer(a.kc, a.cache_stride, layer), kc16_index(h, e, pos, a.hs, a.seq_len), out, true);
            else
                st_f32<COH>(at_layer(a.kc, a.cache_stride, layer) + (((int64_t)h * (a.hs >> 2) + (e >> 2)) * a.seq_len + pos) * 4 + (e & 3), out);
        }
    }
}

// ------------------------------------------------------------------------------------------
// the k-quant kernel.  A workgroup owns a contiguous range of logical rows.  Its work is cut
// into tiles of rt rows x st chunk-steps (rt*st <= NSLOT; a chunk-step = 64 lanes x one chunk);
// the 16 wavefronts take tiles round-robin with the next tile's loads in flight, reduce each
// tile's rows over the lanes and leave fp64 partial sums in LDS; then one thread per row adds
// that row's partials in a fixed order and runs the epilogue.
// ------------------------------------------------------------------------------------------
template <int TYPE>
struct Tile {
    static constexpr int NSLOT = TYPE == L2H_TYPE_Q4_K ? 4 : 2;
    Chunk<TYPE> c[NSLOT];
};

// profiling builds (-DL2H_TIMELINE) stamp the phases of every workgroup with the 100 MHz wall clock
#ifdef L2H_TIMELINE
#define TL(i)                                                                                 \
    if (a.timeline && threadIdx.x == 0) a.timeline[blockIdx.x * 8 + (i)] = wall_clock64();
#else
#define TL(i)
#endif

// One phase of one workgroup `wg`.  `smem` is the dynamic LDS area, `red` 16 doubles, `s_next` the
// tile counter.  If `preloaded`, `cur` already holds tile number `wave` of this phase (its loads
// were issued before the caller waited on the previous phase).
template <int TYPE, int PRO, int EPI, bool DEBUG, bool COH>
__device__ __forceinline__ void matvec_phase(const PhaseArgs &a, int layer, int wg, uint4 *smem, double *red,
                                             int *s_next_p, Tile<TYPE> &cur, bool preloaded) {
    TL(0)
    constexpr int NSLOT = Tile<TYPE>::NSLOT;
    constexpr int CPB = TYPE == L2H_TYPE_Q6_K ? 4 : 8;
    const int64_t K = a.w[0].ne0;
    int8_t *s_qs = (int8_t *)smem;
    int16_t *s_bs = (int16_t *)(s_qs + K);
    float *s_d = (float *)(s_qs + K + K / 8);
    double *s_part = (double *)(s_qs + ((K + K / 8 + K / 64 + 15) & ~(int64_t)15));  // [rows_per_wg][ntpr]
    float *s_val = (float *)(s_part + (int64_t)a.rows_per_wg * a.ntpr);              // [rows_per_wg]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int rt = a.rt, st = a.st, ntpr = a.ntpr;
    const int64_t L_lo = (int64_t)wg * a.rows_per_wg;
    const int64_t L_hi = min(a.n_rows, L_lo + a.rows_per_wg);
    const int n_local = L_hi > L_lo ? (int)(L_hi - L_lo) : 0;
    const int nchunks = (int)a.w[0].nb * CPB;
    const int nsteps = (nchunks + WAVE - 1) / WAVE;
    const int n_rowblocks = (n_local + rt - 1) / rt;
    const int ntiles = n_rowblocks * ntpr;

    // slot k of a tile: row offset k / st, step offset k % st
    auto load_tile = [&](Tile<TYPE> &t, int tt) {
        const int rb = tt / ntpr, sb = tt % ntpr;
#pragma unroll
        for (int k = 0; k < NSLOT; k++) {
            const int ro = k / st, so = k % st;
            const int lr = rb * rt + ro, step = sb * st + so;
            const int ci = lane + WAVE * step;
            if (ro < rt && lr < n_local && step < nsteps && ci < nchunks) {
                const RowRef rr = uniform_row(logical_row<EPI>(a, L_lo + lr));
                if (rr.seg >= 0) load_chunk<TYPE>(t.c[k], seg_ptrs(a, rr.seg, layer), rr.row, ci);
            }
        }
    };

    // the first 16 tiles are handed out statically, the rest on demand (equalises the finish
    // times of the wavefronts); every tile's partial sums have their own LDS slots, so the
    // result does not depend on which wavefront ran which tile
    if (threadIdx.x == 0) *s_next_p = nwaves;
    Tile<TYPE> nxt;
    int tt = wave;
    if (!preloaded && tt < ntiles) load_tile(cur, tt);  // in flight while the activations are staged
    TL(1)

    stage_activations<PRO, true, COH>(a, layer, K, s_qs, s_bs, s_d, nullptr, red);
    TL(2)
    __syncthreads();
    TL(3)
    XLds x{s_qs, s_bs, s_d, nullptr};

    while (tt < ntiles) {
        int tn = 0;
        if (lane == 0) tn = atomicAdd(s_next_p, 1);
        tn = __builtin_amdgcn_readfirstlane(tn);
        if (tn < ntiles) load_tile(nxt, tn);
        const int rb = tt / ntpr, sb = tt % ntpr;
        double acc[NSLOT];
#pragma unroll
        for (int k = 0; k < NSLOT; k++) {
            acc[k] = 0.0;
            const int ro = k / st, so = k % st;
            const int lr = rb * rt + ro, step = sb * st + so;
            const int ci = lane + WAVE * step;
            if (ro < rt && lr < n_local && step < nsteps && ci < nchunks) {
                const RowRef rr = uniform_row(logical_row<EPI>(a, L_lo + lr));
                if (rr.seg >= 0) {
                    int64_t dbg_base = 0;
                    if (DEBUG) dbg_base = rr.row * a.w[0].nb;  // debug launches have one segment
                    acc[k] = chunk_term<DEBUG>(cur.c[k], ci, x, a.dbg_isc, a.dbg_imin, dbg_base);
                }
            }
        }
        // fold the slots of each row, reduce over the lanes, park the partial sum
#pragma unroll
        for (int ro = 0; ro < NSLOT; ro++) {
            if (ro < rt) {  // uniform
                double v = 0.0;
#pragma unroll
                for (int k = 0; k < NSLOT; k++)
                    if (k / st == ro) v += acc[k];
                v = wave_sum_f64_dpp(v);
                const int lr = rb * rt + ro;
                if (lane == 0 && lr < n_local) s_part[lr * ntpr + sb] = v;
            }
        }
        cur = nxt;
        tt = tn;
    }
    TL(4)
    __syncthreads();
    TL(5)
    // one thread per logical row
    for (int lr = threadIdx.x; lr < n_local; lr += blockDim.x) {
        double v = 0.0;
        for (int p = 0; p < ntpr; p++) v += s_part[lr * ntpr + p];
        s_val[lr] = (float)v;
    }
    if (EPI == EPI_SWIGLU || EPI == EPI_ROPE_KV) __syncthreads();
    for (int lr = threadIdx.x; lr < n_local; lr += blockDim.x) {
        const float other = (EPI == EPI_SWIGLU || EPI == EPI_ROPE_KV) ? s_val[lr ^ 1] : 0.0f;
        finish_row<EPI, COH>(a, layer, L_lo + lr, s_val[lr], other);
    }
    TL(6)
}


// Issue the loads of tile number `wave` of a phase (what matvec_phase would do first).
template <int TYPE, int EPI>
__device__ __forceinline__ void matvec_prefetch(const PhaseArgs &a, int layer, int wg, Tile<TYPE> &t) {
    constexpr int NSLOT = Tile<TYPE>::NSLOT;
    constexpr int CPB = TYPE == L2H_TYPE_Q6_K ? 4 : 8;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rt = a.rt, st = a.st, ntpr = a.ntpr;
    const int64_t L_lo = (int64_t)wg * a.rows_per_wg;
    const int64_t L_hi = min(a.n_rows, L_lo + a.rows_per_wg);
    const int n_local = L_hi > L_lo ? (int)(L_hi - L_lo) : 0;
    const int nchunks = (int)a.w[0].nb * CPB;
    const int nsteps = (nchunks + WAVE - 1) / WAVE;
    const int ntiles = ((n_local + rt - 1) / rt) * ntpr;
    // every register of the tile is defined here, so the tile is dead before this call
#pragma unroll
    for (int k = 0; k < NSLOT; k++) zero_chunk(t.c[k]);
    if (wave >= ntiles) return;
    const int rb = wave / ntpr, sb = wave % ntpr;
#pragma unroll
    for (int k = 0; k < NSLOT; k++) {
        const int ro = k / st, so = k % st;
        const int lr = rb * rt + ro, step = sb * st + so;
        const int ci = lane + WAVE * step;
        if (ro < rt && lr < n_local && step < nsteps && ci < nchunks) {
            const RowRef rr = uniform_row(logical_row<EPI>(a, L_lo + lr));
            if (rr.seg >= 0) load_chunk<TYPE>(t.c[k], seg_ptrs(a, rr.seg, layer), rr.row, ci);
        }
    }
}

// Where matvec_phase left the finished fp32 row values of workgroup `wg` (LDS), and how many.
__device__ __forceinline__ const float *matvec_phase_vals(const PhaseArgs &a, int wg, uint4 *smem, int &n_local,
                                                          int64_t &L_lo) {
    const int64_t K = a.w[0].ne0;
    int8_t *s_qs = (int8_t *)smem;
    double *s_part = (double *)(s_qs + ((K + K / 8 + K / 64 + 15) & ~(int64_t)15));
    L_lo = (int64_t)wg * a.rows_per_wg;
    const int64_t L_hi = min(a.n_rows, L_lo + a.rows_per_wg);
    n_local = L_hi > L_lo ? (int)(L_hi - L_lo) : 0;
    return (const float *)(s_part + (int64_t)a.rows_per_wg * a.ntpr);
}

// ------------------------------------------------------------------------------------------
// attention of one head by one workgroup (reference src/inference.jl:263-278):
//   att[t] = fp32(sum_fp64 q[i] K[t][i]) / sqrt(hs); softmax (exp in fp64, fp64 sum); out[i] =
//   fp32(sum_fp64 p[t] V[t][i]).  Same arithmetic as the stand-alone attention kernels.
// LDS: q as fp64 [hs], att fp32 [np], p fp64 [np], partial sums [blockDim/hs][hs].
// ------------------------------------------------------------------------------------------
template <bool COH>
__device__ __forceinline__ void attention_head(const float *q, float *xb, const float *kc, const float *vc, int hs,
                                               int n_heads, int n_kv_heads, int seq_len, int h, int pos, uint4 *smem,
                                               double *redd, float *redf) {
    const int np = pos + 1;
    const int kvh = h / (n_heads / n_kv_heads);
    double *s_q = (double *)smem;
    double *s_p = s_q + hs;
    double *s_red = s_p + seq_len;
    float *s_att = (float *)(s_red + (blockDim.x / hs) * hs);
    const int tid = threadIdx.x;
    for (int i = tid; i < hs; i += blockDim.x) s_q[i] = (double)ld_f32<COH>(q + (int64_t)h * hs + i);
    __syncthreads();
    const float scale = sqrtf((float)hs);
    float mx = -INFINITY;
    for (int t = tid; t < np; t += blockDim.x) {
        const float *kp = kc + ((int64_t)kvh * (hs >> 2) * seq_len + t) * 4;
        double acc = 0.0;
        // four independent 16-byte loads in flight per step (hs is a multiple of 16 for 64/96/128)
        int i4 = 0;
        for (; i4 + 4 <= (hs >> 2); i4 += 4) {
            float4 kv[4];
#pragma unroll
            for (int u = 0; u < 4; u++) kv[u] = ld_f32x4<COH>(kp + (int64_t)(i4 + u) * seq_len * 4);
#pragma unroll
            for (int u = 0; u < 4; u++) {
                acc = fma(s_q[4 * (i4 + u) + 0], (double)kv[u].x, acc);
                acc = fma(s_q[4 * (i4 + u) + 1], (double)kv[u].y, acc);
                acc = fma(s_q[4 * (i4 + u) + 2], (double)kv[u].z, acc);
                acc = fma(s_q[4 * (i4 + u) + 3], (double)kv[u].w, acc);
            }
        }
        for (; i4 < (hs >> 2); i4++) {
            const float4 kv = ld_f32x4<COH>(kp + (int64_t)i4 * seq_len * 4);
            acc = fma(s_q[4 * i4 + 0], (double)kv.x, acc);
            acc = fma(s_q[4 * i4 + 1], (double)kv.y, acc);
            acc = fma(s_q[4 * i4 + 2], (double)kv.z, acc);
            acc = fma(s_q[4 * i4 + 3], (double)kv.w, acc);
        }
        const float a = (float)acc / scale;
        s_att[t] = a;
        mx = fmaxf(mx, a);
    }
    mx = block_max_f32(mx, redf);
    double sum = 0.0;
    for (int t = tid; t < np; t += blockDim.x) {
        const float e = (float)exp((double)(s_att[t] - mx));
        s_att[t] = e;
        sum += (double)e;
    }
    const float sf = (float)block_sum_f64(sum, redd);
    for (int t = tid; t < np; t += blockDim.x) s_p[t] = (double)(s_att[t] / sf);
    __syncthreads();
    const int ngrp = blockDim.x / hs;
    const int i = tid % hs, grp = tid / hs;
    if (grp < ngrp) {
        const float *vp = vc + (int64_t)kvh * seq_len * hs + i;
        double acc = 0.0;
        int t = grp;
        for (; t + 3 * ngrp < np; t += 4 * ngrp) {  // four loads in flight
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = ld_f32<COH>(vp + (int64_t)(t + u * ngrp) * hs);
#pragma unroll
            for (int u = 0; u < 4; u++) acc = fma(s_p[t + u * ngrp], (double)v[u], acc);
        }
        for (; t < np; t += ngrp) acc = fma(s_p[t], (double)ld_f32<COH>(vp + (int64_t)t * hs), acc);
        s_red[grp * hs + i] = acc;
    }
    __syncthreads();
    if (tid < hs) {
        double acc = 0.0;
        for (int k = 0; k < ngrp; k++) acc += s_red[k * hs + tid];
        st_f32<COH>(xb + (int64_t)h * hs + tid, (float)acc);
    }
    __syncthreads();
}

