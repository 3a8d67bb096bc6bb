// Streaming decode kernel: transformer! (reference src/inference.jl:222-315) plus the greedy pick
// (:360) for one token in ONE launch, built around two ideas:
//
//  * The weight bytes never wait for the activations.  At upload every wavefront of every
//    workgroup gets its own contiguous stream holding, in the order it will need them, the pieces
//    (8 q4_K super-blocks of one row, or 16 q6_K super-blocks) of all phases of all layers.  The
//    wavefront copies that stream into a private ring in LDS with global_load_lds_dwordx4, several
//    pieces ahead of the arithmetic and straight across phase boundaries, so HBM keeps streaming
//    while a workgroup waits for the activations of the next phase.
//
//  * No grid barrier.  Activations that cross workgroups travel as 8-byte words {fp32 value, epoch
//    tag}, written and read with device-scope relaxed atomics.  A consumer polls the words it needs
//    until they carry the epoch of the producing phase: data and "ready" arrive in one transaction.
//    Each buffer is rewritten only two or more phases after its last read, and reaching a phase
//    requires every workgroup to have finished the phase before the previous one, so a word is never
//    overwritten while somebody may still want its old value.
//
// The arithmetic is the same as in the per-phase kernels (matvec_dev.h): q8_K activations, integer
// dot products, fp64 sums rounded once.  Every wait is bounded; a workgroup that gives up raises
// `abort`, and all workgroups then leave the kernel.
#include "matvec_dev.h"

#include <string.h>

#define FLOW_D 7            // ring slots per wavefront
#define FLOW_SLOT 1152      // one q4_K piece: 8 headers (128 B) + 8 x 128 B of quants
#define FLOW_Q6_PIECE 3360  // 16 q6_K super-blocks: ql 2048, qh 1024, scales 256, d 32
#define FLOW_NW 16
#ifndef FLOW_FILL
#define FLOW_FILL 0         // pieces a wavefront may fetch per poll while it waits for activations
#endif
#ifndef FLOW_DEFER
#define FLOW_DEFER 0        // 1: inside a phase's loop fetch only that phase's pieces
#endif
#define FLOW_ACT_BYTES 28672
#define FLOW_MAX_PIECES 1024  // per workgroup and phase
#define FLOW_MAX_ROWS 512     // per workgroup and phase

typedef unsigned long long u64;

// Arguments of the model being decoded (everything but the epoch of the launch): constant memory,
// read with scalar loads wherever a phase needs a field.
__constant__ __attribute__((aligned(16))) unsigned char c_flow_raw[(sizeof(FlowArgs) + 15) & ~(size_t)15];
#define c_flow (*(const FlowArgs *)c_flow_raw)

// LDS of the kernel; file scope so that the phases can be separate functions.  The ring is its own
// object: the compiler then knows that ordinary LDS reads of the other areas never touch memory
// that an asynchronous fetch is still writing.
__shared__ __attribute__((aligned(16))) unsigned char s_ring[FLOW_NW * FLOW_D * FLOW_SLOT];
// activation area: q8_K input of the running phase in the first 16 KiB, then the per-piece partial sums
// and the row values; attention (between two matvec phases) uses the whole area for itself
__shared__ uint4 s_act[FLOW_ACT_BYTES / 16];
#define s_part ((double *)((unsigned char *)s_act + 16384))
#define s_val ((float *)((unsigned char *)s_act + 16384 + FLOW_MAX_PIECES * 8))
__shared__ float s_rope[256];
__shared__ double s_red[16];
__shared__ float s_redf[16];
__shared__ int s_flag;

__device__ __forceinline__ void tag_store(u64 *p, float v, unsigned epoch) {
    __hip_atomic_store(p, ((u64)epoch << 32) | (u64)__float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 tag_load(const u64 *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool tag_is(u64 w, unsigned epoch) { return (unsigned)(w >> 32) == epoch; }
__device__ __forceinline__ float tag_val(u64 w) { return __uint_as_float((unsigned)w); }

__host__ __device__ inline int flow_n_local(const FlowGeom &g, int wg) {
    const int lo = wg * g.rpw;
    const int hi = lo + g.rpw < g.n_rows ? lo + g.rpw : g.n_rows;
    return hi > lo ? hi - lo : 0;
}
// pieces of workgroup wg that wavefront `wave` takes: a contiguous run of the workgroup's pieces
// (consecutive pieces of a row stay in one wavefront where possible), the first np % 16 wavefronts
// one piece longer than the rest
__host__ __device__ inline int flow_wave_pieces(const FlowGeom &g, int wg, int wave) {
    const int np = flow_n_local(g, wg) * g.ppr;
    return np / FLOW_NW + (wave < np % FLOW_NW ? 1 : 0);
}
__host__ __device__ inline int flow_wave_start(const FlowGeom &g, int wg, int wave) {
    const int np = flow_n_local(g, wg) * g.ppr;
    const int base = np / FLOW_NW, rem = np % FLOW_NW;
    return wave * base + (wave < rem ? wave : rem);
}

// logical row L of a phase -> (tensor of the phase, row in it).  Logical rows put the two rows an
// epilogue combines next to each other: (w1 row u, w3 row u) and the two halves of a RoPE pair.
__host__ __device__ inline void flow_row_src(int kind, int L, int dim, int kv_dim, int hs, int neox, int &seg,
                                             int &row) {
    if (kind == 2) {  // w1 | w3
        seg = L & 1;
        row = L >> 1;
        return;
    }
    if (kind != 0) {
        seg = 0;
        row = L;
        return;
    }
    seg = L < dim ? 0 : (L < dim + kv_dim ? 1 : 2);
    row = L - (seg == 0 ? 0 : (seg == 1 ? dim : dim + kv_dim));
    if (neox && seg != 2) {  // neox pairs element i with i + hs/2 (reference src/inference.jl:146)
        const int h = row / hs, e = row % hs;
        row = h * hs + (e >> 1) + ((e & 1) ? (hs >> 1) : 0);
    }
}

// ------------------------------------------------------------------------------------------
// the ring of one wavefront
// ------------------------------------------------------------------------------------------
struct Ring;
__device__ __forceinline__ void ring_uniform(Ring &r);
struct Ring {
    const unsigned char *gptr;  // next byte of the stream to fetch
    unsigned lds;               // LDS byte address of slot 0
    int issued, consumed;       // pieces fetched / used so far
    int drain_mark;             // pieces known to have landed (issued before the last full wait)
    int iss_layer, iss_kind, iss_left;
    int iss_seq;                // phases the fetch cursor has passed: 4 * layer + kind of the phase it is in
};

// Headers inside the streams carry the twelve 6-bit scale bytes of a q4_K super-block (reference
// src/kquants.jl:80-109) regrouped so that a lane finds the four values of its sub-block pair j in
// one 24-bit field f_j = sc(2j) | sc(2j+1) << 6 | m(2j) << 12 | m(2j+1) << 18:
//   word 0 = d | dmin << 16;  word 1+k (k = 0..2) = f_k | byte k of f_3 << 24.
__host__ __device__ inline uint32_t flow_pair_field(int sc_a, int sc_b, int m_a, int m_b) {
    return (uint32_t)sc_a | (uint32_t)sc_b << 6 | (uint32_t)m_a << 12 | (uint32_t)m_b << 18;
}
__device__ __forceinline__ uint4 flow_encode_hdr(const uint4 hdr) {
    uint32_t f[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        int sa, sb, ma, mb;
        kq_scales_pair(hdr, j, sa, sb, ma, mb);
        f[j] = flow_pair_field(sa, sb, ma, mb);
    }
    return make_uint4(hdr.x, f[0] | (f[3] & 0xFF) << 24, f[1] | ((f[3] >> 8) & 0xFF) << 24, f[2] | (f[3] >> 16) << 24);
}
// this lane's field (j = 0..3 is fixed per lane: the selects use lane-constant conditions)
__device__ __forceinline__ void flow_decode_pair(const uint4 hdr, int j, int &sc_a, int &sc_b, int &m_a, int &m_b) {
    const uint32_t fw = j == 0 ? hdr.y : (j == 1 ? hdr.z : hdr.w);
    const uint32_t t = __builtin_amdgcn_perm(hdr.z, hdr.y, 0x0c0c0703u);  // byte 3 of word 1, byte 3 of word 2
    const uint32_t g = __builtin_amdgcn_perm(hdr.w, t, 0x0c070100u);      // ... and byte 3 of word 3
    const uint32_t f = j == 3 ? g : fw;
    sc_a = (int)(f & 63);
    sc_b = (int)((f >> 6) & 63);
    m_a = (int)((f >> 12) & 63);
    m_b = (int)((f >> 18) & 63);
}

// geometry of layer phase `kind`, field by field (scalar selects of scalar loads)
__device__ __forceinline__ FlowGeom flow_geom(const FlowArgs &a, int kind) {
    FlowGeom g;
    g.n_rows = kind == 0 ? a.qkv.n_rows : (kind == 1 ? a.wo.n_rows : (kind == 2 ? a.w13.n_rows : a.w2.n_rows));
    g.rpw = kind == 0 ? a.qkv.rpw : (kind == 1 ? a.wo.rpw : (kind == 2 ? a.w13.rpw : a.w2.rpw));
    g.ppr = kind == 0 ? a.qkv.ppr : (kind == 1 ? a.wo.ppr : (kind == 2 ? a.w13.ppr : a.w2.ppr));
    g.K = 0;
    return g;
}

// the ring's bookkeeping is the same on every lane: keep it in scalar registers
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }

__device__ __forceinline__ void ring_uniform(Ring &r) {
    const unsigned long long p = (unsigned long long)r.gptr;
    const unsigned lo = (unsigned)uni((int)(unsigned)p), hi = (unsigned)uni((int)(unsigned)(p >> 32));
    r.gptr = (const unsigned char *)(((unsigned long long)hi << 32) | lo);
    r.lds = (unsigned)uni((int)r.lds);
    r.issued = uni(r.issued);
    r.consumed = uni(r.consumed);
    r.drain_mark = uni(r.drain_mark);
    r.iss_layer = uni(r.iss_layer);
    r.iss_kind = uni(r.iss_kind);
    r.iss_left = uni(r.iss_left);
    r.iss_seq = uni(r.iss_seq);
}

// Between the phases the bookkeeping lives in LDS (one row per wavefront), so that the staging
// function, which is a separate function, can keep fetching while it waits for activations.
__shared__ int s_rs[FLOW_NW][12];
__device__ __forceinline__ void ring_store(const Ring &r) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if ((threadIdx.x & 63) == 0) {
        const unsigned long long p = (unsigned long long)r.gptr;
        int *d = s_rs[wave];
        d[0] = (int)(unsigned)p;
        d[1] = (int)(unsigned)(p >> 32);
        d[2] = (int)r.lds;
        d[3] = r.issued;
        d[4] = r.consumed;
        d[5] = r.drain_mark;
        d[6] = r.iss_layer;
        d[7] = r.iss_kind;
        d[8] = r.iss_left;
        d[9] = r.iss_seq;
    }
}
__device__ __forceinline__ void ring_load(Ring &r) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int *d = s_rs[wave];
    const unsigned lo = (unsigned)uni(d[0]), hi = (unsigned)uni(d[1]);
    r.gptr = (const unsigned char *)(((unsigned long long)hi << 32) | lo);
    r.lds = (unsigned)uni(d[2]);
    r.issued = uni(d[3]);
    r.consumed = uni(d[4]);
    r.drain_mark = uni(d[5]);
    r.iss_layer = uni(d[6]);
    r.iss_kind = uni(d[7]);
    r.iss_left = uni(d[8]);
    r.iss_seq = uni(d[9]);
}

#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))

// fetch the next q4_K piece of this wavefront's stream, if the layer phases have one left
__device__ __forceinline__ void flow_issue_q4(Ring &r, const FlowArgs &a, unsigned char *ring_base, int wg, int wave,
                                              int lane) {
    // (the bookkeeping is the same on every lane; saying so where it steers a branch keeps the
    // branches on the scalar unit)
    while (uni(r.iss_left) == 0) {
        r.iss_layer = uni(r.iss_layer);
        r.iss_kind = uni(r.iss_kind);
        if (r.iss_layer >= a.n_layers) return;
        r.iss_seq = uni(r.iss_seq) + 1;
        if (++r.iss_kind == 4) {
            r.iss_kind = 0;
            if (++r.iss_layer >= a.n_layers) return;
        }
        r.iss_left = uni(flow_wave_pieces(flow_geom(a, r.iss_kind), wg, wave));
    }
    unsigned char *slot = ring_base + (uni(r.issued) % FLOW_D) * FLOW_SLOT;
    const unsigned char *g = r.gptr;
    if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)(g + lane * 16), (AS3 void *)slot, 16, 0, 2);
    __builtin_amdgcn_global_load_lds((const AS1 void *)(g + 128 + lane * 16), (AS3 void *)(slot + 128), 16, 0, 2);
    r.gptr += FLOW_SLOT;
    r.issued++;
    r.iss_left--;
}

// everything this wavefront has fetched so far has landed
__device__ __forceinline__ void flow_drain(Ring &r) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    r.drain_mark = r.issued;
}

// piece number r.consumed has landed (fetches complete in order; OPS fetch instructions per piece)
template <int OPS>
__device__ __forceinline__ void flow_wait_piece(const Ring &r) {
    if (uni(r.consumed) < uni(r.drain_mark)) return;
    const int younger = uni(r.issued - 1 - r.consumed);
    constexpr int DEPTH = OPS == 2 ? FLOW_D : 2;
    if (younger >= DEPTH - 1) {  // the steady state: a full ring
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS * (DEPTH - 1)) : "memory");
        return;
    }
    switch (younger) {
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS * 1) : "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS * 2 > 63 ? 63 : OPS * 2) : "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS * 3 > 63 ? 63 : OPS * 3) : "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS * 4 > 63 ? 63 : OPS * 4) : "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS * 5 > 63 ? 63 : OPS * 5) : "memory"); break;
    }
}

// ------------------------------------------------------------------------------------------
// staging: the input vector of a phase -> q8_K in this workgroup's LDS.  Source: tagged words of
// epoch `epoch`, or (EMB) the embedding row of `tok`.  Returns false if the wait gave up.
// Separate functions (not inlined): the kernel stays small enough to keep its state in registers.
// ------------------------------------------------------------------------------------------
// While it polls, every wavefront keeps fetching pieces of its weight stream into free ring slots
// (`fill` pieces per poll at most; 0 = not at all): the fetches are issued behind the poll's loads, so
// the poll does not wait for them, and they use the time in which the arithmetic has nothing to do.
template <int PRO, bool EMB>
__device__ __noinline__ bool flow_stage(const u64 *src, unsigned epoch, int K, const float *normw, int tok, int fill) {
    const FlowArgs &a = c_flow;
    int8_t *s_qs = (int8_t *)s_act;
    int16_t *s_bs = (int16_t *)(s_qs + 14336);
    float *s_d = (float *)(s_qs + 14336 + 1792);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nb = K >> 8;
    float xv[STAGE_MAX_ROUNDS][4];
    bool ok = true;
    if (EMB) {
#pragma unroll
        for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
            const int b = wave + r * FLOW_NW;
            if (b < nb)
#pragma unroll
                for (int k = 0; k < 4; k++) xv[r][k] = dequant_elem(a.emb, tok, 256 * b + 4 * lane + k);
        }
    } else {
        unsigned spins = 0;
        Ring ring;
        unsigned char *ring_base = s_ring + wave * (FLOW_D * FLOW_SLOT);
        if (fill > 0) ring_load(ring);
        // first pass: every word; later passes: only the words that did not carry the epoch yet, so
        // that waiting for a slow producer costs next to no traffic
        u64 w[STAGE_MAX_ROUNDS][4];
#pragma unroll
        for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
            const int b = wave + r * FLOW_NW;
            if (b < nb)
#pragma unroll
                for (int k = 0; k < 4; k++) w[r][k] = tag_load(src + 256 * b + 4 * lane + k);
        }
        for (;;) {
#pragma nounroll
            for (int f = 0; f < fill; f++) {
                if (uni(ring.issued) - uni(ring.consumed) >= FLOW_D) break;
                flow_issue_q4(ring, a, ring_base, blockIdx.x, wave, lane);
            }
            bool all = true;
#pragma unroll
            for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
                const int b = wave + r * FLOW_NW;
                if (b < nb)
#pragma unroll
                    for (int k = 0; k < 4; k++) all = all && tag_is(w[r][k], epoch);
            }
            // the wavefront leaves the loop as a whole: the fetches above need all of its lanes
            if (__ballot(!all) == 0ull) break;
            if (++spins > a.spin_limit ||
                ((spins & 63) == 0 && __hip_atomic_load(a.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                ok = false;
                break;
            }
#pragma unroll
            for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
                const int b = wave + r * FLOW_NW;
                if (b < nb)
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        if (!tag_is(w[r][k], epoch)) w[r][k] = tag_load(src + 256 * b + 4 * lane + k);
            }
        }
#pragma unroll
        for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
            const int b = wave + r * FLOW_NW;
            if (b < nb)
#pragma unroll
                for (int k = 0; k < 4; k++) xv[r][k] = tag_val(w[r][k]);
        }
        if (fill > 0) ring_store(ring);
    }
    if (threadIdx.x == 0) s_flag = 0;
    __syncthreads();
    if (!ok) s_flag = 1;
    float wv[STAGE_MAX_ROUNDS][4];
    double acc = 0.0;
    if (PRO == PRO_RMSNORM) {  // rmsnorm! (reference src/inference.jl:102-110)
#pragma unroll
        for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
            const int b = wave + r * FLOW_NW;
            if (b < nb) {
                const float4 t = *(const float4 *)(normw + 256 * b + 4 * lane);
                wv[r][0] = t.x;
                wv[r][1] = t.y;
                wv[r][2] = t.z;
                wv[r][3] = t.w;
#pragma unroll
                for (int k = 0; k < 4; k++) acc = fma((double)xv[r][k], (double)xv[r][k], acc);
            }
        }
        acc = wave_sum_f64_dpp(acc);
        if (lane == 0) s_red[wave] = acc;
    }
    __syncthreads();
    if (s_flag) {
        if (threadIdx.x == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return false;
    }
    float ss = 1.0f;
    if (PRO == PRO_RMSNORM) {
        double t = 0.0;
        for (int w = 0; w < FLOW_NW; w++) t += s_red[w];
        ss = (float)t;
        ss /= (float)K;
        ss += 1e-5f;
        ss = 1.0f / sqrtf(ss);
    }
#pragma unroll
    for (int r = 0; r < STAGE_MAX_ROUNDS; r++) {
        const int b = wave + r * FLOW_NW;
        if (b < nb) {
            float v[4];
#pragma unroll
            for (int k = 0; k < 4; k++) v[k] = PRO == PRO_RMSNORM ? wv[r][k] * (ss * xv[r][k]) : xv[r][k];
            uint32_t packed;
            int bsum;
            float d;
            q8k_quantize_wave(v, packed, bsum, d);
            ((uint32_t *)s_qs)[64 * b + lane] = packed;
            if ((lane & 3) == 0) s_bs[16 * b + (lane >> 2)] = (int16_t)bsum;
            if (lane == 0) s_d[b] = d;
        }
    }
    __syncthreads();
    return true;
}

// one tagged word, waited for (the caller has usually seen it already)
__device__ __forceinline__ float flow_read(const u64 *p, unsigned epoch) {
    u64 w = tag_load(p);
    unsigned spins = 0;
    while (!tag_is(w, epoch) && ++spins <= c_flow.spin_limit) w = tag_load(p);
    return tag_val(w);
}

// ------------------------------------------------------------------------------------------
// the arithmetic of one phase for one workgroup: pieces from the ring x q8_K activations in LDS
// -> one fp64 partial sum per piece in s_part[local row * ppr + part]
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ XLds flow_x() {
    int8_t *s_qs = (int8_t *)s_act;
    XLds x;
    x.qs = s_qs;
    x.bsums = (const int16_t *)(s_qs + 14336);
    x.d = (const float *)(s_qs + 14336 + 1792);
    x.xf = nullptr;
    return x;
}

// Fetches are issued inside the loop only while pieces of THIS phase are still missing (an issue
// blocks while the memory pipeline is full, and would hold up the arithmetic); the slots freed
// beyond that are refilled by the staging function of the following phases while it waits.
// cur_seq = 4 * layer + kind of the phase, or -1 for the classifier (which has nothing after it).
__device__ __forceinline__ void flow_loop_q4(const FlowGeom &g, Ring &r, unsigned char *ring_base, int wg, int cur_seq) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ppr = uni(g.ppr);
    const int cnt = uni(flow_wave_pieces(g, wg, wave)), start = uni(flow_wave_start(g, wg, wave));
    const XLds x = flow_x();
    flow_drain(r);
    // whatever the waits before this phase did not fetch of its pieces is requested now
#pragma nounroll
    for (int k = 0; k < FLOW_D; k++) {
        if (uni(r.issued) - uni(r.consumed) >= FLOW_D) break;
        if (FLOW_DEFER && !(cur_seq < 0 || uni(r.iss_seq) < cur_seq || (uni(r.iss_seq) == cur_seq && uni(r.iss_left) > 0))) break;
        flow_issue_q4(r, c_flow, ring_base, wg, wave, lane);
    }
    int part = uni(start % ppr);
    double acc = 0.0;
    for (int k = 0; k < cnt; k++) {
        flow_wait_piece<2>(r);
        const unsigned slot = r.lds + (unsigned)(uni(r.consumed) % FLOW_D) * FLOW_SLOT;
        Chunk<L2H_TYPE_Q4_K> ch;
        asm volatile("ds_read_b128 %0, %2 offset:128\n\tds_read_b128 %1, %3\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(ch.w), "=&v"(ch.hdr)
                     : "v"(slot + lane * 16), "v"(slot + (lane >> 3) * 16)
                     : "memory");
        r.consumed++;
        if (!FLOW_DEFER || cur_seq < 0 || uni(r.iss_seq) < cur_seq || (uni(r.iss_seq) == cur_seq && uni(r.iss_left) > 0))
            flow_issue_q4(r, c_flow, ring_base, wg, wave, lane);  // the slot is free again
#ifdef FLOW_EXP_NOMATH
        acc += (double)(ch.w.x ^ ch.hdr.y);
#else
        {
            int sc_a, sc_b, m_a, m_b, i_sc, i_min;
            flow_decode_pair(ch.hdr, (lane & 7) >> 1, sc_a, sc_b, m_a, m_b);
            acc += q4_term(ch.w, ch.hdr.x, sc_a, sc_b, m_a, m_b, part * 64 + lane, x, i_sc, i_min);
        }
#endif
        // a row's consecutive pieces are reduced over the lanes once; every piece has its own slot
        // in s_part, the run's total goes to its last piece and zero to the others
        const bool last = k == cnt - 1 || uni(part) == ppr - 1;
        if (last) {
            const double v = wave_sum_f64_dpp(acc);
            if (lane == 0) s_part[start + k] = v;
            acc = 0.0;
        } else if (lane == 0) {
            s_part[start + k] = 0.0;
        }
        part = part == ppr - 1 ? 0 : part + 1;
    }
}

// classifier pieces (q6_K): 16 super-blocks per piece, lane = (block lane/4, chunk lane%4); the ring
// holds two pieces
#define FLOW_Q6_D 2
__device__ __forceinline__ void flow_issue_q6(Ring &r, unsigned char *ring_base, int lane) {
    if (uni(r.iss_left) == 0) return;
    unsigned char *slot = ring_base + (uni(r.issued) % FLOW_Q6_D) * FLOW_Q6_PIECE;
    const unsigned char *g = r.gptr;
    __builtin_amdgcn_global_load_lds((const AS1 void *)(g + lane * 16), (AS3 void *)slot, 16, 0, 2);
    __builtin_amdgcn_global_load_lds((const AS1 void *)(g + 1024 + lane * 16), (AS3 void *)(slot + 1024), 16, 0, 2);
    __builtin_amdgcn_global_load_lds((const AS1 void *)(g + 2048 + lane * 16), (AS3 void *)(slot + 2048), 16, 0, 2);
    if (lane < 16)
        __builtin_amdgcn_global_load_lds((const AS1 void *)(g + 3072 + lane * 16), (AS3 void *)(slot + 3072), 16, 0, 2);
    if (lane < 2)
        __builtin_amdgcn_global_load_lds((const AS1 void *)(g + 3328 + lane * 16), (AS3 void *)(slot + 3328), 16, 0, 2);
    r.gptr += FLOW_Q6_PIECE;
    r.issued++;
    r.iss_left--;
}

__device__ __forceinline__ void flow_loop_q6(const FlowGeom &g, Ring &r, unsigned char *ring_base, int wg) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ppr = uni(g.ppr);
    const int cnt = uni(flow_wave_pieces(g, wg, wave)), start = uni(flow_wave_start(g, wg, wave));
    const int b = lane >> 2, c = lane & 3, n = c >> 1, h = c & 1;
    const XLds x = flow_x();
    flow_drain(r);
    int part = uni(start % ppr);
    double acc = 0.0;
    for (int k = 0; k < cnt; k++) {
        flow_wait_piece<5>(r);
        const unsigned slot = r.lds + (unsigned)(uni(r.consumed) % FLOW_Q6_D) * FLOW_Q6_PIECE;
        Chunk<L2H_TYPE_Q6_K> ch;
        uint32_t d16;
        asm volatile("ds_read_b128 %0, %5\n\tds_read_b128 %1, %5 offset:32\n\tds_read_b128 %2, %6 offset:2048\n\t"
                     "ds_read_b32 %3, %7 offset:3072\n\tds_read_u16 %4, %8 offset:3328\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(ch.la), "=&v"(ch.lb), "=&v"(ch.qh), "=&v"(ch.sc), "=&v"(d16)
                     : "v"(slot + b * 128 + 64 * n + 16 * h), "v"(slot + b * 64 + 32 * n + 16 * h),
                       "v"(slot + (b * 4 + 2 * n + h) * 4), "v"(slot + b * 2)
                     : "memory");
        ch.d = d16;
        r.consumed++;
        flow_issue_q6(r, ring_base, lane);
        acc += chunk_term<false>(ch, part * 64 + lane, x, nullptr, nullptr, 0);
        const bool last = k == cnt - 1 || uni(part) == ppr - 1;
        if (last) {
            const double v = wave_sum_f64_dpp(acc);
            if (lane == 0) s_part[start + k] = v;
            acc = 0.0;
        } else if (lane == 0) {
            s_part[start + k] = 0.0;
        }
        part = part == ppr - 1 ? 0 : part + 1;
    }
}

// fp32 value of every local row: the pieces' partial sums added in order
__device__ __forceinline__ void flow_row_values(int n_local, int ppr) {
    __syncthreads();
    for (int lr = threadIdx.x; lr < n_local; lr += blockDim.x) {
        double v = 0.0;
        for (int p = 0; p < ppr; p++) v += s_part[lr * ppr + p];
        s_val[lr] = (float)v;
    }
    __syncthreads();
}

// ---- epilogues -------------------------------------------------------------------------------
// rope! (reference src/inference.jl:112-157) and the cache append (:259-260)
__device__ __noinline__ void flow_finish_qkv(int l, int wg, int pos, unsigned e_q) {
    const FlowArgs &a = c_flow;
    const int n_local = flow_n_local(a.qkv, wg), tid = threadIdx.x;
    flow_row_values(n_local, a.qkv.ppr);
    if (tid >= n_local) return;
    const int L = wg * a.qkv.rpw + tid;
    int seg, row;
    flow_row_src(0, L, a.dim, a.kv_dim, a.hs, a.neox, seg, row);
    const float val = s_val[tid], other = s_val[tid ^ 1];
    const int hh = row / a.hs, e = row % a.hs;
    if (seg == 2) {
        (a.vc + (int64_t)l * a.cache_layer_elems)[((int64_t)hh * a.seq_len + pos) * a.hs + e] = val;
        tag_store(a.vcur + row, val, e_q);
        return;
    }
    const int half = a.hs >> 1;
    const int i = a.neox ? (e % half) : (e >> 1);
    const float c = s_rope[2 * i], s = s_rope[2 * i + 1];
    const int rr = tid & 1;
    // complex product (re + i im)(c + i s), each of the four products rounded
    const float re = rr == 0 ? val : other, im = rr == 0 ? other : val;
    const float out = rr == 0 ? (re * c) - (im * s) : (re * s) + (im * c);
    if (seg == 0) {
        tag_store(a.q + row, out, e_q);
    } else {
        (a.kc + (int64_t)l * a.cache_layer_elems)[(((int64_t)hh * (a.hs >> 2) + (e >> 2)) * a.seq_len + pos) * 4 + (e & 3)] = out;
        tag_store(a.kcur + row, out, e_q);
    }
}

// dst = old + result (x .+= ..., :284,305); which = 1 after wo (-> x_b), 3 after w2 (-> x_a); `old` is
// this thread's row of the other buffer, fetched before the loop
__device__ __noinline__ void flow_finish_resid(int which, int wg, u64 oldw, unsigned e_src, unsigned e_dst) {
    const FlowArgs &a = c_flow;
    const FlowGeom &g = which == 1 ? a.wo : a.w2;
    const u64 *src = which == 1 ? a.x_a : a.x_b;
    u64 *dst = which == 1 ? a.x_b : a.x_a;
    const int n_local = flow_n_local(g, wg), tid = threadIdx.x;
    flow_row_values(n_local, g.ppr);
    if (tid >= n_local) return;
    const int row = wg * g.rpw + tid;
    const float old = tag_is(oldw, e_src) ? tag_val(oldw) : flow_read(src + row, e_src);
    tag_store(dst + row, old + s_val[tid], e_dst);
}

// SwiGLU (:295-299): logical rows (2u, 2u+1) are w1 row u and w3 row u
__device__ __noinline__ void flow_finish_w13(int wg, unsigned e_out) {
    const FlowArgs &a = c_flow;
    const int n_local = flow_n_local(a.w13, wg), tid = threadIdx.x;
    flow_row_values(n_local, a.w13.ppr);
    if (tid >= n_local || (tid & 1)) return;
    const int64_t u = ((int64_t)wg * a.w13.rpw + tid) >> 1;
    tag_store(a.hb + u, swiglu_val(s_val[tid], s_val[tid + 1]), e_out);
}

// logits (:312) and this workgroup's first-maximum key: larger value wins, then the lower index
// (Julia's argmax, :360)
__device__ __noinline__ void flow_finish_cls(int wg, unsigned e_cls) {
    const FlowArgs &a = c_flow;
    const int n_local = flow_n_local(a.cls, wg), tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    flow_row_values(n_local, a.cls.ppr);
    unsigned long long best = 0;
    if (tid < n_local) {
        const int64_t row = (int64_t)wg * a.cls.rpw + tid;
        a.logits[row] = s_val[tid];
        uint32_t b = __float_as_uint(s_val[tid]);
        b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
        if (s_val[tid] == 0.0f) b = 0x80000000u;
        best = ((unsigned long long)b << 32) | (unsigned long long)(0xFFFFFFFFu - (uint32_t)row);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const unsigned long long o = __shfl_xor(best, m, WAVE);
        best = o > best ? o : best;
    }
    unsigned long long *redk = (unsigned long long *)s_red;
    __syncthreads();
    if (lane == 0) redk[wave] = best;
    __syncthreads();
    if (tid == 0) {
        unsigned long long t = redk[0];
        for (int w = 1; w < FLOW_NW; w++) t = redk[w] > t ? redk[w] : t;
        tag_store(a.amax + 2 * wg, __uint_as_float((unsigned)(t >> 32)), e_cls);
        tag_store(a.amax + 2 * wg + 1, __uint_as_float((unsigned)t), e_cls);
    }
}

// argmax(logits) (:360) over the workgroups' keys and the step bookkeeping of the token loop
// (:349-386); run by workgroup 0
__device__ __noinline__ void flow_pick_token(int nwg, unsigned e_cls) {
    const FlowArgs &a = c_flow;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned long long best = 0;
    bool ok = true;
    for (int i = tid; i < nwg; i += blockDim.x) {
        u64 hi = tag_load(a.amax + 2 * i), lo = tag_load(a.amax + 2 * i + 1);
        unsigned spins = 0;
        while (!(tag_is(hi, e_cls) && tag_is(lo, e_cls))) {
            if (++spins > a.spin_limit) {
                ok = false;
                break;
            }
            hi = tag_load(a.amax + 2 * i);
            lo = tag_load(a.amax + 2 * i + 1);
        }
        const unsigned long long k = ((unsigned long long)(unsigned)hi << 32) | (unsigned long long)(unsigned)lo;
        best = k > best ? k : best;
    }
    if (tid == 0) s_flag = 0;
    __syncthreads();
    if (!ok) s_flag = 1;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const unsigned long long o = __shfl_xor(best, m, WAVE);
        best = o > best ? o : best;
    }
    unsigned long long *redk = (unsigned long long *)s_red;
    __syncthreads();
    if (lane == 0) redk[wave] = best;
    __syncthreads();
    if (tid != 0) return;
    if (s_flag) {
        __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    unsigned long long t = redk[0];
    for (int w = 1; w < FLOW_NW; w++) t = redk[w] > t ? redk[w] : t;
    DecodeCtl *ctl = a.ctl;
    const int idx = (int)(0xFFFFFFFFu - (uint32_t)(t & 0xFFFFFFFFull));
    ctl->last_argmax = idx;
    if (ctl->step >= ctl->n_prompt - 1 && ctl->n_out < a.max_out) {
        a.out_tokens[ctl->n_out] = idx;
        ctl->n_out += 1;
    }
    ctl->step += 1;
    ctl->pos += 1;
}

// ------------------------------------------------------------------------------------------
// attention of head h by one workgroup (reference src/inference.jl:263-278); q and the current
// position's k, v arrive as tagged words, earlier positions come from the cache (written by earlier
// launches).  Same arithmetic, in the same order, as attention_head.
// ------------------------------------------------------------------------------------------
__device__ __noinline__ bool flow_attention(int layer, int h, int pos, unsigned e_in, unsigned e_out) {
    const FlowArgs &a = c_flow;
    const int hs = a.hs, seq_len = a.seq_len, np = pos + 1;
    const int kvh = h / (a.n_heads / a.n_kv_heads);
    const float *kc = a.kc + (int64_t)layer * a.cache_layer_elems;
    const float *vc = a.vc + (int64_t)layer * a.cache_layer_elems;
    double *s_q = (double *)s_act;
    double *s_p = s_q + hs;
    double *s_r = s_p + seq_len;
    float *s_att = (float *)(s_r + (FLOW_NW * hs > 1024 ? FLOW_NW * hs : 1024));
    float *s_kcur = s_att + ((seq_len + 3) & ~3);
    float *s_vcur = s_kcur + hs;
    const int tid = threadIdx.x;
    bool ok = true;
#ifdef L2H_TIMELINE
    int atl = 0;
#define ATL()                                                                                                    \
    do {                                                                                                         \
        if (a.timeline && tid == 0 && layer == 2 && atl < 16) a.timeline[256 * 64 + h * 16 + atl++] = wall_clock64(); \
    } while (0)
#else
#define ATL()
#endif
    ATL();
    __syncthreads();  // the activation area is free
    if (tid < 3 * hs) {
        const int which = tid / hs, i = tid % hs;
        const u64 *p = which == 0 ? a.q + (int64_t)h * hs + i : (which == 1 ? a.kcur : a.vcur) + (int64_t)kvh * hs + i;
        u64 w = tag_load(p);
        unsigned spins = 0;
        while (!tag_is(w, e_in)) {
            if (++spins > a.spin_limit ||
                ((spins & 63) == 0 && __hip_atomic_load(a.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                ok = false;
                break;
            }
            w = tag_load(p);
        }
        if (which == 0)
            s_q[i] = (double)tag_val(w);
        else if (which == 1)
            s_kcur[i] = tag_val(w);
        else
            s_vcur[i] = tag_val(w);
    }
    if (tid == 0) s_flag = 0;
    __syncthreads();
    if (!ok) s_flag = 1;
    __syncthreads();
    if (s_flag) {
        if (tid == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return false;
    }
    ATL();
    const float scale = sqrtf((float)hs);
    float mx = -INFINITY;
    // scores: thread = (timestep tl of a block of 256, quarter of the head dimension); the quarter's
    // 16-byte loads are all in flight at once; quarters are added in order (fp64)
    {
        const int tl = tid & 255, part = tid >> 8, per = hs >> 4;  // hs is a multiple of 16, at most 128
        double *s_sp = s_r;                                        // [4][256]
        for (int t0 = 0; t0 < np; t0 += 256) {
            const int t = t0 + tl;
            double acc = 0.0;
            if (t < np) {
                if (t == pos) {
                    for (int i = 4 * part * per; i < 4 * (part + 1) * per; i++) acc = fma(s_q[i], (double)s_kcur[i], acc);
                } else {
                    const float4 *kp = (const float4 *)kc + ((int64_t)kvh * (hs >> 2) + part * per) * seq_len + t;
                    float4 kv[8];
#pragma unroll
                    for (int u = 0; u < 8; u++)
                        if (u < per) kv[u] = kp[(int64_t)u * seq_len];
#pragma unroll
                    for (int u = 0; u < 8; u++)
                        if (u < per) {
                            const double *qq = s_q + 4 * (part * per + u);
                            acc = fma(qq[0], (double)kv[u].x, acc);
                            acc = fma(qq[1], (double)kv[u].y, acc);
                            acc = fma(qq[2], (double)kv[u].z, acc);
                            acc = fma(qq[3], (double)kv[u].w, acc);
                        }
                }
            }
            s_sp[part * 256 + tl] = acc;
            __syncthreads();
            if (part == 0 && t < np) {
                const double v = ((s_sp[tl] + s_sp[256 + tl]) + s_sp[512 + tl]) + s_sp[768 + tl];
                const float sc = (float)v / scale;
                s_att[t] = sc;
                mx = fmaxf(mx, sc);
            }
            __syncthreads();
        }
    }
    ATL();
    mx = block_max_f32(mx, s_redf);
    double sum = 0.0;
    for (int t = tid; t < np; t += blockDim.x) {
        const float e = (float)exp((double)(s_att[t] - mx));
        s_att[t] = e;
        sum += (double)e;
    }
    const float sf = (float)block_sum_f64(sum, s_red);
    for (int t = tid; t < np; t += blockDim.x) s_p[t] = (double)(s_att[t] / sf);
    __syncthreads();
    ATL();
    // values: thread = (16-byte group i4 of the head dimension, timestep group), up to eight loads in
    // flight; the groups of one wavefront are folded with lane exchanges, the rest through LDS
    const int n4 = hs >> 2;         // a power of two (hs 32, 64, 128)
    const int ngrp = blockDim.x / n4;
    {
        const int i4 = tid & (n4 - 1), grp = tid / n4;
        const float4 *vp = (const float4 *)(vc + (int64_t)kvh * seq_len * hs) + i4;
        double acc[4] = {0.0, 0.0, 0.0, 0.0};
        for (int t0 = grp; t0 < np; t0 += 8 * ngrp) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int t = t0 + u * ngrp;
                v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (t < pos) v[u] = vp[(int64_t)t * n4];
                else if (t == pos) v[u] = *(const float4 *)(s_vcur + 4 * i4);
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int t = t0 + u * ngrp;
                if (t < np) {
                    const double p = s_p[t];
                    acc[0] = fma(p, (double)v[u].x, acc[0]);
                    acc[1] = fma(p, (double)v[u].y, acc[1]);
                    acc[2] = fma(p, (double)v[u].z, acc[2]);
                    acc[3] = fma(p, (double)v[u].w, acc[3]);
                }
            }
        }
        for (int off = n4; off < 64; off <<= 1)
#pragma unroll
            for (int c = 0; c < 4; c++) acc[c] += __shfl_xor(acc[c], off, WAVE);
        if ((tid & 63) < n4) {
            const int wv = tid >> 6;
#pragma unroll
            for (int c = 0; c < 4; c++) s_r[wv * hs + 4 * i4 + c] = acc[c];
        }
    }
    __syncthreads();
    ATL();
    if (tid < hs) {
        double acc = 0.0;
        for (int k = 0; k < FLOW_NW; k++) acc += s_r[k * hs + tid];
        tag_store(a.xb + (int64_t)h * hs + tid, (float)acc, e_out);
    }
    __syncthreads();
    return true;
}

// ------------------------------------------------------------------------------------------
// the kernel; gen0 = epoch of this launch's input (advances by 5 * n_layers + 2 per launch)
// ------------------------------------------------------------------------------------------
template <int T_CLS>
__global__ __launch_bounds__(1024) void flow_token_kernel(unsigned int gen0) {
    const FlowArgs &a = c_flow;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = blockIdx.x, nwg = gridDim.x;
    unsigned char *ring_base = s_ring + wave * (FLOW_D * FLOW_SLOT);

    Ring r;
    r.gptr = a.stream + a.wave_off[wg * FLOW_NW + wave];
    r.lds = (unsigned)(size_t)ring_base;
    r.issued = r.consumed = r.drain_mark = 0;
    r.iss_layer = 0;
    r.iss_kind = 0;
    r.iss_seq = 0;
    r.iss_left = flow_wave_pieces(a.qkv, wg, wave);
    ring_uniform(r);  // values that came through vector loads are the same on every lane: make them scalar
#pragma nounroll
    for (int k = 0; k < FLOW_D; k++) flow_issue_q4(r, a, ring_base, wg, wave, lane);

#ifdef L2H_TIMELINE
    int tl_n = 0;
#define FTL()                                                                                   \
    do {                                                                                        \
        if (a.timeline && tid == 0 && tl_n < 64) a.timeline[wg * 64 + tl_n++] = wall_clock64(); \
    } while (0)
#define FTLS()          \
    do {                \
        __syncthreads(); \
        FTL();          \
    } while (0)
#define FTLD()         \
    do {               \
        flow_drain(r); \
        FTL();         \
    } while (0)
#else
#define FTL()
#define FTLS()
#define FTLD()
#endif
    FTL();
#define LEAVE()        \
    do {               \
        flow_drain(r); \
        return;        \
    } while (0)

    // ---- this step's token, position and RoPE angles (reference src/inference.jl:122-127) ----
    const int pos = a.ctl->pos;
    const int tok = a.ctl->step < a.ctl->n_prompt ? a.prompt[a.ctl->step] : a.ctl->last_argmax;
    if (tid < (a.hs >> 1)) {
        float theta = 1.0f * (float)pos;
        for (int k = 0; k < tid; k++) theta *= a.theta_scale;
        s_rope[2 * tid] = (float)cos((double)theta);
        s_rope[2 * tid + 1] = (float)sin((double)theta);
    }
    const unsigned E0 = gen0;
    // the rows of x this workgroup adds to after wo (layer 0): straight from the embedding (:236)
    {
        const int lo = wg * a.wo.rpw, n = flow_n_local(a.wo, wg);
        if (tid < n) tag_store(a.x_a + lo + tid, dequant_elem(a.emb, tok, lo + tid), E0);
    }

    for (int l = 0; l < a.n_layers; l++) {
        const unsigned e_x = E0 + 5u * (unsigned)l;  // x entering the layer
        const unsigned e_q = e_x + 1, e_att = e_x + 2, e_wo = e_x + 3, e_w13 = e_x + 4, e_w2 = e_x + 5;
        // the four matvec phases of the layer share one copy of the streaming loop (the kernel must stay
        // small enough for the instruction cache):
        //   0  rmsnorm (:244), q, k, v (:247-249), rope (:255-256), cache append (:259-260)
        //   1  attention (:263-278) on workgroup h*stride + h%stride, then x += wo * xb (:281-284)
        //   2  rmsnorm (:287), w1, w3 (:291-292), SwiGLU (:295-299)
        //   3  x += w2 * hb (:302-305)
#pragma nounroll
        for (int kind = 0; kind < 4; kind++) {
            bool ok;
            ring_store(r);
            if (kind == 0) {
                const float *nw = a.rms_att + (int64_t)l * a.norm_stride;
                ok = l == 0 ? flow_stage<PRO_RMSNORM, true>(nullptr, 0, a.dim, nw, tok, 0)
                            : flow_stage<PRO_RMSNORM, false>(a.x_a, e_x, a.dim, nw, tok, FLOW_FILL);
            } else if (kind == 1) {
                const int stride = nwg / a.n_heads;
                const int h = wg / stride;
                if (h < a.n_heads && wg % stride == h % stride)
                    if (!uni(flow_attention(l, h, pos, e_q, e_att))) LEAVE();
                FTL();
                ok = flow_stage<PRO_QUANT, false>(a.xb, e_att, a.dim, nullptr, tok, FLOW_FILL);
            } else if (kind == 2) {
                ok = flow_stage<PRO_RMSNORM, false>(a.x_b, e_wo, a.dim, a.rms_ffn + (int64_t)l * a.norm_stride, tok, FLOW_FILL);
            } else {
                ok = flow_stage<PRO_QUANT, false>(a.hb, e_w13, a.hidden, nullptr, tok, FLOW_FILL);
            }
            ring_load(r);
            if (!uni(ok)) LEAVE();
            FTL();
            const FlowGeom g = flow_geom(a, kind);
            // the row of x this thread adds to after wo / w2: fetched now, used after the loop
            u64 oldw = 0;
            if ((kind & 1) && tid < flow_n_local(g, wg)) oldw = tag_load((kind == 1 ? a.x_a : a.x_b) + wg * g.rpw + tid);
            FTLD();
            flow_loop_q4(g, r, ring_base, wg, 4 * l + kind);
            FTL();
            FTLS();
            if (kind == 0)
                flow_finish_qkv(l, wg, pos, e_q);
            else if (kind == 1)
                flow_finish_resid(1, wg, oldw, e_x, e_wo);
            else if (kind == 2)
                flow_finish_w13(wg, e_w13);
            else
                flow_finish_resid(3, wg, oldw, e_wo, e_w2);
            FTL();
        }
    }

    // ---- final rmsnorm (:309) + classifier (:312); the ring restarts on the classifier's pieces ----
    const unsigned e_fin = E0 + 5u * (unsigned)a.n_layers, e_cls = e_fin + 1;
    flow_drain(r);
    r.issued = r.consumed = r.drain_mark = 0;
    r.iss_layer = a.n_layers;  // the layer phases are over: flow_issue_q4 fetches while iss_left lasts
    r.iss_left = flow_wave_pieces(a.cls, wg, wave);
    ring_uniform(r);
    if (T_CLS == L2H_TYPE_Q6_K) {
        for (int k = 0; k < FLOW_Q6_D; k++) flow_issue_q6(r, ring_base, lane);
    } else {
        for (int k = 0; k < FLOW_D; k++) flow_issue_q4(r, a, ring_base, wg, wave, lane);
    }
    if (!uni(flow_stage<PRO_RMSNORM, false>(a.x_a, e_fin, a.dim, a.rms_final, tok, 0))) LEAVE();
    if (T_CLS == L2H_TYPE_Q6_K)
        flow_loop_q6(a.cls, r, ring_base, wg);
    else
        flow_loop_q4(a.cls, r, ring_base, wg, -1);
    flow_finish_cls(wg, e_cls);
    flow_drain(r);
    if (wg == 0) flow_pick_token(nwg, e_cls);
#undef LEAVE
}

// ------------------------------------------------------------------------------------------
// building the streams (once per model)
// ------------------------------------------------------------------------------------------
// bytes a wavefront's stream holds for one layer, and before phase `kind` within a layer
__host__ __device__ inline int64_t flow_layer_bytes(const FlowGeom *g4, int wg, int wave, int upto) {
    int64_t b = 0;
    for (int k = 0; k < upto; k++) b += (int64_t)flow_wave_pieces(g4[k], wg, wave) * FLOW_SLOT;
    return b;
}

struct FlowRepackArgs {
    unsigned char *stream;
    const int64_t *wave_off;
    FlowGeom g4[4];
    FlowGeom cls;
    int kind;  // 0..3 layer phases, 4 classifier
    int layer, n_layers;
    DevTensor w[3];
    int dim, kv_dim, hs, neox;
};

// one 64-thread workgroup copies one piece from the per-tensor field streams into its place
__global__ __launch_bounds__(64) void flow_repack_kernel(FlowRepackArgs p) {
    const FlowGeom g = p.kind == 4 ? p.cls : (p.kind == 0 ? p.g4[0] : (p.kind == 1 ? p.g4[1] : (p.kind == 2 ? p.g4[2] : p.g4[3])));
    const int per_wg = g.rpw * g.ppr;
    const int wg = blockIdx.x / per_wg, j = blockIdx.x % per_wg;
    if (j >= flow_n_local(g, wg) * g.ppr) return;
    const int np = flow_n_local(g, wg) * g.ppr, base = np / FLOW_NW, rem = np % FLOW_NW;
    const int wave = j < rem * (base + 1) ? j / (base + 1) : rem + (j - rem * (base + 1)) / base;
    const int idx = j - flow_wave_start(g, wg, wave);
    const int L = wg * g.rpw + j / g.ppr;
    const int part = j % g.ppr;
    int seg, row32;
    flow_row_src(p.kind == 4 ? 1 : p.kind, L, p.dim, p.kv_dim, p.hs, p.neox, seg, row32);
    const int64_t row = row32;
    const DevTensor &t = seg == 0 ? p.w[0] : (seg == 1 ? p.w[1] : p.w[2]);
    const int64_t layer_b = flow_layer_bytes(p.g4, wg, wave, 4);
    const int lane = threadIdx.x;
    if (t.type == L2H_TYPE_Q4_K) {
        const int64_t off = p.kind == 4 ? (int64_t)p.n_layers * layer_b
                                        : (int64_t)p.layer * layer_b + flow_layer_bytes(p.g4, wg, wave, p.kind);
        uint4 *dst = (uint4 *)(p.stream + p.wave_off[wg * FLOW_NW + wave] + off + (int64_t)idx * FLOW_SLOT);
        const int64_t blk0 = row * t.nb + part * 8;
        if (lane < 8) dst[lane] = flow_encode_hdr(t.hdr[blk0 + lane]);
        dst[8 + lane] = ((const uint4 *)(t.qs + blk0 * 128))[lane];
    } else {  // q6_K classifier
        const int64_t off = (int64_t)p.n_layers * layer_b;
        uint4 *dst = (uint4 *)(p.stream + p.wave_off[wg * FLOW_NW + wave] + off + (int64_t)idx * FLOW_Q6_PIECE);
        const int64_t blk0 = row * t.nb + part * 16;
        const uint4 *ql = (const uint4 *)(t.qs + blk0 * 128), *qh = (const uint4 *)(t.qh + blk0 * 64);
        dst[lane] = ql[lane];
        dst[64 + lane] = ql[64 + lane];
        dst[128 + lane] = qh[lane];
        if (lane < 16) dst[192 + lane] = ((const uint4 *)(t.sc6 + blk0 * 4))[lane];
        if (lane < 2) dst[208 + lane] = ((const uint4 *)(t.d6 + blk0))[lane];
    }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
static FlowGeom make_geom(int64_t n_rows, int64_t K, int type, int grid) {
    FlowGeom g{};
    g.n_rows = (int)n_rows;
    g.K = (int)K;
    int rpw = (int)((n_rows + grid - 1) / grid);
    rpw += rpw & 1;
    g.rpw = rpw;
    g.ppr = (int)(K / 256) / (type == L2H_TYPE_Q6_K ? 16 : 8);
    return g;
}

// Can the model run on this kernel?  q4_K layer matrices with input lengths that are multiples of
// 2048 (whole pieces per row), a q4_K or q6_K classifier (q6_K: multiples of 4096), and sizes that
// fit the kernel's LDS areas.  On success fills the geometry fields of `a` for a grid of `grid`.
bool k_flow_plan(FlowArgs &a, const int *layer_types, int n_layer_types, int cls_type, int grid, std::string *why) {
    auto no = [&](const char *m) {
        if (why) *why = m;
        return false;
    };
    for (int i = 0; i < n_layer_types; i++)
        if (layer_types[i] != L2H_TYPE_Q4_K) return no("layer matrices must be q4_K");
    if (cls_type != L2H_TYPE_Q4_K && cls_type != L2H_TYPE_Q6_K) return no("classifier must be q4_K or q6_K");
    if (a.dim % 2048 != 0 || a.hidden % 2048 != 0) return no("dim and hidden_dim must be multiples of 2048");
    if (cls_type == L2H_TYPE_Q6_K && a.dim % 4096 != 0) return no("a q6_K classifier needs dim to be a multiple of 4096");
    if (a.hidden > 14336 || a.dim > 14336) return no("input vectors longer than 14336");
    if (a.n_heads > grid || (a.hs != 32 && a.hs != 64 && a.hs != 128)) return no("head size must be 32, 64 or 128");
    const size_t att = (size_t)a.hs * 8 + (size_t)a.seq_len * 8 + (size_t)std::max(FLOW_NW * a.hs, 1024) * 8 +
                       (size_t)((a.seq_len + 3) & ~3) * 4 + (size_t)a.hs * 8;
    if (att > FLOW_ACT_BYTES) return no("sequence too long for the attention area");
    a.qkv = make_geom(a.dim + 2 * a.kv_dim, a.dim, L2H_TYPE_Q4_K, grid);
    a.wo = make_geom(a.dim, a.dim, L2H_TYPE_Q4_K, grid);
    a.w13 = make_geom(2 * (int64_t)a.hidden, a.dim, L2H_TYPE_Q4_K, grid);
    a.w2 = make_geom(a.dim, a.hidden, L2H_TYPE_Q4_K, grid);
    a.cls = make_geom(a.vocab, a.dim, cls_type, grid);
    const FlowGeom *gs[5] = {&a.qkv, &a.wo, &a.w13, &a.w2, &a.cls};
    for (const FlowGeom *g : gs)
        if (g->rpw > FLOW_MAX_ROWS || g->rpw * g->ppr > FLOW_MAX_PIECES) return no("too many rows per workgroup");
    if ((a.dim + 2 * a.kv_dim) % 2 != 0) return no("odd row count");
    return true;
}

// byte offset of every wavefront's stream (host array of grid*16 entries); returns the total
int64_t k_flow_offsets(const FlowArgs &a, int cls_type, int grid, std::vector<int64_t> &off) {
    const FlowGeom g4[4] = {a.qkv, a.wo, a.w13, a.w2};
    off.assign((size_t)grid * FLOW_NW, 0);
    int64_t total = 0;
    for (int wg = 0; wg < grid; wg++)
        for (int w = 0; w < FLOW_NW; w++) {
            off[(size_t)wg * FLOW_NW + w] = total;
            total += (int64_t)a.n_layers * flow_layer_bytes(g4, wg, w, 4);
            total += (int64_t)flow_wave_pieces(a.cls, wg, w) * (cls_type == L2H_TYPE_Q6_K ? FLOW_Q6_PIECE : FLOW_SLOT);
            total = (total + 255) & ~(int64_t)255;
        }
    return total + 4096;  // the last fetches of a stream may be issued past a workgroup's final piece: none are, but pad anyway
}

hipError_t k_flow_repack(hipStream_t s, const FlowArgs &a, unsigned char *stream, const int64_t *wave_off_dev, int kind,
                         int layer, const DevTensor *w, int nw, int grid) {
    FlowRepackArgs p{};
    p.stream = stream;
    p.wave_off = wave_off_dev;
    p.g4[0] = a.qkv;
    p.g4[1] = a.wo;
    p.g4[2] = a.w13;
    p.g4[3] = a.w2;
    p.cls = a.cls;
    p.kind = kind;
    p.layer = layer;
    p.n_layers = a.n_layers;
    for (int i = 0; i < nw; i++) p.w[i] = w[i];
    p.dim = a.dim;
    p.kv_dim = a.kv_dim;
    p.hs = a.hs;
    p.neox = a.neox;
    const FlowGeom &g = kind == 4 ? a.cls : p.g4[kind];
    hipLaunchKernelGGL(flow_repack_kernel, dim3((unsigned)(grid * g.rpw * g.ppr)), dim3(64), 0, s, p);
    return hipGetLastError();
}

// copies a model's arguments into the kernel's constant memory (stream-ordered, then waited for)
hipError_t k_flow_bind(hipStream_t s, const FlowArgs &a) {
    hipError_t e = hipMemcpyToSymbolAsync(HIP_SYMBOL(c_flow_raw), &a, sizeof(FlowArgs), 0, hipMemcpyHostToDevice, s);
    if (e != hipSuccess) return e;
    return hipStreamSynchronize(s);
}

hipError_t k_flow_launch(hipStream_t s, unsigned int gen0, int cls_type, int grid) {
    void *args[] = {&gen0};
    const void *fn = cls_type == L2H_TYPE_Q6_K ? (const void *)flow_token_kernel<L2H_TYPE_Q6_K>
                                               : (const void *)flow_token_kernel<L2H_TYPE_Q4_K>;
    return hipLaunchCooperativeKernel(fn, dim3(grid), dim3(1024), args, 0, s);
}
