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
//  * No grid barrier.  Activations that cross workgroups carry their own "ready": the long vectors that
//    every workgroup reads whole (residual stream, attention output, SwiGLU output) are bare fp32 words
//    in which a reserved NaN pattern means "not written yet" (see FLOW_EMPTY), the short ones (q, k, v of
//    the current position, the per-workgroup argmax keys) are 8-byte words {fp32 value, epoch tag}.  All
//    are written and read with device-scope relaxed atomics or their 16-byte equivalent; a consumer polls
//    until its words are there: data and "ready" arrive in one transaction.  Each buffer is rewritten (or
//    marked empty again) only two or more phases after its last read, and reaching a phase requires every
//    workgroup to have finished the phase before the previous one, so a word is never overwritten while
//    somebody may still want its old value.
//    The caller puts all these words into uncached device memory: a store there reaches a poller on another
//    XCD sooner than through the L2s.
//
//  Besides: a few pieces per phase travel through registers, requested while the phase waits for its
//  input (see flow_reg_pieces), and the attention is built for low latency (flow_attention_short).
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
#define FLOW_ACT_BYTES 28672
#define FLOW_MAX_PIECES 1024  // per workgroup and phase
#define FLOW_MAX_ROWS 512     // per workgroup and phase

typedef unsigned long long u64;
typedef unsigned int u32x4v __attribute__((ext_vector_type(4)));

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
__shared__ uint4 s_act[(FLOW_ACT_BYTES + 2048) / 16];  // (+ 2 KiB behind it: the last two of flow_stage's raw blocks)
#define s_part ((double *)((unsigned char *)s_act + 16384))
#define s_val ((float *)((unsigned char *)s_act + 16384 + FLOW_MAX_PIECES * 8))
__shared__ float s_rope[256];
__shared__ double s_red[16];
__shared__ float s_redf[16];
__shared__ int s_flag;
#ifdef L2H_TIMELINE
// profiling build: flow_stage's own stamps (thread 0 of one workgroup, one layer) go to a.timeline[s_tl_fine++]
__shared__ int s_tl_fine;
// ... and where lane 0 of every wavefront of that workgroup stamps the end of its streaming loop (-1: nowhere)
__shared__ int s_tl_wave;
#define STG()                                                                                          \
    do {                                                                                               \
        if (threadIdx.x == 0 && a.timeline && s_tl_fine >= 0) a.timeline[s_tl_fine++] = wall_clock64(); \
    } while (0)
#else
#define STG()
#endif
__shared__ __attribute__((aligned(16))) unsigned char s_sink[256];  // target of fetches made only to warm the L2
__shared__ int s_tok;  // the token of a launch's next step (flow_next_token)
// The rows of the residual stream x that this workgroup adds to after wo and after w2 (the same rows, the same threads:
// k_flow_plan checks it): thread t keeps its row's current value here, so that the addition needs no load of the word
// the thread itself published a phase ago.
#define FLOW_RESID_ROWS 64
__shared__ float s_resid[FLOW_RESID_ROWS];
#define FLOW_TOK_COPIES 8

__device__ __forceinline__ void tag_store(u64 *p, float v, unsigned epoch) {
    __hip_atomic_store(p, ((u64)epoch << 32) | (u64)__float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 tag_load(const u64 *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool tag_is(u64 w, unsigned epoch) { return (unsigned)(w >> 32) == epoch; }
__device__ __forceinline__ float tag_val(u64 w) { return __uint_as_float((unsigned)w); }
// The vectors that every workgroup reads whole — the residual stream x, the attention output, the SwiGLU
// output — travel as bare fp32 words, half the bytes of tagged ones.  A word that has not been written
// holds FLOW_EMPTY, a NaN pattern that no arithmetic here produces (a result that happens to have it is
// stored as the default NaN).  Each comes in two buffers used in turn (x: layer input / after attention;
// the others: by the low bit of the phase's epoch, which consecutive layers, and the last layer of one
// launch and the first of the next, differ in), and whoever writes word i of one buffer puts FLOW_EMPTY
// back into word i of the other: every reader of that one finished with it a phase ago, and it is the
// same thread that writes word i of either.
#define FLOW_EMPTY 0xFFFFFFFFu
// A barrier that orders the workgroup's LDS traffic only.  __syncthreads() also waits for every request to memory that
// the wavefront has under way, the fetches into its ring included; nothing that passes between the wavefronts of a
// workgroup where this one stands goes through memory.
// (In the staging function and the layer epilogues: 769 against 766 tok/s on the headline model.)
__device__ __forceinline__ void flow_barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ unsigned bare_load(const unsigned *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void bare_store(unsigned *p, unsigned v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// the word that stands for v
__device__ __forceinline__ unsigned bare_of(float v) {
    const unsigned u = __float_as_uint(v);
    return u == FLOW_EMPTY ? 0x7FC00000u : u;
}

__host__ __device__ inline int flow_n_local(const FlowGeom &g, int wg) {
    const int lo = wg * g.rpw;
    const int hi = lo + g.rpw < g.n_rows ? lo + g.rpw : g.n_rows;
    return hi > lo ? hi - lo : 0;
}
// Rows that end in the middle of a piece (FlowGeom::ppr == 0) come in pairs of flow_half() pieces: rpw and n_rows are
// even.  H = false: the caller knows that the geometry has none (kernels that are not built for them do not look).
template <bool H = true>
__host__ __device__ inline int flow_half(const FlowGeom &g) {
    return H && g.ppr == 0 ? g.K >> 10 : 0;
}
// pieces of a workgroup's rows
template <bool H = true>
__host__ __device__ inline int flow_wg_pieces(const FlowGeom &g, int wg) {
    const int n = flow_n_local(g, wg), h = flow_half<H>(g);
    return h ? (n >> 1) * h : n * g.ppr;
}
// the first logical row that piece j of a workgroup holds super-blocks of
__host__ __device__ inline int flow_piece_row(const FlowGeom &g, int j) {
    const int h = flow_half(g);
    return h ? 2 * (j / h) : j / g.ppr;
}
// pieces of a workgroup with a full share of rows
__host__ __device__ inline int flow_wg_capacity(const FlowGeom &g) {
    const int h = flow_half(g);
    return h ? (g.rpw >> 1) * h : g.rpw * g.ppr;
}
// pieces of workgroup wg that wavefront `wave` takes: a contiguous run of the workgroup's pieces
// (consecutive pieces of a row stay in one wavefront where possible), the first np % 16 wavefronts
// one piece longer than the rest
template <bool H = true>
__host__ __device__ inline int flow_wave_pieces(const FlowGeom &g, int wg, int wave) {
    const int np = flow_wg_pieces<H>(g, wg);
    return np / FLOW_NW + (wave < np % FLOW_NW ? 1 : 0);
}
template <bool H = true>
__host__ __device__ inline int flow_wave_start(const FlowGeom &g, int wg, int wave) {
    const int np = flow_wg_pieces<H>(g, wg);
    const int base = np / FLOW_NW, rem = np % FLOW_NW;
    return wave * base + (wave < rem ? wave : rem);
}
// While a phase waits for its input vector the memory system is idle and the ring is full.  At the start
// of that wait a wavefront therefore requests the last FLOW_R pieces of its run for the phase into
// registers; the ring's stream passes over them (they sit in a part of the wavefront's stream of their
// own).  That moves their share of the HBM time out of the loops; the price is that the wait's first poll
// returns after them (loads return in order), which is why there are only a few: one is the best count now,
// two were while the waits themselves took longer.
#ifndef FLOW_R
#define FLOW_R 1
#endif
template <bool H = true>
__host__ __device__ inline int flow_reg_pieces(const FlowGeom &g, int wg, int wave) {
    const int cnt = flow_wave_pieces<H>(g, wg, wave);
    return cnt < FLOW_R ? cnt : FLOW_R;
}
// pieces of a layer phase that go through the ring
template <bool H = true>
__host__ __device__ inline int flow_ring_pieces(const FlowGeom &g, int wg, int wave) {
    return flow_wave_pieces<H>(g, wg, wave) - flow_reg_pieces<H>(g, wg, wave);
}

// logical row L of a phase -> (tensor of the phase, row in it).  Logical rows put the two rows an
// epilogue combines next to each other: (w1 row u, w3 row u) and the two halves of a RoPE pair.
// (any_hs: head sizes that are not powers of two)
__host__ __device__ inline void flow_row_src(int kind, int L, int dim, int kv_dim, int hs, int neox, int &seg,
                                             int &row, bool any_hs = false) {
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
        const int e = any_hs ? row % hs : row & (hs - 1);  // (a power of two unless any_hs)
        row = (row - e) + (e >> 1) + ((e & 1) ? (hs >> 1) : 0);
    }
}

// ------------------------------------------------------------------------------------------
// the ring of one wavefront
// ------------------------------------------------------------------------------------------
// A wavefront's stream is one contiguous run of pieces in the order it uses them, so the fetch side
// needs no notion of phases: it keeps the ring full (issued - consumed == FLOW_D) until the stream
// ends, and the slot a piece is fetched into is always the slot that was just emptied.
struct Ring {
    const unsigned char *gptr;  // next byte of the stream to fetch
    unsigned lds;               // LDS byte address of slot 0
    int off;                    // byte offset in the ring of the slot to use (and then refill) next
    int issued, consumed;       // pieces fetched / used so far
    int drain_mark;             // pieces known to have landed (issued before the last full wait)
    int left;                   // pieces of the stream not fetched yet
};

// Headers inside the streams carry the twelve 6-bit scale bytes of a q4_K super-block (reference
// src/kquants.jl:80-109) regrouped so that a lane finds the four values of its sub-block pair j in
// one 24-bit field f_j = sc(2j) | sc(2j+1) << 6 | m(2j) << 12 | m(2j+1) << 18:
//   bytes 0-3 = d | dmin << 16;  bytes 4 + 3j .. 6 + 3j = f_j (little endian), j = 0..3.
// A lane reads the four bytes at 4 + 3j (not aligned; the byte above its field is ignored).
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
    return make_uint4(hdr.x, f[0] | (f[1] & 0xFF) << 24, (f[1] >> 8) | (f[2] & 0xFFFF) << 16, (f[2] >> 16) | f[3] << 8);
}
// field j out of a whole header (j is fixed per lane: the selects use lane-constant conditions).  LDS
// reads that are not aligned are slow, so a lane reads the 16 bytes and shifts its field down.
__device__ __forceinline__ uint32_t flow_field_of(const uint4 hdr, int j) {
    const uint32_t lo = j < 2 ? hdr.y : (j == 2 ? hdr.z : hdr.w), hi = j == 1 ? hdr.z : hdr.w;
    return __builtin_amdgcn_alignbit(hi, lo, (24 * j) & 31);
}
__device__ __forceinline__ void flow_decode_field(uint32_t f, int &sc_a, int &sc_b, int &m_a, int &m_b) {
    sc_a = (int)(f & 63);
    sc_b = (int)((f >> 6) & 63);
    m_a = (int)((f >> 12) & 63);
    m_b = (int)((f >> 18) & 63);
}

// geometry of layer phase `kind`, field by field (scalar selects of scalar loads)
// (HALF: only a kernel built for rows that end inside a piece looks at that field; for the others it is a constant zero)
template <bool HALF = false>
__device__ __forceinline__ FlowGeom flow_geom(const FlowArgs &a, int kind) {
    FlowGeom g;
    g.n_rows = kind == 0 ? a.qkv.n_rows : (kind == 1 ? a.wo.n_rows : (kind == 2 ? a.w13.n_rows : a.w2.n_rows));
    g.rpw = kind == 0 ? a.qkv.rpw : (kind == 1 ? a.wo.rpw : (kind == 2 ? a.w13.rpw : a.w2.rpw));
    g.ppr = kind == 0 ? a.qkv.ppr : (kind == 1 ? a.wo.ppr : (kind == 2 ? a.w13.ppr : a.w2.ppr));
    g.K = 0;
    if (HALF) g.K = kind == 0 ? a.qkv.K : (kind == 1 ? a.wo.K : (kind == 2 ? a.w13.K : a.w2.K));
    return g;
}

// the ring's bookkeeping is the same on every lane: keep it in scalar registers
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ unsigned uni(unsigned v) { return (unsigned)__builtin_amdgcn_readfirstlane((int)v); }
// (arguments of a function that is not inlined arrive in vector registers even when every lane holds
// the same value; made scalar on entry, the arithmetic on them is scalar too)
template <typename T>
__device__ __forceinline__ T *uni(T *p) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = uni((unsigned)v), hi = uni((unsigned)(v >> 32));
    return (T *)(((unsigned long long)hi << 32) | lo);
}

__device__ __forceinline__ void ring_uniform(Ring &r) {
    const unsigned long long p = (unsigned long long)r.gptr;
    const unsigned lo = (unsigned)uni((int)(unsigned)p), hi = (unsigned)uni((int)(unsigned)(p >> 32));
    r.gptr = (const unsigned char *)(((unsigned long long)hi << 32) | lo);
    r.lds = (unsigned)uni((int)r.lds);
    r.off = uni(r.off);
    r.issued = uni(r.issued);
    r.consumed = uni(r.consumed);
    r.drain_mark = uni(r.drain_mark);
    r.left = uni(r.left);
}

#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))

// fetch the next q4_K piece of the stream into the ring slot at byte offset `off`
__device__ __forceinline__ void flow_fetch_q4(const unsigned char *g, unsigned char *ring_base, int off, int lane) {
    // the instruction's immediate offset applies to both the global and the LDS address
    unsigned char *slot = ring_base + off;
    const unsigned char *gl = g + lane * 16;
    if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 0, 2);
    __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 128, 2);
}

// fill the ring from empty or part-empty: pieces go to the slots after the ones in use
__device__ __forceinline__ void flow_top_up_q4(Ring &r, unsigned char *ring_base, int lane) {
#pragma nounroll
    for (int k = 0; k < FLOW_D; k++) {
        const int held = uni(r.issued) - uni(r.consumed);
        if (held >= FLOW_D || uni(r.left) <= 0) break;
        int o = uni(r.off) + held * FLOW_SLOT;
        if (o >= FLOW_D * FLOW_SLOT) o -= FLOW_D * FLOW_SLOT;
        flow_fetch_q4(r.gptr, ring_base, o, lane);
        r.gptr += FLOW_SLOT;
        r.issued++;
        r.left--;
    }
}

// everything this wavefront has fetched so far has landed
__device__ __forceinline__ void flow_drain(Ring &r) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    r.drain_mark = r.issued;
}

// ------------------------------------------------------------------------------------------
// staging: the input vector of a phase -> q8_K in this workgroup's LDS.  Source: tagged words of
// epoch `epoch`, or (EMB) the embedding row of `tok`.  Returns false if the wait gave up.
// Separate functions (not inlined): the kernel stays small enough to keep its state in registers.
// ------------------------------------------------------------------------------------------
// Polls of activation words.  A lane's four words are one contiguous, 16-byte aligned run: fetched with
// 16-byte loads (agent scope; every aligned 4- or 8-byte word of such a load is read whole), so that one
// instruction asks for whole cache lines.  The loads and the wait for them are ONE asm statement: the
// compiler believes an asm's outputs valid as soon as the statement ends and may copy them at once, so no
// statement may end with a load still under way.
#define POLL_BARE1(w0, p0) \
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "+v"(w0) : "v"(p0) : "memory")
#define POLL_BARE2(w0, w1, p0, p1)                                                                                    \
    asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %3, off sc1\n\ts_waitcnt vmcnt(0)" \
                 : "+v"(w0), "+v"(w1)                                                                                 \
                 : "v"(p0), "v"(p1)                                                                                   \
                 : "memory")
#define POLL_BARE3(w0, w1, w2, p0, p1, p2)                                                                 \
    asm volatile("global_load_dwordx4 %0, %3, off sc1\n\tglobal_load_dwordx4 %1, %4, off sc1\n\t"         \
                 "global_load_dwordx4 %2, %5, off sc1\n\ts_waitcnt vmcnt(0)"                               \
                 : "+v"(w0), "+v"(w1), "+v"(w2)                                                            \
                 : "v"(p0), "v"(p1), "v"(p2)                                                               \
                 : "memory")
#define POLL_BARE4(w0, w1, w2, w3, p0, p1, p2, p3)                                                         \
    asm volatile("global_load_dwordx4 %0, %4, off sc1\n\tglobal_load_dwordx4 %1, %5, off sc1\n\t"         \
                 "global_load_dwordx4 %2, %6, off sc1\n\tglobal_load_dwordx4 %3, %7, off sc1\n\ts_waitcnt vmcnt(0)" \
                 : "+v"(w0), "+v"(w1), "+v"(w2), "+v"(w3)                                                  \
                 : "v"(p0), "v"(p1), "v"(p2), "v"(p3)                                                      \
                 : "memory")

// SRC: where the input comes from
#define SRC_EMB 0     // the embedding row of `tok`
#define SRC_BARE 2    // fp32 words; a word is there when it is not FLOW_EMPTY
#define FULL(V_) (V_.x != FLOW_EMPTY && V_.y != FLOW_EMPTY && V_.z != FLOW_EMPTY && V_.w != FLOW_EMPTY)
// Four q8_K blocks per wavefront throughout (q8k_quantize_rows16): a block per row of 16 lanes, a group of 16 values per
// lane.  With a block per wavefront — sixteen wavefronts, four to a SIMD, each through its own chain of reductions and
// divisions for 256 values — the 56 blocks of the hidden vector took 2.4 us of every workgroup's vector pipes, most of it
// after the last word had arrived, and the 16 blocks of a dim-long vector 1.3 us.
//
// A vector that is only quantised (attention output, SwiGLU output): wavefront w waits for blocks 4w .. 4w+3 itself, a
// lane for its 16 words (four 16-byte loads), and quantises them when all are there; one barrier.
//
// A vector that is normalised first (the embedding and norm weights come with dim <= 4096 only: at most 16 blocks) is
// waited for by all sixteen wavefronts, a block each, which also form the sum of squares; its raw values then go through
// LDS to the first four wavefronts, which normalise and quantise.  Block b waits in the part of the activation area
// that nothing else uses while a dim-long vector is staged — except that the last block of each of the four wavefronts
// waits where that same wavefront's quants go (it reads before it writes), and the last two of the others behind the
// activation area.
template <int PRO, int SRC>
__device__ __noinline__ bool flow_stage(const void *src, int K, const float *normw, int tok) {
    src = uni(src), K = uni(K), normw = uni(normw), tok = uni(tok);
    const FlowArgs &a = c_flow;
    int8_t *s_qs = (int8_t *)s_act;
    int16_t *s_bs = (int16_t *)(s_qs + 14336);
    float *s_d = (float *)(s_qs + 14336 + 1792);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nb = K >> 8;
    constexpr bool rms = PRO == PRO_RMSNORM;
    static_assert(rms || SRC == SRC_BARE, "a vector that is only quantised arrives as bare words");
    const int row_b = 4 * wave + (lane >> 4), g16 = lane & 15;  // block and group of this lane where a row is a block
    const bool there = row_b < nb;  // (a row without a block works on block 0's numbers and stores nothing)
    bool ok = true;
    STG();  // entered
    auto quads_store = [&](const float (&v)[16]) {
        q8k_u32x4 packed;
        int bsum;
        float d;
        q8k_quantize_rows16(v, packed, bsum, d);
        if (there) {
            ((q8k_u32x4 *)s_qs)[16 * row_b + g16] = packed;
            s_bs[16 * row_b + g16] = (int16_t)bsum;
            if (g16 == 0) s_d[row_b] = d;
        }
    };
    if constexpr (!rms) {
        if (4 * wave < nb) {
            u32x4v w0 = {FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY}, w1 = w0, w2 = w0, w3 = w0;
            const unsigned *pb = (const unsigned *)src + 256 * (there ? row_b : 0) + 16 * g16;
            unsigned spins = 0;
            for (;;) {
                // (a lane that has all its words does not ask again: waiting for a slow producer costs little traffic)
                if (!(FULL(w0) && FULL(w1) && FULL(w2) && FULL(w3))) POLL_BARE4(w0, w1, w2, w3, pb, pb + 4, pb + 8, pb + 12);
                const bool all = FULL(w0) && FULL(w1) && FULL(w2) && FULL(w3);
                if (spins == 0) STG();  // the first poll is back
                if (__ballot(!all) == 0ull) break;
                if (++spins > a.spin_limit ||
                    ((spins & 63) == 0 && __hip_atomic_load(a.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                    ok = false;
                    break;
                }
            }
            STG();  // this wavefront's words are all there
            const u32x4v ws[4] = {w0, w1, w2, w3};
            float v[16];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                v[4 * q] = __uint_as_float(ws[q].x);
                v[4 * q + 1] = __uint_as_float(ws[q].y);
                v[4 * q + 2] = __uint_as_float(ws[q].z);
                v[4 * q + 3] = __uint_as_float(ws[q].w);
            }
            quads_store(v);
        }
        if (!ok) s_flag = 1;  // zero since the start of the kernel; a kernel that sets it ends
        STG();  // this wavefront's blocks are in LDS
        flow_barrier_lds();
        STG();  // everybody's
        if (s_flag) {
            if (threadIdx.x == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return false;
        }
        return true;
    } else {
        const bool mine = wave < nb;  // this wavefront waits for block `wave`
        float xv[4] = {0.f, 0.f, 0.f, 0.f};
        float nw16[16];
        auto raw_of = [&](int b) -> float * {
            const int w = b >> 2, r = b & 3, i = 3 * w + r;
            const int at = r == 3 ? 256 * w : (i < 10 ? 1024 + 256 * i : FLOW_ACT_BYTES / 4 + 256 * (i - 10));
            return (float *)s_act + at;
        };
        // the norm weights are requested before the wait for the input: their latency passes meanwhile
        if (wave < 4) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                // (a global load: through a plain pointer it would be a flat one, which the LDS waits below would wait for)
                typedef float f32x4v __attribute__((ext_vector_type(4)));
                const f32x4v t = *(const AS1 f32x4v *)(normw + 256 * (there ? row_b : 0) + 16 * g16 + 4 * q);
                nw16[4 * q] = t.x;
                nw16[4 * q + 1] = t.y;
                nw16[4 * q + 2] = t.z;
                nw16[4 * q + 3] = t.w;
            }
        }
        if (SRC == SRC_EMB) {
            if (mine)
#pragma unroll
                for (int k = 0; k < 4; k++) xv[k] = dequant_elem(a.emb, tok, 256 * wave + 4 * lane + k);
        } else if (mine) {
            unsigned spins = 0;
            u32x4v w0 = {FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY};
            const unsigned *pb = (const unsigned *)src + 256 * wave + 4 * lane;
            for (;;) {
                if (!FULL(w0)) POLL_BARE1(w0, pb);
                const bool all = FULL(w0);
                if (spins == 0) STG();  // the first poll is back
                if (__ballot(!all) == 0ull) break;
                if (++spins > a.spin_limit ||
                    ((spins & 63) == 0 && __hip_atomic_load(a.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                    ok = false;
                    break;
                }
            }
            STG();  // this wavefront's words are all there
            xv[0] = __uint_as_float(w0.x);
            xv[1] = __uint_as_float(w0.y);
            xv[2] = __uint_as_float(w0.z);
            xv[3] = __uint_as_float(w0.w);
        }
        if (!ok) s_flag = 1;
        {  // rmsnorm! (reference src/inference.jl:102-110)
            double acc = 0.0;
            if (mine) {
#pragma unroll
                for (int k = 0; k < 4; k++) acc = fma((double)xv[k], (double)xv[k], acc);
            }
            acc = wave_sum_f64_dpp(acc);
            if (lane == 0) s_red[wave] = acc;
            if (mine) *(float4 *)(raw_of(wave) + 4 * lane) = make_float4(xv[0], xv[1], xv[2], xv[3]);
        }
        flow_barrier_lds();
        STG();  // every wavefront's are
        if (s_flag) {
            if (threadIdx.x == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return false;
        }
        if (wave < 4) {
            double t = 0.0;
            for (int w = 0; w < FLOW_NW; w++) t += s_red[w];
            float ss = (float)t;
            ss /= (float)K;
            ss += 1e-5f;
            ss = 1.0f / sqrtf(ss);
            const float *xr = raw_of(there ? row_b : 0) + 16 * g16;
            float v[16];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 x4 = *(const float4 *)(xr + 4 * q);
                v[4 * q] = nw16[4 * q] * (ss * x4.x);
                v[4 * q + 1] = nw16[4 * q + 1] * (ss * x4.y);
                v[4 * q + 2] = nw16[4 * q + 2] * (ss * x4.z);
                v[4 * q + 3] = nw16[4 * q + 3] * (ss * x4.w);
            }
            quads_store(v);
        }
        STG();  // this wavefront's blocks are in LDS
        flow_barrier_lds();
        STG();  // everybody's
        return true;
    }
}
#undef FULL

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

// q4_term on operands that are already in registers: w the lane's 16 bytes of quants, xlo / xhi its 2 x 16
// activations, bs_a / bs_b their block sums, yd the activation block's scale
__device__ __forceinline__ double flow_q4_term(const uint4 w, uint32_t d_dmin, int sc_a, int sc_b, int m_a, int m_b,
                                               const uint4 xlo, const uint4 xhi, int bs_a, int bs_b, float yd) {
    int dot_a, dot_b;
    // (the first product of each sum in the three-operand form with a literal zero: no register to clear)
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(dot_a) : "v"(w.x & 0x0F0F0F0Fu), "v"(xlo.x));
    dot_a = sdot4(w.y & 0x0F0F0F0Fu, xlo.y, dot_a);
    dot_a = sdot4(w.z & 0x0F0F0F0Fu, xlo.z, dot_a);
    dot_a = sdot4(w.w & 0x0F0F0F0Fu, xlo.w, dot_a);
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(dot_b) : "v"((w.x >> 4) & 0x0F0F0F0Fu), "v"(xhi.x));
    dot_b = sdot4((w.y >> 4) & 0x0F0F0F0Fu, xhi.y, dot_b);
    dot_b = sdot4((w.z >> 4) & 0x0F0F0F0Fu, xhi.z, dot_b);
    dot_b = sdot4((w.w >> 4) & 0x0F0F0F0Fu, xhi.w, dot_b);
    // every factor fits 24 bits (scales < 64, |dot| <= 16*15*127, |bsum| <= 16*127): full-rate multiplies
    const int i_sc = mad24(sc_a, dot_a, __mul24(sc_b, dot_b));
    const int i_min = mad24(m_a, bs_a, __mul24(m_b, bs_b));
    const float dy = half_bits_to_float((uint16_t)(d_dmin & 0xFFFF)) * yd;
    const float my = half_bits_to_float((uint16_t)(d_dmin >> 16)) * yd;
    double t = (double)dy * (double)i_sc;
    t = fma(-(double)my, (double)i_min, t);
    return t;
}

// The ring is kept full: as soon as a piece has been read into registers, the next piece of the stream
// is fetched into its slot, whichever phase that piece belongs to.  The loop's bookkeeping is a handful
// of scalars (the scalar unit is shared by the 16 wavefronts of the workgroup, so every scalar
// instruction per piece counts 16-fold):
//   held   pieces fetched and not yet used          ready   of those, known to have landed
//   off    byte offset of the slot to use next      left    pieces of the stream not fetched yet
template <int PIECE_BYTES, int DEPTH, int OPS>
struct RingLoop {
    const unsigned char *gp;
    int off, held, ready, left;
    __device__ __forceinline__ void begin(const Ring &r) {
        gp = r.gptr;
        off = uni(r.off);
        held = uni(r.issued) - uni(r.consumed);
        ready = uni(r.drain_mark) - uni(r.consumed);
        left = uni(r.left);
    }
    // the piece in slot `off` has landed when this returns
    __device__ __forceinline__ void wait() {
        if (ready == 0) {
            if (held == DEPTH) {  // the fetches return in order: all but the DEPTH-1 youngest are back
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS * (DEPTH - 1)) : "memory");
                ready = 1;
            } else {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                ready = held;
            }
        }
    }
    __device__ __forceinline__ void used() {
        ready--;
        held--;
    }
    __device__ __forceinline__ void fetched() {
        gp += PIECE_BYTES;
        left--;
        held++;
    }
    __device__ __forceinline__ void next_slot() {
        off += PIECE_BYTES;
        if (off == DEPTH * PIECE_BYTES) off = 0;
    }
    __device__ __forceinline__ void end(Ring &r, int n_used, int n_fetched) {
        r.gptr = gp;
        r.off = off;
        r.consumed += n_used;
        r.issued += n_fetched;
        r.drain_mark = r.consumed + ready;
        r.left = left;
    }
};

// the pieces of a phase that a wavefront holds in registers (see flow_reg_pieces): per lane its 16 bytes of
// quants, its super-block's d | dmin and the scale field of its sub-block pair
struct RegPieces {
    u32x4v q[FLOW_R];
    uint32_t dm[FLOW_R], f[FLOW_R];
};
// requests them: n pieces at p (every index below is a constant after unrolling: the arrays stay registers)
__device__ __forceinline__ void flow_reg_fetch(RegPieces &rp, const unsigned char *p, int n, int lane) {
    asm volatile("" : "+v"(lane));  // (the addresses below are computed here, not kept in registers across the kernel)
    const AS1 unsigned char *g = (const AS1 unsigned char *)p;  // (a global address: plain global loads)
    const AS1 unsigned char *ph = g + (lane >> 3) * 16, *pq = g + 128 + lane * 16;
    const int fo = 4 + 3 * ((lane & 7) >> 1);
#pragma unroll
    for (int i = 0; i < FLOW_R; i++)
        if (i < n) {
            rp.q[i] = __builtin_nontemporal_load((const AS1 u32x4v *)(pq + i * FLOW_SLOT));
            rp.dm[i] = *(const AS1 uint32_t *)(ph + i * FLOW_SLOT);
            uint32_t f;
            __builtin_memcpy(&f, ph + i * FLOW_SLOT + fo, 4);  // not aligned: one load all the same
            rp.f[i] = f;
        }
}
// After a wait for everything this wavefront has requested: the compiler is told, in its own terms, that
// the register pieces are there (it would otherwise wait for *all* outstanding requests, the ring's
// fetches included, at their first use inside the loop).
__device__ __forceinline__ void flow_reg_arrived(RegPieces &rp) {
#pragma unroll
    for (int i = 0; i < FLOW_R; i++) asm volatile("" : "+v"(rp.q[i]), "+v"(rp.dm[i]), "+v"(rp.f[i]));
}

// REGS: the wavefront's last n_reg pieces are in rp, the ones before them come through the ring
// QUARTERS: a row's sum is left as the four sums of 16 lanes each (s_part holds four doubles per piece)
// for flow_row_values to add, in the order in which wave_sum_f64_dpp would have: the loop is shorter by
// the lane reads and additions; the classifier has too many pieces per workgroup for that layout
template <bool REGS, bool QUARTERS>
__device__ __forceinline__ void flow_loop_q4(const FlowGeom &g, Ring &r, unsigned char *ring_base, int wg, const RegPieces &rp,
                                             int n_reg) {
    // (the lane number through an empty asm: what is derived from it is computed here, at every call, and
    // not once at the top of the kernel, where it would hold registers across all phases and be spilled)
    int lane = threadIdx.x & 63;
    asm volatile("" : "+v"(lane));
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ppr = uni(g.ppr);
    const int cnt = uni(flow_wave_pieces<false>(g, wg, wave)), start = uni(flow_wave_start<false>(g, wg, wave));
    RingLoop<FLOW_SLOT, FLOW_D, 2> q;
    q.begin(r);
    const int left0 = q.left;
    const unsigned rd_w = r.lds + lane * 16, rd_h = r.lds + (lane >> 3) * 16;
    const int pair = (lane & 7) >> 1;
    int part = uni(start % ppr);
    // this lane's activations for piece `part` of a row: block part * 8 + lane / 8, chunk lane % 8
    const int c8 = lane & 7;
    // LDS byte addresses of this lane's activations for piece 0 of a row (quants, block sums, scale); piece
    // `part` lies part * (2048, 256, 32) bytes further on
    const unsigned act = (unsigned)(size_t)s_act;
    const unsigned xq0 = act + (lane >> 3) * 256 + 64 * (c8 >> 1) + 16 * (c8 & 1);
    const unsigned xs0 = act + 14336 + 2 * ((lane >> 3) * 16 + 4 * (c8 >> 1) + (c8 & 1));
    const unsigned xd0 = act + 14336 + 1792 + 4 * (lane >> 3);
    int po = part * 32;  // piece index in units that scale to the three strides (2048, 256, 32 bytes)
    double *out = QUARTERS ? s_part + 4 * start + (lane >> 4) : s_part + start;
    double acc = 0.0;
    int k = cnt;  // pieces to go
    // a row's consecutive pieces are reduced over the lanes once; every piece has its own slot in s_part,
    // the run's total goes to its last piece and zero to the others (every lane stores the same word: no
    // lane-dependent branch in the loop)
#define FLOW_PIECE_DONE()             \
    do {                              \
        part++;                       \
        po += 32;                     \
        double v_ = 0.0;              \
        if (k == 1 || part == ppr) {  \
            v_ = QUARTERS ? row16_sum_f64_dpp(acc) : wave_sum_f64_dpp(acc); \
            acc = 0.0;                \
            po = 0;                   \
            part = 0;                 \
        }                             \
        *out = v_;                    \
        out += QUARTERS ? 4 : 1;      \
        k--;                          \
    } while (0)
    const int n_ring = REGS ? cnt - n_reg : cnt;
#pragma nounroll
    for (int i = 0; i < n_ring; i++) {
        q.wait();
        // all LDS reads of the piece in one statement the compiler does not look into: it would otherwise hold
        // the reads of the activation area back until every asynchronous fetch into the ring had landed
        uint4 w, hdr, xlo, xhi;
        int bs_a, bs_b;
        float yd;
        asm volatile(
            "ds_read_b128 %0, %7 offset:128\n\tds_read_b128 %1, %8\n\tds_read_b128 %2, %9\n\tds_read_b128 %3, %9 offset:32\n\t"
            "ds_read_i16 %4, %10\n\tds_read_i16 %5, %10 offset:4\n\tds_read_b32 %6, %11\n\ts_waitcnt lgkmcnt(0)"
            : "=&v"(w), "=&v"(hdr), "=&v"(xlo), "=&v"(xhi), "=&v"(bs_a), "=&v"(bs_b), "=&v"(yd)
            : "v"(rd_w + q.off), "v"(rd_h + q.off), "v"(xq0 + po * 64), "v"(xs0 + po * 8), "v"(xd0 + po)
            : "memory");
        const uint32_t d_dmin = hdr.x, field = flow_field_of(hdr, pair);
        q.used();
        if (q.left > 0) {  // the slot is free again
            flow_fetch_q4(q.gp, ring_base, q.off, lane);
            q.fetched();
        }
        q.next_slot();
        {
            int sc_a, sc_b, m_a, m_b;
            flow_decode_field(field, sc_a, sc_b, m_a, m_b);
            acc += flow_q4_term(w, d_dmin, sc_a, sc_b, m_a, m_b, xlo, xhi, bs_a, bs_b, yd);
        }
        FLOW_PIECE_DONE();
    }
    q.end(r, n_ring, left0 - q.left);
    if (REGS) {
#pragma unroll
        for (int i = 0; i < FLOW_R; i++)
            if (i < n_reg) {
                uint4 xlo, xhi;
                int bs_a, bs_b;
                float yd;
                asm volatile("ds_read_b128 %0, %5\n\tds_read_b128 %1, %5 offset:32\n\tds_read_i16 %2, %6\n\t"
                             "ds_read_i16 %3, %6 offset:4\n\tds_read_b32 %4, %7\n\ts_waitcnt lgkmcnt(0)"
                             : "=&v"(xlo), "=&v"(xhi), "=&v"(bs_a), "=&v"(bs_b), "=&v"(yd)
                             : "v"(xq0 + po * 64), "v"(xs0 + po * 8), "v"(xd0 + po)
                             : "memory");
                const uint4 w = make_uint4(rp.q[i].x, rp.q[i].y, rp.q[i].z, rp.q[i].w);
                int sc_a, sc_b, m_a, m_b;
                flow_decode_field(rp.f[i], sc_a, sc_b, m_a, m_b);
                acc += flow_q4_term(w, rp.dm[i], sc_a, sc_b, m_a, m_b, xlo, xhi, bs_a, bs_b, yd);
                FLOW_PIECE_DONE();
            }
    }
#undef FLOW_PIECE_DONE
#ifdef L2H_TIMELINE
    if (c_flow.timeline && lane == 0 && s_tl_wave >= 0) c_flow.timeline[s_tl_wave + wave] = wall_clock64();
#endif
}

// classifier pieces (q6_K): 16 super-blocks per piece, lane = (block lane/4, chunk lane%4); the ring
// holds two pieces
#define FLOW_Q6_D 2
__device__ __forceinline__ void flow_fetch_q6(const unsigned char *g, unsigned char *ring_base, int off, int lane) {
    unsigned char *slot = ring_base + off;
    const unsigned char *gl = g + lane * 16;
    __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 0, 2);
    __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 1024, 2);
    __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 2048, 2);
    if (lane < 16) __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 3072, 2);
    if (lane < 2) __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 3328, 2);
}

__device__ __forceinline__ void flow_top_up_q6(Ring &r, unsigned char *ring_base, int lane) {
#pragma nounroll
    for (int k = 0; k < FLOW_Q6_D; k++) {
        const int held = uni(r.issued) - uni(r.consumed);
        if (held >= FLOW_Q6_D || uni(r.left) <= 0) break;
        int o = uni(r.off) + held * FLOW_Q6_PIECE;
        if (o >= FLOW_Q6_D * FLOW_Q6_PIECE) o -= FLOW_Q6_D * FLOW_Q6_PIECE;
        flow_fetch_q6(r.gptr, ring_base, o, lane);
        r.gptr += FLOW_Q6_PIECE;
        r.issued++;
        r.left--;
    }
}

__device__ __forceinline__ void flow_loop_q6(const FlowGeom &g, Ring &r, unsigned char *ring_base, int wg) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ppr = uni(g.ppr);
    const int cnt = uni(flow_wave_pieces<false>(g, wg, wave)), start = uni(flow_wave_start<false>(g, wg, wave));
    const int b = lane >> 2, c = lane & 3, n = c >> 1, h = c & 1;
    const XLds x = flow_x();
    RingLoop<FLOW_Q6_PIECE, FLOW_Q6_D, 5> q;
    q.begin(r);
    const int left0 = q.left;
    int part = uni(start % ppr);
    double acc = 0.0;
#pragma nounroll
    for (int k = 0; k < cnt; k++) {
        q.wait();
        const unsigned slot = r.lds + (unsigned)q.off;
        Chunk<L2H_TYPE_Q6_K> ch;
        uint32_t d16;
        asm volatile("ds_read_b128 %0, %5\n\tds_read_b128 %1, %5 offset:32\n\tds_read_b128 %2, %6 offset:2048\n\t"
                     "ds_read_b32 %3, %7 offset:3072\n\tds_read_u16 %4, %8 offset:3328\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(ch.la), "=&v"(ch.lb), "=&v"(ch.qh), "=&v"(ch.sc), "=&v"(d16)
                     : "v"(slot + b * 128 + 64 * n + 16 * h), "v"(slot + b * 64 + 32 * n + 16 * h),
                       "v"(slot + (b * 4 + 2 * n + h) * 4), "v"(slot + b * 2)
                     : "memory");
        ch.d = d16;
        q.used();
        if (q.left > 0) {
            flow_fetch_q6(q.gp, ring_base, q.off, lane);
            q.fetched();
        }
        q.next_slot();
        acc += chunk_term<false>(ch, part * 64 + lane, x, nullptr, nullptr, 0);
        const bool last = k == cnt - 1 || part == ppr - 1;
        if (last) {
            const double v = wave_sum_f64_dpp(acc);
            if (lane == 0) s_part[start + k] = v;
            acc = 0.0;
        } else if (lane == 0) {
            s_part[start + k] = 0.0;
        }
        part = part == ppr - 1 ? 0 : part + 1;
    }
    q.end(r, cnt, left0 - q.left);
}

// ------------------------------------------------------------------------------------------
// typed pieces: models whose layer matrices are not all q4_K (reference src/kquants.jl:186-408)
// ------------------------------------------------------------------------------------------
// A piece is still eight super-blocks of one row, in one of three formats, each with a 16-byte tag at byte 128:
//   q4_K  1168 B: headers 128 (as above) | tag 16 | quants 1024
//   q5_K  1424 B: headers 128 | tag 16 | high bits 8 x 32 | quants 1024
//   q6_K  1696 B: scales 8 x 16 (bytes permuted: dword 2n+h of a super-block = the scales of its groups 0..3 at
//                 128n + 32g + 16h) | tag 16 | d 8 x 2 | high bits 8 x 64 | low nibbles 1024
// The ring has FLOWM_D slots of the largest size.  Every piece is fetched with two instructions (the first
// `head lanes` x 16 bytes, then 1024 bytes), so the count of fetches under way still tells which pieces have landed.
// The fetch side must know the format of a piece before it has seen it: byte 1 of a piece's tag holds the type of
// the piece FLOWM_D places further on in the wavefront's stream, which is the one that will be fetched into
// the slot this piece leaves (byte 0: the piece's own type); the types of a stream's first FLOWM_D pieces come
// from a table (FlowArgs::wave_types, two bits each).
#define FLOWM_SLOT 1696
#define FLOWM_D 4
__host__ __device__ inline int flowm_piece_bytes(int t) { return t == 0 ? 1168 : (t == 1 ? 1424 : 1696); }
__host__ __device__ inline int flowm_head_lanes(int t) { return t == 0 ? 9 : (t == 1 ? 25 : 42); }

struct MRing {
    const unsigned char *gptr;  // next byte of the stream to fetch
    unsigned lds;               // LDS byte address of slot 0
    int slot;                   // slot of the piece to use next
    int held, ready;            // pieces fetched and not yet used; of those, known to have landed
    int left;                   // pieces of the stream not fetched yet
    unsigned tq;                // types of the held pieces, two bits each, the next to use lowest
};

__device__ __forceinline__ void flowm_fetch(const unsigned char *g, unsigned char *slot, int t, int lane) {
    const int nb = uni(flowm_head_lanes(t));
    const unsigned char *gl = g + lane * 16;
    if (lane < nb) __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 0, 2);
    __builtin_amdgcn_global_load_lds((const AS1 void *)(gl + nb * 16), (AS3 void *)(slot + nb * 16), 16, 0, 2);
}

// the first pieces of a wavefront's stream
__device__ __forceinline__ void flowm_start(MRing &r, unsigned char *ring_base, unsigned types, int lane) {
    r.slot = 0;
    r.held = r.ready = 0;
    r.tq = 0;
#pragma unroll
    for (int j = 0; j < FLOWM_D; j++) {
        if (uni(r.left) > 0) {
            const int t = uni((int)((types >> (2 * j)) & 3u));
            flowm_fetch(r.gptr, ring_base + j * FLOWM_SLOT, t, lane);
            r.gptr += flowm_piece_bytes(t);
            r.tq |= (unsigned)t << (2 * j);
            r.held++;
            r.left--;
        }
    }
}

// the dword of a q6_K super-block's 16 permuted scale bytes that belongs to a lane: dword 2n + h (c8 = 4n + 2w + h)
__device__ __forceinline__ uint32_t flow_q6_scales(const uint4 sc, int c8) {
    const int dn = 2 * (c8 >> 2) + (c8 & 1);
    return dn == 0 ? sc.x : (dn == 1 ? sc.y : (dn == 2 ? sc.z : sc.w));
}

// q5_K: the q4_K term with bit 2j / 2j+1 of the lane's 16 high-bit bytes on top of the nibbles
__device__ __forceinline__ double flow_q5_term(const uint4 w, const uint4 qh, uint32_t d_dmin, int sc_a, int sc_b, int m_a,
                                               int m_b, int sa, const uint4 xlo, const uint4 xhi, int bs_a, int bs_b,
                                               float yd) {
    const int sb = sa + 1;
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
    const int i_sc = mad24(sc_a, dot_a, __mul24(sc_b, dot_b));
    const int i_min = mad24(m_a, bs_a, __mul24(m_b, bs_b));
    const float dy = half_bits_to_float((uint16_t)(d_dmin & 0xFFFF)) * yd;
    const float my = half_bits_to_float((uint16_t)(d_dmin >> 16)) * yd;
    double t = (double)dy * (double)i_sc;
    t = fma(-(double)my, (double)i_min, t);
    return t;
}

// q6_K: the lane's 16 bytes of low nibbles are ql[64n + 32w + 16h ..]: the low nibbles belong to group w (elements
// 128n + 32w + 16h ..), the high nibbles to group 2 + w (64 elements further on); bits 2g, 2g+1 of the lane's 16
// high-bit bytes qh[32n + 16h ..] complete group g (src/kquants.jl:333-336); q - 32 is folded in through the q8_K
// group sums.  scw = the four scales of groups 0..3, d16 the super-block's d.
__device__ __forceinline__ double flow_q6_term(const uint4 ql, const uint4 qh, uint32_t scw, uint32_t d16, int w32,
                                               const uint4 xlo, const uint4 xhi, int bs_lo, int bs_hi, float yd) {
    const int s_lo = 2 * w32, s_hi = 4 + 2 * w32;
    int d_lo = 0, d_hi = 0;
#define Q6LO(L, H) (((L)&0x0F0F0F0Fu) | ((((H) >> s_lo) & 0x03030303u) << 4))
#define Q6HI(L, H) ((((L) >> 4) & 0x0F0F0F0Fu) | ((((H) >> s_hi) & 0x03030303u) << 4))
    d_lo = sdot4(Q6LO(ql.x, qh.x), xlo.x, d_lo);
    d_lo = sdot4(Q6LO(ql.y, qh.y), xlo.y, d_lo);
    d_lo = sdot4(Q6LO(ql.z, qh.z), xlo.z, d_lo);
    d_lo = sdot4(Q6LO(ql.w, qh.w), xlo.w, d_lo);
    d_hi = sdot4(Q6HI(ql.x, qh.x), xhi.x, d_hi);
    d_hi = sdot4(Q6HI(ql.y, qh.y), xhi.y, d_hi);
    d_hi = sdot4(Q6HI(ql.z, qh.z), xhi.z, d_hi);
    d_hi = sdot4(Q6HI(ql.w, qh.w), xhi.w, d_hi);
#undef Q6LO
#undef Q6HI
    const int sc_lo = (int)(int8_t)((scw >> (8 * w32)) & 0xFF), sc_hi = (int)(int8_t)((scw >> (8 * (2 + w32))) & 0xFF);
    // |d - 32 bsum| < 2^18 and |scale| < 2^7: 24-bit (full-rate) multiplies are exact
    const int i_sc = mad24(sc_lo, d_lo - 32 * bs_lo, __mul24(sc_hi, d_hi - 32 * bs_hi));
    const float dy = half_bits_to_float((uint16_t)d16) * yd;
    return (double)dy * (double)i_sc;
}

// the streaming loop over typed pieces; partial sums as in flow_loop_q4<., true> (four doubles per piece)
template <bool HALF = false>
__device__ __forceinline__ void flow_loop_mixed(const FlowGeom &g, MRing &r, unsigned char *ring_base, int wg) {
    int lane = threadIdx.x & 63;
    asm volatile("" : "+v"(lane));
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // rows that end in the middle of a piece (flow_half() pieces per pair of rows): the lane's super-block is number
    // 8 part + blk of the pair's 2 nb_row; from nb_row on it belongs to the odd row
    const int half = uni(flow_half<HALF>(g)), unit = half ? half : uni(g.ppr), mid = half >> 1, nb_row = 4 * half;
    const int cnt = uni(flow_wave_pieces<HALF>(g, wg, wave)), start = uni(flow_wave_start<HALF>(g, wg, wave));
    int part = uni(start % unit);
    const int blk = lane >> 3, c8 = lane & 7;
    // q4_K / q5_K: sub-block pair c8 / 2, half c8 % 2.  q6_K: n = c8 / 4, w = (c8 / 2) % 2, h = c8 % 2.
    const int pair = c8 >> 1, w32 = (c8 >> 1) & 1;
    const unsigned act = (unsigned)(size_t)s_act;
    const unsigned x45 = act + blk * 256 + 64 * (c8 >> 1) + 16 * (c8 & 1);                           // then + 32
    const unsigned x6 = act + blk * 256 + 128 * (c8 >> 2) + 32 * ((c8 >> 1) & 1) + 16 * (c8 & 1);    // then + 64
    const unsigned bs45 = act + 14336 + 2 * (blk * 16 + 4 * (c8 >> 1) + (c8 & 1));                   // then + 4
    const unsigned bs6 = act + 14336 + 2 * (blk * 16 + 8 * (c8 >> 2) + 2 * ((c8 >> 1) & 1) + (c8 & 1));  // then + 8
    const unsigned xd0 = act + 14336 + 1792 + 4 * blk;
    const unsigned q5h = 144 + blk * 32 + 16 * (c8 & 1), q6h = 160 + blk * 64 + 32 * (c8 >> 2) + 16 * (c8 & 1);
    int po = part * 32;
    double *out = s_part + 4 * start + (lane >> 4);
    double acc = 0.0;
    int k = cnt;
    int slot = uni(r.slot), held = uni(r.held), ready = uni(r.ready), left = uni(r.left);
    unsigned tq = uni(r.tq);
    const unsigned char *gp = r.gptr;
#pragma nounroll
    for (int i = 0; i < cnt; i++) {
        if (ready == 0) {
            if (held == FLOWM_D) {  // the fetches return in order: all but the FLOWM_D - 1 youngest pieces are back
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (FLOWM_D - 1)) : "memory");
                ready = 1;
            } else {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                ready = held;
            }
        }
        const int t = (int)(tq & 3u);
        const unsigned sl = r.lds + (unsigned)(slot * FLOWM_SLOT);
        const bool six = t == 2;
        const unsigned a_w = sl + (t == 0 ? 144u : (t == 1 ? 400u : 672u)) + lane * 16;
        const unsigned a_h = sl + blk * 16;
        const unsigned a_q = sl + (six ? q6h : q5h);
        const unsigned back = (half && 8 * part + blk >= nb_row) ? (unsigned)(4 * nb_row) : 0u;  // (the odd row starts anew)
        const unsigned a_xlo = (six ? x6 : x45) + (po - back) * 64, a_xhi = a_xlo + (six ? 64u : 32u);
        const unsigned a_bsa = (six ? bs6 : bs45) + (po - back) * 8, a_bsb = a_bsa + (six ? 8u : 4u);
        const unsigned a_yd = xd0 + (po - back), a_tag = sl + 128, a_d = sl + 144 + 2 * blk;
        uint4 w, hdr, qh, xlo, xhi;
        int bs_a, bs_b;
        float yd;
        uint32_t tag, d16;
        // (one statement that the compiler does not look into, as in flow_loop_q4)
        asm volatile(
            "ds_read_b128 %0, %10\n\tds_read_b128 %1, %11\n\tds_read_b128 %2, %12\n\tds_read_b128 %3, %13\n\t"
            "ds_read_b128 %4, %14\n\tds_read_i16 %5, %15\n\tds_read_i16 %6, %16\n\tds_read_b32 %7, %17\n\t"
            "ds_read_b32 %8, %18\n\tds_read_u16 %9, %19\n\ts_waitcnt lgkmcnt(0)"
            : "=&v"(w), "=&v"(hdr), "=&v"(qh), "=&v"(xlo), "=&v"(xhi), "=&v"(bs_a), "=&v"(bs_b), "=&v"(yd), "=&v"(tag),
              "=&v"(d16)
            : "v"(a_w), "v"(a_h), "v"(a_q), "v"(a_xlo), "v"(a_xhi), "v"(a_bsa), "v"(a_bsb), "v"(a_yd), "v"(a_tag), "v"(a_d)
            : "memory");
        tq >>= 2;
        held--;
        ready--;
        if (left > 0) {  // the slot is free again: the piece FLOWM_D places on, whose type this piece's tag names
            const int nt = uni((int)((tag >> 8) & 3u));
            flowm_fetch(gp, ring_base + slot * FLOWM_SLOT, nt, lane);
            gp += flowm_piece_bytes(nt);
            tq |= (unsigned)nt << (2 * held);
            held++;
            left--;
        }
        slot = slot + 1 == FLOWM_D ? 0 : slot + 1;
        if (six) {
            acc += flow_q6_term(w, qh, flow_q6_scales(hdr, c8), d16, w32, xlo, xhi, bs_a, bs_b, yd);
        } else {
            int sc_a, sc_b, m_a, m_b;
            flow_decode_field(flow_field_of(hdr, pair), sc_a, sc_b, m_a, m_b);
            if (t == 1)
                acc += flow_q5_term(w, qh, hdr.x, sc_a, sc_b, m_a, m_b, 2 * pair, xlo, xhi, bs_a, bs_b, yd);
            else
                acc += flow_q4_term(w, hdr.x, sc_a, sc_b, m_a, m_b, xlo, xhi, bs_a, bs_b, yd);
        }
        // (as FLOW_PIECE_DONE of flow_loop_q4.)  Rows that end inside a piece: the upper half of the lanes goes over to
        // the odd row behind piece mid - 1 and the lower half behind piece mid, and each hands in its sums of the even row
        // there; what a piece's four quarter sums belong to is thereby fixed: to the even row up to the middle piece's
        // second quarter, to the odd row from its third.
        const int done = part;
        part++;
        po += 32;
        double v_ = 0.0;
        if constexpr (!HALF) {
            if (k == 1 || part == unit) {
                v_ = row16_sum_f64_dpp(acc);
                acc = 0.0;
                po = 0;
                part = 0;
            }
        } else {
            const bool last = k == 1 || part == unit;
            if (last || (half && (done == mid || done + 1 == mid))) {
                const double red = row16_sum_f64_dpp(acc);
                const bool mine = last || (done == mid ? lane < 32 : lane >= 32);
                v_ = mine ? red : 0.0;
                acc = mine ? 0.0 : acc;
                if (!half || part == unit) po = 0, part = 0;  // (a wavefront's last piece ends the loop)
            }
        }
        *out = v_;
        out += 4;
        k--;
    }
    r.gptr = gp;
    r.slot = slot;
    r.held = held;
    r.ready = ready;
    r.left = left;
    r.tq = tq;
}

// fp32 value of every local row: the pieces' partial sums added in order
template <bool QUARTERS>
__device__ __forceinline__ void flow_row_values(int n_local, int ppr) {
    __syncthreads();
    for (int lr = threadIdx.x; lr < n_local; lr += blockDim.x) {
        double v = 0.0;
        for (int p = 0; p < ppr; p++) {
            if (QUARTERS) {
                const double *q4 = s_part + 4 * (lr * ppr + p);
                v += (q4[0] + q4[1]) + (q4[2] + q4[3]);
            } else {
                v += s_part[lr * ppr + p];
            }
        }
        s_val[lr] = (float)v;
    }
    __syncthreads();
}

// the same for one row, straight from the partial sums (the layer epilogues: one barrier instead of two)
// (HALF: the geometry may have rows that end inside a piece; see flow_loop_mixed for what belongs to which row)
template <bool HALF = false>
__device__ __forceinline__ float flow_row_value4(int lr, int ppr, int half = 0) {
    if (HALF && half) {
        const int mid = half >> 1, odd = lr & 1;
        const double *h4 = s_part + 4 * (lr >> 1) * half;
        double v = 0.0;
        for (int p = odd ? mid + 1 : 0; p < (odd ? half : mid); p++) v += (h4[4 * p] + h4[4 * p + 1]) + (h4[4 * p + 2] + h4[4 * p + 3]);
        v += h4[4 * mid + 2 * odd] + h4[4 * mid + 2 * odd + 1];
        return (float)v;
    }
    const double *q4 = s_part + 4 * lr * ppr;
    double v = 0.0;
    // (the quarter sums of up to four pieces are read before any is added: one LDS latency per four pieces, not per piece)
    for (int p0 = 0; p0 < ppr; p0 += 4) {
        double q[4][4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (p0 + i < ppr) {
#pragma unroll
                for (int k = 0; k < 4; k++) q[i][k] = q4[4 * (p0 + i) + k];
            }
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (p0 + i < ppr) v += (q[i][0] + q[i][1]) + (q[i][2] + q[i][3]);
    }
    return (float)v;
}
// the value of the row next to this thread's (tid ^ 1), which that thread has just formed in the same way
__device__ __forceinline__ float flow_pair_value(float own) { return dpp_f32<DPP_QUAD_SWAP1>(own); }

// ---- epilogues -------------------------------------------------------------------------------
// (The layer epilogues are inlined: a function waits before it returns for its stores to be acknowledged,
// a round trip to memory that would stand between the publication of a phase's results and the next
// phase's requests.)
// rope! (reference src/inference.jl:112-157) and the cache append (:259-260)
template <bool ANY_HS = false, bool HALF = false>
__device__ __forceinline__ void flow_finish_qkv(int l, int wg, int pos, unsigned e_q) {
    l = uni(l), wg = uni(wg), pos = uni(pos), e_q = uni(e_q);
    const FlowArgs &a = c_flow;
    const int n_local = flow_n_local(a.qkv, wg);
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));  // (what derives from it is computed here and not kept across the kernel)
    flow_barrier_lds();
    if (tid >= n_local) return;
    const int L = wg * a.qkv.rpw + tid;
    int seg, row;
    flow_row_src(0, L, a.dim, a.kv_dim, a.hs, a.neox, seg, row, ANY_HS);
    // (rows come in pairs and a workgroup's run of them is even, so the partner's thread is here too)
    const float val = flow_row_value4<HALF>(tid, a.qkv.ppr, flow_half<HALF>(a.qkv)), other = flow_pair_value(val);
    const int hs_log = 31 - __builtin_clz(a.hs);  // (a power of two unless ANY_HS)
    const int hh = ANY_HS ? row / a.hs : row >> hs_log, e = ANY_HS ? row - hh * a.hs : row & (a.hs - 1);
    if (seg == 2) {
        if (ANY_HS && a.kv16) {  // fp16 cache: the row is rounded on append, and the attention sees the rounded value
            const __half hv = __float2half_rn(val);
            ((__half *)a.vc + (int64_t)l * a.cache_layer_elems)[((int64_t)hh * a.seq_len + pos) * a.hs + e] = hv;
            tag_store(a.vcur + row, __half2float(hv), e_q);
            return;
        }
        (a.vc + (int64_t)l * a.cache_layer_elems)[((int64_t)hh * a.seq_len + pos) * a.hs + e] = val;
        tag_store(a.vcur + row, val, e_q);
        return;
    }
    const int half = a.hs >> 1;
    const int i = a.neox ? (ANY_HS ? (e >= half ? e - half : e) : (e & (half - 1))) : (e >> 1);
    const float c = s_rope[2 * i], s = s_rope[2 * i + 1];
    const int rr = tid & 1;
    // complex product (re + i im)(c + i s), each of the four products rounded
    const float re = rr == 0 ? val : other, im = rr == 0 ? other : val;
    const float out = rr == 0 ? (re * c) - (im * s) : (re * s) + (im * c);
    if (seg == 0) {
        tag_store(a.q + row, out, e_q);
    } else if (ANY_HS && a.kv16) {
        const __half hv = __float2half_rn(out);
        ((__half *)a.kc + (int64_t)l * a.cache_layer_elems)[kc16_index(hh, e, pos, a.hs, a.seq_len)] = hv;
        tag_store(a.kcur + row, __half2float(hv), e_q);
    } else {
        (a.kc + (int64_t)l * a.cache_layer_elems)[(((int64_t)hh * (a.hs >> 2) + (e >> 2)) * a.seq_len + pos) * 4 + (e & 3)] = out;
        tag_store(a.kcur + row, out, e_q);
    }
}

// dst = old + result (x .+= ..., :284,305); which = 1 after wo (-> x_b), 3 after w2 (-> x_a); `old` is
// this thread's row of the other buffer, which the same thread wrote and kept in s_resid
template <bool HALF = false>
__device__ __forceinline__ void flow_finish_resid(int which, int wg) {
    which = uni(which), wg = uni(wg);
    const FlowArgs &a = c_flow;
    const FlowGeom &g = which == 1 ? a.wo : a.w2;
    unsigned *src = which == 1 ? a.x_a : a.x_b;
    unsigned *dst = which == 1 ? a.x_b : a.x_a;
    const int n_local = flow_n_local(g, wg);
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    flow_barrier_lds();
    if (tid >= n_local) return;
    const int row = wg * g.rpw + tid;
    const unsigned neww = bare_of(s_resid[tid] + flow_row_value4<HALF>(tid, g.ppr, flow_half<HALF>(g)));
    bare_store(dst + row, neww);
    s_resid[tid] = __uint_as_float(neww);  // (the value as the other workgroups read it)
    bare_store(src + row, FLOW_EMPTY);  // (its readers are through: see FLOW_EMPTY)
}

// SwiGLU (:295-299): logical rows (2u, 2u+1) are w1 row u and w3 row u.  The arithmetic (an fp64 exp) is a
// function of its own for the registers it takes; the stores are the caller's: a function that stores
// waits before it returns until the stores are acknowledged.
template <bool HALF = false>
__device__ __noinline__ unsigned flow_w13_word(int wg) {
    wg = uni(wg);
    const FlowArgs &a = c_flow;
    const int n_local = flow_n_local(a.w13, wg);
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    flow_barrier_lds();
    if (tid >= n_local) return 0u;
    const float own = flow_row_value4<HALF>(tid, a.w13.ppr, flow_half<HALF>(a.w13)), next = flow_pair_value(own);  // (w1 row u | w3 row u, threads 2u | 2u+1)
    if (tid & 1) return 0u;
    return bare_of(swiglu_val(own, next));
}
template <bool HALF = false>
__device__ __forceinline__ void flow_finish_w13(int wg, unsigned e_out) {
    const FlowArgs &a = c_flow;
    const unsigned v = flow_w13_word<HALF>(wg);
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    if (tid >= flow_n_local(a.w13, wg) || (tid & 1)) return;
    const int64_t u = ((int64_t)wg * a.w13.rpw + tid) >> 1;
    unsigned *mine = a.hbw + (int64_t)(e_out & 1u) * a.hidden, *other = a.hbw + (int64_t)((e_out & 1u) ^ 1u) * a.hidden;
    bare_store(mine + u, v);
    bare_store(other + u, FLOW_EMPTY);
}

// logits (:312) and this workgroup's first-maximum key: larger value wins, then the lower index
// (Julia's argmax, :360)
__device__ __noinline__ void flow_finish_cls(int wg, unsigned e_cls) {
    wg = uni(wg), e_cls = uni(e_cls);
    const FlowArgs &a = c_flow;
    const int n_local = flow_n_local(a.cls, wg), tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    flow_row_values<false>(n_local, a.cls.ppr);
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
// e_next != 0: the launch goes on with another step; the token is handed to all workgroups as a word of that epoch
__device__ __noinline__ void flow_pick_token(int nwg, unsigned e_cls, unsigned e_next) {
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
    if (e_next)
        for (int c = 0; c < FLOW_TOK_COPIES; c++) tag_store(a.tokw + 16 * c, __uint_as_float((unsigned)idx), e_next);
}

// The token of a launch's second and later steps: workgroup 0 publishes it when it has picked (flow_pick_token), and
// since that takes every workgroup's largest logit, a workgroup that has the word also knows that all others are
// through the step before (it may write the next step's first activations).  Polled on the scalar path: a scalar load
// that bypasses the scalar cache does not wait behind the fetches that the rings have just been refilled with, as a
// vector load would.  The word comes in FLOW_TOK_COPIES copies, a 128-byte line each, and a workgroup's first wavefront
// polls copy `workgroup % FLOW_TOK_COPIES` for all sixteen (one line is asked by a thirty-second of the chip).  Returns
// -1 if the wait gave up.
__device__ __forceinline__ int flow_next_token(unsigned epoch) {
    const FlowArgs &a = c_flow;
    if (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) == 0) {
        const u64 *p = a.tokw + 16 * (blockIdx.x % FLOW_TOK_COPIES);
        int tok = -1;
        for (unsigned spins = 0; spins <= a.spin_limit; spins++) {
            u64 w;
            asm volatile("s_load_dwordx2 %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)" : "=s"(w) : "s"(p) : "memory");
            if (tag_is(w, epoch)) {
                tok = (int)(unsigned)w;
                break;
            }
            if ((spins & 63) == 63 && __hip_atomic_load(a.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
            __builtin_amdgcn_s_sleep(1);
        }
        if ((threadIdx.x & 63) == 0) s_tok = tok;
    }
    flow_barrier_lds();
    return s_tok;
}

// The cache lines that head h's attention will read (positions before `pos`) are requested early, while
// the q/k/v matvec still runs: one 4-byte fetch per 128-byte line into a sink in LDS, so that the
// attention's own loads find the lines in the L2 instead of waiting for HBM twice in a row (scores,
// then values).  Position `pos` itself is not read from the cache by this launch.
__device__ __forceinline__ void flow_touch_cache(int layer, int h, int pos) {
    const FlowArgs &a = c_flow;
    if (pos <= 0) return;
    const int hs = a.hs, seq_len = a.seq_len;
    const int kvh = h / (a.n_heads / a.n_kv_heads);
    const unsigned char *kc = (const unsigned char *)(a.kc + (int64_t)layer * a.cache_layer_elems);
    const unsigned char *vc = (const unsigned char *)(a.vc + (int64_t)layer * a.cache_layer_elems);
    const int lane = threadIdx.x & 63;
    unsigned char *sink = s_sink;
    // K: per group of four head dimensions a run of 16 * pos bytes; V: one run of 4 * hs * pos bytes
    const int k_lines = (16 * pos + 127) / 128 + 1, n_k = (hs >> 2) * k_lines;
    const int64_t v_bytes = (int64_t)4 * hs * pos;
    const int n_v = (int)((v_bytes + 127) / 128) + 1;
    for (int i0 = (threadIdx.x & ~63); i0 < n_k + n_v; i0 += blockDim.x) {
        const int i = i0 + lane;
        const unsigned char *g = nullptr;
        if (i < n_k) {
            const int j = i / k_lines, ln = i % k_lines;
            const int64_t lo = ((int64_t)kvh * (hs >> 2) + j) * seq_len * 16, off = (lo & ~(int64_t)127) + 128 * ln;
            if (off < lo + 16 * pos) g = kc + off;
        } else if (i < n_k + n_v) {
            const int64_t lo = (int64_t)kvh * seq_len * hs * 4, off = (lo & ~(int64_t)127) + 128 * (int64_t)(i - n_k);
            if (off < lo + v_bytes) g = vc + off;
        }
        if (g) __builtin_amdgcn_global_load_lds((const AS1 void *)g, (AS3 void *)sink, 4, 0, 0);
    }
}

// ------------------------------------------------------------------------------------------
// attention of head h by one workgroup (reference src/inference.jl:263-278); q and the current
// position's k, v arrive as tagged words, earlier positions come from the cache (written by earlier
// launches).  Same arithmetic, in the same order, as attention_head.
// ------------------------------------------------------------------------------------------
// Caches of up to FLOW_ATT_SHORT positions, the usual case: built for little waiting rather than for
// throughput (one head is a few hundred KiB at most).  All keys are requested at once, before q has
// arrived, all values as soon as the scores are done; barriers separate scores | maximum | sum | values.  HS is a
// template parameter so that nothing below loops or branches on the head size.
#define FLOW_ATT_SHORT 256
template <int HS>
__device__ __noinline__ bool flow_attention_short(int layer, int h, int pos, unsigned e_in, unsigned e_out) {
    layer = uni(layer), h = uni(h), pos = uni(pos), e_in = uni(e_in), e_out = uni(e_out);
    const FlowArgs &a = c_flow;
    // (values: the 16-byte groups of a row are mapped onto n4p lanes, the next power of two; lanes beyond n4 idle)
    constexpr int hs = HS, n4 = HS >> 2, n4p = n4 <= 8 ? 8 : (n4 <= 16 ? 16 : 32), ngrp = FLOW_NW * 64 / n4p, per = HS >> 4,
                  NV = FLOW_ATT_SHORT / ngrp;
    static_assert(HS % 16 == 0 && HS <= 128, "head size");
    const int seq_len = a.seq_len, np = pos + 1;
    const int kvh = h / (a.n_heads / a.n_kv_heads);
    const float *kc = a.kc + (int64_t)layer * a.cache_layer_elems;
    const float *vc = a.vc + (int64_t)layer * a.cache_layer_elems;
    float *s_q = (float *)s_act;             // fp32 as it arrives; widened where it is used
    float *s_kcur = s_q + hs;
    float *s_vcur = s_kcur + hs;
    float *s_att = s_vcur + hs;              // [FLOW_ATT_SHORT]
    double *s_p = (double *)(s_att + FLOW_ATT_SHORT);  // [FLOW_ATT_SHORT]
    double *s_r = s_p + FLOW_ATT_SHORT;      // [FLOW_NW][hs]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
    // scores: lane = (timestep p16 of the wavefront's 16, quarter of the head dimension);
    // values: thread = (16-byte group i4 of the head dimension, timestep group grp), timesteps grp + u * ngrp
    const int p16 = lane & 15, part = lane >> 4, t = 16 * wave + p16;
    const int i4 = tid & (n4p - 1), grp = tid / n4p;
    const bool v_lane = n4p == n4 || i4 < n4;
    typedef float f32x4v __attribute__((ext_vector_type(4)));  // (one 128-bit register: a struct's four floats get split up)
    f32x4v kv[per], v[NV];
    // The keys are requested first of all, before the wait for q: a wavefront none of whose timesteps is in the cache skips
    // them (a scalar branch), a lane beyond the cache reads timestep 0 and does not use it.
    {
        const f32x4v *kp = (const f32x4v *)kc + ((int64_t)kvh * (hs >> 2) + part * per) * seq_len + (t < pos ? t : 0);
#pragma unroll
        for (int u = 0; u < per; u++) {
            kv[u] = f32x4v{0.f, 0.f, 0.f, 0.f};
            if (16 * wave < pos) kv[u] = kp[(int64_t)u * seq_len];
        }
    }
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
        s_q[tid] = tag_val(w);  // s_q, s_kcur, s_vcur lie one behind the other
    }
    if (!ok) s_flag = 1;
    __syncthreads();
    if (s_flag) {
        if (tid == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return false;
    }
    ATL();
    // the current position's key and value are in LDS, the earlier ones came from the cache
    if (t == pos) {
#pragma unroll
        for (int u = 0; u < per; u++) kv[u] = ((const f32x4v *)s_kcur)[part * per + u];
    }
    const float scale = sqrtf((float)hs);
    float sc = -INFINITY;
    {
        double acc = 0.0;
        if (t < np) {
#pragma unroll
            for (int u = 0; u < per; u++) {
                const float4 qq = ((const float4 *)s_q)[part * per + u];
                acc = fma((double)qq.x, (double)kv[u].x, acc);
                acc = fma((double)qq.y, (double)kv[u].y, acc);
                acc = fma((double)qq.z, (double)kv[u].z, acc);
                acc = fma((double)qq.w, (double)kv[u].w, acc);
            }
        }
        // the values are requested now (the keys' registers are free): they arrive during the softmax
        // (No lane-dependent branch around a load and no choice of source at it: either makes the compiler wait for the
        // loads one by one.  A wavefront skips the loads none of whose timesteps is in the cache — a scalar branch — and
        // within a load a lane without a row, or beyond the head size, reads row 0; what the lane really sums is picked
        // after the softmax, when the loads have long landed.)
        const f32x4v *vp0 = (const f32x4v *)(vc + (int64_t)kvh * seq_len * hs) + (v_lane ? i4 : 0);
        const int grp0 = (wave * 64) / n4p;  // the wavefront's first timestep group
#pragma unroll
        for (int u = 0; u < NV; u++) {
            const int tv = grp + u * ngrp;
            v[u] = f32x4v{0.f, 0.f, 0.f, 0.f};
            if (grp0 + u * ngrp < pos) v[u] = vp0[(int64_t)(tv < pos ? tv : 0) * n4];
        }
        // the quarters are added in order (fp64)
        const double a1 = __shfl(acc, p16 + 16, WAVE), a2 = __shfl(acc, p16 + 32, WAVE), a3 = __shfl(acc, p16 + 48, WAVE);
        if (part == 0 && t < np) sc = (float)(((acc + a1) + a2) + a3) / scale;
    }
    float mx = wave_max_f32_dpp(sc);
    if (lane == 0) s_redf[wave] = mx;
    ATL();
    __syncthreads();
#pragma unroll
    for (int w = 0; w < FLOW_NW; w++) mx = fmaxf(mx, s_redf[w]);
    float e = 0.0f;
    if (part == 0 && t < np) e = (float)exp((double)(sc - mx));
    const double sum = wave_sum_f64_dpp((double)e);
    if (lane == 0) s_red[wave] = sum;
    __syncthreads();
    double tot = 0.0;
#pragma unroll
    for (int w = 0; w < FLOW_NW; w++) tot += s_red[w];
    const float sf = (float)tot;
    if (part == 0 && t < np) s_p[t] = (double)(e / sf);  // softmax!, :169-174
    __syncthreads();
    ATL();
    {
        double acc[4] = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int u = 0; u < NV; u++) {
            const int tv = grp + u * ngrp;
            if (tv == pos) v[u] = ((const f32x4v *)s_vcur)[v_lane ? i4 : 0];  // (the current position's row comes from LDS)
            if (!v_lane) v[u] = f32x4v{0.f, 0.f, 0.f, 0.f};
            if (tv < np) {
                const double p = s_p[tv];
                acc[0] = fma(p, (double)v[u].x, acc[0]);
                acc[1] = fma(p, (double)v[u].y, acc[1]);
                acc[2] = fma(p, (double)v[u].z, acc[2]);
                acc[3] = fma(p, (double)v[u].w, acc[3]);
            }
        }
#pragma unroll
        for (int off = n4p; off < 64; off <<= 1)
#pragma unroll
            for (int c = 0; c < 4; c++) acc[c] += __shfl_xor(acc[c], off, WAVE);
        if (lane < n4) {
#pragma unroll
            for (int c = 0; c < 4; c++) s_r[wave * hs + 4 * i4 + c] = acc[c];
        }
    }
    __syncthreads();
    ATL();
    if (tid < hs) {
        double acc = 0.0;
#pragma unroll
        for (int k = 0; k < FLOW_NW; k++) acc += s_r[k * hs + tid];
        bare_store(a.xo + (int64_t)(e_out & 1u) * a.dim + (int64_t)h * hs + tid, bare_of((float)acc));
        bare_store(a.xo + (int64_t)((e_out & 1u) ^ 1u) * a.dim + (int64_t)h * hs + tid, FLOW_EMPTY);
    }
    __syncthreads();
    return true;
}
#undef ATL

// Longer caches: the G = (workgroups / heads) workgroups h*G .. h*G + G-1 share head h, each taking a run of the
// timesteps, so that the whole chip reads the cache.  The arithmetic is that of attention_head with the sums
// regrouped: a member publishes its run's largest score, every member takes the largest of all; then e = fp32(exp(s -
// max)) and the run's fp64 sum of e, published; every member adds the sums in member order and rounds (softmax!'s
// sum); then p = e / sum (fp32) and the run's fp64 partial value sums, published; member j adds the partial sums of
// its hs / G output elements in member order, rounds and stores them.  The exchanged numbers are {32 bits, epoch}
// words like q, k, v (a double travels as two of them); every wait is bounded.
__device__ __forceinline__ void tag_store_f64(u64 *p, double v, unsigned epoch) {
    const unsigned long long b = (unsigned long long)__double_as_longlong(v);
    tag_store(p, __uint_as_float((unsigned)b), epoch);
    tag_store(p + 1, __uint_as_float((unsigned)(b >> 32)), epoch);
}
// waits for the two words of a double; ok is cleared if the wait gave up
__device__ __forceinline__ double tag_wait_f64(const u64 *p, unsigned epoch, bool &ok) {
    u64 lo = tag_load(p), hi = tag_load(p + 1);
    unsigned spins = 0;
    while (!(tag_is(lo, epoch) && tag_is(hi, epoch))) {
        if (++spins > c_flow.spin_limit ||
            ((spins & 63) == 0 && __hip_atomic_load(c_flow.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
            ok = false;
            break;
        }
        lo = tag_load(p);
        hi = tag_load(p + 1);
    }
    return __longlong_as_double((long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned long long)(unsigned)lo));
}

// H16: the cache holds fp16 elements (K as [n_kv][hs/8][seq_len][8], V rows of hs halves): a lane reads eight
// elements per 16-byte load; hs is then a multiple of 32.
template <bool H16>
__device__ __noinline__ bool flow_attention_split(int layer, int pos, unsigned e_in, unsigned e_out) {
    layer = uni(layer), pos = uni(pos), e_in = uni(e_in), e_out = uni(e_out);
    const FlowArgs &a = c_flow;
    // head h runs on workgroups h * G .. h * G + G - 1 (workgroups beyond the last head's take no part)
    const int G = (int)gridDim.x / a.n_heads, h = (int)blockIdx.x / G, j = (int)blockIdx.x - h * G;
    if (h >= a.n_heads) return true;
    const int hs = a.hs, seq_len = a.seq_len, np = pos + 1;
    const int kvh = h / (a.n_heads / a.n_kv_heads);
    const float *kc = (const float *)((const char *)a.kc + (int64_t)layer * a.cache_layer_elems * (H16 ? 2 : 4));
    const float *vc = (const float *)((const char *)a.vc + (int64_t)layer * a.cache_layer_elems * (H16 ? 2 : 4));
    // this member's run of timesteps [lo, hi): runs are multiples of 64 long, the last members' may be empty
    const int C = (((np + G - 1) / G) + 63) & ~63;
    const int lo = min(np, j * C), hi = min(np, lo + C), nj = hi - lo;
    double *s_q = (double *)s_act;                                        // [hs]
    double *s_r = s_q + hs;                                               // [max(16 * hs, 1024)]
    float *s_att = (float *)(s_r + (FLOW_NW * hs > 1024 ? FLOW_NW * hs : 1024));  // [C]: scores, then e
    float *s_kcur = s_att + C;
    float *s_vcur = s_kcur + hs;
    double *s_x = (double *)(s_vcur + hs);                                // [G]: the members' maxima / sums
    u64 *x_max = a.att_x + (int64_t)h * G;
    u64 *x_sum = a.att_x + (int64_t)a.n_heads * G + ((int64_t)h * G) * 2;
    u64 *x_part = a.att_x + (int64_t)a.n_heads * G * 3 + ((int64_t)h * G) * hs * 2;
    const int tid = threadIdx.x;
    bool ok = true;
#ifdef L2H_TIMELINE
    int stl = 0;  // profiling build: member 0 of every head stamps the steps of layer 2
#define STL()                                                                                                         \
    do {                                                                                                              \
        if (a.timeline && tid == 0 && j == 0 && layer == 2 && stl < 16) a.timeline[256 * 64 + h * 16 + stl++] = wall_clock64(); \
    } while (0)
#else
#define STL()
#endif
    STL();
    __syncthreads();  // the activation area is free
    if (tid < 3 * hs) {
        const int which = tid / hs, i = tid % hs;
        // (k and v of the current position are needed by the member whose run holds it)
        if (which == 0 || (pos >= lo && pos < hi)) {
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
    }
    if (!ok) s_flag = 1;
    __syncthreads();
#define SPLIT_CHECK()                                                                                              \
    if (s_flag) {                                                                                                  \
        if (tid == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);             \
        return false;                                                                                              \
    }
    SPLIT_CHECK();
    STL();
    const float scale = sqrtf((float)hs);
    float mx = -INFINITY;
    // (a cache row that only one head reads is read once per token: loaded with the non-temporal hint)
    const bool once = a.n_heads == a.n_kv_heads;
    // scores: a wavefront takes 16 timesteps at a time, lane = (timestep p16, quarter of the head dimension); the
    // quarter's 16-byte loads are all in flight at once; the quarters are added in order (fp64) through lane exchanges,
    // so that the wavefronts run through their timesteps without meeting
    {
        const int lane = tid & 63, wv = tid >> 6, p16 = lane & 15, part = lane >> 4, per = hs >> 4;  // hs: a multiple of 16, at most 128
        for (int t0 = lo + 16 * wv; t0 < hi; t0 += 16 * FLOW_NW) {
            const int t = t0 + p16;
            double acc = 0.0;
            if (H16) {
                if (t < hi) {
                    const int per8 = hs >> 5;  // 16-byte groups of eight elements per quarter
                    const int64_t kg = ((int64_t)kvh * (hs >> 3) + part * per8) * seq_len + t;
                    const float *kl = s_kcur + part * (hs >> 2);
                    Half8 kv[4];
                    h8_bits kb[4];  // (all loads first, then the widening: see the fp32 rows below)
                    // (no branch around a load: a group beyond the head size repeats group 0)
#pragma unroll
                    for (int u = 0; u < 4; u++) kb[u] = ldg_nt_h8_bits(kc, kg + (int64_t)(u < per8 ? u : 0) * seq_len);
#pragma unroll
                    for (int u = 0; u < 4; u++)
                        if (u < per8) kv[u] = h8_widen(kb[u]);
                    if (t == pos) {
#pragma unroll
                        for (int u = 0; u < 4; u++)
                            if (u < per8)
#pragma unroll
                                for (int c = 0; c < 8; c++) kv[u].v[c] = kl[8 * u + c];
                    }
#pragma unroll
                    for (int u = 0; u < 4; u++)
                        if (u < per8) {
                            const double *qq = s_q + part * (hs >> 2) + 8 * u;
#pragma unroll
                            for (int c = 0; c < 8; c++) acc = fma(qq[c], (double)kv[u].v[c], acc);
                        }
                }
            } else if (t < hi) {
                const float4 *kp = (const float4 *)kc + ((int64_t)kvh * (hs >> 2) + part * per) * seq_len + t;
                const float4 *kl = (const float4 *)s_kcur + part * per;
                float4 kv[8];
                // (all of a lane's loads are requested before anything waits for one: the current position's row, which
                // comes from LDS, replaces what was loaded for it afterwards — a choice between the two sources at the
                // load itself makes the compiler wait for every load in turn)
#pragma unroll
                for (int u = 0; u < 8; u++)
                    if (u < per) kv[u] = once ? ldg_nt_f4(kp + (int64_t)u * seq_len) : kp[(int64_t)u * seq_len];
                if (t == pos) {
#pragma unroll
                    for (int u = 0; u < 8; u++)
                        if (u < per) kv[u] = kl[u];
                }
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
            const double a1 = __shfl(acc, p16 + 16, WAVE), a2 = __shfl(acc, p16 + 32, WAVE), a3 = __shfl(acc, p16 + 48, WAVE);
            if (part == 0 && t < hi) {
                const float sc = (float)(((acc + a1) + a2) + a3) / scale;
                s_att[t - lo] = sc;
                mx = fmaxf(mx, sc);
            }
        }
    }
    mx = block_max_f32(mx, s_redf);
    STL();
    if (tid == 0) tag_store(x_max + j, mx, e_out);
    if (tid < G) {  // the largest score of the head: every member's
        const u64 *p = x_max + tid;
        u64 w = tag_load(p);
        unsigned spins = 0;
        while (!tag_is(w, e_out)) {
            if (++spins > a.spin_limit ||
                ((spins & 63) == 0 && __hip_atomic_load(a.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                ok = false;
                break;
            }
            w = tag_load(p);
        }
        s_x[tid] = (double)tag_val(w);
    }
    if (!ok) s_flag = 1;
    __syncthreads();
    SPLIT_CHECK();
    STL();
    float gmx = -INFINITY;
    for (int k = 0; k < G; k++) gmx = fmaxf(gmx, (float)s_x[k]);
    double sum = 0.0;
    for (int t = tid; t < nj; t += blockDim.x) {
        const float e = (float)exp((double)(s_att[t] - gmx));
        s_att[t] = e;
        sum += (double)e;
    }
    sum = block_sum_f64(sum, s_red);  // (ends with every thread past the reads of s_x above)
    STL();
    if (tid == 0) tag_store_f64(x_sum + 2 * j, sum, e_out);
    if (tid < G) s_x[tid] = tag_wait_f64(x_sum + 2 * tid, e_out, ok);
    if (!ok) s_flag = 1;
    __syncthreads();
    SPLIT_CHECK();
    STL();
    double tot = 0.0;
    for (int k = 0; k < G; k++) tot += s_x[k];
    const float sf = (float)tot;  // softmax!'s sum (reference src/inference.jl:169-174)
    // values: thread = (16-byte group i4 of the head dimension, timestep group), four loads in flight (with eight the
    // function needs callee-saved registers, and saving them to scratch costs more than the deeper loads gain); the
    // groups of one wavefront are folded with lane exchanges, the rest through LDS
    // (the 16-byte groups of a row are mapped onto n4p lanes, the next power of two; lanes beyond n4 idle)
    const int n4 = hs >> 2, n4p = n4 <= 8 ? 8 : (n4 <= 16 ? 16 : 32);
    const int ngrp = blockDim.x / n4p;
    if (H16) {
        // thread = (group i8 of eight head dimensions, timestep group of 64); four loads in flight
        const int n8 = hs >> 3, i8 = tid & 15, grp = tid >> 4, ng = blockDim.x >> 4;
        const bool v_lane = i8 < n8;
        double acc[8] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
        for (int t0 = lo + grp; t0 < hi; t0 += 4 * ng) {
            Half8 v[4];
            h8_bits vb[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int t = t0 + u * ng;
                vb[u] = (h8_bits){0u, 0u, 0u, 0u};
                if (t < hi && v_lane) vb[u] = ldg_nt_h8_bits(vc, ((int64_t)kvh * seq_len + t) * n8 + i8);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = h8_widen(vb[u]);
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (t0 + u * ng == pos && v_lane) {
#pragma unroll
                    for (int c = 0; c < 8; c++) v[u].v[c] = s_vcur[8 * i8 + c];
                }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int t = t0 + u * ng;
                if (t < hi) {
                    const double p = (double)(s_att[t - lo] / sf);
#pragma unroll
                    for (int c = 0; c < 8; c++) acc[c] = fma(p, (double)v[u].v[c], acc[c]);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < 8; c++) {
            acc[c] += __shfl_xor(acc[c], 16, WAVE);
            acc[c] += __shfl_xor(acc[c], 32, WAVE);
        }
        if ((tid & 63) < n8) {
            const int wv = tid >> 6;
#pragma unroll
            for (int c = 0; c < 8; c++) s_r[wv * hs + 8 * i8 + c] = acc[c];
        }
    } else {
        const int i4 = tid & (n4p - 1), grp = tid / n4p;
        const bool v_lane = i4 < n4;
        const float4 *vp = (const float4 *)(vc + (int64_t)kvh * seq_len * hs) + i4;
        double acc[4] = {0.0, 0.0, 0.0, 0.0};
#ifndef FLOW_VD
#define FLOW_VD 4
#endif
        constexpr int VD = FLOW_VD;
        for (int t0 = lo + grp; t0 < hi; t0 += VD * ngrp) {
            float4 v[VD];
#pragma unroll
            for (int u = 0; u < VD; u++) {
                const int t = t0 + u * ngrp;
                v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (t < hi && v_lane) v[u] = once ? ldg_nt_f4(vp + (int64_t)t * n4) : vp[(int64_t)t * n4];
            }
#pragma unroll
            for (int u = 0; u < VD; u++) {
                const int t = t0 + u * ngrp;
                if (t == pos && v_lane) v[u] = *(const float4 *)(s_vcur + 4 * i4);  // (see the scores)
                if (t < hi) {
                    const double p = (double)(s_att[t - lo] / sf);
                    acc[0] = fma(p, (double)v[u].x, acc[0]);
                    acc[1] = fma(p, (double)v[u].y, acc[1]);
                    acc[2] = fma(p, (double)v[u].z, acc[2]);
                    acc[3] = fma(p, (double)v[u].w, acc[3]);
                }
            }
        }
        for (int off = n4p; off < 64; off <<= 1)
#pragma unroll
            for (int c = 0; c < 4; c++) acc[c] += __shfl_xor(acc[c], off, WAVE);
        if ((tid & 63) < n4) {
            const int wv = tid >> 6;
#pragma unroll
            for (int c = 0; c < 4; c++) s_r[wv * hs + 4 * i4 + c] = acc[c];
        }
    }
    __syncthreads();
    STL();
    if (tid < hs) {
        double acc = 0.0;
        for (int k = 0; k < FLOW_NW; k++) acc += s_r[k * hs + tid];
        tag_store_f64(x_part + ((int64_t)j * hs + tid) * 2, acc, e_out);
    }
    // member j finishes the hs / G output elements j * hs / G ...: thread (element, member) fetches one partial
    // sum, thread (element, 0) adds them in member order
    const int per_m = hs / G;
    __syncthreads();  // (s_r is free)
    if (tid < per_m * G) {
        const int el = j * per_m + tid / G, m = tid % G;
        s_r[tid] = tag_wait_f64(x_part + ((int64_t)m * hs + el) * 2, e_out, ok);
    }
    if (!ok) s_flag = 1;
    __syncthreads();
    SPLIT_CHECK();
#undef SPLIT_CHECK
    STL();
    if (tid < per_m) {
        double acc = 0.0;
        for (int m = 0; m < G; m++) acc += s_r[tid * G + m];
        const int el = j * per_m + tid;
        bare_store(a.xo + (int64_t)(e_out & 1u) * a.dim + (int64_t)h * hs + el, bare_of((float)acc));
        bare_store(a.xo + (int64_t)((e_out & 1u) ^ 1u) * a.dim + (int64_t)h * hs + el, FLOW_EMPTY);
    }
    __syncthreads();
    STL();
#undef STL
    return true;
}

// ------------------------------------------------------------------------------------------
// the kernel; gen0 = epoch of this launch's input (advances by 5 * n_layers + 2 per launch)
// ------------------------------------------------------------------------------------------
// MIXED: the layers' pieces are typed (flow_loop_mixed) and none travel through registers; the classifier's
// pieces follow them in the stream in their usual form, and the ring starts afresh for them.
// n_tok: steps of the token loop (reference src/inference.jl:349-386) that this launch runs, one after the other; the
// epochs of step t start at gen0 + t * (5 * n_layers + 2).
// HALF (with MIXED): the layer matrices' rows of dim inputs end in the middle of a piece (FlowGeom::half)
template <int T_CLS, bool MIXED, bool HALF = false>
__global__ __launch_bounds__(1024) void flow_token_kernel(unsigned int gen0, int n_tok) {
    const FlowArgs &a = c_flow;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = blockIdx.x, nwg = gridDim.x;
    unsigned char *ring_base = s_ring + wave * (FLOW_D * FLOW_SLOT);
    // the launch's first step as the control block has it; workgroup 0 advances the block after every step
    // (flow_pick_token), the others count for themselves
    const int pos_first = a.ctl->pos, step_first = a.ctl->step, n_prompt = a.ctl->n_prompt, tok_first = a.ctl->last_argmax;
    if (tid == 0) s_flag = 0;
    Ring r;
    MRing mr;
    unsigned char *mring_base = s_ring + wave * (FLOWM_D * FLOWM_SLOT);
    const unsigned char *reg_ptr = nullptr;
    RegPieces rp;
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
#else
#define FTL()
#define FTLS()
#endif
#define LEAVE()        \
    do {               \
        flow_drain(r); \
        return;        \
    } while (0)
    // (flow_drain waits for everything this wavefront has requested, whichever ring it went to)
#pragma nounroll
  for (int t_step = 0; t_step < n_tok; t_step++) {
    // the rings start at the head of the streams (their areas are free: the step before ended with a wait for all of
    // its pieces): requested before the step's token is there
    r.gptr = a.stream + a.wave_off[wg * FLOW_NW + wave];
    r.lds = (unsigned)(size_t)ring_base;
    r.issued = r.consumed = r.drain_mark = 0;
    r.off = 0;
    if constexpr (MIXED) {
        mr.gptr = r.gptr;
        mr.lds = (unsigned)(size_t)mring_base;
        mr.left = a.n_layers * (flow_wave_pieces<HALF>(a.qkv, wg, wave) + flow_wave_pieces<HALF>(a.wo, wg, wave) +
                                flow_wave_pieces<HALF>(a.w13, wg, wave) + flow_wave_pieces<false>(a.w2, wg, wave));
        {
            const unsigned long long p = (unsigned long long)mr.gptr;
            mr.gptr = (const unsigned char *)(((unsigned long long)uni((unsigned)(p >> 32)) << 32) | uni((unsigned)p));
            mr.lds = uni(mr.lds);
            mr.left = uni(mr.left);
        }
        flowm_start(mr, mring_base, uni(a.wave_types[wg * FLOW_NW + wave]), lane);
    } else {
        // the layers' pieces and, where the classifier is q4_K too, its pieces behind them: one stream
        const int ring_layer = flow_ring_pieces<false>(a.qkv, wg, wave) + flow_ring_pieces<false>(a.wo, wg, wave) +
                               flow_ring_pieces<false>(a.w13, wg, wave) + flow_ring_pieces<false>(a.w2, wg, wave);
        r.left = a.n_layers * ring_layer + (T_CLS == L2H_TYPE_Q4_K ? flow_wave_pieces<false>(a.cls, wg, wave) : 0);
        ring_uniform(r);  // values that came through vector loads are the same on every lane: make them scalar
        // the register pieces follow the ring's part of the stream, in the order in which they are used
        reg_ptr = uni(r.gptr + (int64_t)a.n_layers * ring_layer * FLOW_SLOT +
                      (int64_t)flow_wave_pieces<false>(a.cls, wg, wave) * (T_CLS == L2H_TYPE_Q6_K ? FLOW_Q6_PIECE : FLOW_SLOT));
        flow_top_up_q4(r, ring_base, lane);
    }
    FTL();

    // ---- this step's token, position and RoPE angles (reference src/inference.jl:122-127) ----
    const unsigned E0 = gen0 + (unsigned)t_step * (5u * (unsigned)a.n_layers + 2u);
    const int pos = pos_first + t_step, step = step_first + t_step;
    int tok = tok_first;
    if (t_step > 0) {
        tok = uni(flow_next_token(E0));
        if (tok < 0) {
            if (tid == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            LEAVE();
        }
    }
    if (step < n_prompt) tok = a.prompt[step];
    if (tid < (a.hs >> 1)) {
        float theta = 1.0f * (float)pos;
        for (int k = 0; k < tid; k++) theta *= a.theta_scale;
        s_rope[2 * tid] = (float)cos((double)theta);
        s_rope[2 * tid + 1] = (float)sin((double)theta);
    }
    // attention of head h runs on workgroup h * stride + h % stride (spread over the XCDs)
    const int att_stride = nwg / a.n_heads;
    const int att_h = uni(wg / att_stride);
    const bool is_att = uni((int)(att_h < a.n_heads && wg % att_stride == att_h % att_stride)) != 0;
    // the rows of x this workgroup adds to after wo (layer 0): straight from the embedding (:236)
    {
        const int lo = wg * a.wo.rpw, n = flow_n_local(a.wo, wg);
        if (tid < n) s_resid[tid] = __uint_as_float(bare_of(dequant_elem(a.emb, tok, lo + tid)));
    }

    for (int l = 0; l < a.n_layers; l++) {
        const unsigned e_x = E0 + 5u * (unsigned)l;  // x entering the layer
        const unsigned e_q = e_x + 1, e_att = e_x + 2, e_w13 = e_x + 4;  // (e_x + 3 and e_x + 5: the two residual additions)
        // the four matvec phases of the layer share one copy of the streaming loop (the kernel must stay
        // small enough for the instruction cache):
        //   0  rmsnorm (:244), q, k, v (:247-249), rope (:255-256), cache append (:259-260)
        //   1  attention (:263-278) on workgroup h*stride + h%stride, then x += wo * xb (:281-284)
        //   2  rmsnorm (:287), w1, w3 (:291-292), SwiGLU (:295-299)
        //   3  x += w2 * hb (:302-305)
#pragma nounroll
        for (int kind = 0; kind < 4; kind++) {
            bool ok;
            // (thread and lane number anew in every phase: see flow_loop_q4)
            int tid = threadIdx.x;
            asm volatile("" : "+v"(tid));
            const int lane = tid & 63;
            const FlowGeom g = flow_geom<HALF>(a, kind);
            const int n_reg = MIXED ? 0 : uni(flow_reg_pieces<false>(g, wg, wave));
            if (!MIXED && kind != 1) flow_reg_fetch(rp, reg_ptr, n_reg, lane);
#ifdef L2H_TIMELINE
            if (tid == 0) s_tl_fine = ((int)gridDim.x > 101 && wg == 101 && l == 2) ? 256 * 64 + 512 + kind * 8 : -1;
            if (tid == 0) s_tl_wave = ((int)gridDim.x > 101 && wg == 101 && l == 2) ? 256 * 64 + 600 + kind * 16 : -1;
#endif
            if (kind == 0) {
                const float *nw = a.rms_att + (int64_t)l * a.norm_stride;
                ok = l == 0 ? flow_stage<PRO_RMSNORM, SRC_EMB>(nullptr, a.dim, nw, tok)
                            : flow_stage<PRO_RMSNORM, SRC_BARE>(a.x_a, a.dim, nw, tok);
            } else if (kind == 1) {
                // (a long cache is shared by all the workgroups of a head, a short one read by one of them)
                if (is_att || pos >= FLOW_ATT_SHORT || (MIXED && a.kv16)) {
                    const bool fine = (MIXED && a.kv16) ? flow_attention_split<true>(l, pos, e_q, e_att)
                                      : pos >= FLOW_ATT_SHORT ? flow_attention_split<false>(l, pos, e_q, e_att)
                                      : (MIXED && a.hs == 96) ? flow_attention_short<96>(l, att_h, pos, e_q, e_att)
                                      : a.hs == 128 ? flow_attention_short<128>(l, att_h, pos, e_q, e_att)
                                      : a.hs == 64  ? flow_attention_short<64>(l, att_h, pos, e_q, e_att)
                                                    : flow_attention_short<32>(l, att_h, pos, e_q, e_att);
                    if (!uni((int)fine)) LEAVE();
                }
                if (!MIXED) flow_reg_fetch(rp, reg_ptr, n_reg, lane);  // (after the attention: its loads would wait behind these)
                FTL();
                ok = flow_stage<PRO_QUANT, SRC_BARE>(a.xo + (int64_t)(e_att & 1u) * a.dim, a.dim, nullptr, tok);
            } else if (kind == 2) {
                ok = flow_stage<PRO_RMSNORM, SRC_BARE>(a.x_b, a.dim, a.rms_ffn + (int64_t)l * a.norm_stride, tok);
            } else {
                ok = flow_stage<PRO_QUANT, SRC_BARE>(a.hbw + (int64_t)(e_w13 & 1u) * a.hidden, a.hidden, nullptr, tok);
            }
            if (!uni(ok)) LEAVE();
            FTL();
            reg_ptr += n_reg * FLOW_SLOT;
            // what the ring holds has landed by now: after this wait the first FLOW_D pieces need none,
            // and the cache lines requested next do not stand between the loop and its pieces
            flow_drain(r);
            if constexpr (MIXED)
                mr.ready = uni(mr.held);
            else
                flow_reg_arrived(rp);
            FTL();
            if (kind == 0 && is_att && pos < FLOW_ATT_SHORT && !(MIXED && a.kv16)) flow_touch_cache(l, att_h, pos);
            if constexpr (MIXED) {
                // rows of dim inputs padded to whole pieces: the q8_K blocks beyond dim are zero (d = 0, no quants)
                if (kind != 3 && a.dim_pad > a.dim && !flow_half<HALF>(g)) {
                    const int b0 = a.dim >> 8, nbz = (a.dim_pad - a.dim) >> 8;
                    unsigned char *q8 = (unsigned char *)s_act;
                    for (int i = tid; i < nbz * 64; i += 1024) ((uint32_t *)(q8 + 256 * b0))[i] = 0u;
                    if (tid < nbz * 8) ((uint32_t *)(q8 + 14336 + 32 * b0))[tid] = 0u;
                    if (tid < nbz) ((float *)(q8 + 14336 + 1792))[b0 + tid] = 0.f;
                    __syncthreads();
                }
                flow_loop_mixed<HALF>(g, mr, mring_base, wg);
            } else {
                flow_loop_q4<true, true>(g, r, ring_base, wg, rp, n_reg);
            }
            FTL();
            FTLS();
            if (kind == 0)
                flow_finish_qkv<MIXED, HALF>(l, wg, pos, e_q);
            else if (kind == 1)
                flow_finish_resid<HALF>(1, wg);
            else if (kind == 2)
                flow_finish_w13<HALF>(wg, e_w13);
            else
                flow_finish_resid<HALF>(3, wg);
            FTL();
        }
    }

    // ---- final rmsnorm (:309) + classifier (:312); q6_K pieces are larger: the ring starts afresh ----
    const unsigned e_fin = E0 + 5u * (unsigned)a.n_layers, e_cls = e_fin + 1;
    if (MIXED || T_CLS == L2H_TYPE_Q6_K) {
        // (the last epilogue's barrier lies behind every wavefront's last piece: the ring areas can be cut anew)
        flow_drain(r);
        if constexpr (MIXED) r.gptr = mr.gptr;
        r.issued = r.consumed = r.drain_mark = 0;
        r.off = 0;
        r.left = flow_wave_pieces<false>(a.cls, wg, wave);
        ring_uniform(r);
        if (T_CLS == L2H_TYPE_Q6_K)
            flow_top_up_q6(r, ring_base, lane);
        else
            flow_top_up_q4(r, ring_base, lane);
    }
    if (!uni(flow_stage<PRO_RMSNORM, SRC_BARE>(a.x_a, a.dim, a.rms_final, tok))) LEAVE();
    if (MIXED && a.dim_pad > a.dim) {
        const int b0 = a.dim >> 8, nbz = (a.dim_pad - a.dim) >> 8;
        unsigned char *q8 = (unsigned char *)s_act;
        for (int i = tid; i < nbz * 64; i += 1024) ((uint32_t *)(q8 + 256 * b0))[i] = 0u;
        if (tid < nbz * 8) ((uint32_t *)(q8 + 14336 + 32 * b0))[tid] = 0u;
        if (tid < nbz) ((float *)(q8 + 14336 + 1792))[b0 + tid] = 0.f;
        __syncthreads();
    }
    flow_drain(r);
    if (T_CLS == L2H_TYPE_Q6_K)
        flow_loop_q6(a.cls, r, ring_base, wg);
    else
        flow_loop_q4<false, false>(a.cls, r, ring_base, wg, rp, 0);
    flow_finish_cls(wg, e_cls);
    flow_drain(r);
    if (wg == 0) flow_pick_token(nwg, e_cls, t_step + 1 < n_tok ? e_cls + 1 : 0u);
  }
#undef LEAVE
}

// ------------------------------------------------------------------------------------------
// models of fp32 matrices (llama2.c checkpoints, reference src/load_karpathy.jl:32-59; matmul!, src/matmul.jl:3-11):
// the same kernel without streams.  A model of this kind is small (the largest llama2.c checkpoint is 0.4 GB) and
// its rows are read where the tensors lie; what the one launch saves is the 40-odd launches per token.
// Activations stay fp32 in LDS (no q8_K), products are exact in fp64 and summed in fp64, as in matvec_f32_kernel.
// ------------------------------------------------------------------------------------------
// the input vector of a phase -> fp32 in this workgroup's LDS; K <= 4096 and a multiple of 4
#ifndef XF_INLINE
#define XF_INLINE __noinline__
#endif
template <int PRO, int SRC>
__device__ XF_INLINE bool flow_stage_xf(const void *src, int K, const float *normw, int tok) {
    src = uni(src), K = uni(K), normw = uni(normw), tok = uni(tok);
    const FlowArgs &a = c_flow;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int idx = 256 * wave + 4 * lane;
    const bool mine = idx < K;  // (K is a multiple of 4: a lane's four words are all inside or all outside)
    constexpr bool rms = PRO == PRO_RMSNORM;
    float xv[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
    bool ok = true;
    if (rms && mine) {
        const float4 t = *(const float4 *)(normw + idx);
        wv[0] = t.x, wv[1] = t.y, wv[2] = t.z, wv[3] = t.w;
    }
    if (SRC == SRC_EMB) {
        if (mine)
#pragma unroll
            for (int k = 0; k < 4; k++) xv[k] = dequant_elem(a.emb, tok, idx + k);
    } else {
        unsigned spins = 0;
        u32x4v w0 = {FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY, FLOW_EMPTY};
        const unsigned *pb = (const unsigned *)src + idx;
        if (!mine) w0 = (u32x4v){0u, 0u, 0u, 0u};
        for (;;) {
            const bool full = w0.x != FLOW_EMPTY && w0.y != FLOW_EMPTY && w0.z != FLOW_EMPTY && w0.w != FLOW_EMPTY;
            if (!full) POLL_BARE1(w0, pb);
            const bool all = w0.x != FLOW_EMPTY && w0.y != FLOW_EMPTY && w0.z != FLOW_EMPTY && w0.w != FLOW_EMPTY;
            if (__ballot(!all) == 0ull) break;
            if (++spins > a.spin_limit ||
                ((spins & 63) == 0 && __hip_atomic_load(a.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                ok = false;
                break;
            }
        }
        xv[0] = __uint_as_float(w0.x), xv[1] = __uint_as_float(w0.y), xv[2] = __uint_as_float(w0.z), xv[3] = __uint_as_float(w0.w);
    }
    if (!ok) s_flag = 1;
    if (rms) {  // rmsnorm! (reference src/inference.jl:102-110)
        double acc = 0.0;
#pragma unroll
        for (int k = 0; k < 4; k++) acc = fma((double)xv[k], (double)xv[k], acc);
        acc = wave_sum_f64_dpp(acc);
        if (lane == 0) s_red[wave] = acc;
    }
    __syncthreads();
    if (s_flag) {
        if (threadIdx.x == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return false;
    }
    if (rms) {
        double t = 0.0;
        for (int w = 0; w < FLOW_NW; w++) t += s_red[w];
        float ss = (float)t;
        ss /= (float)K;
        ss += 1e-5f;
        ss = 1.0f / sqrtf(ss);
#pragma unroll
        for (int k = 0; k < 4; k++) xv[k] = wv[k] * (ss * xv[k]);
    }
    if (mine) ((float4 *)s_act)[64 * wave + lane] = make_float4(xv[0], xv[1], xv[2], xv[3]);
    __syncthreads();
    return true;
}

// The rows of one phase for one workgroup.  A row is cut into ppr slices of K / ppr inputs (a "piece", chosen so that a
// slice is at most 512 floats where K allows: two 16-byte loads per lane), and a wavefront takes a contiguous run of
// the workgroup's pieces, two at a time; partial sums in the layout the epilogues expect (four doubles per piece,
// the sums of 16 lanes each; CLS: one double per piece).  The weights do not depend on the phase's input: the first
// FLOW_F32_PRE 16-byte loads per lane of the run's first two pieces are requested before the wait for it
// (flow_f32_request), so that their latency passes during the wait (layer phases have one or two pieces per
// wavefront: usually all of their bytes).
#define FLOW_F32_PRE 2
struct F32Pre {
    f32x4v w[2][FLOW_F32_PRE];
};
// piece j of the workgroup -> its floats (n4 groups of four)
__device__ __forceinline__ const float4 *flow_f32_piece(const FlowGeom &g, bool cls, int kind, int layer, int wg, int j, int K,
                                                        int &x_off4) {
    const FlowArgs &a = c_flow;
    const int lr = j / g.ppr, part = j - lr * g.ppr;
    const int L = wg * g.rpw + lr;
    int seg, row;
    flow_row_src(cls ? 1 : kind, L, a.dim, a.kv_dim, a.hs, a.neox, seg, row);
    const int wi = cls ? 7 : (kind == 0 ? seg : (kind == 1 ? 3 : (kind == 2 ? 4 + seg : 6)));
    x_off4 = part * ((K / g.ppr) >> 2);
    return (const float4 *)(a.f_w[wi] + (cls ? (int64_t)0 : (int64_t)layer * a.f_stride[wi]) + (int64_t)row * K) + x_off4;
}
template <bool CLS>
__device__ __forceinline__ void flow_f32_request(F32Pre &pre, const FlowGeom &g, int kind, int layer, int wg, int K) {
    int lane = threadIdx.x & 63;
    asm volatile("" : "+v"(lane));
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cnt = uni(flow_wave_pieces<false>(g, wg, wave)), start = uni(flow_wave_start<false>(g, wg, wave));
    if (cnt <= 0) return;
    const int n4 = (K / g.ppr) >> 2;
#pragma unroll
    for (int r = 0; r < 2; r++) {
        int xo;
        const f32x4v *w4 = (const f32x4v *)flow_f32_piece(g, CLS, kind, layer, wg, start + min(r, cnt - 1), K, xo);
#pragma unroll
        for (int u = 0; u < FLOW_F32_PRE; u++)
            if (lane + 64 * u < n4) pre.w[r][u] = __builtin_nontemporal_load(w4 + lane + 64 * u);
    }
}
template <bool CLS>
__device__ __forceinline__ void flow_loop_f32(const F32Pre &pre, const FlowGeom &g, int kind, int layer, int wg, int K) {
    int lane = threadIdx.x & 63;
    asm volatile("" : "+v"(lane));
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cnt = uni(flow_wave_pieces<false>(g, wg, wave)), start = uni(flow_wave_start<false>(g, wg, wave));
    const int n4 = (K / g.ppr) >> 2;
#define F32_FMA4(ACC_, W_, X_)                       \
    ACC_ = fma((double)W_.x, (double)X_.x, ACC_);    \
    ACC_ = fma((double)W_.y, (double)X_.y, ACC_);    \
    ACC_ = fma((double)W_.z, (double)X_.z, ACC_);    \
    ACC_ = fma((double)W_.w, (double)X_.w, ACC_)
    for (int i = 0; i < cnt; i += 2) {
        int xa, xb;
        const float4 *wa4 = flow_f32_piece(g, CLS, kind, layer, wg, start + i, K, xa);
        const float4 *wb4 = flow_f32_piece(g, CLS, kind, layer, wg, start + min(i + 1, cnt - 1), K, xb);
        const float4 *xa4 = (const float4 *)s_act + xa, *xb4 = (const float4 *)s_act + xb;
        double acc0 = 0.0, acc1 = 0.0;
        int j0 = 0;
        if (i == 0) {  // the run's first two pieces: their first loads were requested before the wait
#pragma unroll
            for (int u = 0; u < FLOW_F32_PRE; u++)
                if (lane + 64 * u < n4) {
                    const float4 xv = xa4[lane + 64 * u], yv = xb4[lane + 64 * u];
                    const f32x4v wa = pre.w[0][u], wb = pre.w[1][u];
                    F32_FMA4(acc0, wa, xv);
                    F32_FMA4(acc1, wb, yv);
                }
            j0 = 64 * FLOW_F32_PRE;
        }
        for (int j = j0 + lane; j < n4; j += 64) {
            const float4 wa = ldg_nt_f4(wa4 + j), wb = ldg_nt_f4(wb4 + j), xv = xa4[j], yv = xb4[j];
            F32_FMA4(acc0, wa, xv);
            F32_FMA4(acc1, wb, yv);
        }
        if (CLS) {
            const double v0 = wave_sum_f64_dpp(acc0), v1 = wave_sum_f64_dpp(acc1);
            if (lane == 0) {
                s_part[start + i] = v0;
                if (i + 1 < cnt) s_part[start + i + 1] = v1;
            }
        } else {
            const double v0 = row16_sum_f64_dpp(acc0), v1 = row16_sum_f64_dpp(acc1);
            s_part[4 * (start + i) + (lane >> 4)] = v0;
            if (i + 1 < cnt) s_part[4 * (start + i + 1) + (lane >> 4)] = v1;
        }
    }
#undef F32_FMA4
}

__global__ __launch_bounds__(1024) void flow_f32_kernel(unsigned int gen0, int n_tok) {
    const FlowArgs &a = c_flow;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = blockIdx.x, nwg = gridDim.x;
    (void)wave;
    const int pos_first = a.ctl->pos, step_first = a.ctl->step, n_prompt = a.ctl->n_prompt, tok_first = a.ctl->last_argmax;
    if (tid == 0) s_flag = 0;
#ifdef L2H_TIMELINE
    int tl_n = 0;
#define XTL()                                                                                   \
    do {                                                                                        \
        if (a.timeline && tid == 0 && tl_n < 64) a.timeline[wg * 64 + tl_n++] = wall_clock64(); \
    } while (0)
#else
#define XTL()
#endif
#pragma nounroll
  for (int t_step = 0; t_step < n_tok; t_step++) {
    XTL();
    // ---- this step's token, position and RoPE angles (reference src/inference.jl:122-127) ----
    const unsigned E0 = gen0 + (unsigned)t_step * (5u * (unsigned)a.n_layers + 2u);
    const int pos = pos_first + t_step, step = step_first + t_step;
    int tok = tok_first;
    if (t_step > 0) {
        tok = uni(flow_next_token(E0));
        if (tok < 0) {
            if (tid == 0) __hip_atomic_store(a.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }
    if (step < n_prompt) tok = a.prompt[step];
    if (tid < (a.hs >> 1)) {
        float theta = 1.0f * (float)pos;
        for (int k = 0; k < tid; k++) theta *= a.theta_scale;
        s_rope[2 * tid] = (float)cos((double)theta);
        s_rope[2 * tid + 1] = (float)sin((double)theta);
    }
    const int att_stride = nwg / a.n_heads;
    const int att_h = uni(wg / att_stride);
    const bool is_att = uni((int)(att_h < a.n_heads && wg % att_stride == att_h % att_stride)) != 0;
    {
        const int lo = wg * a.wo.rpw, n = flow_n_local(a.wo, wg);
        if (tid < n) s_resid[tid] = __uint_as_float(bare_of(dequant_elem(a.emb, tok, lo + tid)));
    }
    for (int l = 0; l < a.n_layers; l++) {
        const unsigned e_x = E0 + 5u * (unsigned)l;
        const unsigned e_q = e_x + 1, e_att = e_x + 2, e_w13 = e_x + 4;
#pragma nounroll
        for (int kind = 0; kind < 4; kind++) {
            bool ok;
            const FlowGeom g = flow_geom(a, kind);
            const int K = kind == 3 ? a.hidden : a.dim;
            F32Pre pre;
            // (after the attention where this workgroup runs one: its loads would wait behind these)
            if (kind != 1) flow_f32_request<false>(pre, g, kind, l, wg, K);
            if (kind == 0) {
                const float *nw = a.rms_att + (int64_t)l * a.norm_stride;
                ok = l == 0 ? flow_stage_xf<PRO_RMSNORM, SRC_EMB>(nullptr, a.dim, nw, tok)
                            : flow_stage_xf<PRO_RMSNORM, SRC_BARE>(a.x_a, a.dim, nw, tok);
            } else if (kind == 1) {
                if (is_att || pos >= FLOW_ATT_SHORT) {
                    const bool fine = pos >= FLOW_ATT_SHORT ? flow_attention_split<false>(l, pos, e_q, e_att)
                                      : a.hs == 128 ? flow_attention_short<128>(l, att_h, pos, e_q, e_att)
                                      : a.hs == 64  ? flow_attention_short<64>(l, att_h, pos, e_q, e_att)
                                                    : flow_attention_short<32>(l, att_h, pos, e_q, e_att);
                    if (!uni((int)fine)) return;
                }
                flow_f32_request<false>(pre, g, kind, l, wg, K);
                ok = flow_stage_xf<PRO_QUANT, SRC_BARE>(a.xo + (int64_t)(e_att & 1u) * a.dim, a.dim, nullptr, tok);
            } else if (kind == 2) {
                ok = flow_stage_xf<PRO_RMSNORM, SRC_BARE>(a.x_b, a.dim, a.rms_ffn + (int64_t)l * a.norm_stride, tok);
            } else {
                ok = flow_stage_xf<PRO_QUANT, SRC_BARE>(a.hbw + (int64_t)(e_w13 & 1u) * a.hidden, a.hidden, nullptr, tok);
            }
            if (!uni(ok)) return;
            XTL();
            if (kind == 0 && is_att && pos < FLOW_ATT_SHORT) flow_touch_cache(l, att_h, pos);
            flow_loop_f32<false>(pre, g, kind, l, wg, K);
            XTL();
            if (kind == 0)
                flow_finish_qkv(l, wg, pos, e_q);
            else if (kind == 1)
                flow_finish_resid(1, wg);
            else if (kind == 2)
                flow_finish_w13(wg, e_w13);
            else
                flow_finish_resid(3, wg);
            XTL();
        }
    }
    // ---- final rmsnorm (:309) + classifier (:312) ----
    const unsigned e_fin = E0 + 5u * (unsigned)a.n_layers, e_cls = e_fin + 1;
    F32Pre pre;
    flow_f32_request<true>(pre, a.cls, 4, 0, wg, a.dim);
    if (!uni(flow_stage_xf<PRO_RMSNORM, SRC_BARE>(a.x_a, a.dim, a.rms_final, tok))) return;
    flow_loop_f32<true>(pre, a.cls, 4, 0, wg, a.dim);
    flow_finish_cls(wg, e_cls);
    if (wg == 0) flow_pick_token(nwg, e_cls, t_step + 1 < n_tok ? e_cls + 1 : 0u);
  }
#undef XTL
}

// ------------------------------------------------------------------------------------------
// building the streams (once per model)
// ------------------------------------------------------------------------------------------
// bytes a wavefront's stream holds for one layer, and before phase `kind` within a layer
__host__ __device__ inline int64_t flow_layer_bytes(const FlowGeom *g4, int wg, int wave, int upto) {
    int64_t b = 0;
    for (int k = 0; k < upto; k++) b += (int64_t)flow_ring_pieces(g4[k], wg, wave) * FLOW_SLOT;
    return b;
}
// register pieces of a wavefront in one layer, before phase `upto`
__host__ __device__ inline int flow_layer_regs(const FlowGeom *g4, int wg, int wave, int upto) {
    int n = 0;
    for (int k = 0; k < upto; k++) n += flow_reg_pieces(g4[k], wg, wave);
    return n;
}
// a wavefront's stream: the ring's pieces of every layer, the classifier's, then the register pieces of every layer
__host__ __device__ inline int64_t flow_reg_base(const FlowGeom *g4, const FlowGeom &cls, int cls_piece_bytes, int n_layers,
                                                 int wg, int wave) {
    return (int64_t)n_layers * flow_layer_bytes(g4, wg, wave, 4) + (int64_t)flow_wave_pieces(cls, wg, wave) * cls_piece_bytes;
}

struct FlowRepackArgs {
    unsigned char *stream;
    const int64_t *wave_off;
    FlowGeom g4[4];
    FlowGeom cls;
    int kind;  // 0..3 layer phases, 4 classifier
    int layer, n_layers, cls_piece_bytes;
    DevTensor w[3];
    int dim, kv_dim, hs, neox;
    int mixed;  // typed pieces: placed by the tables
    FlowTypedDev typed;
};

// one 64-thread workgroup copies one piece from the per-tensor field streams into its place
__global__ __launch_bounds__(64) void flow_repack_kernel(FlowRepackArgs p) {
    const FlowGeom g = p.kind == 4 ? p.cls : (p.kind == 0 ? p.g4[0] : (p.kind == 1 ? p.g4[1] : (p.kind == 2 ? p.g4[2] : p.g4[3])));
    const int per_wg = flow_wg_capacity(g);
    const int wg = blockIdx.x / per_wg, j = blockIdx.x % per_wg;
    if (j >= flow_wg_pieces(g, wg)) return;
    const int np = flow_wg_pieces(g, wg), base = np / FLOW_NW, rem = np % FLOW_NW;
    const int wave = j < rem * (base + 1) ? j / (base + 1) : rem + (j - rem * (base + 1)) / base;
    const int idx = j - flow_wave_start(g, wg, wave);
    const int L = wg * g.rpw + flow_piece_row(g, j);
    const int half = flow_half(g), part = half ? j % half : j % g.ppr;
    int seg, row32;
    flow_row_src(p.kind == 4 ? 1 : p.kind, L, p.dim, p.kv_dim, p.hs, p.neox, seg, row32, true);
    const int64_t row = row32;
    const DevTensor &t = seg == 0 ? p.w[0] : (seg == 1 ? p.w[1] : p.w[2]);
    const int64_t layer_b = flow_layer_bytes(p.g4, wg, wave, 4);
    const int lane = threadIdx.x;
    if (p.mixed && p.kind < 4) {
        // typed piece: entry of the tables = the wavefront's pieces of earlier layers and phases + idx
        int before = 0, per_layer = 0;
        for (int k = 0; k < 4; k++) {
            const int c = flow_wave_pieces(p.g4[k], wg, wave);
            per_layer += c;
            if (k < p.kind) before += c;
        }
        const int64_t e = p.typed.piece_base[wg * FLOW_NW + wave] + (int64_t)p.layer * per_layer + before + idx;
        uint4 *dst = (uint4 *)(p.stream + p.wave_off[wg * FLOW_NW + wave] + p.typed.piece_off[e]);
        // super-block b of the piece: which tensor and which of its super-blocks (valid: the row has it; a row that is
        // padded to whole pieces has fewer than 8 in its last piece, and the others are written as zeros, d = 0).
        // Rows that end inside a piece: super-block 8 part + b of the pair's, the odd row's from t.nb on.
        auto at = [&](int b_, const DevTensor *&tt, int64_t &bi) -> bool {
            if (half) {
                const int pb = 8 * part + b_, odd = pb >= (int)t.nb ? 1 : 0;
                int sg, rw;
                flow_row_src(p.kind, L + odd, p.dim, p.kv_dim, p.hs, p.neox, sg, rw, true);
                tt = sg == 0 ? &p.w[0] : (sg == 1 ? &p.w[1] : &p.w[2]);
                bi = (int64_t)rw * tt->nb + (pb - odd * (int)t.nb);
                return true;
            }
            tt = &t;
            bi = row * t.nb + part * 8 + b_;
            return (int64_t)part * 8 + b_ < t.nb;
        };
        const uint4 z4 = make_uint4(0u, 0u, 0u, 0u);
        const DevTensor *tt;
        int64_t bi;
        if (lane == 0) dst[8] = make_uint4((uint32_t)p.typed.piece_tag[e], 0u, 0u, 0u);
        if (t.type == L2H_TYPE_Q4_K) {
            if (lane < 8) dst[lane] = at(lane, tt, bi) ? flow_encode_hdr(tt->hdr[bi]) : z4;
            dst[9 + lane] = at(lane >> 3, tt, bi) ? ((const uint4 *)(tt->qs + bi * 128))[lane & 7] : z4;
        } else if (t.type == L2H_TYPE_Q5_K) {
            if (lane < 8) dst[lane] = at(lane, tt, bi) ? flow_encode_hdr(tt->hdr[bi]) : z4;
            if (lane < 16) dst[9 + lane] = at(lane >> 1, tt, bi) ? ((const uint4 *)(tt->qh + bi * 32))[lane & 1] : z4;
            dst[25 + lane] = at(lane >> 3, tt, bi) ? ((const uint4 *)(tt->qs + bi * 128))[lane & 7] : z4;
        } else {  // q6_K
            if (lane < 8) dst[lane] = at(lane, tt, bi) ? ((const uint4 *)(tt->sc6 + bi * 4))[0] : z4;
            if (lane == 1) {
                uint16_t dd[8];
                for (int b_ = 0; b_ < 8; b_++) dd[b_] = at(b_, tt, bi) ? tt->d6[bi] : (uint16_t)0;
                dst[9] = make_uint4(dd[0] | (uint32_t)dd[1] << 16, dd[2] | (uint32_t)dd[3] << 16, dd[4] | (uint32_t)dd[5] << 16,
                                    dd[6] | (uint32_t)dd[7] << 16);
            }
            if (lane < 32) dst[10 + lane] = at(lane >> 2, tt, bi) ? ((const uint4 *)(tt->qh + bi * 64))[lane & 3] : z4;
            dst[42 + lane] = at(lane >> 3, tt, bi) ? ((const uint4 *)(tt->qs + bi * 128))[lane & 7] : z4;
        }
        return;
    }
    const int64_t cls_at = p.mixed ? p.typed.cls_off[wg * FLOW_NW + wave] : (int64_t)p.n_layers * layer_b;
    if (t.type == L2H_TYPE_Q4_K) {
        int64_t off = p.kind == 4 ? cls_at : (int64_t)p.layer * layer_b + flow_layer_bytes(p.g4, wg, wave, p.kind);
        int at = idx;
        if (p.kind < 4) {
            const int n_ring = flow_ring_pieces(g, wg, wave);
            if (idx >= n_ring) {
                off = flow_reg_base(p.g4, p.cls, p.cls_piece_bytes, p.n_layers, wg, wave) +
                      ((int64_t)p.layer * flow_layer_regs(p.g4, wg, wave, 4) + flow_layer_regs(p.g4, wg, wave, p.kind)) * FLOW_SLOT;
                at = idx - n_ring;
            }
        }
        uint4 *dst = (uint4 *)(p.stream + p.wave_off[wg * FLOW_NW + wave] + off + (int64_t)at * FLOW_SLOT);
        const int64_t blk0 = row * t.nb + part * 8;
        const int nbv = (int)min((int64_t)8, max((int64_t)0, t.nb - (int64_t)part * 8));  // (8 unless the row is padded)
        const uint4 z4 = make_uint4(0u, 0u, 0u, 0u);
        if (lane < 8) dst[lane] = lane < nbv ? flow_encode_hdr(t.hdr[blk0 + lane]) : z4;
        dst[8 + lane] = (lane >> 3) < nbv ? ((const uint4 *)(t.qs + blk0 * 128))[lane] : z4;
    } else {  // q6_K classifier
        const int64_t off = cls_at;
        uint4 *dst = (uint4 *)(p.stream + p.wave_off[wg * FLOW_NW + wave] + off + (int64_t)idx * FLOW_Q6_PIECE);
        const int64_t blk0 = row * t.nb + part * 16;
        const int nbv = (int)min((int64_t)16, max((int64_t)0, t.nb - (int64_t)part * 16));  // (16 unless the row is padded)
        const uint4 z4 = make_uint4(0u, 0u, 0u, 0u);
        const uint4 *ql = (const uint4 *)(t.qs + blk0 * 128), *qh = (const uint4 *)(t.qh + blk0 * 64);
        dst[lane] = (lane >> 3) < nbv ? ql[lane] : z4;
        dst[64 + lane] = 8 + (lane >> 3) < nbv ? ql[64 + lane] : z4;
        dst[128 + lane] = (lane >> 2) < nbv ? qh[lane] : z4;
        if (lane < 16) dst[192 + lane] = lane < nbv ? ((const uint4 *)(t.sc6 + blk0 * 4))[lane] : z4;
        if (lane < 2) {
            uint16_t dd[8];
            for (int b = 0; b < 8; b++) dd[b] = 8 * lane + b < nbv ? t.d6[blk0 + 8 * lane + b] : (uint16_t)0;
            dst[208 + lane] = make_uint4(dd[0] | (uint32_t)dd[1] << 16, dd[2] | (uint32_t)dd[3] << 16,
                                         dd[4] | (uint32_t)dd[5] << 16, dd[6] | (uint32_t)dd[7] << 16);
        }
    }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
static FlowGeom make_geom(int64_t n_rows, int64_t K, int type, int grid, bool halves = false) {
    FlowGeom g{};
    g.n_rows = (int)n_rows;
    g.K = (int)K;
    int rpw = (int)((n_rows + grid - 1) / grid);
    rpw += rpw & 1;
    g.rpw = rpw;
    if (type == L2H_TYPE_F32) {
        // fp32 rows: slices of at most 512 floats where K allows it (1, 2, 4 or 8 slices of a multiple of 4 floats):
        // two loads per lane, which flow_f32_request covers
        int ppr = 1;
        while (ppr < 8 && K / ppr > 512 && K % (8 * ppr) == 0) ppr *= 2;
        g.ppr = ppr;
    } else {
        g.ppr = (int)(K / 256) / (type == L2H_TYPE_Q6_K ? 16 : 8);
        if (halves) g.ppr = 0;  // K = 256 * (8 i + 4): a piece and a half per row (or 2 1/2, ...), whole pieces per pair of rows
    }
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
    a.mixed = 0;
    a.f32 = 0;
    {
        bool all_f32 = cls_type == L2H_TYPE_F32;
        for (int i = 0; i < n_layer_types; i++) all_f32 = all_f32 && layer_types[i] == L2H_TYPE_F32;
        if (all_f32 && a.kv16) return no("fp32 models keep an fp32 cache in this kernel");
        if (all_f32) {  // rows of fp32 weights, read where they lie: a row is one "piece"
            if (a.dim % 4 != 0 || a.hidden % 4 != 0 || a.dim > 4096 || a.hidden > 4096)
                return no("fp32 models: dim and hidden_dim must be multiples of 4, at most 4096");
            if (a.n_heads > grid || (a.hs != 32 && a.hs != 64 && a.hs != 128)) return no("head size must be 32, 64 or 128");
            const int G = grid / a.n_heads;
            if (G < 1 || a.hs % G != 0 || G > 64) return no("head size must be a multiple of workgroups / heads");
            const size_t run = (size_t)((((a.seq_len + G - 1) / G) + 63) & ~63);
            const size_t att = (size_t)a.hs * 8 + (size_t)std::max(FLOW_NW * a.hs, 1024) * 8 + run * 4 + (size_t)a.hs * 8 + 64 * 8;
            if (att > FLOW_ACT_BYTES) return no("sequence too long for the attention area");
            a.qkv = make_geom(a.dim + 2 * a.kv_dim, a.dim, L2H_TYPE_F32, grid);
            a.wo = make_geom(a.dim, a.dim, L2H_TYPE_F32, grid);
            a.w13 = make_geom(2 * (int64_t)a.hidden, a.dim, L2H_TYPE_F32, grid);
            a.w2 = make_geom(a.dim, a.hidden, L2H_TYPE_F32, grid);
            a.cls = make_geom(a.vocab, a.dim, L2H_TYPE_F32, grid);
            const FlowGeom *gs[5] = {&a.qkv, &a.wo, &a.w13, &a.w2, &a.cls};
            for (const FlowGeom *g : gs)
                if (g->rpw > FLOW_MAX_ROWS || g->rpw * g->ppr > (g == &a.cls ? FLOW_MAX_PIECES : FLOW_MAX_PIECES / 4))
                    return no("too many rows per workgroup");
            if ((a.dim + 2 * a.kv_dim) % 2 != 0) return no("odd row count");
            if (a.wo.rpw != a.w2.rpw || a.wo.rpw > FLOW_RESID_ROWS) return no("too many rows of x per workgroup");
            a.f32 = 1;
            a.dim_pad = a.dim;
            return true;
        }
    }
    for (int i = 0; i < n_layer_types; i++) {
        const int t = layer_types[i];
        if (t != L2H_TYPE_Q4_K && t != L2H_TYPE_Q5_K && t != L2H_TYPE_Q6_K) return no("layer matrices must be q4_K, q5_K or q6_K");
        if (t != L2H_TYPE_Q4_K) a.mixed = 1;
    }
    for (int l = 0; l * 7 + 6 < n_layer_types; l++)  // (w1 and w3 rows alternate within a workgroup's pieces)
        if (layer_types[l * 7 + 4] != layer_types[l * 7 + 6]) return no("w1 and w3 of a layer must have one type");
    if (cls_type != L2H_TYPE_Q4_K && cls_type != L2H_TYPE_Q6_K) return no("classifier must be q4_K or q6_K");
    // rows of dim inputs may be padded with zero super-blocks to whole pieces if that adds a third at most (dim 3584
    // -> 4096); such a model, and one with head size 96, runs as typed pieces.  Where half a piece is missing (dim 3072)
    // the layer matrices are not padded: their rows go in pairs, a pair's middle piece shared by the two (the
    // classifier's rows, which are not paired, stay padded).
    a.dim_pad = (a.dim + 2047) / 2048 * 2048;
    const bool halves = a.dim % 2048 == 1024;
    if (a.dim % 256 != 0 || (int64_t)a.dim * 4 < (int64_t)a.dim_pad * 3 || a.hidden % 2048 != 0)
        return no("dim must be a multiple of 2048 (or of 256 and within a quarter below one), hidden_dim a multiple of 2048");
    if (a.dim_pad != a.dim) a.mixed = 1;
    if (cls_type == L2H_TYPE_Q6_K && a.dim_pad % 4096 != 0) return no("a q6_K classifier needs dim to be a multiple of 4096");
    if (a.hidden > 14336 || a.dim_pad > 4096) return no("dim above 4096 or hidden_dim above 14336");
    if (a.n_heads > grid || (a.hs != 32 && a.hs != 64 && a.hs != 96 && a.hs != 128)) return no("head size must be 32, 64, 96 or 128");
    if (a.hs == 96) a.mixed = 1;
    if (a.kv16) {  // (set by the caller) the fp16 cache is read by the typed-piece instantiation's attention only
        if (a.hs % 32 != 0) return no("an fp16 cache needs a head size that is a multiple of 32");
        a.mixed = 1;
    }
    // the split attention of long caches: q, the partial sums, one member's run of scores, k and v of the position, G numbers
    const int G = grid / a.n_heads;
    if (G < 1 || a.hs % G != 0 || G > 64) return no("head size must be a multiple of workgroups / heads");
    const size_t run = (size_t)((((a.seq_len + G - 1) / G) + 63) & ~63);
    const size_t att = (size_t)a.hs * 8 + (size_t)std::max(FLOW_NW * a.hs, 1024) * 8 + run * 4 + (size_t)a.hs * 8 + 64 * 8;
    if (att > FLOW_ACT_BYTES) return no("sequence too long for the attention area");
    a.qkv = make_geom(a.dim + 2 * a.kv_dim, halves ? a.dim : a.dim_pad, L2H_TYPE_Q4_K, grid, halves);
    a.wo = make_geom(a.dim, halves ? a.dim : a.dim_pad, L2H_TYPE_Q4_K, grid, halves);
    a.w13 = make_geom(2 * (int64_t)a.hidden, halves ? a.dim : a.dim_pad, L2H_TYPE_Q4_K, grid, halves);
    a.w2 = make_geom(a.dim, a.hidden, L2H_TYPE_Q4_K, grid);
    a.cls = make_geom(a.vocab, a.dim_pad, cls_type, grid);
    const FlowGeom *gs[5] = {&a.qkv, &a.wo, &a.w13, &a.w2, &a.cls};
    for (const FlowGeom *g : gs)
        if (g->rpw > FLOW_MAX_ROWS || flow_wg_capacity(*g) > (g == &a.cls ? FLOW_MAX_PIECES : FLOW_MAX_PIECES / 4))
            return no("too many rows per workgroup");  // (layer phases keep four partial sums per piece)
    if ((a.dim + 2 * a.kv_dim) % 2 != 0 || (halves && (a.dim % 2 != 0 || a.kv_dim % 2 != 0)))
        return no("odd row count");
    if (a.wo.rpw != a.w2.rpw) return no("row split of wo and w2 differs");  // (a row of x has one owner)
    if (a.wo.rpw > FLOW_RESID_ROWS) return no("too many rows of x per workgroup");
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
            total += flow_reg_base(g4, a.cls, cls_type == L2H_TYPE_Q6_K ? FLOW_Q6_PIECE : FLOW_SLOT, a.n_layers, wg, w);
            total += (int64_t)a.n_layers * flow_layer_regs(g4, wg, w, 4) * FLOW_SLOT;
            total = (total + 255) & ~(int64_t)255;
        }
    return total + 4096;  // the last fetches of a stream may be issued past a workgroup's final piece: none are, but pad anyway
}

void k_flow_typed_tables(const FlowArgs &a, const int *layer_types, int cls_type, int grid, FlowTypedTables &t) {
    const FlowGeom g4[4] = {a.qkv, a.wo, a.w13, a.w2};
    const size_t nw = (size_t)grid * FLOW_NW;
    t.wave_off.assign(nw, 0);
    t.piece_base.assign(nw, 0);
    t.cls_off.assign(nw, 0);
    t.wave_types.assign(nw, 0u);
    t.piece_off.clear();
    t.piece_tag.clear();
    const int cls_piece = cls_type == L2H_TYPE_Q6_K ? FLOW_Q6_PIECE : FLOW_SLOT;
    int64_t total = 0;
    std::vector<int> types;
    for (int wg = 0; wg < grid; wg++)
        for (int w = 0; w < FLOW_NW; w++) {
            const size_t wi = (size_t)wg * FLOW_NW + w;
            t.wave_off[wi] = total;
            t.piece_base[wi] = (int64_t)t.piece_off.size();
            types.clear();
            int64_t off = 0;
            for (int l = 0; l < a.n_layers; l++)
                for (int kind = 0; kind < 4; kind++) {
                    const FlowGeom &g = g4[kind];
                    const int cnt = flow_wave_pieces(g, wg, w), start = flow_wave_start(g, wg, w);
                    for (int i = 0; i < cnt; i++) {
                        const int L = wg * g.rpw + flow_piece_row(g, start + i);
                        int seg, row;
                        flow_row_src(kind, L, a.dim, a.kv_dim, a.hs, a.neox, seg, row, true);
                        const int slot = kind == 0 ? seg : (kind == 1 ? 3 : (kind == 2 ? 4 : 5));
                        const int ty = layer_types[l * 7 + slot] - L2H_TYPE_Q4_K;
                        t.piece_off.push_back(off);
                        types.push_back(ty);
                        off += flowm_piece_bytes(ty);
                    }
                }
            const size_t n = types.size();
            for (size_t i = 0; i < n; i++)
                t.piece_tag.push_back((uint16_t)(types[i] | ((i + FLOWM_D < n ? types[i + FLOWM_D] : 3) << 8)));
            unsigned first = 0;
            for (size_t j = 0; j < (size_t)FLOWM_D && j < n; j++) first |= (unsigned)types[j] << (2 * j);
            t.wave_types[wi] = first;
            t.cls_off[wi] = off;
            off += (int64_t)flow_wave_pieces(a.cls, wg, w) * cls_piece;
            total += (off + 255) & ~(int64_t)255;
        }
    t.total = total + 4096;
}

hipError_t k_flow_repack(hipStream_t s, const FlowArgs &a, unsigned char *stream, const int64_t *wave_off_dev, int kind,
                         int layer, const DevTensor *w, int nw, int grid, int cls_type, const FlowTypedDev &typed) {
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
    p.cls_piece_bytes = cls_type == L2H_TYPE_Q6_K ? FLOW_Q6_PIECE : FLOW_SLOT;
    for (int i = 0; i < nw; i++) p.w[i] = w[i];
    p.dim = a.dim;
    p.kv_dim = a.kv_dim;
    p.hs = a.hs;
    p.neox = a.neox;
    p.mixed = a.mixed;
    p.typed = typed;
    const FlowGeom &g = kind == 4 ? a.cls : p.g4[kind];
    hipLaunchKernelGGL(flow_repack_kernel, dim3((unsigned)(grid * flow_wg_capacity(g))), dim3(64), 0, s, p);
    return hipGetLastError();
}

// copies a model's arguments into the kernel's constant memory (stream-ordered, then waited for)
hipError_t k_flow_bind(hipStream_t s, const FlowArgs &a) {
    hipError_t e = hipMemcpyToSymbolAsync(HIP_SYMBOL(c_flow_raw), &a, sizeof(FlowArgs), 0, hipMemcpyHostToDevice, s);
    if (e != hipSuccess) return e;
    return hipStreamSynchronize(s);
}

// Whether `grid` workgroups of the kernel can be resident at once on a device of n_cu CUs that runs nothing
// else.  The kernel has no grid-wide barrier and every wait in it is bounded, so residency is what makes it
// fast, not what makes it correct: workgroups that had to wait for a CU would let the others run into their
// wait limit, and the launch would end with the error that l2h_model_set_wait_limit describes.
// form: 0 q4_K pieces, 1 typed pieces, 2 typed pieces and rows that end inside a piece
static const void *flow_kernel_fn(int cls_type, int form) {
    if (cls_type == L2H_TYPE_F32) return (const void *)flow_f32_kernel;
    if (form == 2)
        return cls_type == L2H_TYPE_Q6_K ? (const void *)flow_token_kernel<L2H_TYPE_Q6_K, true, true>
                                         : (const void *)flow_token_kernel<L2H_TYPE_Q4_K, true, true>;
    if (form == 1)
        return cls_type == L2H_TYPE_Q6_K ? (const void *)flow_token_kernel<L2H_TYPE_Q6_K, true>
                                         : (const void *)flow_token_kernel<L2H_TYPE_Q4_K, true>;
    return cls_type == L2H_TYPE_Q6_K ? (const void *)flow_token_kernel<L2H_TYPE_Q6_K, false>
                                     : (const void *)flow_token_kernel<L2H_TYPE_Q4_K, false>;
}

bool k_flow_fits(int cls_type, int grid, int n_cu, int form) {
    const void *fn = flow_kernel_fn(cls_type, form);
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, 1024, 0) != hipSuccess) return false;
    return per_cu >= 1 && (int64_t)per_cu * n_cu >= grid;
}

// A plain launch: a cooperative one costs about 20 µs more per token on this stack, and all it would add is the
// residency check that k_flow_fits makes once.
hipError_t k_flow_launch(hipStream_t s, unsigned int gen0, int n_tok, int cls_type, int grid, int form) {
    void *args[] = {&gen0, &n_tok};
    const void *fn = flow_kernel_fn(cls_type, form);
    return hipLaunchKernel(fn, dim3(grid), dim3(1024), args, 0, s);
}
