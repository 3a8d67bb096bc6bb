// Persistent decode kernel: transformer! (reference src/inference.jl:222-315) plus the greedy
// pick (:360) for one token in ONE launch.  One workgroup of 16 wavefronts per compute unit runs
// the phases of every layer back to back, separated by a grid-wide barrier:
//     embed | per layer: [rmsnorm+q,k,v+rope+cache] | attention | [wo+residual] |
//             [rmsnorm+w1,w3+SwiGLU] | [w2+residual] | [rmsnorm+classifier] | argmax
// Before it waits at a barrier, every wavefront issues the loads of its first weight tile of the
// next phase, so the HBM pipes stay busy while the barrier and the activation staging complete.
// The phases are the same device functions the per-phase kernels run (matvec_dev.h); activations
// that cross workgroups use device-scope accesses (COH = true).
#include "matvec_dev.h"

#include <string.h>

// ------------------------------------------------------------------------------------------
// grid barrier.  Arrival: 16 workgroups share a counter, the last of them bumps the root counter,
// the last root arrival publishes the generation number in 8 flag copies; waiters poll "their"
// copy.  All accesses are relaxed device-scope atomics; data published before the barrier was
// written with device-scope stores that have completed (s_waitcnt) before the arrival.
// A wait is bounded: after `spin_limit` polls the workgroup raises `abort`, and every workgroup
// leaves the kernel at its next barrier.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ bool grid_barrier(GridBar *b, unsigned long long gen, unsigned int spin_limit,
                                             int *s_abort) {
    __builtin_amdgcn_s_waitcnt(0);  // this thread's stores have reached their coherence point
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned nwg = gridDim.x, wg = blockIdx.x;
        const unsigned ngrp = (nwg + 15) >> 4, grp = wg >> 4;
        const unsigned in_grp = min(16u, nwg - (grp << 4));
        bool last = false;
        const unsigned long long prev =
            __hip_atomic_fetch_add(&b->count[16 * (1 + grp)], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == (unsigned long long)in_grp * gen - 1) {
            const unsigned long long p2 =
                __hip_atomic_fetch_add(&b->count[0], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last = (p2 == (unsigned long long)ngrp * gen - 1);
        }
        int aborted = 0;
        if (last) {
            for (int k = 0; k < 8; k++)
                __hip_atomic_store(&b->flag[16 * k], gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            unsigned int spins = 0;
            const unsigned fi = 16 * (wg & 7);
            while (__hip_atomic_load(&b->flag[fi], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < gen) {
                if (++spins > spin_limit) {
                    __hip_atomic_store(&b->abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    aborted = 1;
                    break;
                }
                if ((spins & 63) == 0 && __hip_atomic_load(&b->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                    aborted = 1;
                    break;
                }
            }
        }
        if (!aborted && __hip_atomic_load(&b->abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) aborted = 1;
        *s_abort = aborted;
    }
    __syncthreads();
    return *s_abort == 0;
}

// first-maximum key of (value, index): larger value wins, then lower index (Julia's argmax)
__device__ __forceinline__ unsigned long long mega_argmax_key(float v, uint32_t idx) {
    uint32_t b = __float_as_uint(v);
    b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    if (v == 0.0f) b = 0x80000000u;
    return ((unsigned long long)b << 32) | (unsigned long long)(0xFFFFFFFFu - idx);
}

__device__ __forceinline__ unsigned long long block_max_key(unsigned long long key, unsigned long long *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const unsigned long long o = __shfl_xor(key, m, WAVE);
        key = o > key ? o : key;
    }
    __syncthreads();
    if (lane == 0) red[wave] = key;
    __syncthreads();
    unsigned long long t = red[0];
    for (int w = 1; w < nw; w++) t = red[w] > t ? red[w] : t;
    return t;
}

// Phase arguments of the model being decoded: q/k/v, wo, w1+w3, w2 of layer 0 (later layers are
// addressed by stride) and the classifier.  Constant memory: read with scalar loads that the
// compiler may treat as invariant; the phase index goes through `opaque` so that each phase
// loads what it needs when it starts instead of everything being loaded at kernel entry.
#define PHASE_BYTES ((sizeof(PhaseArgs) + 15) & ~(size_t)15)
__constant__ __attribute__((aligned(16))) unsigned char c_phase_raw[5 * PHASE_BYTES];

__device__ __forceinline__ int opaque(int k) {
    asm volatile("" : "+s"(k));
    return k;
}
#define PHASE(k) (*(const PhaseArgs *)(c_phase_raw + (size_t)opaque(k) * PHASE_BYTES))

template <int T_QKV, int T_WO, int T_W13, int T_W2, int T_OUT>
__global__ __launch_bounds__(1024) void decode_token_kernel(MegaArgs g) {
    extern __shared__ uint4 smem[];
    __shared__ double red[16];
    __shared__ float redf[16];
    __shared__ int s_next, s_abort;
    // phase arguments live in the kernel-argument segment (layer 0 + per-layer strides)
    const int wg = blockIdx.x, nwg = gridDim.x, tid = threadIdx.x;
    unsigned long long gen = g.gen0;
#define BARRIER()                                                       \
    do {                                                                \
        if (!grid_barrier(g.bar, ++gen, g.spin_limit, &s_abort)) return; \
    } while (0)

#ifdef L2H_TIMELINE
    int tl_n = 0;
#define MTL()                                                                                        \
    do {                                                                                             \
        if (g.timeline && tid == 0 && tl_n < 64) g.timeline[wg * 64 + tl_n++] = wall_clock64();      \
    } while (0)
#else
#define MTL()
#endif
    MTL();
    // ---- token embedding (:236) and this position's RoPE table (:122-127) ----
    const int pos = g.ctl->pos;
    {
        const int tok = g.ctl->step < g.ctl->n_prompt ? g.prompt[g.ctl->step] : g.ctl->last_argmax;
        for (int e = wg * blockDim.x + tid; e < g.dim; e += nwg * blockDim.x)
            st_f32<true>(g.x + e, dequant_elem(g.emb, tok, e));
        if (wg == nwg - 1 && tid < (g.hs >> 1)) {
            float theta = 1.0f * (float)pos;
            for (int k = 0; k < tid; k++) theta *= g.theta_scale;
            st_f32<true>(g.rope_cs + 2 * tid, (float)cos((double)theta));
            st_f32<true>(g.rope_cs + 2 * tid + 1, (float)sin((double)theta));
        }
    }
    Tile<T_QKV> t_qkv;
    Tile<T_WO> t_wo;
    Tile<T_W13> t_w13;
    Tile<T_W2> t_w2;
    matvec_prefetch<T_QKV, EPI_ROPE_KV>(PHASE(0), 0, wg, t_qkv);
    MTL();
    BARRIER();
    MTL();

    for (int l = 0; l < g.n_layers; l++) {
        // q, k, v
        matvec_phase<T_QKV, PRO_RMSNORM, EPI_ROPE_KV, false, true>(PHASE(0), l, wg, smem, red, &s_next, t_qkv, true);
        matvec_prefetch<T_WO, EPI_RESID>(PHASE(1), l, wg, t_wo);
        MTL();
        BARRIER();
        MTL();
        // attention: one head per workgroup
        for (int h = wg; h < g.n_heads; h += nwg) attention_head<true>(g.q, g.xb, g.kc + (int64_t)l * g.cache_layer_elems, g.vc + (int64_t)l * g.cache_layer_elems, g.hs,
                                                                   g.n_heads, g.n_kv_heads, g.seq_len, h, pos, smem, red, redf);
        MTL();
        BARRIER();
        MTL();
        // wo + residual
        matvec_phase<T_WO, PRO_QUANT, EPI_RESID, false, true>(PHASE(1), l, wg, smem, red, &s_next, t_wo, true);
        matvec_prefetch<T_W13, EPI_SWIGLU>(PHASE(2), l, wg, t_w13);
        MTL();
        BARRIER();
        MTL();
        // w1, w3 + SwiGLU
        matvec_phase<T_W13, PRO_RMSNORM, EPI_SWIGLU, false, true>(PHASE(2), l, wg, smem, red, &s_next, t_w13, true);
        matvec_prefetch<T_W2, EPI_RESID>(PHASE(3), l, wg, t_w2);
        MTL();
        BARRIER();
        MTL();
        // w2 + residual
        matvec_phase<T_W2, PRO_QUANT, EPI_RESID, false, true>(PHASE(3), l, wg, smem, red, &s_next, t_w2, true);
        if (l + 1 < g.n_layers) matvec_prefetch<T_QKV, EPI_ROPE_KV>(PHASE(0), l + 1, wg, t_qkv);
        MTL();
        BARRIER();
        MTL();
    }

    // ---- final rmsnorm (:309) + classifier (:312), then argmax over this workgroup's rows ----
    {
        Tile<T_OUT> t_out;
        const PhaseArgs &po = PHASE(4);
        matvec_phase<T_OUT, PRO_RMSNORM, EPI_STORE, false, true>(po, 0, wg, smem, red, &s_next, t_out, false);
        int n_local;
        int64_t L_lo;
        const float *vals = matvec_phase_vals(po, wg, smem, n_local, L_lo);
        unsigned long long best = 0;
        for (int lr = tid; lr < n_local; lr += blockDim.x) {
            const unsigned long long key = mega_argmax_key(vals[lr], (uint32_t)(L_lo + lr));
            best = key > best ? key : best;
        }
        best = block_max_key(best, (unsigned long long *)red);
        if (tid == 0) __hip_atomic_store(g.argmax_partial + wg, best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    BARRIER();
    if (wg == 0) {  // argmax(logits) (:360) and the step bookkeeping of the token loop (:349-386)
        unsigned long long best = 0;
        for (int i = tid; i < nwg; i += blockDim.x) {
            const unsigned long long k =
                __hip_atomic_load(g.argmax_partial + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            best = k > best ? k : best;
        }
        best = block_max_key(best, (unsigned long long *)red);
        if (tid == 0) {
            DecodeCtl *ctl = g.ctl;
            const int idx = (int)(0xFFFFFFFFu - (uint32_t)(best & 0xFFFFFFFFull));
            ctl->last_argmax = idx;
            if (ctl->step >= ctl->n_prompt - 1 && ctl->n_out < g.max_out) {
                g.out_tokens[ctl->n_out] = idx;
                ctl->n_out += 1;
            }
            ctl->step += 1;
            ctl->pos += 1;
        }
    }
#undef BARRIER
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
struct MegaCombo {
    int t_qkv, t_wo, t_w13, t_w2, t_out;
    const void *fn;
};

#define Q4 L2H_TYPE_Q4_K
#define Q5 L2H_TYPE_Q5_K
#define Q6 L2H_TYPE_Q6_K
static const MegaCombo kCombos[] = {
    {Q4, Q4, Q4, Q4, Q6, (const void *)decode_token_kernel<Q4, Q4, Q4, Q4, Q6>},  // Q4_K_S style
    {Q4, Q4, Q4, Q4, Q4, (const void *)decode_token_kernel<Q4, Q4, Q4, Q4, Q4>},  // all q4_K
    {Q5, Q5, Q5, Q6, Q6, (const void *)decode_token_kernel<Q5, Q5, Q5, Q6, Q6>},  // Q5_K_M style
};
#undef Q4
#undef Q5
#undef Q6

static const MegaCombo *find_combo(int a, int b, int c, int d, int e) {
    for (const MegaCombo &k : kCombos)
        if (k.t_qkv == a && k.t_wo == b && k.t_w13 == c && k.t_w2 == d && k.t_out == e) return &k;
    return nullptr;
}

bool k_mega_supported(int t_qkv, int t_wo, int t_w13, int t_w2, int t_out) {
    return find_combo(t_qkv, t_wo, t_w13, t_w2, t_out) != nullptr;
}

size_t k_mega_lds_bytes(const MegaArgs &g, const PhaseArgs *ph) {
    size_t need = 0;
    for (int i = 0; i < 5; i++) {
        const PhaseArgs &p = ph[i];
        const int64_t K = p.w[0].ne0;
        const size_t b = (size_t)((K + K / 8 + K / 64 + 15) & ~(int64_t)15) + (size_t)p.rows_per_wg * p.ntpr * 8 +
                         (size_t)p.rows_per_wg * 4 + 16;
        need = std::max(need, b);
    }
    const size_t att = (size_t)g.hs * 8 + (size_t)g.seq_len * 8 + (size_t)(1024 / g.hs) * g.hs * 8 + (size_t)g.seq_len * 4;
    return std::max(need, att);
}

// copies the phase arguments of a model into the kernel's constant memory (stream-ordered)
hipError_t k_mega_bind(hipStream_t s, const PhaseArgs *ph) {
    std::vector<unsigned char> raw(5 * PHASE_BYTES, 0);
    for (int k = 0; k < 5; k++) memcpy(raw.data() + k * PHASE_BYTES, &ph[k], sizeof(PhaseArgs));
    hipError_t e = hipMemcpyToSymbolAsync(HIP_SYMBOL(c_phase_raw), raw.data(), raw.size(), 0, hipMemcpyHostToDevice, s);
    if (e != hipSuccess) return e;
    return hipStreamSynchronize(s);  // raw goes out of scope
}

hipError_t k_mega_launch(hipStream_t s, const MegaArgs &g, int t_qkv, int t_wo, int t_w13, int t_w2, int t_out, int grid,
                         size_t lds) {
    const MegaCombo *c = find_combo(t_qkv, t_wo, t_w13, t_w2, t_out);
    if (!c) return hipErrorInvalidValue;
    MegaArgs copy = g;
    void *args[] = {&copy};
    return hipLaunchCooperativeKernel(c->fn, dim3(grid), dim3(1024), args, (unsigned)lds, s);
}
