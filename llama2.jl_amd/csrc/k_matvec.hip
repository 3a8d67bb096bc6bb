// matmul!(y, A, x) for one input vector (reference src/matmul.jl:3-23) with the neighbouring
// element-wise steps of transformer! (src/inference.jl:244-305) fused in:
//   prologue  rmsnorm! (+ q8_K quantization of the activations) or plain quantization,
//             done by every workgroup into its own LDS copy;
//   body      k-quant weights x q8_K activations: nibbles/bit-planes unpacked in registers,
//             packed-int8 dot instructions, per-chunk integers scaled and summed in fp64;
//             F32 weights x fp32 activations: fp64 sum of exact products;
//   epilogue  store | residual add | SwiGLU | RoPE + KV-cache append.
// Every output row is fp32(sum of exact fp64 terms), so the value does not depend on how
// lanes, wavefronts and workgroups split the row.
//
// Work split: each workgroup owns a contiguous range of rows (one contiguous region of each
// weight stream, read with non-temporal 16-byte lane loads) and cuts it into equal tiles that its
// 16 wavefronts take round-robin; because fp64 sums may be split anywhere, a row can be shared
// by several wavefronts when a workgroup has few rows.
#include "matvec_dev.h"

template <int TYPE, int PRO, int EPI, bool DEBUG>
__global__ __launch_bounds__(1024) void matvec_kq_kernel(PhaseArgs a) {
    extern __shared__ uint4 smem[];
    __shared__ double red[16];
    __shared__ int s_next;
    Tile<TYPE> cur;
    matvec_phase<TYPE, PRO, EPI, DEBUG, false>(a, 0, blockIdx.x, smem, red, &s_next, cur, false);
}

// F32 weights: y[row] = fp32(sum_fp64 A[row][k] * x[k]); same prologues and epilogues; one
// wavefront per pair of logical rows.
template <int PRO, int EPI>
__global__ __launch_bounds__(1024) void matvec_f32_kernel(PhaseArgs a) {
    extern __shared__ uint4 smem[];
    __shared__ double red[16];
    const int64_t K = a.w[0].ne0;
    float *s_x = (float *)smem;
    stage_activations<PRO, false, false>(a, 0, K, nullptr, nullptr, nullptr, s_x, red);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int64_t L_lo = (int64_t)blockIdx.x * a.rows_per_wg;
    const int64_t L_hi = min(a.n_rows, L_lo + a.rows_per_wg);
    for (int64_t L = L_lo + 2 * wave; L < L_hi; L += 2 * nwaves) {
        double acc[2] = {0.0, 0.0};
#pragma unroll
        for (int r = 0; r < 2; r++) {
            if (L + r >= L_hi) continue;
            const RowRef rr = logical_row<EPI>(a, L + r);
            if (rr.seg < 0) continue;
            const float *wr = (rr.seg == 0 ? a.w[0].f32 : (rr.seg == 1 ? a.w[1].f32 : a.w[2].f32)) + rr.row * K;
            if ((K & 3) == 0) {
                const float4 *w4 = (const float4 *)wr;
                const float4 *x4 = (const float4 *)s_x;
                for (int64_t i = lane; i < K / 4; i += WAVE) {
                    const float4 wv = w4[i], xv = x4[i];
                    acc[r] = fma((double)wv.x, (double)xv.x, acc[r]);
                    acc[r] = fma((double)wv.y, (double)xv.y, acc[r]);
                    acc[r] = fma((double)wv.z, (double)xv.z, acc[r]);
                    acc[r] = fma((double)wv.w, (double)xv.w, acc[r]);
                }
            } else {
                for (int64_t i = lane; i < K; i += WAVE) acc[r] = fma((double)wr[i], (double)s_x[i], acc[r]);
            }
        }
        const float v0 = (float)wave_sum_f64_dpp(acc[0]), v1 = (float)wave_sum_f64_dpp(acc[1]);
        if (lane < 2 && L + lane < L_hi) finish_row<EPI, false>(a, 0, L + lane, lane == 0 ? v0 : v1, lane == 0 ? v1 : v0);
    }
}

// ------------------------------------------------------------------------------------------
// launch
// ------------------------------------------------------------------------------------------
template <int TYPE, int PRO, int EPI, bool DEBUG>
static hipError_t launch_one(hipStream_t s, const PhaseArgs &a, int grid) {
    const int64_t K = a.w[0].ne0;
    if constexpr (TYPE == L2H_TYPE_F32) {
        const size_t lds = (size_t)K * 4;
        if (lds > 64 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void *)matvec_f32_kernel<PRO, EPI>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL((matvec_f32_kernel<PRO, EPI>), dim3(grid), dim3(1024), lds, s, a);
    } else {
        const size_t lds = (size_t)((K + K / 8 + K / 64 + 15) & ~(int64_t)15) + (size_t)a.rows_per_wg * a.ntpr * 8 +
                           (size_t)a.rows_per_wg * 4 + 16;
        if (lds > 64 * 1024) return hipErrorInvalidValue;
        hipLaunchKernelGGL((matvec_kq_kernel<TYPE, PRO, EPI, DEBUG>), dim3(grid), dim3(1024), lds, s, a);
    }
    return hipGetLastError();
}

template <int TYPE>
static hipError_t launch_type(hipStream_t s, const PhaseArgs &a, int pro, int epi, int grid) {
    const bool dbg = a.dbg_isc != nullptr;
#define CASE(P, E)                                                    \
    if (pro == P && epi == E) {                                       \
        if constexpr (TYPE != L2H_TYPE_F32 && E == EPI_STORE) {       \
            if (dbg) return launch_one<TYPE, P, E, true>(s, a, grid); \
        }                                                             \
        return launch_one<TYPE, P, E, false>(s, a, grid);             \
    }
    CASE(PRO_RMSNORM, EPI_ROPE_KV)
    CASE(PRO_QUANT, EPI_RESID)
    CASE(PRO_RMSNORM, EPI_SWIGLU)
    CASE(PRO_RMSNORM, EPI_STORE)
    CASE(PRO_QUANT, EPI_STORE)
#undef CASE
    return hipErrorInvalidValue;
}

int k_matvec_plan(PhaseArgs &a, int epi) {
    const int type = a.w[0].type;
    for (int i = 1; i < a.nseg; i++)
        if (a.w[i].type != type || a.w[i].ne0 != a.w[0].ne0) return -1;
    int64_t rows = 0;
    for (int i = 0; i < a.nseg; i++) {
        if (epi == EPI_ROPE_KV && (a.w[i].ne1 & 1)) return -1;
        rows += a.w[i].ne1;
    }
    if (epi == EPI_SWIGLU && (a.nseg != 2 || a.w[0].ne1 != a.w[1].ne1)) return -1;
    a.n_rows = rows;
    if (rows == 0) return 0;
    // contiguous, even-sized row ranges; at most max_grid workgroups, at most 2048 rows each
    int64_t grid = std::min<int64_t>(a.max_grid, (rows + 1) / 2);
    grid = std::max<int64_t>(grid, (rows + 2047) / 2048);
    if (grid < 1) grid = 1;
    int64_t rpw = (rows + grid - 1) / grid;
    rpw += rpw & 1;
    grid = (rows + rpw - 1) / rpw;
    a.rows_per_wg = (int)rpw;
    a.rt = a.st = a.ntpr = 1;
    if (type != L2H_TYPE_F32) {
        const int nslot = type == L2H_TYPE_Q4_K ? 4 : 2;
        const int cpb = type == L2H_TYPE_Q6_K ? 4 : 8;
        const int nsteps = (int)((a.w[0].nb * cpb + 63) / 64);
        int st = std::min(nsteps, nslot);
        int rt = nslot / st;
        // keep all 16 wavefronts busy when the workgroup has few rows
        while (rt > 1 && ((rpw + rt - 1) / rt) * ((nsteps + st - 1) / st) < 16) rt >>= 1;
        while (st > 1 && rt == 1 && rpw * ((nsteps + st - 1) / st) < 16) st = (st + 1) / 2;
        a.rt = rt;
        a.st = st;
        a.ntpr = (nsteps + st - 1) / st;
    }
    return (int)grid;
}

hipError_t k_matvec(hipStream_t s, PhaseArgs a, int pro, int epi) {
    const int type = a.w[0].type;
    const int grid = k_matvec_plan(a, epi);
    if (grid < 0) return hipErrorInvalidValue;
    if (grid == 0) return hipSuccess;
    switch (type) {
    case L2H_TYPE_Q4_K: return launch_type<L2H_TYPE_Q4_K>(s, a, pro, epi, (int)grid);
    case L2H_TYPE_Q5_K: return launch_type<L2H_TYPE_Q5_K>(s, a, pro, epi, (int)grid);
    case L2H_TYPE_Q6_K: return launch_type<L2H_TYPE_Q6_K>(s, a, pro, epi, (int)grid);
    case L2H_TYPE_F32: return launch_type<L2H_TYPE_F32>(s, a, pro, epi, (int)grid);
    }
    return hipErrorInvalidValue;
}

// ------------------------------------------------------------------------------------------
// The prologue alone, with its LDS image copied out: what the single-operator entry points
// (rmsnorm, q8_K quantization) run, so that they exercise the code the matvec kernels use.
// ------------------------------------------------------------------------------------------
template <int PRO, bool KQ>
__global__ __launch_bounds__(1024) void stage_dump_kernel(PhaseArgs a, int64_t n, Q8Dev q8_out, float *f32_out) {
    extern __shared__ uint4 smem[];
    __shared__ double red[16];
    // PRO_QUANT blocks are independent: each workgroup takes a slice of up to 8192 elements
    const int64_t off = PRO == PRO_QUANT ? (int64_t)blockIdx.x * 8192 : 0;
    const int64_t len = PRO == PRO_QUANT ? min((int64_t)8192, n - off) : n;
    a.xf += off;
    int8_t *s_qs = (int8_t *)smem;
    int16_t *s_bs = (int16_t *)(s_qs + len);
    float *s_d = (float *)(s_qs + len + len / 8);
    float *s_xf = (float *)smem;
    stage_activations<PRO, KQ, false>(a, 0, len, s_qs, s_bs, s_d, s_xf, red);
    __syncthreads();
    if (KQ) {
        for (int64_t i = threadIdx.x; i < len; i += blockDim.x) q8_out.qs[off + i] = s_qs[i];
        for (int64_t i = threadIdx.x; i < len / 16; i += blockDim.x) q8_out.bsums[off / 16 + i] = s_bs[i];
        for (int64_t i = threadIdx.x; i < len / 256; i += blockDim.x) q8_out.d[off / 256 + i] = s_d[i];
    } else {
        for (int64_t i = threadIdx.x; i < len; i += blockDim.x) f32_out[off + i] = s_xf[i];
    }
}

// quantize_row_q8_K with four blocks per wavefront, a block per row of 16 lanes: the form in which the streaming decode
// kernel stages its inputs (q8k_quantize_rows16); the stand-alone quantizer runs it beside the one-block-per-wavefront
// form and compares, so that its tests pin both
__global__ __launch_bounds__(64) void quantize_rows16_kernel(const float *x, int64_t nb, Q8Dev out) {
    const int lane = threadIdx.x, g = lane & 15;
    const int64_t b = 4 * (int64_t)blockIdx.x + (lane >> 4);
    const bool there = b < nb;  // (a row without a block works on zeros and stores nothing)
    float v[16];
#pragma unroll
    for (int k = 0; k < 16; k++) v[k] = there ? x[256 * b + 16 * g + k] : 0.0f;
    q8k_u32x4 packed;
    int bsum;
    float d;
    q8k_quantize_rows16(v, packed, bsum, d);
    if (there) {
        ((q8k_u32x4 *)out.qs)[16 * b + g] = packed;
        out.bsums[16 * b + g] = (int16_t)bsum;
        if (g == 0) out.d[b] = d;
    }
}

hipError_t k_quantize_rows16(hipStream_t s, const float *x, int64_t n, Q8Dev q8_out) {
    const int64_t nb = n / 256;
    hipLaunchKernelGGL(quantize_rows16_kernel, dim3((unsigned)((nb + 3) / 4)), dim3(64), 0, s, x, nb, q8_out);
    return hipGetLastError();
}

hipError_t k_stage_dump(hipStream_t s, const float *x, const float *normw, int64_t n, int pro, Q8Dev q8_out,
                        float *f32_out) {
    PhaseArgs a{};
    a.xf = x;
    a.normw = normw;
    const bool kq = f32_out == nullptr;
    if (pro == PRO_QUANT && kq) {
        const int grid = (int)((n + 8191) / 8192);
        hipLaunchKernelGGL((stage_dump_kernel<PRO_QUANT, true>), dim3(grid), dim3(1024), 8192 + 1024 + 128 + 16, s, a, n,
                           q8_out, f32_out);
    } else if (pro == PRO_RMSNORM) {
        if (n > 16384 - 1024) return hipErrorInvalidValue;
        const size_t lds = kq ? (size_t)(n + n / 8 + n / 64 + 16) : (size_t)n * 4;
        if (kq)
            hipLaunchKernelGGL((stage_dump_kernel<PRO_RMSNORM, true>), dim3(1), dim3(1024), lds, s, a, n, q8_out, f32_out);
        else
            hipLaunchKernelGGL((stage_dump_kernel<PRO_RMSNORM, false>), dim3(1), dim3(1024), lds, s, a, n, q8_out,
                               f32_out);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
