// The streaming decode kernel's q4_K piece loop (flow_loop_q4) alone: every wavefront runs it over its own stream,
// seven pieces a call, with the ring's fetches ("fetch") or over the same seven resident pieces again and again
// ("no fetch": the arithmetic and LDS traffic only), with 16, 8 or 4 wavefronts of the workgroup taking part.
// GB/s-equivalent = pieces x 1152 bytes per second over the whole chip.
#include "../k_flow.hip"
#include <stdio.h>
#include <stdlib.h>
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

template <int FETCH, int NW>
__global__ __launch_bounds__(1024) void mb_loop(const unsigned char *stream, int iters, long long per_wave_bytes, float *out) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned char *ring_base = s_ring + wave * (FLOW_D * FLOW_SLOT);
    for (int i = tid; i < FLOW_ACT_BYTES / 16; i += 1024) s_act[i] = make_uint4(0x01020304u * (i & 3), 0x7f017f01u, 0x01010101u, 0x02020202u);
    __syncthreads();
    Ring r;
    r.gptr = stream + ((long long)blockIdx.x * 16 + wave) * per_wave_bytes;
    r.lds = (unsigned)(size_t)ring_base;
    r.issued = r.consumed = r.drain_mark = 0;
    r.off = 0;
    r.left = 1 << 30;
    ring_uniform(r);
    if (wave >= NW) return;
    flow_top_up_q4(r, ring_base, lane);
    flow_drain(r);
    FlowGeom g;
    g.rpw = 56;
    g.ppr = 2;
    g.n_rows = gridDim.x * g.rpw;
    g.K = 4096;
    RegPieces rp;
    for (int it = 0; it < iters; it++) {
        if (!FETCH) {
            r.left = 0;
            r.issued = r.consumed + FLOW_D;
            r.drain_mark = r.issued;
        }
        flow_loop_q4<false, true>(g, r, ring_base, blockIdx.x, rp, 0);
    }
    flow_drain(r);
    if (s_part[tid & 255] == 1.2345) out[0] = 1.f;
}

int main() {
    const int iters = 120;  // x 7 pieces per wave per iteration
    const long long per_wave = (long long)(iters * 7 + 8) * FLOW_SLOT;
    const long long bytes = 256LL * 16 * per_wave;
    unsigned char *buf; float *out;
    CHECK(hipMalloc(&buf, bytes + 65536)); CHECK(hipMalloc(&out, 64));
    CHECK(hipMemset(buf, 0x11, bytes + 65536));
    hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    const double pieces = 256.0 * 16 * iters * 7;
#define RUN(name, launch, frac) do { for (int rep = 0; rep < 3; rep++) { CHECK(hipEventRecord(e0)); launch; CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1)); float ms; CHECK(hipEventElapsedTime(&ms, e0, e1)); if (rep == 2) printf("%-34s %8.3f ms  %7.1f GB/s-equivalent  %6.3f us per piece per wave\n", name, ms, pieces * (frac) * 1152 / ms / 1e6, ms * 1e3 / (iters * 7)); } CHECK(hipGetLastError()); fflush(stdout); } while (0)
    RUN("loop, no fetch, 16 waves", (mb_loop<0, 16><<<256, 1024>>>(buf, iters, per_wave, out)), 1.0);
    RUN("loop, fetch, 16 waves", (mb_loop<1, 16><<<256, 1024>>>(buf, iters, per_wave, out)), 1.0);
    RUN("loop, no fetch, 8 waves", (mb_loop<0, 8><<<256, 1024>>>(buf, iters, per_wave, out)), 0.5);
    RUN("loop, fetch, 8 waves", (mb_loop<1, 8><<<256, 1024>>>(buf, iters, per_wave, out)), 0.5);
    RUN("loop, no fetch, 4 waves", (mb_loop<0, 4><<<256, 1024>>>(buf, iters, per_wave, out)), 0.25);
    RUN("loop, fetch, 4 waves", (mb_loop<1, 4><<<256, 1024>>>(buf, iters, per_wave, out)), 0.25);
    return 0;
}
