// How fast can NF wavefronts per CU (256 workgroups) stream with global_load_lds_dwordx4, each keeping D requests of
// 1 KiB in flight (s_waitcnt vmcnt(D - 1) after every request)?  Nothing else runs: the ceiling of a design in which
// a few wavefronts do all the fetching.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))
__shared__ __attribute__((aligned(16))) unsigned char s_ring[16 * 8192];
template <int D>
__global__ __launch_bounds__(1024) void k(const unsigned char *src, int nf, int iters, float *out) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (wave >= nf) return;
    const unsigned char *g = src + ((long long)blockIdx.x * 16 + wave) * (long long)iters * 1024 + lane * 16;
    unsigned char *base = s_ring + wave * 8192;
    for (int i = 0; i < iters; i++) {
        __builtin_amdgcn_global_load_lds((const AS1 void *)g, (AS3 void *)(base + (i & 7) * 1024), 16, 0, 2);
        g += 1024;
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D - 1) : "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (s_ring[tid] == 77 && out) out[0] = 1.f;
}
int main() {
    const int iters_total = 16 * 1200;  // KB per CU
    unsigned char *buf; float *out;
    const long long bytes = 256LL * iters_total * 1024;
    CHECK(hipMalloc(&buf, bytes + 65536)); CHECK(hipMalloc(&out, 64));
    CHECK(hipMemset(buf, 1, bytes));
    hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
#define RUN(D, NF) do { const int iters = iters_total / 16; for (int rep = 0; rep < 3; rep++) { CHECK(hipEventRecord(e0)); k<D><<<256, 1024>>>(buf, NF, iters, out); CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1)); float ms; CHECK(hipEventElapsedTime(&ms, e0, e1)); if (rep == 2) printf("in flight %2d, %2d wavefronts per CU: %7.1f GB/s  (%5.2f KB/us per wavefront)\n", D, NF, 256.0 * NF * iters * 1024 / ms / 1e6, iters * 1.024 / (ms * 1e3)); } CHECK(hipGetLastError()); fflush(stdout); } while (0)
    RUN(8, 1); RUN(16, 1); RUN(32, 1); RUN(60, 1);
    RUN(8, 2); RUN(16, 2); RUN(32, 2); RUN(60, 2);
    RUN(8, 4); RUN(32, 4); RUN(60, 4);
    RUN(8, 8); RUN(32, 8);
    RUN(8, 16); RUN(32, 16);
    return 0;
}
