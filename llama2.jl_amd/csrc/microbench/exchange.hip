// The cost of one "every workgroup reads the whole vector" hand-over through device memory in the style of the
// streaming decode kernel: 256 workgroups each store their share of a vector of n words (bare words, 0xFFFFFFFF =
// not there yet, three buffers in rotation), then all poll the whole vector with 16-byte coherent loads until no
// word is missing; nothing else happens between two hand-overs.  Uncached and ordinary device memory.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
#define EMPTY 0xFFFFFFFFu
typedef unsigned int u32x4v __attribute__((ext_vector_type(4)));

template <int CACHED_POLICY>
__global__ __launch_bounds__(1024) void k_exchange(unsigned *buf, int n, int iters, unsigned spin_limit, long long *t_out, unsigned *fail) {
    const int tid = threadIdx.x, wg = blockIdx.x, nwg = gridDim.x;
    const int per = n / nwg;  // words owned by a workgroup
    __shared__ int s_bad;
    if (tid == 0) s_bad = 0;
    __syncthreads();
    long long t0 = 0;
    for (int it = 0; it < iters; it++) {
        if (it == 8 && wg == 0 && tid == 0) t0 = wall_clock64();
        unsigned *cur = buf + (size_t)(it % 3) * n, *nxt = buf + (size_t)((it + 1) % 3) * n;
        if (tid < per) {
            __hip_atomic_store(cur + wg * per + tid, (unsigned)(it + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(nxt + wg * per + tid, EMPTY, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        unsigned spins = 0;
        for (int base = 0; base < n; base += 4096) {
            const int i = base + 4 * tid;
            if (i >= n) break;
            const u32x4v *p = (const u32x4v *)(cur + i);
            for (;;) {
                u32x4v w;
                asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(w) : "v"(p) : "memory");
                const bool full = w.x != EMPTY && w.y != EMPTY && w.z != EMPTY && w.w != EMPTY;
                if (__ballot(!full) == 0ull) break;
                if (++spins > spin_limit || ((spins & 1023) == 0 && __hip_atomic_load(fail, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                    s_bad = 1;
                    break;
                }
            }
        }
        __syncthreads();
        if (s_bad) {
            if (tid == 0) __hip_atomic_store(fail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }
    if (wg == 0 && tid == 0) t_out[0] = wall_clock64() - t0;
}

int main(int argc, char **argv) {
    const int iters = 2008;
    unsigned *buf_c, *buf_u; long long *t_out; unsigned *fail;
    const size_t words = 3 * 16384;
    CHECK(hipMalloc(&buf_c, words * 4));
    CHECK(hipExtMallocWithFlags((void **)&buf_u, words * 4, hipDeviceMallocUncached));
    CHECK(hipMalloc(&t_out, 64)); CHECK(hipMalloc(&fail, 64));
    int rate_khz = 0;
    CHECK(hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, 0));
#define RUN(name, buf, n) do { CHECK(hipMemset(buf, 0xFF, words * 4)); CHECK(hipMemset(fail, 0, 64)); CHECK(hipMemset(t_out, 0, 64)); int n_ = n; \
        void *args[] = {&buf, (void *)&n_, (void *)&iters, (void *)&spin, &t_out, &fail}; \
        CHECK(hipLaunchCooperativeKernel((const void *)k_exchange<0>, dim3(256), dim3(1024), args, 0, 0)); CHECK(hipDeviceSynchronize()); \
        long long t; unsigned f; CHECK(hipMemcpy(&t, t_out, 8, hipMemcpyDeviceToHost)); CHECK(hipMemcpy(&f, fail, 4, hipMemcpyDeviceToHost)); \
        printf("%-46s %s %8.3f us per exchange\n", name, f ? "GAVE UP" : "ok", (double)t / rate_khz * 1e3 / (iters - 8)); fflush(stdout); } while (0)
    const unsigned spin = 100000;
    RUN("uncached, 256 words (1 per wg)", buf_u, 256);
    RUN("uncached, 1024 words", buf_u, 1024);
    RUN("uncached, 4096 words", buf_u, 4096);
    RUN("uncached, 14336 words", buf_u, 14336);
    RUN("cached, 256 words", buf_c, 256);
    RUN("cached, 4096 words", buf_c, 4096);
    RUN("cached, 14336 words", buf_c, 14336);
    return 0;
}
