// One-way latency of a word handed from one workgroup to another: thread 0 of workgroup A stores a counter, thread 0
// of workgroup B polls it and answers in a second word, A polls that; half the round trip is printed.  Uncached or
// ordinary device memory, partner on the same XCD (workgroup 8) or on another one (workgroup 1); all other workgroups
// of the launch exit at once.  Stores and polls are the streaming decode kernel's (relaxed device-scope atomics).
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

__global__ __launch_bounds__(64) void k(unsigned *w, int partner, int rounds, long long *out) {
    if (threadIdx.x != 0) return;
    unsigned *ping = w, *pong = w + 64;  // (different 128-byte lines)
    if (blockIdx.x == 0) {
        const long long t0 = wall_clock64();
        for (int i = 1; i <= rounds; i++) {
            __hip_atomic_store(ping, (unsigned)i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            unsigned spins = 0;
            while (__hip_atomic_load(pong, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != (unsigned)i)
                if (++spins > 10000000u) return;
        }
        out[0] = wall_clock64() - t0;
    } else if ((int)blockIdx.x == partner) {
        for (int i = 1; i <= rounds; i++) {
            unsigned spins = 0;
            while (__hip_atomic_load(ping, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != (unsigned)i)
                if (++spins > 10000000u) return;
            __hip_atomic_store(pong, (unsigned)i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

int main() {
    unsigned *unc, *ord;
    long long *out;
    CHECK(hipExtMallocWithFlags((void **)&unc, 4096, hipDeviceMallocUncached));  // (never freed: the process ends)
    CHECK(hipMalloc(&ord, 4096));
    CHECK(hipMalloc(&out, 64));
    const int rounds = 2000;
    for (int mem = 0; mem < 2; mem++)
        for (int partner : {8, 1}) {
            unsigned *w = mem == 0 ? unc : ord;
            long long h = 0;
            for (int rep = 0; rep < 2; rep++) {
                CHECK(hipMemset(w, 0, 4096)); CHECK(hipMemset(out, 0, 64));
                k<<<16, 64>>>(w, partner, rounds, out);
                CHECK(hipDeviceSynchronize());
                CHECK(hipMemcpy(&h, out, 8, hipMemcpyDeviceToHost));
            }
            printf("%-9s memory, partner on %-12s: %6.3f us one way\n", mem == 0 ? "uncached" : "ordinary", partner == 8 ? "the same XCD" : "another XCD",
                   h * 0.01 / rounds / 2);
            fflush(stdout);
        }
    return 0;
}
