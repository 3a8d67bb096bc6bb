// What delays a poll: the requests that its own wavefront has in flight, those of the other wavefronts of its CU, or
// the load on the memory system as a whole?  Wavefront 0 of a workgroup reads one 16-byte word of uncached memory
// after the other (each read waited for, as a poll is) and reports the average round trip, while
//   A  nothing else runs,
//   B  the other 15 wavefronts of every workgroup stream their own bytes through LDS rings (7 pieces of 1152 B in
//      flight each),
//   C  as B, and wavefront 0 itself has six such pieces in flight in front of every poll,
//   D  the streaming wavefronts are those of the odd workgroups only (all 16 of them, 14 pieces in flight each); the
//      polls come from the even workgroups, whose CUs do nothing else.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
typedef unsigned int u32x4v __attribute__((ext_vector_type(4)));

template <int DEPTH>
__device__ __forceinline__ void stream_wave(const unsigned char *g, unsigned char *rb, long long n, int lane, const unsigned *stop) {
    long long issued = 0;
    for (; issued < DEPTH; issued++) {
        if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)(g + issued * 1152 + lane * 16), (AS3 void *)(rb + (issued % 7) * 1152), 16, 0, 2);
        __builtin_amdgcn_global_load_lds((const AS1 void *)(g + issued * 1152 + lane * 16), (AS3 void *)(rb + (issued % 7) * 1152), 16, 128, 2);
    }
    for (long long i = 0; i < n; i++) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (DEPTH - 1)) : "memory");
        if ((i & 15) == 0 && __hip_atomic_load(stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
        if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)(g + issued * 1152 + lane * 16), (AS3 void *)(rb + (issued % 7) * 1152), 16, 0, 2);
        __builtin_amdgcn_global_load_lds((const AS1 void *)(g + issued * 1152 + lane * 16), (AS3 void *)(rb + (issued % 7) * 1152), 16, 128, 2);
        issued++;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// mode 0 = A, 1 = B, 2 = C, 3 = D
__global__ __launch_bounds__(1024) void k(const unsigned char *buf, long long per_wave, const u32x4v *words, int n_polls, int mode,
                                          unsigned *stop, long long *out) {
    __shared__ __attribute__((aligned(16))) unsigned char ring[16 * 7 * 1152];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned char *g = buf + ((long long)blockIdx.x * 16 + wave) * (per_wave + 16) * 1152;
    unsigned char *rb = ring + wave * 7 * 1152;
    const bool poller = wave == 0 && (mode != 3 || (blockIdx.x & 1) == 0);
    const bool streamer = mode == 3 ? (blockIdx.x & 1) == 1 : (mode != 0 && wave != 0);
    if (poller) {
        // a lane reads its own 16 bytes of a 1 KiB record; records are visited in a scattered order
        unsigned acc = 0;
        long long fetched = 0;
        __builtin_amdgcn_s_sleep(64);  // (let the streams get going)
        const long long t0 = wall_clock64();
        for (int i = 0; i < n_polls; i++) {
            if (mode == 2) {
                for (int u = 0; u < 6; u++, fetched++) {
                    if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)(g + (fetched % per_wave) * 1152 + lane * 16), (AS3 void *)(rb + u * 1152), 16, 0, 2);
                    __builtin_amdgcn_global_load_lds((const AS1 void *)(g + (fetched % per_wave) * 1152 + lane * 16), (AS3 void *)(rb + u * 1152), 16, 128, 2);
                }
            }
            const u32x4v *p = words + (((long long)blockIdx.x * 997 + (long long)i * 61) & 4095) * 64 + lane;
            u32x4v w;
            asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(w) : "v"(p) : "memory");
            acc += w.x;
        }
        const long long t1 = wall_clock64();
        if (lane == 0) out[blockIdx.x] = t1 - t0;
        if (acc == 0x12345678u) out[300] = acc;
        if (lane == 0) __hip_atomic_fetch_add(stop + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the last poller to finish stops the streams
        const unsigned n_pollers = mode == 3 ? gridDim.x / 2 : gridDim.x;
        if (lane == 0 && __hip_atomic_load(stop + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= n_pollers)
            __hip_atomic_store(stop, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if (streamer) {
        if (mode == 3) stream_wave<14>(g, rb, per_wave, lane, stop);
        else stream_wave<7>(g, rb, per_wave, lane, stop);
    }
}

int main() {
    const long long per_wave = 900;
    const long long bytes = 256LL * 16 * (per_wave + 16) * 1152;
    unsigned char *buf; u32x4v *words; unsigned *stop; long long *out;
    CHECK(hipMalloc(&buf, bytes)); CHECK(hipMemset(buf, 1, bytes));
    CHECK(hipExtMallocWithFlags((void **)&words, 4096 * 1024, hipDeviceMallocUncached));  // (never freed: the process ends)
    CHECK(hipMemset(words, 0, 4096 * 1024));
    CHECK(hipMalloc(&stop, 64)); CHECK(hipMalloc(&out, 4096));
    const char *names[4] = {"A  nothing else runs", "B  the CU's other 15 wavefronts stream", "C  as B, and six pieces of its own in front of every poll",
                            "D  polls from idle CUs, the other half of the chip streams"};
    const int n_polls = 100;
    for (int mode = 0; mode < 4; mode++) {
        for (int rep = 0; rep < 2; rep++) {
            CHECK(hipMemset(stop, 0, 64)); CHECK(hipMemset(out, 0, 4096));
            k<<<256, 1024>>>(buf, per_wave, words, n_polls, mode, stop, out);
            CHECK(hipDeviceSynchronize());
        }
        long long h[256]; CHECK(hipMemcpy(h, out, 2048, hipMemcpyDeviceToHost));
        double sum = 0, mx = 0; int n = 0;
        for (int i = 0; i < 256; i++) if (h[i]) { const double us = h[i] * 0.01 / n_polls; sum += us; mx = us > mx ? us : mx; n++; }
        printf("%-62s: %6.2f us per poll (average over %d polling wavefronts; slowest %6.2f)\n", names[mode], sum / n, n, mx);
        fflush(stdout);
    }
    return 0;
}
