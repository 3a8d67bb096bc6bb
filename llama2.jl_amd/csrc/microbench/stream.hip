// How fast 256 workgroups x 16 wavefronts read 4.5 GB in the access patterns of the streaming decode kernel:
// a contiguous stream per wavefront in pieces of 1152 bytes moved into an LDS ring with global_load_lds (ring
// depth 7, 4, 2; nt or default cache policy), the same per workgroup, plain 16-byte loads into registers, and
// the usual grid-strided read for comparison.  (The register variants read 1024 of every 1152 bytes: their
// byte rate is 8/9 of the figure printed.)
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
typedef unsigned int u32x4v __attribute__((ext_vector_type(4)));

// mode 0: per-wave contiguous stream, pieces of 1152 B through LDS-DMA, ring of D slots
// mode 1: per-workgroup contiguous stream, piece i of a step belongs to wave i
// mode 2: per-wave stream, pieces of 1024 B (64 lanes x 16 B) only
template <int D, int MODE, int AUX>
__global__ __launch_bounds__(1024) void k_lds(const unsigned char *base, long long per_wave_pieces, unsigned *out) {
    __shared__ __attribute__((aligned(16))) unsigned char ring[16 * D * 1152];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    unsigned char *rb = ring + wave * D * 1152;
    const long long n = per_wave_pieces;
    const unsigned char *g;
    long long stride;
    if (MODE == 1) { g = base + ((long long)blockIdx.x * n * 16 + wave) * 1152; stride = 16 * 1152; }
    else { g = base + ((long long)blockIdx.x * 16 + wave) * n * 1152; stride = 1152; }
    int off = 0;
    unsigned acc = 0;
    long long issued = 0;
    for (; issued < D && issued < n; issued++) {
        const unsigned char *gl = g + issued * stride + lane * 16;
        unsigned char *slot = rb + (int)issued * 1152;
        if (MODE != 2) { if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 0, AUX); }
        __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 128, AUX);
    }
    for (long long i = 0; i < n; i++) {
        if (MODE != 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (D - 1)) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D - 1) : "memory");
        acc += *(volatile unsigned *)(rb + off + 128 + lane * 16);
        if (issued < n) {
            const unsigned char *gl = g + issued * stride + lane * 16;
            unsigned char *slot = rb + off;
            if (MODE != 2) { if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 0, AUX); }
            __builtin_amdgcn_global_load_lds((const AS1 void *)gl, (AS3 void *)slot, 16, 128, AUX);
            issued++;
        } else {
            // keep the count of outstanding operations constant: nothing to do, the waits become stricter
        }
        off += 1152;
        if (off == D * 1152) off = 0;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (acc == 0x12345678u) out[0] = acc;
}

// registers: each wave reads 1024-B pieces of its own stream with plain 16-byte loads, U in flight
template <int U, int NT>
__global__ __launch_bounds__(1024) void k_reg(const unsigned char *base, long long per_wave_pieces, unsigned *out) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const u32x4v *g = (const u32x4v *)(base + ((long long)blockIdx.x * 16 + wave) * per_wave_pieces * 1152) + lane;
    unsigned acc = 0;
    for (long long i = 0; i + U <= per_wave_pieces; i += U) {
        u32x4v v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = NT ? __builtin_nontemporal_load(g + (i + u) * 72) : g[(i + u) * 72];
#pragma unroll
        for (int u = 0; u < U; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x12345678u) out[0] = acc;
}

// plain grid-strided coalesced read of the whole buffer (the usual bandwidth test)
__global__ __launch_bounds__(1024) void k_plain(const u32x4v *base, long long n16, unsigned *out) {
    unsigned acc = 0;
    for (long long i = (long long)blockIdx.x * 1024 + threadIdx.x; i < n16; i += (long long)gridDim.x * 1024) {
        const u32x4v v = __builtin_nontemporal_load(base + i);
        acc += v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x12345678u) out[0] = acc;
}

int main() {
    const long long per_wave = 960;  // pieces per wave: 256*16*960*1152 = 4.53 GB
    const long long bytes = 256LL * 16 * per_wave * 1152;
    unsigned char *buf; unsigned *out;
    CHECK(hipMalloc(&buf, bytes + 65536)); CHECK(hipMalloc(&out, 64));
    CHECK(hipMemset(buf, 1, bytes + 65536));
    hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
#define RUN(name, launch) do { for (int rep = 0; rep < 3; rep++) { CHECK(hipEventRecord(e0)); launch; CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1)); float ms; CHECK(hipEventElapsedTime(&ms, e0, e1)); if (rep == 2) printf("%-40s %8.3f ms  %7.1f GB/s\n", name, ms, bytes / ms / 1e6); } CHECK(hipGetLastError()); fflush(stdout); } while (0)
    RUN("plain coalesced nt, 2048 wgs", (k_plain<<<2048, 1024>>>((const u32x4v *)buf, bytes / 16, out)));
    RUN("plain coalesced nt, 256 wgs", (k_plain<<<256, 1024>>>((const u32x4v *)buf, bytes / 16, out)));
    RUN("lds per-wave 1152 D7 nt", (k_lds<7, 0, 2><<<256, 1024>>>(buf, per_wave, out)));
    RUN("lds per-wave 1152 D7 aux0", (k_lds<7, 0, 0><<<256, 1024>>>(buf, per_wave, out)));
    RUN("lds per-wave 1152 D4 nt", (k_lds<4, 0, 2><<<256, 1024>>>(buf, per_wave, out)));
    RUN("lds per-wave 1152 D2 nt", (k_lds<2, 0, 2><<<256, 1024>>>(buf, per_wave, out)));
    RUN("lds per-wg interleaved 1152 D7 nt", (k_lds<7, 1, 2><<<256, 1024>>>(buf, per_wave, out)));
    RUN("lds per-wave 1024-only D7 nt", (k_lds<7, 2, 2><<<256, 1024>>>(buf, per_wave, out)));
    RUN("reg per-wave U4 nt", (k_reg<4, 1><<<256, 1024>>>(buf, per_wave, out)));
    RUN("reg per-wave U8 nt", (k_reg<8, 1><<<256, 1024>>>(buf, per_wave, out)));
    RUN("reg per-wave U8 plain", (k_reg<8, 0><<<256, 1024>>>(buf, per_wave, out)));
    return 0;
}
