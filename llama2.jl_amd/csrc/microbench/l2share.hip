// Does a workgroup find in its XCD's L2 what another workgroup of the same XCD loaded a moment ago?
// Workgroup (xcd, slot 0) loads a private region; then (xcd, slot 1) reads the same region, (xcd, slot 2) the region
// of the next XCD, (xcd, slot 3) a region nobody touched; each times its read with the wall clock.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
typedef unsigned int u32x4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned read_region(const u32x4v *p, long long n16) {
    unsigned acc = 0;
    for (long long i = threadIdx.x; i < n16; i += 4 * 1024) {
        u32x4v v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = i + u * 1024 < n16 ? p[i + u * 1024] : u32x4v{0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < 4; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    return acc;
}

__global__ __launch_bounds__(1024) void k(const unsigned char *buf, long long region, unsigned *flags, long long *out) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const long long n16 = region / 16;
    unsigned acc = 0;
    if (slot == 0) {
        acc = read_region((const u32x4v *)(buf + xcd * region), n16);
        __syncthreads();
        if (threadIdx.x == 0) __hip_atomic_store(flags + xcd, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    } else if (slot <= 3) {
        // wait until every loader is done
        if (threadIdx.x < 8) {
            unsigned spins = 0;
            while (__hip_atomic_load(flags + threadIdx.x, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) == 0u)
                if (++spins > 20000000u) break;
        }
        __syncthreads();
        const int r = slot == 1 ? xcd : (slot == 2 ? (xcd + 1) & 7 : 8 + xcd);
        const long long t0 = wall_clock64();
        acc = read_region((const u32x4v *)(buf + r * region), n16);
        __syncthreads();
        if (threadIdx.x == 0) out[slot * 8 + xcd] = wall_clock64() - t0;
    }
    if (acc == 0x12345678u) out[63] = acc;
}

int main() {
    unsigned char *buf; unsigned *flags; long long *out;
    const long long max_region = 4 << 20;
    CHECK(hipMalloc(&buf, 16 * max_region)); CHECK(hipMemset(buf, 1, 16 * max_region));
    CHECK(hipMalloc(&flags, 64)); CHECK(hipMalloc(&out, 512));
    // scrub the caches between runs by reading something large
    unsigned char *big; CHECK(hipMalloc(&big, 1LL << 30));
    for (long long region : {256LL << 10, 1LL << 20, 2LL << 20, 4LL << 20}) {
        CHECK(hipMemset(big, 2, 1LL << 30));
        CHECK(hipMemset(flags, 0, 64)); CHECK(hipMemset(out, 0, 512));
        k<<<256, 1024>>>(buf, region, flags, out);
        CHECK(hipDeviceSynchronize());
        long long h[64]; CHECK(hipMemcpy(h, out, 512, hipMemcpyDeviceToHost));
        const char *names[4] = {"", "same XCD's region", "next XCD's region", "untouched region"};
        for (int s = 1; s <= 3; s++) {
            double sum = 0; for (int x = 0; x < 8; x++) sum += h[s * 8 + x] * 0.01;
            printf("region %5lld KiB, %-18s: %7.2f us on average = %6.1f GB/s per workgroup\n", region >> 10, names[s], sum / 8,
                   region / (sum / 8) / 1e3);
        }
        fflush(stdout);
    }
    return 0;
}
