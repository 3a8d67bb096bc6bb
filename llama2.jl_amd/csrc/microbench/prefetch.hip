// Do workgroups that only pull the weight streams into their XCD's L2 (ahead of the workgroups that consume them)
// shorten a layer?  Consumers: per-wavefront streams in pieces of 1152 B through a 7-slot LDS ring, a loop per phase
// (pieces per phase given), between the loops an exchange among all consumers plus a minimum wait; the arithmetic of
// a piece is emulated by a sleep.  Prefetchers: K workgroups per XCD touch one word per 128-byte line of the
// streams of their XCD's consumers, at most AHEAD pieces beyond what consumer 0 of the XCD has fetched.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#define AS1 __attribute__((address_space(1)))
#define AS3 __attribute__((address_space(3)))
#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)
#define D 7

struct Args {
    const unsigned char *buf;
    unsigned *xw;        // exchange words [256]
    unsigned *prog;      // [8] pieces fetched by consumer 0 of each XCD
    long long *out;      // [0] total ticks, [1] loop ticks (consumer 0)
    int n_layers, k_pref, ahead, aux, full;
    int pieces[4];       // per phase
    int wait_ticks[4];   // minimum wait before each phase's loop (10 ns ticks)
    int piece_ticks;     // emulated arithmetic per piece
    int ppl;             // pieces per layer and wavefront
};

__device__ __forceinline__ void sleep_until(long long t) {
    while ((long long)wall_clock64() < t) __builtin_amdgcn_s_sleep(1);
}

__global__ __launch_bounds__(1024) void mb_prefetch(Args a) {
    __shared__ __attribute__((aligned(16))) unsigned char ring[16 * D * 1152];
    __shared__ unsigned sink[16 * 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int NC = 32 - a.k_pref;  // consumers per XCD
    const long long total = (long long)a.n_layers * a.ppl;
    if (slot >= NC) {
        // ---- prefetcher j of this XCD ----
        const int j = slot - NC;
        const int n_lines = NC * 16 * 9;
        long long r = D;
        unsigned spins = 0;
        while (r < total) {
            long long p = (long long)__hip_atomic_load(a.prog + xcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            p = __builtin_amdgcn_readfirstlane((int)p);
            if (p >= total) break;
            if (r < p) r = p;
            long long limit = p + a.ahead;
            if (limit > total) limit = total;
            if (r >= limit) {
                if (++spins > 4000000u) break;
                __builtin_amdgcn_s_sleep(8);
                continue;
            }
            if (a.full) {
                // whole pieces, as the consumers fetch them, into a sink
                for (; r < limit; r++) {
                    for (int st = j * 16 + wave; st < NC * 16; st += a.k_pref * 16) {
                        const unsigned char *g = a.buf + ((((long long)xcd * NC * 16 + st) * total + r) * 1152) + lane * 16;
                        if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)g, (AS3 void *)(ring + wave * 1152), 16, 0, 0);
                        __builtin_amdgcn_global_load_lds((const AS1 void *)g, (AS3 void *)(ring + wave * 1152), 16, 128, 0);
                    }
                    asm volatile("s_waitcnt vmcnt(40)" ::: "memory");
                }
                continue;
            }
            for (; r < limit; r++) {
                for (int q = j * 1024 + tid; q < n_lines; q += a.k_pref * 1024) {
                    const int stream = q / 9, line = q - stream * 9;
                    const int cs = stream >> 4, cw = stream & 15;
                    const unsigned char *g = a.buf + ((((long long)xcd * NC + cs) * 16 + cw) * total + r) * 1152 + line * 128;
                    __builtin_amdgcn_global_load_lds((const AS1 void *)g, (AS3 void *)(sink + wave * 64), 4, 0, 0);
                }
                if ((r & 7) == 7) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        return;
    }
    // ---- consumer ----
    const int n_cons = NC * 8, cid = xcd * NC + slot;
    unsigned char *rb = ring + wave * D * 1152;
    const unsigned char *g = a.buf + (((long long)cid * 16 + wave) * total) * 1152 + lane * 16;
    long long issued = 0;
    auto fetch = [&](unsigned char *dst) {
        if (a.aux) {
            if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)(g + issued * 1152), (AS3 void *)dst, 16, 0, 2);
            __builtin_amdgcn_global_load_lds((const AS1 void *)(g + issued * 1152), (AS3 void *)dst, 16, 128, 2);
        } else {
            if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)(g + issued * 1152), (AS3 void *)dst, 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const AS1 void *)(g + issued * 1152), (AS3 void *)dst, 16, 128, 0);
        }
        issued++;
    };
    for (int i = 0; i < D; i++) fetch(rb + i * 1152);
    if (slot == 0 && tid == 0) __hip_atomic_store(a.prog + xcd, (unsigned)issued, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    int off = 0;
    unsigned acc = 0, epoch = 0;
    long long loop_ticks = 0;
    __syncthreads();
    const long long t_start = wall_clock64();
    long long t_end_loop = t_start;
    for (int l = 0; l < a.n_layers; l++) {
        for (int ph = 0; ph < 4; ph++) {
            // the hand-over: every consumer stores a word, everybody waits for all of them
            epoch++;
            if (tid == 0) __hip_atomic_store(a.xw + cid, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (tid < n_cons) {
                unsigned spins = 0;
                while (__hip_atomic_load(a.xw + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < epoch)
                    if (++spins > 2000000u) break;
            }
            __syncthreads();
            sleep_until(t_end_loop + a.wait_ticks[ph]);
            const long long t0 = wall_clock64();
            for (int i = 0; i < a.pieces[ph]; i++) {
                const long long tp = wall_clock64();
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (D - 1)) : "memory");
                acc += *(volatile unsigned *)(rb + off + 128 + lane * 16);
                if (issued < total) {
                    fetch(rb + off);
                } else {
                    // (the waits become stricter: fine)
                }
                if (slot == 0 && tid == 0) __hip_atomic_store(a.prog + xcd, (unsigned)issued, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                off += 1152;
                if (off == D * 1152) off = 0;
                sleep_until(tp + a.piece_ticks);
            }
            __syncthreads();
            t_end_loop = wall_clock64();
            loop_ticks += t_end_loop - t0;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (blockIdx.x == 0 && tid == 0) {
        a.out[0] = wall_clock64() - t_start;
        a.out[1] = loop_ticks;
    }
    if (acc == 0x12345678u) a.out[2] = acc;
}

// the prefetchers' own rate: K workgroups per XCD touch every 128-byte line of the pieces (vm 8) or load the pieces
// whole (vm 100); nothing else runs
__global__ __launch_bounds__(1024) void mb_touch(const unsigned char *buf, int k_pref, long long rounds, int vm) {
    __shared__ unsigned sink[16 * 64];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int NC = 32 - k_pref;
    if (slot < NC) return;
    const int j = slot - NC, n_lines = NC * 16 * 9;
    if (vm >= 100) {
        __shared__ __attribute__((aligned(16))) unsigned char rs[16 * 1152];
        const int lane = tid & 63;
        for (long long r = 0; r < rounds; r++) {
            for (int st = j * 16 + wave; st < NC * 16; st += k_pref * 16) {
                const unsigned char *g = buf + ((((long long)xcd * NC * 16 + st) * rounds + r) * 1152) + lane * 16;
                if (lane < 8) __builtin_amdgcn_global_load_lds((const AS1 void *)g, (AS3 void *)(rs + wave * 1152), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((const AS1 void *)g, (AS3 void *)(rs + wave * 1152), 16, 128, 0);
            }
            asm volatile("s_waitcnt vmcnt(40)" ::: "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        return;
    }
    for (long long r = 0; r < rounds; r++) {
        for (int q = j * 1024 + tid; q < n_lines; q += k_pref * 1024) {
            const int stream = q / 9, line = q - stream * 9;
            const int cs = stream >> 4, cw = stream & 15;
            const unsigned char *g = buf + ((((long long)xcd * NC + cs) * 16 + cw) * rounds + r) * 1152 + line * 128;
            __builtin_amdgcn_global_load_lds((const AS1 void *)g, (AS3 void *)(sink + wave * 64), 4, 0, 0);
        }
        if ((r & 7) == 7) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

int main(int argc, char **argv) {
    const int n_layers = 32;
    unsigned char *buf;
    const long long max_bytes = 256LL * 16 * 36 * n_layers * 1152 + (1 << 20);
    CHECK(hipMalloc(&buf, max_bytes));
    CHECK(hipMemset(buf, 1, max_bytes));
    unsigned *xw, *prog;
    long long *out;
    CHECK(hipExtMallocWithFlags((void **)&xw, 4096, hipDeviceMallocUncached));  // (never freed: the process ends)
    CHECK(hipMalloc(&prog, 64));
    CHECK(hipMalloc(&out, 64));
    {
        hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
        for (int k : {2, 4, 8, 16}) for (int vm : {8, 100}) {
            const long long rounds = 960; const int NC = 32 - k;
            float ms = 0;
            for (int rep = 0; rep < 2; rep++) {
                CHECK(hipEventRecord(e0)); mb_touch<<<256, 1024>>>(buf, k, rounds, vm); CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1));
                CHECK(hipEventElapsedTime(&ms, e0, e1));
            }
            const double bytes = NC * 8 * 16.0 * rounds * 1152;
            printf("prefetchers alone: %2d per XCD, %-13s: %7.3f ms  %7.1f GB/s of lines\n", k, vm == 8 ? "lines touched" : "whole pieces", ms, bytes / ms / 1e6);
            fflush(stdout);
        }
    }
    struct Case { const char *name; int k, ahead, aux, pieces[4], piece_ticks, full; };
    // 32 consumers per XCD: 3+2+14+7 = 26 pieces per wavefront and layer = 122.7 MB; 28: 3+3+16+8 = 30 -> 123.9 MB;
    // 24: 4+3+18+10 = 35 -> 123.9 MB
    const Case cases[] = {
        {"no prefetchers, 0.53 us/piece, nt", 0, 0, 1, {3, 2, 14, 7}, 53, 0},
        {"no prefetchers, 0.21 us/piece, nt", 0, 0, 1, {3, 2, 14, 7}, 21, 0},
        {"2 per XCD, lines touched, 6 pieces ahead", 2, 6, 0, {3, 2, 15, 8}, 21, 0},
        {"4 per XCD, lines touched, 6 pieces ahead", 4, 6, 0, {3, 3, 16, 8}, 21, 0},
        {"4 per XCD, whole pieces, 6 ahead", 4, 6, 0, {3, 3, 16, 8}, 21, 1},
        {"4 per XCD, whole pieces, 30 ahead (a layer)", 4, 30, 0, {3, 3, 16, 8}, 21, 1},
        {"8 per XCD, whole pieces, 6 ahead", 8, 6, 0, {4, 3, 18, 10}, 21, 1},
        {"8 per XCD, whole pieces, 35 ahead (a layer)", 8, 35, 0, {4, 3, 18, 10}, 21, 1},
    };
    for (const Case &c : cases) {
        Args a;
        a.buf = buf; a.xw = xw; a.prog = prog; a.out = out;
        a.n_layers = n_layers; a.k_pref = c.k; a.ahead = c.ahead; a.aux = c.aux; a.full = c.full;
        a.ppl = 0;
        for (int i = 0; i < 4; i++) { a.pieces[i] = c.pieces[i]; a.ppl += c.pieces[i]; }
        // waits of the kernel's timeline: before q|k|v 3.4 + 0.6 (epilogue of w2), wo 6.0 + 1.2 + 0.6, w1|w3 3.2 + 0.4, w2 5.0 + 0.8
        const int w[4] = {400, 780, 360, 580};
        for (int i = 0; i < 4; i++) a.wait_ticks[i] = w[i];
        a.piece_ticks = c.piece_ticks;
        const double mb = (32 - c.k) * 8 * 16.0 * a.ppl * 1152 / 1e6;
        for (int rep = 0; rep < 2; rep++) {
            CHECK(hipMemset(xw, 0, 4096)); CHECK(hipMemset(prog, 0, 64)); CHECK(hipMemset(out, 0, 64));
            mb_prefetch<<<256, 1024>>>(a);
            CHECK(hipDeviceSynchronize());
        }
        long long h[2];
        CHECK(hipMemcpy(h, out, 16, hipMemcpyDeviceToHost));
        printf("%-48s %6.1f MB/layer  %6.2f us/layer  loops %6.2f  waits %6.2f\n", c.name, mb, h[0] * 0.01 / n_layers,
               h[1] * 0.01 / n_layers, (h[0] - h[1]) * 0.01 / n_layers);
        fflush(stdout);
    }
    return 0;
}
