// Memory-system ceilings for the access patterns of the search and build kernels, measured on the
// GPU this runs on: what a kernel that does nothing but the loads can reach. The evaluation kernels
// are gathers of whole records at random addresses; HBM delivers such chunks well below its streaming
// rate, the more so the shorter they are, and returning atomics on a large visited bitmap take a
// share of the same memory system. Prints one line per case; no input, about a second of GPU time.
//
//   chunk reads:  every wave reads random, 128-byte aligned chunks of a 5 GiB buffer, DEPTH chunks in
//                 flight (the loads of all of them are issued before the first is consumed)
//   with atomics: the same 1 KiB reads plus `per_chunk` random 4-byte atomicOr (value returned) on a
//                 private 128 KiB region per workgroup (the visited bitmap of one query at 1 M docs)
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#define CK(x)                                                                         \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            fprintf(stderr, "membench: %s (line %d)\n", hipGetErrorString(e_), __LINE__); \
            exit(1);                                                                  \
        }                                                                             \
    } while (0)

__device__ inline uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

constexpr int DEPTH = 3;

// LOADS x 1 KiB per chunk (dwordx4 per lane and load) or, with SMALL, LOADS x 256 B (dword per lane).
template <int LOADS, bool SMALL>
__global__ __launch_bounds__(256) void chunk_reads(const char* buf, uint64_t lines, uint32_t iters, uint32_t* bitmap, uint32_t words_per_block,
                                                   uint32_t atomic_lanes, uint32_t* sink) {
    const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) / 64, lane = threadIdx.x & 63;
    uint32_t* mine = bitmap + (size_t)blockIdx.x * words_per_block;
    uint32_t acc = 0;
    for (uint32_t it = 0; it < iters; it++) {
        uint4 v[DEPTH][LOADS];
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            const uint64_t r = mix64(((uint64_t)wave << 32) | (it * DEPTH + d));
            const char* p = buf + (r % lines) * 128;
#pragma unroll
            for (int c = 0; c < LOADS; c++) {
                if (SMALL) v[d][c] = make_uint4(reinterpret_cast<const uint32_t*>(p)[lane + 64 * c], 0, 0, 0);
                else v[d][c] = reinterpret_cast<const uint4*>(p)[lane + 64 * c];
            }
        }
        if (lane < atomic_lanes) {
            const uint64_t r = mix64(((uint64_t)(wave * 64 + lane) << 32) | (0x80000000u + it));
            acc ^= atomicOr(&mine[(r >> 8) % words_per_block], 1u << (r & 31));
        }
#pragma unroll
        for (int d = 0; d < DEPTH; d++)
#pragma unroll
            for (int c = 0; c < LOADS; c++) acc ^= v[d][c].x ^ v[d][c].y ^ v[d][c].z ^ v[d][c].w;
    }
    if (acc == 0x12345678u) sink[0] = acc; // keeps the loads alive
}

template <int LOADS, bool SMALL>
static void run(const char* buf, uint64_t bytes, uint32_t* bitmap, uint32_t words_per_block, uint32_t atomic_lanes, uint32_t* sink, uint32_t grid,
                hipEvent_t e0, hipEvent_t e1) {
    const uint32_t chunk = LOADS * (SMALL ? 256u : 1024u);
    const uint32_t iters = 6000000u / chunk + 200;
    const uint64_t lines = (bytes - 16384) / 128;
    chunk_reads<LOADS, SMALL><<<grid, 256>>>(buf, lines, iters / 4, bitmap, words_per_block, atomic_lanes, sink);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    chunk_reads<LOADS, SMALL><<<grid, 256>>>(buf, lines, iters, bitmap, words_per_block, atomic_lanes, sink);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double chunks = (double)grid * 4 * iters * DEPTH;
    if (atomic_lanes == 0)
        printf("random reads, %5u B chunks, %d in flight per wave, %u waves per CU: %6.0f GB/s  (%5.2f G chunks/s)\n", chunk, DEPTH, grid / 64,
               chunks * chunk / ms / 1e6, chunks / ms / 1e6);
    else
        printf("random reads, %5u B chunks + %.2f returning atomics per chunk:        %6.0f GB/s  (%5.2f G chunks/s, %5.2f G atomics/s)\n", chunk,
               atomic_lanes / (double)DEPTH, chunks * chunk / ms / 1e6, chunks / ms / 1e6, (double)grid * 4 * iters * atomic_lanes / ms / 1e6);
    fflush(stdout);
}

int main() {
    int dev = 0;
    hipDeviceProp_t prop;
    CK(hipGetDevice(&dev));
    CK(hipGetDeviceProperties(&prop, dev));
    const uint32_t cus = prop.multiProcessorCount, grid = cus * 5; // 5 workgroups of 4 waves per CU: the occupancy of the search kernel
    const uint64_t bytes = 5ull << 30;                            // the size of the 1 M-doc corpus
    const uint32_t words_per_block = 32768;                       // 128 KiB of visited bitmap per workgroup
    char* buf = nullptr;
    uint32_t *bitmap = nullptr, *sink = nullptr;
    CK(hipMalloc(&buf, bytes));
    CK(hipMalloc(&bitmap, (size_t)grid * words_per_block * 4));
    CK(hipMalloc(&sink, 4));
    CK(hipMemset(buf, 1, bytes));
    CK(hipMemset(bitmap, 0, (size_t)grid * words_per_block * 4));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    printf("membench on %s (%s), %u CUs\n", prop.name, prop.gcnArchName, cus);
    run<1, true>(buf, bytes, bitmap, words_per_block, 0, sink, grid, e0, e1);
    run<2, true>(buf, bytes, bitmap, words_per_block, 0, sink, grid, e0, e1);
    run<3, true>(buf, bytes, bitmap, words_per_block, 0, sink, grid, e0, e1);
    run<1, false>(buf, bytes, bitmap, words_per_block, 0, sink, grid, e0, e1);
    run<2, false>(buf, bytes, bitmap, words_per_block, 0, sink, grid, e0, e1);
    run<5, false>(buf, bytes, bitmap, words_per_block, 0, sink, grid, e0, e1);
    run<1, false>(buf, bytes, bitmap, words_per_block, 3, sink, grid, e0, e1);
    run<1, false>(buf, bytes, bitmap, words_per_block, 5, sink, grid, e0, e1);
    run<1, false>(buf, bytes, bitmap, words_per_block, 9, sink, grid, e0, e1);
    CK(hipFree(buf));
    CK(hipFree(bitmap));
    CK(hipFree(sink));
    return 0;
}
