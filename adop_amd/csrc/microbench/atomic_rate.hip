// atomic_rate.hip - stand-alone microbenchmark (not linked into the library): throughput of device-scope fp32 atomic add,
// plain stores and loads on one GPU for different lane -> address patterns.  Its result decided the data layout of the
// blend accumulators (one 64-byte line per pixel) and the per-wavefront merging of point-levels.
//   hipcc --offload-arch=gfx950 -O3 -munsafe-fp-atomics adop_amd/csrc/microbench/atomic_rate.hip -o atomic_rate && ./atomic_rate
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#include <vector>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("err %s line %d\n", hipGetErrorString(e), __LINE__); return 1;}}while(0)

__device__ __forceinline__ uint32_t hash32(uint32_t x){ x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16; return x; }

// mode 0: every lane a random line (lane-scattered)
// mode 1: groups of G consecutive lanes hit G consecutive floats of one random line-aligned chunk
// mode 2: plain stores to the same addresses as mode 1 (reference)
template<int G, int MODE>
__global__ void k(float* buf, uint32_t nchunks, int iters)
{
    uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t grp = tid / G, lane = tid % G;
    for (int it = 0; it < iters; ++it)
    {
        uint32_t c = hash32(grp * 9781u + it * 6271u) % nchunks;
        float* p = buf + (size_t)(c - c % (G > 16 ? G / 16 : 1)) * 16 + lane;
        if (MODE == 0) unsafeAtomicAdd(p, 1.0f);
        else if (MODE == 1) __builtin_nontemporal_store(1.0f, p);
        else { float v = __builtin_nontemporal_load(p); if (v == 123.f) buf[0] = v; }
    }
}

template<int G, int MODE>
float run(float* buf, uint32_t nchunks, int blocks, int iters)
{
    hipEvent_t a, b; hipEventCreate(&a); hipEventCreate(&b);
    hipLaunchKernelGGL((k<G,MODE>), dim3(blocks), dim3(256), 0, 0, buf, nchunks, iters);
    hipDeviceSynchronize();
    hipEventRecord(a);
    hipLaunchKernelGGL((k<G,MODE>), dim3(blocks), dim3(256), 0, 0, buf, nchunks, iters);
    hipEventRecord(b); hipEventSynchronize(b);
    float ms; hipEventElapsedTime(&ms, a, b); return ms;
}

int main()
{
    const uint32_t nchunks = 2750000;  // 64 B chunks = 176 MB (like the 1080p pyramid with 16 floats/pixel)
    float* buf; CK(hipMalloc(&buf, (size_t)nchunks * 64)); CK(hipMemset(buf, 0, (size_t)nchunks * 64));
    int blocks = 39063, iters = 8;     // 10M threads x 8 = 80M lane-ops
    double ops = (double)blocks * 256 * iters;
    #define R(G,MODE,name) { float ms = run<G,MODE>(buf, nchunks, blocks, iters); printf("%-42s G=%2d  %8.3f ms  %8.2f G lane-ops/s  %8.2f G groups/s\n", name, G, ms, ops/ms/1e6, ops/G/ms/1e6); }
    R(1,0,"atomic, 1 lane per random line");
    R(2,0,"atomic, 2 lanes per line");
    R(4,0,"atomic, 4 lanes per line");
    R(8,0,"atomic, 8 lanes per line");
    R(16,0,"atomic, 16 lanes per line");
    R(32,0,"atomic, 32 lanes per 128B");
    R(64,0,"atomic, 64 lanes per 256B");
    R(1,1,"store, 1 lane per random line");
    R(16,1,"store, 16 lanes per line");
    R(1,2,"load, 1 lane per random line");
    R(16,2,"load, 16 lanes per line");
    // small footprint: 4 MB (fits L2): contention / locality effect
    const uint32_t small = 65536;
    { float ms = run<1,0>(buf, small, blocks, iters); printf("atomic 1 lane, 4MB footprint               %8.3f ms %8.2f G/s\n", ms, ops/ms/1e6); }
    { float ms = run<16,0>(buf, small, blocks, iters); printf("atomic 16 lanes, 4MB footprint             %8.3f ms %8.2f G/s\n", ms, ops/ms/1e6); }
    { float ms = run<16,0>(buf, 256, blocks, iters); printf("atomic 16 lanes, 16KB footprint (contended) %8.3f ms %8.2f G/s\n", ms, ops/ms/1e6); }
    { float ms = run<1,0>(buf, 256, blocks, iters); printf("atomic 1 lane, 16KB footprint (contended)   %8.3f ms %8.2f G/s\n", ms, ops/ms/1e6); }
    return 0;
}
