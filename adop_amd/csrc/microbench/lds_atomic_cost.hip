// lds_atomic_cost.hip — stand-alone microbenchmark (not linked into the library): cost of LDS atomics on gfx950 for
// different conflict patterns (ds_add_f32, ds_min_u64, ds_add_u32, ds_wrxchg_rtn_b32, a compare-and-swap float add),
// global float atomics at agent / workgroup / wavefront scope, and scattered 16-byte stores in runs of 1 .. 64 records.
// The tile kernels' choice of integer LDS atomics + per-pixel lists over float accumulation in LDS rests on its table.
//   make -C adop_amd/csrc microbench && adop_amd/csrc/microbench/lds_atomic_cost
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("err %s line %d\n", hipGetErrorString(e), __LINE__); return 1;}}while(0)

__device__ __forceinline__ uint32_t hash32(uint32_t x){ x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16; return x; }

// MODE 0: ds_add_f32, lanes -> addresses with CONF lanes sharing one address (consecutive lanes)
// MODE 1: ds_min_u64 same pattern
// MODE 2: plain LDS read-modify-write (non atomic) same pattern (reference)
// MODE 3: ds_add_f32 random addresses in a 1280*9 float tile
template<int MODE, int CONF>
__global__ __launch_bounds__(256) void k(float* out, int iters)
{
    __shared__ float s[12288];
    __shared__ unsigned long long s64[2048];
    for (int i = threadIdx.x; i < 12288; i += 256) s[i] = 0;
    for (int i = threadIdx.x; i < 2048; i += 256) s64[i] = ~0ull;
    __syncthreads();
    uint32_t tid = threadIdx.x;
    for (int it = 0; it < iters; ++it)
    {
        uint32_t a = (tid / CONF) + it * 67u;
        if (MODE == 0) atomicAdd(&s[a % 12288], 1.0f);
        else if (MODE == 1) atomicMin(&s64[a % 2048], (unsigned long long)(tid * 7919u + it));
        else if (MODE == 2) { float v = s[a % 12288]; s[a % 12288] = v + 1.0f; }
        else if (MODE == 4) { // CAS float add
            uint32_t* p = (uint32_t*)&s[a % 12288];
            uint32_t old = *p, assumed;
            do { assumed = old; old = atomicCAS(p, assumed, __float_as_uint(__uint_as_float(assumed) + 1.0f)); } while (old != assumed);
        }
        else if (MODE == 5) atomicAdd((uint32_t*)&s[a % 12288], 1u);
        else if (MODE == 6) { uint32_t o = atomicExch((uint32_t*)&s[a % 12288], tid); if (o == 0xffffffffu) s[0] = 1; }
        else if (MODE == 3) { uint32_t r = hash32(tid * 9781u + it * 6271u + blockIdx.x) % (1280u); atomicAdd(&s[r * 9 + (tid & 7)], 1.0f); }
    }
    __syncthreads();
    float acc = 0;
    for (int i = threadIdx.x; i < 12288; i += 256) acc += s[i];
    for (int i = threadIdx.x; i < 2048; i += 256) acc += (float)(s64[i] & 0xff);
    if (acc == -1.f) out[0] = acc;
}

template<int MODE, int CONF>
float run(float* buf, int blocks, int iters)
{
    hipEvent_t a, b; hipEventCreate(&a); hipEventCreate(&b);
    hipLaunchKernelGGL((k<MODE,CONF>), dim3(blocks), dim3(256), 0, 0, buf, iters);
    hipDeviceSynchronize();
    hipEventRecord(a);
    hipLaunchKernelGGL((k<MODE,CONF>), dim3(blocks), dim3(256), 0, 0, buf, iters);
    hipEventRecord(b); hipEventSynchronize(b);
    float ms; hipEventElapsedTime(&ms, a, b); return ms;
}

// global atomics at different scopes: every lane a random line of a 176 MB buffer
template<int SCOPE>
__global__ void g(float* buf, uint32_t nchunks, int iters)
{
    uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    for (int it = 0; it < iters; ++it)
    {
        uint32_t c = hash32(tid * 9781u + it * 6271u) % nchunks;
        float* p = buf + (size_t)c * 16;
        if (SCOPE == 0) __hip_atomic_fetch_add(p, 1.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else if (SCOPE == 1) __hip_atomic_fetch_add(p, 1.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else __hip_atomic_fetch_add(p, 1.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
    }
}
template<int SCOPE>
float rung(float* buf, uint32_t nchunks, int blocks, int iters)
{
    hipEvent_t a, b; hipEventCreate(&a); hipEventCreate(&b);
    hipLaunchKernelGGL((g<SCOPE>), dim3(blocks), dim3(256), 0, 0, buf, nchunks, iters);
    hipDeviceSynchronize();
    hipEventRecord(a);
    hipLaunchKernelGGL((g<SCOPE>), dim3(blocks), dim3(256), 0, 0, buf, nchunks, iters);
    hipEventRecord(b); hipEventSynchronize(b);
    float ms; hipEventElapsedTime(&ms, a, b); return ms;
}

// 16-byte stores: runs of RUN consecutive lanes write RUN consecutive 16 B records at a random place
template<int RUN>
__global__ void st16(float4* buf, uint32_t nrec, int iters)
{
    uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t grp = tid / RUN, lane = tid % RUN;
    for (int it = 0; it < iters; ++it)
    {
        uint32_t c = hash32(grp * 9781u + it * 6271u) % (nrec / RUN);
        buf[(size_t)c * RUN + lane] = make_float4(1, 2, 3, 4);
    }
}
template<int RUN>
float runst(float4* buf, uint32_t nrec, int blocks, int iters)
{
    hipEvent_t a, b; hipEventCreate(&a); hipEventCreate(&b);
    hipLaunchKernelGGL((st16<RUN>), dim3(blocks), dim3(256), 0, 0, buf, nrec, iters);
    hipDeviceSynchronize();
    hipEventRecord(a);
    hipLaunchKernelGGL((st16<RUN>), dim3(blocks), dim3(256), 0, 0, buf, nrec, iters);
    hipEventRecord(b); hipEventSynchronize(b);
    float ms; hipEventElapsedTime(&ms, a, b); return ms;
}

int main()
{
    float* buf; CK(hipMalloc(&buf, (size_t)2750000 * 64)); CK(hipMemset(buf, 0, (size_t)2750000 * 64));
    int blocks = 4096, iters = 256;
    double ops = (double)blocks * 256 * iters;  // lane-ops
    // 256 CUs; clock ~2.4 GHz: cycles per wave-instruction per CU = (ms*1e-3*2.4e9) / (ops/64/256)
    #define R(MODE,CONF,name) { float ms = run<MODE,CONF>(buf, blocks, iters); printf("%-36s conf=%2d %8.3f ms %8.2f G lane-ops/s  %6.1f clk/wave-instr/CU\n", name, CONF, ms, ops/ms/1e6, ms*1e-3*2.4e9/(ops/64/256)); }
    R(0,1,"ds_add_f32"); R(0,2,"ds_add_f32"); R(0,4,"ds_add_f32"); R(0,16,"ds_add_f32"); R(0,64,"ds_add_f32");
    R(1,1,"ds_min_u64"); R(1,2,"ds_min_u64"); R(1,4,"ds_min_u64"); R(1,16,"ds_min_u64"); R(1,64,"ds_min_u64");
    R(2,1,"plain rmw");
    R(4,1,"cas float add"); R(4,2,"cas float add"); R(4,4,"cas float add"); R(4,16,"cas float add");
    R(5,1,"ds_add_u32"); R(5,4,"ds_add_u32"); R(5,64,"ds_add_u32");
    R(6,1,"ds_wrxchg_rtn"); R(6,4,"ds_wrxchg_rtn");
    R(3,1,"ds_add_f32 random tile");
    int gb = 39063, gi = 8; double gops = (double)gb * 256 * gi;
    { float ms = rung<0>(buf, 2750000, gb, gi); printf("global atomic agent scope      %8.3f ms %8.2f G/s\n", ms, gops/ms/1e6); }
    { float ms = rung<1>(buf, 2750000, gb, gi); printf("global atomic workgroup scope  %8.3f ms %8.2f G/s\n", ms, gops/ms/1e6); }
    { float ms = rung<2>(buf, 2750000, gb, gi); printf("global atomic wavefront scope  %8.3f ms %8.2f G/s\n", ms, gops/ms/1e6); }
    { float ms = runst<1>((float4*)buf, 11000000, gb, gi); printf("16B stores run=1   %8.3f ms %8.2f G rec/s %8.1f GB/s\n", ms, gops/ms/1e6, gops*16/ms/1e6); }
    { float ms = runst<4>((float4*)buf, 11000000, gb, gi); printf("16B stores run=4   %8.3f ms %8.2f G rec/s %8.1f GB/s\n", ms, gops/ms/1e6, gops*16/ms/1e6); }
    { float ms = runst<16>((float4*)buf, 11000000, gb, gi); printf("16B stores run=16  %8.3f ms %8.2f G rec/s %8.1f GB/s\n", ms, gops/ms/1e6, gops*16/ms/1e6); }
    { float ms = runst<64>((float4*)buf, 11000000, gb, gi); printf("16B stores run=64  %8.3f ms %8.2f G rec/s %8.1f GB/s\n", ms, gops/ms/1e6, gops*16/ms/1e6); }
    return 0;
}
