// Issue-rate probe for two ways of applying a 6-bit sub-block scale to an int8 product on the matrix cores.
//  TWO : the scale is split in base 8 and folded into two int8 weight operands; two v_mfma_i32_32x32x32_i8 per
//        sub-block and token tile accumulate in place; FILL other vector instructions per iteration stand for
//        conversion, flush and bookkeeping.
//  ONE : raw nibbles as the operand, one matrix instruction per sub-block and token tile into a zero accumulator,
//        then 16 v_mad_i32_i24 (result x per-lane scale + running sum), plus FILL other vector instructions.
// One iteration = one sub-block (K = 32) x four token tiles of 32, for a wave's 32 weight rows.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %s:%d\n", hipGetErrorString(e), __FILE__, __LINE__); exit(1);} } while (0)
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

template <int FILL>
__device__ __forceinline__ void filler(uint32_t (&x)[4], uint32_t y) {
#pragma unroll
    for (int i = 0; i < FILL; ++i) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(x[i & 3]) : "v"(y));
}

template <int VAR, int FILL>
__global__ __launch_bounds__(512, 2) void probe(int iters, int sc, int *out) {
    const int lane = threadIdx.x & 63;
    __shared__ __align__(16) unsigned char lds[32 * 1024];   // one 128-token activation tile: 32 fragments of 1 KB
    const int lane_off = (lane & 31) * 256 / 8 + 16 * ((lane >> 5) ^ (lane & 1));   // any conflict-free 16-byte pattern
    if (VAR == 4) {
        for (int k = threadIdx.x; k < 32 * 1024 / 4; k += blockDim.x) reinterpret_cast<int *>(lds)[k] = k;
        __syncthreads();
    }
    v4i a[4], b = {lane * 3, 7, 9, 11}, b2 = {lane, 5, 3, 1};
    for (int t = 0; t < 4; ++t) a[t] = (v4i){lane + t, lane + 1, lane + 2, lane + 3};
    uint32_t x[4] = {1u, 2u, 3u, (uint32_t)lane};
    v16i acc[4], hi[4];
    const v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (int t = 0; t < 4; ++t) { acc[t] = z; hi[t] = z; }
    for (int i = 0; i < iters; ++i) {
        if (VAR == 0) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b, acc[t], 0, 0, 0);
                hi[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b2, hi[t], 0, 0, 0);
                filler<FILL / 4>(x, (uint32_t)sc);
            }
        } else if (VAR == 2) {   // the same eight matrix instructions on TWO accumulators: each depends on the one two back
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b, acc[0], 0, 0, 0);
                hi[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b2, hi[0], 0, 0, 0);
                filler<FILL / 4>(x, (uint32_t)sc);
            }
        } else if (VAR == 4) {   // as VAR 2, every pair fed by a fresh 16-byte operand read from LDS four pairs earlier
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b, acc[0], 0, 0, 0);
                hi[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b2, hi[0], 0, 0, 0);
                a[t] = *reinterpret_cast<const v4i *>(lds + ((i * 4 + t) & 31) * 1024 + lane_off);
                filler<FILL / 4>(x, (uint32_t)sc);
            }
        } else if (VAR == 3) {   // on FOUR accumulators (two token tiles interleaved)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                acc[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b, acc[t & 1], 0, 0, 0);
                hi[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b2, hi[t & 1], 0, 0, 0);
                filler<FILL / 4>(x, (uint32_t)sc);
            }
        } else {
            v16i I[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) I[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b, z, 0, 0, 0);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[t][v] = __mul24(I[t][v], sc) + acc[t][v];
                filler<FILL / 4>(x, (uint32_t)sc);
            }
        }
    }
    int s = (int)(x[0] + x[1] + x[2] + x[3]);
    for (int t = 0; t < 4; ++t)
        for (int v = 0; v < 16; ++v) s += acc[t][v] + hi[t][v];
    if (s == 0x12345678) out[0] = s;
}

template <int VAR, int FILL>
void run(const char *name, int cus, int *out) {
    const int iters = 20000;
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    hipLaunchKernelGGL((probe<VAR, FILL>), dim3(cus), dim3(512), 0, 0, iters, 5, out); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL((probe<VAR, FILL>), dim3(cus), dim3(512), 0, 0, iters, 5, out);
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    // per SIMD: two waves, each `iters` iterations of four sub-block x token-tile products
    const double ns_per_product = ms * 1e6 / (iters * 4.0 * 2.0);
    const double tops = (double)cus * 8 * iters * 4 * 65536.0 / (ms * 1e-3) / 1e12;
    printf("%-44s %8.3f ms  %6.1f ns per product and SIMD  %7.1f TOPS of useful int8 work\n", name, ms, ns_per_product, tops);
    fflush(stdout);
}

int main() {
    hipDeviceProp_t prop; CK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    int *out; CK(hipMalloc(&out, 4));
    printf("CUs %d, 8 waves a workgroup, one workgroup a CU (two waves a SIMD)\n", cus);
    run<0, 0>("two chains, no other vector work", cus, out);
    run<0, 40>("two chains + 5 vector instr / matrix instr", cus, out);
    run<0, 60>("two chains + 7.5 (the wide kernel's mix)", cus, out);
    run<0, 80>("two chains + 10", cus, out);
    run<2, 0>("two chains on TWO accumulators, no other work", cus, out);
    run<2, 60>("two chains on TWO accumulators + 7.5", cus, out);
    run<4, 0>("two chains, operands from LDS, no other work", cus, out);
    run<4, 40>("two chains, operands from LDS + 5", cus, out);
    run<4, 60>("two chains, operands from LDS + 7.5", cus, out);
    run<3, 0>("two chains on FOUR accumulators, no other work", cus, out);
    run<3, 60>("two chains on FOUR accumulators + 7.5", cus, out);
    run<1, 0>("one chain + 16 mad24, nothing else", cus, out);
    run<1, 8>("one chain + 16 mad24 + 2", cus, out);
    run<1, 16>("one chain + 16 mad24 + 4", cus, out);
    run<1, 24>("one chain + 16 mad24 + 6", cus, out);
    run<1, 32>("one chain + 16 mad24 + 8", cus, out);
    return 0;
}
