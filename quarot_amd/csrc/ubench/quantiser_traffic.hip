// Quantiser-traffic microbenchmark (stand-alone; not part of the library): the memory traffic of an fp16 -> int4
// quantiser and of its inverse with NOTHING else -- 16-byte loads of RD bytes in all, 16-byte stores of RD / 4 bytes
// (or the other way round), eight buffers in turn so that no launch re-reads what the last-level cache holds.
// The times are the floor for quant_rows_kernel / kv_quant_kernel (4 : 1) and kv_dequant_kernel (1 : 4).
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops -o quantiser_traffic quantiser_traffic.hip && ./quantiser_traffic
#include <hip/hip_runtime.h>
#include <cstdio>
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// each thread: 4 loads -> 1 store (QUANT) or 1 load -> 4 stores
template <bool QUANT>
__global__ __launch_bounds__(256) void traffic(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t small_units) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < small_units; i += stride) {
        if (QUANT) {
            u32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(src + (size_t)u * small_units + i);
            __builtin_nontemporal_store(v[0] ^ v[1] ^ v[2] ^ v[3], dst + i);
        } else {
            const u32x4 v = __builtin_nontemporal_load(src + i);
#pragma unroll
            for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(v + (unsigned)u, dst + (size_t)u * small_units + i);
        }
    }
}
int main() {
    const size_t big = (size_t)256 << 20, small = big / 4;               // 268 MB of fp16, 67 MB of codes: the K or V cache of [32, 4096, 8, 128]
    char *a, *b;
    hipMalloc(&a, 8 * big); hipMalloc(&b, 8 * big);
    hipMemset(a, 1, 8 * big); hipMemset(b, 2, 8 * big);
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    for (int wgs_per_cu : {4, 8, 16}) {
        for (int quant = 1; quant >= 0; --quant) {
            int turn = 0;
            auto launch = [&]() {
                const size_t w = (size_t)(turn++ % 8) * big;
                if (quant) traffic<true><<<256 * wgs_per_cu, 256>>>((const u32x4*)(a + w), (u32x4*)(b + w), small / 16);
                else traffic<false><<<256 * wgs_per_cu, 256>>>((const u32x4*)(a + w), (u32x4*)(b + w), small / 16);
            };
            launch(); hipDeviceSynchronize();
            hipEventRecord(e0);
            for (int r = 0; r < 6; ++r) launch();
            hipEventRecord(e1); hipEventSynchronize(e1);
            float ms; hipEventElapsedTime(&ms, e0, e1); ms /= 6;
            printf("%s  workgroups/CU %2d: %6.1f us  %5.2f TB/s (read + written)\n", quant ? "268 MB read, 67 MB written" : "67 MB read, 268 MB written", wgs_per_cu,
                   ms * 1e3, (double)(big + small) / (ms * 1e-3) / 1e12);
            fflush(stdout);
        }
    }
    return 0;
}
