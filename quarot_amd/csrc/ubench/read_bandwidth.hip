// Read-bandwidth microbenchmark (stand-alone; not part of the library): what one workgroup per CU can pull
// from HBM (a 2 GiB buffer, every launch reads all of it) and from L2 (a 2 MB window read over and over), as a
// function of waves per CU and 16-byte loads in flight per lane.  The ceilings that the memory-bound kernels
// are measured against come from here.
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops -o read_bandwidth read_bandwidth.hip && ./read_bandwidth
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <int U>
__global__ __launch_bounds__(1024) void readk(const u32x4* __restrict__ src, size_t units_per_wg, size_t wrap_units, unsigned* out) {
    const int nthr = blockDim.x;
    size_t base = (size_t)blockIdx.x * units_per_wg;
    u32x4 acc = {0, 0, 0, 0};
    for (size_t i = threadIdx.x; i + (size_t)(U - 1) * nthr < units_per_wg; i += (size_t)U * nthr) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(src + (base + i + (size_t)u * nthr) % wrap_units);
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[0] = 1;
}
int main() {
    const size_t bytes = (size_t)2 << 30;
    u32x4* src; unsigned* out;
    hipMalloc(&src, bytes); hipMalloc(&out, 4);
    hipMemset(src, 1, bytes);
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    const int cus = 256;
    for (int hbm = 1; hbm >= 0; --hbm)
        for (int waves : {4, 8, 16}) {
            for (int U : {1, 2, 4, 8}) {
                const size_t total_units = bytes / 16;
                const size_t per_wg = total_units / cus / (hbm ? 1 : 1);
                const size_t wrap = hbm ? total_units : (size_t)(1 << 20) / 16 * 2;      // 2 MB window: L2 hits
                auto launch = [&]() {
                    switch (U) {
                        case 1: readk<1><<<cus, waves * 64>>>(src, per_wg, wrap, out); break;
                        case 2: readk<2><<<cus, waves * 64>>>(src, per_wg, wrap, out); break;
                        case 4: readk<4><<<cus, waves * 64>>>(src, per_wg, wrap, out); break;
                        default: readk<8><<<cus, waves * 64>>>(src, per_wg, wrap, out); break;
                    }
                };
                launch(); hipDeviceSynchronize();
                hipEventRecord(e0);
                for (int r = 0; r < 3; ++r) launch();
                hipEventRecord(e1); hipEventSynchronize(e1);
                float ms; hipEventElapsedTime(&ms, e0, e1); ms /= 3;
                const double gbs = (double)per_wg * cus * 16 / (ms * 1e-3) / 1e9;
                printf("%s waves/CU %2d loads in flight/wave %d (%5.1f KB per CU): %7.1f GB/s total, %5.1f GB/s per CU\n", hbm ? "HBM" : "L2 ", waves, U,
                       waves * 64 * U * 16 / 1024.0, gbs, gbs / cus);
                fflush(stdout);
            }
        }
    return 0;
}
