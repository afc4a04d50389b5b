// Decode-traffic microbenchmark (stand-alone; not part of the library): the memory traffic of decode against
// the narrow weight (8192 x 28672 int4 = 117 MB, 32 rows per CU) with NOTHING else -- every workgroup streams
// its private 1/256 of 117 MB from HBM (eight 128 MB windows in turn, so that no launch re-reads what the
// last-level cache holds) and reads a shared 1 MB region (the tokens' codes, L2 hits) XS 16-byte loads for
// every 4 private ones: 4:1, 4:4, 4:8 are the byte ratios of 8, 32 and 64 tokens.  The times are the floor
// for any kernel with that decomposition of the work.
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops -o decode_traffic decode_traffic.hip && ./decode_traffic
#include <hip/hip_runtime.h>
#include <cstdio>
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <int XP, int XS>
__global__ __launch_bounds__(1024) void mixk(const u32x4* __restrict__ priv, const u32x4* __restrict__ shared, size_t priv_units_per_wg,
                                             size_t shared_units, unsigned* out, size_t window) {
    priv += window;
    const int nthr = blockDim.x;
    const size_t base = (size_t)blockIdx.x * priv_units_per_wg;
    u32x4 acc = {0, 0, 0, 0};
    size_t j = threadIdx.x;
    for (size_t i = threadIdx.x; i + (size_t)(XP - 1) * nthr < priv_units_per_wg; i += (size_t)XP * nthr) {
        u32x4 v[XP + XS];
#pragma unroll
        for (int u = 0; u < XP; ++u) v[u] = __builtin_nontemporal_load(priv + base + i + (size_t)u * nthr);
#pragma unroll
        for (int u = 0; u < XS; ++u) {
            v[XP + u] = shared[j];
            j += nthr;
            if (j >= shared_units) j -= shared_units;
        }
#pragma unroll
        for (int u = 0; u < XP + XS; ++u) acc ^= v[u];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[0] = 1;
}
int main() {
    const size_t bytes = (size_t)1 << 30;
    u32x4 *priv, *shared; unsigned* out;
    hipMalloc(&priv, bytes); hipMalloc(&shared, 1 << 20); hipMalloc(&out, 4);
    hipMemset(priv, 1, bytes); hipMemset(shared, 2, 1 << 20);
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    const int cus = 256;
    const size_t per_wg = (size_t)(117 << 20) / 16 / cus;          // 117 MB of private data in all: the narrow weight
    for (int waves : {8, 16}) {
        for (int mode = 0; mode < 4; ++mode) {
            int turn = 0;
            auto launch = [&]() {
                const size_t win = (size_t)(turn++ % 8) * ((size_t)(128 << 20) / 16);     // eight windows of 128 MB: no launch re-reads what the last-level cache holds
                switch (mode) {
                    case 0: mixk<4, 0><<<cus, waves * 64>>>(priv, shared, per_wg, (1 << 20) / 16, out, win); break;
                    case 1: mixk<4, 1><<<cus, waves * 64>>>(priv, shared, per_wg, (1 << 20) / 16, out, win); break;
                    case 2: mixk<4, 4><<<cus, waves * 64>>>(priv, shared, per_wg, (1 << 20) / 16, out, win); break;
                    default: mixk<4, 8><<<cus, waves * 64>>>(priv, shared, per_wg, (1 << 20) / 16, out, win); break;
                }
            };
            const int xs = mode == 0 ? 0 : mode == 1 ? 1 : mode == 2 ? 4 : 8;
            launch(); hipDeviceSynchronize();
            hipEventRecord(e0);
            for (int r = 0; r < 5; ++r) launch();
            hipEventRecord(e1); hipEventSynchronize(e1);
            float ms; hipEventElapsedTime(&ms, e0, e1); ms /= 5;
            const double pb = (double)per_wg * cus * 16, sb = pb * xs / 4;
            printf("waves/CU %2d private:shared 4:%d  %6.1f us  private %5.2f TB/s  per CU total %5.1f GB/s (shared bytes per CU %.2f MB)\n", waves, xs, ms * 1e3,
                   pb / (ms * 1e-3) / 1e12, (pb + sb) / cus / (ms * 1e-3) / 1e9, sb / cus / 1e6);
            fflush(stdout);
        }
    }
    return 0;
}
