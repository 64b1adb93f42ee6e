// What a backward that accumulates dK and dV in LDS would pay for its additions: every head-query adds 36 taps x 32
// channels x 2 arrays into accumulators that cover the 21 x 13 pixels a 16 x 8 tile's windows reach (one head: 32
// channels), with window origins drawn at random inside the tile.  fp32 additions (ds_add_f32), 32-bit integer additions
// (what a fixed-point accumulator would use) and a read-add-write that is not atomic (timing only), at pixel strides of
// 32 and 33 dwords.  A measuring tool, not part of the library:  make microbench && microbench/lds_add
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
constexpr int BW = 21, BH = 13, NPX = BW * BH, WN = 6;
template <int STRIDE, int MAP, int KIND>
__global__ __launch_bounds__(256) void k_add(float *out, int passes, uint32_t seed) {
    __shared__ float acc[2][NPX * STRIDE];
    for (int i = threadIdx.x; i < 2 * NPX * STRIDE; i += 256) (&acc[0][0])[i] = 0.f;
    __syncthreads();
    const int hq = threadIdx.x >> 1, sub = threadIdx.x & 1;
    for (int p = 0; p < passes; ++p) {
        uint32_t hsh = (uint32_t)(hq * 2654435761u) ^ (uint32_t)(p * 40503u) ^ seed ^ (blockIdx.x * 97u);
        hsh ^= hsh >> 13; hsh *= 0x5bd1e995u; hsh ^= hsh >> 15;
        const int cx = (int)(hsh & 15u), cy = (int)((hsh >> 4) & 7u);        // window origin inside the box: 0..15, 0..7
        const float val = (float)(hsh & 255u) * 0.01f;
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i) {
                const int pix = (cy + j) * BW + cx + i;                     // <= 12 * 21 + 20 = 272
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int ch = MAP == 0 ? sub * 16 + e : e * 2 + sub;
                    if constexpr (KIND == 0) {
                        __hip_atomic_fetch_add(&acc[0][pix * STRIDE + ch], val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        __hip_atomic_fetch_add(&acc[1][pix * STRIDE + ch], val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    } else if constexpr (KIND == 1) {        // 32-bit integer additions (what a fixed-point accumulator would use)
                        __hip_atomic_fetch_add((unsigned *)&acc[0][pix * STRIDE + ch], (unsigned)hsh, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        __hip_atomic_fetch_add((unsigned *)&acc[1][pix * STRIDE + ch], (unsigned)hsh, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    } else {                                 // not atomic: read, add, write (wrong sums when lanes collide; timing only)
                        volatile float *a0 = &acc[0][pix * STRIDE + ch], *a1 = &acc[1][pix * STRIDE + ch];
                        *a0 = *a0 + val; *a1 = *a1 + val;
                    }
                }
            }
    }
    __syncthreads();
    float s = 0.f;
    for (int i = threadIdx.x; i < 2 * NPX * STRIDE; i += 256) s += (&acc[0][0])[i];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}
template <typename K> void run(const char *name, K k, float *d, int per_cu) {
    const int passes = 40, blocks = 256 * per_cu;
    hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    hipLaunchKernelGGL(k, dim3(blocks), dim3(256), 0, 0, d, passes, 1u);
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(e0);
    hipLaunchKernelGGL(k, dim3(blocks), dim3(256), 0, 0, d, passes, 2u);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    float ms; (void)hipEventElapsedTime(&ms, e0, e1);
    // wave-passes per SIMD = passes * per_cu (4 waves per block, one per SIMD)
    const double cyc = ms * 1e-3 * 2.27e9 / (passes * per_cu);
    printf("%-28s %d workgroups per CU: %8.3f ms, %8.0f cycles per wavefront-pass (32 head-queries, 2304 additions per lane pair)\n", name, per_cu, ms, cyc);
    fflush(stdout);
}
int main() {
    float *d; (void)hipMalloc(&d, 256 * 4 * 256 * sizeof(float));
    for (int w : {1, 2}) {
        run("f32 add, stride 32", k_add<32, 0, 0>, d, w);
        run("f32 add, stride 33", k_add<33, 0, 0>, d, w);
        run("u32 add, stride 32", k_add<32, 0, 1>, d, w);
        run("u32 add, stride 33", k_add<33, 0, 1>, d, w);
        run("u32 add, stride 33, dealt", k_add<33, 1, 1>, d, w);
        run("read-add-write, stride 33", k_add<33, 0, 2>, d, w);
    }
    return 0;
}
