// Microbenchmark behind two design decisions of the fused MoE kernels (MI355X):
//   * weight streams use non-temporal loads: a cold read of a large buffer with plain loads runs well below what the
//     same read reaches with the non-temporal hint (modes 3 and 2 below);
//   * per-slot result rows that are written by one kernel and read back by the next gain little from the 256 MiB
//     Infinity Cache even when they fit (mode 0 against mode 2), and nothing when written non-temporally (mode 1).
// Build and run (one MI355X):
//     hipcc --offload-arch=gfx950 -O3 -o /tmp/mall_readback alpha-moe_amd/microbench/mall_readback.hip && /tmp/mall_readback
// Every line: a kernel writes `size` bytes, another reads them back; 2 GiB of other data is written before each pair so
// that nothing older survives in L2 or the Infinity Cache.
//   mode 0: plain stores, plain loads        mode 1: non-temporal stores, plain loads
//   mode 2: plain stores, non-temporal loads mode 3: plain stores, 2 GiB of other writes, then plain loads (cold)
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <vector>
typedef int v4i __attribute__((ext_vector_type(4)));
__global__ void wr(v4i *p, size_t n, int v) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = (v4i){v, v, v, v};
}
__global__ void wr_nt(v4i *p, size_t n, int v) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) __builtin_nontemporal_store((v4i){v, v, v, v}, p + i);
}
__global__ void rd(const v4i *p, size_t n, int *out) {
    v4i a = {0, 0, 0, 0};
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) { v4i v = p[i]; a += v; }
    if (a.x + a.y + a.z + a.w == 12345) *out = 1;
}
__global__ void rd_nt(const v4i *p, size_t n, int *out) {
    v4i a = {0, 0, 0, 0};
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) { v4i v = __builtin_nontemporal_load(p + i); a += v; }
    if (a.x + a.y + a.z + a.w == 12345) *out = 1;
}
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
int main() {
    size_t maxb = (size_t)2 << 30;
    v4i *buf, *other; int *flag;
    CK(hipMalloc(&buf, maxb)); CK(hipMalloc(&other, maxb)); CK(hipMalloc(&flag, 4));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const int grid = 256 * 8, th = 256;
    size_t sizes[] = {16u << 20, 32u << 20, 64u << 20, 96u << 20, 128u << 20, 192u << 20, 256u << 20, 384u << 20, 512u << 20, (size_t)1 << 30};
    for (int mode = 0; mode < 4; mode++) {   // 0: wr + rd, 1: wr_nt + rd, 2: wr + rd_nt, 3: cold read (after flushing with `other`)
        for (size_t b : sizes) {
            size_t n = b / 16;
            float tw = 0, tr = 0; int reps = 5;
            for (int r = 0; r < reps + 1; r++) {
                hipLaunchKernelGGL(wr, dim3(grid), dim3(th), 0, 0, other, maxb / 16, r);   // evict everything
                CK(hipEventRecord(e0));
                if (mode == 1) hipLaunchKernelGGL(wr_nt, dim3(grid), dim3(th), 0, 0, buf, n, r); else hipLaunchKernelGGL(wr, dim3(grid), dim3(th), 0, 0, buf, n, r);
                CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
                float ms; CK(hipEventElapsedTime(&ms, e0, e1)); if (r) tw += ms;
                if (mode == 3) hipLaunchKernelGGL(wr, dim3(grid), dim3(th), 0, 0, other, maxb / 16, r);
                CK(hipEventRecord(e0));
                if (mode == 2) hipLaunchKernelGGL(rd_nt, dim3(grid), dim3(th), 0, 0, buf, n, flag); else hipLaunchKernelGGL(rd, dim3(grid), dim3(th), 0, 0, buf, n, flag);
                CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
                CK(hipEventElapsedTime(&ms, e0, e1)); if (r) tr += ms;
            }
            printf("mode %d size %4zu MiB: write %.2f TB/s  read-back %.2f TB/s\n", mode, b >> 20, b / (tw / reps * 1e-3) / 1e12, b / (tr / reps * 1e-3) / 1e12);
            fflush(stdout);
        }
    }
    return 0;
}
