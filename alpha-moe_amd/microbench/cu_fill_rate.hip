// Microbenchmark: how fast can ONE compute unit pull data that sits in L2 / Infinity Cache / HBM, and does it matter
// whether the loads go straight to LDS (global_load_lds_dwordx4, what the kernels use) or to registers?
// One workgroup of 8 wavefronts per compute unit streams its own region `passes` times.
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/cu_fill_rate alpha-moe_amd/microbench/cu_fill_rate.hip && /tmp/cu_fill_rate
// Modes:
//   lds  D : direct-to-LDS, every instruction covers 8 whole 128-byte lines, D instructions (KiB) in flight per wavefront
//   lds16 D: direct-to-LDS, every instruction covers 16 rows x 64 bytes (the matrix-operand register layout)
//   ldsnt D: as lds, with the non-temporal hint
//   reg  U : non-temporal loads to registers, bursts of U instructions of 1 KiB per wavefront (regpl: plain loads)
// Region per workgroup: 64 KiB (stays in L2), 1 MiB (L2 + Infinity Cache), 16 MiB (HBM; 4 GiB in total at 256 workgroups).
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

typedef int v4i __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

template <int N> __device__ inline void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

template <int D, bool ROWS16, int AUX = 0>
__global__ __launch_bounds__(512) void fill_lds(const uint8_t *src, size_t region, int passes, int *sink)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint8_t *base = src + (size_t)blockIdx.x * region;
    uint8_t *ring = lds + wave * (D * 1024);
    // a wavefront takes every 8th KiB of the region
    const size_t n_chunks = region / 1024 / 8;
    // ROWS16: the 1 KiB of an instruction is spread over 16 rows of 128 bytes, 64 bytes from each (two instructions
    // cover the 2 KiB block); otherwise it is 8 whole lines
    const size_t lane_off = ROWS16 ? (size_t)(lane & 15) * 128 + (lane >> 4) * 16 : (size_t)lane * 16;
    for (int p = 0; p < passes; p++) {
        for (size_t c = 0; c < n_chunks; c++) {
            size_t off = (c * 8 + wave) * 1024;
            if (ROWS16) off = (off & ~(size_t)2047) + ((off >> 10) & 1) * 64;
            __builtin_amdgcn_global_load_lds((gptr_t)(base + off + lane_off), (lptr_t)(ring + (c % D) * 1024), 16, 0, AUX);
            wait_vmcnt<D - 1>();
        }
    }
    wait_vmcnt<0>();
    __syncthreads();
    if (threadIdx.x == 0 && lds[0] == 0x5a && lds[1] == 0x11) sink[0] = 1;
}

template <int U, bool NT = true>
__global__ __launch_bounds__(512) void fill_reg(const uint8_t *src, size_t region, int passes, int *sink)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint8_t *base = src + (size_t)blockIdx.x * region + (size_t)lane * 16;
    const size_t n_chunks = region / 1024 / 8;
    v4i acc = {0, 0, 0, 0};
    for (int p = 0; p < passes; p++) {
        for (size_t c = 0; c + U <= n_chunks; c += U) {
            v4i r[U];
#pragma unroll
            for (int u = 0; u < U; u++)
                r[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<const v4i *>(base + ((c + u) * 8 + wave) * 1024))
                          : *reinterpret_cast<const v4i *>(base + ((c + u) * 8 + wave) * 1024);
#pragma unroll
            for (int u = 0; u < U; u++) acc ^= r[u];
        }
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678) sink[1] = 1;
}

int main()
{
    const size_t total = (size_t)4 << 30;
    uint8_t *buf; int *sink;
    CHECK(hipMalloc(&buf, total)); CHECK(hipMemset(buf, 1, total)); CHECK(hipMalloc(&sink, 64));
    hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&fill_lds<16, false>), hipFuncAttributeMaxDynamicSharedMemorySize, 8 * 16 * 1024));
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&fill_lds<16, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 8 * 16 * 1024));
    struct Case { const char *name; int kind, depth; };
    const Case cases[] = {{"lds   D=2", 0, 2}, {"lds   D=4", 0, 4}, {"lds   D=8", 0, 8}, {"lds   D=16", 0, 16},
                          {"lds16 D=4", 1, 4}, {"lds16 D=16", 1, 16}, {"ldsnt D=4", 3, 4}, {"ldsnt D=8", 3, 8},
                          {"regpl U=4", 4, 4}, {"regpl U=8", 4, 8},
                          {"reg   U=4", 2, 4}, {"reg   U=8", 2, 8}, {"reg   U=16", 2, 16}, {"reg   U=32", 2, 32}};
    printf("%-12s %-8s %-6s %10s %12s %14s\n", "mode", "region", "wgs", "us", "GB/s total", "GB/s per CU");
    for (size_t region : {(size_t)64 << 10, (size_t)1 << 20, (size_t)16 << 20})
        for (int nwg : {1, 256})
            for (const Case &c : cases) {
                // about 16 MiB per workgroup and measurement, at least one pass
                int passes = (int)(((size_t)16 << 20) / region);
                if (passes < 1) passes = 1;
                float best = 1e9f;
                for (int rep = 0; rep < 3; rep++) {
                    CHECK(hipEventRecord(e0, 0));
#define LDS(D, R) hipLaunchKernelGGL((fill_lds<D, R>), dim3(nwg), dim3(512), 8 * D * 1024, 0, buf, region, passes, sink)
#define REG(U) hipLaunchKernelGGL((fill_reg<U>), dim3(nwg), dim3(512), 0, 0, buf, region, passes, sink)
                    if (c.kind == 0) { if (c.depth == 2) LDS(2, false); else if (c.depth == 4) LDS(4, false); else if (c.depth == 8) LDS(8, false); else LDS(16, false); }
                    else if (c.kind == 1) { if (c.depth == 4) LDS(4, true); else LDS(16, true); }
                    else if (c.kind == 3) { if (c.depth == 4) hipLaunchKernelGGL((fill_lds<4, false, 2>), dim3(nwg), dim3(512), 8 * 4 * 1024, 0, buf, region, passes, sink); else hipLaunchKernelGGL((fill_lds<8, false, 2>), dim3(nwg), dim3(512), 8 * 8 * 1024, 0, buf, region, passes, sink); }
                    else if (c.kind == 4) { if (c.depth == 4) hipLaunchKernelGGL((fill_reg<4, false>), dim3(nwg), dim3(512), 0, 0, buf, region, passes, sink); else hipLaunchKernelGGL((fill_reg<8, false>), dim3(nwg), dim3(512), 0, 0, buf, region, passes, sink); }
                    else { if (c.depth == 4) REG(4); else if (c.depth == 8) REG(8); else if (c.depth == 16) REG(16); else REG(32); }
                    CHECK(hipEventRecord(e1, 0)); CHECK(hipEventSynchronize(e1));
                    float ms; CHECK(hipEventElapsedTime(&ms, e0, e1)); best = best < ms ? best : ms;
                }
                const double bytes = (double)region * passes * nwg;
                printf("%-12s %-8zu %-6d %10.1f %12.1f %14.1f\n", c.name, region >> 10, nwg, best * 1e3, bytes / best / 1e6, bytes / best / 1e6 / nwg);
                fflush(stdout);
            }
    return 0;
}
