// Microbenchmark: what does it cost to add top_k partial rows per token into one [M, C] accumulator in memory, compared
// with writing the rows once (and summing them in a second pass)?  M * top_k rows of C values in a shuffled order, dealt to
// persistent workgroups as blocks of 128 rows x one eighth of the columns.  "xcd-owned": the workgroups of XCD x only
// ever touch column slab x, so that one L2 could own those lines; "mixed": every XCD touches every slab.
//   hipcc --offload-arch=gfx950 -O3 -munsafe-fp-atomics -o /tmp/accumulate_rows alpha-moe_amd/microbench/accumulate_rows.hip
//   /tmp/accumulate_rows 8192
// Prints microseconds per mode and, at the end, how workgroup index % 8 maps to the hardware XCC_ID.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
#include <algorithm>
#include <random>
#include <cstring>

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

typedef short v2s __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

__device__ inline int xcc_id() { return __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15; }

enum { kAtomF32 = 0, kAtomPkBf16 = 1, kRmwF32 = 2, kStoreY = 3, kAtomF32Tile = 4 };

// rows: [nblk][128] token ids.  An item is (block b, slab s): 128 rows x slab_cols columns.
// owner != 0: the workgroups of XCD x take exactly the items of slab x.  owner == 0: slab = (x + b) % 8 (every XCD
// touches every slab over the run).
template <int MODE>
__global__ __launch_bounds__(256) void add_rows(float *acc, unsigned short *y, const int *rows, int nblk, int C,
                                                int owner, int *xcd_seen)
{
    const int x = xcc_id();
    const int nslab = 8, slab_cols = C / nslab;
    const int wg_in_x = blockIdx.x >> 3, nwg_x = gridDim.x >> 3;
    if (threadIdx.x == 0) atomicAdd(&xcd_seen[(blockIdx.x & 7) * 8 + (x & 7)], 1);
    const int tid = threadIdx.x;
    for (int b = wg_in_x; b < nblk; b += nwg_x) {
        const int s = owner ? x : (x + b) & 7;
        for (int r = 0; r < 128; r++) {
            const int tok = rows[b * 128 + r];
            if (MODE == kAtomF32) {
                float *base = acc + (size_t)tok * C + s * slab_cols;
                for (int c = tid; c < slab_cols; c += 256) unsafeAtomicAdd(base + c, 1.0f);
            } else if (MODE == kAtomF32Tile) {
                // lane owns 16 consecutive floats; instruction i touches float i of every lane's chunk
                float *base = acc + (size_t)tok * C + s * slab_cols;
                for (int c0 = tid * 16; c0 < slab_cols; c0 += 256 * 16)
#pragma unroll
                    for (int i = 0; i < 16; i++) unsafeAtomicAdd(base + c0 + i, 1.0f);
            } else if (MODE == kAtomPkBf16) {
                unsigned short *base = (unsigned short *)acc + (size_t)tok * C + s * slab_cols;
                v2bf one = {(__bf16)1.0f, (__bf16)1.0f};
                for (int c = tid * 2; c < slab_cols; c += 512)
                    __builtin_amdgcn_global_atomic_fadd_v2bf16((v2s __attribute__((address_space(1))) *)(base + c), __builtin_bit_cast(v2s, one));
            } else if (MODE == kRmwF32) {
                float4 *base = (float4 *)(acc + (size_t)tok * C + s * slab_cols);
                for (int c = tid; c < slab_cols / 4; c += 256) {
                    float4 v = base[c];
                    v.x += 1.f; v.y += 1.f; v.z += 1.f; v.w += 1.f;
                    base[c] = v;
                }
            } else if (MODE == kStoreY) {
                uint4 *base = (uint4 *)(y + ((size_t)b * 128 + r) * C + s * slab_cols);
                for (int c = tid; c < slab_cols / 8; c += 256) base[c] = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);
            }
        }
    }
}

int main(int argc, char **argv)
{
    const int M = argc > 1 ? atoi(argv[1]) : 8192, C = 7168, topk = 9;
    const int nrows = M * topk, nblk = nrows / 128;
    std::vector<int> rows(nrows);
    for (int i = 0; i < nrows; i++) rows[i] = i % M;
    std::mt19937 rng(1);
    std::shuffle(rows.begin(), rows.end(), rng);
    int *d_rows, *d_seen; float *acc; unsigned short *y;
    CHECK(hipMalloc(&d_rows, nrows * 4)); CHECK(hipMemcpy(d_rows, rows.data(), nrows * 4, hipMemcpyHostToDevice));
    CHECK(hipMalloc(&d_seen, 64 * 4)); CHECK(hipMemset(d_seen, 0, 64 * 4));
    CHECK(hipMalloc(&acc, (size_t)M * C * 4)); CHECK(hipMalloc(&y, (size_t)nrows * C * 2));
    hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    const char *names[] = {"atomic f32 coalesced", "atomic pk_bf16 coalesced", "plain rmw f32x4", "plain store y bf16", "atomic f32 16-per-lane"};
    printf("M=%d C=%d rows=%d blocks=%d; acc f32 %.0f MB, y %.0f MB\n", M, C, nrows, nblk, M * (double)C * 4 / 1e6, nrows * (double)C * 2 / 1e6);
    for (int grid : {256, 512, 1024}) for (int owner = 1; owner >= 0; owner--) for (int mode = 0; mode < 5; mode++) {
        float best = 1e9f;
        for (int rep = 0; rep < 3; rep++) {
            CHECK(hipMemsetAsync(acc, 0, (size_t)M * C * 4, 0));
            CHECK(hipEventRecord(e0, 0));
            switch (mode) {
            case 0: add_rows<0><<<grid, 256>>>(acc, y, d_rows, nblk, C, owner, d_seen); break;
            case 1: add_rows<1><<<grid, 256>>>(acc, y, d_rows, nblk, C, owner, d_seen); break;
            case 2: add_rows<2><<<grid, 256>>>(acc, y, d_rows, nblk, C, owner, d_seen); break;
            case 3: add_rows<3><<<grid, 256>>>(acc, y, d_rows, nblk, C, owner, d_seen); break;
            case 4: add_rows<4><<<grid, 256>>>(acc, y, d_rows, nblk, C, owner, d_seen); break;
            }
            CHECK(hipEventRecord(e1, 0)); CHECK(hipEventSynchronize(e1));
            float ms; CHECK(hipEventElapsedTime(&ms, e0, e1)); best = std::min(best, ms);
        }
        // spot check
        std::vector<float> h(1024);
        CHECK(hipMemcpy(h.data(), acc + (size_t)(M / 2) * C + 3000, 1024 * 4, hipMemcpyDeviceToHost));
        float lo = 1e9f, hi = -1e9f;
        if (mode == 1) { unsigned short *p = (unsigned short *)acc; std::vector<unsigned short> hb(1024); CHECK(hipMemcpy(hb.data(), p + (size_t)(M / 2) * C + 3000, 2048, hipMemcpyDeviceToHost)); for (auto v : hb) { unsigned u = (unsigned)v << 16; float f; memcpy(&f, &u, 4); lo = std::min(lo, f); hi = std::max(hi, f); } }
        else for (float v : h) { lo = std::min(lo, v); hi = std::max(hi, v); }
        printf("grid %4d %-9s %-26s %8.1f us  (check min %.1f max %.1f)\n", grid, owner ? "xcd-owned" : "mixed", names[mode], best * 1e3f, lo, hi);
        fflush(stdout);
    }
    std::vector<int> seen(64); CHECK(hipMemcpy(seen.data(), d_seen, 256, hipMemcpyDeviceToHost));
    printf("blockIdx%%8 (row) vs XCC_ID (col) counts:\n");
    for (int i = 0; i < 8; i++) { for (int j = 0; j < 8; j++) printf("%8d", seen[i * 8 + j]); printf("\n"); }
    return 0;
}
