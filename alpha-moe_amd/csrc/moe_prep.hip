// Input preparation of the fused MoE operator on the GPU: the two steps every caller runs right before it.
//
//   * per-token-group FP8 quantisation of the activations (the reference calls SGLang's
//     sglang_per_token_group_quant_fp8(x, 128), jit_moe.py:142; the kernel consumes the result at
//     fused_moe_w8a8_up_down_acc.cu:793,800-807): scale = max(amax, 1e-10) / 448, q = fp8_rne(clamp(x / scale, +-448));
//   * grouping of the routing slots by expert, padded to the row-block size (SGLang's moe_align_block_size,
//     jit_moe.py:158; consumed at fused_moe_w8a8_up_down_acc.cu:676-679,756-758): flat slot ids in ascending expert
//     order, ascending id within an expert (stable: the result depends on nothing but the input), padding entries
//     equal to numel, one expert id per block (-1 past the padded total), and the padded total.
//
// Both are HBM-bound integer/byte passes: 16-byte loads, no matrix instructions.
#include "moe_common.hpp"

namespace alpha_moe {
namespace {

constexpr int kAlignSeg = 1024;        // routing slots per workgroup of the histogram and placement kernels
constexpr int kAlignMaxExperts = 4096;

// ---- quantisation ------------------------------------------------------------------------------------------
// A group of 128 values is held by 16 lanes x 8 values; a wavefront works on 4 groups at a time.
template <typename T>
__device__ __forceinline__ void load8(const T *p, float (&v)[8]);

template <>
__device__ __forceinline__ void load8<uint16_t>(const uint16_t *p, float (&v)[8])   // bf16
{
    const v4i raw = *reinterpret_cast<const v4i *>(p);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[2 * i] = __builtin_bit_cast(float, (uint32_t)raw[i] << 16);
        v[2 * i + 1] = __builtin_bit_cast(float, (uint32_t)raw[i] & 0xffff0000u);
    }
}

template <>
__device__ __forceinline__ void load8<float>(const float *p, float (&v)[8])
{
    const v4f a = *reinterpret_cast<const v4f *>(p), b = *reinterpret_cast<const v4f *>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[i] = a[i];
        v[4 + i] = b[i];
    }
}

template <typename T>
__global__ __launch_bounds__(256) void quant_group128_kernel(const T *__restrict__ x, uint8_t *__restrict__ q,
                                                             float *__restrict__ scale, long long n_groups)
{
    const int sub = threadIdx.x & 15;
    const long long stride = (long long)gridDim.x * 16;
    for (long long g = (long long)blockIdx.x * 16 + (threadIdx.x >> 4); g < n_groups; g += stride) {
        float v[8];
        load8<T>(x + g * 128 + sub * 8, v);
        float m = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) m = fmaxf(m, fabsf(v[i]));
#pragma unroll
        for (int d = 1; d < 16; d <<= 1) m = fmaxf(m, __shfl_xor(m, d));
        const float s = fmaxf(m, kAmaxFloor) / kFp8Max;
        uint2 o;
        o.x = pack_fp8x4(clamp_fp8(v[0] / s), clamp_fp8(v[1] / s), clamp_fp8(v[2] / s), clamp_fp8(v[3] / s));
        o.y = pack_fp8x4(clamp_fp8(v[4] / s), clamp_fp8(v[5] / s), clamp_fp8(v[6] / s), clamp_fp8(v[7] / s));
        *reinterpret_cast<uint2 *>(q + g * 128 + sub * 8) = o;
        if (sub == 0) scale[g] = s;
    }
}

// ---- alignment ---------------------------------------------------------------------------------------------
// Exclusive prefix sum over `n` values held in LDS (n <= kAlignMaxExperts), in place; returns the total.
// Every thread of the workgroup calls it.
__device__ int block_exclusive_scan(int *vals, int n, int *partial /* [blockDim.x + 1] */)
{
    const int per = (n + blockDim.x - 1) / blockDim.x;
    const int lo = threadIdx.x * per, hi = lo + per < n ? lo + per : n;
    int sum = 0;
    for (int i = lo; i < hi; i++) sum += vals[i];
    partial[threadIdx.x] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (unsigned i = 0; i < blockDim.x; i++) {
            const int t = partial[i];
            partial[i] = run;
            run += t;
        }
        partial[blockDim.x] = run;
    }
    __syncthreads();
    int run = partial[threadIdx.x];
    for (int i = lo; i < hi; i++) {
        const int t = vals[i];
        vals[i] = run;
        run += t;
    }
    __syncthreads();
    return partial[blockDim.x];
}

// Stable placement of one wavefront's 64 consecutive slots: lanes with the same expert take consecutive positions
// in lane order behind cursor[expert]; the cursor advances by their number.  All 64 lanes call it (e < 0: no slot).
__device__ __forceinline__ void place_chunk(int e, int flat_id, int *cursor, int32_t *sorted_ids)
{
    const int lane = threadIdx.x & 63;
    unsigned long long todo = __ballot(e >= 0);
    while (todo) {
        const int leader_lane = __builtin_ctzll(todo);
        const int leader = __shfl(e, leader_lane);
        const unsigned long long same = __ballot(e == leader) & todo;
        if (e == leader) {
            const int rank = __builtin_popcountll(same & ((1ull << lane) - 1));
            sorted_ids[cursor[leader] + rank] = flat_id;
        }
        __builtin_amdgcn_wave_barrier();
        if (lane == leader_lane) cursor[leader] += __builtin_popcountll(same);
        __builtin_amdgcn_wave_barrier();
        todo &= ~same;
    }
}

// Fills expert_ids and the padded total from the experts' padded segment starts (`start`, exclusive scan of `padded`).
__device__ void write_blocks(const int *start, const int *padded, int E, int block_size, int total, int32_t *expert_ids,
                             int n_blocks, int32_t *ntpp)
{
    for (int e = threadIdx.x; e < E; e += blockDim.x)
        for (int b = start[e] / block_size, end = (start[e] + padded[e]) / block_size; b < end && b < n_blocks; b++)
            expert_ids[b] = e;
    for (int b = total / block_size + threadIdx.x; b < n_blocks; b += blockDim.x) expert_ids[b] = -1;
    if (threadIdx.x == 0) ntpp[0] = total;
}

// One workgroup does everything: up to a few thousand slots (decode).
__global__ __launch_bounds__(256) void align_small_kernel(const int32_t *__restrict__ ids, int numel, int E, int block_size,
                                                          int32_t *sorted_ids, int sorted_num, int32_t *expert_ids,
                                                          int n_blocks, int32_t *ntpp)
{
    extern __shared__ int lds[];   // [E] counts -> cursors | [E] padded | [257] scan partials
    int *cnt = lds, *padded = lds + E, *partial = lds + 2 * E;
    for (int i = threadIdx.x; i < E; i += blockDim.x) cnt[i] = 0;
    for (int i = threadIdx.x; i < sorted_num; i += blockDim.x) sorted_ids[i] = numel;
    __syncthreads();
    for (int i = threadIdx.x; i < numel; i += blockDim.x) {
        const int e = ids[i];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < E; i += blockDim.x) {
        padded[i] = (cnt[i] + block_size - 1) / block_size * block_size;
        cnt[i] = padded[i];
    }
    __syncthreads();
    const int total = block_exclusive_scan(cnt, E, partial);   // cnt: start of each expert's padded segment
    write_blocks(cnt, padded, E, block_size, total, expert_ids, n_blocks, ntpp);
    __syncthreads();   // the sentinel fill is done and write_blocks has read the starts before the cursors move
    if (threadIdx.x < 64) {
        for (int base = 0; base < numel; base += 64) {
            const int i = base + threadIdx.x;
            int e = i < numel ? ids[i] : -1;
            if (e >= E) e = -1;
            place_chunk(e, i, cnt, sorted_ids);
        }
    }
}

// Large inputs, pass 1: per-segment expert histograms; also the sentinel fill.
__global__ __launch_bounds__(256) void align_hist_kernel(const int32_t *__restrict__ ids, int numel, int E, int *hist,
                                                         int32_t *sorted_ids, int sorted_num)
{
    extern __shared__ int lds[];
    for (int i = threadIdx.x; i < E; i += blockDim.x) lds[i] = 0;
    __syncthreads();
    const int lo = blockIdx.x * kAlignSeg, hi = lo + kAlignSeg < numel ? lo + kAlignSeg : numel;
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const int e = ids[i];
        if (e >= 0 && e < E) atomicAdd(&lds[e], 1);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < E; i += blockDim.x) hist[(size_t)blockIdx.x * E + i] = lds[i];
    const int per = (sorted_num + gridDim.x - 1) / gridDim.x;
    const int flo = blockIdx.x * per, fhi = flo + per < sorted_num ? flo + per : sorted_num;
    for (int i = flo + threadIdx.x; i < fhi; i += blockDim.x) sorted_ids[i] = numel;
}

// Pass 2 (one workgroup): hist[s][e] becomes the position where segment s starts writing expert e.
__global__ __launch_bounds__(1024) void align_scan_kernel(int *hist, int n_seg, int E, int block_size, int32_t *expert_ids,
                                                          int n_blocks, int32_t *ntpp)
{
    extern __shared__ int lds[];   // [E] starts | [E] padded | [1025] scan partials
    int *start = lds, *padded = lds + E, *partial = lds + 2 * E;
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
        for (int s = 0; s < n_seg; s++) {
            const int t = hist[(size_t)s * E + e];
            hist[(size_t)s * E + e] = run;
            run += t;
        }
        padded[e] = (run + block_size - 1) / block_size * block_size;
        start[e] = padded[e];
    }
    __syncthreads();
    const int total = block_exclusive_scan(start, E, partial);
    write_blocks(start, padded, E, block_size, total, expert_ids, n_blocks, ntpp);
    for (int e = threadIdx.x; e < E; e += blockDim.x)
        for (int s = 0; s < n_seg; s++) hist[(size_t)s * E + e] += start[e];
}

// Pass 3: one wavefront per segment places its slots in order.
__global__ __launch_bounds__(64) void align_place_kernel(const int32_t *__restrict__ ids, int numel, int E, const int *hist,
                                                         int32_t *sorted_ids)
{
    extern __shared__ int lds[];   // [E] cursors
    for (int i = threadIdx.x; i < E; i += 64) lds[i] = hist[(size_t)blockIdx.x * E + i];
    __builtin_amdgcn_wave_barrier();
    __syncthreads();
    const int lo = blockIdx.x * kAlignSeg, hi = lo + kAlignSeg < numel ? lo + kAlignSeg : numel;
    for (int base = lo; base < hi; base += 64) {
        const int i = base + threadIdx.x;
        int e = i < hi ? ids[i] : -1;
        if (e >= E) e = -1;
        place_chunk(e, i, lds, sorted_ids);
    }
}

}  // namespace
}  // namespace alpha_moe

using namespace alpha_moe;

extern "C" int alpha_moe_per_token_group_quant_fp8(const void *x, int x_is_f32, uint8_t *q, float *scale, int M, int K,
                                                   void *stream)
{
    if (!x || !q || !scale) return ALPHA_MOE_ERR_NULL_POINTER;
    if (M <= 0 || K <= 0 || K % 128 != 0) return ALPHA_MOE_ERR_SHAPE;
    const long long n_groups = (long long)M * (K / 128);
    const long long want = (n_groups + 15) / 16;
    const unsigned grid = (unsigned)(want < 8192 ? want : 8192);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    if (x_is_f32)
        hipLaunchKernelGGL(quant_group128_kernel<float>, dim3(grid), dim3(256), 0, hs, static_cast<const float *>(x), q,
                           scale, n_groups);
    else
        hipLaunchKernelGGL(quant_group128_kernel<uint16_t>, dim3(grid), dim3(256), 0, hs,
                           static_cast<const uint16_t *>(x), q, scale, n_groups);
    return hipGetLastError() == hipSuccess ? ALPHA_MOE_OK : ALPHA_MOE_ERR_LAUNCH;
}

extern "C" size_t alpha_moe_align_workspace_bytes(int numel, int num_experts)
{
    if (numel <= 0 || num_experts <= 0) return 0;
    const size_t n_seg = ((size_t)numel + kAlignSeg - 1) / kAlignSeg;
    return n_seg * (size_t)num_experts * sizeof(int);
}

extern "C" int alpha_moe_moe_align_block_size(const int32_t *topk_ids, int numel, int num_experts, int block_size,
                                              int32_t *sorted_token_ids, int sorted_num, int32_t *expert_ids,
                                              int n_blocks, int32_t *num_tokens_post_padded, void *workspace,
                                              size_t workspace_bytes, void *stream)
{
    if (!topk_ids || !sorted_token_ids || !expert_ids || !num_tokens_post_padded) return ALPHA_MOE_ERR_NULL_POINTER;
    if (numel <= 0 || num_experts <= 0 || num_experts > kAlignMaxExperts || block_size <= 0) return ALPHA_MOE_ERR_SHAPE;
    if ((long long)sorted_num != (long long)numel + (long long)num_experts * (block_size - 1) ||
        (long long)n_blocks != ((long long)sorted_num + block_size - 1) / block_size)
        return ALPHA_MOE_ERR_SHAPE;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const int E = num_experts;
    if (numel <= 4 * kAlignSeg) {
        hipLaunchKernelGGL(align_small_kernel, dim3(1), dim3(256), (2 * E + 257) * sizeof(int), hs, topk_ids, numel, E,
                           block_size, sorted_token_ids, sorted_num, expert_ids, n_blocks, num_tokens_post_padded);
        return hipGetLastError() == hipSuccess ? ALPHA_MOE_OK : ALPHA_MOE_ERR_LAUNCH;
    }
    if (!workspace || workspace_bytes < alpha_moe_align_workspace_bytes(numel, E)) return ALPHA_MOE_ERR_WORKSPACE;
    const int n_seg = (numel + kAlignSeg - 1) / kAlignSeg;
    int *hist = static_cast<int *>(workspace);
    hipLaunchKernelGGL(align_hist_kernel, dim3(n_seg), dim3(256), E * sizeof(int), hs, topk_ids, numel, E, hist,
                       sorted_token_ids, sorted_num);
    hipLaunchKernelGGL(align_scan_kernel, dim3(1), dim3(1024), (2 * E + 1025) * sizeof(int), hs, hist, n_seg, E,
                       block_size, expert_ids, n_blocks, num_tokens_post_padded);
    hipLaunchKernelGGL(align_place_kernel, dim3(n_seg), dim3(64), E * sizeof(int), hs, topk_ids, numel, E, hist,
                       sorted_token_ids);
    return hipGetLastError() == hipSuccess ? ALPHA_MOE_OK : ALPHA_MOE_ERR_LAUNCH;
}
