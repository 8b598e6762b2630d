// Fused W8A8 MoE, "direct" kernel: one workgroup per unit, weights HBM -> VGPR in the MFMA operand layout.
//
// Work decomposition (one workgroup per unit, like the reference's CTA at
// csrc/kernels/fused_moe_w8a8/fused_moe_w8a8_up_down_acc.cu:676-679,767):
//   unit = (block of block_m rows of sorted_token_ids, 128-column slice `ib` of the intermediate)
//        = 256 interleaved w1 rows x K, then K output columns x 128 of w2.
// Each wavefront owns its own weight rows, so nothing is shared between wavefronts until the 128-column
// requantisation group is reduced; the requantised block_m x 128 FP8 tile crosses lanes once through LDS
// (accumulator layout != B layout).  Down projection: w2 rows (= output columns) as A gives each lane 4 adjacent
// output columns of one token.  Partial output rows are summed in an fp32 scratch row (cleared by a fill kernel
// first) with hardware fp32 atomics and rounded to bf16 once by the finalize kernel (adding every partial straight into the bf16 output would round
// the running sum top_k * I/128 times, ~1.5e-2 of the output range for DeepSeek-V3 routing weights).
//
// Handles every block_m in 8..128; the persistent streaming kernel in moe_stream.hip is the fast path for
// block_m <= 32.
#include "moe_common.hpp"

namespace alpha_moe {
namespace {

// One K block of operands for one wavefront: NP gate/up row pairs, TM token tiles.
template <int TM, int NP>
struct UpStage {
    v4i ag[NP][2], au[NP][2];
    v4i b[TM][2];
    float xs[TM];
};

struct DownStage {
    v4i a[2];
    float ws;
};

// TM: 16-token tiles per block (block_m <= 16*TM); WN: wavefronts per workgroup; STAGES: K blocks in flight.
template <int TM, int WN, int STAGES>
__global__ __launch_bounds__(WN * 64) void fused_moe_w8a8_direct_kernel(const MoeParams p)
{
    constexpr int RW = 256 / WN;    // interleaved w1 rows per wavefront
    constexpr int NP = RW / 32;     // gate/up MFMA pairs per wavefront per K block
    const int n_ib = p.N >> 8;
    const int mb = blockIdx.x / n_ib;
    const int ib = blockIdx.x - mb * n_ib;
    if (mb * p.block_m >= p.ntpp[0]) return;
    const int e = p.expert_ids[mb];
    if (e < 0 || e >= p.E) return;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;        // MFMA row (weights) / column (tokens) this lane feeds
    const int q = lane >> 4;        // K group this lane feeds; also the row quad of its accumulators
    const int K = p.K, I = p.N >> 1;
    const int nkb = K >> 7;

    // ---- routing: which token each B column is -------------------------------------------------
    int tok[TM];
    int slot[TM];
    bool valid[TM];
#pragma unroll
    for (int t = 0; t < TM; t++) {
        const int r = t * 16 + n;
        const int idx = mb * p.block_m + r;
        int id = -1;
        if (r < p.block_m && idx < p.sorted_num) id = p.sorted_ids[idx];
        const int tk = id / p.top_k;
        valid[t] = id >= 0 && tk < p.M;
        tok[t] = valid[t] ? tk : 0;
        slot[t] = valid[t] ? id : 0;
    }

    const uint8_t *xp[TM];
    const float *xsp[TM];
#pragma unroll
    for (int t = 0; t < TM; t++) {
        xp[t] = p.x + (size_t)tok[t] * K + 16 * q;
        xsp[t] = p.x_scale + (size_t)tok[t] * nkb;
    }
    // A row m of the gate MFMA of pair pr <- slab row pr*32 + (m/8)*16 + m%8; its up partner is 8 rows below
    const uint8_t *wg[NP];
#pragma unroll
    for (int pr = 0; pr < NP; pr++) {
        const int row = ib * 256 + wave * RW + pr * 32 + (n >> 3) * 16 + (n & 7);
        wg[pr] = p.w + ((size_t)e * p.N + row) * K + 16 * q;
    }
    // This unit's two w1 scale rows (gate = row 2*ib, up = row 2*ib+1 of the interleaved scale tensor) go to LDS
    // once: reading them per K block with scalar loads would put an out-of-order counter into the pipelined loop.
    __shared__ float s_ws[2][kMaxKBlocks];
    {
        const float *ws_rows = p.w_scale + ((size_t)e * (p.N >> 7) + 2 * ib) * nkb;
        for (int i = threadIdx.x; i < 2 * nkb; i += WN * 64) s_ws[i >= nkb][i >= nkb ? i - nkb : i] = ws_rows[i];
    }
    __syncthreads();

    v4f accg[NP][TM], accu[NP][TM];
#pragma unroll
    for (int pr = 0; pr < NP; pr++)
#pragma unroll
        for (int t = 0; t < TM; t++) {
            accg[pr][t] = (v4f){0.f, 0.f, 0.f, 0.f};
            accu[pr][t] = (v4f){0.f, 0.f, 0.f, 0.f};
        }

    UpStage<TM, NP> st[STAGES];
    // kb is clamped so that prefetches past the end stay in bounds; their data is never used
    auto load_up = [&](UpStage<TM, NP> &s, int kb) {
        kb = kb < nkb ? kb : nkb - 1;
        const int ko = kb << 7;
#pragma unroll
        for (int pr = 0; pr < NP; pr++) {
            s.ag[pr][0] = ldg128(wg[pr] + ko);
            s.ag[pr][1] = ldg128(wg[pr] + ko + 64);
            s.au[pr][0] = ldg128(wg[pr] + (size_t)8 * K + ko);
            s.au[pr][1] = ldg128(wg[pr] + (size_t)8 * K + ko + 64);
        }
#pragma unroll
        for (int t = 0; t < TM; t++) {
            s.b[t][0] = ldg128(xp[t] + ko);
            s.b[t][1] = ldg128(xp[t] + ko + 64);
            s.xs[t] = xsp[t][kb];
        }
    };
    auto compute_up = [&](const UpStage<TM, NP> &s, int kb) {
        const float wsg = s_ws[0][kb], wsu = s_ws[1][kb];
#pragma unroll
        for (int t = 0; t < TM; t++) {
            const v8i b = cat(s.b[t][0], s.b[t][1]);
            const float sg = wsg * s.xs[t];
            const float su = wsu * s.xs[t];
#pragma unroll
            for (int pr = 0; pr < NP; pr++) {
                const v4f tg = mfma_fp8(cat(s.ag[pr][0], s.ag[pr][1]), b);
                const v4f tu = mfma_fp8(cat(s.au[pr][0], s.au[pr][1]), b);
                accg[pr][t] += tg * sg;
                accu[pr][t] += tu * su;
            }
        }
    };

    // Software pipeline, STAGES K blocks deep.  The steady-state loop is branch-free (every prefetch is issued
    // unconditionally) so that the compiler's s_waitcnt vmcnt(N) leaves the younger prefetches in flight; the
    // last nkb % STAGES blocks are drained afterwards.
#pragma unroll
    for (int s = 0; s < STAGES - 1; s++) load_up(st[s], s);
    const int nkb_full = nkb - nkb % STAGES;
    for (int kb0 = 0; kb0 < nkb_full; kb0 += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            load_up(st[(s + STAGES - 1) % STAGES], kb0 + s + STAGES - 1);
            __builtin_amdgcn_sched_barrier(0);   // keep the prefetch ahead of the MFMAs that hide its latency
            compute_up(st[s], kb0 + s);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int s = 0; s < STAGES - 1; s++)
        if (nkb_full + s < nkb) compute_up(st[s], nkb_full + s);

    // ---- SwiGLU, per-token amax over the 128 columns, FP8 requant -----------------------------
    __shared__ float s_amax[WN][TM * 16];
    __shared__ __attribute__((aligned(16))) uint8_t s_aq[TM * 16][kLdsRowStride];

#pragma unroll
    for (int t = 0; t < TM; t++) {
        float m = 0.f;
#pragma unroll
        for (int pr = 0; pr < NP; pr++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float a = swiglu_bf16(accg[pr][t][j], accu[pr][t][j]);
                accg[pr][t][j] = a;
                m = fmaxf(m, fabsf(a));
            }
        m = fmaxf(m, __shfl_xor(m, 16));
        m = fmaxf(m, __shfl_xor(m, 32));
        if (q == 0) s_amax[wave][t * 16 + n] = m;
    }
    __syncthreads();
    float tscale[TM];
#pragma unroll
    for (int t = 0; t < TM; t++) {
        float m = kAmaxFloor;
#pragma unroll
        for (int wv = 0; wv < WN; wv++) m = fmaxf(m, s_amax[wv][t * 16 + n]);
        const float s_a = m / kFp8Max;
#pragma unroll
        for (int pr = 0; pr < NP; pr++) {
            const uint32_t packed = pack_fp8x4(clamp_fp8(accg[pr][t][0] / s_a), clamp_fp8(accg[pr][t][1] / s_a),
                                               clamp_fp8(accg[pr][t][2] / s_a), clamp_fp8(accg[pr][t][3] / s_a));
            const int col = wave * (RW / 2) + pr * 16 + 4 * q;
            *reinterpret_cast<uint32_t *>(&s_aq[t * 16 + n][col]) = packed;
        }
        tscale[t] = s_a * (p.topk_w[slot[t]] * p.scaling);
    }
    __syncthreads();

    // ---- down projection: 16 output columns x all tokens per MFMA -----------------------------
    v8i ba[TM];
#pragma unroll
    for (int t = 0; t < TM; t++) {
        const v4i lo = *reinterpret_cast<const v4i *>(&s_aq[t * 16 + n][16 * q]);
        const v4i hi = *reinterpret_cast<const v4i *>(&s_aq[t * 16 + n][64 + 16 * q]);
        ba[t] = cat(lo, hi);
    }
    float *accp[TM];
#pragma unroll
    for (int t = 0; t < TM; t++) accp[t] = p.acc + (size_t)tok[t] * K + 4 * q;

    const int n_ct = K >> 4;                      // 16-column tiles
    const int n_it = (n_ct - wave + WN - 1) / WN; // tiles of this wavefront: ct = wave + WN*i
    const uint8_t *w2p = p.w2 + ((size_t)e * K + wave * 16 + n) * I + ib * 128 + 16 * q;
    const size_t w2_step = (size_t)WN * 16 * I;
    const int n_ibk = I >> 7;
    const float *w2s_p = p.w2_scale + (size_t)e * (K >> 7) * n_ibk + ib;

    DownStage ds[STAGES];
    auto load_down = [&](DownStage &s, int i) {
        i = i < n_it ? i : n_it - 1;
        const uint8_t *a = w2p + (size_t)i * w2_step;
        s.a[0] = ldg128(a);
        s.a[1] = ldg128(a + 64);
        s.ws = w2s_p[(size_t)(((wave + WN * i) << 4) >> 7) * n_ibk];
    };
    auto compute_down = [&](const DownStage &s, int i) {
        const int c0 = (wave + WN * i) << 4;
        const v8i a = cat(s.a[0], s.a[1]);
#pragma unroll
        for (int t = 0; t < TM; t++) {
            const v4f d = mfma_fp8(a, ba[t]);
            const float sc = tscale[t] * s.ws;
            if (valid[t]) {
#pragma unroll
                for (int j = 0; j < 4; j++) atomic_add_f32(accp[t] + c0 + j, d[j] * sc);
            }
        }
    };
    if (n_it > 0) {
#pragma unroll
        for (int s = 0; s < STAGES - 1; s++) load_down(ds[s], s);
        const int n_full = n_it - n_it % STAGES;
        for (int i0 = 0; i0 < n_full; i0 += STAGES) {
#pragma unroll
            for (int s = 0; s < STAGES; s++) {
                load_down(ds[(s + STAGES - 1) % STAGES], i0 + s + STAGES - 1);
                __builtin_amdgcn_sched_barrier(0);
                compute_down(ds[s], i0 + s);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int s = 0; s < STAGES - 1; s++)
            if (n_full + s < n_it) compute_down(ds[s], n_full + s);
    }
}

__global__ __launch_bounds__(256) void moe_zero_kernel(float *__restrict__ acc, int n4)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n4) reinterpret_cast<v4f *>(acc)[i] = (v4f){0.f, 0.f, 0.f, 0.f};
}

// out[i] = bf16(float(out[i]) + acc[i]), or bf16(acc[i]) when overwriting.  n4 = M*K/4 (K % 128 == 0, so rows never
// straddle).
__global__ __launch_bounds__(256) void moe_finalize_kernel(float *__restrict__ acc, uint16_t *__restrict__ out, int n4,
                                                           int overwrite)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    v4f a = reinterpret_cast<v4f *>(acc)[i];
    uint2 o = {0u, 0u};
    if (!overwrite) o = reinterpret_cast<uint2 *>(out)[i];
    const float o0 = __builtin_bit_cast(float, o.x << 16), o1 = __builtin_bit_cast(float, o.x & 0xffff0000u);
    const float o2 = __builtin_bit_cast(float, o.y << 16), o3 = __builtin_bit_cast(float, o.y & 0xffff0000u);
    o.x = pack_bf16x2(o0 + a[0], o1 + a[1]);
    o.y = pack_bf16x2(o2 + a[2], o3 + a[3]);
    reinterpret_cast<uint2 *>(out)[i] = o;
}

typedef void (*KernelFn)(const MoeParams);

// Registers bound how many K blocks a wavefront can keep in flight (accumulators 16*NP*TM, one stage
// 16*NP + 9*TM + 2 VGPRs).  Deepest depth per (WN, TM) that compiles without scratch spills; deeper requests
// are clamped, which does not change the result.
constexpr int max_stages(int tm, int wn)
{
    constexpr int wn4[8] = {5, 5, 5, 5, 4, 3, 3, 2};
    constexpr int wn8[8] = {5, 5, 4, 3, 2, 1, 1, 1};
    return wn == 4 ? wn4[tm - 1] : wn8[tm - 1];
}

template <int TM, int WN, int S>
KernelFn pick_stages(int stages)
{
    if constexpr (S > max_stages(TM, WN)) {
        return pick_stages<TM, WN, S - 1>(stages);
    } else {
        if (stages >= S || S == 1) return fused_moe_w8a8_direct_kernel<TM, WN, S>;
        if constexpr (S > 1) return pick_stages<TM, WN, S - 1>(stages);
        return nullptr;
    }
}

template <int WN>
KernelFn pick_tm(int tm, int stages)
{
    switch (tm) {
    case 1: return pick_stages<1, WN, 5>(stages);
    case 2: return pick_stages<2, WN, 5>(stages);
    case 3: return pick_stages<3, WN, 5>(stages);
    case 4: return pick_stages<4, WN, 5>(stages);
    case 5: return pick_stages<5, WN, 5>(stages);
    case 6: return pick_stages<6, WN, 5>(stages);
    case 7: return pick_stages<7, WN, 5>(stages);
    default: return pick_stages<8, WN, 5>(stages);
    }
}

}  // namespace

hipError_t launch_direct(const MoeParams &p, int warp_n, int stages, hipStream_t stream)
{
    const int tm = (p.block_m + 15) / 16;
    const KernelFn fn = warp_n == 4 ? pick_tm<4>(tm, stages) : pick_tm<8>(tm, stages);
    const int n_blocks = (p.sorted_num + p.block_m - 1) / p.block_m;
    const dim3 grid((unsigned)(n_blocks * (p.N / 256)));
    hipLaunchKernelGGL(fn, grid, dim3((unsigned)(warp_n * 64)), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_zero_acc(const MoeParams &p, hipStream_t stream)
{
    // a fill kernel, not hipMemsetAsync: the call may be captured into a HIP graph
    const int n4 = (int)((int64_t)p.M * p.K / 4);
    hipLaunchKernelGGL(moe_zero_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, stream, p.acc, n4);
    return hipGetLastError();
}

hipError_t launch_finalize(const MoeParams &p, hipStream_t stream)
{
    const int n4 = (int)((int64_t)p.M * p.K / 4);
    hipLaunchKernelGGL(moe_finalize_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, stream, p.acc, p.out, n4,
                       p.overwrite);
    return hipGetLastError();
}

}  // namespace alpha_moe
