// Fused W8A8 MoE up/gate -> SwiGLU -> FP8 requant -> down -> scatter-add, written for gfx950 (MI355X).
//
// Work decomposition (one workgroup per unit, like the reference's CTA at
// csrc/kernels/fused_moe_w8a8/fused_moe_w8a8_up_down_acc.cu:676-679,767):
//   unit = (block of block_m rows of sorted_token_ids, 128-column slice `ib` of the intermediate)
//        = 256 interleaved w1 rows x K, then K output columns x 128 of w2.
//
// CDNA4 mapping, not a translation of the Hopper pipeline:
//   * v_mfma_f32_16x16x128_f8f6f4 with WEIGHT rows as the A operand and TOKENS as the B operand.  One
//     instruction contracts exactly one 128-wide scale block, so block scales are applied to its fp32 result.
//   * Each wavefront owns its own weight rows, so weights go HBM -> VGPR directly in the MFMA operand layout
//     (lane = (row m = lane%16, K group q = lane/16); the lane's 32 bytes are bytes [16q,16q+16) and
//     [64+16q,64+16q+16) of the 128-byte K block - any K permutation is legal as long as A and B agree - so
//     that the four lanes of a row read 64 contiguous bytes per load).  No LDS staging, no barrier in the loop.
//   * Gate/up pairing under the interleave-8 layout: one MFMA takes the 8+8 gate rows of two 16-row chunks,
//     a second takes their up rows; accumulator register j of a lane is then gate/up of the SAME intermediate
//     column, and a lane owns 4 consecutive columns -> SwiGLU and the FP8 pack stay in registers.
//   * The requantised block_m x 128 FP8 tile crosses lanes once through LDS (accumulator layout != B layout).
//   * Down projection: w2 rows (= output columns) as A gives each lane 4 adjacent output columns of one token
//     -> two global_atomic_pk_add_bf16 per accumulator quad, no transpose.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/alpha_moe_hip.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef short v2s __attribute__((ext_vector_type(2)));

constexpr float kFp8Max = 448.0f;
constexpr float kAmaxFloor = 1e-10f;
constexpr int kLdsRowStride = 144;   // 128 FP8 + 16 pad: dword writes of 16 tokens x 4 quads hit 64 distinct banks

struct MoeParams {
    const uint8_t *x;
    const float *x_scale;
    const uint8_t *w;
    const float *w_scale;
    const uint8_t *w2;
    const float *w2_scale;
    uint16_t *out;
    const int32_t *sorted_ids;
    const int32_t *expert_ids;
    const int32_t *ntpp;
    const float *topk_w;
    int top_k, M, K, N, E, sorted_num, block_m;
    float scaling;
};

__device__ __forceinline__ v4i ldg128(const uint8_t *p) { return *reinterpret_cast<const v4i *>(p); }

__device__ __forceinline__ v8i cat(v4i lo, v4i hi)
{
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

__device__ __forceinline__ v4f mfma_fp8(v8i a, v8i b)
{
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    // cbsz = blgp = 0: both operands OCP e4m3; scale operands 0 -> plain v_mfma_f32_16x16x128_f8f6f4
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, zero, 0, 0, 0, 0, 0, 0);
}

__device__ __forceinline__ float round_bf16(float v) { return static_cast<float>(static_cast<__bf16>(v)); }

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 p = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ float clamp_fp8(float v) { return fminf(fmaxf(v, -kFp8Max), kFp8Max); }

__device__ __forceinline__ uint32_t pack_fp8x4(float a, float b, float c, float d)
{
    int p = 0;
    p = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, p, false);   // RNE to OCP e4m3 on gfx950
    p = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, p, true);
    return static_cast<uint32_t>(p);
}

__device__ __forceinline__ void atomic_add_bf16x2(uint16_t *addr, uint32_t packed)
{
    typedef v2s __attribute__((address_space(1))) * gptr;
    __builtin_amdgcn_global_atomic_fadd_v2bf16(reinterpret_cast<gptr>(reinterpret_cast<uintptr_t>(addr)),
                                               __builtin_bit_cast(v2s, packed));
}

// One K block of operands for one wavefront: NP gate/up row pairs, TM token tiles.
template <int TM, int NP>
struct UpStage {
    v4i ag[NP][2], au[NP][2];
    v4i b[TM][2];
    float xs[TM];
    float wsg, wsu;
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
    const float *wsg_p = p.w_scale + ((size_t)e * (p.N >> 7) + 2 * ib) * nkb;   // gate scale row 2*ib, up row 2*ib+1
    const float *wsu_p = wsg_p + nkb;

    v4f accg[NP][TM], accu[NP][TM];
#pragma unroll
    for (int pr = 0; pr < NP; pr++)
#pragma unroll
        for (int t = 0; t < TM; t++) {
            accg[pr][t] = (v4f){0.f, 0.f, 0.f, 0.f};
            accu[pr][t] = (v4f){0.f, 0.f, 0.f, 0.f};
        }

    UpStage<TM, NP> st[STAGES];
    auto load_up = [&](UpStage<TM, NP> &s, int kb) {
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
        s.wsg = wsg_p[kb];
        s.wsu = wsu_p[kb];
    };
    auto compute_up = [&](const UpStage<TM, NP> &s) {
#pragma unroll
        for (int t = 0; t < TM; t++) {
            const v8i b = cat(s.b[t][0], s.b[t][1]);
            const float sg = s.wsg * s.xs[t];
            const float su = s.wsu * s.xs[t];
#pragma unroll
            for (int pr = 0; pr < NP; pr++) {
                const v4f tg = mfma_fp8(cat(s.ag[pr][0], s.ag[pr][1]), b);
                const v4f tu = mfma_fp8(cat(s.au[pr][0], s.au[pr][1]), b);
                accg[pr][t] += tg * sg;
                accu[pr][t] += tu * su;
            }
        }
    };

#pragma unroll
    for (int s = 0; s < STAGES - 1; s++)
        if (s < nkb) load_up(st[s], s);
    for (int kb0 = 0; kb0 < nkb; kb0 += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            const int kb = kb0 + s;
            if (kb < nkb) {
                const int kpre = kb + STAGES - 1;
                if (kpre < nkb) load_up(st[(s + STAGES - 1) % STAGES], kpre);
                compute_up(st[s]);
            }
        }
    }

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
                const float g = round_bf16(accg[pr][t][j]);
                const float u = round_bf16(accu[pr][t][j]);
                const float a = round_bf16(g / (1.0f + __expf(-g)) * u);
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
    uint16_t *outp[TM];
#pragma unroll
    for (int t = 0; t < TM; t++) outp[t] = p.out + (size_t)tok[t] * K + 4 * q;

    const int n_ct = K >> 4;                      // 16-column tiles
    const int n_it = (n_ct - wave + WN - 1) / WN; // tiles of this wavefront: ct = wave + WN*i
    const uint8_t *w2p = p.w2 + ((size_t)e * K + wave * 16 + n) * I + ib * 128 + 16 * q;
    const size_t w2_step = (size_t)WN * 16 * I;
    const int n_ibk = I >> 7;
    const float *w2s_p = p.w2_scale + (size_t)e * (K >> 7) * n_ibk + ib;

    DownStage ds[STAGES];
    auto load_down = [&](DownStage &s, int i) {
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
                atomic_add_bf16x2(outp[t] + c0, pack_bf16x2(d[0] * sc, d[1] * sc));
                atomic_add_bf16x2(outp[t] + c0 + 2, pack_bf16x2(d[2] * sc, d[3] * sc));
            }
        }
    };
#pragma unroll
    for (int s = 0; s < STAGES - 1; s++)
        if (s < n_it) load_down(ds[s], s);
    for (int i0 = 0; i0 < n_it; i0 += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            const int i = i0 + s;
            if (i < n_it) {
                const int ipre = i + STAGES - 1;
                if (ipre < n_it) load_down(ds[(s + STAGES - 1) % STAGES], ipre);
                compute_down(ds[s], i);
            }
        }
    }
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

extern "C" int alpha_moe_validate(int top_k, int M, int K, int N, int num_experts, int sorted_num, int block_m,
                                  int block_n, int warp_n, int stages)
{
    if (M <= 0 || K <= 0 || N <= 0 || num_experts <= 0 || top_k <= 0 || sorted_num <= 0) return ALPHA_MOE_ERR_SHAPE;
    if (K % 128 != 0 || N % 256 != 0) return ALPHA_MOE_ERR_SHAPE;
    if ((int64_t)M * top_k > INT32_MAX) return ALPHA_MOE_ERR_SHAPE;
    if (block_m < 8 || block_m > 128 || block_m % 8 != 0) return ALPHA_MOE_ERR_BLOCK_M;
    if (!((block_n == 64 && warp_n == 4) || (block_n == 32 && warp_n == 8))) return ALPHA_MOE_ERR_BLOCK_N_WARP_N;
    if (stages < 1 || stages > 5) return ALPHA_MOE_ERR_STAGES;
    const int64_t n_blocks = ((int64_t)sorted_num + block_m - 1) / block_m;
    if (n_blocks * (N / 256) > INT32_MAX) return ALPHA_MOE_ERR_SHAPE;
    return ALPHA_MOE_OK;
}

extern "C" int alpha_moe_fused_moe_w8a8_up_down(const uint8_t *x, const float *x_scale, const uint8_t *w,
                                                const float *w_scale, const uint8_t *w2, const float *w2_scale,
                                                uint16_t *out, const int32_t *sorted_token_ids,
                                                const int32_t *expert_ids, const int32_t *num_tokens_post_padded,
                                                const float *topk_weights, int top_k, int M, int K, int N,
                                                int num_experts, int sorted_num, int block_m, int block_n, int warp_n,
                                                int stages, float scaling_factor, void *stream)
{
    if (!x || !x_scale || !w || !w_scale || !w2 || !w2_scale || !out || !sorted_token_ids || !expert_ids ||
        !num_tokens_post_padded || !topk_weights)
        return ALPHA_MOE_ERR_NULL_POINTER;
    const int rc = alpha_moe_validate(top_k, M, K, N, num_experts, sorted_num, block_m, block_n, warp_n, stages);
    if (rc != ALPHA_MOE_OK) return rc;

    MoeParams p;
    p.x = x; p.x_scale = x_scale; p.w = w; p.w_scale = w_scale; p.w2 = w2; p.w2_scale = w2_scale;
    p.out = out; p.sorted_ids = sorted_token_ids; p.expert_ids = expert_ids; p.ntpp = num_tokens_post_padded;
    p.topk_w = topk_weights;
    p.top_k = top_k; p.M = M; p.K = K; p.N = N; p.E = num_experts; p.sorted_num = sorted_num; p.block_m = block_m;
    p.scaling = scaling_factor;

    const int tm = (block_m + 15) / 16;
    const KernelFn fn = warp_n == 4 ? pick_tm<4>(tm, stages) : pick_tm<8>(tm, stages);
    const int n_blocks = (sorted_num + block_m - 1) / block_m;
    const dim3 grid((unsigned)(n_blocks * (N / 256)));
    const dim3 block((unsigned)(warp_n * 64));
    hipLaunchKernelGGL(fn, grid, block, 0, static_cast<hipStream_t>(stream), p);
    return hipGetLastError() == hipSuccess ? ALPHA_MOE_OK : ALPHA_MOE_ERR_LAUNCH;
}

extern "C" const char *alpha_moe_status_string(int status)
{
    switch (status) {
    case ALPHA_MOE_OK: return "ok";
    case ALPHA_MOE_ERR_NULL_POINTER: return "a required pointer is null";
    case ALPHA_MOE_ERR_SHAPE: return "unsupported shape: need M>0, top_k>0, K % 128 == 0, N % 256 == 0, sizes within int32";
    case ALPHA_MOE_ERR_BLOCK_M: return "block_m must be a multiple of 8 in [8, 128]";
    case ALPHA_MOE_ERR_BLOCK_N_WARP_N: return "(block_n, warp_n) must be (64, 4) or (32, 8)";
    case ALPHA_MOE_ERR_STAGES: return "stages must be in [1, 5]";
    case ALPHA_MOE_ERR_LAUNCH: return "the HIP runtime refused the kernel launch";
    default: return "unknown status";
    }
}

extern "C" const char *alpha_moe_version(void) { return "0.1"; }
