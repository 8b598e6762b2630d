// Fused W8A8 MoE, "streaming" kernel for decode-sized batches (block_m <= 32): ONE persistent launch that moves
// every active expert's weights through the chip once at HBM speed.
//
// Why not one workgroup per (row block, 128-column slice) like the reference's CTA
// (fused_moe_w8a8_up_down_acc.cu:676-679,767)?  On MI355X one CU sustains ~45 GB/s of HBM reads, the chip ~6.9 TB/s,
// so a decode step (DeepSeek-V3 shard, M=1: 18 such units of 2.75 MB) must be cut into hundreds of pieces to
// engage all 256 CUs.  The 128-column requantisation group forces a dependency between the pieces, so the kernel
// is a small dataflow over a work queue (items are taken in queue order with one atomic):
//
//   UP item   (unit u = (row block mb, slice ib), K split ks): 256 interleaved w1 rows x kbpi K blocks.  Partial
//             gate/up sums of the VALID tokens are added into h[u] (fp32 atomics); the item that arrives last at
//             arrive[u] reads h[u], applies SwiGLU, quantises the block_m x 128 tile to FP8 (aq[u], sa[u]) and
//             publishes flag[u] = 1.  With a single K split the sums never leave registers.
//   DOWN item (unit u, column slab cs): waits for flag[u], then tpi 16-column tiles of w2[e][:, 128*ib : +128];
//             results are added into acc[token] (fp32 atomics), then down_done is bumped.
//   FIN item  (chunk of acc): waits for down_done == number of DOWN items, then out = bf16(out + acc), acc = 0,
//             and clears its share of flag/aq/sa.
//
// Every wait is on items EARLIER in the queue, which are already held by running workgroups that never wait on
// later ones, so the queue drains whatever the number of resident workgroups; each spin is bounded and sets
// ctl->error instead of hanging.  Everything in the workspace is zero again when the kernel ends (arrive, h and acc
// are cleared by their last reader, flag/aq/sa by the FIN items, head/done/down_done by the last workgroup to
// leave), so one zero-filled buffer serves calls of any size without a memset in between.
//
// Data movement: weights go HBM -> LDS with non-temporal global_load_lds_dwordx4 (measured: 6.9 TB/s against
// 3.4 TB/s for the same loads without the non-temporal hint, and 5.5 TB/s for direct-to-VGPR loads in the MFMA
// lane order), into a per-wavefront ring of 16-row x 128-byte tiles, so the loop needs no workgroup barrier.  Inside
// a tile, 16-byte chunk c of row m sits at position c ^ ((m >> 1) & 7): the MFMA operand read (16 rows at a fixed
// chunk) then touches 16 distinct bank quads.  Token rows (a few KB, L2-resident) are loaded straight to VGPRs.
#include <stdlib.h>

#include <mutex>
#include <vector>

#include "moe_common.hpp"

namespace alpha_moe {
namespace {

struct StreamCtl {
    int head;        // next work item
    int done;        // workgroups that have left
    int reserved;
    int down_done;   // finished DOWN items of this launch
    int error;       // sticky: a bounded wait ran out
    int pad[59];
};
static_assert(sizeof(StreamCtl) == 256, "control block is one 256-byte line group");

struct StreamPlan {
    MoeParams p;
    StreamCtl *ctl;
    int *arrive;     // [units]
    int *flag;       // [units]
    float *sa;       // [units][bm_pad]           requantisation scale per token
    uint8_t *aq;     // [units][bm_pad][128]      requantised SwiGLU output, FP8
    float *h;        // [units][bm_pad][2][128]   partial gate/up sums (K-split only)
    int n_ib, nkb, n_ct, n_mb_max;
    int kbpi, ks;    // K blocks per UP item, UP items per unit
    int tpi, n_cs;   // 16-column tiles per DOWN item, DOWN items per unit
    int n_fin;       // FIN items
    int bm_pad;
};

typedef const void __attribute__((address_space(1))) * gptr_t;
typedef void __attribute__((address_space(3))) * lptr_t;

// 64 lanes x 16 bytes, HBM -> LDS at lds + lane*16, bypassing VGPRs; aux 2 = non-temporal
__device__ __forceinline__ void dma16_nt(const uint8_t *g, uint8_t *lds)
{
    __builtin_amdgcn_global_load_lds((gptr_t)(uintptr_t)g, (lptr_t)(uint32_t)(uintptr_t)lds, 16, 0, 2);
}

// Global loads the compiler does not track: the pipelines below count vector-memory operations themselves and
// place their own s_waitcnt vmcnt(N) (the compiler cannot see direct-to-LDS loads complete and, left to insert the
// waits for ordinary loads mixed in between them, drains the whole queue every iteration).
__device__ __forceinline__ v4i ldg128_untracked(const uint8_t *p, int byte_offset)
{
    v4i r;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r) : "v"(p + byte_offset) : "memory");
    return r;
}
__device__ __forceinline__ float ldg32_untracked(const float *p)
{
    float r;
    asm volatile("global_load_dword %0, %1, off" : "=v"(r) : "v"(p) : "memory");
    return r;
}

// Agent-scope (sc1) accesses for data that crosses workgroups inside one launch: they are served at the point
// where all XCDs agree, so no L2-wide write-back / invalidate (what a __threadfence() costs here) is needed.
__device__ __forceinline__ v4i ldg128_agent(const void *p)
{
    v4i r;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(r) : "v"(p) : "memory");
    return r;
}
__device__ __forceinline__ void stg32_agent(void *p, uint32_t v)
{
    asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void stg128_agent(void *p, v4i v)
{
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void atomic_add_f32_agent(float *p, float v)
{
    asm volatile("global_atomic_add_f32 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
// all of this wavefront's vector-memory operations (loads, stores, atomics) have completed
__device__ __forceinline__ void drain_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
    __builtin_amdgcn_sched_barrier(0);   // consumers of untracked loads must not be scheduled above the wait
}

// STAGES-deep software pipeline over n steps.  issue(slot, step) must clamp `step` itself (prefetches past the end
// are issued unconditionally so that the steady-state loop is branch-free) and issues exactly LPS vector-memory
// instructions; compute(slot, step) consumes them.
template <int STAGES, int LPS, class Issue, class Compute>
__device__ __forceinline__ void pipeline(int n, Issue issue, Compute compute)
{
#pragma unroll
    for (int s = 0; s < STAGES - 1; s++) issue(s, s);
    const int n_full = n - n % STAGES;
    for (int i0 = 0; i0 < n_full; i0 += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            issue((s + STAGES - 1) % STAGES, i0 + s + STAGES - 1);
            __builtin_amdgcn_sched_barrier(0);
            wait_vmcnt<(STAGES - 1) * LPS>();
            compute(s, i0 + s);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if constexpr (STAGES > 1) {
        // drain: slots 0..STAGES-2 are in flight, oldest first.  Waiting for all of them at once costs nothing here.
        wait_vmcnt<0>();
#pragma unroll
        for (int s = 0; s < STAGES - 1; s++)
            if (n_full + s < n) compute(s, n_full + s);
    }
    wait_vmcnt<0>();
}

__device__ __forceinline__ int load_agent(const int *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_agent(int *p, int v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Bounded wait for *addr >= target (one thread).  ~4M polls with a sleep between them, i.e. seconds.
__device__ __noinline__ void spin_until_ge(const int *addr, int target, StreamCtl *ctl)
{
    for (int it = 0; it < (1 << 22); it++) {
        if (load_agent(addr) >= target) return;
        __builtin_amdgcn_s_sleep(8);
    }
    store_agent(&ctl->error, 1);
}

template <int TM>
struct Routing {
    int tok[TM];
    int slot[TM];
    bool valid[TM];
};

template <int TM>
__device__ __forceinline__ Routing<TM> load_routing(const MoeParams &p, int mb, int n)
{
    Routing<TM> r;
#pragma unroll
    for (int t = 0; t < TM; t++) {
        const int row = t * 16 + n;
        const int idx = mb * p.block_m + row;
        int id = -1;
        if (row < p.block_m && idx < p.sorted_num) id = p.sorted_ids[idx];
        const int tk = id / p.top_k;
        r.valid[t] = id >= 0 && tk < p.M;
        r.tok[t] = r.valid[t] ? tk : 0;
        r.slot[t] = r.valid[t] ? id : 0;
    }
    return r;
}

template <int TM, int WN, int STAGES>
__global__ __launch_bounds__(WN * 64) void moe_stream_kernel(const StreamPlan s)
{
    constexpr int RW = 256 / WN;            // w1 rows per wavefront
    constexpr int NP = RW / 32;             // gate/up MFMA pairs per wavefront per K block
    constexpr int NT = 2 * NP;              // 16x128 weight tiles per wavefront per UP stage
    constexpr int DT = RW / 16;             // 16x128 weight tiles per wavefront per DOWN stage
    constexpr int STAGE_BYTES = RW * 128;
    constexpr int THREADS = WN * 64;
    constexpr int FIN_CHUNK = THREADS * 4;  // float4 elements per FIN item

    extern __shared__ __attribute__((aligned(1024))) uint8_t ring_all[];
    __shared__ float s_ws[2][kMaxKBlocks];
    __shared__ float s_amax[WN][TM * 16];
    __shared__ int s_bcast[2];

    const MoeParams &p = s.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int n = lane & 15;
    const int q = lane >> 4;
    const int K = p.K, I = p.N >> 1;
    uint8_t *ring = ring_all + wave * (STAGES * STAGE_BYTES);

    // operand read offsets inside a 16x128 tile (see the swizzle note at the top of the file)
    const int f_n = (n >> 1) & 7;
    const int frag_lo = n * 128 + 16 * (q ^ f_n);
    const int frag_hi = n * 128 + 16 * ((q ^ f_n) ^ 4);
    // loader side: this lane fills position (row l/8 (+8 for the second instruction), chunk slot l%8) of a tile
    const int ld_row = lane >> 3;
    int ld_chunk[2];
#pragma unroll
    for (int i = 0; i < 2; i++) ld_chunk[i] = (lane & 7) ^ (((8 * i + ld_row) >> 1) & 7);

    int n_mb = (s.p.ntpp[0] + p.block_m - 1) / p.block_m;
    n_mb = n_mb < s.n_mb_max ? n_mb : s.n_mb_max;
    const int n_units = n_mb * s.n_ib;
    const int n_up = n_units * s.ks;
    const int n_down = n_units * s.n_cs;
    const int total = n_up + n_down + s.n_fin;

    auto read_tile = [&](const uint8_t *tile) -> v8i {
        return cat(*reinterpret_cast<const v4i *>(tile + frag_lo), *reinterpret_cast<const v4i *>(tile + frag_hi));
    };

    // SwiGLU + per-token amax over the 128 columns + FP8 requant of one unit, from accumulators in the MFMA layout.
    auto activate_and_publish = [&](int u, v4f (&accg)[NP][TM], v4f (&accu)[NP][TM]) {
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
        uint8_t *aq_u = s.aq + (size_t)u * s.bm_pad * 128;
#pragma unroll
        for (int t = 0; t < TM; t++) {
            float m = kAmaxFloor;
#pragma unroll
            for (int wv = 0; wv < WN; wv++) m = fmaxf(m, s_amax[wv][t * 16 + n]);
            const float s_a = m / kFp8Max;
#pragma unroll
            for (int pr = 0; pr < NP; pr++) {
                const uint32_t packed =
                    pack_fp8x4(clamp_fp8(accg[pr][t][0] / s_a), clamp_fp8(accg[pr][t][1] / s_a),
                               clamp_fp8(accg[pr][t][2] / s_a), clamp_fp8(accg[pr][t][3] / s_a));
                const int col = wave * (RW / 2) + pr * 16 + 4 * q;
                stg32_agent(aq_u + (t * 16 + n) * 128 + col, packed);
            }
            if (wave == 0 && q == 0)
                stg32_agent(&s.sa[(size_t)u * s.bm_pad + t * 16 + n], __builtin_bit_cast(uint32_t, s_a));
        }
        drain_vmem();
        __syncthreads();
        if (tid == 0) store_agent(&s.flag[u], 1);
    };

    auto up_item = [&](int item) {
        const int u = item / s.ks;
        const int ksp = item - u * s.ks;
        const int mb = u / s.n_ib;
        const int ib = u - mb * s.n_ib;
        const int e = p.expert_ids[mb];
        if (e < 0 || e >= p.E) return;
        const int kb0 = ksp * s.kbpi;
        const int nk = (s.nkb - kb0) < s.kbpi ? (s.nkb - kb0) : s.kbpi;
        const Routing<TM> r = load_routing<TM>(p, mb, n);

        // this unit's gate (row 2*ib) and up (row 2*ib+1) scale rows, K range of the item
        {
            const float *ws_rows = p.w_scale + ((size_t)e * (p.N >> 7) + 2 * ib) * s.nkb + kb0;
            for (int i = tid; i < 2 * nk; i += THREADS) {
                const int up = i >= nk;
                s_ws[up][i - up * nk] = ws_rows[up * s.nkb + (i - up * nk)];
            }
        }
        __syncthreads();

        const uint8_t *ga[NT][2];
#pragma unroll
        for (int a = 0; a < NT; a++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                // tile a = (pair a/2, gate|up a%2); tile row 8i + l/8 is slab row pair*32 + 16i + l/8 (+8 for up)
                const int row = ib * 256 + wave * RW + (a >> 1) * 32 + 16 * i + ld_row + 8 * (a & 1);
                ga[a][i] = p.w + ((size_t)e * p.N + row) * K + (size_t)kb0 * 128 + 16 * ld_chunk[i];
            }
        const uint8_t *xp[TM];
        const float *xsp[TM];
#pragma unroll
        for (int t = 0; t < TM; t++) {
            xp[t] = p.x + (size_t)r.tok[t] * K + (size_t)kb0 * 128 + 16 * q;
            xsp[t] = p.x_scale + (size_t)r.tok[t] * s.nkb + kb0;
        }

        v4f accg[NP][TM], accu[NP][TM];
#pragma unroll
        for (int pr = 0; pr < NP; pr++)
#pragma unroll
            for (int t = 0; t < TM; t++) {
                accg[pr][t] = (v4f){0.f, 0.f, 0.f, 0.f};
                accu[pr][t] = (v4f){0.f, 0.f, 0.f, 0.f};
            }

        struct BStage {
            v4i b[TM][2];
            float xs[TM];
        } bst[STAGES];
        constexpr int LPS = NT * 2 + TM * 3;

        auto issue = [&](int slot, int kb) {
            kb = kb < nk ? kb : nk - 1;
            uint8_t *dst = ring + slot * STAGE_BYTES;
#pragma unroll
            for (int a = 0; a < NT; a++)
#pragma unroll
                for (int i = 0; i < 2; i++) dma16_nt(ga[a][i] + (size_t)kb * 128, dst + a * 2048 + i * 1024);
#pragma unroll
            for (int t = 0; t < TM; t++) {
                bst[slot].b[t][0] = ldg128_untracked(xp[t] + (size_t)kb * 128, 0);
                bst[slot].b[t][1] = ldg128_untracked(xp[t] + (size_t)kb * 128, 64);
                bst[slot].xs[t] = ldg32_untracked(xsp[t] + kb);
            }
        };
        auto compute = [&](int slot, int kb) {
            const uint8_t *src = ring + slot * STAGE_BYTES;
            const float wsg = s_ws[0][kb], wsu = s_ws[1][kb];
            v8i ag[NP], au[NP];
#pragma unroll
            for (int pr = 0; pr < NP; pr++) {
                ag[pr] = read_tile(src + (2 * pr) * 2048);
                au[pr] = read_tile(src + (2 * pr + 1) * 2048);
            }
#pragma unroll
            for (int t = 0; t < TM; t++) {
                const v8i b = cat(bst[slot].b[t][0], bst[slot].b[t][1]);
                const float sg = wsg * bst[slot].xs[t];
                const float su = wsu * bst[slot].xs[t];
#pragma unroll
                for (int pr = 0; pr < NP; pr++) {
                    accg[pr][t] += mfma_fp8(ag[pr], b) * sg;
                    accu[pr][t] += mfma_fp8(au[pr], b) * su;
                }
            }
        };
        pipeline<STAGES, LPS>(nk, issue, compute);

        if (s.ks > 1) {
            // K-split: add the valid tokens' partial sums into h[u]; the last arrival takes the totals back
            float *h_u = s.h + (size_t)u * s.bm_pad * 256;
#pragma unroll
            for (int t = 0; t < TM; t++) {
                if (!r.valid[t]) continue;
#pragma unroll
                for (int pr = 0; pr < NP; pr++) {
                    float *dst = h_u + (t * 16 + n) * 256 + wave * (RW / 2) + pr * 16 + 4 * q;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        atomic_add_f32_agent(dst + j, accg[pr][t][j]);
                        atomic_add_f32_agent(dst + 128 + j, accu[pr][t][j]);
                    }
                }
            }
            drain_vmem();
            __syncthreads();
            if (tid == 0)
                s_bcast[1] = __hip_atomic_fetch_add(&s.arrive[u], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            if (s_bcast[1] != s.ks - 1) return;
#pragma unroll
            for (int t = 0; t < TM; t++)
#pragma unroll
                for (int pr = 0; pr < NP; pr++) {
                    float *src = h_u + (t * 16 + n) * 256 + wave * (RW / 2) + pr * 16 + 4 * q;
                    v4i g = {0, 0, 0, 0}, up = {0, 0, 0, 0};
                    if (r.valid[t]) {
                        g = ldg128_agent(src);
                        up = ldg128_agent(src + 128);
                    }
                    drain_vmem();
                    accg[pr][t] = __builtin_bit_cast(v4f, g);
                    accu[pr][t] = __builtin_bit_cast(v4f, up);
                    if (r.valid[t]) {
                        stg128_agent(src, (v4i){0, 0, 0, 0});
                        stg128_agent(src + 128, (v4i){0, 0, 0, 0});
                    }
                }
            if (tid == 0) store_agent(&s.arrive[u], 0);
        }
        activate_and_publish(u, accg, accu);
    };

    auto down_item = [&](int item) {
        const int u = item / s.n_cs;
        const int cs = item - u * s.n_cs;
        const int mb = u / s.n_ib;
        const int ib = u - mb * s.n_ib;
        const int e = p.expert_ids[mb];
        if (e >= 0 && e < p.E) {
            if (tid == 0) spin_until_ge(&s.flag[u], 1, s.ctl);
            __syncthreads();
            const Routing<TM> r = load_routing<TM>(p, mb, n);

            const int t0 = cs * s.tpi;
            const int t1 = (t0 + s.tpi) < s.n_ct ? (t0 + s.tpi) : s.n_ct;
            const int tpw = s.tpi / WN;
            const int wt0 = t0 + wave * tpw;
            int wnt = (wt0 + tpw < t1 ? wt0 + tpw : t1) - wt0;   // tiles of this wavefront, may be <= 0
            // w2 scales of the 128-column blocks this item touches
            const int blk0 = (t0 * 16) >> 7;
            const int nblk = (((t1 * 16) - 1) >> 7) - blk0 + 1;
            for (int i = tid; i < nblk; i += THREADS)
                s_ws[0][i] = p.w2_scale[((size_t)e * (K >> 7) + blk0 + i) * s.n_ib + ib];
            __syncthreads();

            v8i ba[TM];
            float tsc[TM];
            float *accp[TM];
            const uint8_t *aq_u = s.aq + (size_t)u * s.bm_pad * 128;
#pragma unroll
            for (int t = 0; t < TM; t++) {
                const v4i lo = ldg128_agent(aq_u + (t * 16 + n) * 128 + 16 * q);
                const v4i hi = ldg128_agent(aq_u + (t * 16 + n) * 128 + 64 + 16 * q);
                const int sa_bits = load_agent(reinterpret_cast<const int *>(&s.sa[(size_t)u * s.bm_pad + t * 16 + n]));
                drain_vmem();
                ba[t] = cat(lo, hi);
                tsc[t] = __builtin_bit_cast(float, sa_bits) * (p.topk_w[r.slot[t]] * p.scaling);
                accp[t] = p.acc + (size_t)r.tok[t] * K + 4 * q;
            }
            if (wnt > 0) {
                const uint8_t *gd[2];
#pragma unroll
                for (int i = 0; i < 2; i++)
                    gd[i] = p.w2 + ((size_t)e * K + (size_t)wt0 * 16 + 8 * i + ld_row) * I + ib * 128 + 16 * ld_chunk[i];
                const size_t tile_step = (size_t)16 * I;
                const int n_st = (wnt + DT - 1) / DT;
                constexpr int LPS = DT * 2;
                auto issue = [&](int slot, int st) {
                    uint8_t *dst = ring + slot * STAGE_BYTES;
#pragma unroll
                    for (int j = 0; j < DT; j++) {
                        int tile = st * DT + j;
                        tile = tile < wnt ? tile : wnt - 1;
#pragma unroll
                        for (int i = 0; i < 2; i++) dma16_nt(gd[i] + tile * tile_step, dst + j * 2048 + i * 1024);
                    }
                };
                auto compute = [&](int slot, int st) {
                    const uint8_t *src = ring + slot * STAGE_BYTES;
#pragma unroll
                    for (int j = 0; j < DT; j++) {
                        const int tile = st * DT + j;
                        if (tile < wnt) {
                            const v8i a = read_tile(src + j * 2048);
                            const int c0 = (wt0 + tile) << 4;
                            const float ws = s_ws[0][(c0 >> 7) - blk0];
#pragma unroll
                            for (int t = 0; t < TM; t++) {
                                const v4f d = mfma_fp8(a, ba[t]);
                                const float sc = tsc[t] * ws;
                                if (r.valid[t]) {
#pragma unroll
                                    for (int jj = 0; jj < 4; jj++) atomic_add_f32_agent(accp[t] + c0 + jj, d[jj] * sc);
                                }
                            }
                        }
                    }
                };
                pipeline<STAGES, LPS>(n_st, issue, compute);
            }
        }
        drain_vmem();
        __syncthreads();
        if (tid == 0) __hip_atomic_fetch_add(&s.ctl->down_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };

    auto fin_item = [&](int f) {
        if (tid == 0) spin_until_ge(&s.ctl->down_done, n_down, s.ctl);
        __syncthreads();
        const int n4 = (int)(((int64_t)p.M * K) >> 2);
        const int i = f * FIN_CHUNK + tid;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int idx = i + k * THREADS;
            if (idx < n4) {
                const v4i a_bits = ldg128_agent(reinterpret_cast<const v4f *>(p.acc) + idx);
                uint2 o = reinterpret_cast<uint2 *>(p.out)[idx];
                drain_vmem();
                const v4f a = __builtin_bit_cast(v4f, a_bits);
                const float o0 = __builtin_bit_cast(float, o.x << 16), o1 = __builtin_bit_cast(float, o.x & 0xffff0000u);
                const float o2 = __builtin_bit_cast(float, o.y << 16), o3 = __builtin_bit_cast(float, o.y & 0xffff0000u);
                o.x = pack_bf16x2(o0 + a[0], o1 + a[1]);
                o.y = pack_bf16x2(o2 + a[2], o3 + a[3]);
                reinterpret_cast<uint2 *>(p.out)[idx] = o;
                reinterpret_cast<v4f *>(p.acc)[idx] = (v4f){0.f, 0.f, 0.f, 0.f};
            }
        }
        // this item's share of the per-unit state: nothing reads it any more
        const int upf = (n_units + s.n_fin - 1) / s.n_fin;
        const int u0 = f * upf;
        const int u1 = (u0 + upf) < n_units ? (u0 + upf) : n_units;
        for (int u = u0 + tid; u < u1; u += THREADS) s.flag[u] = 0;
        if (u1 > u0) {
            const int aq16 = s.bm_pad * 8;   // 16-byte pieces of aq per unit
            v4i *aq = reinterpret_cast<v4i *>(s.aq + (size_t)u0 * s.bm_pad * 128);
            for (int i = tid; i < (u1 - u0) * aq16; i += THREADS) aq[i] = (v4i){0, 0, 0, 0};
            float *sa = s.sa + (size_t)u0 * s.bm_pad;
            for (int i = tid; i < (u1 - u0) * s.bm_pad; i += THREADS) sa[i] = 0.f;
        }
    };

    // ---- work queue ---------------------------------------------------------------------------------------
    if (tid == 0) s_bcast[0] = __hip_atomic_fetch_add(&s.ctl->head, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    int item = s_bcast[0];
    while (item < total) {
        int next = 0;
        if (tid == 0) next = __hip_atomic_fetch_add(&s.ctl->head, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (item < n_up)
            up_item(item);
        else if (item < n_up + n_down)
            down_item(item - n_up);
        else
            fin_item(item - n_up - n_down);
        __syncthreads();
        if (tid == 0) s_bcast[0] = next;
        __syncthreads();
        item = s_bcast[0];
    }
    if (tid == 0) {
        const int left = __hip_atomic_fetch_add(&s.ctl->done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left == (int)gridDim.x - 1) {
            store_agent(&s.ctl->head, 0);
            store_agent(&s.ctl->done, 0);
            store_agent(&s.ctl->down_done, 0);
        }
    }
}

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

struct Layout {
    size_t ctl, acc, arrive, flag, sa, aq, h, total;
    int units, bm_pad;
};

Layout make_layout(int M, int K, int N, int sorted_num, int block_m)
{
    Layout L;
    L.bm_pad = (block_m + 15) / 16 * 16;
    const size_t n_mb = ((size_t)sorted_num + block_m - 1) / block_m;
    L.units = (int)(n_mb * (N / 256));
    size_t off = 0;
    L.ctl = off; off = align_up(off + sizeof(StreamCtl));
    L.acc = off; off = align_up(off + (size_t)M * K * sizeof(float));
    L.arrive = off; off = align_up(off + (size_t)L.units * sizeof(int));
    L.flag = off; off = align_up(off + (size_t)L.units * sizeof(int));
    L.sa = off; off = align_up(off + (size_t)L.units * L.bm_pad * sizeof(float));
    L.aq = off; off = align_up(off + (size_t)L.units * L.bm_pad * 128);
    L.h = off; off = align_up(off + (size_t)L.units * L.bm_pad * 256 * sizeof(float));
    L.total = off;
    return L;
}

int env_int(const char *name, int dflt)
{
    const char *e = getenv(name);
    return e ? atoi(e) : dflt;
}

typedef void (*StreamFn)(const StreamPlan);

struct Variant {
    StreamFn fn;
    int lds_bytes;
    int threads;
};

template <int TM, int WN, int ST>
Variant variant()
{
    return Variant{moe_stream_kernel<TM, WN, ST>, 256 * 128 * ST, WN * 64};
}

template <int TM, int WN>
Variant pick_stages(int stages)
{
    switch (stages) {
    case 1: return variant<TM, WN, 1>();
    case 2: return variant<TM, WN, 2>();
    case 3: return variant<TM, WN, 3>();
    default: return variant<TM, WN, 4>();   // 4 x 32 KiB of ring is what 160 KiB of LDS holds
    }
}

Variant pick(int tm, int wn, int stages)
{
    if (tm == 1) return wn == 4 ? pick_stages<1, 4>(stages) : pick_stages<1, 8>(stages);
    return wn == 4 ? pick_stages<2, 4>(stages) : pick_stages<2, 8>(stages);
}

// Workgroups of this variant the current device keeps resident at once; the attribute and occupancy queries run
// once per (variant, device).
hipError_t resident_slots(const Variant &v, int *slots)
{
    struct Entry {
        StreamFn fn;
        int dev;
        int slots;
    };
    static std::mutex mu;
    static std::vector<Entry> cache;
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    std::lock_guard<std::mutex> lock(mu);
    for (const Entry &e : cache)
        if (e.fn == v.fn && e.dev == dev) {
            *slots = e.slots;
            return hipSuccess;
        }
    int cus = 0;
    err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess) return err;
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(v.fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                              v.lds_bytes);
    if (err != hipSuccess) return err;
    int occ = 0;
    err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, reinterpret_cast<const void *>(v.fn), v.threads,
                                                       v.lds_bytes);
    if (err != hipSuccess) return err;
    if (occ < 1) occ = 1;
    *slots = cus * occ;
    cache.push_back(Entry{v.fn, dev, *slots});
    return hipSuccess;
}

}  // namespace

bool stream_supported(int block_m) { return block_m <= 32; }

size_t stream_workspace_bytes(int M, int K, int N, int sorted_num, int block_m)
{
    return make_layout(M, K, N, sorted_num, block_m).total;
}

hipError_t launch_stream(const MoeParams &p, int warp_n, int stages, void *workspace, hipStream_t stream)
{
    const Layout L = make_layout(p.M, p.K, p.N, p.sorted_num, p.block_m);
    uint8_t *ws = static_cast<uint8_t *>(workspace);
    StreamPlan s;
    s.p = p;
    s.p.acc = reinterpret_cast<float *>(ws + L.acc);
    s.ctl = reinterpret_cast<StreamCtl *>(ws + L.ctl);
    s.arrive = reinterpret_cast<int *>(ws + L.arrive);
    s.flag = reinterpret_cast<int *>(ws + L.flag);
    s.sa = reinterpret_cast<float *>(ws + L.sa);
    s.aq = ws + L.aq;
    s.h = reinterpret_cast<float *>(ws + L.h);
    s.bm_pad = L.bm_pad;
    s.n_ib = p.N / 256;
    s.nkb = p.K / 128;
    s.n_ct = p.K / 16;
    s.n_mb_max = (p.sorted_num + p.block_m - 1) / p.block_m;

    const Variant v = pick((p.block_m + 15) / 16, warp_n, stages);

    int slots = 0;
    const hipError_t err = resident_slots(v, &slots);
    if (err != hipSuccess) return err;

    // Item sizes: aim at ~4 items per resident workgroup, between 64 KiB and 512 KiB of weights each.
    const int64_t rows = (int64_t)p.M * p.top_k;
    int64_t mb_est = (rows < p.E ? rows : p.E) + rows / p.block_m;
    if (mb_est > s.n_mb_max) mb_est = s.n_mb_max;
    const int64_t unit_bytes = (int64_t)256 * p.K + (int64_t)p.K * 128;
    int64_t target = mb_est * s.n_ib * unit_bytes / ((int64_t)slots * 4);
    if (target < (64 << 10)) target = 64 << 10;
    if (target > (512 << 10)) target = 512 << 10;
    int kbpi = (int)((target + (1 << 14)) / (1 << 15));   // 32 KiB of w1 per K block
    kbpi = env_int("ALPHA_MOE_KBPI", kbpi);
    if (kbpi < 1) kbpi = 1;
    if (kbpi > s.nkb) kbpi = s.nkb;
    s.ks = (s.nkb + kbpi - 1) / kbpi;
    s.kbpi = (s.nkb + s.ks - 1) / s.ks;                    // even split
    s.ks = (s.nkb + s.kbpi - 1) / s.kbpi;
    int tpi = (int)(target / (16 * 2048)) * 16;            // 2 KiB of w2 per tile, whole multiples of 16 tiles
    tpi = env_int("ALPHA_MOE_TPI", tpi);
    if (tpi < 16) tpi = 16;
    tpi = (tpi + 15) / 16 * 16;
    if (tpi > (s.n_ct + 15) / 16 * 16) tpi = (s.n_ct + 15) / 16 * 16;
    s.n_cs = (s.n_ct + tpi - 1) / tpi;
    s.tpi = ((s.n_ct + s.n_cs - 1) / s.n_cs + 15) / 16 * 16;   // even split, whole multiples of 16 tiles
    s.n_cs = (s.n_ct + s.tpi - 1) / s.tpi;
    const int64_t n4 = (int64_t)p.M * p.K / 4;
    s.n_fin = (int)((n4 + v.threads * 4 - 1) / (v.threads * 4));

    const int64_t max_items = (int64_t)L.units * (s.ks + s.n_cs) + s.n_fin;
    int grid = env_int("ALPHA_MOE_GRID", slots);
    if (grid > max_items) grid = (int)max_items;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL(v.fn, dim3((unsigned)grid), dim3((unsigned)v.threads), v.lds_bytes, stream, s);
    return hipGetLastError();
}

}  // namespace alpha_moe
