// Fused W8A8 MoE, "streaming" kernel for decode-sized batches (block_m <= 32): ONE persistent launch that moves
// every active expert's weights through the chip once at HBM speed.
//
// Why not one workgroup per (row block, 128-column slice) like the reference's CTA
// (fused_moe_w8a8_up_down_acc.cu:676-679,767)?  On MI355X one CU sustains ~45 GB/s of HBM reads, the chip ~6.9 TB/s,
// so a decode step (DeepSeek-V3 shard, M=1: 18 such units of 2.75 MB) must be cut into hundreds of pieces to
// engage all 256 CUs.  The 128-column requantisation group forces a dependency between the pieces, so the kernel
// is a small dataflow over a work queue (items are taken in queue order with one atomic):
//
//   UP item   (unit u = (row block mb, slice ib), K split ks): 256 interleaved w1 rows x kbpi K blocks.  With one
//             K split the gate/up sums stay in registers; otherwise the VALID tokens' partial sums are stored to
//             hpart[u][ks] and the item that arrives last at arrive[u] adds the slices up in a fixed order.  That
//             workgroup applies SwiGLU, quantises the block_m x 128 tile to FP8 (aq[u], sa[u]) and publishes
//             flag[u] = epoch.
//   DOWN item (row block mb, column slab cs): waits for the flags of all I/128 slices of mb, then contracts the
//             full intermediate against tpi 16-column tiles of w2[e] and stores each valid (token, slot) row's
//             fp32 result to y[slot] - every element of y has exactly one writer.  Bumps down_done.
//   FIN item  (token t, 1024 output columns): waits for down_done == number of DOWN items, then
//             out[t] = bf16(out[t] + sum over the token's live slots of y[slot]) - one rounding, fixed order.
//
// There is no floating-point atomic anywhere: the result is bit-reproducible from run to run.
//
// Every wait is on items EARLIER in the queue, and items never wait on later ones.  Every item, the first one of a
// workgroup too, comes from one counter: only running workgroups ever hold items, so the queue drains with any number
// of workgroups resident - launches may overlap on a device (several streams, other persistent kernels) without
// being able to starve each other.  (ALPHA_MOE_STRICT_QUEUE=0 hands the first gridDim.x items out by workgroup index
// instead, which saves the first round trip to the counter but is only correct when the whole grid is resident at
// once; it is an experiment switch, not a mode to serve with.)  Each spin is bounded and sets ctl->error instead of
// hanging; the items that write `out` then fill it with NaN, in that launch and in every later one on the workspace.
// The workspace starts zero-filled; its first kPrefixBytes hold the control block, the arrival counters (reset by the
// last arrival) and epoch-stamped flags, so nothing has to be cleared between launches; the rest (aq, sa, hpart, y)
// is only ever read after it was written in the same launch.
//
// Data movement: weights go HBM -> LDS with non-temporal global_load_lds_dwordx4 (measured on MI355X: 6.9 TB/s
// against 3.4 TB/s for the same loads without the non-temporal hint, and 5.5 TB/s for direct-to-VGPR loads in the
// MFMA lane order), into a per-wavefront ring of 2 KiB tiles (16 rows x 128 bytes), so the loops need no workgroup
// barrier.  Inside a tile, 16-byte chunk c of row m sits at position c ^ ((m >> 1) & 7): the MFMA operand read (16
// rows at a fixed chunk) then touches 16 distinct bank quads.  A tile is exactly two load instructions, so "tile j
// has landed" is "at most 2*(S-1) vector-memory operations outstanding" once the S-1 tiles behind it are issued;
// result stores issued in between only make that wait stricter, never wrong.
// Data that crosses workgroups inside the launch uses agent-scope (sc1) loads and stores: an L2-wide write-back /
// invalidate (__threadfence) per hand-over costs ~4x the whole kernel on this 8-XCD part.
#include <mutex>
#include <vector>

#include "moe_common.hpp"

namespace alpha_moe {
namespace {

constexpr int kItemKBlocks = 64;     // most K blocks one UP item covers
constexpr int kMaxIb = 16;           // most 128-column slices of the intermediate (I <= 2048)
constexpr int kFinCols = 1024;       // output columns per FIN item
constexpr int kMaxDynamicLds = 140 << 10;   // of the 160 KiB of a compute unit; the kernel's static tables take ~16 KiB

struct StreamPlan {
    MoeParams p;
    StreamCtl *ctl;
    int *arrive;     // [units]  K-split items that have delivered their partial sums
    int *flag;       // [units]  == epoch once aq/sa of the unit are published
    int *live;       // [slots]  == epoch once y[slot] is being written this launch
    float *sa;       // [units][bm_pad]              requantisation scale per token
    uint8_t *aq;     // [units][bm_pad][128]         requantised SwiGLU output, FP8
    float *hpart;    // [units][ks][bm_pad][2][128]  partial gate/up sums (K-split only)
    float *y;        // [slots][K]                   down-projection result per (token, slot) row
    int n_ib, nkb, n_ct, n_mb_max;
    int kbpi, ks;    // K blocks per UP item, UP items per unit
    int tpi, n_cs;   // 16-column tiles per DOWN item, DOWN items per row block
    int n_fc;        // 1024-column chunks per token
    int fin_w;       // chunks per FIN item (1 or 2)
    int lag;         // row blocks between a block's UP items and its DOWN items in the queue
    int bm_pad;
    int strict_queue;   // every item, the first one too, comes from the counter: correct with any number of resident workgroups
};

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

// TM: 16-token tiles per row block; WN: wavefronts per workgroup; S: 2 KiB tiles in each wavefront's LDS ring
template <int TM, int WN, int S>
__global__ __launch_bounds__(WN * 64) void moe_stream_kernel(const StreamPlan s)
{
    constexpr int RW = 256 / WN;            // w1 rows per wavefront
    constexpr int NP = RW / 32;             // gate/up MFMA pairs per wavefront per K block
    constexpr int NT = 2 * NP;              // 16x128 weight tiles per wavefront per K block
    constexpr int TPK = NT + TM;            // ring tiles per wavefront per K block (token tiles first)
    constexpr int THREADS = WN * 64;
    static_assert(S >= 2 && 2 * (S - 1) < 64, "ring depth must fit the 6-bit vmcnt");
    // Ring reuse is ordered, not padded: before a load is issued the wavefront waits for all of its own LDS reads
    // (wait_lds_reads() at the top of every step), so the tile a load overwrites has been read into registers whatever
    // the ring size.  The hazard this closes: a token tile's LDS read has no consumer until the K block's first matrix
    // instruction, so with S slots a fast load (the cached dummy line behind the end of an item) could land in the slot
    // while that read was still queued - seen as one wavefront's 16 intermediate columns wrong in ~1 of 30 short UP
    // items.  The ring still keeps one slot more than tiles in flight: a load then targets the tile read TWO steps ago.
    constexpr int R = S + 1;

    // dynamic LDS: [WN rings of S + 1 tiles][n_ib * TM tiles of requantised activations (DOWN items)]
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds_dyn[];
    __shared__ float s_sc[1024];                       // UP: gate scales [0,64), up scales [64,128); DOWN: w2 scales [blk][ib]
    __shared__ float s_xs[TM * 16][kItemKBlocks + 1];  // UP: activation scales [row][K block]; DOWN: sa [row][ib]
    __shared__ int s_tok[TM * 16];
    __shared__ float s_amax[WN][TM * 16];
    __shared__ int s_bcast[2];

    const MoeParams &p = s.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform, and the compiler should know it
    const int n = lane & 15;
    const int q = lane >> 4;
    const int K = p.K, I = p.N >> 1;
    uint8_t *ring = lds_dyn + wave * (R * 2048);
    uint8_t *s_aq = lds_dyn + WN * (R * 2048);

    // operand read offsets inside a 16x128 tile (see the swizzle note at the top of the file)
    const int f_n = (n >> 1) & 7;
    const int frag_lo = n * 128 + 16 * (q ^ f_n);
    const int frag_hi = n * 128 + 16 * ((q ^ f_n) ^ 4);
    // loader side: this lane fills position (row l/8 (+8 for the second instruction), chunk slot l%8) of a tile
    const int ld_row = lane >> 3;
    int ld_chunk[2];
#pragma unroll
    for (int i = 0; i < 2; i++) ld_chunk[i] = (lane & 7) ^ (((8 * i + ld_row) >> 1) & 7);

    int n_mb = (__builtin_amdgcn_readfirstlane(s.p.ntpp[0]) + p.block_m - 1) / p.block_m;
    n_mb = n_mb < s.n_mb_max ? n_mb : s.n_mb_max;
    const int n_units = n_mb * s.n_ib;
    const int n_up = n_units * s.ks;
    const int n_down = n_mb * s.n_cs;
    const int n_fin = (p.M * s.n_fc + s.fin_w - 1) / s.fin_w;
    const int total = n_up + n_down + n_fin;
    const int epoch = (int)((unsigned)__builtin_amdgcn_readfirstlane(s.ctl->epoch) + 1u);
    const uint8_t *dummy = p.x;   // where loads past the end of an item are pointed: always mapped, always cached

    auto read_tile = [&](const uint8_t *tile) -> v8i {
        return cat(*reinterpret_cast<const v4i *>(tile + frag_lo), *reinterpret_cast<const v4i *>(tile + frag_hi));
    };

    // The next item is taken from the queue when the current one has finished streaming (its atomic's round trip
    // hides behind the item's epilogue).  Taking it any earlier lets busy workgroups sit on items that idle ones
    // could already run.
    int next_item = -1;
    auto fetch_next = [&]() {
        // the first gridDim.x items are handed out by workgroup index, the counter hands out the rest
        if (tid == 0 && next_item < 0)
            next_item = (s.strict_queue ? 0 : (int)gridDim.x) +
                        __hip_atomic_fetch_add(&s.ctl->head, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
                stg32_agent(aq_u, (uint32_t)((t * 16 + n) * 128 + col), packed);
            }
            if (wave == 0 && q == 0)
                stg32_agent(s.sa + (size_t)u * s.bm_pad, (uint32_t)(t * 16 + n) * 4u, __builtin_bit_cast(uint32_t, s_a));
        }
        drain_vmem();
        __syncthreads();
        if (tid == 0) store_agent(&s.flag[u], epoch);
    };

    auto up_item = [&](int item) {
        const int u = item / s.ks;
        const int ksp = item - u * s.ks;
        const int mb = u / s.n_ib;
        const int ib = u - mb * s.n_ib;
        // the rows' slot ids do not depend on the expert id: their loads go out before the wait for it (one memory
        // round trip less at the head of every item)
        const Routing<TM> r = load_routing<TM>(p, mb, n);
        int row_id = -1;
        if (tid < TM * 16) {
            const int idx = mb * p.block_m + tid;
            if (tid < p.block_m && idx < p.sorted_num) row_id = p.sorted_ids[idx];
        }
        const int e = __builtin_amdgcn_readfirstlane(p.expert_ids[mb]);
        if (e < 0 || e >= p.E) return;
        const int kb0 = ksp * s.kbpi;
        const int nk = (s.nkb - kb0) < s.kbpi ? (s.nkb - kb0) : s.kbpi;

        // per-item tables in LDS: token of every row, the unit's gate (row 2*ib) / up (row 2*ib+1) weight scales and
        // the tokens' activation scales over the item's K range
        if (tid < TM * 16) {
            const int tk = row_id / p.top_k;
            s_tok[tid] = (row_id >= 0 && tk < p.M) ? tk : 0;
        }
        {
            const float *ws_rows = p.w_scale + ((size_t)e * (p.N >> 7) + 2 * ib) * s.nkb + kb0;
            for (int i = tid; i < 2 * nk; i += THREADS) {
                const int up = i >= nk;
                s_sc[up * kItemKBlocks + i - up * nk] = ws_rows[up * s.nkb + (i - up * nk)];
            }
        }
        __syncthreads();
        for (int i = tid; i < TM * 16 * nk; i += THREADS) {
            const int row = i / nk, k = i - row * nk;
            s_xs[row][k] = p.x_scale[(size_t)s_tok[row] * s.nkb + kb0 + k];
        }

        // loader-side row pointers: tile position (row 8i + l/8, chunk slot l%8) <- global (row, chunk slot ^ f(row))
        const uint8_t *ga[NT][2];
#pragma unroll
        for (int a = 0; a < NT; a++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                // weight tile a = (pair a/2, gate|up a%2): tile row 8i + l/8 is slab row pair*32 + 16i + l/8 (+8 for up)
                const int row = ib * 256 + wave * RW + (a >> 1) * 32 + 16 * i + ld_row + 8 * (a & 1);
                ga[a][i] = p.w + (size_t)e * p.N * K + row * p.w_rs + kb0 * p.w_ks + 16 * ld_chunk[i];
            }
        const uint8_t *gb[TM][2];
#pragma unroll
        for (int t = 0; t < TM; t++)
#pragma unroll
            for (int i = 0; i < 2; i++)
                gb[t][i] = p.x + (size_t)s_tok[t * 16 + 8 * i + ld_row] * K + (size_t)kb0 * 128 + 16 * ld_chunk[i];

        v4f accg[NP][TM], accu[NP][TM];
#pragma unroll
        for (int pr = 0; pr < NP; pr++)
#pragma unroll
            for (int t = 0; t < TM; t++) {
                accg[pr][t] = (v4f){0.f, 0.f, 0.f, 0.f};
                accu[pr][t] = (v4f){0.f, 0.f, 0.f, 0.f};
            }

        // Tile stream of this wavefront: K block kb contributes TPK tiles in the order [tokens t=0..TM-1, G0, U0, G1, ...].
        auto issue = [&](int kb, int a, int slot) {   // `a` is a compile-time constant after unrolling
            uint8_t *dst = ring + slot * 2048;
            const bool past_end = kb >= nk;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                if (a < TM)
                    dma16<0>(past_end ? dummy : gb[a < TM ? a : 0][i] + (size_t)kb * 128, dst + i * 1024);
                else
                    dma16<2>(past_end ? dummy : ga[a >= TM ? a - TM : 0][i] + kb * p.w_ks, dst + i * 1024);
            }
        };
        int slot_w = 0, slot_r = 0;
#pragma unroll
        for (int j = 0; j < S - 1; j++) {
            issue(j / TPK, j % TPK, slot_w);
            slot_w = slot_w + 1 == R ? 0 : slot_w + 1;
        }
        __syncthreads();   // s_xs is complete
        v8i bfrag[TM];
        for (int kb = 0; kb < nk; kb++) {
            float sg[TM], su[TM];
#pragma unroll
            for (int a = 0; a < TPK; a++) {
                // Every LDS read this wavefront has issued is complete before a new direct-to-LDS load may land: a
                // token tile's read has no consumer until the first matrix instruction of the K block, and nothing
                // else orders it against the load that re-targets its slot.
                wait_lds_reads();
                issue(kb + (a + S - 1) / TPK, (a + S - 1) % TPK, slot_w);
                slot_w = slot_w + 1 == R ? 0 : slot_w + 1;
                __builtin_amdgcn_sched_barrier(0);
                if (a == 0) {   // the K block's scales: read behind the step's load so that their latency hides there
                    const float wsg = s_sc[kb], wsu = s_sc[kItemKBlocks + kb];
#pragma unroll
                    for (int t = 0; t < TM; t++) {
                        const float xs = s_xs[t * 16 + n][kb];
                        sg[t] = wsg * xs;
                        su[t] = wsu * xs;
                    }
                }
                wait_vmcnt<2 * (S - 1)>();
                const v8i frag = read_tile(ring + slot_r * 2048);
                slot_r = slot_r + 1 == R ? 0 : slot_r + 1;
                if (a < TM) {
                    bfrag[a < TM ? a : 0] = frag;
                } else {
                    const int pr = (a - TM) >> 1;
#pragma unroll
                    for (int t = 0; t < TM; t++) {
                        if (((a - TM) & 1) == 0)
                            accg[pr < NP ? pr : 0][t] += mfma_fp8(frag, bfrag[t]) * sg[t];
                        else
                            accu[pr < NP ? pr : 0][t] += mfma_fp8(frag, bfrag[t]) * su[t];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        fetch_next();
        drain_vmem();

        if (s.ks > 1) {
            // K-split: store the valid tokens' partial sums to this item's slice; the last arrival adds the slices up
            const size_t slice = (size_t)s.bm_pad * 256;
            float *h_u = s.hpart + (size_t)u * s.ks * slice;
            const int my_off = n * 256 + wave * (RW / 2) + 4 * q;
#pragma unroll
            for (int t = 0; t < TM; t++) {
                if (!r.valid[t]) continue;
#pragma unroll
                for (int pr = 0; pr < NP; pr++) {
                    const uint32_t off = (uint32_t)(t * 16 * 256 + my_off + pr * 16) * 4u;
                    stg128_agent(h_u + ksp * slice, off, accg[pr][t]);
                    stg128_agent(h_u + ksp * slice, off + 512u, accu[pr][t]);
                }
            }
            drain_vmem();
            __syncthreads();
            if (tid == 0)
                s_bcast[1] = __hip_atomic_fetch_add(&s.arrive[u], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            if (s_bcast[1] != s.ks - 1) return;
            acquire_fence();   // the other splits' partial sums are read from here on, not before
            if (tid == 0) store_agent(&s.arrive[u], 0);
#pragma unroll
            for (int t = 0; t < TM; t++)
#pragma unroll
                for (int pr = 0; pr < NP; pr++) {
                    v4f g = {0.f, 0.f, 0.f, 0.f}, up = {0.f, 0.f, 0.f, 0.f};
                    if (r.valid[t]) {
                        const uint32_t off = (uint32_t)(t * 16 * 256 + my_off + pr * 16) * 4u;
                        // fixed order: the sum does not depend on arrival order.  Eight splits (16 loads) are in flight
                        // at a time: one memory round trip per batch, not per split.
                        for (int k0 = 0; k0 < s.ks; k0 += 8) {
                            v4i gk[8], uk[8];
#pragma unroll
                            for (int k = 0; k < 8; k++) {
                                const int kk = k0 + k < s.ks ? k0 + k : s.ks - 1;
                                gk[k] = ldg128_agent(h_u + kk * slice, off);
                                uk[k] = ldg128_agent(h_u + kk * slice, off + 512u);
                            }
#pragma unroll
                            for (int k = 0; k < 8; k++)
                                if (k0 + k < s.ks) {
                                    g += __builtin_bit_cast(v4f, gk[k]);
                                    up += __builtin_bit_cast(v4f, uk[k]);
                                }
                        }
                    }
                    accg[pr][t] = g;
                    accu[pr][t] = up;
                }
        }
        activate_and_publish(u, accg, accu);
    };

    // (DOWN items of two sizes - a block's last columns in quarter-size items queued behind everything else, so that
    // the phase ends on short items - were tried: the short items stream at half the rate of the long ones, a call got
    // 3 % slower at M = 64 and 10 % at M = 4.)
    auto down_item = [&](int item) {
        const int mb = item / s.n_cs;
        const int cs = item - mb * s.n_cs;
        const Routing<TM> r = load_routing<TM>(p, mb, n);   // in flight together with the expert id
        // so is every wavefront's own look at the flags of the block's slices (one lane each): a wavefront that has seen
        // them up may read what the UP items published without meeting the others first
        const int flag0 = lane < s.n_ib ? load_agent(&s.flag[mb * s.n_ib + lane]) : epoch;
        const int e = __builtin_amdgcn_readfirstlane(p.expert_ids[mb]);
        if (e >= 0 && e < p.E) {
            const int n_ib = s.n_ib;
            const int t0 = cs * s.tpi;
            const int t1 = (t0 + s.tpi) < s.n_ct ? (t0 + s.tpi) : s.n_ct;
            const int tpw = s.tpi / WN;
            const int wt0 = t0 + wave * tpw;
            const int wng = (wt0 + tpw < t1 ? wt0 + tpw : t1) - wt0;   // 16-column groups of this wavefront, may be <= 0
            const int wnt = wng > 0 ? wng * n_ib : 0;                  // ring tiles: group-major, slice-minor
            // weights first: they do not depend on the up phase
            const uint8_t *gd[2];
#pragma unroll
            for (int i = 0; i < 2; i++)
                gd[i] = p.w2 + (size_t)e * K * I + ((wng > 0 ? wt0 : 0) * 16 + 8 * i + ld_row) * p.w2_rs + 16 * ld_chunk[i];
            const size_t group_step = 16 * p.w2_rs;
            int ig = 0, iib = 0;   // (group, slice) of the next tile to issue
            auto issue = [&](int slot) {
                uint8_t *dst = ring + slot * 2048;
                const bool past_end = ig >= wng;
#pragma unroll
                for (int i = 0; i < 2; i++)
                    dma16<2>(past_end ? dummy : gd[i] + ig * group_step + iib * p.w2_ks, dst + i * 1024);
                iib++;
                if (iib == n_ib) {
                    iib = 0;
                    ig++;
                }
            };
            int slot_w = 0, slot_r = 0;
            auto prime = [&]() {
#pragma unroll
                for (int j = 0; j < S - 1; j++) {
                    issue(slot_w);
                    slot_w = slot_w + 1 == S ? 0 : slot_w + 1;
                }
            };
            // Everything the item needs goes out before anything is waited for: the w2 scales of the 128-column blocks
            // the item touches (s_sc[blk * n_ib + ib], at most four per thread), the ring's first tiles, and - once
            // this wavefront has seen the flags up - the requantised activations and their scales.
            const int blk0 = (t0 * 16) >> 7;
            const int nblk = (((t1 * 16) - 1) >> 7) - blk0 + 1;
            const float *w2s = p.w2_scale + ((size_t)e * (K >> 7) + blk0) * n_ib;
            float sc_reg[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int i = tid + k * THREADS;
                sc_reg[k] = i < nblk * n_ib ? w2s[i] : 0.f;
            }
            prime();
            // rare (a DOWN item is queued long after the UP items it needs): a poll returns behind the ring's loads
            if (!__all(reached(flag0, epoch))) spin_all_ge(&s.flag[mb * n_ib], n_ib, epoch, s.ctl, &s.ctl->down_done);

            // requantised activations of all slices -> LDS as operand tiles, their scales -> s_xs[row][ib]
            for (int i = wave; i < n_ib * TM; i += WN) {
                const int ib = i / TM, t = i - ib * TM;
                const uint8_t *src = s.aq + ((size_t)(mb * n_ib + ib) * s.bm_pad + t * 16) * 128;
#pragma unroll
                for (int k = 0; k < 2; k++)
                    dma16<16>(src + (8 * k + ld_row) * 128 + 16 * ld_chunk[k], s_aq + i * 2048 + k * 1024);
            }
            static_assert(kMaxIb * TM * 16 <= 2 * THREADS, "at most two activation scales per thread");
            int sa_bits[2] = {0, 0};
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int i = tid + k * THREADS;
                const int ib = i / (TM * 16), row = i - ib * (TM * 16);
                if (i < n_ib * TM * 16)
                    sa_bits[k] = load_agent(reinterpret_cast<const int *>(&s.sa[(size_t)(mb * n_ib + ib) * s.bm_pad + row]));
            }
            float tw[TM];
            uint32_t yoff[TM];   // byte offset of this lane's 4 columns in the slot's row of y (rows * K * 4 <= 2^30)
#pragma unroll
            for (int t = 0; t < TM; t++) {
                tw[t] = r.valid[t] ? p.topk_w[r.slot[t]] * p.scaling : 0.f;
                yoff[t] = ((uint32_t)r.slot[t] * (uint32_t)K + 4u * q) * 4u;
                if (cs == 0 && wave == 0 && q == 0 && r.valid[t]) store_agent(&s.live[r.slot[t]], epoch);
            }
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int i = tid + k * THREADS;
                if (i < nblk * n_ib) s_sc[i] = sc_reg[k];
            }
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int i = tid + k * THREADS;
                const int ib = i / (TM * 16), row = i - ib * (TM * 16);
                if (i < n_ib * TM * 16) s_xs[row][ib] = __builtin_bit_cast(float, sa_bits[k]);
            }
            // everything issued so far (the ring's first S-1 tiles, the activation tiles) has landed
            drain_vmem();
            __syncthreads();

            // Result rows are kept in registers and stored NG column groups at a time, normally once, behind the
            // item's last tile: the wait counter that tells a wavefront that a ring tile has landed counts stores as
            // well, in issue order, so a store between the loads holds every later tile back until it is acknowledged
            // by memory (measured on the DeepSeek-V3 shard at M = 64: 234 -> 215 us per call with the stores taken out).
            constexpr int NG = 16 / TM;
            for (int g0 = 0; g0 < wng; g0 += NG) {
                v4f res[NG][TM];
#pragma unroll
                for (int gg = 0; gg < NG; gg++) {
                    if (g0 + gg < wng) {   // wavefront-uniform
                        const int c0 = (wt0 + g0 + gg) << 4;
                        v4f d[TM];
#pragma unroll
                        for (int t = 0; t < TM; t++) d[t] = (v4f){0.f, 0.f, 0.f, 0.f};
                        for (int cib = 0; cib < n_ib; cib++) {
                            issue(slot_w);
                            slot_w = slot_w + 1 == S ? 0 : slot_w + 1;
                            __builtin_amdgcn_sched_barrier(0);
                            wait_vmcnt<2 * (S - 1)>();
                            const v8i a = read_tile(ring + slot_r * 2048);
                            slot_r = slot_r + 1 == S ? 0 : slot_r + 1;
                            const float ws = s_sc[((c0 >> 7) - blk0) * n_ib + cib];
#pragma unroll
                            for (int t = 0; t < TM; t++) {
                                const v8i b = read_tile(s_aq + (cib * TM + t) * 2048);
                                d[t] += mfma_fp8(a, b) * (s_xs[t * 16 + n][cib] * ws);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
#pragma unroll
                        for (int t = 0; t < TM; t++) res[gg][t] = d[t] * tw[t];
                    }
                }
#pragma unroll
                for (int gg = 0; gg < NG; gg++)
                    if (g0 + gg < wng) {
#pragma unroll
                        for (int t = 0; t < TM; t++)
                            if (r.valid[t]) stg128_agent(s.y, yoff[t] + ((uint32_t)(wt0 + g0 + gg) << 6), res[gg][t]);
                    }
            }
        }
        // (Asking for the next item when the last tile is issued, and counting the item only behind the next item's
        // prologue instead of waiting for its rows here, were both tried: 1 - 3 % slower at M = 16 and 64.)
        fetch_next();
        drain_vmem();
        __syncthreads();
        if (tid == 0) __hip_atomic_fetch_add(&s.ctl->down_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };

    // FIN item: two dependent round trips.  (1) Wavefront 0 polls the DOWN counter; an expired wait anywhere in this
    // launch has set kExpiredBit in that very counter, and lane 1 reads the sticky error word of earlier launches
    // with the same instruction.  (2) The stamps of the token's slots, the rows of ALL its slots and the prior output
    // go out together; rows of slots that are not live this launch are dropped after the fact (they are stale bytes of
    // this workspace, nothing else).
    auto fin_item = [&](int f) {
        if (wave == 0) {
            int v = 0;
            bool up = false;
            for (int it = 0; it < (1 << 22) && !up; it++) {
                v = load_agent(lane == 1 ? &s.ctl->error : &s.ctl->down_done);
                up = reached(__builtin_amdgcn_readlane(v, 0), n_down);
                if (!up) {
                    if (it < 16) __builtin_amdgcn_s_sleep(4);
                    else __builtin_amdgcn_s_sleep(32);
                }
            }
            if (lane == 0) {
                if (!up) store_agent(&s.ctl->error, 1);
                // a result row may be missing: the output says so itself, NaN in every element
                s_bcast[1] = !up || __builtin_amdgcn_readlane(v, 1) != 0 || (__builtin_amdgcn_readlane(v, 0) & kExpiredBit) != 0;
            }
        }
        __syncthreads();
        acquire_fence();   // the result rows are read from here on, not before the DOWN counter was seen up
        // an item sums fin_w (1 or 2) chunks of 1024 columns: with more chunks than workgroups, two per item halve the
        // rounds of dependent memory round trips that close the call
        const bool poisoned = s_bcast[1] != 0;
        const int n_chunks = p.M * s.n_fc;
        int tk[2], col[2], stamp[2];
        bool mine[2];
        uint2 *op[2];
        uint2 o[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int ch = f * s.fin_w + j;
            const bool on = j < s.fin_w && ch < n_chunks;
            tk[j] = on ? ch / s.n_fc : 0;
            col[j] = (on ? ch - tk[j] * s.n_fc : 0) * kFinCols + tid * 4;
            mine[j] = on && tid < kFinCols / 4 && col[j] < K;
            // lane k fetches the stamp of the token's slot k (top_k <= 64)
            stamp[j] = load_agent(&s.live[tk[j] * p.top_k + (lane < p.top_k ? lane : 0)]);
            op[j] = reinterpret_cast<uint2 *>(p.out + (size_t)tk[j] * K + (mine[j] ? col[j] : 0));
            o[j] = make_uint2(0u, 0u);
            if (mine[j] && !p.overwrite && !poisoned) o[j] = *op[j];
        }
        v4f sum[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        // slot order: the sum depends on nothing but the inputs.  Sixteen rows per chunk are in flight at a time.
        for (int s0 = 0; s0 < p.top_k; s0 += 16) {
            v4i lo[2][8], hi[2][8];
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    lo[j][k] = (v4i){0, 0, 0, 0};
                    hi[j][k] = (v4i){0, 0, 0, 0};
                    const uint32_t row = ((uint32_t)(tk[j] * p.top_k + s0 + k) * (uint32_t)K + (uint32_t)col[j]) * 4u;
                    if (mine[j] && s0 + k < p.top_k) lo[j][k] = ldg128_agent(s.y, row);
                    if (mine[j] && s0 + 8 + k < p.top_k) hi[j][k] = ldg128_agent(s.y, row + 32u * (uint32_t)K);
                }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const unsigned long long live_mask = __ballot(lane < p.top_k && stamp[j] == epoch) >> s0;
#pragma unroll
                for (int k = 0; k < 8; k++)
                    if ((live_mask >> k) & 1) sum[j] += __builtin_bit_cast(v4f, lo[j][k]);
#pragma unroll
                for (int k = 0; k < 8; k++)
                    if ((live_mask >> (8 + k)) & 1) sum[j] += __builtin_bit_cast(v4f, hi[j][k]);
            }
        }
#pragma unroll
        for (int j = 0; j < 2; j++)
            if (mine[j]) {
                uint2 r = o[j];
                if (poisoned) {
                    r = make_uint2(0x7fc07fc0u, 0x7fc07fc0u);
                } else {
                    const float o0 = __builtin_bit_cast(float, r.x << 16), o1 = __builtin_bit_cast(float, r.x & 0xffff0000u);
                    const float o2 = __builtin_bit_cast(float, r.y << 16), o3 = __builtin_bit_cast(float, r.y & 0xffff0000u);
                    r.x = pack_bf16x2(o0 + sum[j][0], o1 + sum[j][1]);
                    r.y = pack_bf16x2(o2 + sum[j][2], o3 + sum[j][3]);
                }
                *op[j] = r;
            }
    };

    // ---- work queue ---------------------------------------------------------------------------------------
    // Order: round r holds the UP items of row block r followed by the DOWN items of row block r - lag, so the two
    // kinds overlap, a DOWN item is taken long after the UP items it waits for, and only `lag` blocks' worth of
    // DOWN items remain when the UP items run out.  FIN items come last.
    const int per_up = s.n_ib * s.ks, per_down = s.n_cs;
    const int lag = s.lag < n_mb ? s.lag : n_mb;
    const int head_items = lag * per_up;                          // rounds 0 .. lag-1: UP only
    const int mid_items = (n_mb - lag) * (per_up + per_down);     // rounds lag .. n_mb-1: UP then DOWN
    // every item kind has exactly one call site: the compiler inlines the item bodies into the loop
    auto run_item = [&](int item) {
        int up = -1, down = -1, fin = -1;
        if (item >= n_up + n_down) {
            fin = item - n_up - n_down;
        } else if (item < head_items) {
            up = item;
        } else if (item < head_items + mid_items) {
            const int i = item - head_items;
            const int round = i / (per_up + per_down);
            const int off = i - round * (per_up + per_down);
            if (off < per_up)
                up = (lag + round) * per_up + off;
            else
                down = round * per_down + (off - per_up);
        } else {
            down = (n_mb - lag) * per_down + (item - head_items - mid_items);
        }
        if (up >= 0) up_item(up);
        else if (down >= 0) down_item(down);
        else fin_item(fin);
        return up >= 0 ? 1 : down >= 0 ? 2 : 3;
    };
    int item = blockIdx.x;   // no round trip to the queue before the first item
    if (s.strict_queue) {    // unless the caller cannot promise that the whole grid is resident at once
        fetch_next();
        if (tid == 0) s_bcast[0] = next_item;
        __syncthreads();
        item = __builtin_amdgcn_readfirstlane(s_bcast[0]);
        __syncthreads();
    }
    while (item < total) {
        next_item = -1;
        const int kind = run_item(item);
        (void)kind;
        fetch_next();   // paths that did not get there themselves (skipped blocks, FIN items)
        __syncthreads();
        if (tid == 0) s_bcast[0] = next_item;
        __syncthreads();
        item = __builtin_amdgcn_readfirstlane(s_bcast[0]);
    }
    if (tid == 0) {
        const int left = __hip_atomic_fetch_add(&s.ctl->done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left == (int)gridDim.x - 1) {
            store_agent(&s.ctl->head, 0);
            store_agent(&s.ctl->done, 0);
            store_agent(&s.ctl->down_done, 0);
            store_agent(&s.ctl->epoch, epoch);
        }
    }
}

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

// Everything the host decides about one launch; a pure function of the sizes (and of the tuning overrides), so the
// workspace query and the launch agree.
struct HostPlan {
    bool ok;
    int bm_pad, n_ib, nkb, n_ct, n_mb_max, units;
    int kbpi, ks, tpi, n_cs, n_fc, fin_w, lag;
    size_t off_sa, off_aq, off_hpart, off_y, total;
};

// Compute units of the current device (256 on MI355X); read once.
int compute_units()
{
    static const int n = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            return 256;
        return cus;
    }();
    return n;
}

HostPlan make_plan(int top_k, int M, int K, int N, int E, int sorted_num, int block_m)
{
    HostPlan h = {};
    h.bm_pad = (block_m + 15) / 16 * 16;
    h.n_ib = N / 256;
    h.nkb = K / 128;
    h.n_ct = K / 16;
    const int64_t rows = (int64_t)M * top_k;
    // a live row block holds at least one (token, slot) row, so there are at most M*top_k of them
    int64_t n_mb_max = ((int64_t)sorted_num + block_m - 1) / block_m;
    if (n_mb_max > rows) n_mb_max = rows;
    h.n_mb_max = (int)n_mb_max;
    const int64_t units = n_mb_max * h.n_ib;
    h.ok = block_m <= 32 && top_k <= 64 && h.n_ib <= kMaxIb && units <= kMaxUnits && rows <= kMaxSlots &&
           rows * (int64_t)K * 4 <= ((int64_t)1 << 30);
    if (!h.ok) return h;
    h.units = (int)units;

    // Item sizes (from sweeps on MI355X, DeepSeek-V3 shard, M = 1..64).  UP: whole K per item once there are about as
    // many (row block, slice) units as compute units - no partial sums, no arrival counter - and otherwise K split so
    // that the UP items about fill the chip once; items below ~128 KiB of w1 drown in their fixed cost (a dozen
    // dependent memory round trips).  DOWN: items of 256 KiB of w2, 128 KiB when there would be too few of them.
    const int cus = compute_units();
    int64_t mb_est = (rows < E ? rows : E) + rows / block_m;
    if (mb_est > n_mb_max) mb_est = n_mb_max;
    const int64_t units_est = mb_est * h.n_ib;
    int ks_want = (int)((cus + units_est - 1) / units_est);
    if (ks_want < 1) ks_want = 1;
    int kbpi = (h.nkb + ks_want - 1) / ks_want;
    if (kbpi < 4) kbpi = 4;
    kbpi = tunable(kTunKbpi, kbpi);
    if (kbpi < 1) kbpi = 1;
    if (kbpi > h.nkb) kbpi = h.nkb;
    if (kbpi > kItemKBlocks) kbpi = kItemKBlocks;
    h.ks = (h.nkb + kbpi - 1) / kbpi;
    h.kbpi = (h.nkb + h.ks - 1) / h.ks;                    // even split
    h.ks = (h.nkb + h.kbpi - 1) / h.kbpi;
    // a DOWN item reads all n_ib slices of its columns: 2 KiB * n_ib per 16-column tile
    int64_t down_target = 256 << 10;
    if (mb_est * ((h.n_ct * 2048 * h.n_ib + down_target - 1) / down_target) < cus / 2) down_target = 128 << 10;
    // small experts, about a row block per compute unit: one DOWN item per block (Qwen3-Next shard, M = 32: -7 %)
    if ((int64_t)h.n_ct * 2048 * h.n_ib <= (512 << 10) && mb_est * 4 >= cus * 3) down_target = 512 << 10;
    int tpi = (int)(down_target / (2048 * h.n_ib)) / 16 * 16;
    tpi = tunable(kTunTpi, tpi);
    if (tpi < 16) tpi = 16;
    tpi = (tpi + 15) / 16 * 16;
    if (tpi > (h.n_ct + 15) / 16 * 16) tpi = (h.n_ct + 15) / 16 * 16;
    if (tpi / 8 * h.n_ib > 1024) tpi = 1024 / h.n_ib * 8 / 16 * 16;   // w2 scales of one item fit s_sc
    h.n_cs = (h.n_ct + tpi - 1) / tpi;
    h.tpi = ((h.n_ct + h.n_cs - 1) / h.n_cs + 15) / 16 * 16;   // even split, whole multiples of 16 tiles
    h.n_cs = (h.n_ct + h.tpi - 1) / h.tpi;
    h.n_fc = (K + kFinCols - 1) / kFinCols;
    h.fin_w = (int64_t)M * h.n_fc > cus ? 2 : 1;
    // how many row blocks later a block's DOWN items enter the queue than its UP items
    // (measured: overlapping the two kinds lowers the total rate - DOWN items stream less efficiently than UP items -
    // so by default the lag is "all blocks", i.e. UP items first, then DOWN items)
    h.lag = tunable(kTunLag, 1 << 30);
    if (h.lag < 1) h.lag = 1;

    size_t off = align_up(kPrefixBytes);
    h.off_sa = off; off = align_up(off + (size_t)h.units * h.bm_pad * sizeof(float));
    h.off_aq = off; off = align_up(off + (size_t)h.units * h.bm_pad * 128);
    h.off_hpart = off; off = align_up(off + (h.ks > 1 ? (size_t)h.units * h.ks * h.bm_pad * 256 * sizeof(float) : 0));
    h.off_y = off; off = align_up(off + (size_t)rows * K * sizeof(float));
    h.total = off;
    return h;
}

typedef void (*StreamFn)(const StreamPlan);

struct Variant {
    StreamFn fn;
    int ring_bytes;
    int threads;
    int tm;
};

template <int TM, int WN, int S>
Variant variant()
{
    return Variant{moe_stream_kernel<TM, WN, S>, WN * (S + 1) * 2048, WN * 64, TM};
}

// `stages` sizes the LDS ring: 16 KiB per workgroup per stage, i.e. S = 8 * stages / WN tiles of 2 KiB per
// wavefront (at least 2).  Up to 4 stages, two workgroups share a CU's 160 KiB of LDS.
template <int TM>
Variant pick_ring(int wn, int stages)
{
    int tiles = 8 * stages / wn;
    if (tiles < 2) tiles = 2;
    if (wn == 4) {
        switch (tiles) {
        case 2: return variant<TM, 4, 2>();
        case 4: return variant<TM, 4, 4>();
        case 6: return variant<TM, 4, 6>();
        case 8: return variant<TM, 4, 8>();
        default: return variant<TM, 4, 10>();
        }
    }
    switch (tiles) {
    case 2: return variant<TM, 8, 2>();
    case 3: return variant<TM, 8, 3>();
    case 4: return variant<TM, 8, 4>();
    default: return variant<TM, 8, 5>();
    }
}

Variant pick(int tm, int wn, int stages) { return tm == 1 ? pick_ring<1>(wn, stages) : pick_ring<2>(wn, stages); }

// Workgroups of this variant the current device keeps resident at once; the attribute and occupancy queries run
// once per (variant, LDS size, device).
hipError_t resident_slots(const Variant &v, int lds_bytes, int *slots)
{
    struct Entry {
        StreamFn fn;
        int dev, lds, slots;
    };
    static std::mutex mu;
    static std::vector<Entry> cache;
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    std::lock_guard<std::mutex> lock(mu);
    for (const Entry &e : cache)
        if (e.fn == v.fn && e.dev == dev && e.lds == lds_bytes) {
            *slots = e.slots;
            return hipSuccess;
        }
    int cus = 0;
    err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess) return err;
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(v.fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                              kMaxDynamicLds);
    if (err != hipSuccess) return err;
    int occ = 0;
    err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, reinterpret_cast<const void *>(v.fn), v.threads,
                                                       lds_bytes);
    if (err != hipSuccess) return err;
    // The runtime's answer divides the CU's LDS by the byte count; the hardware hands LDS out in granules (1280 bytes
    // on gfx950), so three workgroups of 54 272 bytes each do NOT fit the 160 KiB although 3 * 54 272 < 163 840.  A grid
    // one workgroup per CU too large is fatal here: the workgroups that are not resident own their first items (see
    // the kernel's item loop) and the resident ones end up waiting for them.  Round up to both granules in use on
    // CDNA parts and take the smaller count.
    hipFuncAttributes attr;
    err = hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(v.fn));
    if (err != hipSuccess) return err;
    const size_t need = attr.sharedSizeBytes + (size_t)lds_bytes;
    const size_t g1 = (need + 1279) / 1280 * 1280, g2 = (need + 2047) / 2048 * 2048;
    const int occ_lds = (int)(((size_t)160 << 10) / (g1 > g2 ? g1 : g2));
    if (occ > occ_lds) occ = occ_lds;
    if (occ < 1) occ = 1;
    *slots = cus * occ;
    cache.push_back(Entry{v.fn, dev, lds_bytes, *slots});
    return hipSuccess;
}

}  // namespace

size_t stream_prefix_bytes() { return align_up(kPrefixBytes); }

bool stream_supported(int top_k, int M, int K, int N, int E, int sorted_num, int block_m)
{
    return make_plan(top_k, M, K, N, E, sorted_num, block_m).ok;
}

size_t stream_workspace_bytes(int top_k, int M, int K, int N, int E, int sorted_num, int block_m)
{
    return make_plan(top_k, M, K, N, E, sorted_num, block_m).total;
}

hipError_t launch_stream(const MoeParams &p, int warp_n, int stages, void *workspace, hipStream_t stream)
{
    const HostPlan h = make_plan(p.top_k, p.M, p.K, p.N, p.E, p.sorted_num, p.block_m);
    if (!h.ok) return hipErrorInvalidValue;
    uint8_t *ws = static_cast<uint8_t *>(workspace);
    StreamPlan s;
    s.p = p;
    s.ctl = reinterpret_cast<StreamCtl *>(ws);
    s.arrive = reinterpret_cast<int *>(ws + kOffArrive);
    s.flag = reinterpret_cast<int *>(ws + kOffFlag);
    s.live = reinterpret_cast<int *>(ws + kOffLive);
    s.sa = reinterpret_cast<float *>(ws + h.off_sa);
    s.aq = ws + h.off_aq;
    s.hpart = reinterpret_cast<float *>(ws + h.off_hpart);
    s.y = reinterpret_cast<float *>(ws + h.off_y);
    s.bm_pad = h.bm_pad;
    s.n_ib = h.n_ib;
    s.nkb = h.nkb;
    s.n_ct = h.n_ct;
    s.n_mb_max = h.n_mb_max;
    s.kbpi = h.kbpi;
    s.ks = h.ks;
    s.tpi = h.tpi;
    s.n_cs = h.n_cs;
    s.n_fc = h.n_fc;
    s.fin_w = h.fin_w;
    s.lag = h.lag;
    s.strict_queue = tunable(kTunStrictQueue, 1) != 0;

    // `stages` asks for a ring depth; what LDS holds next to the item tables decides.  The shallowest ring always fits.
    const int tm = (p.block_m + 15) / 16;
    const int tail_bytes = h.n_ib * tm * 2048;   // DOWN items: the requantised tiles of all slices
    Variant v = pick(tm, warp_n, stages);
    int lds_bytes = v.ring_bytes + tail_bytes;
    while (lds_bytes > kMaxDynamicLds && stages > 1) {
        stages--;
        v = pick(tm, warp_n, stages);
        lds_bytes = v.ring_bytes + tail_bytes;
    }
    if (lds_bytes > kMaxDynamicLds) return hipErrorInvalidValue;
    int slots = 0;
    const hipError_t err = resident_slots(v, lds_bytes, &slots);
    if (err != hipSuccess) return err;

    const int64_t max_items = (int64_t)h.units * h.ks + (int64_t)h.n_mb_max * h.n_cs + (int64_t)p.M * h.n_fc;
    int grid = tunable(kTunGrid, slots);
    if (grid > max_items) grid = (int)max_items;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL(v.fn, dim3((unsigned)grid), dim3((unsigned)v.threads), lds_bytes, stream, s);
    return hipGetLastError();
}

}  // namespace alpha_moe
