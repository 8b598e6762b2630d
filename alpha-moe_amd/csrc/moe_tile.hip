// Fused W8A8 MoE, "tile" kernel for large batches: persistent workgroups of 8 wavefronts (two per SIMD, one workgroup
// per compute unit) that take work items from eight queues.  A row block of block_m sorted rows is I/128 UP items (one
// 128-column slice of the intermediate each) and a few DOWN items (a slab of output columns each).
//
// UP item.  The workgroup contracts the slice's 256 interleaved w1 rows against the block's tokens over all of K, one
// 128-byte K block per step.  Every operand reaches the matrix cores through LDS, filled by direct-to-LDS loads that
// cover whole 128-byte lines: measured on MI355X, a compute unit takes ~38 GB/s from L2 when a load instruction touches
// 16 rows x 64 bytes (the matrix-operand register layout) and ~100 GB/s when it touches 8 rows x 128 bytes, and at full
// matrix rate a 128-token block needs ~110 GB/s.  Wavefront (w, g) multiplies weight rows 64 w .. 64 w + 63 (4 operand
// tiles) with token half g; the two wavefronts of a pair w share a 3-stage ring of weight tiles and each loads half of
// it; the token tiles (16 tokens x 128 bytes, gathered through the routing) and their scales go through a 3-stage ring
// shared by everybody, one tile per wavefront, with one workgroup barrier per step.  A wavefront issues 4 x TH matrix
// instructions per step; the 4 multiply-adds that scale a 16x16 product into the fp32 accumulators are placed right
// behind the NEXT matrix instruction so that vector and matrix pipes overlap (75% of the FP8 peak for this loop in
// isolation against 35% when the compiler orders it), and the step's loads are spread between them: a direct-to-LDS
// load blocks the issuing wavefront for 30-60 ns, during which the SIMD's other wavefront computes.
// SwiGLU and the FP8 requantisation of the 128-column group happen in registers (cross-wavefront amax through LDS);
// the block_m x 128 FP8 tile goes to a scratch area of the workspace in operand-tile layout, its per-token scales
// beside it, and the unit's flag is stamped with the launch epoch.
//
// DOWN item.  Waits for the flags of the block's slices, fetches their tiles and scales into LDS (where the token ring
// was) and contracts them with w2: 64 output columns at a time (4 operand tiles of w2 rows through the pair's ring),
// all slices, the wavefront's token half.  The w2 rows of a tile are picked so that a lane ends up with 16 adjacent
// output columns of its token: each valid (token, slot) row is written ONCE, in bf16, as whole 128-byte lines, to
// y[slot]: top_k result rows per token instead of the top_k * I/128 partial rows the reference's decomposition
// (fused_moe_w8a8_up_down_acc.cu:676-679,1085-1091) adds into the output.  A second kernel sums a token's live rows
// in fp32 and rounds into `out` once.  No atomics: at M = 8192 fp32 atomics alone cost 13 ms on MI355X.
//
// What bounds it (measured on the DeepSeek-V3 shard): a compute unit keeps about 32 KiB of L2 misses in flight whatever
// the ring depth (two or three stages, one or four wavefronts issuing: same rate), so alone it streams ~37 GB/s and a
// step takes ~1.5 us against 0.43 us of matrix time; 256 of them together reach what HBM and the fabric deliver.
// Everything therefore hinges on keeping all compute units busy and on the bytes they pull: items instead of whole row
// blocks (one workgroup per block left 16 of 272 blocks at M = 1024 to a second round: 547 us, now 391 us), the
// blocks of one expert next to each other on one XCD so that they share its L2, and non-temporal loads for the
// weights of experts that have a single block.
#include <mutex>
#include <type_traits>

#include "moe_common.hpp"

namespace alpha_moe {
namespace {

constexpr int kTileMaxIb = 8;        // most 128-column slices of the intermediate (I <= 1024)
constexpr int kTileMaxKb = 128;      // most 128-byte K blocks (K <= 16384)
constexpr int kTileMaxW2s = 512;     // most w2 block scales of one expert, (K/128) * (I/128)
constexpr int kStages = 3;
constexpr int kARingBytes = 4 * kStages * 8192;   // 4 wavefronts x 3 stages x 4 tiles of 2 KiB
constexpr int kMaxTailBytes = 48 << 10;           // token-tile ring / requantised tiles next to the weight rings

struct TileParams {
    MoeParams p;
    StreamCtl *ctl;
    int *flag;        // [row blocks][n_ib] == epoch once the unit's requantised tiles are in scratch
    int *live;        // [slots] == epoch once y[slot] is written this launch
    uint16_t *y;      // [slots][K] bf16
    uint8_t *aqs;     // [row blocks][n_ib][TM] requantised operand tiles of 2 KiB
    float *sas;       // [row blocks][n_ib][TM * 16] their per-token scales
    int n_ib, nkb, n_mb_max;
    int gps, n_cs;    // 64-column groups per DOWN item, column slabs per row block
    int nh;           // token parts per column slab (a DOWN item is one part of one slab)
    int lag;          // row blocks whose up/gate items precede the first down items of a queue
    int w_nt;         // weights with non-temporal loads: 1 always, 0 never, -1 for experts with a single row block
    int xs_chunk;     // 1: a token's activation scales are fetched four K steps at a time (K / 128 a multiple of 4,
                      // x_scale 16-byte aligned), 0: one step at a time
};

// One step of a wavefront: 4 weight tiles x TH token tiles, all from LDS.  acc[k][t] += (A_k x B_t) * row[t] * sc[k & 1]
// with row[] a per-token factor in LDS (16 floats per tile, already offset to this lane's token).  The product of
// (k, t) is scaled into its accumulator behind the matrix instruction of (k, t + 1).
// The step's NOPS direct-to-LDS loads (issue(i), i < NOPS) are spread evenly between the 4 TH matrix instructions: a
// load instruction blocks its wavefront for 30-60 ns (measured), and the other wavefront of the SIMD computes then.
// The factor of token tile t is row[t * row_stride].
template <int TH, int NOPS, typename Issue>
__device__ __forceinline__ void mma_step(const uint8_t *a_tiles, const uint8_t *b_tiles, const float *row, int row_stride,
                                         float sc0, float sc1, v4f (&acc)[4][TH], int frag_lo, int frag_hi, Issue issue)
{
    constexpr int GROUPS = 4 * TH;
    auto read_tile = [&](const uint8_t *tile) -> v8i {
        return cat(*reinterpret_cast<const v4i *>(tile + frag_lo), *reinterpret_cast<const v4i *>(tile + frag_hi));
    };
    v8i a[4];
#pragma unroll
    for (int k = 0; k < 4; k++) a[k] = read_tile(a_tiles + k * 2048);
    v8i b = read_tile(b_tiles);
    float f = row[0];
    v4f prev[4];
    float p0 = 0.f, p1 = 0.f;
#pragma unroll
    for (int t = 0; t < TH; t++) {
        v8i b_next = b;
        float f_next = f;
        if (t + 1 < TH) {
            b_next = read_tile(b_tiles + (t + 1) * 2048);
            f_next = row[(t + 1) * row_stride];
        }
        v4f cur[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            cur[k] = mfma_fp8(a[k], b);
            if (t > 0) {
                acc[k][t - 1] += prev[k] * ((k & 1) ? p1 : p0);
                asm volatile("" : "+v"(acc[k][t - 1]));   // the multiply-adds stay here, behind this matrix instruction
            }
            __builtin_amdgcn_sched_barrier(0);
            // loads i with i * GROUPS / NOPS == g go behind group g
#pragma unroll
            for (int i = 0; i < NOPS; i++)
                if (i * GROUPS / NOPS == t * 4 + k) issue(i);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) prev[k] = cur[k];
        p0 = f * sc0;
        p1 = f * sc1;
        b = b_next;
        f = f_next;
    }
#pragma unroll
    for (int k = 0; k < 4; k++) acc[k][TH - 1] += prev[k] * ((k & 1) ? p1 : p0);
}

// TH: 16-token tiles per wavefront; a row block has TM = 2 TH of them (block_m rounded up to 32 rows).
// Wavefront v = (w = v % 4, g = v / 4): weight rows 64 w .. 64 w + 63 of the slice, token tiles g TH .. g TH + TH - 1.
template <int TH>
__global__ __launch_bounds__(512) void moe_tile_kernel(const TileParams s)
{
    constexpr int TM = 2 * TH;
    constexpr int THREADS = 512;
    constexpr int AOPS = 4;                   // 2 of the pair's 4 weight tiles x 2 halves
    constexpr int XOPS = 3;                   // one token tile (2 halves) + its 16 scales
    constexpr int OPS1 = AOPS + XOPS;

    // [4 pairs][3 stages][4 tiles] weight rings | UP items: [3 stages][TM] token tiles; DOWN items: the requantised
    // tiles [n_ib][TM] in the same place
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds_dyn[];
    __shared__ __attribute__((aligned(1024))) uint8_t s_dummy[2048 + 256];
    __shared__ float s_xs[kStages][TM * 16];
    __shared__ float s_ws[2][kTileMaxKb];
    __shared__ float s_amax[4][TM * 16];
    __shared__ __attribute__((aligned(16))) float s_sa[kTileMaxIb][TM * 16];
    // chunked activation scales of UP items, [chunk & 1][tile][token][step & 3], in the place of the DOWN items' s_sa:
    // items of the two kinds never overlap in a workgroup (a barrier separates them, and an item's loads have landed)
    static_assert(kTileMaxIb * 16 >= 2 * 64, "s_xc does not fit s_sa");
    float (*s_xc)[TM * 64] = reinterpret_cast<float (*)[TM * 64]>(&s_sa[0][0]);
    __shared__ float s_w2s[kTileMaxW2s];
    __shared__ int s_tok[TM * 16];
    __shared__ int s_item[2];

    const MoeParams &p = s.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int w = wave & 3, g = wave >> 2;
    const int n = lane & 15;
    const int q = lane >> 4;
    const int K = p.K, I = p.N >> 1;
    const int n_ib = s.n_ib, nkb = s.nkb;
    const int epoch = (int)((unsigned)__builtin_amdgcn_readfirstlane(s.ctl->epoch) + 1u);
    uint8_t *a_ring = lds_dyn + w * (kStages * 8192);
    uint8_t *xbuf = lds_dyn + kARingBytes;

    // Row blocks are dealt to eight queues in contiguous runs (the blocks of one expert are neighbours), and a
    // workgroup serves the queue of its XCD first (the hardware deals workgroup i to XCD i % 8): the workgroups that
    // stream the same expert's weights at the same time then share one L2.
    int n_live = (__builtin_amdgcn_readfirstlane(p.ntpp[0]) + p.block_m - 1) / p.block_m;
    n_live = n_live < s.n_mb_max ? n_live : s.n_mb_max;
    const int per_q = (n_live + 7) >> 3;
    const int per_up = n_ib, per_down = s.n_cs * s.nh;

    // operand fragment of lane (n, q): chunks q and q+4 of row n; chunk c of row r sits at position c ^ ((r >> 1) & 7)
    const int f_n = (n >> 1) & 7;
    const int frag_lo = n * 128 + 16 * (q ^ f_n);
    const int frag_hi = n * 128 + 16 * ((q ^ f_n) ^ 4);
    // direct-to-LDS load h of a tile: lane l fills position l & 7 of row 8h + l / 8
    const int ld_row = lane >> 3;
    int ld_chunk[2];
#pragma unroll
    for (int h = 0; h < 2; h++) ld_chunk[h] = 16 * ((lane & 7) ^ (((8 * h + ld_row) >> 1) & 7));

    v4f acc[4][TH];

    // ---- UP item: slice ib of row block mb -> requantised operand tiles + scales in scratch, then the unit's flag ----
    // An expert with a single row block streams its weights with non-temporal loads (measured on the DeepSeek-V3 shard:
    // -13 % at M = 512 where nearly every expert has one block, +8 % at M = 8192 if applied to experts whose blocks run
    // side by side and share the lines in L2).
    auto lone_block = [&](int mb, int e) {
        if (s.w_nt >= 0) return s.w_nt != 0;
        const bool left = mb > 0 && __builtin_amdgcn_readfirstlane(p.expert_ids[mb - 1]) == e;
        const bool right = mb + 1 < n_live && __builtin_amdgcn_readfirstlane(p.expert_ids[mb + 1]) == e;
        return !left && !right;
    };

    const bool xs_chunk = s.xs_chunk != 0;
    auto up_item = [&](int mb, int ib) {
        int e = __builtin_amdgcn_readfirstlane(p.expert_ids[mb]);
        if (e < 0 || e >= p.E) return;
        const bool nt = lone_block(mb, e);
        if (tid < TM * 16) {
            const int idx = mb * p.block_m + tid;
            int id = -1;
            if (tid < p.block_m && idx < p.sorted_num) id = p.sorted_ids[idx];
            const int tk = id / p.top_k;
            s_tok[tid] = (id >= 0 && tk < p.M) ? tk : 0;
        }
        // this slice's gate (row 2*ib) and up (row 2*ib+1) scale rows
        {
            const float *ws_rows = p.w_scale + ((size_t)e * (p.N >> 7) + 2 * ib) * nkb;
            for (int i = tid; i < 2 * nkb; i += THREADS) s_ws[i >= nkb][i >= nkb ? i - nkb : i] = ws_rows[i];
        }
        __syncthreads();

        // token-tile gather: wavefront v loads tile v (a dummy where the block has no such tile)
        const bool x_real = wave < TM;
        const uint8_t *gx[2];
#pragma unroll
        for (int h = 0; h < 2; h++)
            gx[h] = p.x + (size_t)s_tok[x_real ? wave * 16 + 8 * h + ld_row : 0] * K + ld_chunk[h];
        const float *gxs = p.x_scale + (size_t)s_tok[x_real ? wave * 16 + (lane & 15) : 0] * nkb;
        // Weight rows of the pair: tile a = (32-row group a / 2, gate | up a % 2); matrix row r of the tile is slab row
        // group * 32 + (r / 8) * 16 + r % 8 (+ 8 for up), so load h of a tile covers slab rows ... + 16 h + lane / 8.
        // Wavefront (w, g) loads tiles 2g and 2g + 1 of pair w.
        const uint8_t *wbase = p.w + (size_t)e * p.N * K + (ib * 256 + w * 64 + g * 32 + ld_row) * p.w_rs;
        // operation i of a step's OPS1: weight tile half (i < AOPS), token tile half, token scales
        auto issue_op = [&](int kb, int stage, int i) {
            const int kc = kb < nkb ? kb : nkb - 1;
            if (i < AOPS) {
                const int up = i >> 1, h = i & 1;
                const uint8_t *src = wbase + (h * 16 + 8 * up) * p.w_rs + kc * p.w_ks + ld_chunk[h];
                uint8_t *dst = a_ring + stage * 8192 + (2 * g + up) * 2048 + h * 1024;
                if (nt) dma16<2>(src, dst);
                else dma16<0>(src, dst);
            } else if (i < AOPS + 2) {
                const int part = i - AOPS;
                uint8_t *dst = x_real ? xbuf + stage * (TM * 2048) + wave * 2048 : s_dummy;
                dma16<0>(gx[part] + (size_t)kc * 128, dst + part * 1024);
            } else if (xs_chunk) {
                // steps kb .. kb + 3 of the tile's 16 tokens, 16 bytes per token, with the loads of step kb & ~3
                float *sdst = x_real ? &s_xc[(kb >> 2) & 1][wave * 64] : reinterpret_cast<float *>(s_dummy + 2048);
                if ((kb & 3) == 0 && lane < 16) dma16<0>(reinterpret_cast<const uint8_t *>(gxs + (kb < nkb ? kb : nkb - 4)), reinterpret_cast<uint8_t *>(sdst));
            } else {
                float *sdst = x_real ? &s_xs[stage][wave * 16] : reinterpret_cast<float *>(s_dummy + 2048);
                if (lane < 16) dma4(gxs + kc, sdst);
            }
        };
        // load instructions of step kb: the scales come with every fourth step when they are fetched in chunks
        auto ops_of = [&](int kb) { return xs_chunk ? OPS1 - 1 + ((kb & 3) == 0 ? 1 : 0) : OPS1; };
        auto issue_all = [&](int kb, int stage) {
#pragma unroll
            for (int i = 0; i < OPS1; i++) issue_op(kb, stage, i);
        };
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int t = 0; t < TH; t++) acc[a][t] = (v4f){0.f, 0.f, 0.f, 0.f};

        // Per wavefront the loads of step kb are issued two steps ahead.  Step kb: wait for the own loads of kb (those of
        // kb + 1 stay in flight), meet the others (their tiles of kb have landed, and everybody is done reading
        // stage (kb + 2) % 3), then compute while refilling that stage.
        issue_all(0, 0);
        issue_all(1, 1);
        for (int kb0 = 0; kb0 < nkb; kb0 += kStages) {
#pragma unroll
            for (int h = 0; h < kStages; h++) {
                const int kb = kb0 + h;
                if (kb < nkb) {
                    if (ops_of(kb + 1) == OPS1) wait_vmcnt<OPS1>();
                    else wait_vmcnt<OPS1 - 1>();
                    lds_barrier();
                    const float *row = xs_chunk ? &s_xc[(kb >> 2) & 1][g * (TH * 64) + n * 4 + (kb & 3)]
                                                : &s_xs[h][g * (TH * 16) + n];
                    mma_step<TH, OPS1>(a_ring + h * 8192, xbuf + h * (TM * 2048) + g * (TH * 2048), row,
                                       xs_chunk ? 64 : 16, s_ws[0][kb], s_ws[1][kb], acc, frag_lo, frag_hi,
                                       [&](int i) { issue_op(kb + 2, (h + 2) % kStages, i); });
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        wait_vmcnt<0>();

        // SwiGLU, per-token amax over the slice's 128 columns, FP8 requant into operand tiles
#pragma unroll
        for (int t = 0; t < TH; t++) {
            float m = 0.f;
#pragma unroll
            for (int pr = 0; pr < 2; pr++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float a = swiglu_bf16(acc[2 * pr][t][j], acc[2 * pr + 1][t][j]);
                    acc[2 * pr][t][j] = a;
                    m = fmaxf(m, fabsf(a));
                }
            m = fmaxf(m, __shfl_xor(m, 16));
            m = fmaxf(m, __shfl_xor(m, 32));
            if (q == 0) s_amax[w][(g * TH + t) * 16 + n] = m;
        }
        __syncthreads();
        const int unit = mb * n_ib + ib;
#pragma unroll
        for (int t = 0; t < TH; t++) {
            const int tg = g * TH + t;
            float m = kAmaxFloor;
#pragma unroll
            for (int wv = 0; wv < 4; wv++) m = fmaxf(m, s_amax[wv][tg * 16 + n]);
            const float s_a = m / kFp8Max;
            uint8_t *tile = s.aqs + ((size_t)unit * TM + tg) * 2048;
#pragma unroll
            for (int pr = 0; pr < 2; pr++) {
                const uint32_t packed =
                    pack_fp8x4(clamp_fp8(acc[2 * pr][t][0] / s_a), clamp_fp8(acc[2 * pr][t][1] / s_a),
                               clamp_fp8(acc[2 * pr][t][2] / s_a), clamp_fp8(acc[2 * pr][t][3] / s_a));
                // columns w*32 + pr*16 + 4q .. +3 of token n: chunk w*2 + pr of the row, bytes 4q .. 4q+3 in it
                stg32_agent(tile, (uint32_t)(n * 128 + 16 * ((w * 2 + pr) ^ f_n) + 4 * q), packed);
            }
            if (w == 0 && q == 0)
                stg32_agent(s.sas + (size_t)unit * (TM * 16) + tg * 16, 4u * n, __builtin_bit_cast(uint32_t, s_a));
        }
        wait_vmcnt<0>();
        __syncthreads();
        if (tid == 0) store_agent(&s.flag[unit], epoch);
    };

    // ---- DOWN item: column groups [cs * gps, (cs + 1) * gps) of row block mb, all slices, token part `part` ------------
    // 64 output columns per step group.  Pair w takes the slab's groups w, w + 4, ...; its two wavefronts split the
    // tokens as before and each loads two of the four w2 tiles of a step.  Matrix row r of tile k is output column
    // c0 + 16 (r / 4) + 4 k + r % 4, so lane (n, q) collects columns c0 + 16 q .. c0 + 16 q + 15 of token n over the
    // four tiles.  Load h of a tile: rows 8h + lane / 8.
    // The requantised tiles of ALL slices have to sit in LDS next to the weight ring.  Where I/128 slices of a whole
    // block do not fit, the block's token tiles are served in TH / THD parts, each by an item of its own with THD
    // tiles per wavefront: part `part` covers token tiles [part * 2 THD, (part + 1) * 2 THD).
    auto down_item = [&](int mb, int cs, int part, auto thd_c) {
        constexpr int THD = decltype(thd_c)::value;
        constexpr int TMD = 2 * THD;
        const int e = __builtin_amdgcn_readfirstlane(p.expert_ids[mb]);
        if (e < 0 || e >= p.E) return;
        const bool nt = lone_block(mb, e);
        int slot[THD];
        bool valid[THD];
        float tw[THD];
#pragma unroll
        for (int t = 0; t < THD; t++) {
            const int row = (part * TMD + g * THD + t) * 16 + n;
            const int idx = mb * p.block_m + row;
            int id = -1;
            if (row < p.block_m && idx < p.sorted_num) id = p.sorted_ids[idx];
            valid[t] = id >= 0 && id / p.top_k < p.M;
            slot[t] = valid[t] ? id : 0;
            tw[t] = valid[t] ? p.topk_w[slot[t]] * p.scaling : 0.f;
            if (cs == 0 && w == 0 && q == 0 && valid[t]) s.live[slot[t]] = epoch;
        }
        for (int i = tid; i < (K >> 7) * n_ib; i += THREADS) s_w2s[i] = p.w2_scale[(size_t)e * (K >> 7) * n_ib + i];

        const int n_groups = K >> 6;
        const int g0 = cs * s.gps;
        const int g1 = g0 + s.gps < n_groups ? g0 + s.gps : n_groups;
        const int span = g1 - g0;
        int my_groups = (span - w + 3) >> 2;                      // the slab's groups w, w + 4, ... (none: 0)
        my_groups = my_groups > 0 ? my_groups : 0;
        const int n_steps = ((span + 3) >> 2) * n_ib;             // (group, slice) steps of the longest pair, slice-minor
        const uint8_t *w2base = p.w2 + (size_t)e * K * I + (16 * (lane >> 5) + (ld_row & 3)) * p.w2_rs;
        int lg = 0, lib = 0;   // (group index, slice) of the next step to load
        auto group_of = [&](int i) {   // i-th group of this pair, clamped into the slab for loads past its end
            int grp = g0 + w + 4 * (i < my_groups ? i : my_groups - 1);
            grp = grp < g0 ? g0 : grp;
            return grp < g1 ? grp : g1 - 1;
        };
        auto issue2_op = [&](int stage, int i) {   // operation i of AOPS of the step (lg, lib)
            const int c0 = group_of(lg) << 6;
            const int k = 2 * g + (i >> 1), h = i & 1;
            const uint8_t *src = w2base + (c0 + 32 * h + 4 * k) * p.w2_rs + lib * p.w2_ks + ld_chunk[h];
            uint8_t *dst = a_ring + stage * 8192 + k * 2048 + h * 1024;
            if (nt) dma16<2>(src, dst);
            else dma16<0>(src, dst);
        };
        auto advance2 = [&]() {
            lib++;
            if (lib == n_ib) {
                lib = 0;
                lg++;
            }
        };
        auto issue2 = [&](int stage) {
#pragma unroll
            for (int i = 0; i < AOPS; i++) issue2_op(stage, i);
            advance2();
        };
        // the weights do not depend on the up/gate phase: first two steps go out before the wait
        issue2(0);
        issue2(1);
        if (wave == 0) spin_all_ge(&s.flag[mb * n_ib], n_ib, epoch, s.ctl);
        __syncthreads();
        // the requantised tiles of this part and their scales come from scratch into LDS: [slice][tile of the part]
        uint8_t *aq = xbuf;
        for (int i = wave; i < n_ib * TMD; i += 8) {
            const int ib = i / TMD, tt = i - ib * TMD;
            const uint8_t *src = s.aqs + ((size_t)(mb * n_ib + ib) * TM + part * TMD + tt) * 2048 + lane * 16;
            dma16<16>(src, aq + i * 2048);
            dma16<16>(src + 1024, aq + i * 2048 + 1024);
        }
        for (int i = tid; i < n_ib * TMD * 16; i += THREADS) {
            const int ib = i / (TMD * 16), r = i - ib * (TMD * 16);
            const int bits = load_agent(
                reinterpret_cast<const int *>(&s.sas[(size_t)(mb * n_ib + ib) * (TM * 16) + part * (TMD * 16) + r]));
            s_sa[ib][r] = __builtin_bit_cast(float, bits);
        }
        wait_vmcnt<0>();
        __syncthreads();

        v4f accd[4][THD];
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int t = 0; t < THD; t++) accd[a][t] = (v4f){0.f, 0.f, 0.f, 0.f};
        int cg = 0, cib = 0;
        // the ring's first two steps were issued above and have landed (wait_vmcnt<0>): from here on one younger step
        // stays in flight
        for (int s0 = 0; s0 < n_steps; s0 += kStages) {
#pragma unroll
            for (int h = 0; h < kStages; h++) {
                if (s0 + h < n_steps) {
                    // one younger step of AOPS loads stays in flight; result stores only make this stricter
                    wait_vmcnt<AOPS>();
                    lds_barrier();
                    const int c0 = group_of(cg) << 6;
                    const float ws2 = s_w2s[(c0 >> 7) * n_ib + cib];
                    mma_step<THD, AOPS>(a_ring + h * 8192, aq + cib * (TMD * 2048) + g * (THD * 2048),
                                        &s_sa[cib][g * (THD * 16) + n], 16, ws2, ws2, accd, frag_lo, frag_hi,
                                        [&](int i) { issue2_op((h + 2) % kStages, i); });
                    advance2();
                    __builtin_amdgcn_sched_barrier(0);
                    cib++;
                    if (cib == n_ib) {
#pragma unroll
                        for (int t = 0; t < THD; t++) {
                            if (valid[t] && cg < my_groups) {
                                uint16_t *yp = s.y + (size_t)slot[t] * K + c0 + 16 * q;
#pragma unroll
                                for (int half = 0; half < 2; half++) {
                                    const v4f lo = accd[2 * half][t] * tw[t], hi = accd[2 * half + 1][t] * tw[t];
                                    v4i o;
                                    o.x = (int)pack_bf16x2(lo[0], lo[1]);
                                    o.y = (int)pack_bf16x2(lo[2], lo[3]);
                                    o.z = (int)pack_bf16x2(hi[0], hi[1]);
                                    o.w = (int)pack_bf16x2(hi[2], hi[3]);
                                    *reinterpret_cast<v4i *>(yp + 8 * half) = o;
                                }
                            }
#pragma unroll
                            for (int a = 0; a < 4; a++) accd[a][t] = (v4f){0.f, 0.f, 0.f, 0.f};
                        }
                        cib = 0;
                        cg++;
                    }
                }
            }
        }
        wait_vmcnt<0>();
    };
    // token parts of a DOWN item: the host picks the smallest divisor of TH whose tiles fit next to the weight ring
    auto run_down = [&](int mb, int sub) {
        const int cs = sub / s.nh, part = sub - cs * s.nh;
        if (s.nh == 1) {
            down_item(mb, cs, 0, std::integral_constant<int, TH>());
        } else if (TH % 2 == 0 && s.nh == 2) {
            down_item(mb, cs, part, std::integral_constant<int, (TH % 2 == 0 ? TH / 2 : TH)>());
        } else if (TH % 3 == 0 && s.nh == 3) {
            down_item(mb, cs, part, std::integral_constant<int, (TH % 3 == 0 ? TH / 3 : TH)>());
        } else if (TH % 4 == 0 && s.nh == 4) {
            down_item(mb, cs, part, std::integral_constant<int, (TH % 4 == 0 ? TH / 4 : TH)>());
        }
    };

    // ---- item loop ------------------------------------------------------------------------------------------------
    // Queue qq holds row blocks [qq * per_q, ...) as items: the up/gate items of `lag` blocks first, then alternately
    // the up/gate items of block lag + r and the down items of block r, at the end the down items of the last `lag`
    // blocks.  A down item waits for the flags of its block's up/gate items, which are EARLIER in the same queue:
    // whoever took them is running and waits for nothing later, so the queues drain with any number of resident
    // workgroups.  A workgroup that finds its queue empty moves on to the next one.
    auto blocks_of = [&](int qq) {
        const int left = n_live - qq * per_q;
        return left < 0 ? 0 : (left < per_q ? left : per_q);
    };
    // (Asking for the next item's ticket while the current item runs was tried: the round trip it hides, ~2 us per item,
    // does not show in a call's time - the kernel is bound by what all compute units pull together, not by one of them.)
    int qq = blockIdx.x & 7, visited = 0;   // state of thread 0
    while (true) {
        if (tid == 0) {
            int it = -1;
            while (visited < 8) {
                const int nb = blocks_of(qq);
                const int idx = nb > 0 ? __hip_atomic_fetch_add(&s.ctl->tile_head[qq], 1, __ATOMIC_RELAXED,
                                                                __HIP_MEMORY_SCOPE_AGENT)
                                       : 0;
                if (idx < nb * (per_up + per_down)) {
                    it = idx;
                    break;
                }
                qq = (qq + 1) & 7;
                visited++;
            }
            s_item[0] = it;
            s_item[1] = qq;
        }
        __syncthreads();
        const int item = __builtin_amdgcn_readfirstlane(s_item[0]);
        const int qi = __builtin_amdgcn_readfirstlane(s_item[1]);
        if (item < 0) break;
        const int nb = blocks_of(qi);
        const int lag = s.lag < nb ? s.lag : nb;
        const int head_items = lag * per_up, mid_items = (nb - lag) * (per_up + per_down);
        int up = -1, down = -1;
        if (item < head_items) {
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
            down = (nb - lag) * per_down + (item - head_items - mid_items);
        }
        if (up >= 0) {
            up_item(qi * per_q + up / per_up, up % per_up);
        } else {
            run_down(qi * per_q + down / per_down, down % per_down);
        }
        __syncthreads();   // everybody is done with the item's LDS tables and rings before the next item refills them
    }
    if (tid == 0) {
        const int left = __hip_atomic_fetch_add(&s.ctl->tile_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left == (int)gridDim.x - 1) {
            for (int i = 0; i < 8; i++) store_agent(&s.ctl->tile_head[i], 0);
            store_agent(&s.ctl->tile_done, 0);
        }
    }
}

// out[t] = bf16(out[t] + sum over the token's live slots of y[slot]); the last workgroup to leave closes the epoch.
// A unit is (token, 2048 columns): a thread owns 8 columns and keeps up to 8 row loads in flight.  Workgroups stride
// over the units so that the closing counter sees a few thousand arrivals, not one per unit.
__global__ __launch_bounds__(256) void moe_tile_reduce_kernel(const RowsReduce s, int chunks_per_token, int n_units)
{
    const MoeParams &p = s.p;
    const int epoch = (int)((unsigned)s.ctl->epoch + 1u);
    // a bounded wait that ran out (in this call's tile kernel or in any earlier launch on this workspace: the word is
    // sticky) means result rows may be missing: the output then says so itself, NaN in every element
    // (an ordinary load: this kernel starts after the tile kernel has ended, and every wavefront asking the memory side
    // for the same word with an agent-scope load cost ~100 us per call)
    const bool poisoned = s.ctl->error != 0;
    for (int unit = blockIdx.x; unit < n_units; unit += gridDim.x) {
        const int t = unit / chunks_per_token;
        const int c = (unit - t * chunks_per_token) * 2048 + threadIdx.x * 8;
        if (c >= p.K) continue;
        float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        auto add = [&](const v4i v) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                sum[2 * i] += __builtin_bit_cast(float, (uint32_t)v[i] << 16);
                sum[2 * i + 1] += __builtin_bit_cast(float, (uint32_t)v[i] & 0xffff0000u);
            }
        };
        v4i *op = reinterpret_cast<v4i *>(p.out + (size_t)t * p.K + c);
        v4i prior = {0, 0, 0, 0};
        if (!p.overwrite) prior = *op;
        const int *live = s.live + t * p.top_k;
        const uint16_t *yrow = s.y + (size_t)t * p.top_k * p.K + c;
        for (int s0 = 0; s0 < p.top_k; s0 += 8) {   // slot order: the sum depends on nothing but the inputs
            bool on[8];
            v4i v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) on[j] = s0 + j < p.top_k && live[s0 + j] == epoch;
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (on[j]) v[j] = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(yrow + (size_t)(s0 + j) * p.K));
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (on[j]) add(v[j]);
        }
        add(prior);
        v4i o;
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = poisoned ? 0x7fc07fc0 : (int)pack_bf16x2(sum[2 * i], sum[2 * i + 1]);
        *op = o;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int left = __hip_atomic_fetch_add(&s.ctl->fin_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left == (int)gridDim.x - 1) {
            __hip_atomic_store(&s.ctl->fin_done, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&s.ctl->epoch, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

// Token parts of a DOWN item: the smallest divisor nh of th such that the requantised tiles of all n_ib slices of a
// part (2 th / nh tiles per slice) fit next to the weight rings; 0 if none does.
int token_parts(int th, int n_ib)
{
    for (int nh = 1; nh <= th; nh++)
        if (th % nh == 0 && n_ib * (2 * th / nh) * 2048 <= kMaxTailBytes) return nh;
    return 0;
}

// LDS behind the weight rings: the 3-stage ring of token tiles (UP items) or the requantised tiles of a part (DOWN)
int tail_bytes(int th, int n_ib)
{
    const int up = kStages * 2 * th * 2048, down = n_ib * (2 * th / token_parts(th, n_ib)) * 2048;
    return up > down ? up : down;
}

typedef void (*TileFn)(const TileParams);

// 16-token tiles per wavefront: a row block is rounded up to 32 th rows
int tiles_per_wave(int block_m) { return (block_m + 31) / 32; }

TileFn pick(int th)
{
    switch (th) {
    case 1: return moe_tile_kernel<1>;
    case 2: return moe_tile_kernel<2>;
    case 3: return moe_tile_kernel<3>;
    default: return moe_tile_kernel<4>;
    }
}

// The variant's dynamic LDS limit is raised once per (variant, device), not on every launch.
hipError_t allow_dynamic_lds(int th, TileFn fn)
{
    static std::mutex mu;
    static bool done[5][64];
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    std::lock_guard<std::mutex> lock(mu);
    if (dev >= 0 && dev < 64 && done[th][dev]) return hipSuccess;
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                              kARingBytes + kMaxTailBytes);
    if (err == hipSuccess && dev >= 0 && dev < 64) done[th][dev] = true;
    return err;
}

}  // namespace

// 64-column groups per DOWN item: about 5 * stages ring steps (a step is one group x one slice; 14 at stages = 3), a
// multiple of 4 so that every pair of wavefronts gets the same number of groups
static int groups_per_item(int n_ib, int stages)
{
    const int e = tunable(kTunTileGps, 0);
    if (e > 0) return (e + 3) / 4 * 4;
    const int steps = stages == 3 ? 14 : 5 * stages;
    return 4 * ((steps + n_ib - 1) / n_ib);
}

bool tile_supported(int top_k, int M, int K, int N, int E, int sorted_num, int block_m)
{
    (void)E;
    const int tm = 2 * tiles_per_wave(block_m);
    const int n_ib = N / 256;
    const int64_t n_mb = ((int64_t)sorted_num + block_m - 1) / block_m;
    return n_ib <= kTileMaxIb && token_parts(tm / 2, n_ib) > 0 && K <= 128 * kTileMaxKb &&
           (K / 128) * n_ib <= kTileMaxW2s && (int64_t)M * top_k <= kMaxSlots && n_mb * n_ib <= kMaxUnits;
}

size_t tile_workspace_bytes(int top_k, int M, int K, int N, int E, int sorted_num, int block_m)
{
    (void)E;
    const int tm = 2 * tiles_per_wave(block_m);
    const size_t n_mb = ((size_t)sorted_num + block_m - 1) / block_m;
    return align_up(kPrefixBytes) + align_up((size_t)M * top_k * K * sizeof(uint16_t)) +
           align_up(n_mb * (N / 256) * tm * 2048) + align_up(n_mb * (N / 256) * tm * 16 * sizeof(float));
}

hipError_t launch_tile(const MoeParams &p, int stages, void *workspace, hipStream_t stream)
{
    uint8_t *ws = static_cast<uint8_t *>(workspace);
    TileParams s;
    s.p = p;
    s.n_ib = p.N / 256;
    s.nkb = p.K / 128;
    s.n_mb_max = (p.sorted_num + p.block_m - 1) / p.block_m;
    const int tm = 2 * tiles_per_wave(p.block_m);
    size_t off = align_up(kPrefixBytes);
    s.ctl = reinterpret_cast<StreamCtl *>(ws);
    s.flag = reinterpret_cast<int *>(ws + kOffFlag);
    s.live = reinterpret_cast<int *>(ws + kOffLive);
    s.y = reinterpret_cast<uint16_t *>(ws + off);
    off += align_up((size_t)p.M * p.top_k * p.K * sizeof(uint16_t));
    s.aqs = ws + off;
    off += align_up((size_t)s.n_mb_max * s.n_ib * tm * 2048);
    s.sas = reinterpret_cast<float *>(ws + off);
    s.gps = groups_per_item(s.n_ib, stages);
    s.n_cs = ((p.K >> 6) + s.gps - 1) / s.gps;
    // up/gate items of this many row blocks run ahead of the first down items of a queue: with ~32 workgroups
    // on a queue, a down item's up/gate items were taken at least two rounds of the queue earlier
    s.lag = tunable(kTunTileLag, 64);
    s.w_nt = tunable(kTunTileNt, -1);
    s.xs_chunk = (s.nkb % 4 == 0 && reinterpret_cast<uintptr_t>(p.x_scale) % 16 == 0) ? 1 : 0;
    if (s.lag < 1) s.lag = 1;
    const TileFn fn = pick(tm / 2);
    s.nh = token_parts(tm / 2, s.n_ib);
    const int lds_bytes = kARingBytes + tail_bytes(tm / 2, s.n_ib);
    hipError_t err = allow_dynamic_lds(tm / 2, fn);   // once per variant and device
    if (err != hipSuccess) return err;
    // persistent workgroups, one per compute unit (the rings take most of a CU's LDS); fewer when there is less work
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            return 256;
        return n;
    }();
    const int64_t items = (int64_t)s.n_mb_max * (s.n_ib + s.n_cs * s.nh);
    int grid = tunable(kTunTileGrid, cus);
    if (grid > items) grid = (int)((items + 7) / 8 * 8);
    if (grid < 8) grid = 8;
    hipLaunchKernelGGL(fn, dim3((unsigned)grid), dim3(512), lds_bytes, stream, s);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    RowsReduce r;
    r.p = p;
    r.ctl = s.ctl;
    r.live = s.live;
    r.y = s.y;
    return launch_rows_reduce(r, stream);
}

hipError_t launch_rows_reduce(const RowsReduce &r, hipStream_t stream)
{
    const int chunks = (r.p.K + 2047) / 2048;
    const int n_units = r.p.M * chunks;
    hipLaunchKernelGGL(moe_tile_reduce_kernel, dim3((unsigned)(n_units < 4096 ? n_units : 4096)), dim3(256), 0, stream, r,
                       chunks, n_units);
    return hipGetLastError();
}

}  // namespace alpha_moe
