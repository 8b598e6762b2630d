// Fused W8A8 MoE, "wide" kernel for large batches: the work unit is a MACRO BLOCK of up to 256 consecutive sorted rows
// of one expert (as many whole row blocks of block_m rows as fit), not a single row block.
//
// Why: on MI355X the tile kernel's up/gate items spend their time bringing operands to LDS, not multiplying them.  A
// 256-row weight slab against 128 tokens is 48 KiB through L2 per 128-byte K step for 8.4 MFLOP; against 256 tokens it
// is 64 KiB for 16.8 MFLOP, a third fewer bytes per flop, and the weight bytes - the ones that miss L2 because an
// expert's slab is streamed once - are halved.  The 256 x 256 fp32 accumulators are 128 registers of each of the
// workgroup's eight wavefronts, which is what the register file holds next to the operands.
//
// Persistent workgroups of 8 wavefronts (two per SIMD, one workgroup per compute unit) take items from eight queues,
// one per XCD, exactly as in the tile kernel.  A macro block is I/128 UP items (one 128-column slice each) and a few
// DOWN items (a slab of output columns each).  Which row blocks form a macro block is decided on the device by
// moe_wide_plan_kernel (the host does not know expert_ids): consecutive blocks of one expert, floor(256 / block_m) at
// a time.
//
// Wavefront (w, g): weight rows 64 w .. 64 w + 63 (four operand tiles, shared with the pair's other wavefront through
// a two-stage LDS ring), token tiles g, g + 2, ..., g + 14 (interleaved so that a partly filled macro block loads
// both wavefronts of a pair alike).  Token tiles past the block's last valid row are neither loaded nor multiplied.
// Two ring stages of 64 KiB (32 KiB of weights, 32 KiB of tokens): the loads of step k + 1 are issued while step k
// is multiplied, and one workgroup barrier per step orders everything.
//
// UP item: SwiGLU and the FP8 requantisation of the 128-column group in registers, operand tiles + per-token scales
// to scratch, then the unit's flag (fused_moe_w8a8_up_down_acc.cu:863-994 of the reference).  DOWN item: waits for
// the flags of the block's slices and contracts their tiles with w2, 64 output columns per pair of wavefronts and
// step; the tiles either sit in LDS for the whole item (I/128 <= 2: they fit where the token ring was) or stream
// through the ring like tokens do.  Each valid (token, slot) row is written once, bf16, whole 128-byte lines, to
// y[slot]; the tile kernel's reduce kernel sums a token's rows in fp32 and rounds into `out` once
// (fused_moe_w8a8_up_down_acc.cu:1007-1096 adds top_k * I/128 partial rows per token into the output instead).
#include <mutex>
#include <type_traits>

#include "moe_common.hpp"

namespace alpha_moe {
namespace {

constexpr int kWRows = 256;                 // token rows of a macro block
constexpr int kWTiles = kWRows / 16;        // 16-token operand tiles of a macro block
constexpr int kWStageA = 4 * 4 * 2048;      // 4 pairs x 4 weight tiles of 2 KiB
constexpr int kWStageX = kWTiles * 2048;    // 16 token tiles
constexpr int kWDynLds = 2 * kWStageA + 2 * kWStageX;
constexpr int kWMaxKb = 128;                // most 128-byte K blocks (K <= 16384)
constexpr int kWMaxW2s = 1024;              // most w2 block scales of one expert, (K/128) * (I/128)
constexpr int kWResidentIb = 2;             // slices whose requantised tiles fit LDS for a whole DOWN item

struct WideParams {
    MoeParams p;
    StreamCtl *ctl;
    int *flag;        // [first row block of a macro block][n_ib] == epoch once the slice's tiles are in scratch
    int *live;        // [slots] == epoch once y[slot] is written this launch
    uint16_t *y;      // [slots][K] bf16
    uint8_t *aqs;     // [n_ib][n_tiles_total] requantised operand tiles of 2 KiB
    float *sas;       // [n_ib][n_tiles_total * 16] their per-token scales
    int *plan;        // [0] macro blocks of this launch; [4 + 4 m ..]: first row block, expert, row blocks, "the expert's
                      // only macro block" of macro block m
    int n_ib, nkb, n_mb_max;
    int blocks_per_macro;   // floor(256 / block_m)
    int tpb;                // 16-row tile slots per row block in scratch, ceil(block_m / 16)
    int n_tiles_total;      // n_mb_max * tpb
    int gps, n_cs;          // 64-column groups per DOWN item, column slabs per macro block
    int lag;                // macro blocks whose up/gate items precede the first down items of a queue
    int w_nt;               // weights with non-temporal loads: 1 always, 0 never, -1 for experts with one macro block
    int xs_chunk;           // 1: a token's activation scales are fetched four K steps at a time (K / 128 a multiple of 4,
                            // x_scale 16-byte aligned), 0: one step at a time
};

__device__ __forceinline__ int rfl(int v) { return __builtin_amdgcn_readfirstlane(v); }

// A wavefront-uniform pointer the compiler cannot fold into per-lane address arithmetic: added to a 32-bit per-lane
// offset it gives the "scalar base + vector offset" form of a load, one address register per lane instead of two
// and no 64-bit vector adds per step.
template <typename T>
__device__ __forceinline__ const T *uniform_ptr(const T *ptr)
{
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = (uint32_t)rfl((int)(uint32_t)v), hi = (uint32_t)rfl((int)(uint32_t)(v >> 32));
    return reinterpret_cast<const T *>(((uint64_t)hi << 32) | lo);
}

// Direct-to-LDS loads of 16 and 4 bytes per lane from (uniform base + 32-bit per-lane offset).  The empty asm keeps the
// address addition in the load's own basic block, where instruction selection can fold it into the load.
template <int AUX>
__device__ __forceinline__ void dma16_sv(const void *ubase, unsigned voff, void *lds)
{
    asm volatile("" : "+v"(voff));
    const uint8_t *g = uniform_ptr(static_cast<const uint8_t *>(ubase)) + (size_t)voff;
    __builtin_amdgcn_global_load_lds((gptr_t)(uintptr_t)g, (lptr_t)(uint32_t)(uintptr_t)lds, 16, 0, AUX);
}
template <int AUX>
__device__ __forceinline__ void dma4_sv(const void *ubase, unsigned voff, void *lds)
{
    asm volatile("" : "+v"(voff));
    const uint8_t *g = uniform_ptr(static_cast<const uint8_t *>(ubase)) + (size_t)voff;
    __builtin_amdgcn_global_load_lds((gptr_t)(uintptr_t)g, (lptr_t)(uint32_t)(uintptr_t)lds, 4, 0, AUX);
}

// ---- which row blocks form the macro blocks ------------------------------------------------------------------------
// One workgroup.  Row block mb leads a macro block when its distance from the first block of its expert's run is a
// multiple of blocks_per_macro; blocks whose expert id is outside [0, E) lead nothing and belong to nothing.
__global__ __launch_bounds__(1024) void moe_wide_plan_kernel(const WideParams s)
{
    __shared__ int s_last_start[16];
    __shared__ int s_count[16];
    __shared__ int s_carry[2];   // run start before this chunk, leaders before this chunk
    const MoeParams &p = s.p;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int n_live = (p.ntpp[0] + p.block_m - 1) / p.block_m;
    n_live = n_live < s.n_mb_max ? n_live : s.n_mb_max;
    if (tid == 0) {
        s_carry[0] = 0;
        s_carry[1] = 0;
    }
    __syncthreads();
    for (int base = 0; base < n_live; base += 1024) {
        const int mb = base + tid;
        const bool in = mb < n_live;
        const int e = in ? p.expert_ids[mb] : -1;
        const int e_prev = (in && mb > 0) ? p.expert_ids[mb - 1] : -2;
        const bool starts = in && (mb == 0 || e != e_prev);
        const unsigned long long smask = __ballot(starts);
        const unsigned long long upto = smask & (~0ull >> (63 - lane));
        int start = upto ? (base + wave * 64 + 63 - __builtin_clzll(upto)) : -1;
        if (lane == 63) s_last_start[wave] = start;
        __syncthreads();
        if (start < 0) {
            for (int v = wave - 1; v >= 0 && start < 0; v--) start = s_last_start[v];
            if (start < 0) start = s_carry[0];
        }
        const bool leader = in && e >= 0 && e < p.E && ((mb - start) % s.blocks_per_macro) == 0;
        const unsigned long long lmask = __ballot(leader);
        if (lane == 0) s_count[wave] = __builtin_popcountll(lmask);
        __syncthreads();
        int pos = s_carry[1] + __builtin_popcountll(lmask & ((1ull << lane) - 1ull));
        for (int v = 0; v < wave; v++) pos += s_count[v];
        if (leader) {
            // the macro block's row blocks: up to blocks_per_macro consecutive ones of this expert
            int nb = 1;
            while (nb < s.blocks_per_macro && mb + nb < n_live && p.expert_ids[mb + nb] == e) nb++;
            const bool more_after = mb + nb < n_live && p.expert_ids[mb + nb] == e;
            *reinterpret_cast<v4i *>(&s.plan[4 + 4 * pos]) = (v4i){mb, e, nb, (mb == start && !more_after) ? 1 : 0};
        }
        __syncthreads();
        if (tid == 1023) {
            int total = pos + (leader ? 1 : 0);
            s_carry[0] = start;
            s_carry[1] = total;
        }
        __syncthreads();
    }
    if (tid == 0) s.plan[0] = s_carry[1];
}

// One step of a wavefront: the pair's 4 weight tiles x up to 8 token tiles, all from LDS.
//   acc[k][t] += (A_k x B_t) * row[t] * (k odd ? sc1 : sc0)
// with row[] a per-token factor in LDS.  Token tile t of the wavefront sits 4 KiB behind tile t - 1 (the other
// wavefront of the pair owns the tiles in between); only the first nt_w tiles are live.  The product of (k, t) is
// scaled into its accumulator behind the matrix instruction of (k + 1, t).  issue(t) puts the step's loads between the
// token tiles, whatever nt_w is.
template <typename Issue>
__device__ __forceinline__ void wide_step(const uint8_t *a_tiles, const uint8_t *b_tiles, const float *row, float sc0,
                                          float sc1, v4f (&acc)[4][8], int frag_lo, int frag_hi, int nt_w, Issue issue)
{
    auto read_tile = [&](const uint8_t *tile) -> v8i {
        return cat(*reinterpret_cast<const v4i *>(tile + frag_lo), *reinterpret_cast<const v4i *>(tile + frag_hi));
    };
    v8i a[4];
#pragma unroll
    for (int k = 0; k < 4; k++) a[k] = read_tile(a_tiles + k * 2048);
    v8i b = read_tile(b_tiles);
    float f = row[0];
#pragma unroll
    for (int t = 0; t < 8; t++) {
        issue(t);
        v8i b_next = b;
        float f_next = f;
        if (t + 1 < 8) {
            b_next = read_tile(b_tiles + (t + 1) * 4096);
            // per-token factors of tile tt sit at (tt & 7) * 32 + (tt >> 3) * 16; tt = 2 t + g, g folded into `row`
            f_next = row[(t + 1) < 4 ? (t + 1) * 64 : (t + 1 - 4) * 64 + 16];
        }
        if (t < nt_w) {
            const float p0 = f * sc0, p1 = f * sc1;
            v4f prev;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const v4f cur = mfma_fp8(a[k], b);
                __builtin_amdgcn_sched_barrier(0);
                if (k > 0) {
                    acc[k - 1][t] += prev * (((k - 1) & 1) ? p1 : p0);
                    asm volatile("" : "+v"(acc[k - 1][t]));   // the multiply-adds stay behind this matrix instruction
                }
                prev = cur;
                __builtin_amdgcn_sched_barrier(0);
            }
            acc[3][t] += prev * p1;
            asm volatile("" : "+v"(acc[3][t]));
        }
        b = b_next;
        f = f_next;
    }
}

// Half a step: token tiles T0 .. T0 + 3 of the wavefront (TS bytes apart in LDS) against weight fragments already in
// registers.  Same arithmetic and order as wide_step.
// The per-token factor of the wavefront's token tile t is row[t * row_a + (t >= 4 ? row_b : 0)].
template <int T0, int TS, typename Issue>
__device__ __forceinline__ void wide_half(const v8i (&a)[4], const uint8_t *b_tiles, const float *row, int row_a, int row_b,
                                          float sc0, float sc1, v4f (&acc)[4][8], int frag_lo, int frag_hi, int nt_w,
                                          Issue issue)
{
    auto read_tile = [&](const uint8_t *tile) -> v8i {
        return cat(*reinterpret_cast<const v4i *>(tile + frag_lo), *reinterpret_cast<const v4i *>(tile + frag_hi));
    };
    auto row_at = [&](int t) { return row[t * row_a + (t >= 4 ? row_b : 0)]; };
    v8i b = read_tile(b_tiles + T0 * TS);
    float f = row_at(T0);
#pragma unroll
    for (int t = T0; t < T0 + 4; t++) {
        issue(t);
        v8i b_next = b;
        float f_next = f;
        if (t + 1 < T0 + 4) {
            b_next = read_tile(b_tiles + (t + 1) * TS);
            f_next = row_at(t + 1);
        }
        if (t < nt_w) {
            const float p0 = f * sc0, p1 = f * sc1;
            v4f prev;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const v4f cur = mfma_fp8(a[k], b);
                __builtin_amdgcn_sched_barrier(0);
                if (k > 0) {
                    acc[k - 1][t] += prev * (((k - 1) & 1) ? p1 : p0);
                    asm volatile("" : "+v"(acc[k - 1][t]));
                }
                prev = cur;
                __builtin_amdgcn_sched_barrier(0);
            }
            acc[3][t] += prev * p1;
            asm volatile("" : "+v"(acc[3][t]));
        }
        b = b_next;
        f = f_next;
    }
}

// A whole step of a wavefront that has the matrix pipe to itself: its token tiles (TS bytes apart in LDS) against weight
// fragments in registers, same arithmetic and order per accumulator as wide_step.  A lone wavefront issues one
// instruction every four cycles and a matrix instruction occupies the pipe for 32, so a token tile (four matrix
// instructions) has 32 issue slots and the stream must be straight-line and free of wait states to keep the pipe fed:
//  - a product is scaled into its accumulator D matrix instructions after its own (a vector instruction may read a
//    product 11 slots after the matrix instruction was issued; a group of one matrix instruction and four
//    multiply-adds is 5), and the queue of D products lives on from one step to the next: it is cleared before an
//    item's first step and drained after its last (wide_queue_drain);
//  - the tiles run from the top down and only in blocks of four: tiles 7 .. 4 when the wavefront has more than four
//    live tiles, then tiles 3 .. 0, so a step always ends with tile 0 and the products a step finds in the queue are
//    those of tile 0.  A dead tile of a block is multiplied like a live one (whatever its LDS holds; nobody reads a dead
//    tile's accumulators);
//  - the first tile's operands are read at the start of the step (wide_top_read), every other tile's while the tile
//    before it is multiplied; the weight-block factors and the weight fragments are in registers before the barrier
//    that starts the step.
// The operand reads are written as instructions the compiler knows nothing about, and waited for by hand: it would
// wait for ALL outstanding LDS reads before a tile's first matrix instruction, the next tile's (just issued) included,
// which puts an LDS round trip into every other tile.  LDS reads complete in order, so "at most the three reads just
// issued are outstanding" is what a tile needs.
template <int OFF>
__device__ __forceinline__ v4i lds_read16_raw(unsigned addr)
{
    v4i v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
__device__ __forceinline__ float lds_read4_raw(unsigned addr)
{
    float v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
template <int N>
__device__ __forceinline__ void lds_landed_but(v4i &lo, v4i &hi, float &f)
{
    asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(lo), "+v"(hi), "+v"(f) : "n"(N));
}

// operands of the first tile of a step: tile 7 (upper) or 3
template <int TS>
__device__ __forceinline__ void wide_top_read(const uint8_t *b_tiles, const float *row, int row_a, int frag_lo, int frag_hi,
                                              bool upper, v4i &b_lo, v4i &b_hi, float &f)
{
    const unsigned a_lo = (uint32_t)(uintptr_t)b_tiles + (unsigned)frag_lo, a_hi = (uint32_t)(uintptr_t)b_tiles + (unsigned)frag_hi;
    const unsigned a_f = (uint32_t)(uintptr_t)row, f_stride = 4u * (unsigned)row_a;
    if (upper) {
        b_lo = lds_read16_raw<7 * TS>(a_lo);
        b_hi = lds_read16_raw<7 * TS>(a_hi);
        f = lds_read4_raw(a_f + 7u * f_stride);
    } else {
        b_lo = lds_read16_raw<3 * TS>(a_lo);
        b_hi = lds_read16_raw<3 * TS>(a_hi);
        f = lds_read4_raw(a_f + 3u * f_stride);
    }
}

template <int TS, int D>
__device__ __forceinline__ void wide_tiles8(const v8i (&a)[4], const uint8_t *b_tiles, const float *row, int row_a, float sc0,
                                            float sc1, v4f (&acc)[4][8], int frag_lo, int frag_hi, bool upper, v4i &b_lo,
                                            v4i &b_hi, float &f, v4f (&prod)[D], float (&fac)[D])
{
    static_assert(D >= 1 && D <= 3, "queue depth");
    static_assert(7 * TS < 65536, "tile offsets are instruction immediates");
    const unsigned a_lo = (uint32_t)(uintptr_t)b_tiles + (unsigned)frag_lo, a_hi = (uint32_t)(uintptr_t)b_tiles + (unsigned)frag_hi;
    const unsigned a_f = (uint32_t)(uintptr_t)row, f_stride = 4u * (unsigned)row_a;
    // tile t; the tile multiplied before it was tile `before` (of this step, or tile 0 of the step before)
    auto tile = [&](auto tc, auto bc) {
        constexpr int t = decltype(tc)::value, before = decltype(bc)::value;
        v4i n_lo = b_lo, n_hi = b_hi;
        float n_f = f;
        if constexpr (t > 0) {
            n_lo = lds_read16_raw<(t > 0 ? t - 1 : 0) * TS>(a_lo);
            n_hi = lds_read16_raw<(t > 0 ? t - 1 : 0) * TS>(a_hi);
            n_f = lds_read4_raw(a_f + (unsigned)(t - 1) * f_stride);
            lds_landed_but<3>(b_lo, b_hi, f);
        } else {
            lds_landed_but<0>(b_lo, b_hi, f);
        }
        const v8i b = cat(b_lo, b_hi);
        const float p0 = f * sc0, p1 = f * sc1;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const v4f cur = mfma_fp8(a[k], b);
            __builtin_amdgcn_sched_barrier(0);
            // the oldest product of the queue: D matrix instructions back
            v4f &dst = k >= D ? acc[k - D][t] : acc[4 - D + k][before];
            dst += prod[0] * fac[0];
            asm volatile("" : "+v"(dst));
#pragma unroll
            for (int i = 0; i + 1 < D; i++) {
                prod[i] = prod[i + 1];
                fac[i] = fac[i + 1];
            }
            prod[D - 1] = cur;
            fac[D - 1] = (k & 1) ? p1 : p0;
            __builtin_amdgcn_sched_barrier(0);
        }
        b_lo = n_lo;
        b_hi = n_hi;
        f = n_f;
    };
    using std::integral_constant;
    if (upper) {
        tile(integral_constant<int, 7>{}, integral_constant<int, 0>{});
        tile(integral_constant<int, 6>{}, integral_constant<int, 7>{});
        tile(integral_constant<int, 5>{}, integral_constant<int, 6>{});
        tile(integral_constant<int, 4>{}, integral_constant<int, 5>{});
        tile(integral_constant<int, 3>{}, integral_constant<int, 4>{});
    } else {
        tile(integral_constant<int, 3>{}, integral_constant<int, 0>{});
    }
    tile(integral_constant<int, 2>{}, integral_constant<int, 3>{});
    tile(integral_constant<int, 1>{}, integral_constant<int, 2>{});
    tile(integral_constant<int, 0>{}, integral_constant<int, 1>{});
}

template <int D>
__device__ __forceinline__ void wide_queue_clear(v4f (&prod)[D], float (&fac)[D])
{
#pragma unroll
    for (int i = 0; i < D; i++) {
        prod[i] = (v4f){0.f, 0.f, 0.f, 0.f};
        fac[i] = 0.f;
    }
}

// after an item's last step: the queue holds the last D products of tile 0
template <int D>
__device__ __forceinline__ void wide_queue_drain(v4f (&acc)[4][8], v4f (&prod)[D], float (&fac)[D])
{
#pragma unroll
    for (int i = 0; i < D; i++) acc[4 - D + i][0] += prod[i] * fac[i];
}

// "At most n of this wavefront's loads are still outstanding", n known only at run time (the same for all lanes).
// Loads complete in the order they were issued, so this is "every load issued before the last n has landed".
__device__ __forceinline__ void wait_pending(int n)
{
    switch (n) {
    case 0: wait_vmcnt<0>(); break;
    case 1: wait_vmcnt<1>(); break;
    case 2: wait_vmcnt<2>(); break;
    case 3: wait_vmcnt<3>(); break;
    case 4: wait_vmcnt<4>(); break;
    case 5: wait_vmcnt<5>(); break;
    case 6: wait_vmcnt<6>(); break;
    case 7: wait_vmcnt<7>(); break;
    case 8: wait_vmcnt<8>(); break;
    case 9: wait_vmcnt<9>(); break;
    case 10: wait_vmcnt<10>(); break;
    case 11: wait_vmcnt<11>(); break;
    case 12: wait_vmcnt<12>(); break;
    case 13: wait_vmcnt<13>(); break;
    case 14: wait_vmcnt<14>(); break;
    case 15: wait_vmcnt<15>(); break;
    default: wait_vmcnt<16>(); break;
    }
}

// Products in flight between a matrix instruction and its scaled accumulate in the ping-pong loop: two leave one wait
// state per matrix instruction and keep the loops free of register spills (three would leave none, and spill).
constexpr int kPpDepth = 2;

// PP: the up/gate items run the two wavefronts of a SIMD half a step apart (see up_item).
template <bool PP>
__global__ __launch_bounds__(512) void moe_wide_kernel(const WideParams s)
{
    constexpr int THREADS = 512;
    // [2 stages][4 pairs][4 tiles] weight ring | [2 stages][16] token tiles (UP, streamed DOWN) or the requantised
    // tiles [n_ib][16] of a resident DOWN item in the same place
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds_dyn[];
    __shared__ float s_xs[2][kWRows];        // per-token factors of a ring stage, tile tt at (tt & 7) * 32 + (tt >> 3) * 16
    __shared__ __attribute__((aligned(16))) float s_xc[2][kWRows * 4];   // UP, chunked: [chunk & 1][tile][token][step & 3]
    __shared__ float s_ws[2][kWMaxKb];
    __shared__ float s_amax[4][kWRows];
    __shared__ float s_w2s[kWMaxW2s];
    __shared__ int s_tok[kWRows];            // UP: token of each row (-1: none); DOWN: slot of each row (-1: none)
    __shared__ float s_tw[kWRows];
    __shared__ int s_last[4];
    __shared__ int s_item[2];

    const MoeParams &p = s.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = rfl(tid >> 6);
    const int w = wave & 3, g = wave >> 2;
    const int n = lane & 15;
    const int q = lane >> 4;
    const int K = p.K, I = p.N >> 1;
    const int n_ib = s.n_ib, nkb = s.nkb;
    const int epoch = (int)((unsigned)rfl(s.ctl->epoch) + 1u);
    uint8_t *a_ring = lds_dyn;
    uint8_t *xbuf = lds_dyn + 2 * kWStageA;

    int n_live = (rfl(p.ntpp[0]) + p.block_m - 1) / p.block_m;
    n_live = n_live < s.n_mb_max ? n_live : s.n_mb_max;
    const int n_macro = rfl(s.plan[0]);
    const int per_q = (n_macro + 7) >> 3;
    const int per_up = n_ib, per_down = s.n_cs;

    // operand fragment of lane (n, q): chunks q and q+4 of row n; chunk c of row r sits at position c ^ ((r >> 1) & 7)
    const int f_n = (n >> 1) & 7;
    const int frag_lo = n * 128 + 16 * (q ^ f_n);
    const int frag_hi = n * 128 + 16 * ((q ^ f_n) ^ 4);
    // direct-to-LDS load h of a tile: lane l fills position l & 7 of row 8h + l / 8
    const int ld_row = lane >> 3;
    unsigned ld_chunk[2];
#pragma unroll
    for (int h = 0; h < 2; h++) ld_chunk[h] = 16u * ((lane & 7) ^ (((8 * h + ld_row) >> 1) & 7));
    // per-token factors of this lane's token in tile g (later tiles: see wide_step)
    const int row_off = g * 32 + n;

    v4f acc[4][8];
    auto clear_acc = [&]() {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int t = 0; t < 8; t++) acc[a][t] = (v4f){0.f, 0.f, 0.f, 0.f};
    };

    // Rows of macro block m: row blocks mb0 .. mb0 + nb - 1 of expert e, sorted rows row0 .. row0 + n_rows - 1.
    struct Macro {
        int mb0, e, row0, n_rows;
        bool lone;   // the expert has no other macro block
    };
    auto macro_of = [&](int m) {   // one load: the plan kernel has looked the expert ids up
        const v4i ent = *reinterpret_cast<const v4i *>(&s.plan[4 + 4 * m]);
        Macro mc;
        mc.mb0 = rfl(ent.x);
        mc.e = rfl(ent.y);
        mc.row0 = mc.mb0 * p.block_m;
        mc.n_rows = rfl(ent.z) * p.block_m;
        if (mc.row0 + mc.n_rows > p.sorted_num) mc.n_rows = p.sorted_num - mc.row0;
        mc.lone = s.w_nt >= 0 ? s.w_nt != 0 : rfl(ent.w) != 0;
        return mc;
    };
    // Routing of the block's rows into LDS; returns the number of 16-row tiles up to the last valid row.
    auto load_rows = [&](const Macro &mc, bool for_down, int cs) {
        if (tid < kWRows) {
            int id = -1;
            if (tid < mc.n_rows) id = p.sorted_ids[mc.row0 + tid];
            const int tk = id / p.top_k;
            const bool ok = id >= 0 && tk < p.M;
            if (!for_down) {
                s_tok[tid] = ok ? tk : -1;
            } else {
                s_tok[tid] = ok ? id : -1;
                s_tw[tid] = ok ? p.topk_w[id] * p.scaling : 0.f;
                if (ok && cs == 0) s.live[id] = epoch;
            }
            const unsigned long long okm = __ballot(ok);
            if (lane == 0) s_last[wave] = okm ? wave * 64 + 63 - __builtin_clzll(okm) : -1;
        }
    };
    auto tiles_of = [&]() {
        int last = s_last[0];
#pragma unroll
        for (int v = 1; v < 4; v++) last = s_last[v] > last ? s_last[v] : last;
        return rfl((last >> 4) + 1);   // 0 when no row is valid
    };

    // ---- UP item: slice ib of macro block m -> requantised operand tiles + scales in scratch, then the unit's flag --
    auto up_item = [&](int m, int ib) {
        const Macro mc = macro_of(m);
        load_rows(mc, false, 0);
        {
            // this slice's gate (row 2*ib) and up (row 2*ib+1) scale rows
            const float *ws_rows = p.w_scale + ((size_t)mc.e * (p.N >> 7) + 2 * ib) * nkb;
            for (int i = tid; i < 2 * nkb; i += THREADS) s_ws[i >= nkb][i >= nkb ? i - nkb : i] = ws_rows[i];
        }
        __syncthreads();
        const int n_tiles = tiles_of();
        const int nt_w = n_tiles > g ? (n_tiles - g + 1) >> 1 : 0;
        const int unit = mc.mb0 * n_ib + ib;
        if (n_tiles > 0) {
            if constexpr (PP) {
                // Ping-pong: the wavefronts with g = 0 and those with g = 1 - the two wavefronts of every SIMD - run half a
                // step apart.  In one half step a wavefront multiplies (the matrix instructions of a K step with their
                // scaled accumulates and operand reads, nothing else: wide_tiles8), in the other it issues its loads,
                // waits for the batch before, and reads the weight fragments and factors of its next step; a barrier ends
                // each half step.  So on every SIMD one wavefront is at its memory instructions while the other has the
                // matrix pipe to itself (matrix and memory instructions of different wavefronts overlap completely; those
                // of one wavefront, or of two in the same phase, add up).
                //   half step 2 kb:     g = 0 multiplies step kb          g = 1 loads odd token tiles of step kb + 1
                //   half step 2 kb + 1: g = 0 loads weights and even      g = 1 multiplies step kb
                //                       token tiles of step kb + 2
                // Weights of step kb: ring slot kb & 1 (its fragments are in everybody's registers one half step before
                // it is refilled).  Token tiles: the even tiles of step kb are half 2 kb of a stream, the odd ones half
                // 2 kb + 1; half hh sits in quarter hh & 3 of the token region and is refilled with half hh + 4 one half
                // step after its use.  Every load is issued three half steps before its first use.
                const bool xs_chunk = s.xs_chunk != 0;
                const int row_a = xs_chunk ? 128 : 16;
                float *s_xs4 = &s_xs[0][0];   // per-step scales (not chunked): [half & 3][tile of the half][token]
                // this wavefront's two token tiles of its half: e = 2 w, 2 w + 1 (token tile 2 e + g)
                unsigned x_off[2][2], xs_off[2];
                bool x_live[2];
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int tt = 2 * (2 * w + j) + g;
                    x_live[j] = rfl(tt < n_tiles ? 1 : 0) != 0;   // (the same in all lanes; a scalar for the compiler too)
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const int tk = s_tok[tt * 16 + 8 * h + ld_row];
                        x_off[j][h] = (unsigned)(tk < 0 ? 0 : tk) * (unsigned)K + ld_chunk[h];
                    }
                    const int tk = s_tok[tt * 16 + n];
                    xs_off[j] = (unsigned)(tk < 0 ? 0 : tk) * (unsigned)nkb;
                }
                // weights (g = 0 only): all four tiles of pair w; tile a = (32-row group a / 2, gate | up a % 2)
                unsigned w_voff[2];
#pragma unroll
                for (int h = 0; h < 2; h++) w_voff[h] = (unsigned)((ib * 256 + w * 64 + ld_row) * p.w_rs) + ld_chunk[h];
                const uint8_t *wexp = p.w + (size_t)mc.e * p.N * K;
                const bool nt = mc.lone;
                // the wavefront's loads of step kn; returns how many instructions went out
                auto issue_batch = [&](int kn) {
                    int cnt = 0;
                    if (kn >= nkb) return cnt;
                    if (g == 0) {
#pragma unroll
                        for (int a = 0; a < 4; a++)
#pragma unroll
                            for (int h = 0; h < 2; h++) {
                                const uint8_t *src = wexp + (size_t)kn * p.w_ks + (size_t)((a >> 1) * 32 + h * 16 + 8 * (a & 1)) * p.w_rs;
                                uint8_t *dst = a_ring + (kn & 1) * kWStageA + w * 8192 + a * 2048 + h * 1024;
                                if (nt) dma16_sv<2>(src, w_voff[h], dst);
                                else dma16_sv<0>(src, w_voff[h], dst);
                                cnt++;
                            }
                    }
                    const int hh = 2 * kn + g;
                    uint8_t *xq = xbuf + (hh & 3) * 16384;
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        if (!x_live[j]) continue;
                        const int e = 2 * w + j;
#pragma unroll
                        for (int h = 0; h < 2; h++)
                            dma16_sv<0>(p.x + (size_t)kn * 128, x_off[j][h], xq + e * 2048 + h * 1024);
                        cnt += 2;
                        if (xs_chunk) {
                            if ((kn & 3) == 0) {
                                if (lane < 16) dma16_sv<0>(p.x_scale + kn, xs_off[j] * 4u, &s_xc[(kn >> 2) & 1][(2 * e + g) * 64]);
                                cnt++;
                            }
                        } else {
                            if (lane < 16) dma4_sv<0>(p.x_scale + kn, xs_off[j] * 4u, s_xs4 + (hh & 3) * 128 + e * 16);
                            cnt++;
                        }
                    }
                    return rfl(cnt);
                };
                v8i a[4];
                auto read_a = [&](int kb) {
                    const uint8_t *a_tiles = a_ring + (kb & 1) * kWStageA + w * 8192;
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        a[k] = cat(*reinterpret_cast<const v4i *>(a_tiles + k * 2048 + frag_lo),
                                   *reinterpret_cast<const v4i *>(a_tiles + k * 2048 + frag_hi));
                    // waited for here: a wait of the compiler's in the multiply phase would also cover the operand reads
                    // in flight there, which it does not know of
                    asm volatile("" ::"v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]));
                };
                const bool upper = nt_w > 4;
                v4i top_lo, top_hi;   // operands of the first tile of the next step, and its weight-block factors
                float top_f, top_sc0, top_sc1;
                v4f q_prod[kPpDepth];
                float q_fac[kPpDepth];
                wide_queue_clear(q_prod, q_fac);
                auto row_of = [&](int kb) {
                    return xs_chunk ? &s_xc[(kb >> 2) & 1][g * 64 + n * 4 + (kb & 3)] : s_xs4 + ((2 * kb + g) & 3) * 128 + n;
                };
                // before the barrier that starts a multiply phase: the step's weight-block factors
                auto read_sc = [&](int kb) {
                    top_sc0 = s_ws[0][kb];
                    top_sc1 = s_ws[1][kb];
                    asm volatile("" ::"v"(top_sc0), "v"(top_sc1));   // (as in read_a)
                };
                auto multiply = [&](int kb) {
                    if (nt_w > 0) {
                        wide_top_read<2048>(xbuf + ((2 * kb + g) & 3) * 16384, row_of(kb), row_a, frag_lo, frag_hi, upper, top_lo,
                                            top_hi, top_f);
                        wide_tiles8<2048, kPpDepth>(a, xbuf + ((2 * kb + g) & 3) * 16384, row_of(kb), row_a, top_sc0, top_sc1, acc,
                                                    frag_lo, frag_hi, upper, top_lo, top_hi, top_f, q_prod, q_fac);
                    }
                };
                clear_acc();
                if (g == 0) {
                    issue_batch(0);
                    const int c1 = issue_batch(1);
                    wait_pending(c1);
                    read_a(0);
                    read_sc(0);
                    lds_barrier();
                    for (int kb = 0; kb < nkb; kb++) {
                        multiply(kb);
                        lds_barrier();
                        const int cnt = issue_batch(kb + 2);
                        wait_pending(cnt);   // the loads of step kb + 1 have landed
                        if (kb + 1 < nkb) {
                            read_a(kb + 1);
                            read_sc(kb + 1);
                        }
                        lds_barrier();
                    }
                } else {
                    issue_batch(0);
                    lds_barrier();
                    for (int kb = 0; kb < nkb; kb++) {
                        const int cnt = issue_batch(kb + 1);
                        wait_pending(cnt);   // the odd token tiles of step kb have landed
                        read_a(kb);          // (its weights: g = 0 waited for them before the barrier)
                        read_sc(kb);
                        lds_barrier();
                        multiply(kb);
                        lds_barrier();
                    }
                }
                wide_queue_drain(acc, q_prod, q_fac);
            } else {
            // token-tile gather: wavefront v loads tiles v and v + 8
            const bool xs_chunk = s.xs_chunk != 0;
            const int row_a = xs_chunk ? 128 : 64, row_b = xs_chunk ? 0 : -240;
            unsigned x_off[2][2], xs_off[2];
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int tk = s_tok[(wave + 8 * j) * 16 + 8 * h + ld_row];
                    x_off[j][h] = (unsigned)(tk < 0 ? 0 : tk) * (unsigned)K + ld_chunk[h];
                }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int tk = s_tok[(wave + 8 * j) * 16 + n];
                xs_off[j] = (unsigned)(tk < 0 ? 0 : tk) * (unsigned)nkb;
            }
            // Weight rows of the pair: tile a = (32-row group a / 2, gate | up a % 2); matrix row r of the tile is slab
            // row group * 32 + (r / 8) * 16 + r % 8 (+ 8 for up), so load h of a tile covers slab rows ... + 16 h +
            // lane / 8.  Wavefront (w, g) loads tiles 2g and 2g + 1 of pair w.
            unsigned w_off[2][2];
#pragma unroll
            for (int up = 0; up < 2; up++)
#pragma unroll
                for (int h = 0; h < 2; h++)
                    w_off[up][h] =
                        (unsigned)((ib * 256 + w * 64 + g * 32 + ld_row + h * 16 + 8 * up) * p.w_rs) + ld_chunk[h];
            const uint8_t *wexp = p.w + (size_t)mc.e * p.N * K;
            const bool nt = mc.lone;
            // Loads of a step, in three groups that are issued - and waited for - separately:
            //   A    the wavefront's 4 weight tile halves
            //   XLO  token tile `wave` (tiles 0..7: the first half of a step) and its scales
            //   XHI  token tile `wave + 8` and its scales
            // `issued` counts this wavefront's load instructions; a group's mark is the count right after its last one.
            int issued = 0;
            auto issue_a_op = [&](int kb, int stage, int i) {   // i < 4
                const int up = i >> 1, h = i & 1;
                const uint8_t *src = wexp + (size_t)kb * p.w_ks;
                uint8_t *dst = a_ring + stage * kWStageA + w * 8192 + (2 * g + up) * 2048 + h * 1024;
                if (nt) dma16_sv<2>(src, w_off[up][h], dst);
                else dma16_sv<0>(src, w_off[up][h], dst);
                issued++;
            };
            auto issue_x_op = [&](int kb, int stage, int j, int i) {   // i < 3: two tile halves, the scales
                if (wave + 8 * j >= n_tiles) return;
                if (i < 2) {
                    dma16_sv<0>(p.x + (size_t)kb * 128, x_off[j][i],
                                xbuf + stage * kWStageX + (wave + 8 * j) * 2048 + i * 1024);
                } else if (xs_chunk) {
                    // steps kb .. kb + 3 of the tile's 16 tokens, 16 bytes per token, with the loads of step kb & ~3
                    if (kb & 3) return;
                    if (lane < 16) dma16_sv<0>(p.x_scale + kb, xs_off[j] * 4u, &s_xc[(kb >> 2) & 1][(wave + 8 * j) * 64]);
                } else if (lane < 16) {
                    dma4_sv<0>(p.x_scale + kb, xs_off[j] * 4u, &s_xs[stage][wave * 32 + 16 * j]);
                }
                issued++;
            };
            clear_acc();
            // Step kb reads stage kb & 1.  Its weight tiles are in registers right after the step's first barrier, so the
            // weight stage is refilled (step kb + 2) behind a second barrier; the first half of the token stage is
            // refilled behind a third one in the middle of the step, the second half from the start of the next step.
            // The loads go out one at a time between the matrix instructions of the token tiles: a load instruction
            // holds its wavefront until the memory pipeline takes it, and a burst of them holds the matrix work up.
            int mark_a[2], mark_lo[2], mark_hi[2];
            for (int i = 0; i < 4; i++) issue_a_op(0, 0, i);
            mark_a[0] = issued;
            for (int i = 0; i < 3; i++) issue_x_op(0, 0, 0, i);
            mark_lo[0] = issued;
            for (int i = 0; i < 3; i++) issue_x_op(0, 0, 1, i);
            mark_hi[0] = issued;
            if (nkb > 1) {
                for (int i = 0; i < 4; i++) issue_a_op(1, 1, i);
                mark_a[1] = issued;
                for (int i = 0; i < 3; i++) issue_x_op(1, 1, 0, i);
                mark_lo[1] = issued;
            }
            for (int kb0 = 0; kb0 < nkb; kb0 += 2) {
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int kb = kb0 + h;
                    if (kb < nkb) {
                        wait_pending(issued - mark_a[h]);
                        lds_barrier();   // everybody's weight tiles of step kb have landed; step kb - 1 is done with
                        v8i a[4];
                        {
                            const uint8_t *a_tiles = a_ring + h * kWStageA + w * 8192;
#pragma unroll
                            for (int k = 0; k < 4; k++)
                                a[k] = cat(*reinterpret_cast<const v4i *>(a_tiles + k * 2048 + frag_lo),
                                           *reinterpret_cast<const v4i *>(a_tiles + k * 2048 + frag_hi));
                        }
                        wait_pending(issued - mark_lo[h]);
                        lds_barrier();   // weight fragments are in registers everywhere; token tiles 0..7 have landed
                        const float sc0 = s_ws[0][kb], sc1 = s_ws[1][kb];
                        const float *row = xs_chunk ? &s_xc[(kb >> 2) & 1][g * 64 + n * 4 + (kb & 3)] : &s_xs[h][row_off];
                        // loads of the step, five or so per half: weights of step kb + 2 (halves 0, 1 | 2, 3), the
                        // second token half of step kb + 1 | the first token half of step kb + 2
                        wide_half<0, 4096>(a, xbuf + h * kWStageX + g * 2048, row, row_a, row_b, sc0, sc1, acc, frag_lo,
                                     frag_hi, nt_w, [&](int t) {
                                         if (kb + 2 < nkb && (t & 1) == 0) issue_a_op(kb + 2, h, t >> 1);
                                         if (kb + 1 < nkb) {
                                             if (t & 1) issue_x_op(kb + 1, h ^ 1, 1, t >> 1);
                                             if (t == 3) issue_x_op(kb + 1, h ^ 1, 1, 2);
                                         }
                                     });
                        mark_hi[h ^ 1] = issued;
                        wait_pending(issued - mark_hi[h]);
                        lds_barrier();   // everybody is done with token tiles 0..7; tiles 8..15 have landed
                        wide_half<4, 4096>(a, xbuf + h * kWStageX + g * 2048, row, row_a, row_b, sc0, sc1, acc, frag_lo,
                                     frag_hi, nt_w, [&](int t) {
                                         if (kb + 2 < nkb) {
                                             if ((t & 1) == 0) issue_a_op(kb + 2, h, 2 + ((t - 4) >> 1));
                                             if (t == 6) mark_a[h] = issued;
                                             if (t & 1) issue_x_op(kb + 2, h, 0, (t - 4) >> 1);
                                             if (t == 7) issue_x_op(kb + 2, h, 0, 2);
                                         }
                                     });
                        mark_lo[h] = issued;
                    }
                }
            }
            }
            wait_vmcnt<0>();

            // SwiGLU, per-token amax over the slice's 128 columns, FP8 requant into operand tiles
#pragma unroll
            for (int t = 0; t < 8; t++) {
                if (t < nt_w) {
                    float mx = 0.f;
#pragma unroll
                    for (int pr = 0; pr < 2; pr++)
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const float a = swiglu_bf16(acc[2 * pr][t][j], acc[2 * pr + 1][t][j]);
                            acc[2 * pr][t][j] = a;
                            mx = fmaxf(mx, fabsf(a));
                        }
                    mx = fmaxf(mx, __shfl_xor(mx, 16));
                    mx = fmaxf(mx, __shfl_xor(mx, 32));
                    if (q == 0) s_amax[w][(2 * t + g) * 16 + n] = mx;
                }
            }
            __syncthreads();
#pragma unroll
            for (int t = 0; t < 8; t++) {
                if (t < nt_w) {
                    const int tt = 2 * t + g;
                    float mx = kAmaxFloor;
#pragma unroll
                    for (int wv = 0; wv < 4; wv++) mx = fmaxf(mx, s_amax[wv][tt * 16 + n]);
                    const float s_a = mx / kFp8Max;
                    const size_t gt = (size_t)ib * s.n_tiles_total + (size_t)mc.mb0 * s.tpb + tt;
                    uint8_t *tile = s.aqs + gt * 2048;
#pragma unroll
                    for (int pr = 0; pr < 2; pr++) {
                        const uint32_t packed =
                            pack_fp8x4(clamp_fp8(acc[2 * pr][t][0] / s_a), clamp_fp8(acc[2 * pr][t][1] / s_a),
                                       clamp_fp8(acc[2 * pr][t][2] / s_a), clamp_fp8(acc[2 * pr][t][3] / s_a));
                        // columns w*32 + pr*16 + 4q .. +3 of token n: chunk w*2 + pr of the row, bytes 4q .. 4q+3 in it
                        stg32_agent(tile, (uint32_t)(n * 128 + 16 * ((w * 2 + pr) ^ f_n) + 4 * q), packed);
                    }
                    if (w == 0 && q == 0) stg32_agent(s.sas + gt * 16, 4u * n, __builtin_bit_cast(uint32_t, s_a));
                }
            }
            wait_vmcnt<0>();
        }
        __syncthreads();
        if (tid == 0) store_agent(&s.flag[unit], epoch);
    };

    // ---- DOWN item: column groups [cs * gps, (cs + 1) * gps) of macro block m, all slices ---------------------------
    // 64 output columns per pair of wavefronts and step.  Pair w takes the slab's groups w, w + 4, ...; its two
    // wavefronts split the token tiles as above and each loads two of the four w2 tiles of a step.  Matrix row r of tile
    // k is output column c0 + 16 (r / 4) + 4 k + r % 4, so lane (n, q) collects columns c0 + 16 q .. c0 + 16 q + 15 of
    // token n over the four tiles.  Load h of a tile: rows 8h + lane / 8.
    auto down_item = [&](int m, int cs, auto resident_c) {
        constexpr bool RESIDENT = decltype(resident_c)::value;
        const Macro mc = macro_of(m);
        load_rows(mc, true, cs);
        for (int i = tid; i < (K >> 7) * n_ib; i += THREADS) s_w2s[i] = p.w2_scale[(size_t)mc.e * (K >> 7) * n_ib + i];
        const bool nt = mc.lone;

        const int n_groups = K >> 6;
        const int g0 = cs * s.gps;
        const int g1 = g0 + s.gps < n_groups ? g0 + s.gps : n_groups;
        const int span = g1 - g0;
        int my_groups = (span - w + 3) >> 2;                      // the slab's groups w, w + 4, ... (none: 0)
        my_groups = my_groups > 0 ? my_groups : 0;
        const int n_steps = ((span + 3) >> 2) * n_ib;             // (group, slice) steps of the longest pair, slice-minor
        const uint8_t *w2exp = p.w2 + (size_t)mc.e * K * I;
        unsigned w2_off[2][2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int h = 0; h < 2; h++)
                w2_off[kk][h] =
                    (unsigned)((16 * (lane >> 5) + (ld_row & 3) + 32 * h + 4 * (2 * g + kk)) * p.w2_rs) + ld_chunk[h];
        int lg = 0, lib = 0;   // (group index, slice) of the next step to load
        auto group_of = [&](int i) {   // i-th group of this pair, clamped into the slab for loads past its end
            int grp = g0 + w + 4 * (i < my_groups ? i : my_groups - 1);
            grp = grp < g0 ? g0 : grp;
            return grp < g1 ? grp : g1 - 1;
        };
        const size_t tile0 = (size_t)mc.mb0 * s.tpb;
        int n_tiles = 0;
        // operation i of the step (lg, lib) into ring stage `stage`: 4 w2 tile halves; streamed: 4 requantised tile
        // halves of slice lib and their scales
        auto issue_op = [&](int stage, int i) {
            if (i < 4) {
                const int kk = i >> 1, h = i & 1;
                const int c0 = group_of(lg) << 6;
                const uint8_t *src = w2exp + (size_t)c0 * p.w2_rs + (size_t)lib * p.w2_ks;
                uint8_t *dst = a_ring + stage * kWStageA + w * 8192 + (2 * g + kk) * 2048 + h * 1024;
                if (nt) dma16_sv<2>(src, w2_off[kk][h], dst);
                else dma16_sv<0>(src, w2_off[kk][h], dst);
            } else if (!RESIDENT) {
                if (i < 8) {
                    const int j = (i - 4) >> 1, h = i & 1;
                    if (wave + 8 * j < n_tiles)
                        dma16_sv<16>(s.aqs + ((size_t)lib * s.n_tiles_total + tile0 + wave + 8 * j) * 2048 + h * 1024,
                                     (unsigned)(lane * 16), xbuf + stage * kWStageX + (wave + 8 * j) * 2048 + h * 1024);
                } else if (lane < 32) {
                    const int tt = wave + 8 * ((lane >> 4) & 1);
                    dma4_sv<16>(s.sas + ((size_t)lib * s.n_tiles_total + tile0) * 16,
                                (unsigned)((tt < n_tiles ? tt : 0) * 16 + n) * 4u, &s_xs[stage][wave * 32]);
                }
            }
        };
        auto advance = [&]() {
            lib++;
            if (lib == n_ib) {
                lib = 0;
                lg++;
            }
        };
        // the weights do not depend on the up/gate phase: the first step's go out before the wait
#pragma unroll
        for (int i = 0; i < 4; i++) issue_op(0, i);
        if (wave == 0) spin_all_ge(&s.flag[mc.mb0 * n_ib], n_ib, epoch, s.ctl);
        __syncthreads();
        n_tiles = tiles_of();
        const int nt_w = n_tiles > g ? (n_tiles - g + 1) >> 1 : 0;
        if (RESIDENT) {
            // the requantised tiles of all slices and their scales come from scratch into LDS: [slice][tile]
            for (int i = wave; i < n_ib * kWTiles; i += 8) {
                const int ib = i >> 4, tt = i & 15;
                if (tt < n_tiles) {
                    const uint8_t *src = s.aqs + ((size_t)ib * s.n_tiles_total + tile0 + tt) * 2048;
                    dma16_sv<16>(src, (unsigned)(lane * 16), xbuf + i * 2048);
                    dma16_sv<16>(src + 1024, (unsigned)(lane * 16), xbuf + i * 2048 + 1024);
                }
            }
            for (int i = tid; i < n_ib * kWRows; i += THREADS) {
                const int ib = i >> 8, r = i & 255;
                const int tt = r >> 4;
                if (tt < n_tiles) {
                    const int bits = load_agent(reinterpret_cast<const int *>(
                        &s.sas[((size_t)ib * s.n_tiles_total + tile0 + tt) * 16 + (r & 15)]));
                    s_xs[ib][(tt & 7) * 32 + (tt >> 3) * 16 + (r & 15)] = __builtin_bit_cast(float, bits);
                }
            }
        } else {
#pragma unroll
            for (int i = 4; i < 9; i++) issue_op(0, i);
        }
        advance();
        wait_vmcnt<0>();
        clear_acc();
        int cg = 0, cib = 0;
        for (int s0 = 0; s0 < n_steps; s0 += 2) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                if (s0 + h < n_steps) {
                    lds_barrier();
                    const int c0 = group_of(cg) << 6;
                    const float ws2 = s_w2s[(c0 >> 7) * n_ib + cib];
                    const bool more = s0 + h + 1 < n_steps;
                    const uint8_t *b_tiles = RESIDENT ? xbuf + cib * kWStageX + g * 2048 : xbuf + h * kWStageX + g * 2048;
                    const float *row = RESIDENT ? &s_xs[cib][row_off] : &s_xs[h][row_off];
                    wide_step(a_ring + h * kWStageA + w * 8192, b_tiles, row, ws2, ws2, acc, frag_lo, frag_hi, nt_w,
                              [&](int t) {
                                  if (more) {
                                      if (RESIDENT) {
                                          if (t < 4) issue_op(h ^ 1, t);
                                      } else if (t == 0) {
                                          issue_op(h ^ 1, 0);
                                          issue_op(h ^ 1, 4);
                                          issue_op(h ^ 1, 8);
                                      } else if (t < 4) {
                                          issue_op(h ^ 1, t);
                                          issue_op(h ^ 1, t + 4);
                                      }
                                  }
                              });
                    if (more) advance();
                    // the next step's loads have landed before any result store is issued: the stores are then only
                    // waited for a whole step later
                    wait_vmcnt<0>();
                    cib++;
                    if (cib == n_ib) {
#pragma unroll
                        for (int t = 0; t < 8; t++) {
                            if (t < nt_w) {
                                const int r = (2 * t + g) * 16 + n;
                                const int slot = s_tok[r];
                                if (slot >= 0 && cg < my_groups) {
                                    const float tw = s_tw[r];
                                    uint16_t *yp = s.y + (size_t)slot * K + c0 + 16 * q;
#pragma unroll
                                    for (int half = 0; half < 2; half++) {
                                        const v4f lo = acc[2 * half][t] * tw, hi = acc[2 * half + 1][t] * tw;
                                        v4i o;
                                        o.x = (int)pack_bf16x2(lo[0], lo[1]);
                                        o.y = (int)pack_bf16x2(lo[2], lo[3]);
                                        o.z = (int)pack_bf16x2(hi[0], hi[1]);
                                        o.w = (int)pack_bf16x2(hi[2], hi[3]);
                                        *reinterpret_cast<v4i *>(yp + 8 * half) = o;
                                    }
                                }
#pragma unroll
                                for (int a = 0; a < 4; a++) acc[a][t] = (v4f){0.f, 0.f, 0.f, 0.f};
                            }
                        }
                        cib = 0;
                        cg++;
                    }
                }
            }
        }
        wait_vmcnt<0>();
    };

    // ---- item loop ------------------------------------------------------------------------------------------------
    // Queue qq holds macro blocks [qq * per_q, ...) as items: the up/gate items of `lag` blocks first, then alternately
    // the up/gate items of block lag + r and the down items of block r, at the end the down items of the last `lag`
    // blocks.  A down item waits for the flags of its block's up/gate items, which are EARLIER in the same queue:
    // whoever took them is running and waits for nothing later, so the queues drain with any number of resident
    // workgroups.  A workgroup that finds its queue empty moves on to the next one.
    auto blocks_of = [&](int qq) {
        const int left = n_macro - qq * per_q;
        return left < 0 ? 0 : (left < per_q ? left : per_q);
    };
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
        const int item = rfl(s_item[0]);
        const int qi = rfl(s_item[1]);
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
        } else if (n_ib <= kWResidentIb) {
            down_item(qi * per_q + down / per_down, down % per_down, std::true_type());
        } else {
            down_item(qi * per_q + down / per_down, down % per_down, std::false_type());
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

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

hipError_t allow_dynamic_lds()
{
    static std::mutex mu;
    static bool done[64];
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    std::lock_guard<std::mutex> lock(mu);
    if (dev >= 0 && dev < 64 && done[dev]) return hipSuccess;
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(moe_wide_kernel<false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kWDynLds);
    if (err == hipSuccess)
        err = hipFuncSetAttribute(reinterpret_cast<const void *>(moe_wide_kernel<true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kWDynLds);
    if (err == hipSuccess && dev >= 0 && dev < 64) done[dev] = true;
    return err;
}

// 64-column groups per DOWN item: about 8 * stages ring steps (a step is four groups x one slice), a multiple of 4 so
// that every pair of wavefronts gets the same number of groups
int groups_per_item(int n_ib, int stages)
{
    const int e = tunable(kTunTileGps, 0);
    if (e > 0) return (e + 3) / 4 * 4;
    return 4 * ((8 * stages + n_ib - 1) / n_ib);
}

}  // namespace

bool wide_supported(int top_k, int M, int K, int N, int E, int sorted_num, int block_m)
{
    (void)E;
    const int n_ib = N / 256;
    const int64_t n_mb = ((int64_t)sorted_num + block_m - 1) / block_m;
    return block_m > 32 && K <= 128 * kWMaxKb && (K / 128) * n_ib <= kWMaxW2s && (int64_t)M * top_k <= kMaxSlots &&
           n_mb * n_ib <= kMaxUnits && (int64_t)N * K < ((int64_t)1 << 31) && (int64_t)M * K < ((int64_t)1 << 32);
}

size_t wide_workspace_bytes(int top_k, int M, int K, int N, int E, int sorted_num, int block_m)
{
    (void)E;
    const size_t n_mb = ((size_t)sorted_num + block_m - 1) / block_m;
    const size_t tiles = n_mb * ((block_m + 15) / 16);
    return align_up(kPrefixBytes) + align_up((size_t)M * top_k * K * sizeof(uint16_t)) +
           align_up((size_t)(N / 256) * tiles * 2048) + align_up((size_t)(N / 256) * tiles * 16 * sizeof(float)) +
           align_up((n_mb + 1) * 4 * sizeof(int));
}

hipError_t launch_wide(const MoeParams &p, int stages, void *workspace, hipStream_t stream)
{
    uint8_t *ws = static_cast<uint8_t *>(workspace);
    WideParams s;
    s.p = p;
    s.n_ib = p.N / 256;
    s.nkb = p.K / 128;
    s.n_mb_max = (p.sorted_num + p.block_m - 1) / p.block_m;
    s.blocks_per_macro = kWRows / p.block_m;
    s.tpb = (p.block_m + 15) / 16;
    s.n_tiles_total = s.n_mb_max * s.tpb;
    size_t off = align_up(kPrefixBytes);
    s.ctl = reinterpret_cast<StreamCtl *>(ws);
    s.flag = reinterpret_cast<int *>(ws + kOffFlag);
    s.live = reinterpret_cast<int *>(ws + kOffLive);
    s.y = reinterpret_cast<uint16_t *>(ws + off);
    off += align_up((size_t)p.M * p.top_k * p.K * sizeof(uint16_t));
    s.aqs = ws + off;
    off += align_up((size_t)s.n_ib * s.n_tiles_total * 2048);
    s.sas = reinterpret_cast<float *>(ws + off);
    off += align_up((size_t)s.n_ib * s.n_tiles_total * 16 * sizeof(float));
    s.plan = reinterpret_cast<int *>(ws + off);
    s.gps = groups_per_item(s.n_ib, stages);
    s.n_cs = ((p.K >> 6) + s.gps - 1) / s.gps;
    s.lag = tunable(kTunTileLag, 32);
    s.w_nt = tunable(kTunTileNt, -1);
    s.xs_chunk = (s.nkb % 4 == 0 && reinterpret_cast<uintptr_t>(p.x_scale) % 16 == 0) ? 1 : 0;
    if (s.lag < 1) s.lag = 1;
    hipError_t err = allow_dynamic_lds();
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(moe_wide_plan_kernel, dim3(1), dim3(1024), 0, stream, s);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            return 256;
        return n;
    }();
    const int64_t items = (int64_t)s.n_mb_max * (s.n_ib + s.n_cs);
    int grid = tunable(kTunTileGrid, cus);
    if (grid > items) grid = (int)((items + 7) / 8 * 8);
    if (grid < 8) grid = 8;
    // The ping-pong up/gate loop multiplies a wavefront's token tiles in blocks of four, dead ones included, and so pays
    // off when an expert's rows fill its 256-row blocks: by default it is used from 192 routed rows per expert on
    // average (measured: 2 - 3 % on whole calls there; slower below).  The result does not depend on the choice.
    const int pp_default = (int64_t)p.M * p.top_k >= (int64_t)192 * p.E ? 1 : 0;
    if (tunable(kTunWidePp, pp_default) != 0)
        hipLaunchKernelGGL(moe_wide_kernel<true>, dim3((unsigned)grid), dim3(512), kWDynLds, stream, s);
    else
        hipLaunchKernelGGL(moe_wide_kernel<false>, dim3((unsigned)grid), dim3(512), kWDynLds, stream, s);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    RowsReduce r;
    r.p = p;
    r.ctl = s.ctl;
    r.live = s.live;
    r.y = s.y;
    return launch_rows_reduce(r, stream);
}

}  // namespace alpha_moe
