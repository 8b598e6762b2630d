// Shared device helpers and launch interfaces of the gfx950 fused W8A8 MoE kernels.
//
// Conventions used by every kernel in this directory:
//   * v_mfma_f32_16x16x128_f8f6f4 with WEIGHT rows as the A operand and TOKENS as the B operand; one instruction
//     contracts exactly one 128-wide scale block, so block scales multiply its fp32 result.
//   * Operand lane layout: lane = (m = lane % 16, q = lane / 16); the lane feeds row/column m with the 32 bytes
//     [16q, 16q+16) ++ [64+16q, 64+16q+16) of the 128-byte K block ("chunk q" and "chunk q+4" of eight 16-byte
//     chunks).  Any K permutation is legal as long as A and B use the same one.
//   * Accumulator lane layout: register j of lane (n, q) is (row 4q + j, token n).
//   * Gate/up pairing under the interleave-8 weight layout: the gate MFMA of a 32-row group takes the 8+8 gate rows
//     of its two 16-row chunks, the up MFMA their up rows, so accumulator j of a lane is gate/up of the SAME
//     intermediate column and a lane owns 4 consecutive columns.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/alpha_moe_hip.h"
#include "alpha_moe_tuning.h"

namespace alpha_moe {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr float kFp8Max = 448.0f;
constexpr float kAmaxFloor = 1e-10f;
constexpr int kMaxKBlocks = 512;     // K <= 65536
constexpr int kLdsRowStride = 144;   // 128 FP8 + 16 pad: dword writes of 16 tokens x 4 quads hit 64 distinct banks

struct MoeParams {
    const uint8_t *x;
    const float *x_scale;
    const uint8_t *w;
    const float *w_scale;
    const uint8_t *w2;
    const float *w2_scale;
    uint16_t *out;              // [M, K] bf16
    float *acc;                 // [M, K] fp32 scratch (direct kernel only)
    const int32_t *sorted_ids;
    const int32_t *expert_ids;
    const int32_t *ntpp;
    const float *topk_w;
    int top_k, M, K, N, E, sorted_num, block_m;
    float scaling;
    int overwrite;              // 1: out = bf16(sum), whatever out held; 0: out = bf16(out + sum)
    // Byte strides of the two weight tensors inside one expert: from one row to the next, and from one 128-byte K
    // block of a row to the next.  The operator's layout ([N][K] and [K][I] row-major) has (K, 128) and (I, 128); the
    // pre-packed layout ([K/128][N][128] and [I/128][K][128]: a K block of consecutive rows is contiguous) has
    // (128, N * 128) and (128, K * 128).
    size_t w_rs, w_ks, w2_rs, w2_ks;
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

// SwiGLU on bf16-rounded gate/up, result rounded to bf16 (the reference keeps all three in bf16,
// fused_moe_w8a8_up_down_acc.cu:76-79,919-946)
__device__ __forceinline__ float swiglu_bf16(float gate, float up)
{
    const float g = round_bf16(gate);
    const float u = round_bf16(up);
    return round_bf16(g / (1.0f + __expf(-g)) * u);
}

__device__ __forceinline__ void atomic_add_f32(float *addr, float v)
{
    typedef float __attribute__((address_space(1))) * gptr;
    __builtin_amdgcn_global_atomic_fadd_f32(reinterpret_cast<gptr>(reinterpret_cast<uintptr_t>(addr)), v);
}

// ---- memory helpers shared by the persistent kernels ---------------------------------------------------------
typedef const void __attribute__((address_space(1))) * gptr_t;
typedef void __attribute__((address_space(3))) * lptr_t;

// Memory -> LDS without passing VGPRs: lane l's 16 bytes land at lds + 16 l; the global address is per lane.
// AUX: 0 default, 2 non-temporal (measured on MI355X: weight streams reach 6.9 TB/s with it, 3.4 TB/s without), 16 agent
// scope (sc1: for data another workgroup wrote during this launch).
template <int AUX>
__device__ __forceinline__ void dma16(const void *g, void *lds)
{
    __builtin_amdgcn_global_load_lds((gptr_t)(uintptr_t)g, (lptr_t)(uint32_t)(uintptr_t)lds, 16, 0, AUX);
}
// The same for 4 bytes per lane.
__device__ __forceinline__ void dma4(const void *g, void *lds)
{
    __builtin_amdgcn_global_load_lds((gptr_t)(uintptr_t)g, (lptr_t)(uint32_t)(uintptr_t)lds, 4, 0, 0);
}

// "At most N of this wavefront's vector-memory operations are still outstanding".  The kernels count their
// direct-to-LDS loads themselves.
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
    __builtin_amdgcn_sched_barrier(0);   // nothing that consumes the awaited data may be scheduled above the wait
}
// all of this wavefront's vector-memory operations (loads, stores, direct-to-LDS loads) have completed
__device__ __forceinline__ void drain_vmem() { wait_vmcnt<0>(); }

// all of this wavefront's LDS operations (reads into registers included) have completed
__device__ __forceinline__ void wait_lds_reads()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// Workgroup barrier that waits for this wavefront's LDS operations only (__syncthreads would also drain every
// outstanding global load, and with them the prefetches in flight).
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// Agent-scope (sc1) accesses for data that crosses workgroups - and XCDs, whose L2s are not coherent with each other -
// inside one launch.  The 16- and 4-byte ones are raw buffer operations on a buffer that starts at a wavefront-uniform
// base and has no end, addressed by a 32-bit per-lane byte offset: the cache-policy bits are an argument of the builtin
// (no flat or global builtin takes them), and unlike inline asm the compiler sees these accesses - it places the wait
// before the first use of a loaded register, keeps that register live until then, and honours the hazard between a
// wide store and the next write of its data registers.  drain_vmem() before telling anybody about what was stored;
// acquire_fence() between seeing another workgroup's flag and loading what it published.
typedef unsigned v4u __attribute__((ext_vector_type(4)));
constexpr int kAuxAgent = 16;   // sc1
__device__ __forceinline__ __amdgpu_buffer_rsrc_t agent_buffer(const void *uniform_base)
{
    const uint64_t v = reinterpret_cast<uint64_t>(uniform_base);
    const uint64_t u = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32)) << 32) |
                       (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>(u), 0, -1, 0x00020000);
}
__device__ __forceinline__ v4i ldg128_agent(const void *uniform_base, uint32_t byte_off)
{
    return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(agent_buffer(uniform_base), (int)byte_off, 0, kAuxAgent));
}
__device__ __forceinline__ void stg32_agent(void *uniform_base, uint32_t byte_off, uint32_t v)
{
    __builtin_amdgcn_raw_buffer_store_b32(v, agent_buffer(uniform_base), (int)byte_off, 0, kAuxAgent);
}
__device__ __forceinline__ void stg128_agent(void *uniform_base, uint32_t byte_off, v4f v)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), agent_buffer(uniform_base), (int)byte_off, 0, kAuxAgent);
}
// nothing that reads memory may be moved by the compiler from behind this point to before it
__device__ __forceinline__ void acquire_fence() { asm volatile("" ::: "memory"); }
__device__ __forceinline__ int load_agent(const int *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_agent(int *p, int v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- workspace prefix shared by the kernel families --------------------------------------------------------
// The first kPrefixBytes of the workspace are zero-initialised by the caller once and maintained by the kernels:
// counters return to zero by themselves, flags are stamped with a launch epoch that grows by one per launch and is
// compared modulo 2^32 (reached()), so it may wrap.  Its size does not depend on the problem, so calls of different
// sizes can share one buffer.
constexpr int kMaxUnits = 1 << 16;   // most (row block, slice) units of one streaming launch
constexpr int kMaxSlots = 1 << 18;   // most (token, slot) rows whose results go through per-slot rows

struct StreamCtl {
    int head;        // streaming kernel: next work item
    int done;        // streaming kernel: workgroups that have left
    int epoch;       // completed launches on this workspace (any kernel family)
    int pad_e;
    int fin_done;    // tile kernels: reduce-kernel workgroups that have left
    int tile_done;   // tile kernel: workgroups that have left
    int pad0[2];
    int tile_head[8];   // tile kernel: next work item of each of the eight queues
    int pad1a[16];
    // a 128-byte line of its own: idle workgroups poll it while the others still fetch items through `head`
    int down_done;   // streaming kernel: finished DOWN items of this launch (+ kExpiredBit after an expired wait)
    int error;       // sticky: a bounded wait ran out (word kErrorWord of the workspace); read with the same poll
    int pad1[30];
};
constexpr int kErrorWord = 33;
static_assert(sizeof(StreamCtl) == 256, "control block is one 256-byte line group");
static_assert(offsetof(StreamCtl, error) == kErrorWord * sizeof(int) && offsetof(StreamCtl, down_done) % 128 == 0,
              "the error word sits right behind the DOWN counter, on that counter's line");

constexpr size_t kOffArrive = 256;
constexpr size_t kOffFlag = kOffArrive + sizeof(int) * kMaxUnits;
constexpr size_t kOffLive = kOffFlag + sizeof(int) * kMaxUnits;
constexpr size_t kPrefixBytes = kOffLive + sizeof(int) * kMaxSlots;

// Bounded waits between workgroups: ~4M polls with a sleep between them, i.e. seconds, then the sticky error word of
// the control block instead of a hang.  The sleep grows from 0.1 us to 0.9 us: a hundred workgroups polling one address
// every 0.2 us keep that L2 channel busy enough to slow the loads of the workgroups still streaming weights threefold
// (measured).
// "a >= b" for counters and epochs that wrap around: true while a is at most 2^31 - 1 steps ahead of b
__device__ __forceinline__ bool reached(int a, int b) { return (int)((unsigned)a - (unsigned)b) >= 0; }

// A whole wavefront, `count` <= 64 consecutive flags, one per lane: every poll is ONE load, so the wait costs one round
// trip however many flags there are.
// `also`: a counter that other workgroups are (or will be) waiting on; an expiry sets kExpiredBit in it (an OR: several
// wavefronts of a workgroup may expire together and must not cancel each other), so that they stop waiting and learn
// about the expiry from the very word they poll.
constexpr int kExpiredBit = 1 << 30;
__device__ __noinline__ inline void spin_all_ge(const int *addr, int count, int target, StreamCtl *ctl,
                                                int *also = nullptr)
{
    const int lane = threadIdx.x & 63;
    for (int it = 0; it < (1 << 22); it++) {
        const int v = lane < count ? load_agent(addr + lane) : target;
        if (__all(reached(v, target))) {
            acquire_fence();
            return;
        }
        if (it < 16) __builtin_amdgcn_s_sleep(4);
        else __builtin_amdgcn_s_sleep(32);
    }
    if (lane == 0) {
        store_agent(&ctl->error, 1);
        if (also) __hip_atomic_fetch_or(also, kExpiredBit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- tuning overrides (experiments and tests) ---------------------------------------------------------------
// Read from the environment ONCE, when the library is first used, and changed afterwards only through
// alpha_moe_set_tunable(): no launch ever calls getenv.  A value of kTunableUnset means "the library decides".
constexpr int kTunableUnset = INT32_MIN;
enum Tunable {
    kTunPath,          // ALPHA_MOE_PATH: 1 direct, 2 stream, 3 tile (where the family applies)
    kTunStrictQueue,   // ALPHA_MOE_STRICT_QUEUE: 0 hands the first gridDim.x items of the streaming kernel out by index
    kTunKbpi,          // ALPHA_MOE_KBPI: K blocks per UP item of the streaming kernel
    kTunTpi,           // ALPHA_MOE_TPI: 16-column tiles per DOWN item of the streaming kernel
    kTunLag,           // ALPHA_MOE_LAG: row blocks between a block's UP and DOWN items in the streaming queue
    kTunGrid,          // ALPHA_MOE_GRID: workgroups of the streaming kernel
    kTunTileGps,       // ALPHA_MOE_TILE_GPS: 64-column groups per DOWN item of the tile kernel
    kTunTileLag,       // ALPHA_MOE_TILE_LAG
    kTunTileGrid,      // ALPHA_MOE_TILE_GRID
    kTunTileNt,        // ALPHA_MOE_TILE_NT: non-temporal weight loads 1 always, 0 never
    kTunWidePp,        // ALPHA_MOE_WIDE_PP: up/gate items of the wide kernel with the wavefronts of a SIMD half a step apart
    kTunCount
};
int tunable(Tunable which, int dflt);   // the override if one is set, else dflt

// ---- host-side launchers, one per kernel family (each in its own translation unit) -------------------------

// One workgroup per (block of block_m sorted rows, 128-column intermediate slice), weights HBM -> VGPR.
// Any block_m in 8..128.  Adds into p.acc (M*K floats, cleared by launch_zero_acc first); launch_finalize then
// rounds the sums into p.out.
hipError_t launch_zero_acc(const MoeParams &p, hipStream_t stream);
hipError_t launch_direct(const MoeParams &p, int warp_n, int stages, hipStream_t stream);
hipError_t launch_finalize(const MoeParams &p, hipStream_t stream);   // out = bf16(out + acc), or bf16(acc)

// Persistent work-queue kernel for decode-sized batches (block_m <= 32 and bounded sizes): split-K up items ->
// SwiGLU/requant -> column-slab down items -> per-token reduction, chained through counters in the workspace.
// Weights HBM -> LDS with direct-to-LDS loads.  The first stream_prefix_bytes() of the workspace belong to it.
size_t stream_prefix_bytes();
bool stream_supported(int top_k, int M, int K, int N, int E, int sorted_num, int block_m);
size_t stream_workspace_bytes(int top_k, int M, int K, int N, int E, int sorted_num, int block_m);
hipError_t launch_stream(const MoeParams &p, int warp_n, int stages, void *workspace, hipStream_t stream);


// Tiled kernel for large batches: one workgroup per row block, token tiles shared through LDS, all I/128 slices in
// one workgroup, per-slot bf16 result rows reduced by a second kernel.
bool tile_supported(int top_k, int M, int K, int N, int E, int sorted_num, int block_m);
size_t tile_workspace_bytes(int top_k, int M, int K, int N, int E, int sorted_num, int block_m);
hipError_t launch_tile(const MoeParams &p, int stages, void *workspace, hipStream_t stream);

// Wide kernel for large batches: macro blocks of up to 256 consecutive sorted rows of one expert (several row blocks),
// twice the tokens per weight byte of the tile kernel; same per-slot result rows and reduce kernel.  block_m > 32.
bool wide_supported(int top_k, int M, int K, int N, int E, int sorted_num, int block_m);
size_t wide_workspace_bytes(int top_k, int M, int K, int N, int E, int sorted_num, int block_m);
hipError_t launch_wide(const MoeParams &p, int stages, void *workspace, hipStream_t stream);

// out[t] = bf16(out[t] + sum over the token's live slots of y[slot]) (or bf16(sum) when p.overwrite); closes the
// workspace's launch epoch.  Shared by the tile and wide kernels, which write each (token, slot) row once into y.
struct RowsReduce {
    MoeParams p;
    StreamCtl *ctl;
    const int *live;      // [slots] == epoch + 1 of the control block for rows written in this launch
    const uint16_t *y;    // [slots][K] bf16
};
hipError_t launch_rows_reduce(const RowsReduce &r, hipStream_t stream);

}  // namespace alpha_moe
