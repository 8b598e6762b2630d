/*
 * C ABI of the MI355X (gfx950) fused W8A8 MoE operator: libalpha_moe_hip.so.
 *
 * Plain pointers and sizes only; no torch types.  Every pointer is DEVICE memory, borrowed for the
 * duration of the enqueued work; nothing is allocated, freed or synchronised; the call is asynchronous on
 * `stream` and can be captured into a HIP graph.  No function here prints or exits: each returns a status.
 */
#ifndef ALPHA_MOE_HIP_H
#define ALPHA_MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum alpha_moe_status {
    ALPHA_MOE_OK = 0,
    ALPHA_MOE_ERR_NULL_POINTER = 1,   /* a required pointer is null */
    ALPHA_MOE_ERR_SHAPE = 2,          /* M<=0, K%128!=0, N%256!=0, top_k<=0, sizes overflow int32 ... */
    ALPHA_MOE_ERR_BLOCK_M = 3,        /* block_m not in {8,16,...,128} */
    ALPHA_MOE_ERR_BLOCK_N_WARP_N = 4, /* (block_n, warp_n) not (64,4) or (32,8) */
    ALPHA_MOE_ERR_STAGES = 5,         /* stages not in 1..5 */
    ALPHA_MOE_ERR_LAUNCH = 6,         /* the HIP runtime refused the launch (see hipGetLastError) */
    ALPHA_MOE_ERR_WORKSPACE = 7,      /* workspace null, misaligned or smaller than alpha_moe_workspace_bytes() */
    ALPHA_MOE_ERR_WAIT_EXPIRED = 8,   /* alpha_moe_workspace_check: a bounded wait between workgroups ran out */
    ALPHA_MOE_ERR_SCRATCH_LIMIT = 9   /* ..._static: the call needs more than ALPHA_MOE_STATIC_SCRATCH_BYTES of scratch */
};

/*
 * out[t, :] += scaling_factor * sum_s topk_weights[t, s] * W2_e . requant(SwiGLU(W1_e . x_t)),  e = expert of slot (t, s).
 *
 * Replaces the reference's C++ seam `fused_moe_w8a8_wgmma_up_down_acc`
 * (declared csrc/torch_interface.cpp:12-34, defined
 * csrc/kernels/fused_moe_w8a8/fused_moe_w8a8_up_down_acc.cu:1258-1303): same parameters in the same order, with
 * fp8 as uint8_t codes (OCP e4m3fn), bf16 as uint16_t, the stream as an opaque hipStream_t, an int status
 * instead of stderr prints / exit(), and a caller-owned scratch buffer before the stream (the reference has none:
 * it adds every partial row straight into the bf16 output).
 *
 *   x                [M, K]            fp8, row-major, K % 128 == 0
 *   x_scale          [M, K/128]        f32, per token per 128 columns
 *   w                [E, N, K]         fp8, N = 2*I, gate/up rows interleaved in chunks of 8, N % 256 == 0
 *   w_scale          [E, N/128, K/128] f32, gate/up rows interleaved in chunks of 1
 *   w2               [E, K, N/2]       fp8
 *   w2_scale         [E, K/128, N/256] f32
 *   out              [M, K]            bf16, the result is ADDED once per call (out = bf16(out + sum)); caller zero-fills
 *   sorted_token_ids [sorted_num]      flat slot ids t*top_k+s grouped by expert in blocks of block_m; ids >= M*top_k are padding
 *   expert_ids       [ceil(sorted_num/block_m)]  expert of each block (blocks with an id outside [0,E) are skipped)
 *   num_tokens_post_padded [1]         blocks starting at or past this row are skipped
 *   topk_weights     [M*top_k]         f32, indexed by the flat slot id
 *   block_m          8..128 step 8     must equal the block size sorted_token_ids was built with
 *   (block_n, warp_n) (64,4) or (32,8) wavefronts per workgroup = warp_n, w1 rows per wavefront = block_n
 *   stages           1..5              K-blocks of loads kept in flight per wavefront
 *   workspace        device scratch of at least alpha_moe_workspace_bytes(top_k, M, K, N, num_experts, sorted_num,
 *                    block_m) bytes, 256-byte aligned.  Its first alpha_moe_workspace_zero_bytes() bytes must be
 *                    ZERO-FILLED once, before its first use (zero-filling all of it is fine too); after
 *                    that its contents belong to the library (self-resetting counters, per-launch epochs) and the
 *                    same buffer serves any number of calls, of any sizes it is large enough for, without being
 *                    cleared.  Calls that share a workspace must be ordered on one stream.
 */
int alpha_moe_fused_moe_w8a8_up_down(
    const uint8_t *x, const float *x_scale,
    const uint8_t *w, const float *w_scale,
    const uint8_t *w2, const float *w2_scale,
    uint16_t *out,
    const int32_t *sorted_token_ids, const int32_t *expert_ids, const int32_t *num_tokens_post_padded,
    const float *topk_weights,
    int top_k, int M, int K, int N, int num_experts, int sorted_num,
    int block_m, int block_n, int warp_n, int stages,
    float scaling_factor, void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * The same call with store semantics: out = bf16(sum), whatever `out` held before, so the caller's zero-fill of
 * `out` (README.md:49,62 and extra/sglang.patch:31 of the reference: `torch.zeros_like(hidden_states)` before every
 * call) and its launch are not needed.  Every element of out[0:M, 0:K] is written, also for tokens none of whose
 * slots is live.  Same arguments, checks, workspace and status codes as alpha_moe_fused_moe_w8a8_up_down.
 * The reference has no such variant: its kernel can only add, because top_k * I/128 workgroups contribute to a row.
 */
int alpha_moe_fused_moe_w8a8_up_down_store(
    const uint8_t *x, const float *x_scale,
    const uint8_t *w, const float *w_scale,
    const uint8_t *w2, const float *w2_scale,
    uint16_t *out,
    const int32_t *sorted_token_ids, const int32_t *expert_ids, const int32_t *num_tokens_post_padded,
    const float *topk_weights,
    int top_k, int M, int K, int N, int num_experts, int sorted_num,
    int block_m, int block_n, int warp_n, int stages,
    float scaling_factor, void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * The same operator on PRE-PACKED weights (an optional offline re-layout; the interleave-8 layout above stays the
 * operator's API).  No counterpart in the reference, whose TMA box loads take the row-major tensors as they are; it
 * builds on the reference's interleave step (alpha_moe_python/utils.py:5-17, README.md:94-102) and is applied after it:
 *   w_packed   [E, K/128, N, 128]  = w  viewed as [E, N, K/128, 128] with the two middle axes swapped
 *   w2_packed  [E, I/128, K, 128]  = w2 viewed as [E, K, I/128, 128] with the two middle axes swapped
 * so that one 128-byte K block of consecutive rows is contiguous in memory: the 256 rows of a slice are one 32 KiB
 * burst per K step instead of 256 row pieces K bytes apart.  alpha_moe_python.utils.prepack_weights builds both.
 * Scales, routing arrays, knobs, workspace and status codes are those of alpha_moe_fused_moe_w8a8_up_down; store != 0
 * gives the semantics of ..._store.  Shapes that only the fallback kernel takes (more than eight 128-column slices, K
 * above 16384) return ALPHA_MOE_ERR_SHAPE: that kernel reads the operator's layout only.
 */
int alpha_moe_fused_moe_w8a8_up_down_prepacked(
    const uint8_t *x, const float *x_scale,
    const uint8_t *w_packed, const float *w_scale,
    const uint8_t *w2_packed, const float *w2_scale,
    uint16_t *out,
    const int32_t *sorted_token_ids, const int32_t *expert_ids, const int32_t *num_tokens_post_padded,
    const float *topk_weights,
    int top_k, int M, int K, int N, int num_experts, int sorted_num,
    int block_m, int block_n, int warp_n, int stages,
    float scaling_factor, int store, void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * The adding call for callers that cannot allocate device memory or pass a buffer through: code under HIP graph
 * capture that has no workspace at hand, tight serving loops, harnesses that forbid hipMalloc.  It has NO counterpart
 * in the reference (whose kernel needs no scratch).  Same arguments, checks and result as
 * alpha_moe_fused_moe_w8a8_up_down without `workspace` / `workspace_bytes`: the scratch memory is a buffer of
 * ALPHA_MOE_STATIC_SCRATCH_BYTES built into the library's code object (every device the library runs on holds its own
 * copy until the process ends).  The call allocates and frees nothing.  A call whose alpha_moe_workspace_bytes()
 * exceeds that size returns ALPHA_MOE_ERR_SCRATCH_LIMIT and launches nothing: 64 MiB cover every decode-sized batch of
 * the shipped shard shapes (DeepSeek-V3 shard with the shipped knobs: up to M = 128, and M = 256 with 16-row blocks;
 * the other two shards up to M = 1024) but not prefill, whose scratch grows with M * top_k * K.  All calls on one device share the one
 * buffer, which keeps the last call's contents: calls that overlap in time on one device race (order them on one
 * stream), and a bounded wait that ran out stays recorded (every later call then fills `out` with NaN) until
 * alpha_moe_static_scratch_reset clears it.  The first call on a device looks the buffer's address up; make that call outside graph capture.
 */
#define ALPHA_MOE_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
int alpha_moe_fused_moe_w8a8_up_down_static(
    const uint8_t *x, const float *x_scale,
    const uint8_t *w, const float *w_scale,
    const uint8_t *w2, const float *w2_scale,
    uint16_t *out,
    const int32_t *sorted_token_ids, const int32_t *expert_ids, const int32_t *num_tokens_post_padded,
    const float *topk_weights,
    int top_k, int M, int K, int N, int num_experts, int sorted_num,
    int block_m, int block_n, int warp_n, int stages,
    float scaling_factor, void *stream /* hipStream_t */);

/*
 * Health and repair of the built-in scratch buffer of alpha_moe_fused_moe_w8a8_up_down_static on the current device
 * (callers have no address for it, so alpha_moe_workspace_check cannot be pointed at it).  No counterpart in the
 * reference.  alpha_moe_static_scratch_check waits for `stream` and returns ALPHA_MOE_ERR_WAIT_EXPIRED if a bounded wait
 * ever ran out on that buffer, ALPHA_MOE_OK otherwise.  alpha_moe_static_scratch_reset clears the buffer's control
 * prefix on `stream` (a fill kernel; no allocation), which also clears a recorded expiry: call it with no call on that
 * device in flight, outside graph capture.
 */
int alpha_moe_static_scratch_check(void *stream /* hipStream_t */);
int alpha_moe_static_scratch_reset(void *stream /* hipStream_t */);

/* Bytes of scratch the calls above need for these sizes (0 if any is not positive). */
size_t alpha_moe_workspace_bytes(int top_k, int M, int K, int N, int num_experts, int sorted_num, int block_m);

/*
 * How many bytes at the start of a workspace have to be zero before its first use (the control block, counters and
 * flags; independent of the problem size).  The rest may hold anything.  No counterpart in the reference, which has
 * no scratch memory.
 */
size_t alpha_moe_workspace_zero_bytes(void);

/*
 * Health of a workspace: waits for `stream`, then returns ALPHA_MOE_ERR_WAIT_EXPIRED if in any earlier launch on this
 * workspace a workgroup gave up waiting for another (each such wait is bounded at a few seconds so that nothing
 * hangs; the results of that launch are not valid), ALPHA_MOE_OK otherwise.  The flag is sticky until the prefix is
 * zero-filled again.  Synchronises, so it is for tests and health checks, not for the serving loop.  The reference's
 * kernel has no waits between thread blocks and no counterpart.  Callers need not poll it to notice: while the flag
 * is set, every call on the workspace fills `out` with NaN.
 */
int alpha_moe_workspace_check(const void *workspace, void *stream /* hipStream_t */);

/*
 * The argument checks of the call above without touching the device: returns the status the launch would
 * return for these sizes and knobs.  Replaces the knob dispatch of fused_moe_w8a8_up_down_acc.cu:1200-1256,1282-1302
 * (which prints to stderr and silently does nothing) and the TORCH_CHECKs of torch_interface.cpp:59-64.
 */
int alpha_moe_validate(int top_k, int M, int K, int N, int num_experts, int sorted_num,
                       int block_m, int block_n, int warp_n, int stages);

/*
 * Input preparation, the two steps every caller runs right before the fused call.  The reference takes both from
 * SGLang (jit_moe.py:142,158; extra/sglang.patch:30-35); here they are part of the library.
 *
 * alpha_moe_per_token_group_quant_fp8 replaces sglang_per_token_group_quant_fp8(x, 128) (jit_moe.py:142): x is
 * [M, K] row-major bf16 (x_is_f32 == 0) or fp32 (x_is_f32 != 0), K % 128 == 0; writes q [M, K] FP8 e4m3 and
 * scale [M, K/128] fp32 with scale = max(amax, 1e-10) / 448, q = rne(clamp(x / scale, -448, 448)): the arrays the
 * fused kernel reads at fused_moe_w8a8_up_down_acc.cu:793,800-807.
 */
int alpha_moe_per_token_group_quant_fp8(const void *x, int x_is_f32, uint8_t *q, float *scale, int M, int K,
                                        void *stream /* hipStream_t */);

/*
 * alpha_moe_moe_align_block_size replaces SGLang's moe_align_block_size(topk_ids, block_size, num_experts)
 * (jit_moe.py:158): topk_ids holds the expert of each of the numel = M * top_k routing slots.  Writes
 *   sorted_token_ids [sorted_num = numel + num_experts * (block_size - 1)]: slot ids in ascending expert order,
 *       ascending within an expert, every expert's segment padded to a multiple of block_size with the value numel;
 *   expert_ids [n_blocks = ceil(sorted_num / block_size)]: the expert of each block, -1 past the padded total;
 *   num_tokens_post_padded [1]: the padded total
 * as the fused kernel reads them (fused_moe_w8a8_up_down_acc.cu:676-679,756-758).  Slots whose expert is outside
 * [0, num_experts) are dropped.  num_experts <= 4096.  Inputs of more than 4096 slots need a scratch buffer of
 * alpha_moe_align_workspace_bytes(numel, num_experts) bytes (any contents); smaller ones accept workspace == NULL.
 */
size_t alpha_moe_align_workspace_bytes(int numel, int num_experts);
int alpha_moe_moe_align_block_size(const int32_t *topk_ids, int numel, int num_experts, int block_size,
                                   int32_t *sorted_token_ids, int sorted_num, int32_t *expert_ids, int n_blocks,
                                   int32_t *num_tokens_post_padded, void *workspace, size_t workspace_bytes,
                                   void *stream /* hipStream_t */);

/* Human-readable text for a status code (static storage). */
const char *alpha_moe_status_string(int status);

/* Library version, "major.minor". */
const char *alpha_moe_version(void);

#ifdef __cplusplus
}
#endif
#endif /* ALPHA_MOE_HIP_H */
