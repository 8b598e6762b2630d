// C ABI of libalpha_moe_hip.so (include/alpha_moe_hip.h): argument checks, kernel-family choice, launches.
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "moe_common.hpp"

using namespace alpha_moe;

namespace {

// Tuning overrides: name (also the environment variable read once at first use), current value.
struct TunableSlot {
    const char *name;
    int value;
};
TunableSlot g_tunables[kTunCount] = {
    {"ALPHA_MOE_PATH", kTunableUnset},        {"ALPHA_MOE_STRICT_QUEUE", kTunableUnset},
    {"ALPHA_MOE_KBPI", kTunableUnset},        {"ALPHA_MOE_TPI", kTunableUnset},
    {"ALPHA_MOE_LAG", kTunableUnset},         {"ALPHA_MOE_GRID", kTunableUnset},
    {"ALPHA_MOE_TILE_GPS", kTunableUnset},    {"ALPHA_MOE_TILE_LAG", kTunableUnset},
    {"ALPHA_MOE_TILE_GRID", kTunableUnset},   {"ALPHA_MOE_TILE_NT", kTunableUnset},
    {"ALPHA_MOE_WIDE_PP", kTunableUnset},
};

void load_tunables_once()
{
    static const bool done = [] {
        for (TunableSlot &t : g_tunables) {
            const char *e = getenv(t.name);
            if (!e) continue;
            if (!strcmp(t.name, "ALPHA_MOE_PATH"))
                t.value = !strcmp(e, "direct") ? 1 : !strcmp(e, "stream") ? 2 : !strcmp(e, "tile") ? 3 : !strcmp(e, "wide") ? 4 : kTunableUnset;
            else
                t.value = atoi(e);
        }
        return true;
    }();
    (void)done;
}

enum Path { kDirect, kStream, kTile, kWide };

// Streaming kernel for row blocks of at most 32 rows (decode); above that (prefill) warp_n picks the token tiles a
// wavefront multiplies per step: 8 -> wide kernel (macro blocks of 256 rows), 4 -> tile kernel (one row block).  The
// direct kernel is the fallback for shapes none of them takes.
Path choose_path(int top_k, int M, int K, int N, int E, int sorted_num, int block_m, int warp_n)
{
    const bool s_ok = stream_supported(top_k, M, K, N, E, sorted_num, block_m);
    const bool t_ok = tile_supported(top_k, M, K, N, E, sorted_num, block_m);
    const bool w_ok = wide_supported(top_k, M, K, N, E, sorted_num, block_m);
    const int f = tunable(kTunPath, 0);
    if (f == 1) return kDirect;
    if (f == 2 && s_ok) return kStream;
    if (f == 3 && t_ok) return kTile;
    if (f == 4 && w_ok) return kWide;
    if (s_ok) return kStream;
    if (w_ok && (warp_n == 8 || !t_ok)) return kWide;
    if (t_ok) return kTile;
    return kDirect;
}

}  // namespace

int alpha_moe::tunable(Tunable which, int dflt)
{
    load_tunables_once();
    const int v = g_tunables[which].value;
    return v == kTunableUnset ? dflt : v;
}

extern "C" int alpha_moe_set_tunable(const char *name, int value, int set)
{
    if (!name) return ALPHA_MOE_ERR_NULL_POINTER;
    load_tunables_once();
    for (TunableSlot &t : g_tunables)
        if (!strcmp(t.name, name)) {
            t.value = set ? value : kTunableUnset;
            return ALPHA_MOE_OK;
        }
    return ALPHA_MOE_ERR_SHAPE;
}

extern "C" int alpha_moe_validate(int top_k, int M, int K, int N, int num_experts, int sorted_num, int block_m,
                                  int block_n, int warp_n, int stages)
{
    if (M <= 0 || K <= 0 || N <= 0 || num_experts <= 0 || top_k <= 0 || sorted_num <= 0) return ALPHA_MOE_ERR_SHAPE;
    if (K % 128 != 0 || N % 256 != 0 || K > 128 * kMaxKBlocks) return ALPHA_MOE_ERR_SHAPE;
    if ((int64_t)M * top_k > INT32_MAX || (int64_t)M * K / 4 > INT32_MAX) return ALPHA_MOE_ERR_SHAPE;
    if (block_m < 8 || block_m > 128 || block_m % 8 != 0) return ALPHA_MOE_ERR_BLOCK_M;
    if (!((block_n == 64 && warp_n == 4) || (block_n == 32 && warp_n == 8))) return ALPHA_MOE_ERR_BLOCK_N_WARP_N;
    if (stages < 1 || stages > 5) return ALPHA_MOE_ERR_STAGES;
    const int64_t n_blocks = ((int64_t)sorted_num + block_m - 1) / block_m;
    if (n_blocks * (N / 256) * (K / 128) > INT32_MAX) return ALPHA_MOE_ERR_SHAPE;
    return ALPHA_MOE_OK;
}

extern "C" size_t alpha_moe_workspace_bytes(int top_k, int M, int K, int N, int num_experts, int sorted_num,
                                            int block_m)
{
    if (top_k <= 0 || M <= 0 || K <= 0 || N <= 0 || num_experts <= 0 || sorted_num <= 0 || block_m <= 0) return 0;
    // both kernel families keep their bookkeeping out of each other's way: the streaming kernel's self-maintaining
    // prefix comes first, the direct kernel's accumulator (cleared on every call) after it
    const size_t direct = stream_prefix_bytes() + (size_t)M * (size_t)K * sizeof(float);
    const size_t stream = stream_supported(top_k, M, K, N, num_experts, sorted_num, block_m)
                              ? stream_workspace_bytes(top_k, M, K, N, num_experts, sorted_num, block_m)
                              : 0;
    const size_t tile = tile_supported(top_k, M, K, N, num_experts, sorted_num, block_m)
                            ? tile_workspace_bytes(top_k, M, K, N, num_experts, sorted_num, block_m)
                            : 0;
    const size_t wide = wide_supported(top_k, M, K, N, num_experts, sorted_num, block_m)
                            ? wide_workspace_bytes(top_k, M, K, N, num_experts, sorted_num, block_m)
                            : 0;
    size_t m = direct > stream ? direct : stream;
    m = m > tile ? m : tile;
    return m > wide ? m : wide;
}

namespace {

int run_fused_moe(const uint8_t *x, const float *x_scale, const uint8_t *w, const float *w_scale, const uint8_t *w2,
                  const float *w2_scale, uint16_t *out, const int32_t *sorted_token_ids, const int32_t *expert_ids,
                  const int32_t *num_tokens_post_padded, const float *topk_weights, int top_k, int M, int K, int N,
                  int num_experts, int sorted_num, int block_m, int block_n, int warp_n, int stages,
                  float scaling_factor, void *workspace, size_t workspace_bytes, void *stream, int overwrite,
                  int prepacked = 0)
{
    if (!x || !x_scale || !w || !w_scale || !w2 || !w2_scale || !out || !sorted_token_ids || !expert_ids ||
        !num_tokens_post_padded || !topk_weights)
        return ALPHA_MOE_ERR_NULL_POINTER;
    const int rc = alpha_moe_validate(top_k, M, K, N, num_experts, sorted_num, block_m, block_n, warp_n, stages);
    if (rc != ALPHA_MOE_OK) return rc;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0 ||
        workspace_bytes < alpha_moe_workspace_bytes(top_k, M, K, N, num_experts, sorted_num, block_m))
        return ALPHA_MOE_ERR_WORKSPACE;

    MoeParams p;
    p.x = x; p.x_scale = x_scale; p.w = w; p.w_scale = w_scale; p.w2 = w2; p.w2_scale = w2_scale;
    p.out = out;
    p.acc = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + stream_prefix_bytes());
    p.sorted_ids = sorted_token_ids; p.expert_ids = expert_ids; p.ntpp = num_tokens_post_padded;
    p.topk_w = topk_weights;
    p.top_k = top_k; p.M = M; p.K = K; p.N = N; p.E = num_experts; p.sorted_num = sorted_num; p.block_m = block_m;
    p.scaling = scaling_factor;
    p.overwrite = overwrite;
    const size_t I = (size_t)N / 2;
    p.w_rs = prepacked ? 128 : (size_t)K;
    p.w_ks = prepacked ? (size_t)N * 128 : 128;
    p.w2_rs = prepacked ? 128 : I;
    p.w2_ks = prepacked ? (size_t)K * 128 : 128;

    hipStream_t hs = static_cast<hipStream_t>(stream);
    hipError_t err;
    const Path path = choose_path(top_k, M, K, N, num_experts, sorted_num, block_m, warp_n);
    if (path == kStream) {
        err = launch_stream(p, warp_n, stages, workspace, hs);
    } else if (path == kWide) {
        err = launch_wide(p, stages, workspace, hs);
    } else if (path == kTile) {
        err = launch_tile(p, stages, workspace, hs);
    } else {
        // the fallback kernel reads the operator's own layout only
        if (prepacked) return ALPHA_MOE_ERR_SHAPE;
        err = launch_zero_acc(p, hs);
        if (err == hipSuccess) err = launch_direct(p, warp_n, stages, hs);
        if (err == hipSuccess) err = launch_finalize(p, hs);
    }
    return err == hipSuccess ? ALPHA_MOE_OK : ALPHA_MOE_ERR_LAUNCH;
}

}  // namespace

extern "C" int alpha_moe_fused_moe_w8a8_up_down(const uint8_t *x, const float *x_scale, const uint8_t *w,
                                                const float *w_scale, const uint8_t *w2, const float *w2_scale,
                                                uint16_t *out, const int32_t *sorted_token_ids,
                                                const int32_t *expert_ids, const int32_t *num_tokens_post_padded,
                                                const float *topk_weights, int top_k, int M, int K, int N,
                                                int num_experts, int sorted_num, int block_m, int block_n, int warp_n,
                                                int stages, float scaling_factor, void *workspace,
                                                size_t workspace_bytes, void *stream)
{
    return run_fused_moe(x, x_scale, w, w_scale, w2, w2_scale, out, sorted_token_ids, expert_ids,
                         num_tokens_post_padded, topk_weights, top_k, M, K, N, num_experts, sorted_num, block_m, block_n,
                         warp_n, stages, scaling_factor, workspace, workspace_bytes, stream, 0);
}

extern "C" int alpha_moe_fused_moe_w8a8_up_down_store(const uint8_t *x, const float *x_scale, const uint8_t *w,
                                                      const float *w_scale, const uint8_t *w2, const float *w2_scale,
                                                      uint16_t *out, const int32_t *sorted_token_ids,
                                                      const int32_t *expert_ids,
                                                      const int32_t *num_tokens_post_padded, const float *topk_weights,
                                                      int top_k, int M, int K, int N, int num_experts, int sorted_num,
                                                      int block_m, int block_n, int warp_n, int stages,
                                                      float scaling_factor, void *workspace, size_t workspace_bytes,
                                                      void *stream)
{
    return run_fused_moe(x, x_scale, w, w_scale, w2, w2_scale, out, sorted_token_ids, expert_ids,
                         num_tokens_post_padded, topk_weights, top_k, M, K, N, num_experts, sorted_num, block_m, block_n,
                         warp_n, stages, scaling_factor, workspace, workspace_bytes, stream, 1);
}

extern "C" int alpha_moe_fused_moe_w8a8_up_down_prepacked(const uint8_t *x, const float *x_scale, const uint8_t *w_packed,
                                                          const float *w_scale, const uint8_t *w2_packed,
                                                          const float *w2_scale, uint16_t *out,
                                                          const int32_t *sorted_token_ids, const int32_t *expert_ids,
                                                          const int32_t *num_tokens_post_padded,
                                                          const float *topk_weights, int top_k, int M, int K, int N,
                                                          int num_experts, int sorted_num, int block_m, int block_n,
                                                          int warp_n, int stages, float scaling_factor, int store,
                                                          void *workspace, size_t workspace_bytes, void *stream)
{
    return run_fused_moe(x, x_scale, w_packed, w_scale, w2_packed, w2_scale, out, sorted_token_ids, expert_ids,
                         num_tokens_post_padded, topk_weights, top_k, M, K, N, num_experts, sorted_num, block_m, block_n,
                         warp_n, stages, scaling_factor, workspace, workspace_bytes, stream, store != 0, 1);
}

// ---- the entry point for callers that cannot allocate ------------------------------------------------------
// Same call as alpha_moe_fused_moe_w8a8_up_down, with the scratch memory in this array instead of a caller's buffer.
// Zero when the code object is loaded, which is the state the kernels' control prefix has to start in; afterwards the
// kernels maintain it like any workspace.  Every device the library runs on holds its own copy until the process ends.
static __device__ __align__(256) unsigned char scratch[ALPHA_MOE_STATIC_SCRATCH_BYTES];

namespace {

// Device address of `scratch` on the current device: looked up once per device, with that device current (in host code
// the array's name is a host-side handle, not a device address).
void *static_scratch_of_current_device()
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void *ptrs[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        ptrs[dev] = ptr;
    }
    return ptrs[dev];
}

}  // namespace

extern "C" int alpha_moe_fused_moe_w8a8_up_down_static(const uint8_t *x, const float *x_scale, const uint8_t *w,
                                                       const float *w_scale, const uint8_t *w2, const float *w2_scale,
                                                       uint16_t *out, const int32_t *sorted_token_ids,
                                                       const int32_t *expert_ids,
                                                       const int32_t *num_tokens_post_padded, const float *topk_weights,
                                                       int top_k, int M, int K, int N, int num_experts, int sorted_num,
                                                       int block_m, int block_n, int warp_n, int stages,
                                                       float scaling_factor, void *stream)
{
    if (!x || !x_scale || !w || !w_scale || !w2 || !w2_scale || !out || !sorted_token_ids || !expert_ids ||
        !num_tokens_post_padded || !topk_weights)
        return ALPHA_MOE_ERR_NULL_POINTER;
    const int rc = alpha_moe_validate(top_k, M, K, N, num_experts, sorted_num, block_m, block_n, warp_n, stages);
    if (rc != ALPHA_MOE_OK) return rc;
    if (alpha_moe_workspace_bytes(top_k, M, K, N, num_experts, sorted_num, block_m) > ALPHA_MOE_STATIC_SCRATCH_BYTES)
        return ALPHA_MOE_ERR_SCRATCH_LIMIT;
    void *ptr = static_scratch_of_current_device();
    if (!ptr) return ALPHA_MOE_ERR_LAUNCH;
    return run_fused_moe(x, x_scale, w, w_scale, w2, w2_scale, out, sorted_token_ids, expert_ids,
                         num_tokens_post_padded, topk_weights, top_k, M, K, N, num_experts, sorted_num, block_m, block_n,
                         warp_n, stages, scaling_factor, ptr, ALPHA_MOE_STATIC_SCRATCH_BYTES, stream, 0);
}

namespace {
// clears `words` ints (a fill kernel: unlike a memset node it may be recorded into a HIP graph)
__global__ void zero_words_kernel(int *dst, size_t words)
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < words; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = 0;
}
}  // namespace

extern "C" int alpha_moe_static_scratch_check(void *stream)
{
    void *ptr = static_scratch_of_current_device();
    if (!ptr) return ALPHA_MOE_ERR_LAUNCH;
    return alpha_moe_workspace_check(ptr, stream);
}

extern "C" int alpha_moe_static_scratch_reset(void *stream)
{
    void *ptr = static_scratch_of_current_device();
    if (!ptr) return ALPHA_MOE_ERR_LAUNCH;
    hipLaunchKernelGGL(zero_words_kernel, dim3(64), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<int *>(ptr), alpha_moe_workspace_zero_bytes() / sizeof(int));
    return hipGetLastError() == hipSuccess ? ALPHA_MOE_OK : ALPHA_MOE_ERR_LAUNCH;
}

extern "C" int alpha_moe_workspace_check(const void *workspace, void *stream)
{
    if (!workspace) return ALPHA_MOE_ERR_NULL_POINTER;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    int flag = 0;
    const StreamCtl *ctl = static_cast<const StreamCtl *>(workspace);
    if (hipMemcpyAsync(&flag, &ctl->error, sizeof(int), hipMemcpyDeviceToHost, hs) != hipSuccess ||
        hipStreamSynchronize(hs) != hipSuccess)
        return ALPHA_MOE_ERR_LAUNCH;
    return flag ? ALPHA_MOE_ERR_WAIT_EXPIRED : ALPHA_MOE_OK;
}

extern "C" size_t alpha_moe_workspace_zero_bytes(void) { return (stream_prefix_bytes() + 255) & ~(size_t)255; }

extern "C" const char *alpha_moe_status_string(int status)
{
    switch (status) {
    case ALPHA_MOE_OK: return "ok";
    case ALPHA_MOE_ERR_NULL_POINTER: return "a required pointer is null";
    case ALPHA_MOE_ERR_SHAPE: return "unsupported shape: need M>0, top_k>0, K % 128 == 0, K <= 65536, N % 256 == 0, sizes within int32";
    case ALPHA_MOE_ERR_BLOCK_M: return "block_m must be a multiple of 8 in [8, 128]";
    case ALPHA_MOE_ERR_BLOCK_N_WARP_N: return "(block_n, warp_n) must be (64, 4) or (32, 8)";
    case ALPHA_MOE_ERR_STAGES: return "stages must be in [1, 5]";
    case ALPHA_MOE_ERR_WORKSPACE: return "workspace is null, not 256-byte aligned, or smaller than alpha_moe_workspace_bytes()";
    case ALPHA_MOE_ERR_LAUNCH: return "the HIP runtime refused the kernel launch";
    case ALPHA_MOE_ERR_WAIT_EXPIRED:
        return "a workgroup's bounded wait for another workgroup ran out in an earlier launch on this workspace: its "
               "results are not valid (launches overlapping on one device, or a device that cannot hold the grid)";
    case ALPHA_MOE_ERR_SCRATCH_LIMIT:
        return "the call needs more scratch memory than the library's built-in buffer holds "
               "(alpha_moe_fused_moe_w8a8_up_down_static): use the entry point that takes a workspace";
    default: return "unknown status";
    }
}

extern "C" const char *alpha_moe_version(void) { return "0.6"; }
