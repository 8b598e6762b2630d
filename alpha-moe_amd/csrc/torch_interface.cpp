// PyTorch-ROCm binding of the fused W8A8 MoE operator: registers
// torch.ops.alpha_moe.fused_moe_w8a8_up_down with the schema of the reference
// (csrc/torch_interface.cpp:105-125), checks the arguments, and forwards raw device pointers plus the
// current HIP stream to the C ABI in include/alpha_moe_hip.h.  No kernel code lives here.
//
// Differences from the reference binding (csrc/torch_interface.cpp:37-103), all on the strict side:
//   * dtype, device and shape of every tensor are checked (the reference checks contiguity only);
//   * the device guard is installed before the stream is fetched;
//   * a refused launch or an unsupported knob raises instead of printing or doing nothing.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include "../../include/alpha_moe_hip.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <tuple>
#include <utility>
#include <vector>

namespace {

// Scratch for the C ABI, one buffer per (device, stream): zero-filled when created and maintained by the library
// afterwards, so the steady state allocates and clears nothing.  When a call needs more than the buffer holds, a new one
// of at least 1.5 times the old size takes over (geometric growth: a stream that sees growing sizes reallocates a
// logarithmic number of times).  What happens to the old one depends on whether a HIP graph may hold its address: a
// buffer that was handed out while its stream was being captured is kept alive beside the new one (graphs captured
// before keep replaying into it: control block, flags and result rows); a buffer only eager calls ever used is dropped,
// which is safe because the caching allocator hands its memory out again in stream order, behind the kernels that used it.
// Growth while the stream is being captured is refused: the fill of the new buffer's control prefix would be recorded
// into the graph and run on every replay, and the allocation would belong to the graph's private pool.
// reserve_workspace() sizes the buffer ahead of time.
struct StreamScratch {
    at::Tensor current;
    bool current_seen_by_capture = false;
    std::vector<at::Tensor> retired;
};

std::mutex g_scratch_mu;
std::map<std::pair<int, void *>, StreamScratch> g_scratch;

at::Tensor workspace_for(const at::Device &dev, hipStream_t stream, size_t bytes)
{
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    StreamScratch &slot = g_scratch[{dev.index(), static_cast<void *>(stream)}];
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(stream, &capturing);
    if (!slot.current.defined() || static_cast<size_t>(slot.current.numel()) < bytes) {
        TORCH_CHECK(capturing == hipStreamCaptureStatusNone,
                    "alpha_moe: this call needs ", bytes, " bytes of scratch memory on a stream that is being captured "
                    "and holds ", slot.current.defined() ? slot.current.numel() : 0, ": run the operator once with "
                    "these sizes before the capture, or call torch.ops.alpha_moe.reserve_workspace(x, bytes) there");
        size_t cap = bytes;
        if (slot.current.defined()) {
            cap = std::max(cap, static_cast<size_t>(slot.current.numel()) * 3 / 2);
            if (slot.current_seen_by_capture) slot.retired.push_back(slot.current);
        }
        cap = (cap + 255) & ~static_cast<size_t>(255);
        slot.current = at::Tensor();   // an eager-only buffer goes back to the allocator before the new one is taken
        slot.current = at::empty({static_cast<int64_t>(cap)}, at::TensorOptions().dtype(at::kByte).device(dev));
        slot.current_seen_by_capture = false;
        // only the control block, counters and flags have to start at zero (1.5 MiB, not the whole buffer)
        slot.current.narrow(0, 0, static_cast<int64_t>(alpha_moe_workspace_zero_bytes())).zero_();
    }
    if (capturing != hipStreamCaptureStatusNone) slot.current_seen_by_capture = true;
    return slot.current;
}

// scratch_buffers(like): [buffers alive, bytes of the current one, bytes kept for earlier graph captures] of
// (like's device, the current stream) - for tests and memory accounting.
std::vector<int64_t> scratch_buffers(const at::Tensor &like)
{
    TORCH_CHECK(like.is_cuda(), "scratch_buffers: `like` must be a GPU tensor (it names the device)");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(like.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    auto it = g_scratch.find({like.device().index(), static_cast<void *>(stream)});
    if (it == g_scratch.end()) return {0, 0, 0};
    int64_t retired = 0;
    for (const at::Tensor &t : it->second.retired) retired += t.numel();
    return {static_cast<int64_t>(it->second.retired.size()) + (it->second.current.defined() ? 1 : 0),
            it->second.current.defined() ? it->second.current.numel() : 0, retired};
}

// reserve_workspace(like, bytes): make the scratch buffer of (like's device, the current stream) at least `bytes`
// large now, e.g. alpha_moe_workspace_bytes() of the largest call a graph captured later on this stream will make.
void reserve_workspace(const at::Tensor &like, int64_t bytes)
{
    TORCH_CHECK(like.is_cuda(), "reserve_workspace: `like` must be a GPU tensor (it names the device)");
    TORCH_CHECK(bytes >= 0, "reserve_workspace: bytes must not be negative");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(like.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const size_t need = std::max(static_cast<size_t>(bytes), alpha_moe_workspace_zero_bytes());
    (void)workspace_for(like.device(), stream, need);
}

// bytes of scratch a call with these sizes needs (alpha_moe_workspace_bytes of the C ABI)
int64_t workspace_bytes(int64_t top_k, int64_t M, int64_t K, int64_t N, int64_t E, int64_t sorted_num, int64_t block_m)
{
    return static_cast<int64_t>(alpha_moe_workspace_bytes(static_cast<int>(top_k), static_cast<int>(M), static_cast<int>(K),
                                                          static_cast<int>(N), static_cast<int>(E),
                                                          static_cast<int>(sorted_num), static_cast<int>(block_m)));
}

void check_tensor(const at::Tensor &t, const char *name, at::ScalarType dtype, const at::Device &dev)
{
    TORCH_CHECK(t.defined(), name, " is undefined");
    TORCH_CHECK(t.device() == dev, name, " must be on ", dev, ", got ", t.device());
    TORCH_CHECK(t.scalar_type() == dtype, name, " must have dtype ", dtype, ", got ", t.scalar_type());
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

void run_fused_moe(const at::Tensor &x, const at::Tensor &x_scale, const at::Tensor &w, const at::Tensor &w_scale,
                   const at::Tensor &w2, const at::Tensor &w2_scale, const at::Tensor &sorted_token_ids,
                   const at::Tensor &expert_ids, const at::Tensor &num_tokens_post_padded,
                   const at::Tensor &topk_weights, at::Tensor &out, int64_t top_k, int64_t block_m, int64_t block_n,
                   int64_t warp_n, int64_t stages, double scaling_factor, bool store, bool prepacked = false)
{
    TORCH_CHECK(x.is_cuda(), "x must be a GPU tensor");
    const at::Device dev = x.device();
    check_tensor(x, "x", at::kFloat8_e4m3fn, dev);
    check_tensor(x_scale, "x_scale", at::kFloat, dev);
    check_tensor(w, "w", at::kFloat8_e4m3fn, dev);
    check_tensor(w_scale, "w_scale", at::kFloat, dev);
    check_tensor(w2, "w2", at::kFloat8_e4m3fn, dev);
    check_tensor(w2_scale, "w2_scale", at::kFloat, dev);
    check_tensor(sorted_token_ids, "sorted_token_ids", at::kInt, dev);
    check_tensor(expert_ids, "expert_ids", at::kInt, dev);
    check_tensor(num_tokens_post_padded, "num_tokens_post_padded", at::kInt, dev);
    check_tensor(topk_weights, "topk_weights", at::kFloat, dev);
    check_tensor(out, "out", at::kBFloat16, dev);

    TORCH_CHECK(x.dim() == 2 && x.size(0) > 0, "x must be [M, K] with M > 0");
    const int64_t M = x.size(0), K = x.size(1);
    TORCH_CHECK(K % 128 == 0, "K dimension must be a multiple of 128");
    int64_t E, N;
    if (!prepacked) {
        TORCH_CHECK(w.dim() == 3 && w.size(2) == K, "w must be [E, N, K] with the K of x");
        E = w.size(0), N = w.size(1);
        TORCH_CHECK(N % 256 == 0, "N (= 2 * intermediate size) must be a multiple of 256");
        TORCH_CHECK(w2.dim() == 3 && w2.size(0) == E && w2.size(1) == K && w2.size(2) == N / 2, "w2 must be [E, K, N/2]");
    } else {
        TORCH_CHECK(w.dim() == 4 && w.size(1) == K / 128 && w.size(3) == 128,
                    "w_packed must be [E, K/128, N, 128] with the K of x (alpha_moe_python.utils.prepack_weights)");
        E = w.size(0), N = w.size(2);
        TORCH_CHECK(N % 256 == 0, "N (= 2 * intermediate size) must be a multiple of 256");
        TORCH_CHECK(w2.dim() == 4 && w2.size(0) == E && w2.size(1) == N / 256 && w2.size(2) == K && w2.size(3) == 128,
                    "w2_packed must be [E, N/256, K, 128]");
    }
    TORCH_CHECK(x_scale.numel() == M * (K / 128), "x_scale must be [M, K/128]");
    TORCH_CHECK(w_scale.numel() == E * (N / 128) * (K / 128), "w_scale must be [E, N/128, K/128]");
    TORCH_CHECK(w2_scale.numel() == E * (K / 128) * (N / 256), "w2_scale must be [E, K/128, N/256]");
    TORCH_CHECK(out.dim() == 2 && out.size(0) == M && out.size(1) == K, "out must be [M, K]");
    TORCH_CHECK(top_k > 0 && topk_weights.numel() == M * top_k, "topk_weights must hold M * top_k values");
    TORCH_CHECK((block_n == 64 && warp_n == 4) || (block_n == 32 && warp_n == 8),
                "(block_n, warp_n) must be (64, 4) or (32, 8)");
    TORCH_CHECK(stages > 0 && stages < 6, "stages must be in [1, 5]");
    TORCH_CHECK(block_m > 0 && block_m <= 128 && block_m % 8 == 0, "block_m must be a multiple of 8 in [8, 128]");
    const int64_t sorted_num = sorted_token_ids.numel();
    TORCH_CHECK(sorted_num > 0, "sorted_token_ids is empty");
    TORCH_CHECK(expert_ids.numel() >= (sorted_num + block_m - 1) / block_m,
                "expert_ids must hold one entry per block_m rows of sorted_token_ids");
    TORCH_CHECK(num_tokens_post_padded.numel() >= 1, "num_tokens_post_padded must hold one value");
    TORCH_CHECK(M * top_k <= INT32_MAX && sorted_num <= INT32_MAX && E <= INT32_MAX, "sizes exceed int32");

    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(dev);
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();

    const size_t ws_bytes =
        alpha_moe_workspace_bytes(static_cast<int>(top_k), static_cast<int>(M), static_cast<int>(K), static_cast<int>(N),
                                  static_cast<int>(E), static_cast<int>(sorted_num), static_cast<int>(block_m));
    at::Tensor ws = workspace_for(dev, stream, ws_bytes);

    const int rc = (prepacked ?
        alpha_moe_fused_moe_w8a8_up_down_prepacked(
            static_cast<const uint8_t *>(x.const_data_ptr()), x_scale.const_data_ptr<float>(),
            static_cast<const uint8_t *>(w.const_data_ptr()), w_scale.const_data_ptr<float>(),
            static_cast<const uint8_t *>(w2.const_data_ptr()), w2_scale.const_data_ptr<float>(),
            static_cast<uint16_t *>(out.data_ptr()), sorted_token_ids.const_data_ptr<int32_t>(),
            expert_ids.const_data_ptr<int32_t>(), num_tokens_post_padded.const_data_ptr<int32_t>(),
            topk_weights.const_data_ptr<float>(), static_cast<int>(top_k), static_cast<int>(M), static_cast<int>(K),
            static_cast<int>(N), static_cast<int>(E), static_cast<int>(sorted_num), static_cast<int>(block_m),
            static_cast<int>(block_n), static_cast<int>(warp_n), static_cast<int>(stages),
            static_cast<float>(scaling_factor), store ? 1 : 0, ws.data_ptr(), static_cast<size_t>(ws.numel()),
            static_cast<void *>(stream))
        : (store ? alpha_moe_fused_moe_w8a8_up_down_store : alpha_moe_fused_moe_w8a8_up_down)(
            static_cast<const uint8_t *>(x.const_data_ptr()), x_scale.const_data_ptr<float>(),
            static_cast<const uint8_t *>(w.const_data_ptr()), w_scale.const_data_ptr<float>(),
            static_cast<const uint8_t *>(w2.const_data_ptr()), w2_scale.const_data_ptr<float>(),
            static_cast<uint16_t *>(out.data_ptr()), sorted_token_ids.const_data_ptr<int32_t>(),
            expert_ids.const_data_ptr<int32_t>(), num_tokens_post_padded.const_data_ptr<int32_t>(),
            topk_weights.const_data_ptr<float>(), static_cast<int>(top_k), static_cast<int>(M), static_cast<int>(K),
            static_cast<int>(N), static_cast<int>(E), static_cast<int>(sorted_num), static_cast<int>(block_m),
            static_cast<int>(block_n), static_cast<int>(warp_n), static_cast<int>(stages),
            static_cast<float>(scaling_factor), ws.data_ptr(), static_cast<size_t>(ws.numel()),
            static_cast<void *>(stream)));
    TORCH_CHECK(rc == ALPHA_MOE_OK, "alpha_moe_fused_moe_w8a8_up_down failed: ", alpha_moe_status_string(rc));
}

void fused_moe_w8a8_up_down(const at::Tensor &x, const at::Tensor &x_scale, const at::Tensor &w,
                            const at::Tensor &w_scale, const at::Tensor &w2, const at::Tensor &w2_scale,
                            const at::Tensor &sorted_token_ids, const at::Tensor &expert_ids,
                            const at::Tensor &num_tokens_post_padded, const at::Tensor &topk_weights,
                            at::Tensor &out, int64_t top_k, int64_t block_m, int64_t block_n, int64_t warp_n,
                            int64_t stages, double scaling_factor)
{
    run_fused_moe(x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
                  topk_weights, out, top_k, block_m, block_n, warp_n, stages, scaling_factor, false);
}

// Store semantics: out = bf16(sum) whatever it held, so the caller need not zero-fill it first.
void fused_moe_w8a8_up_down_store(const at::Tensor &x, const at::Tensor &x_scale, const at::Tensor &w,
                                  const at::Tensor &w_scale, const at::Tensor &w2, const at::Tensor &w2_scale,
                                  const at::Tensor &sorted_token_ids, const at::Tensor &expert_ids,
                                  const at::Tensor &num_tokens_post_padded, const at::Tensor &topk_weights,
                                  at::Tensor &out, int64_t top_k, int64_t block_m, int64_t block_n, int64_t warp_n,
                                  int64_t stages, double scaling_factor)
{
    run_fused_moe(x, x_scale, w, w_scale, w2, w2_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
                  topk_weights, out, top_k, block_m, block_n, warp_n, stages, scaling_factor, true);
}

// The operator on weights re-laid-out by alpha_moe_python.utils.prepack_weights: w_packed [E, K/128, N, 128],
// w2_packed [E, I/128, K, 128]; store selects the overwriting variant.
void fused_moe_w8a8_up_down_prepacked(const at::Tensor &x, const at::Tensor &x_scale, const at::Tensor &w_packed,
                                      const at::Tensor &w_scale, const at::Tensor &w2_packed, const at::Tensor &w2_scale,
                                      const at::Tensor &sorted_token_ids, const at::Tensor &expert_ids,
                                      const at::Tensor &num_tokens_post_padded, const at::Tensor &topk_weights,
                                      at::Tensor &out, int64_t top_k, int64_t block_m, int64_t block_n, int64_t warp_n,
                                      int64_t stages, double scaling_factor, bool store)
{
    run_fused_moe(x, x_scale, w_packed, w_scale, w2_packed, w2_scale, sorted_token_ids, expert_ids,
                  num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n, stages, scaling_factor, store,
                  true);
}

// (q, scale) = per_token_group_quant_fp8(x, 128): what the reference's callers get from SGLang (jit_moe.py:142).
std::tuple<at::Tensor, at::Tensor> per_token_group_quant_fp8(const at::Tensor &x, int64_t group_size)
{
    TORCH_CHECK(x.is_cuda(), "x must be a GPU tensor");
    TORCH_CHECK(group_size == 128, "group_size must be 128");
    TORCH_CHECK(x.dim() == 2 && x.size(1) % 128 == 0 && x.size(0) > 0, "x must be [M, K] with K % 128 == 0");
    TORCH_CHECK(x.scalar_type() == at::kBFloat16 || x.scalar_type() == at::kFloat, "x must be bfloat16 or float32");
    TORCH_CHECK(x.is_contiguous(), "x must be contiguous");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(x.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    at::Tensor q = at::empty(x.sizes(), x.options().dtype(at::kFloat8_e4m3fn));
    at::Tensor scale = at::empty({x.size(0), x.size(1) / 128}, x.options().dtype(at::kFloat));
    const int rc = alpha_moe_per_token_group_quant_fp8(x.const_data_ptr(), x.scalar_type() == at::kFloat,
                                                       static_cast<uint8_t *>(q.data_ptr()), scale.data_ptr<float>(),
                                                       static_cast<int>(x.size(0)), static_cast<int>(x.size(1)),
                                                       static_cast<void *>(stream));
    TORCH_CHECK(rc == ALPHA_MOE_OK, "alpha_moe_per_token_group_quant_fp8 failed: ", alpha_moe_status_string(rc));
    return {q, scale};
}

// (sorted_token_ids, expert_ids, num_tokens_post_padded) = moe_align_block_size(topk_ids, block_size, num_experts):
// what the reference's callers get from SGLang (jit_moe.py:158).
std::tuple<at::Tensor, at::Tensor, at::Tensor> moe_align_block_size(const at::Tensor &topk_ids, int64_t block_size,
                                                                    int64_t num_experts)
{
    TORCH_CHECK(topk_ids.is_cuda(), "topk_ids must be a GPU tensor");
    TORCH_CHECK(topk_ids.scalar_type() == at::kInt, "topk_ids must be int32");
    TORCH_CHECK(topk_ids.is_contiguous() && topk_ids.numel() > 0, "topk_ids must be contiguous and not empty");
    TORCH_CHECK(block_size > 0 && num_experts > 0, "block_size and num_experts must be positive");
    const int64_t numel = topk_ids.numel();
    const int64_t sorted_num = numel + num_experts * (block_size - 1);
    const int64_t n_blocks = (sorted_num + block_size - 1) / block_size;
    TORCH_CHECK(sorted_num <= INT32_MAX, "too many routing slots");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(topk_ids.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const auto opts = topk_ids.options();
    at::Tensor sorted_ids = at::empty({sorted_num}, opts), expert_ids = at::empty({n_blocks}, opts),
               total = at::empty({1}, opts);
    const size_t ws_bytes = alpha_moe_align_workspace_bytes(static_cast<int>(numel), static_cast<int>(num_experts));
    at::Tensor ws = at::empty({static_cast<int64_t>(ws_bytes)}, opts.dtype(at::kByte));
    const int rc = alpha_moe_moe_align_block_size(
        topk_ids.const_data_ptr<int32_t>(), static_cast<int>(numel), static_cast<int>(num_experts),
        static_cast<int>(block_size), sorted_ids.data_ptr<int32_t>(), static_cast<int>(sorted_num),
        expert_ids.data_ptr<int32_t>(), static_cast<int>(n_blocks), total.data_ptr<int32_t>(), ws.data_ptr(), ws_bytes,
        static_cast<void *>(stream));
    TORCH_CHECK(rc == ALPHA_MOE_OK, "alpha_moe_moe_align_block_size failed: ", alpha_moe_status_string(rc));
    return {sorted_ids, expert_ids, total};
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(alpha_moe, m)
{
    m.def("per_token_group_quant_fp8(Tensor x, int group_size) -> (Tensor, Tensor)");
    m.impl("per_token_group_quant_fp8", c10::DispatchKey::CUDA, &per_token_group_quant_fp8);
    m.def("moe_align_block_size(Tensor topk_ids, int block_size, int num_experts) -> (Tensor, Tensor, Tensor)");
    m.impl("moe_align_block_size", c10::DispatchKey::CUDA, &moe_align_block_size);
    m.def("reserve_workspace(Tensor like, int bytes) -> ()");
    m.impl("reserve_workspace", c10::DispatchKey::CUDA, &reserve_workspace);
    m.def("scratch_buffers(Tensor like) -> int[]");
    m.impl("scratch_buffers", c10::DispatchKey::CUDA, &scratch_buffers);
    m.def("workspace_bytes(int top_k, int M, int K, int N, int E, int sorted_num, int block_m) -> int", &workspace_bytes);
    m.def("fused_moe_w8a8_up_down("
          "Tensor x, Tensor x_scale, Tensor w, Tensor w_scale, Tensor w2, Tensor w2_scale, "
          "Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, Tensor topk_weights, "
          "Tensor(a!) out, int top_k, int block_m, int block_n, int warp_n, int stages, float scaling_factor"
          ") -> ()");
    // GPU tensors of PyTorch-ROCm carry the dispatch key named CUDA
    m.impl("fused_moe_w8a8_up_down", c10::DispatchKey::CUDA, &fused_moe_w8a8_up_down);
    m.def("fused_moe_w8a8_up_down_store("
          "Tensor x, Tensor x_scale, Tensor w, Tensor w_scale, Tensor w2, Tensor w2_scale, "
          "Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, Tensor topk_weights, "
          "Tensor(a!) out, int top_k, int block_m, int block_n, int warp_n, int stages, float scaling_factor"
          ") -> ()");
    m.impl("fused_moe_w8a8_up_down_store", c10::DispatchKey::CUDA, &fused_moe_w8a8_up_down_store);
    m.def("fused_moe_w8a8_up_down_prepacked("
          "Tensor x, Tensor x_scale, Tensor w_packed, Tensor w_scale, Tensor w2_packed, Tensor w2_scale, "
          "Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, Tensor topk_weights, "
          "Tensor(a!) out, int top_k, int block_m, int block_n, int warp_n, int stages, float scaling_factor, bool store"
          ") -> ()");
    m.impl("fused_moe_w8a8_up_down_prepacked", c10::DispatchKey::CUDA, &fused_moe_w8a8_up_down_prepacked);
}
