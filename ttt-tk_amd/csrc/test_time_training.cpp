// Python operator module `test_time_training` for ROCm: the same two functions, positional
// argument lists, tensor layouts and return value as the upstream binding
// (test_time_training.cpp:25-42, :47-91, :95-105), implemented on top of the C ABI in
// include/ttt_mlp.h.  Shape / dtype / device / contiguity problems raise (TORCH_CHECK ->
// RuntimeError) like upstream (kernels/ttt/ttt.cu:621-630, kernels/ttt_backward/ttt.cu:1507-1760);
// unlike upstream, launch and execution errors raise as well instead of being printed.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include "../../include/ttt_mlp.h"

namespace {

constexpr int64_t F = TTT_MLP_F, CS = TTT_MLP_CS, HID = TTT_MLP_HID;
bool g_synchronize = true;  // upstream blocks the host until the kernel has finished
bool g_fill_group_tensors = false;   // leave the values of checkpoint group 0 in the sixteen *_group tensors
bool g_accumulate = true;            // grad_L_XQ / XK / XV / last_eta are added to (upstream behaviour) rather than overwritten
bool g_overlap = true;      // two workgroups per (batch, head) whenever they fit the device
unsigned long long g_wait_ticks = 2000000000ull;   // mirrors the library's limit, for the error text
torch::Tensor* g_sticky = nullptr;   // a device int, non-zero once a launch that nobody waited for gave up a wait (never freed:
                                     // a static tensor would be destroyed after the runtime at process exit)
torch::Tensor* g_workspace = nullptr;   // caller-owned workspace of the multi-workgroup launches (set_workspace); never freed here
int g_last_forward_mode = -1;    // 0 = one workgroup per (batch, head), 1 = two
int g_last_backward_mode = -1;

void check_tensor(const torch::Tensor& t, const char* name, c10::ScalarType dtype, std::initializer_list<int64_t> shape) {
  TORCH_CHECK(t.device().is_cuda(), "Invalid dims for ", name, ": not a GPU tensor");
  TORCH_CHECK(t.is_contiguous(), "Invalid dims for ", name, ": not contiguous");
  TORCH_CHECK(t.scalar_type() == dtype, "Invalid dtype for ", name, ": expected ", c10::toString(dtype), ", got ",
              c10::toString(t.scalar_type()));
  TORCH_CHECK(t.dim() == (int64_t)shape.size(), "Invalid dims for ", name, ": expected ", shape.size(), " dims, got ", t.dim());
  int64_t d = 0;
  for (int64_t s : shape) {
    TORCH_CHECK(s < 0 || t.size(d) == s, "Invalid dims for ", name, ": size(", d, ") is ", t.size(d), ", expected ", s);
    ++d;
  }
}

// last_eta is [B,NH,NC,CS,1]; the upstream forward also accepts [B,NH,NC,CS] (same bytes).
void check_eta(const torch::Tensor& t, const char* name, int64_t B, int64_t NH, int64_t NC, bool allow_4d) {
  if (allow_4d && t.dim() == 4) check_tensor(t, name, torch::kBFloat16, {B, NH, NC, CS});
  else check_tensor(t, name, torch::kBFloat16, {B, NH, NC, CS, 1});
}

const uint16_t* bfp(const torch::Tensor& t) { return reinterpret_cast<const uint16_t*>(t.data_ptr<at::BFloat16>()); }
uint16_t* bfp_mut(const torch::Tensor& t) { return reinterpret_cast<uint16_t*>(t.data_ptr<at::BFloat16>()); }

// `status` (may be null): device address of the status word of a launch with several workgroups per
// (batch, head); it can only be looked at when the host waits for the stream anyway.
std::string gave_up_text() {
  return "a workgroup waited " + std::to_string(g_wait_ticks / 100000000.0) + " s for its partner and gave up (were all "
         "compute units available to this launch?); the outputs are invalid - set_overlap(False) avoids the mode";
}

// The device int that collects the status words of launches the host did not wait for.
int* sticky_word(const torch::Device& dev) {
  if (g_sticky == nullptr || g_sticky->device() != dev)
    g_sticky = new torch::Tensor(torch::zeros({1}, torch::TensorOptions().dtype(torch::kInt32).device(dev)));
  return g_sticky->data_ptr<int>();
}

void finish(int rc, hipStream_t stream, const char* what, const torch::Device& dev, const void* status = nullptr) {
  TORCH_CHECK(rc == TTT_MLP_OK, what, " launch failed: ", ttt_mlp_error_string(rc));
  if (!g_synchronize && status != nullptr) {
    // nobody looks at the status word before the workspace goes back to the allocator: fold it into a word that stays
    rc = ttt_mlp_status_accumulate(status, sticky_word(dev), stream);
    TORCH_CHECK(rc == TTT_MLP_OK, what, " launch failed: ", ttt_mlp_error_string(rc));
  }
  if (g_synchronize) {
    hipError_t e = hipStreamSynchronize(stream);
    TORCH_CHECK(e == hipSuccess, what, " execution failed: ", hipGetErrorString(e));
    if (status != nullptr) {
      int word = 0;
      e = hipMemcpy(&word, status, sizeof(int), hipMemcpyDeviceToHost);
      TORCH_CHECK(e == hipSuccess, what, " execution failed: ", hipGetErrorString(e));
      TORCH_CHECK(word == 0, what, ": ", gave_up_text());
    }
  }
}

// The multi-workgroup launches are an optimisation: not worth failing (or evicting the caller's cached
// blocks) for.  They are used only if their workspace fits comfortably into what the device has free
// (memory held by torch's caching allocator counts as free for torch, so this is conservative).
bool workspace_is_affordable(size_t bytes) {
  if (bytes == 0) return false;
  size_t free_b = 0, total_b = 0;
  if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return false;
  return bytes <= free_b / 2;
}

// Where the workspace of a multi-workgroup launch comes from.  With a caller-owned workspace (set_workspace) the
// operators allocate nothing and ask the device nothing: the launch uses it if it is large enough and on the right
// device, and falls back to one workgroup per (batch, head) otherwise.  Without one the workspace comes from torch's
// caching allocator (which orders its reuse after the launch on the same stream) if the device has room to spare.
// Whether the launcher would cut the sequences of this shape at checkpoints even with a workspace at hand (it then runs
// one workgroup per pair and the workspace would go unused).
bool sequences_cut(int which, int64_t pairs, int64_t NC, int64_t cgs) {
  int seg = 0, launches = 0;
  if (ttt_mlp_segment_plan(which, (long long)pairs, 0, (int)NC, (int)cgs, 1, &seg, &launches) != 0) return false;
  return seg > 0;
}

struct Workspace {
  void* ptr = nullptr;
  torch::Tensor held;   // keeps an allocated workspace alive until the launch has been enqueued
};
Workspace take_workspace(size_t bytes, const torch::Device& dev) {
  Workspace w;
  if (bytes == 0) return w;
  if (g_workspace != nullptr) {
    if (g_workspace->device() == dev && (size_t)g_workspace->numel() >= bytes) w.ptr = g_workspace->data_ptr();
    return w;
  }
  if (!workspace_is_affordable(bytes)) return w;
  w.held = torch::empty({(int64_t)bytes}, torch::TensorOptions().dtype(torch::kUInt8).device(dev));
  w.ptr = w.held.data_ptr();
  return w;
}

}  // namespace

torch::Tensor ttt_forward(const torch::Tensor XQ, const torch::Tensor XK, const torch::Tensor XV,
                          const torch::Tensor last_eta, const torch::Tensor ttt_norm_weight,
                          const torch::Tensor ttt_norm_bias, const torch::Tensor W1, const torch::Tensor b1,
                          const torch::Tensor W2, const torch::Tensor b2, const torch::Tensor W1_checkpoints,
                          const torch::Tensor b1_checkpoints, const torch::Tensor W2_checkpoints,
                          const torch::Tensor b2_checkpoints, const torch::Tensor Out, const int checkpoint_group_size) {
  TORCH_CHECK(XQ.dim() == 5, "Invalid dims for XQ");
  const int64_t B = XQ.size(0), NH = XQ.size(1), NC = XQ.size(2);
  TORCH_CHECK(W1_checkpoints.dim() == 5, "Invalid dims for W1_checkpoints");
  const int64_t K = W1_checkpoints.size(2);
  TORCH_CHECK(checkpoint_group_size > 0, "checkpoint_group_size must be positive");
  TORCH_CHECK(K == (NC + checkpoint_group_size - 1) / checkpoint_group_size,
              "Invalid dims for W1_checkpoints: ", K, " checkpoints for ", NC, " mini-batches in groups of ", checkpoint_group_size);
  check_tensor(XQ, "XQ", torch::kBFloat16, {B, NH, NC, CS, F});
  check_tensor(XK, "XK", torch::kBFloat16, {B, NH, NC, CS, F});
  check_tensor(XV, "XV", torch::kBFloat16, {B, NH, NC, CS, F});
  check_eta(last_eta, "last_eta", B, NH, NC, true);
  check_tensor(ttt_norm_weight, "ttt_norm_weight", torch::kFloat32, {1, NH, 1, F});
  check_tensor(ttt_norm_bias, "ttt_norm_bias", torch::kFloat32, {1, NH, 1, F});
  check_tensor(W1, "W1", torch::kFloat32, {B, NH, F, HID});
  check_tensor(b1, "b1", torch::kFloat32, {B, NH, 1, HID});
  check_tensor(W2, "W2", torch::kFloat32, {B, NH, HID, F});
  check_tensor(b2, "b2", torch::kFloat32, {B, NH, 1, F});
  check_tensor(W1_checkpoints, "W1_checkpoints", torch::kFloat32, {B, NH, K, F, HID});
  check_tensor(b1_checkpoints, "b1_checkpoints", torch::kFloat32, {B, NH, K, 1, HID});
  check_tensor(W2_checkpoints, "W2_checkpoints", torch::kFloat32, {B, NH, K, HID, F});
  check_tensor(b2_checkpoints, "b2_checkpoints", torch::kFloat32, {B, NH, K, 1, F});
  check_tensor(Out, "Out", torch::kBFloat16, {B, NH, NC, CS, F});

  ttt_mlp_fwd_args a;
  a.XQ = bfp(XQ); a.XK = bfp(XK); a.XV = bfp(XV); a.last_eta = bfp(last_eta);
  a.ttt_norm_weight = ttt_norm_weight.data_ptr<float>(); a.ttt_norm_bias = ttt_norm_bias.data_ptr<float>();
  a.W1 = W1.data_ptr<float>(); a.b1 = b1.data_ptr<float>(); a.W2 = W2.data_ptr<float>(); a.b2 = b2.data_ptr<float>();
  a.W1_checkpoints = W1_checkpoints.data_ptr<float>(); a.b1_checkpoints = b1_checkpoints.data_ptr<float>();
  a.W2_checkpoints = W2_checkpoints.data_ptr<float>(); a.b2_checkpoints = b2_checkpoints.data_ptr<float>();
  a.Out = bfp_mut(Out);
  a.checkpoint_group_size = checkpoint_group_size;
  a.B = (int32_t)B; a.NH = (int32_t)NH; a.NC = (int32_t)NC; a.K = (int32_t)K;
  const c10::DeviceGuard guard(XQ.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(XQ.device().index()).stream();
  // With few (batch, head) pairs most CUs would idle: then a second workgroup per pair computes Out behind
  // the state recurrence.  Its workspace: the caller's (set_workspace) or torch's caching allocator's.
  // (more pairs than CUs and sequences that the launcher cuts at checkpoints: no second workgroup, no workspace)
  const size_t ws_bytes = (g_overlap && NC >= 2 && !sequences_cut(0, B * NH, NC, checkpoint_group_size))
                              ? ttt_mlp_fwd_workspace_bytes((int32_t)B, (int32_t)NH) : 0;
  const Workspace ws = take_workspace(ws_bytes, XQ.device());
  if (ws.ptr != nullptr) {
    g_last_forward_mode = 1;
    const char* status = static_cast<const char*>(ws.ptr) + ttt_mlp_fwd_status_offset((int32_t)B, (int32_t)NH);
    finish(ttt_mlp_fwd_launch_overlapped(&a, ws.ptr, ws_bytes, stream), stream, "ttt_forward", XQ.device(), status);
  } else {
    g_last_forward_mode = 0;
    finish(ttt_mlp_fwd_launch(&a, stream), stream, "ttt_forward", XQ.device());
  }
  return Out;
}

torch::Tensor ttt_backward(
    const torch::Tensor XQ, const torch::Tensor XK, const torch::Tensor XV, const torch::Tensor last_eta,
    const torch::Tensor ttt_norm_weight, const torch::Tensor ttt_norm_bias, const torch::Tensor W1_checkpoints,
    const torch::Tensor b1_checkpoints, const torch::Tensor W2_checkpoints, const torch::Tensor b2_checkpoints,
    const torch::Tensor Out, const torch::Tensor W1_init_group, const torch::Tensor b1_init_group,
    const torch::Tensor W2_init_group, const torch::Tensor b2_init_group, const torch::Tensor x_hat_ln_group,
    const torch::Tensor std_ln_group, const torch::Tensor X2_group, const torch::Tensor Z1_group,
    const torch::Tensor Z1_bar_group, const torch::Tensor X2_bar_group, const torch::Tensor grad_l_wrt_Z2_group,
    const torch::Tensor grad_l_wrt_Z1_group, const torch::Tensor x_hat_fused_group,
    const torch::Tensor grad_x_hat_fused_group, const torch::Tensor grad_output_fused_group,
    const torch::Tensor std_fused_group, const torch::Tensor grad_L_W1_last, const torch::Tensor grad_L_b1_last,
    const torch::Tensor grad_L_W2_last, const torch::Tensor grad_L_b2_last, const torch::Tensor grad_L_XQW_mini_batch,
    const torch::Tensor grad_L_ttt_norm_weight, const torch::Tensor grad_L_ttt_norm_bias,
    const torch::Tensor grad_L_W1_init, const torch::Tensor grad_L_b1_init, const torch::Tensor grad_L_W2_init,
    const torch::Tensor grad_L_b2_init, const torch::Tensor grad_L_last_eta, const torch::Tensor grad_L_XQ,
    const torch::Tensor grad_L_XK, const torch::Tensor grad_L_XV, const int checkpoint_group_size) {
  TORCH_CHECK(XQ.dim() == 5, "Invalid dims for XQ");
  const int64_t B = XQ.size(0), NH = XQ.size(1), NC = XQ.size(2);
  TORCH_CHECK(W1_checkpoints.dim() == 5, "Invalid dims for W1_checkpoints");
  const int64_t K = W1_checkpoints.size(2);
  const int64_t G = checkpoint_group_size;
  TORCH_CHECK(G > 0, "checkpoint_group_size must be positive");
  TORCH_CHECK(K == (NC + G - 1) / G, "Invalid dims for W1_checkpoints: ", K, " checkpoints for ", NC,
              " mini-batches in groups of ", G);
  const auto bf = torch::kBFloat16;
  const auto f32 = torch::kFloat32;
  check_tensor(XQ, "XQ", bf, {B, NH, NC, CS, F});
  check_tensor(XK, "XK", bf, {B, NH, NC, CS, F});
  check_tensor(XV, "XV", bf, {B, NH, NC, CS, F});
  check_eta(last_eta, "last_eta", B, NH, NC, false);
  check_tensor(ttt_norm_weight, "ttt_norm_weight", f32, {1, NH, 1, F});
  check_tensor(ttt_norm_bias, "ttt_norm_bias", f32, {1, NH, 1, F});
  check_tensor(W1_checkpoints, "W1_checkpoints", f32, {B, NH, K, F, HID});
  check_tensor(b1_checkpoints, "b1_checkpoints", f32, {B, NH, K, 1, HID});
  check_tensor(W2_checkpoints, "W2_checkpoints", f32, {B, NH, K, HID, F});
  check_tensor(b2_checkpoints, "b2_checkpoints", f32, {B, NH, K, 1, F});
  check_tensor(Out, "Out", bf, {B, NH, NC, CS, F});
  check_tensor(W1_init_group, "W1_init_group", f32, {B, NH, G, F, HID});
  check_tensor(b1_init_group, "b1_init_group", f32, {B, NH, G, 1, HID});
  check_tensor(W2_init_group, "W2_init_group", f32, {B, NH, G, HID, F});
  check_tensor(b2_init_group, "b2_init_group", f32, {B, NH, G, 1, F});
  check_tensor(x_hat_ln_group, "x_hat_ln_group", bf, {B, NH, G, CS, F});
  check_tensor(std_ln_group, "std_ln_group", f32, {B, NH, G, CS, 1});
  check_tensor(X2_group, "X2_group", bf, {B, NH, G, CS, HID});
  check_tensor(Z1_group, "Z1_group", bf, {B, NH, G, CS, HID});
  check_tensor(Z1_bar_group, "Z1_bar_group", bf, {B, NH, G, CS, HID});
  check_tensor(X2_bar_group, "X2_bar_group", bf, {B, NH, G, CS, HID});
  check_tensor(grad_l_wrt_Z2_group, "grad_l_wrt_Z2_group", bf, {B, NH, G, CS, F});
  check_tensor(grad_l_wrt_Z1_group, "grad_l_wrt_Z1_group", bf, {B, NH, G, CS, HID});
  check_tensor(x_hat_fused_group, "x_hat_fused_group", bf, {B, NH, G, CS, F});
  check_tensor(grad_x_hat_fused_group, "grad_x_hat_fused_group", bf, {B, NH, G, CS, F});
  check_tensor(grad_output_fused_group, "grad_output_fused_group", bf, {B, NH, G, CS, F});
  check_tensor(std_fused_group, "std_fused_group", f32, {B, NH, G, CS, 1});
  check_tensor(grad_L_W1_last, "grad_L_W1_last", f32, {B, NH, F, HID});
  check_tensor(grad_L_b1_last, "grad_L_b1_last", f32, {B, NH, 1, HID});
  check_tensor(grad_L_W2_last, "grad_L_W2_last", f32, {B, NH, HID, F});
  check_tensor(grad_L_b2_last, "grad_L_b2_last", f32, {B, NH, 1, F});
  check_tensor(grad_L_XQW_mini_batch, "grad_L_XQW_mini_batch", bf, {B, NH, NC, CS, F});
  check_tensor(grad_L_ttt_norm_weight, "grad_L_ttt_norm_weight", f32, {B, NH, 1, F});
  check_tensor(grad_L_ttt_norm_bias, "grad_L_ttt_norm_bias", f32, {B, NH, 1, F});
  check_tensor(grad_L_W1_init, "grad_L_W1_init", f32, {B, NH, F, HID});
  check_tensor(grad_L_b1_init, "grad_L_b1_init", f32, {B, NH, 1, HID});
  check_tensor(grad_L_W2_init, "grad_L_W2_init", f32, {B, NH, HID, F});
  check_tensor(grad_L_b2_init, "grad_L_b2_init", f32, {B, NH, 1, F});
  check_tensor(grad_L_last_eta, "grad_L_last_eta", bf, {B, NH, NC, CS, 1});
  check_tensor(grad_L_XQ, "grad_L_XQ", bf, {B, NH, NC, CS, F});
  check_tensor(grad_L_XK, "grad_L_XK", bf, {B, NH, NC, CS, F});
  check_tensor(grad_L_XV, "grad_L_XV", bf, {B, NH, NC, CS, F});

  ttt_mlp_bwd_args a;
  a.XQ = bfp(XQ); a.XK = bfp(XK); a.XV = bfp(XV); a.last_eta = bfp(last_eta);
  a.ttt_norm_weight = ttt_norm_weight.data_ptr<float>(); a.ttt_norm_bias = ttt_norm_bias.data_ptr<float>();
  a.W1_checkpoints = W1_checkpoints.data_ptr<float>(); a.b1_checkpoints = b1_checkpoints.data_ptr<float>();
  a.W2_checkpoints = W2_checkpoints.data_ptr<float>(); a.b2_checkpoints = b2_checkpoints.data_ptr<float>();
  a.Out = bfp_mut(Out);
  a.W1_init_group = W1_init_group.data_ptr<float>(); a.b1_init_group = b1_init_group.data_ptr<float>();
  a.W2_init_group = W2_init_group.data_ptr<float>(); a.b2_init_group = b2_init_group.data_ptr<float>();
  a.x_hat_ln_group = bfp_mut(x_hat_ln_group); a.std_ln_group = std_ln_group.data_ptr<float>();
  a.X2_group = bfp_mut(X2_group); a.Z1_group = bfp_mut(Z1_group);
  a.Z1_bar_group = bfp_mut(Z1_bar_group); a.X2_bar_group = bfp_mut(X2_bar_group);
  a.grad_l_wrt_Z2_group = bfp_mut(grad_l_wrt_Z2_group); a.grad_l_wrt_Z1_group = bfp_mut(grad_l_wrt_Z1_group);
  a.x_hat_fused_group = bfp_mut(x_hat_fused_group); a.grad_x_hat_fused_group = bfp_mut(grad_x_hat_fused_group);
  a.grad_output_fused_group = bfp_mut(grad_output_fused_group); a.std_fused_group = std_fused_group.data_ptr<float>();
  a.grad_L_W1_last = grad_L_W1_last.data_ptr<float>(); a.grad_L_b1_last = grad_L_b1_last.data_ptr<float>();
  a.grad_L_W2_last = grad_L_W2_last.data_ptr<float>(); a.grad_L_b2_last = grad_L_b2_last.data_ptr<float>();
  a.grad_L_XQW_mini_batch = bfp(grad_L_XQW_mini_batch);
  a.grad_L_ttt_norm_weight = grad_L_ttt_norm_weight.data_ptr<float>();
  a.grad_L_ttt_norm_bias = grad_L_ttt_norm_bias.data_ptr<float>();
  a.grad_L_W1_init = grad_L_W1_init.data_ptr<float>(); a.grad_L_b1_init = grad_L_b1_init.data_ptr<float>();
  a.grad_L_W2_init = grad_L_W2_init.data_ptr<float>(); a.grad_L_b2_init = grad_L_b2_init.data_ptr<float>();
  a.grad_L_last_eta = bfp_mut(grad_L_last_eta);
  a.grad_L_XQ = bfp_mut(grad_L_XQ); a.grad_L_XK = bfp_mut(grad_L_XK); a.grad_L_XV = bfp_mut(grad_L_XV);
  a.checkpoint_group_size = checkpoint_group_size;
  a.B = (int32_t)B; a.NH = (int32_t)NH; a.NC = (int32_t)NC; a.K = (int32_t)K;
  a.overwrite = g_accumulate ? 0 : 1;
  const c10::DeviceGuard guard(XQ.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(XQ.device().index()).stream();
  // With few (batch, head) pairs most CUs would idle: then a second workgroup per pair recomputes the
  // checkpoint groups ahead of the reverse walk.  Its workspace (further sets of the per-group tensors): the
  // caller's (set_workspace) or torch's caching allocator's.
  const size_t ws_bytes = (g_overlap && K >= 2 && !sequences_cut(1, B * NH, NC, checkpoint_group_size))
                              ? ttt_mlp_bwd_workspace_bytes((int32_t)B, (int32_t)NH, checkpoint_group_size) : 0;
  const Workspace ws = take_workspace(ws_bytes, XQ.device());
  if (ws.ptr != nullptr) {
    g_last_backward_mode = 1;
    const char* status = static_cast<const char*>(ws.ptr) + ttt_mlp_bwd_status_offset((int32_t)B, (int32_t)NH);
    int rc = ttt_mlp_bwd_launch_overlapped(&a, ws.ptr, ws_bytes, stream);
    if (rc == 0 && g_fill_group_tensors) rc = ttt_mlp_bwd_export_group0(&a, stream);
    finish(rc, stream, "ttt_backward", XQ.device(), status);
  } else {
    g_last_backward_mode = 0;
    int rc = ttt_mlp_bwd_launch(&a, stream);
    if (rc == 0 && g_fill_group_tensors) rc = ttt_mlp_bwd_export_group0(&a, stream);
    finish(rc, stream, "ttt_backward", XQ.device());
  }
  return Out;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "Test Time Training Kernels";
  m.def("ttt_forward", &ttt_forward, "TTT Forward.");
  m.def("ttt_backward", &ttt_backward, "TTT Backward.");
  // Not part of the upstream module: lets a harness time launches with events instead of paying
  // the host synchronisation the upstream operator performs on every call.
  m.def("set_synchronize", [](bool on) { g_synchronize = on; }, "Block the host after each launch (default true).");
  m.def("abi_version", []() { return ttt_mlp_abi_version(); });
  // Also not upstream: choice of the launch shape (results are bit-identical either way).
  m.def("set_overlap", [](bool on) { g_overlap = on; },
        "Use a second workgroup per (batch, head) when the device has room: the forward's output branch, the "
        "backward's recomputation of checkpoint groups (default true).");
  m.def("set_fill_group_tensors", [](bool on) { g_fill_group_tensors = on; },
        "After ttt_backward, leave the values of checkpoint group 0 in the sixteen *_group tensors, row-major, as the "
        "upstream kernel does (its harness compares them); costs one more, slower kernel (default false: the tensors "
        "are workspace with unspecified contents).");
  m.def("set_accumulate", [](bool on) { g_accumulate = on; },
        "True (default, the upstream behaviour): ttt_backward adds to grad_L_last_eta / grad_L_XQ / grad_L_XK / "
        "grad_L_XV, which the caller zero-fills.  False: it overwrites them - no zero-fill needed, and the kernels "
        "skip the read of the old values.");
  m.def("get_accumulate", []() { return g_accumulate; });
  m.def("check_last_status", []() {
          if (g_sticky == nullptr) return;
          const c10::DeviceGuard guard(g_sticky->device());
          hipStream_t stream = c10::hip::getCurrentHIPStream(g_sticky->device().index()).stream();
          hipError_t e = hipStreamSynchronize(stream);
          TORCH_CHECK(e == hipSuccess, "check_last_status: ", hipGetErrorString(e));
          int word = 0;
          e = hipMemcpy(&word, g_sticky->data_ptr<int>(), sizeof(int), hipMemcpyDeviceToHost);
          TORCH_CHECK(e == hipSuccess, "check_last_status: ", hipGetErrorString(e));
          if (word != 0) {
            (void)hipMemset(g_sticky->data_ptr<int>(), 0, sizeof(int));
            TORCH_CHECK(false, "ttt_forward / ttt_backward: ", gave_up_text());
          }
        },
        "With set_synchronize(False) the operators cannot report a multi-workgroup launch whose workgroups gave up "
        "waiting for each other (the reference reports execution errors after its own synchronisation, "
        "kernels/ttt/ttt.cu:708-718).  Call this after such launches: it waits for the current stream and raises if "
        "any launch since the last call gave up (the outputs of that launch are invalid).");
  m.def("set_wait_limit", [](unsigned long long ticks) { g_wait_ticks = ticks; ttt_mlp_set_wait_limit(ticks); },
        "Ticks of the GPU's 100 MHz clock a workgroup waits for its partner before giving up (default 2e9 = 20 s).");
  // The upstream operator allocates nothing: every tensor, scratch included, is the caller's
  // (kernels/ttt_backward/ttt.cu:1451-1917).  The launches with several workgroups per (batch, head) need a workspace
  // beyond the upstream argument list; a caller that wants the same guarantee hands it over once.
  m.def("workspace_bytes", [](int B, int NH, int checkpoint_group_size) {
          const size_t f = ttt_mlp_fwd_workspace_bytes(B, NH), b = ttt_mlp_bwd_workspace_bytes(B, NH, checkpoint_group_size);
          return (unsigned long long)(f > b ? f : b);
        },
        "Bytes of workspace that let ttt_forward and ttt_backward of this shape use several workgroups per (batch, head) "
        "(0: the shape runs with one workgroup per pair and needs none).");
  m.def("set_workspace", [](c10::optional<torch::Tensor> ws) {
          if (!ws.has_value()) { delete g_workspace; g_workspace = nullptr; return; }
          TORCH_CHECK(ws->device().is_cuda() && ws->is_contiguous() && ws->scalar_type() == torch::kUInt8 && ws->dim() == 1,
                      "set_workspace: a contiguous 1-D uint8 GPU tensor is expected");
          TORCH_CHECK(reinterpret_cast<uintptr_t>(ws->data_ptr()) % 256 == 0, "set_workspace: the tensor must be 256-byte aligned");
          (void)sticky_word(ws->device());   // the one device word check_last_status reads exists before the first launch
          delete g_workspace;
          g_workspace = new torch::Tensor(*ws);
        },
        "Hand the operators a workspace (1-D uint8 GPU tensor of at least workspace_bytes(...) bytes) that they use for "
        "every later call instead of allocating one: with it ttt_forward / ttt_backward allocate nothing and do not query "
        "the device's free memory; a call whose shape needs more than the tensor holds, or that runs on another device, "
        "uses one workgroup per (batch, head).  The contents are scratch; calls that overlap in time must not share it.  "
        "None returns to the default (workspace from torch's caching allocator per call).");
  m.def("set_compute_units", [](int n) { ttt_mlp_set_compute_units(n); },
        "CUs the multi-workgroup launches may count on (their workgroups wait for each other and must all be resident): "
        "say so when the process runs under a CU mask or beside a kernel that holds CUs; 0 (default) = all of the device.");
  m.def("last_forward_mode", []() { return g_last_forward_mode; },
        "0: the last ttt_forward used one workgroup per (batch, head); 1: two; -1: none yet.");
  m.def("last_backward_mode", []() { return g_last_backward_mode; },
        "0: the last ttt_backward used one workgroup per (batch, head); 1: two; -1: none yet.");
}
