// extern "C" entry points declared in include/ttt_mlp.h: argument validation on the host, then
// one asynchronous kernel launch.  Nothing here allocates or synchronises.
#include "../../include/ttt_mlp.h"
#include "ttt_mlp_kernels.hpp"

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename... P>
inline bool any_null(P... ptrs) { return ((ptrs == nullptr) || ...); }

template <typename... P>
inline bool all_aligned(P... ptrs) { return (aligned16(ptrs) && ...); }

int check_sizes(int B, int NH, int NC, int K, int cgs) {
  if (B <= 0 || NH <= 0 || NC <= 0 || K <= 0 || cgs <= 0) return TTT_MLP_ERR_BAD_ARG;
  if ((long long)K != ((long long)NC + cgs - 1) / cgs) return TTT_MLP_ERR_BAD_CKPT;
  if ((long long)B * NH > 0x7fffffffLL) return TTT_MLP_ERR_TOO_LARGE;
  // the kernels address one (batch, head) with 32-bit byte offsets: 8 KiB per mini-batch, 32 KiB per group slot
  if (NC > (1 << 18) || cgs > (1 << 16)) return TTT_MLP_ERR_TOO_LARGE;
  return TTT_MLP_OK;
}

inline const __bf16* bf(const uint16_t* p) { return reinterpret_cast<const __bf16*>(p); }
inline __bf16* bf(uint16_t* p) { return reinterpret_cast<__bf16*>(p); }

}  // namespace

extern "C" int ttt_mlp_abi_version(void) { return TTT_MLP_ABI_VERSION; }

extern "C" const char* ttt_mlp_error_string(int code) {
  switch (code) {
    case TTT_MLP_OK: return "success";
    case TTT_MLP_ERR_BAD_ARG: return "ttt_mlp: null pointer or non-positive size";
    case TTT_MLP_ERR_BAD_CKPT: return "ttt_mlp: number of checkpoints K must equal ceil(NC / checkpoint_group_size)";
    case TTT_MLP_ERR_ALIGN: return "ttt_mlp: every tensor pointer must be 16-byte aligned";
    case TTT_MLP_ERR_TOO_LARGE: return "ttt_mlp: B*NH exceeds the launch grid limit, or NC > 262144, or checkpoint_group_size > 65536";
    default: return hipGetErrorString(static_cast<hipError_t>(code));
  }
}

extern "C" int ttt_mlp_fwd_launch(const ttt_mlp_fwd_args* a, void* stream) {
  if (a == nullptr) return TTT_MLP_ERR_BAD_ARG;
  if (any_null(a->XQ, a->XK, a->XV, a->last_eta, a->ttt_norm_weight, a->ttt_norm_bias, a->W1, a->b1, a->W2, a->b2,
               a->W1_checkpoints, a->b1_checkpoints, a->W2_checkpoints, a->b2_checkpoints, a->Out))
    return TTT_MLP_ERR_BAD_ARG;
  if (int rc = check_sizes(a->B, a->NH, a->NC, a->K, a->checkpoint_group_size)) return rc;
  if (!all_aligned(a->XQ, a->XK, a->XV, a->last_eta, a->ttt_norm_weight, a->ttt_norm_bias, a->W1, a->b1, a->W2,
                   a->b2, a->W1_checkpoints, a->b1_checkpoints, a->W2_checkpoints, a->b2_checkpoints, a->Out))
    return TTT_MLP_ERR_ALIGN;
  ttt::FwdParams p;
  p.XQ = bf(a->XQ); p.XK = bf(a->XK); p.XV = bf(a->XV); p.last_eta = bf(a->last_eta);
  p.ttt_norm_weight = a->ttt_norm_weight; p.ttt_norm_bias = a->ttt_norm_bias;
  p.W1 = a->W1; p.b1 = a->b1; p.W2 = a->W2; p.b2 = a->b2;
  p.W1_ck = a->W1_checkpoints; p.b1_ck = a->b1_checkpoints; p.W2_ck = a->W2_checkpoints; p.b2_ck = a->b2_checkpoints;
  p.Out = bf(a->Out);
  p.B = a->B; p.NH = a->NH; p.NC = a->NC; p.K = a->K; p.cgs = a->checkpoint_group_size;
  return static_cast<int>(ttt_mlp_fwd_enqueue(p, static_cast<hipStream_t>(stream)));
}

extern "C" int ttt_mlp_bwd_launch(const ttt_mlp_bwd_args* a, void* stream) {
  if (a == nullptr) return TTT_MLP_ERR_BAD_ARG;
  if (any_null(a->XQ, a->XK, a->XV, a->last_eta, a->ttt_norm_weight, a->ttt_norm_bias, a->W1_checkpoints,
               a->b1_checkpoints, a->W2_checkpoints, a->b2_checkpoints, a->W1_init_group, a->b1_init_group,
               a->W2_init_group, a->b2_init_group, a->x_hat_ln_group, a->std_ln_group, a->X2_group, a->Z1_group,
               a->Z1_bar_group, a->X2_bar_group, a->grad_l_wrt_Z2_group, a->grad_l_wrt_Z1_group, a->x_hat_fused_group,
               a->grad_x_hat_fused_group, a->grad_output_fused_group, a->std_fused_group, a->grad_L_W1_last,
               a->grad_L_b1_last, a->grad_L_W2_last, a->grad_L_b2_last, a->grad_L_XQW_mini_batch,
               a->grad_L_ttt_norm_weight, a->grad_L_ttt_norm_bias, a->grad_L_W1_init, a->grad_L_b1_init,
               a->grad_L_W2_init, a->grad_L_b2_init, a->grad_L_last_eta, a->grad_L_XQ, a->grad_L_XK, a->grad_L_XV))
    return TTT_MLP_ERR_BAD_ARG;  // `Out` is unused and may be null
  if (int rc = check_sizes(a->B, a->NH, a->NC, a->K, a->checkpoint_group_size)) return rc;
  if (!all_aligned(a->XQ, a->XK, a->XV, a->last_eta, a->ttt_norm_weight, a->ttt_norm_bias, a->W1_checkpoints,
                   a->b1_checkpoints, a->W2_checkpoints, a->b2_checkpoints, a->W1_init_group, a->b1_init_group,
                   a->W2_init_group, a->b2_init_group, a->x_hat_ln_group, a->std_ln_group, a->Z1_group,
                   a->Z1_bar_group, a->grad_l_wrt_Z2_group, a->x_hat_fused_group, a->grad_output_fused_group,
                   a->std_fused_group, a->grad_L_W1_last, a->grad_L_b1_last, a->grad_L_W2_last, a->grad_L_b2_last,
                   a->grad_L_XQW_mini_batch, a->grad_L_ttt_norm_weight, a->grad_L_ttt_norm_bias, a->grad_L_W1_init,
                   a->grad_L_b1_init, a->grad_L_W2_init, a->grad_L_b2_init, a->grad_L_last_eta, a->grad_L_XQ,
                   a->grad_L_XK, a->grad_L_XV))
    return TTT_MLP_ERR_ALIGN;
  ttt::BwdParams p;
  p.XQ = bf(a->XQ); p.XK = bf(a->XK); p.XV = bf(a->XV); p.last_eta = bf(a->last_eta);
  p.ttt_norm_weight = a->ttt_norm_weight; p.ttt_norm_bias = a->ttt_norm_bias;
  p.W1_ck = a->W1_checkpoints; p.b1_ck = a->b1_checkpoints; p.W2_ck = a->W2_checkpoints; p.b2_ck = a->b2_checkpoints;
  p.W1_init_group = a->W1_init_group; p.b1_init_group = a->b1_init_group;
  p.W2_init_group = a->W2_init_group; p.b2_init_group = a->b2_init_group;
  p.x_hat_ln_group = bf(a->x_hat_ln_group); p.std_ln_group = a->std_ln_group;
  p.X2_group = bf(a->X2_group); p.Z1_group = bf(a->Z1_group);
  p.Z1_bar_group = bf(a->Z1_bar_group); p.X2_bar_group = bf(a->X2_bar_group);
  p.grad_l_wrt_Z2_group = bf(a->grad_l_wrt_Z2_group); p.grad_l_wrt_Z1_group = bf(a->grad_l_wrt_Z1_group);
  p.x_hat_fused_group = bf(a->x_hat_fused_group); p.grad_x_hat_fused_group = bf(a->grad_x_hat_fused_group);
  p.grad_output_fused_group = bf(a->grad_output_fused_group); p.std_fused_group = a->std_fused_group;
  p.grad_L_W1_last = a->grad_L_W1_last; p.grad_L_b1_last = a->grad_L_b1_last;
  p.grad_L_W2_last = a->grad_L_W2_last; p.grad_L_b2_last = a->grad_L_b2_last;
  p.grad_L_XQW = bf(a->grad_L_XQW_mini_batch);
  p.grad_L_ttt_norm_weight = a->grad_L_ttt_norm_weight; p.grad_L_ttt_norm_bias = a->grad_L_ttt_norm_bias;
  p.grad_L_W1_init = a->grad_L_W1_init; p.grad_L_b1_init = a->grad_L_b1_init;
  p.grad_L_W2_init = a->grad_L_W2_init; p.grad_L_b2_init = a->grad_L_b2_init;
  p.grad_L_last_eta = bf(a->grad_L_last_eta);
  p.grad_L_XQ = bf(a->grad_L_XQ); p.grad_L_XK = bf(a->grad_L_XK); p.grad_L_XV = bf(a->grad_L_XV);
  p.B = a->B; p.NH = a->NH; p.NC = a->NC; p.K = a->K; p.cgs = a->checkpoint_group_size;
  return static_cast<int>(ttt_mlp_bwd_enqueue(p, static_cast<hipStream_t>(stream)));
}

extern "C" int ttt_mlp_kernel_info(int which, int* lds_bytes, int* threads_per_workgroup) {
  if (lds_bytes == nullptr || threads_per_workgroup == nullptr) return TTT_MLP_ERR_BAD_ARG;
  if (which == 0) { *lds_bytes = ttt_mlp_fwd_lds_bytes(); *threads_per_workgroup = ttt_mlp_fwd_threads(); return TTT_MLP_OK; }
  if (which == 1) { *lds_bytes = ttt_mlp_bwd_lds_bytes(); *threads_per_workgroup = ttt_mlp_bwd_threads(); return TTT_MLP_OK; }
  return TTT_MLP_ERR_BAD_ARG;
}
