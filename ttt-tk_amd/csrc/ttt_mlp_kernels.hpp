// Internal interface between the C ABI and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ttt {

struct FwdParams {
  const __bf16 *XQ, *XK, *XV, *last_eta;
  const float *ttt_norm_weight, *ttt_norm_bias;
  const float *W1, *b1, *W2, *b2;
  float *W1_ck, *b1_ck, *W2_ck, *b2_ck;
  __bf16* Out;
  int B, NH, NC, K, cgs;
};

}  // namespace ttt

hipError_t ttt_mlp_fwd_enqueue(const ttt::FwdParams& p, hipStream_t stream);
extern "C" int ttt_mlp_fwd_lds_bytes();
extern "C" int ttt_mlp_bwd_lds_bytes();
