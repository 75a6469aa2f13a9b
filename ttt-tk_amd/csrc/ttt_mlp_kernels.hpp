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
  // Two-workgroup mode only (sync != nullptr): per (batch, head) a ring of 2 * FWD_RING_MAX mini-batch slots
  // (2 << ring_log2 of them in use: 1 << ring_log2 mini-batches per hand-over, chosen by the launcher from NC)
  // with the bf16 operand images (64 KiB) and the bias vectors (256 + 64 floats) of the state after a
  // mini-batch, and the words the two workgroups signal with (layout as in the backward).
  // The workspace pointers are indexed by the global (batch, head) number like everything else: the
  // launcher passes them moved back by bh0 entries.
  __bf16* state_img;
  float* bias_img;
  int ring_log2;
  int* sync;
  int* status;    // the status word behind the synchronisation words
  unsigned long long wait_limit;   // ticks of the 100 MHz clock a workgroup waits for another before it gives up
  int bh0, nbh;   // this launch covers (batch, head) pairs bh0 .. bh0 + nbh - 1
};
constexpr int FWD_RING_MAX = 32;               // most mini-batches per hand-over (8 or 32 are compiled)
constexpr int FWD_IMG_BYTES = 64 * 256 * 2 * 2;  // W1 and W2 as bf16 operands
constexpr int FWD_BIAS_FLOATS = 256 + 64;

struct BwdParams {
  const __bf16 *XQ, *XK, *XV, *last_eta;
  const float *ttt_norm_weight, *ttt_norm_bias;
  const float *W1_ck, *b1_ck, *W2_ck, *b2_ck;
  float *W1_init_group, *b1_init_group, *W2_init_group, *b2_init_group;
  __bf16* x_hat_ln_group;
  float* std_ln_group;
  __bf16 *X2_group, *Z1_group, *Z1_bar_group, *X2_bar_group;
  __bf16 *grad_l_wrt_Z2_group, *grad_l_wrt_Z1_group;
  __bf16 *x_hat_fused_group, *grad_x_hat_fused_group, *grad_output_fused_group;
  float* std_fused_group;
  const float *grad_L_W1_last, *grad_L_b1_last, *grad_L_W2_last, *grad_L_b2_last;
  const __bf16* grad_L_XQW;
  float *grad_L_ttt_norm_weight, *grad_L_ttt_norm_bias;
  float *grad_L_W1_init, *grad_L_b1_init, *grad_L_W2_init, *grad_L_b2_init;
  __bf16 *grad_L_last_eta, *grad_L_XQ, *grad_L_XK, *grad_L_XV;
  int B, NH, NC, K, cgs;
  // Several workgroups per (batch, head) only (sync != nullptr): n_replay = 1 or 2 workgroups replay the
  // checkpoint groups (taking turns), one walks them backwards.  Group number g (0 = the last group of the
  // sequence) is replayed into set g % (2 * n_replay) of the per-group tensors that carry it to the walk:
  // set 0 = the caller's tensors, sets 1.. = alt_*[set - 1] from the workspace.
  __bf16 *alt_X2_group[3], *alt_Z1_group[3], *alt_Z1_bar_group[3], *alt_X2_bar_group[3];
  __bf16 *alt_grad_l_wrt_Z2_group[3], *alt_grad_l_wrt_Z1_group[3];
  __bf16 *alt_x_hat_fused_group[3], *alt_grad_x_hat_fused_group[3], *alt_grad_output_fused_group[3];
  float* alt_std_fused_group[3];
  float* alt_W1_init_group[3];
  float* norm_partial;   // [B*NH][2][8 waves][2][64]: the replay's share of the norm-weight / norm-bias gradients, by group parity
  float* norm_park;      // [B*NH][8 waves][2][64]: n_replay = 1: the share of the parity that is not being added to
  __bf16* walk_park;     // [B*NH][64][256]: one register image the walking workgroup parks across its LayerNorm stage
  int n_replay;
  // n_finish = 1: a further workgroup forms grad_L_XK, grad_L_XV and the walk's share of the norm gradients from
  // what the walk hands it per mini-batch - one register image (dZ1: [B*NH][2 sets][cgs][64][256] bf16) and two
  // fp32 tiles (g_y and the norm-weight gradient terms: [B*NH][2][cgs][2][64][64]); the two sets alternate by
  // group.  It keeps its own copy of the running gradient wrt W1 and forms G1 = -eta * dl/dZ1 itself.
  __bf16* fin_dz;
  float* fin_gy;
  int n_finish;
  int* sync;
  int* status;    // the status word behind the synchronisation words
  unsigned long long wait_limit;   // ticks of the 100 MHz clock a workgroup waits for another before it gives up
  int overwrite;  // non-zero: grad_L_XQ / XK / XV / last_eta are stored, not added to (every element is written exactly once)
  int bh0, nbh;   // this launch covers (batch, head) pairs bh0 .. bh0 + nbh - 1 (workspace pointers moved back by bh0 entries)
};

// Layout of `sync` (ints): 32 per (batch, head) - words 0 and 8 count the groups replayed by the first /
// second replaying workgroup (norm_partial is written before the last count), word 16 the groups the
// reverse walk has finished, word 24 the groups the grad_L_XK workgroup has finished - then one status
// word (non-zero: a wait gave up).
constexpr int BWD_SYNC_STRIDE = 32;
inline size_t bwd_sync_ints(long long BH) { return (size_t)BH * BWD_SYNC_STRIDE + 32; }

}  // namespace ttt

// p.sync == nullptr: one workgroup per (batch, head); otherwise two (state recurrence / output branch).
hipError_t ttt_mlp_fwd_enqueue(const ttt::FwdParams& p, hipStream_t stream);
// p.sync == nullptr: one workgroup per (batch, head); otherwise two (replay / reverse walk).
hipError_t ttt_mlp_bwd_enqueue(const ttt::BwdParams& p, hipStream_t stream);
// Replays checkpoint group 0 and writes the sixteen per-group tensors row-major (side path, one workgroup per pair).
hipError_t ttt_mlp_export_group0_enqueue(const ttt::BwdParams& p, hipStream_t stream);
extern "C" int ttt_mlp_fwd_lds_bytes();
extern "C" int ttt_mlp_bwd_lds_bytes();
extern "C" int ttt_mlp_fwd_threads();
extern "C" int ttt_mlp_bwd_threads();
