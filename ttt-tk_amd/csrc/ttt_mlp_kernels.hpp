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
  // One workgroup per pair, sequence cut into segments (seg_len > 0, a multiple of cgs): workgroup i of the launch
  // runs job job0 + i, job q = segment q / (B*NH) of pair q % (B*NH); a segment starts from the checkpoint that the
  // segment before it left (an earlier launch on the same stream) and leaves the one the next starts from.
  int seg_len, job0;
#ifdef TTT_STAGE_CLOCKS
  unsigned* stage_clocks;   // [B*NH][2 roles][8 waves][STAGE_SLOTS] or nullptr (see below)
#endif
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
  // n_prefetch = 1 (with n_finish = 1 only): one more workgroup reads nothing for itself; it touches every cache
  // line that the walk is about to ask for, one mini-batch ahead of it, so that the walk's own requests are
  // answered by the L2 the two share instead of by HBM.
  int n_prefetch;
  int* sync;
  int* status;    // the status word behind the synchronisation words
  unsigned long long wait_limit;   // ticks of the 100 MHz clock a workgroup waits for another before it gives up
  int overwrite;  // non-zero: grad_L_XQ / XK / XV / last_eta are stored, not added to (every element is written exactly once)
  int bh0, nbh;   // this launch covers (batch, head) pairs bh0 .. bh0 + nbh - 1 (workspace pointers moved back by bh0 entries)
  // One workgroup per pair, sequence cut into segments of seg_groups checkpoint groups (> 0): workgroup i of the launch
  // runs job job0 + i, job q = segment q / (B*NH) of pair q % (B*NH), segment 0 being the sequence's last groups.  A
  // segment takes the running gradients from grad_L_*_init, where the segment before it (an earlier launch on the same
  // stream) left them, and the norm-gradient sums from the pair's slots of x_hat_ln_group.
  int seg_groups, job0;
#ifdef TTT_STAGE_CLOCKS
  unsigned* stage_clocks;   // [B*NH][4 roles][8 waves][STAGE_SLOTS] or nullptr (see below)
#endif
};

// Layout of `sync` (ints): 32 per (batch, head) - words 0 and 8 count the groups replayed by the first /
// second replaying workgroup (norm_partial is written before the last count), word 16 the groups the
// reverse walk has finished, word 12 the mini-batches of the last group it walks that it has handed to the grad_L_XK
// workgroup (that group is handed over in chunks), word 20 the mini-batches it has started (a pacing hint for the prefetching workgroup,
// no data is ordered by it), word 24 the groups the grad_L_XK workgroup has finished - then one status
// word (non-zero: a wait gave up).
constexpr int BWD_SYNC_STRIDE = 32;
inline size_t bwd_sync_ints(long long BH) { return (size_t)BH * BWD_SYNC_STRIDE + 32; }

// ---- optional stage clocks.  A library built with -DTTT_STAGE_CLOCKS (stage_clocks.py builds one beside the product
// library) reads the shader clock at the boundaries of the stages named here and adds up, per wave, the clocks
// spent in each; every wave stores its sums when the kernel ends.  The product library
// is built without the macro and contains none of this.  Reading the clock is a scalar-memory operation: every
// boundary also waits for the wave's outstanding LDS reads, which makes an instrumented kernel some 10 % slower.
// Slot of a workgroup in the buffer: forward 0 = the recurrence (or the one workgroup), 1 = the output branch;
// backward 0 / 1 = the replaying workgroups, 2 = the reverse walk (or the one workgroup), 3 = unused.
constexpr int STAGE_SLOTS = 24;
enum FwdStage {
  FS_TOP,            // barrier that opens the mini-batch, checkpoint store, wait for the other workgroup
  FS_F1_GELU,        // Z1 = XK W1 + b1, GELU and its derivative
  FS_X2_SPLIT,       // X2 in two terms, high-order term to LDS
  FS_F2_PAIRSUM,     // Z2 = X2 W2 and its sum over the wave pairs (two barriers)
  FS_LN,             // LayerNorm + loss gradient of 8 tokens per wave, G2 to LDS
  FS_LN_BARRIER,     // barrier after it
  FS_F3,             // G1 = (G2 W2^T) * GELU'(Z1), including the transposition of W2's terms through LDS
  FS_F4,             // W1 step
  FS_F5,             // W2 step and b2
  FS_HANDOVER,       // recurrence workgroup: state images for the output branch
  FS_PUBLISH,        // recurrence workgroup: counter for the output branch
  FS_OUT_FORWARD,    // output branch: Z1_bar, GELU, Z2_bar and its pair sum
  FS_OUT_LN,         // output branch: LayerNorm, residual, store; next inputs
  FS_COUNT
};
enum BwdStage {
  BS_GROUP,          // per checkpoint group: waits for the other workgroups, parking / loading of state and gradients
  BS_R_TOP,          // replay: barrier that opens the mini-batch
  BS_R_F1_GELU,      // replay: Z1, GELU family, images of Z1
  BS_R_F2_PAIRSUM,   // replay: Z2 and its pair sum
  BS_R_LN,           // replay: fused LayerNorm + loss gradient, saved tiles, barrier
  BS_R_F3,           // replay: G1
  BS_R_WSTEP,        // replay: W1 and W2 steps
  BS_R_IMAGES,       // replay: operand images of the state after the step
  BS_R_OUT_FORWARD,  // replay: output branch forward with its pair sum
  BS_R_OUT_LN,       // replay: output LayerNorm forward and backward, next inputs, barrier
  BS_R_OUT_BACKWARD, // replay: gZ1_bar, grad_L_XQ with its pair sum, images for the walk
  BS_W_TOP,          // walk: tiles of the mini-batch into LDS (two barriers)
  BS_W_BAR_TERMS,    // walk: what the output branch adds to the running gradients
  BS_W_STEP_BACK,    // walk: the weight step backwards up to its pair sum
  BS_W_PAIRSUM,      // walk: pair sum of it
  BS_W_LN,           // walk: second-order pass through the fused LayerNorm loss
  BS_W_LN_BARRIER,   // walk: barrier after it
  BS_W_MLP_BACK,     // walk: inner MLP backwards (to the second wave-level fence)
  BS_W_UPDATES,      // walk: updates of the running gradients
  BS_W_DXK,          // walk: grad_L_XK with its pair sum (not with a grad_L_XK workgroup)
  BS_PUBLISH,        // counters for the other workgroups
  BS_X_GROUP,        // grad_L_XK workgroup, per checkpoint group: waits for the walk to have finished the group
  BS_X_PRODUCTS,     // grad_L_XK workgroup: operands of the mini-batch from HBM, G1 and the products, to the pair sum
  BS_X_SUMS,         // grad_L_XK workgroup: pair sum, grad_L_XK / grad_L_XV, token sums of the norm gradients, barrier
  BS_COUNT
};
static_assert(FS_COUNT <= STAGE_SLOTS && BS_COUNT <= STAGE_SLOTS, "stage slots");

}  // namespace ttt

#ifdef TTT_STAGE_CLOCKS
// Device buffers the next launches write their stage clocks to (nullptr: none): forward [B*NH][2][8][STAGE_SLOTS],
// backward [B*NH][4][8][STAGE_SLOTS] unsigned ints, zero-filled by the caller.
extern "C" void ttt_mlp_set_stage_clocks(unsigned* forward, unsigned* backward);
#endif

// p.sync == nullptr: one workgroup per (batch, head); otherwise two (state recurrence / output branch).
hipError_t ttt_mlp_fwd_enqueue(const ttt::FwdParams& p, hipStream_t stream);
hipError_t ttt_mlp_fwd_clear_words(int* words, int n, hipStream_t stream);   // zeroes n ints with a small kernel
// p.sync == nullptr: one workgroup per (batch, head); otherwise two (replay / reverse walk).
hipError_t ttt_mlp_bwd_enqueue(const ttt::BwdParams& p, hipStream_t stream);
// Replays checkpoint group 0 and writes the sixteen per-group tensors row-major (side path, one workgroup per pair).
hipError_t ttt_mlp_export_group0_enqueue(const ttt::BwdParams& p, hipStream_t stream);
extern "C" int ttt_mlp_fwd_lds_bytes();
extern "C" int ttt_mlp_bwd_lds_bytes();
extern "C" int ttt_mlp_fwd_threads();
extern "C" int ttt_mlp_bwd_threads();
