/*
 * C ABI of the MI355X (gfx950) TTT-MLP forward / remat-backward kernels.
 *
 * This is the drop-in boundary below the Python operator module
 * `test_time_training`: plain pointers and sizes, no torch types.  Every
 * pointer is a DEVICE pointer to a contiguous row-major tensor owned by the
 * caller; the library allocates nothing, keeps no state between calls and
 * never synchronises the stream (the launch is asynchronous on `stream`).
 *
 * Fixed sizes of the shipped kernels: mini-batch CS = 64 tokens, head dim
 * F = 64, hidden dim H = 256.  B = batch, NH = heads, NC = mini-batches,
 * K = ceil(NC / checkpoint_group_size) checkpoints.
 *
 * Reference interfaces replaced (upstream repository paths):
 *   ttt_mlp_fwd_launch  <- host launcher `ttt_forward`   kernels/ttt/ttt.cu:594-721
 *                          + kernel fwd_ttt_mlp_ker<64>   kernels/ttt/ttt.cu:85-586
 *   ttt_mlp_bwd_launch  <- host launcher `ttt_backward`  kernels/ttt_backward/ttt.cu:1451-1917
 *                          + kernel bwd_ttt_mlp_ker<64>   kernels/ttt_backward/ttt.cu:179-1443
 * The argument structs list the tensors in the exact order of the operator's
 * positional arguments (test_time_training.cpp:25-42 and :47-91).
 */
#ifndef TTT_MLP_H_
#define TTT_MLP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTT_MLP_ABI_VERSION 2

#define TTT_MLP_CS 64   /* tokens per mini-batch        */
#define TTT_MLP_F 64    /* head dimension               */
#define TTT_MLP_HID 256 /* inner MLP hidden dimension   */

/* Return codes (0 = success; positive values below 1000 are hipError_t codes). */
#define TTT_MLP_OK 0
#define TTT_MLP_ERR_BAD_ARG 1001   /* null pointer or non-positive size           */
#define TTT_MLP_ERR_BAD_CKPT 1002  /* K != ceil(NC / checkpoint_group_size)       */
#define TTT_MLP_ERR_ALIGN 1003     /* a pointer is not 16-byte aligned            */
#define TTT_MLP_ERR_TOO_LARGE 1004 /* B*NH > 2^31-1, NC > 2^18, cgs > 2^16 or K > 2^15 */
#define TTT_MLP_ERR_NO_ROOM 1005   /* 2*B*NH workgroups exceed the CUs of the device */
#define TTT_MLP_ERR_WORKSPACE 1006 /* workspace smaller than required              */
#define TTT_MLP_ERR_SCRATCH 1007   /* more (batch, head) pairs than the fixed scratch of ttt_mlp_fwd_launch_static serves */

/* Forward scan.  Replaces the 16 positional arguments of `ttt_forward`
 * (test_time_training.cpp:25-42).  bf16 tensors are passed as uint16_t bit patterns. */
typedef struct ttt_mlp_fwd_args {
  const uint16_t* XQ;              /* [B,NH,NC,CS,F]  bf16 in  */
  const uint16_t* XK;              /* [B,NH,NC,CS,F]  bf16 in  */
  const uint16_t* XV;              /* [B,NH,NC,CS,F]  bf16 in  */
  const uint16_t* last_eta;        /* [B,NH,NC,CS,1]  bf16 in  */
  const float* ttt_norm_weight;    /* [1,NH,1,F]      fp32 in  */
  const float* ttt_norm_bias;      /* [1,NH,1,F]      fp32 in  */
  const float* W1;                 /* [B,NH,F,HID]    fp32 in (initial state, not modified) */
  const float* b1;                 /* [B,NH,1,HID]    fp32 in  */
  const float* W2;                 /* [B,NH,HID,F]    fp32 in  */
  const float* b2;                 /* [B,NH,1,F]      fp32 in  */
  float* W1_checkpoints;           /* [B,NH,K,F,HID]  fp32 out */
  float* b1_checkpoints;           /* [B,NH,K,1,HID]  fp32 out */
  float* W2_checkpoints;           /* [B,NH,K,HID,F]  fp32 out */
  float* b2_checkpoints;           /* [B,NH,K,1,F]    fp32 out */
  uint16_t* Out;                   /* [B,NH,NC,CS,F]  bf16 out */
  int32_t checkpoint_group_size;
  int32_t B, NH, NC, K;
} ttt_mlp_fwd_args;

/* Remat backward.  Replaces the 43 positional arguments of `ttt_backward`
 * (test_time_training.cpp:47-91).  The sixteen *_group tensors are caller-owned
 * scratch of checkpoint_group_size mini-batches; the library uses them as
 * workspace and leaves their contents unspecified.  grad_L_last_eta / grad_L_XQ /
 * grad_L_XK / grad_L_XV are accumulated into (the caller zero-fills them) unless
 * `overwrite` is set, all other outputs are overwritten.  `Out` is not touched. */
typedef struct ttt_mlp_bwd_args {
  const uint16_t* XQ;
  const uint16_t* XK;
  const uint16_t* XV;
  const uint16_t* last_eta;
  const float* ttt_norm_weight;
  const float* ttt_norm_bias;
  const float* W1_checkpoints;     /* [B,NH,K,F,HID]  fp32 in */
  const float* b1_checkpoints;
  const float* W2_checkpoints;
  const float* b2_checkpoints;
  uint16_t* Out;                   /* unused */
  float* W1_init_group;            /* [B,NH,cgs,F,HID]  fp32 scratch */
  float* b1_init_group;            /* [B,NH,cgs,1,HID]  fp32 scratch */
  float* W2_init_group;            /* [B,NH,cgs,HID,F]  fp32 scratch */
  float* b2_init_group;            /* [B,NH,cgs,1,F]    fp32 scratch */
  uint16_t* x_hat_ln_group;        /* [B,NH,cgs,CS,F]   bf16 scratch */
  float* std_ln_group;             /* [B,NH,cgs,CS,1]   fp32 scratch */
  uint16_t* X2_group;              /* [B,NH,cgs,CS,HID] bf16 scratch */
  uint16_t* Z1_group;
  uint16_t* Z1_bar_group;
  uint16_t* X2_bar_group;
  uint16_t* grad_l_wrt_Z2_group;   /* [B,NH,cgs,CS,F]   bf16 scratch */
  uint16_t* grad_l_wrt_Z1_group;   /* [B,NH,cgs,CS,HID] bf16 scratch */
  uint16_t* x_hat_fused_group;     /* [B,NH,cgs,CS,F]   bf16 scratch */
  uint16_t* grad_x_hat_fused_group;
  uint16_t* grad_output_fused_group;
  float* std_fused_group;          /* [B,NH,cgs,CS,1]   fp32 scratch */
  const float* grad_L_W1_last;     /* [B,NH,F,HID] fp32 in: grads wrt the state after the last mini-batch */
  const float* grad_L_b1_last;
  const float* grad_L_W2_last;
  const float* grad_L_b2_last;
  const uint16_t* grad_L_XQW_mini_batch; /* [B,NH,NC,CS,F] bf16 in */
  float* grad_L_ttt_norm_weight;   /* [B,NH,1,F] fp32 out (per batch element) */
  float* grad_L_ttt_norm_bias;
  float* grad_L_W1_init;           /* as W1 ... fp32 out */
  float* grad_L_b1_init;
  float* grad_L_W2_init;
  float* grad_L_b2_init;
  uint16_t* grad_L_last_eta;       /* [B,NH,NC,CS,1] bf16, accumulated into */
  uint16_t* grad_L_XQ;             /* [B,NH,NC,CS,F] bf16, accumulated into */
  uint16_t* grad_L_XK;
  uint16_t* grad_L_XV;
  int32_t checkpoint_group_size;
  int32_t B, NH, NC, K;
  /* 0: grad_L_last_eta / grad_L_XQ / grad_L_XK / grad_L_XV are added to, as the reference's kernel does with
   * its four thread blocks per head (the caller zero-fills them, kernels/ttt_backward/matching.py:406-415).
   * 1: they are overwritten - these kernels write every element exactly once, so the zero-fill and the
   * read of the old value can both be left out.  Same values either way when the tensors start at zero. */
  int32_t overwrite;
} ttt_mlp_bwd_args;

/* Version of this header the library was built against. */
int ttt_mlp_abi_version(void);

/* Validates sizes / alignment and enqueues the forward kernel on `stream`
 * (a hipStream_t, NULL = the default stream).  Returns TTT_MLP_OK, one of the
 * TTT_MLP_ERR_* codes, or the hipError_t of a failed launch. */
int ttt_mlp_fwd_launch(const ttt_mlp_fwd_args* args, void* stream);

/* Same for the remat backward. */
int ttt_mlp_bwd_launch(const ttt_mlp_bwd_args* args, void* stream);

/* The same backward (bit-identical results) with two to five workgroups per
 * (batch, head) where the device has CUs to spare: one or two recompute checkpoint
 * group after checkpoint group, one walks each recomputed group backwards, a
 * fourth forms grad_L_XK, grad_L_XV and part of the norm gradients from what the
 * walk hands it, so that only the chain through the running gradients stays on
 * the critical path, and a fifth (with a multiple of 8 pairs, if 5*n fits) only
 * reads ahead of the walk so that the walk's requests hit the L2.  The reference launcher
 * (kernels/ttt_backward/ttt.cu:1451-1917) has no counterpart: it spreads one
 * (batch, head) over a cluster of four thread blocks instead.
 * Workgroups that wait for each other must be resident together (one per CU),
 * so the pairs are covered by up to two launches in a row: the largest multiple
 * of the CU count with one workgroup per pair, then the remaining n pairs with
 * four each if 4*n fits the CUs, else three if 3*n fits, else two if 2*n fits.
 * ttt_mlp_bwd_workspace_bytes() returns 0 when neither does (n = 0 or 2*n > CUs of
 * the current device); the launcher then returns TTT_MLP_ERR_NO_ROOM and the caller
 * uses ttt_mlp_bwd_launch.
 * The caller owns the device workspace (256-byte aligned, contents unspecified
 * before and after; calls that overlap in time need separate workspaces).  The int
 * at index n*32 of the workspace is a status word: once the stream has drained
 * it reads non-zero only if a workgroup waited 20 s for another and gave up, in
 * which case the outputs are invalid. */
size_t ttt_mlp_bwd_workspace_bytes(int32_t B, int32_t NH, int32_t checkpoint_group_size);
/* Byte offset of that status word (an int) inside the workspace; 0 when the mode does not apply. */
size_t ttt_mlp_bwd_status_offset(int32_t B, int32_t NH);

/* The forward with two workgroups per (batch, head), under the same conditions and with the same
 * conventions (launches, workspace, status word at int index n*32, TTT_MLP_ERR_NO_ROOM, bit-identical
 * results): one workgroup carries the state through the mini-batches and leaves every new state
 * in the workspace as bf16 operands, the other computes Out from them, 8 mini-batches behind
 * (32 when NC >= 512).
 * Pairs are covered as in the backward: full rounds of the device with one workgroup per pair, then the
 * remaining n pairs with two each if 2*n fits the CUs.
 * No counterpart in the reference launcher (kernels/ttt/ttt.cu:594-721). */
size_t ttt_mlp_fwd_workspace_bytes(int32_t B, int32_t NH);
size_t ttt_mlp_fwd_status_offset(int32_t B, int32_t NH);
int ttt_mlp_fwd_launch_overlapped(const ttt_mlp_fwd_args* args, void* workspace, size_t workspace_bytes, void* stream);
int ttt_mlp_bwd_launch_overlapped(const ttt_mlp_bwd_args* args, void* workspace, size_t workspace_bytes, void* stream);

/* ttt_mlp_fwd_launch_overlapped for callers that cannot allocate device memory and have no workspace to
 * pass - code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart
 * in the reference.  Same kernels and bit-identical results; the workspace is a fixed array in the
 * library's device memory (32.6 MiB per GPU, held until the process ends), so the call allocates nothing
 * and serves at most 8 (batch, head) pairs: B*NH > 8 returns TTT_MLP_ERR_SCRATCH, a device without room
 * for two workgroups per pair TTT_MLP_ERR_NO_ROOM, before anything is enqueued.  Every call on a GPU uses
 * that GPU's one array: calls that overlap in time on one GPU (two streams, two threads) race - serialise
 * them.  The launch goes to the current device (make it the stream's); the first call on a device looks the
 * array's address up, which is not a stream operation: a caller that captures the call into a HIP graph makes
 * one ordinary call on that device first.  `sticky_word` (may be NULL): a device int owned by the caller; as ttt_mlp_status_accumulate, the
 * call enqueues `if (status != 0) *sticky_word = 1` behind the kernels. */
int ttt_mlp_fwd_launch_static(const ttt_mlp_fwd_args* args, int* sticky_word, void* stream);

/* For callers that do not wait for the stream after an overlapped launch (and may free or reuse the
 * workspace before they do): enqueues, behind the launch on the same stream, `if (*status_word != 0)
 * *sticky_word = 1`.  `status_word` = workspace + ttt_mlp_*_status_offset(); `sticky_word` = a device int
 * owned by the caller that outlives the workspace (zero it once).  After any later synchronisation a
 * non-zero sticky word says that some launch since it was last zeroed gave up a wait: the reference's
 * launchers report execution errors right after their own device synchronisation
 * (kernels/ttt/ttt.cu:708-718); this is the same report for callers that synchronise later. */
int ttt_mlp_status_accumulate(const void* status_word, int* sticky_word, void* stream);

/* Optional: fills the sixteen *_group tensors with the values of checkpoint group 0 (the group the
 * backward processes last) in the layouts of the struct above, as the reference's kernel leaves them
 * (kernels/ttt_backward/ttt.cu:518-521, 551-552, 607-610, 636-637, 669, 699, 744-745, 798-800; its
 * harness compares them, kernels/ttt_backward/matching.py:667-690).  Slot i holds, for mini-batch i:
 * the state before it (W1/b1/W2/b2_init_group), Z1, X2 = gelu(Z1), the LayerNorm-fused loss
 * gradient's x_hat / std / grad_output / grad_x_hat (*_fused_group), grad_l_wrt_Z2, grad_l_wrt_Z1,
 * and of the output branch with the state after it Z1_bar, X2_bar and the LayerNorm's x_hat / std
 * (*_ln_group).  The backward launchers use these tensors as workspace in formats of their own, so
 * this is a separate, slower kernel (fp32 on the vector units, values rounded only when stored) that
 * replays group 0 from checkpoint 0: enqueue it behind the backward on the same stream.  Reads XQ,
 * XK, XV, last_eta, the norm parameters and the checkpoints; slots of mini-batches beyond NC are
 * left as they are.  Takes the argument struct of ttt_mlp_bwd_launch and validates it the same way. */
int ttt_mlp_bwd_export_group0(const ttt_mlp_bwd_args* args, void* stream);

/* How long a workgroup of an overlapped launch waits for another before it gives up and raises the
 * status word, in ticks of the GPU's 100 MHz clock (default 2,000,000,000 = 20 s).  Process-wide; meant
 * for tests of that path (a limit of 1 makes the first wait give up) and for hosts that want a shorter one. */
void ttt_mlp_set_wait_limit(unsigned long long ticks_100mhz);

/* Workgroups of an overlapped launch wait for each other, so all of them must be resident at once; the launch
 * plans count on every compute unit the device reports.  A host that runs these launches under a CU mask, or
 * beside another kernel that holds CUs for their whole duration, says here how many CUs they can count on
 * (process-wide; 0 = all the device reports, the default): shapes that no longer fit run with one workgroup per
 * (batch, head), and ttt_mlp_*_workspace_bytes() follow.  No counterpart in the reference. */
void ttt_mlp_set_compute_units(int compute_units);

/* Human-readable text for a return code of the two launchers. */
const char* ttt_mlp_error_string(int code);

/* How an overlapped launch of `pairs` = B*NH (batch, head) pairs is laid out on a device with
 * `compute_units` CUs (no device needed): the first *one_workgroup_pairs pairs run with one workgroup each,
 * the remaining *other_pairs with *workgroups_per_other_pair each (0 if there are none).  which = 0
 * forward (1 or 2 per pair), 1 backward (1 to 5: one or two that replay the checkpoint groups, one that walks
 * them backwards, one for grad_L_XK / grad_L_XV, one that fetches the walk's operands into the L2 ahead of it). */
int ttt_mlp_launch_plan(int which, long long pairs, int compute_units, long long* one_workgroup_pairs,
                        long long* other_pairs, int* workgroups_per_other_pair);

/* With more (batch, head) pairs than CUs the launchers cut every sequence into segments at checkpoint boundaries
 * where that shortens the call: a forward segment starts from the checkpoint that the segment before it left in
 * the caller's checkpoint tensors; a backward segment (the sequence's last groups first) takes the running
 * gradients from grad_L_W1/b1/W2/b2_init, where the one before it left them, and the norm-gradient sums from
 * x_hat_ln_group (needs checkpoint_group_size >= 2).  The (segment, pair) jobs are launched `compute_units` at a
 * time, so a last round that is not full costs a fraction of a sequence instead of a whole one (384 pairs on
 * 256 CUs: 3 launches of half a sequence).  Results do not change by a bit.  This query (no device needed) says
 * what the launchers do for `pairs` pairs of `NC` mini-batches (which = 0 forward, 1 backward; compute_units = 0:
 * the current device's, as the launchers count them):
 * *segment_minibatches = mini-batches per segment (0: sequences are not cut) and *launches = kernel launches of
 * the call; with_workspace = 0 for ttt_mlp_*_launch, 1 for ttt_mlp_*_launch_overlapped.  No counterpart in the
 * reference (kernels/ttt/ttt.cu:699-706 launches one grid of B*NH clusters for whole sequences). */
int ttt_mlp_segment_plan(int which, long long pairs, int compute_units, int NC, int checkpoint_group_size, int with_workspace,
                         int* segment_minibatches, int* launches);

/* Static facts about the compiled kernels, for harnesses: LDS bytes per
 * workgroup and threads per workgroup of the forward (which = 0) or backward
 * (which = 1) kernel.  Returns 0 on success. */
int ttt_mlp_kernel_info(int which, int* lds_bytes, int* threads_per_workgroup);

#ifdef __cplusplus
}
#endif
#endif /* TTT_MLP_H_ */
