// extern "C" entry points declared in include/ttt_mlp.h: argument validation on the host, then
// one asynchronous kernel launch.  Nothing here allocates or synchronises.
#include <atomic>

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
  // ... and one checkpoint slot (64 KiB) with a 32-bit byte offset too
  if (K > (1 << 15)) return TTT_MLP_ERR_TOO_LARGE;
  return TTT_MLP_OK;
}

unsigned long long g_wait_limit = 2000000000ull;   // 20 s of the 100 MHz clock
int g_cu_budget = 0;   // CUs the caller says these launches can count on (0: all the device reports)

inline const __bf16* bf(const uint16_t* p) { return reinterpret_cast<const __bf16*>(p); }
inline __bf16* bf(uint16_t* p) { return reinterpret_cast<__bf16*>(p); }

}  // namespace

extern "C" int ttt_mlp_abi_version(void) { return TTT_MLP_ABI_VERSION; }

extern "C" void ttt_mlp_set_wait_limit(unsigned long long ticks_100mhz) { g_wait_limit = ticks_100mhz; }

extern "C" void ttt_mlp_set_compute_units(int compute_units) { g_cu_budget = compute_units > 0 ? compute_units : 0; }

extern "C" const char* ttt_mlp_error_string(int code) {
  switch (code) {
    case TTT_MLP_OK: return "success";
    case TTT_MLP_ERR_BAD_ARG: return "ttt_mlp: null pointer or non-positive size";
    case TTT_MLP_ERR_BAD_CKPT: return "ttt_mlp: number of checkpoints K must equal ceil(NC / checkpoint_group_size)";
    case TTT_MLP_ERR_ALIGN: return "ttt_mlp: every tensor pointer must be 16-byte aligned";
    case TTT_MLP_ERR_TOO_LARGE: return "ttt_mlp: B*NH exceeds the launch grid limit, or NC > 262144, or checkpoint_group_size > 65536, or more than 32768 checkpoints";
    case TTT_MLP_ERR_NO_ROOM: return "ttt_mlp: two workgroups per (batch, head) do not fit the compute units of this device; use ttt_mlp_fwd_launch / ttt_mlp_bwd_launch";
    case TTT_MLP_ERR_WORKSPACE: return "ttt_mlp: workspace smaller than ttt_mlp_fwd_workspace_bytes() / ttt_mlp_bwd_workspace_bytes()";
    case TTT_MLP_ERR_SCRATCH: return "ttt_mlp: ttt_mlp_fwd_launch_static serves at most 8 (batch, head) pairs (B*NH <= 8): its workspace is a fixed array in device memory";
    default: return hipGetErrorString(static_cast<hipError_t>(code));
  }
}

#ifdef TTT_STAGE_CLOCKS
namespace {
unsigned* g_stage_clocks_fwd = nullptr;
unsigned* g_stage_clocks_bwd = nullptr;
}  // namespace
extern "C" void ttt_mlp_set_stage_clocks(unsigned* forward, unsigned* backward) {
  g_stage_clocks_fwd = forward;
  g_stage_clocks_bwd = backward;
}
#endif

namespace {
int make_fwd_params(const ttt_mlp_fwd_args* a, ttt::FwdParams& p) {
  if (a == nullptr) return TTT_MLP_ERR_BAD_ARG;
  if (any_null(a->XQ, a->XK, a->XV, a->last_eta, a->ttt_norm_weight, a->ttt_norm_bias, a->W1, a->b1, a->W2, a->b2,
               a->W1_checkpoints, a->b1_checkpoints, a->W2_checkpoints, a->b2_checkpoints, a->Out))
    return TTT_MLP_ERR_BAD_ARG;
  if (int rc = check_sizes(a->B, a->NH, a->NC, a->K, a->checkpoint_group_size)) return rc;
  if (!all_aligned(a->XQ, a->XK, a->XV, a->last_eta, a->ttt_norm_weight, a->ttt_norm_bias, a->W1, a->b1, a->W2,
                   a->b2, a->W1_checkpoints, a->b1_checkpoints, a->W2_checkpoints, a->b2_checkpoints, a->Out))
    return TTT_MLP_ERR_ALIGN;
  p = ttt::FwdParams{};
  p.XQ = bf(a->XQ); p.XK = bf(a->XK); p.XV = bf(a->XV); p.last_eta = bf(a->last_eta);
  p.ttt_norm_weight = a->ttt_norm_weight; p.ttt_norm_bias = a->ttt_norm_bias;
  p.W1 = a->W1; p.b1 = a->b1; p.W2 = a->W2; p.b2 = a->b2;
  p.W1_ck = a->W1_checkpoints; p.b1_ck = a->b1_checkpoints; p.W2_ck = a->W2_checkpoints; p.b2_ck = a->b2_checkpoints;
  p.Out = bf(a->Out);
  p.B = a->B; p.NH = a->NH; p.NC = a->NC; p.K = a->K; p.cgs = a->checkpoint_group_size;
#ifdef TTT_STAGE_CLOCKS
  p.stage_clocks = g_stage_clocks_fwd;
#endif
  return TTT_MLP_OK;
}
}  // namespace

namespace {

// Validates the backward arguments and translates them for the kernels.
int make_bwd_params(const ttt_mlp_bwd_args* a, ttt::BwdParams& p) {
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
                   a->W2_init_group, a->b2_init_group, a->x_hat_ln_group, a->std_ln_group, a->X2_group, a->Z1_group,
                   a->Z1_bar_group, a->X2_bar_group, a->grad_l_wrt_Z2_group, a->grad_l_wrt_Z1_group, a->x_hat_fused_group,
                   a->grad_x_hat_fused_group, a->grad_output_fused_group, a->std_fused_group, a->grad_L_W1_last, a->grad_L_b1_last, a->grad_L_W2_last, a->grad_L_b2_last,
                   a->grad_L_XQW_mini_batch, a->grad_L_ttt_norm_weight, a->grad_L_ttt_norm_bias, a->grad_L_W1_init,
                   a->grad_L_b1_init, a->grad_L_W2_init, a->grad_L_b2_init, a->grad_L_last_eta, a->grad_L_XQ,
                   a->grad_L_XK, a->grad_L_XV))
    return TTT_MLP_ERR_ALIGN;
  p = ttt::BwdParams{};
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
  p.overwrite = a->overwrite != 0;
#ifdef TTT_STAGE_CLOCKS
  p.stage_clocks = g_stage_clocks_bwd;
#endif
  return TTT_MLP_OK;
}

// Two workgroups per (batch, head) wait for each other, so all of them must be resident at once: one
// workgroup fills a CU (LDS), hence such a launch may not exceed the CUs of the current device.  The
// (batch, head) pairs are therefore covered by two launches in a row: as many full rounds of one
// workgroup per pair as there are (a multiple of the CU count), then the rest - with two workgroups per
// pair if that fits the device (split), otherwise with one.
struct LaunchPlan {
  long long n_single = 0;   // pairs 0 .. n_single-1: one workgroup each
  long long n_rest = 0;     // pairs n_single .. n_single+n_rest-1
  bool rest_split = false;
  int per_pair = 1;         // workgroups per pair of the rest: 2, or 3 / 4 where the kernel can use them and they fit
  bool prefetch = false;    // backward with 4 per pair: a fifth that fetches ahead of the walk
};
// `three_way`: the backward can use three to five workgroups per pair, the forward two.
LaunchPlan plan_for(long long BH, int cus, bool three_way) {
  LaunchPlan pl;
  if (BH <= 0 || cus <= 0) {
    pl.n_single = BH > 0 ? BH : 0;
    return pl;
  }
  pl.n_single = BH / cus * cus;
  pl.n_rest = BH - pl.n_single;
  pl.rest_split = pl.n_rest > 0 && 2 * pl.n_rest <= cus;
  if (!pl.rest_split) { pl.n_single = BH; pl.n_rest = 0; }
  else pl.per_pair = !three_way ? 2 : 4 * pl.n_rest <= cus ? 4 : 3 * pl.n_rest <= cus ? 3 : 2;
  // the fifth workgroup helps only from the walk's own XCD, which the kernel arranges for a multiple of 8 pairs
  pl.prefetch = pl.per_pair == 4 && 5 * pl.n_rest <= cus && pl.n_rest % 8 == 0;
  return pl;
}
LaunchPlan plan_launches(long long BH, bool three_way) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    cus = 0;
  if (g_cu_budget > 0 && g_cu_budget < cus) cus = g_cu_budget;
  return plan_for(BH, cus, three_way);
}

// More (batch, head) pairs than CUs, one workgroup each: the hardware runs them in rounds, and a last round that is
// not full leaves CUs idle for a whole sequence.  The forward can cut every sequence into segments at checkpoint
// boundaries instead - a segment starts from the checkpoint before its first mini-batch, which the segment before it
// left in the caller's checkpoint tensors - and launch the (segment, pair) jobs segment-major, one launch per `cus`
// jobs: a pair's earlier segment is always in an earlier launch (pairs >= cus), and the rounds are a fraction of a
// sequence long, so 384 pairs on 256 CUs take 3 launches of half a sequence, 1.5 sequences instead of 2 (or 1.76 with
// the last 128 pairs on two workgroups each).  Same arithmetic on the same state: results do not change.
struct SegmentPlan {
  int seg_len = 0;      // mini-batches per segment, a multiple of cgs; 0 = sequences are not cut
  int groups = 0;       // checkpoint groups per segment
  int launches = 1;
  long long jobs = 0;
};
#ifndef TTT_CUT_PERCENT
#define TTT_CUT_PERCENT 99   // a cut must gain 1 % by the estimate below
#endif
// `alt_x1000`: what the alternative costs, in thousandths of a mini-batch of one workgroup.
SegmentPlan plan_segments(long long pairs, int cus, int NC, int cgs, long long alt_x1000) {
  SegmentPlan best;
#ifndef TTT_STAGE_CLOCKS   // the stage clocks are kept per pair and sequence
  if (pairs <= cus || pairs > (1 << 27) || cus <= 0 || NC <= 0 || cgs <= 0) return best;   // (job numbers are ints)
  const int K = (NC + cgs - 1) / cgs;
  long long best_t = alt_x1000 * TTT_CUT_PERCENT / 100;
  for (int S = 2; S <= 8 && S <= K; S++) {
    const int groups = (K + S - 1) / S, segs = (K + groups - 1) / groups;
    const long long len = (long long)groups * cgs, jobs = segs * pairs, launches = (jobs + cus - 1) / cus;
    const long long t = launches * (len * 1000 + 2000);   // + 2 mini-batches' worth per launch: gaps, state in and out
    if (t < best_t) {
      best_t = t;
      best.seg_len = static_cast<int>(len);
      best.groups = groups;
      best.launches = static_cast<int>(launches);
      best.jobs = jobs;
    }
  }
#endif
  return best;
}
// Thousandths of a one-workgroup mini-batch that the pairs take uncut: full rounds, and the rest either one more
// round or, with several workgroups per pair, a shorter one - measured with every CU busy: the forward's recurrence
// workgroup runs at 0.755 of one workgroup's time per mini-batch; the backward's walk with one replaying workgroup
// at 0.56, and about 0.4 / 0.3 with more workgroups per pair.
long long uncut_x1000(const LaunchPlan& pl, long long pairs, int cus, int NC, bool with_workspace, bool backward) {
  if (cus <= 0) return (long long)NC * 1000;
  if (with_workspace && pl.rest_split) {
    const int rest = !backward ? 755 : pl.per_pair == 2 ? 560 : pl.per_pair == 3 ? 400 : 300;
    return (pl.n_single / cus * 1000 + rest) * NC;
  }
  return (pairs + cus - 1) / cus * 1000 * NC;
}
int device_cus() {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return 0;
  return g_cu_budget > 0 && g_cu_budget < cus ? g_cu_budget : cus;
}
// The launches of a call with the sequences cut: `cus` jobs each, in job order, on the one stream.
template <class Params, class Enqueue>
int launch_segments(Params p, const SegmentPlan& plan, int cus, Enqueue enqueue) {
  p.sync = nullptr;
  p.bh0 = 0;
  for (long long j0 = 0; j0 < plan.jobs; j0 += cus) {
    p.job0 = static_cast<int>(j0);
    p.nbh = static_cast<int>(plan.jobs - j0 < cus ? plan.jobs - j0 : cus);
    if (hipError_t e = enqueue(p)) return static_cast<int>(e);
  }
  return TTT_MLP_OK;
}
int launch_fwd_segments(ttt::FwdParams p, const SegmentPlan& plan, int cus, hipStream_t stream) {
  p.seg_len = plan.seg_len;
  return launch_segments(p, plan, cus, [stream](const ttt::FwdParams& q) { return ttt_mlp_fwd_enqueue(q, stream); });
}
// Backward: segment 0 = the last groups of every sequence.  The third parked norm-gradient sum needs a second
// mini-batch slot in x_hat_ln_group, hence cgs >= 2 (plan_bwd_segments).
int launch_bwd_segments(ttt::BwdParams p, const SegmentPlan& plan, int cus, hipStream_t stream) {
  p.seg_groups = plan.groups;
  return launch_segments(p, plan, cus, [stream](const ttt::BwdParams& q) { return ttt_mlp_bwd_enqueue(q, stream); });
}
SegmentPlan plan_bwd_segments(const LaunchPlan& pl, long long pairs, int cus, int NC, int cgs, bool with_workspace) {
  if (cgs < 2) return SegmentPlan{};
  return plan_segments(pairs, cus, NC, cgs, uncut_x1000(pl, pairs, cus, NC, with_workspace, true));
}

// Workspace of the backward with 2 or 3 workgroups per pair, for n (batch, head) pairs: the synchronisation
// words, the replay's shares of the norm gradients (two sums per pair + one parking slot), then 1 or 3
// alternate sets of the ten per-group tensors that carry a replayed group to the reverse walk; each part
// 256-byte aligned.
struct BwdWorkspace {
  static constexpr int PER_SET = 11;
  static constexpr int PARTS = 8 + PER_SET * 3;
  size_t off[PARTS];
  size_t total;
  BwdWorkspace(long long n, long long cgs, int alt_sets, bool finish) {
    const size_t slot = (size_t)n * (size_t)cgs;
    const size_t tile = TTT_MLP_CS * TTT_MLP_F * 2, img = TTT_MLP_CS * TTT_MLP_HID * 2, vec = TTT_MLP_CS * 4;
    const size_t norm = (size_t)n * 8 * 2 * TTT_MLP_F * sizeof(float);
    // per set: X2, Z1, Z1_bar, X2_bar (images), gZ2 (tile), gZ1 (image), x_hat_fused, g_x_hat_fused, g_out_fused
    // (tiles), std_fused, W1_init (two images per slot)
    const size_t per_set[PER_SET] = {slot * img, slot * img, slot * img, slot * img, slot * tile, slot * img,
                                     slot * tile, slot * tile, slot * tile, slot * vec, slot * 2 * img};
    size_t o = 0;
    auto put = [&](int i, size_t bytes) { off[i] = o; o += (bytes + 255) & ~(size_t)255; };
    put(0, ttt::bwd_sync_ints(n) * sizeof(int));
    put(1, 2 * norm);
    put(2, norm);
    put(3, (size_t)n * img);
    // hand-over to the grad_L_XK workgroup: one image (dZ1) and two fp32 tiles (g_y, norm-weight gradient terms) per slot, two sets
    put(4, 0);
    put(5, 0);
    put(6, finish ? 2 * slot * img : 0);
    put(7, finish ? 2 * slot * 4 * tile : 0);
    for (int s = 0; s < 3; s++)
      for (int t = 0; t < PER_SET; t++) put(8 + PER_SET * s + t, s < alt_sets ? per_set[t] : 0);
    total = o;
  }
};

// Workspace of the forward's two-workgroup mode: synchronisation words, then per (batch, head) a ring of
// 2 * FWD_RING_MAX slots of state images and of bias vectors.
struct FwdWorkspace {
  size_t off[3];
  size_t total;
  explicit FwdWorkspace(long long n) {
    const size_t slots = (size_t)n * 2 * ttt::FWD_RING_MAX;
    const size_t bytes[3] = {ttt::bwd_sync_ints(n) * sizeof(int), slots * ttt::FWD_IMG_BYTES,
                             slots * ttt::FWD_BIAS_FLOATS * sizeof(float)};
    size_t o = 0;
    for (int i = 0; i < 3; i++) { off[i] = o; o += (bytes[i] + 255) & ~(size_t)255; }
    total = o;
  }
};

int check_workspace(const void* workspace) {
  if (workspace == nullptr) return TTT_MLP_ERR_BAD_ARG;
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return TTT_MLP_ERR_ALIGN;
  return TTT_MLP_OK;
}

}  // namespace

extern "C" int ttt_mlp_bwd_launch(const ttt_mlp_bwd_args* a, void* stream) {
  ttt::BwdParams p;
  if (int rc = make_bwd_params(a, p)) return rc;
  {
    const long long pairs = (long long)p.B * p.NH;
    const int cus = device_cus();
    const SegmentPlan seg = plan_bwd_segments(LaunchPlan{}, pairs, cus, p.NC, p.cgs, false);
    if (seg.seg_len > 0) return launch_bwd_segments(p, seg, cus, static_cast<hipStream_t>(stream));
  }
  p.bh0 = 0;
  p.nbh = p.B * p.NH;
  return static_cast<int>(ttt_mlp_bwd_enqueue(p, static_cast<hipStream_t>(stream)));
}

extern "C" int ttt_mlp_bwd_export_group0(const ttt_mlp_bwd_args* a, void* stream) {
  ttt::BwdParams p;
  if (int rc = make_bwd_params(a, p)) return rc;
  p.bh0 = 0;
  p.nbh = p.B * p.NH;
  return static_cast<int>(ttt_mlp_export_group0_enqueue(p, static_cast<hipStream_t>(stream)));
}

extern "C" size_t ttt_mlp_bwd_workspace_bytes(int B, int NH, int checkpoint_group_size) {
  if (B <= 0 || NH <= 0 || checkpoint_group_size <= 0 || checkpoint_group_size > (1 << 16)) return 0;
  const LaunchPlan pl = plan_launches((long long)B * NH, true);
  if (!pl.rest_split) return 0;
  const int n_replay = pl.per_pair >= 3 ? 2 : 1;
  return BwdWorkspace(pl.n_rest, checkpoint_group_size, 2 * n_replay - 1, pl.per_pair == 4).total;
}

extern "C" size_t ttt_mlp_bwd_status_offset(int B, int NH) {
  if (B <= 0 || NH <= 0) return 0;
  const LaunchPlan pl = plan_launches((long long)B * NH, true);
  return pl.rest_split ? (size_t)pl.n_rest * ttt::BWD_SYNC_STRIDE * sizeof(int) : 0;
}

extern "C" int ttt_mlp_bwd_launch_overlapped(const ttt_mlp_bwd_args* a, void* workspace, size_t workspace_bytes, void* stream) {
  ttt::BwdParams p;
  if (int rc = make_bwd_params(a, p)) return rc;
  if (int rc = check_workspace(workspace)) return rc;
  const LaunchPlan pl = plan_launches((long long)p.B * p.NH, true);
  if (!pl.rest_split) return TTT_MLP_ERR_NO_ROOM;
  const int n_replay = pl.per_pair >= 3 ? 2 : 1, alt_sets = 2 * n_replay - 1;
  const bool finish = pl.per_pair == 4;
  const BwdWorkspace w(pl.n_rest, p.cgs, alt_sets, finish);
  if (workspace_bytes < w.total) return TTT_MLP_ERR_WORKSPACE;
  char* base = static_cast<char*>(workspace);
  {
    // cut sequences where they beat a last round on several workgroups per pair (see the forward)
    const long long pairs = (long long)p.B * p.NH;
    const int cus = device_cus();
    const SegmentPlan seg = plan_bwd_segments(pl, pairs, cus, p.NC, p.cgs, true);
    if (seg.seg_len > 0) {
      if (hipError_t e = ttt_mlp_fwd_clear_words(reinterpret_cast<int*>(base + w.off[0]), static_cast<int>(ttt::bwd_sync_ints(pl.n_rest)),
                                                 static_cast<hipStream_t>(stream)))
        return static_cast<int>(e);
      return launch_bwd_segments(p, seg, cus, static_cast<hipStream_t>(stream));
    }
  }
  if (pl.n_single > 0) {
    p.bh0 = 0;
    p.nbh = static_cast<int>(pl.n_single);
    if (hipError_t e = ttt_mlp_bwd_enqueue(p, static_cast<hipStream_t>(stream))) return static_cast<int>(e);
  }
  // The kernels index the workspace by the global pair number: every pointer is moved back by bh0 entries.
  const size_t b0 = (size_t)pl.n_single;
  const size_t tile = (size_t)p.cgs * TTT_MLP_CS * TTT_MLP_F, img = (size_t)p.cgs * TTT_MLP_CS * TTT_MLP_HID, vec = (size_t)p.cgs * TTT_MLP_CS;
  const size_t norm = 8 * 2 * TTT_MLP_F;
  p.bh0 = static_cast<int>(pl.n_single);
  p.nbh = static_cast<int>(pl.n_rest);
  p.n_replay = n_replay;
  p.n_finish = finish ? 1 : 0;
  p.n_prefetch = pl.prefetch ? 1 : 0;
  p.wait_limit = g_wait_limit;
  if (finish) {
    p.fin_dz = reinterpret_cast<__bf16*>(base + w.off[6]) - b0 * 2 * img;
    p.fin_gy = reinterpret_cast<float*>(base + w.off[7]) - b0 * 2 * 2 * tile;
  }
  int* words = reinterpret_cast<int*>(base + w.off[0]);
  p.status = words + (size_t)pl.n_rest * ttt::BWD_SYNC_STRIDE;
  p.sync = words - b0 * ttt::BWD_SYNC_STRIDE;
  p.norm_partial = reinterpret_cast<float*>(base + w.off[1]) - b0 * 2 * norm;
  p.norm_park = reinterpret_cast<float*>(base + w.off[2]) - b0 * norm;
  p.walk_park = reinterpret_cast<__bf16*>(base + w.off[3]) - b0 * (TTT_MLP_CS * TTT_MLP_HID);
  for (int s = 0; s < alt_sets; s++) {
    const size_t* o = w.off + 8 + BwdWorkspace::PER_SET * s;
    p.alt_X2_group[s] = reinterpret_cast<__bf16*>(base + o[0]) - b0 * img;
    p.alt_Z1_group[s] = reinterpret_cast<__bf16*>(base + o[1]) - b0 * img;
    p.alt_Z1_bar_group[s] = reinterpret_cast<__bf16*>(base + o[2]) - b0 * img;
    p.alt_X2_bar_group[s] = reinterpret_cast<__bf16*>(base + o[3]) - b0 * img;
    p.alt_grad_l_wrt_Z2_group[s] = reinterpret_cast<__bf16*>(base + o[4]) - b0 * tile;
    p.alt_grad_l_wrt_Z1_group[s] = reinterpret_cast<__bf16*>(base + o[5]) - b0 * img;
    p.alt_x_hat_fused_group[s] = reinterpret_cast<__bf16*>(base + o[6]) - b0 * tile;
    p.alt_grad_x_hat_fused_group[s] = reinterpret_cast<__bf16*>(base + o[7]) - b0 * tile;
    p.alt_grad_output_fused_group[s] = reinterpret_cast<__bf16*>(base + o[8]) - b0 * tile;
    p.alt_std_fused_group[s] = reinterpret_cast<float*>(base + o[9]) - b0 * vec;
    p.alt_W1_init_group[s] = reinterpret_cast<float*>(base + o[10]) - b0 * img;   // [cgs][64][256] floats = 2 images per slot
  }
  return static_cast<int>(ttt_mlp_bwd_enqueue(p, static_cast<hipStream_t>(stream)));
}

extern "C" int ttt_mlp_fwd_launch(const ttt_mlp_fwd_args* a, void* stream) {
  ttt::FwdParams p;
  if (int rc = make_fwd_params(a, p)) return rc;
  const long long pairs = (long long)p.B * p.NH;
  const int cus = device_cus();
  const SegmentPlan seg = plan_segments(pairs, cus, p.NC, p.cgs, uncut_x1000(LaunchPlan{}, pairs, cus, p.NC, false, false));
  if (seg.seg_len > 0) return launch_fwd_segments(p, seg, cus, static_cast<hipStream_t>(stream));
  p.bh0 = 0;
  p.nbh = p.B * p.NH;
  return static_cast<int>(ttt_mlp_fwd_enqueue(p, static_cast<hipStream_t>(stream)));
}

extern "C" size_t ttt_mlp_fwd_workspace_bytes(int B, int NH) {
  if (B <= 0 || NH <= 0) return 0;
  const LaunchPlan pl = plan_launches((long long)B * NH, false);
  return pl.rest_split ? FwdWorkspace(pl.n_rest).total : 0;
}

extern "C" size_t ttt_mlp_fwd_status_offset(int B, int NH) {
  if (B <= 0 || NH <= 0) return 0;
  const LaunchPlan pl = plan_launches((long long)B * NH, false);
  return pl.rest_split ? (size_t)pl.n_rest * ttt::BWD_SYNC_STRIDE * sizeof(int) : 0;
}

extern "C" int ttt_mlp_fwd_launch_overlapped(const ttt_mlp_fwd_args* a, void* workspace, size_t workspace_bytes, void* stream) {
  ttt::FwdParams p;
  if (int rc = make_fwd_params(a, p)) return rc;
  if (int rc = check_workspace(workspace)) return rc;
  const LaunchPlan pl = plan_launches((long long)p.B * p.NH, false);
  if (!pl.rest_split) return TTT_MLP_ERR_NO_ROOM;
  const FwdWorkspace w(pl.n_rest);
  if (workspace_bytes < w.total) return TTT_MLP_ERR_WORKSPACE;
  char* base = static_cast<char*>(workspace);
  {
    // cut sequences beat a last round on two workgroups per pair where there are full rounds before it: the
    // workspace then only has its words cleared (callers read the status word behind them)
    const long long pairs = (long long)p.B * p.NH;
    const int cus = device_cus();
    const SegmentPlan seg = plan_segments(pairs, cus, p.NC, p.cgs, uncut_x1000(pl, pairs, cus, p.NC, true, false));
    if (seg.seg_len > 0) {
      if (hipError_t e = ttt_mlp_fwd_clear_words(reinterpret_cast<int*>(base + w.off[0]), static_cast<int>(ttt::bwd_sync_ints(pl.n_rest)),
                                                 static_cast<hipStream_t>(stream)))
        return static_cast<int>(e);
      return launch_fwd_segments(p, seg, cus, static_cast<hipStream_t>(stream));
    }
  }
  if (pl.n_single > 0) {
    p.bh0 = 0;
    p.nbh = static_cast<int>(pl.n_single);
    if (hipError_t e = ttt_mlp_fwd_enqueue(p, static_cast<hipStream_t>(stream))) return static_cast<int>(e);
  }
  const size_t b0 = (size_t)pl.n_single;
  p.bh0 = static_cast<int>(pl.n_single);
  p.nbh = static_cast<int>(pl.n_rest);
  int* words = reinterpret_cast<int*>(base + w.off[0]);
  p.status = words + (size_t)pl.n_rest * ttt::BWD_SYNC_STRIDE;
  p.sync = words - b0 * ttt::BWD_SYNC_STRIDE;
  p.wait_limit = g_wait_limit;
  p.ring_log2 = p.NC >= 512 ? 5 : 3;   // 32 or 8 mini-batches per hand-over
  p.state_img = reinterpret_cast<__bf16*>(base + w.off[1]) - b0 * 2 * ttt::FWD_RING_MAX * (ttt::FWD_IMG_BYTES / 2);
  p.bias_img = reinterpret_cast<float*>(base + w.off[2]) - b0 * 2 * ttt::FWD_RING_MAX * ttt::FWD_BIAS_FLOATS;
  return static_cast<int>(ttt_mlp_fwd_enqueue(p, static_cast<hipStream_t>(stream)));
}

// ---------------------------------------------------------------------------------------------------------
// The two-workgroup forward for callers that cannot allocate and have no workspace to bring: its workspace
// is this fixed array (one copy per GPU, held until the process ends).  Host code never passes the array's
// name to a kernel - the name is a host-side stand-in, not a device address; the address on each device
// comes from hipGetSymbolAddress, once per device.
namespace {
constexpr int STATIC_MAX_PAIRS = 8;
constexpr size_t static_scratch_bytes() {
  // FwdWorkspace(STATIC_MAX_PAIRS): synchronisation words, state images, bias vectors; each part 256-byte aligned
  const size_t slots = (size_t)STATIC_MAX_PAIRS * 2 * ttt::FWD_RING_MAX;
  const size_t a = ((STATIC_MAX_PAIRS * ttt::BWD_SYNC_STRIDE + 32) * sizeof(int) + 255) & ~(size_t)255;
  const size_t b = (slots * ttt::FWD_IMG_BYTES + 255) & ~(size_t)255;
  const size_t c = (slots * ttt::FWD_BIAS_FLOATS * sizeof(float) + 255) & ~(size_t)255;
  return a + b + c;
}
static __device__ __align__(256) unsigned char scratch[static_scratch_bytes()];   // 32.6 MiB

constexpr int MAX_DEVICES = 64;
// address of `scratch` on each device, looked up at the first call there; host threads may race to the first
// call - every one of them finds the same address, so an atomic slot per device is all the guard it needs
std::atomic<void*> g_scratch_ptr[MAX_DEVICES] = {};

// The current device's copy of the array (the device that the launch goes to).  Looked up once per device.
int static_scratch(void** ptr) {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return static_cast<int>(e);
  if (dev < 0 || dev >= MAX_DEVICES) return TTT_MLP_ERR_BAD_ARG;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) return static_cast<int>(e);
    if (p == nullptr) return TTT_MLP_ERR_BAD_ARG;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *ptr = p;
  return TTT_MLP_OK;
}

__global__ void ttt_mlp_or_status(const int* status, int* sticky) {
  if (*status != 0) *sticky = 1;
}
}  // namespace

extern "C" int ttt_mlp_status_accumulate(const void* status_word, int* sticky_word, void* stream) {
  if (status_word == nullptr || sticky_word == nullptr) return TTT_MLP_ERR_BAD_ARG;
  hipLaunchKernelGGL(ttt_mlp_or_status, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream),
                     static_cast<const int*>(status_word), sticky_word);
  return static_cast<int>(hipGetLastError());
}

extern "C" int ttt_mlp_fwd_launch_static(const ttt_mlp_fwd_args* a, int* sticky_word, void* stream) {
  ttt::FwdParams p;
  if (int rc = make_fwd_params(a, p)) return rc;
  const long long pairs = (long long)p.B * p.NH;
  if (pairs > STATIC_MAX_PAIRS) return TTT_MLP_ERR_SCRATCH;
  const LaunchPlan pl = plan_launches(pairs, false);
  if (!pl.rest_split || pl.n_single != 0) return TTT_MLP_ERR_NO_ROOM;
  const FwdWorkspace w(pl.n_rest);
  static_assert(static_scratch_bytes() % 256 == 0, "scratch parts are 256-byte aligned");
  if (w.total > static_scratch_bytes()) return TTT_MLP_ERR_SCRATCH;
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // From here on as ttt_mlp_fwd_launch_overlapped with `ws` as the workspace: the launch clears the
  // synchronisation words and the status word itself (a small kernel ahead of the main one), everything
  // else in the workspace is written before it is read.
  if (int rc = ttt_mlp_fwd_launch_overlapped(a, ws, static_scratch_bytes(), stream)) return rc;
  if (sticky_word != nullptr) {
    const int* status = reinterpret_cast<const int*>(static_cast<const char*>(ws) + w.off[0]) + (size_t)pl.n_rest * ttt::BWD_SYNC_STRIDE;
    return ttt_mlp_status_accumulate(status, sticky_word, stream);
  }
  return TTT_MLP_OK;
}

extern "C" int ttt_mlp_launch_plan(int which, long long pairs, int compute_units, long long* one_workgroup_pairs,
                                   long long* other_pairs, int* workgroups_per_other_pair) {
  if (one_workgroup_pairs == nullptr || other_pairs == nullptr || workgroups_per_other_pair == nullptr || (which != 0 && which != 1))
    return TTT_MLP_ERR_BAD_ARG;
  const LaunchPlan pl = plan_for(pairs, compute_units, which == 1);
  *one_workgroup_pairs = pl.n_single;
  *other_pairs = pl.n_rest;
  *workgroups_per_other_pair = pl.n_rest > 0 ? pl.per_pair + (pl.prefetch ? 1 : 0) : 0;
  return TTT_MLP_OK;
}

extern "C" int ttt_mlp_segment_plan(int which, long long pairs, int compute_units, int NC, int checkpoint_group_size, int with_workspace,
                                    int* segment_minibatches, int* launches) {
  if (compute_units == 0) compute_units = device_cus();   // the current device's, or the budget set for it
  if (segment_minibatches == nullptr || launches == nullptr || pairs <= 0 || compute_units <= 0 || NC <= 0 ||
      checkpoint_group_size <= 0 || (which != 0 && which != 1))
    return TTT_MLP_ERR_BAD_ARG;
  const LaunchPlan pl = plan_for(pairs, compute_units, which == 1);
  const SegmentPlan seg = which == 1 ? plan_bwd_segments(pl, pairs, compute_units, NC, checkpoint_group_size, with_workspace != 0)
                                     : plan_segments(pairs, compute_units, NC, checkpoint_group_size,
                                                     uncut_x1000(pl, pairs, compute_units, NC, with_workspace != 0, false));
  *segment_minibatches = seg.seg_len;
  *launches = seg.seg_len > 0 ? seg.launches : (with_workspace != 0 && pl.rest_split && pl.n_single > 0 ? 2 : 1);
  return TTT_MLP_OK;
}

extern "C" int ttt_mlp_kernel_info(int which, int* lds_bytes, int* threads_per_workgroup) {
  if (lds_bytes == nullptr || threads_per_workgroup == nullptr) return TTT_MLP_ERR_BAD_ARG;
  if (which == 0) { *lds_bytes = ttt_mlp_fwd_lds_bytes(); *threads_per_workgroup = ttt_mlp_fwd_threads(); return TTT_MLP_OK; }
  if (which == 1) { *lds_bytes = ttt_mlp_bwd_lds_bytes(); *threads_per_workgroup = ttt_mlp_bwd_threads(); return TTT_MLP_OK; }
  return TTT_MLP_ERR_BAD_ARG;
}
