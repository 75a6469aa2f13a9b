// Remat backward of the non-causal TTT-MLP layer for gfx950 (MI355X).
//
// Behaviour follows the upstream operator `ttt_backward` (kernel kernels/ttt_backward/ttt.cu:179-1443,
// mathematics kernels/ttt_backward/matching.py:57-342, group walk :539-663): for every checkpoint
// group, last to first, the forward is replayed from the checkpoint while the per-mini-batch
// activations are saved, then the group is walked backwards producing the ten output gradients.
//
// Mapping: workgroups of 8 wavefronts (two per SIMD, at most 256 registers each); one per (batch,
// head), or two to five where the device has CUs to spare - then one or two replay the checkpoint
// groups (taking turns), one walks them backwards, a group or more behind, a fourth forms
// grad_L_XK from what the walk hands it, and a fifth reads ahead of the walk into the L2.  Wave v owns hidden columns [32v, 32v+32).  All [tokens x hidden] activations live in
// registers in the "Q" orientation (accumulator rows = hidden, lane = token), so per-token scalars
// (eta, dEta partial sums) are per-lane values.  An activation that is also needed with tokens as the
// contraction index is bounced once through a wave-private LDS tile (row store + transposing read).
//
// Waves v and v^4 form a pair.  A wave keeps the two token blocks of a Q tile in the order (r, 1-r),
// r = v / 4: of every product summed over the hidden dimension it keeps token block r and hands token
// block 1-r to its partner through LDS, which adds its own share; the LayerNorm lanes (8 per token,
// 8 tokens per wave) then add the four pair sums.  Every sum has a fixed order.
//
// State in registers:
//   replay : W1s [F x hid], W2s [hid x F] (fp32 accumulator tiles; where W2 is needed with F contracted, the bf16
//            terms of W2s are transposed through a wave-private LDS tile); b1, b2 in LDS
//   reverse: gW1s [F x hid], gW2s [hid x F] (running gradients) only; gb1, gb2 in LDS.  The weights
//            enter the reverse walk as ready-made bf16 MFMA operands: after every mini-batch the replay
//            stores the operand images of W1^T[shard] and W2[shard]^T, and the walk reads the image of
//            the state after and before the step (before the first step of a group: converted straight
//            from the fp32 checkpoint).
// The output branch (Out depends on the state after a step, nothing later depends on it) is taken
// backwards inside the replay, where that state is still in registers: the replay writes dXQ and
// leaves dL/dZ2_bar and the operands X2_bar^T, (dL/dZ1_bar)^T, so that the walk only accumulates their
// products into the running gradients.
// While a group is replayed by the workgroup that also walks, the running gradients are parked in the
// caller's W*_init_group scratch.
// Saved per mini-batch (caller's *_group scratch): Z1 as a bf16 register image (Z1_group); the operand
// images X2_bar^T (X2_bar_group) and (dL/dZ1_bar)^T (Z1_bar_group); the two weight operand images
// (X2_group: W1^T[shard], grad_l_wrt_Z1_group: W2[shard]^T); x_hat / grad_output of the fused LayerNorm
// loss, dl/dZ2 and dL/dZ2_bar (grad_x_hat_fused_group) as bf16 [tok][F] tiles; the fused std in fp32.
#include "ttt_mlp_common.hpp"
#include "ttt_mlp_kernels.hpp"

namespace ttt {

// Zeros standing in for the old contents of an output tile (8 KiB) when the outputs are overwritten rather
// than added to: the load stays where it is in the instruction stream and is served by the L2.
__device__ __attribute__((aligned(256))) const uint4 zero_tile[512] = {};

constexpr int BW_NWAVE = 8;
constexpr int BW_THREADS = 64 * BW_NWAVE;
constexpr int BW_NS = HID / BW_NWAVE;     // hidden columns per wave: 32
constexpr int LDX = 68;                   // row stride (elements) of the shared [64][64] bf16 tiles
constexpr int LDH = 36;                   // row stride of wave-private [64][32 hid] bf16 tiles
constexpr int LDF = 68;                   // row stride of wave-private [32 hid][64 F] bf16 tiles
constexpr int LDR = 68;                   // row stride (floats) of a pair-sum region [32 tok][64 F]: 16-byte accesses of
                                          // 16 consecutive rows fall on 64 distinct banks
constexpr int RGN = 2304;                 // floats per pair-sum region

constexpr int SB_TILE = 64 * LDX * 2;     // 8704
constexpr int SB_XQ = 0;                  // reverse: XQ until the post-update stage is done, then (with SB_E2)
constexpr int SB_E2 = SB_XQ + SB_TILE;    //          the fp32 park of g_y ; replay: XQ and XV
constexpr int SB_XK = SB_E2 + SB_TILE;
constexpr int SB_GZ2 = SB_XK + SB_TILE;   // replay: G2 = -eta*dl/dZ2 ; reverse: raw dl/dZ2
constexpr int SB_A = SB_GZ2 + SB_TILE;    // reverse: gZ2_bar, later dZ2
static_assert(2 * SB_TILE >= CS * FD * 4, "g_y park does not fit");
static_assert(32 * XPAIR * 2 <= SB_TILE, "a tile of row pairs fits a tile slot");
constexpr int SB_P = SB_A + SB_TILE;      // 8 pair-sum regions (one per wave), fp32 [32][LDR]
constexpr int SB_REGION = RGN * 4;        // 9216: also two wave-private bf16 tiles
static_assert(32 * LDR <= RGN, "pair-sum rows do not fit their region");
constexpr int SB_WTILE = 64 * LDH * 2;    // 4608
static_assert(2 * SB_WTILE <= SB_REGION && 32 * LDF * 2 <= SB_WTILE, "private tiles do not fit a region");
constexpr int SB_BNC = SB_P + BW_NWAVE * SB_REGION;   // 8 wave-private bounce tiles [64][LDH]
constexpr int SB_B1 = SB_BNC + BW_NWAVE * SB_WTILE;   // b1 during a replay, 256 floats
constexpr int SB_B2 = SB_B1 + HID * 4;        // b2 during a replay, 64 floats
constexpr int SB_GB1 = SB_B2 + FD * 4;        // running gradient wrt b1
constexpr int SB_GB2 = SB_GB1 + HID * 4;      // running gradient wrt b2
constexpr int SB_GAM = SB_GB2 + FD * 4;       // ttt_norm_weight of this head
constexpr int SB_BET = SB_GAM + FD * 4;       // ttt_norm_bias of this head
constexpr int SB_ETA = SB_BET + FD * 4;
constexpr int SB_DETA = SB_ETA + CS * 4;                  // [8 waves][64 tokens] partial dEta sums
constexpr int SB_RED = SB_DETA + BW_NWAVE * CS * 4;       // [8 waves][2][64] norm-gradient accumulators
constexpr int SB_FLAG = SB_RED + BW_NWAVE * 2 * FD * 4;   // outcome of a wait on the other workgroup
constexpr int SM_BWD_BYTES = SB_FLAG + 16;
static_assert(SM_BWD_BYTES <= 160 * 1024, "LDS budget of one gfx950 CU exceeded");

#define WAVE_SYNC() TTT_WAVE_SYNC()
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16((a), (b), (c), 0, 0, 0)

// ------------------------------------------------------------------ register images in HBM
// A [64 tok x 32 hid] (or [64 F x 32 hid]) bf16 operand as 4 chunks of 8 bf16 per lane; chunk n of
// thread tid sits at (n*512 + tid)*16 bytes, so every load/store instruction of a wave moves 1 KiB.
// `img` = byte offset of the image inside the buffer, `t16` = 16 * tid.
constexpr unsigned IMG_BYTES = CS * HID * 2;          // 32 KiB
constexpr unsigned CHUNK_BYTES = BW_THREADS * 16;     // 8 KiB
constexpr unsigned TILE_BYTES = CS * FD * 2;          // one [64][64] bf16 tile in HBM: 8 KiB
TTT_DEV void chunk_store(gptr_t b, unsigned img, int n, unsigned t16, bf16x8 v) { g_st8h(b, t16, img + n * CHUNK_BYTES, v); }
// The replay's images: written once and read a checkpoint group later.  When another workgroup reads them
// (STREAM) they bypass the cache hierarchy as far as the hardware lets them, so that they do not push out
// lines that are re-used; with one workgroup per (batch, head) keeping them cached measured faster.
template <bool STREAM>
TTT_DEV void image_store(gptr_t b, unsigned img, int n, unsigned t16, bf16x8 v) {
  if constexpr (STREAM) g_st_stream<bf16x8>(b, t16, img + n * CHUNK_BYTES, v);
  else g_st8h(b, t16, img + n * CHUNK_BYTES, v);
}
template <bool STREAM>
TTT_DEV bf16x8 image_load(gptr_t b, unsigned img, int n, unsigned t16) {
  if constexpr (STREAM) return g_ld_stream<bf16x8>(b, t16, img + n * CHUNK_BYTES);
  else return g_ld8h(b, t16, img + n * CHUNK_BYTES);
}
TTT_DEV bf16x8 chunk_load(gptr_t b, unsigned img, int n, unsigned t16) { return g_ld8h(b, t16, img + n * CHUNK_BYTES); }

// fp32 accumulator tile <-> HBM in the caller's row-major layout.  `ld` = row length, (r0, c0) =
// origin of this wave's block (wave-uniform); accumulator rows are tensor rows.
template <int RB, int CB>
TTT_DEV void acc_load_rows(AccT<RB, CB>& a, gptr_t g, unsigned off, int ld, int r0, int c0, int c, int h) {
  const unsigned vo = (4 * h * ld + c) * 4;
#pragma unroll
  for (int rb = 0; rb < RB; rb++)
#pragma unroll
    for (int cb = 0; cb < CB; cb++)
#pragma unroll
      for (int i = 0; i < 16; i++)
        a.b[rb][cb][i] = g_ldf(g, vo, off + ((r0 + 32 * rb + 8 * (i >> 2) + (i & 3)) * ld + c0 + 32 * cb) * 4);
}
template <int RB, int CB>
TTT_DEV void acc_store_rows(const AccT<RB, CB>& a, gptr_t g, unsigned off, int ld, int r0, int c0, int c, int h) {
  const unsigned vo = (4 * h * ld + c) * 4;
#pragma unroll
  for (int rb = 0; rb < RB; rb++)
#pragma unroll
    for (int cb = 0; cb < CB; cb++)
#pragma unroll
      for (int i = 0; i < 16; i++)
        g_stf(g, vo, off + ((r0 + 32 * rb + 8 * (i >> 2) + (i & 3)) * ld + c0 + 32 * cb) * 4, a.b[rb][cb][i]);
}
// Same, but accumulator rows are tensor COLUMNS (the tile holds the transpose of the block).
template <int RB, int CB>
TTT_DEV void acc_load_cols(AccT<RB, CB>& a, gptr_t g, unsigned off, int ld, int r0, int c0, int c, int h) {
  const unsigned vo = (c * ld + 4 * h) * 4;
#pragma unroll
  for (int rb = 0; rb < RB; rb++)
#pragma unroll
    for (int cb = 0; cb < CB; cb++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const f32x4 x = g_ld4f(g, vo, off + ((r0 + 32 * cb) * ld + c0 + 32 * rb + 8 * g4) * 4);
#pragma unroll
        for (int e = 0; e < 4; e++) a.b[rb][cb][4 * g4 + e] = x[e];
      }
}

// ------------------------------------------------------------------ LayerNorm-lane helpers
// A lane of a LayerNorm stage owns token `tok` and the 8 features f0 .. f0+7.
TTT_DEV void ln_load(float (&x)[8], const bf16* p) {      // p 8-byte aligned
  const bf16x4 a = *reinterpret_cast<const bf16x4*>(p), b = *reinterpret_cast<const bf16x4*>(p + 4);
#pragma unroll
  for (int e = 0; e < 4; e++) { x[e] = (float)a[e]; x[4 + e] = (float)b[e]; }
}
TTT_DEV void ln_store_h(bf16* p, bf16x8 v) {
  *reinterpret_cast<bf16x4*>(p) = __builtin_shufflevector(v, v, 0, 1, 2, 3);
  *reinterpret_cast<bf16x4*>(p + 4) = __builtin_shufflevector(v, v, 4, 5, 6, 7);
}
TTT_DEV void ln_store(bf16* p, const float (&x)[8]) {
  bf16x4 a, b;
#pragma unroll
  for (int e = 0; e < 4; e++) { a[e] = (bf16)x[e]; b[e] = (bf16)x[4 + e]; }
  *reinterpret_cast<bf16x4*>(p) = a;
  *reinterpret_cast<bf16x4*>(p + 4) = b;
}
// 8 features of this lane's token to / from a [tok][F] bf16 tile in HBM (16 bytes per lane).
template <bool STREAM = false>
TTT_DEV void ln_store_g(gptr_t b, unsigned voff, unsigned soff, const float (&x)[8]) {
  bf16x8 v;
#pragma unroll
  for (int e = 0; e < 8; e++) v[e] = (bf16)x[e];
  if constexpr (STREAM) g_st_stream<bf16x8>(b, voff, soff, v);
  else g_st8h(b, voff, soff, v);
}
TTT_DEV void ln_cvt8(float (&x)[8], bf16x8 v) {
#pragma unroll
  for (int e = 0; e < 8; e++) x[e] = (float)v[e];
}
TTT_DEV void ln_load_f32(float (&x)[8], const float* p) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
  for (int e = 0; e < 4; e++) { x[e] = a[e]; x[4 + e] = b[e]; }
}
// Sum of the four pair sums of this lane's token / features.  `row` points at this token's row of the
// first pair's region; the regions of successive pairs are 2 regions apart.
TTT_DEV void ln_gather(float (&z)[8], const float* row) {
  f32x4 a = *reinterpret_cast<const f32x4*>(row), b = *reinterpret_cast<const f32x4*>(row + 4);
#pragma unroll
  for (int pp = 1; pp < 4; pp++) {
    a += *reinterpret_cast<const f32x4*>(row + pp * 2 * RGN);
    b += *reinterpret_cast<const f32x4*>(row + pp * 2 * RGN + 4);
  }
#pragma unroll
  for (int e = 0; e < 4; e++) { z[e] = a[e]; z[4 + e] = b[e]; }
}
TTT_DEV float sum8(const float (&x)[8]) {
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) s += x[e];
  return s;
}
TTT_DEV float dot8(const float (&x)[8], const float (&y)[8]) {
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) s = __builtin_fmaf(x[e], y[e], s);
  return s;
}
// z -> x_hat in place, returns 1/std; *std_out = std.
TTT_DEV float ln_normalize(float (&z)[8], float* std_out) {
  const float mu = oct_sum(sum8(z)) * (1.f / FD);
  float var = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) { z[e] -= mu; var = __builtin_fmaf(z[e], z[e], var); }
  const float v = oct_sum(var) * (1.f / FD) + LN_EPS;
  const float rstd = __builtin_amdgcn_rsqf(v);
#pragma unroll
  for (int e = 0; e < 8; e++) z[e] *= rstd;
  *std_out = v * rstd;  // sqrt(v)
  return rstd;
}
// acc[f0 + e] += sum over this wave's tokens of x[e]   (wave-private LDS vector).  The 8 tokens sit in the lanes
// that share lane % 8: lanes 8 apart inside a row of 16 (one rotation), then the four rows, two values per swap
// (row_pair_sum2, half_sum2): in the end row r of one register holds the total of x[r], of the other that of
// x[4 + r], and lanes 0..7 of every row add their two totals to the vector.
TTT_DEV void ln_token_sum_add(float* s_acc, const float (&x)[8], int lane, int f0) {
  float y[8];
#pragma unroll
  for (int e = 0; e < 8; e++)
    y[e] = x[e] + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x[e]), 0x128, 0xF, 0xF, false));  // row_ror:8
  const float lo = half_sum2(row_pair_sum2(y[0], y[1]), row_pair_sum2(y[2], y[3]));
  const float hi = half_sum2(row_pair_sum2(y[4], y[5]), row_pair_sum2(y[6], y[7]));
  if ((lane & 8) == 0) {
    float* d = s_acc + f0 + (lane >> 4);
    d[0] += lo;
    d[4] += hi;
  }
}

// 16-byte chunk staging of one [64][64] bf16 tile from HBM into an LDS tile with row stride LDX
// (rows are 8-byte aligned): thread tid moves chunk tid.
// The same into a tile of row pairs (XQ, XK, XV: the layout LDS-direct loads deliver).
TTT_DEV void lds_put16x(bf16* s_tile, int tid, u32x4 v) {
  uint2* d = reinterpret_cast<uint2*>(s_tile + xrow(tid >> 3) + (tid & 7) * 8);
  d[0] = make_uint2(v[0], v[1]);
  d[1] = make_uint2(v[2], v[3]);
}
TTT_DEV void lds_put16(bf16* s_tile, int tid, u32x4 v) {
  uint2* d = reinterpret_cast<uint2*>(s_tile + (tid >> 3) * LDX + (tid & 7) * 8);
  d[0] = make_uint2(v[0], v[1]);
  d[1] = make_uint2(v[2], v[3]);
}

// ---------------------------------------------------------------- just-in-time operand pieces
// Piece (free block fb, k-step s) of the chained operand of an accumulator tile.
template <int RB, int CB>
TTT_DEV bf16x8 piece_state(const AccT<RB, CB>& x, int fb, int s) { return pack8(x.b[s >> 1][fb], s & 1); }
// Chained operand of an accumulator tile written as an LDS tile stored [free index][contraction index].
template <int LD, int RB, int CB>
TTT_DEV void store_state_rows(bf16* tile, const AccT<RB, CB>& x, int c, int h) {
#pragma unroll
  for (int fb = 0; fb < CB; fb++)
#pragma unroll
    for (int s = 0; s < 2 * RB; s++) store_piece_rows<LD>(tile, fb, s, c, h, piece_state(x, fb, s));
}
// s_vec[row] += sum over the 64-long contraction of the 32-row operand whose pieces fa(s) yields; the
// sum is formed on the matrix cores, lanes with c == 0 fold it into the LDS vector.
template <class FA>
TTT_DEV void lds_rowsum_add_jit(float* s_vec, FA fa, bf16x8 ones, int c, int h) {
  f32x16 t;
#pragma unroll
  for (int i = 0; i < 16; i++) t[i] = 0.f;
#pragma unroll
  for (int s = 0; s < 4; s++) t = MFMA(fa(s), ones, t);
  if (c == 0) {
#pragma unroll
    for (int g = 0; g < 4; g++) {
      f32x4* q = reinterpret_cast<f32x4*>(s_vec + 8 * g + 4 * h);
      f32x4 v = *q;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] += t[4 * g + e];
      *q = v;
    }
  }
  // Other lanes of this wave read the vector next; without a fence the compiler may forward the
  // values each lane saw before the update.
  WAVE_SYNC();
}
// C-init of the rows of a Q-orientation tile from an LDS vector indexed by accumulator row (32 floats).
template <int CB>
TTT_DEV void acc_init_rows_lds(AccT<1, CB>& a, const float* s_vec, int h) {
#pragma unroll
  for (int g = 0; g < 4; g++) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(s_vec + 8 * g + 4 * h);
#pragma unroll
    for (int cb = 0; cb < CB; cb++)
#pragma unroll
      for (int e = 0; e < 4; e++) a.b[0][cb][4 * g + e] = v[e];
  }
}

TTT_DEV bf16x8 cvt8(const f32x4 lo, const f32x4 hi) {
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 4; e++) { o[e] = (bf16)lo[e]; o[4 + e] = (bf16)hi[e]; }
  return o;
}
// Piece (kappa order) straight from a row-major fp32 matrix in HBM: lane = row row0 + c, contraction =
// columns col0 + 16 s ...; row0, col0, s wave-uniform.
TTT_DEV bf16x8 piece_from_f32(gptr_t g, unsigned off, int ld, int row0, int col0, int s, int c, int h) {
  const unsigned vo = (c * ld + 4 * h) * 4, so = off + (row0 * ld + col0 + 16 * s) * 4;
  return cvt8(g_ld4f(g, vo, so), g_ld4f(g, vo, so + 32));
}

// Pair sum of a product z (rows F, column block 0 = the token block this wave keeps, column block 1 =
// the one it hands over): leaves the pair sum of the kept block in the PARTNER's region, stored
// [tok in block][F].  Contains two workgroup barriers; the caller makes sure that this wave's own
// reads of its region (the private tiles T1 / T2) are complete.
TTT_DEV void pair_sum(float* own, float* partner, const AccT<2, 2>& z, int c, int h) {
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const f32x16& x = z.b[rb][1];
      f32x4 v = {x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]};
      *reinterpret_cast<f32x4*>(own + c * LDR + 32 * rb + 8 * g + 4 * h) = v;
    }
  __syncthreads();
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      float* q = partner + c * LDR + 32 * rb + 8 * g + 4 * h;
      const f32x16& x = z.b[rb][0];
      f32x4 v = *reinterpret_cast<const f32x4*>(q);
      v[0] += x[4 * g]; v[1] += x[4 * g + 1]; v[2] += x[4 * g + 2]; v[3] += x[4 * g + 3];
      *reinterpret_cast<f32x4*>(q) = v;
    }
  __syncthreads();
}

// Three [64][64] bf16 tiles + the eta vector of one mini-batch in flight from HBM (per thread).
struct Staged3 {
  u32x4 a, b, c;
  bf16 eta;
};
// `mb` = mini-batch index inside this (batch, head); t16 = 16 * tid.
TTT_DEV void stage3_load(Staged3& s, gptr_t ga, gptr_t gb, gptr_t gc, gptr_t geta, int mb, int tid, unsigned t16) {
  s.a = g_ld16(ga, t16, mb * TILE_BYTES);
  s.b = g_ld16(gb, t16, mb * TILE_BYTES);
  s.c = g_ld16(gc, t16, mb * TILE_BYTES);
  s.eta = g_ldh(geta, 2 * (tid & (CS - 1)), mb * (CS * 2));   // in bounds for every thread; threads >= CS drop it
}
TTT_DEV void stage3_store(const Staged3& s, bf16* sa, bf16* sb, bf16* sc, bf16* s_eta, int tid) {
  lds_put16x(sa, tid, s.a);
  lds_put16x(sb, tid, s.b);
  lds_put16x(sc, tid, s.c);
  if (tid < CS) s_eta[tid] = s.eta;   // the replay keeps eta as bf16 in LDS
}

// Piece s of W2[shard] before mini-batch j of the group as an operand (lane = hid row, contraction =
// F): the image the replay stored after mini-batch j-1, or straight from the fp32 checkpoint.
// STREAM: the caller reads the image once (the grad_L_XK workgroup), so it need not stay in the L2.
template <bool STREAM = false>
TTT_DEV bf16x8 w2_before(gptr_t img, gptr_t ck, unsigned ck_off, int j, int s, int hid0, int c, int h, unsigned t16) {
  // the image offset is clamped so that the load stays inside the buffer even if it is hoisted above the branch
  bf16x8 r = image_load<STREAM>(img, (j > 0 ? j - 1 : 0) * IMG_BYTES, s, t16);
  if (j == 0) r = piece_from_f32(ck, ck_off, FD, hid0, 0, s, c, h);
  return r;
}
// Piece (row block rb, k-step s) of W1[:, shard]^T before mini-batch j (lane = F row, contraction = hid).
template <bool STREAM = false>
TTT_DEV bf16x8 w1_before(gptr_t img, gptr_t ck, unsigned ck_off, int j, int rb, int s, int hid0, int c, int h, unsigned t16) {
  bf16x8 r = image_load<STREAM>(img, (j > 0 ? j - 1 : 0) * IMG_BYTES, 2 * rb + s, t16);
  if (j == 0) r = piece_from_f32(ck, ck_off, HID, 32 * rb, hid0, s, c, h);
  return r;
}

constexpr int FIN_CHUNK = 8;   // mini-batches per hand-over to the grad_L_XK workgroup within the last group walked (a power of two)

// ------------------------------------------------------------------ two workgroups per (batch, head)
// The replay of a checkpoint group needs only the checkpoint, so it can run ahead of the reverse walk
// on another CU: one workgroup replays group after group into two alternating sets of the per-group
// tensors, the other walks each group backwards as soon as it is complete.  They signal through two
// counters in HBM (agent scope); both are resident at once because the launcher uses this mode only
// when the grid fits the CUs of the device.  A wait that sees no progress for SPIN_LIMIT ticks of the
// 100 MHz clock raises the status word and both workgroups leave, so every wave always exits.
// ROLE 0: replay and reverse walk of every group in one workgroup; 1: replays only - every n_replay-th group,
// starting with group number `turn` (counted from the end of the sequence); 2: the reverse walks only.
// IMG (with two replaying workgroups): the replay has time to spare and evaluates gelu, gelu', gelu'' of the
// rounded Z1 for the walk, which gets them as three images instead of the image of Z1.  Same values either way.
// FIN: grad_L_XK is a leaf of the walk - it needs the running gradients, but nothing needs it.  With a
// fourth workgroup the walk hands over the operands of its two products (gW1, G1, dZ1 as register images)
// and g_y, and that workgroup (bwd_finish_dxk) forms the products, their pair sum and the final sum.
template <int ROLE, bool IMG, bool FIN>
// k_hi, k_lo: the checkpoint groups k_hi, k_hi - 1, .. k_lo of the sequence (ROLE 0: a segment; the other roles take
// the whole sequence, K - 1 .. 0).
TTT_DEV void bwd_body(const BwdParams& p, unsigned char* smem, const int bh, const int turn, const int k_hi, const int k_lo) {
  static_assert(!(ROLE == 0 && (IMG || FIN)), "one workgroup per (batch, head) does everything itself");
  bf16* s_xq = reinterpret_cast<bf16*>(smem + SB_XQ);
  bf16* s_xk = reinterpret_cast<bf16*>(smem + SB_XK);
  bf16* s_gz2 = reinterpret_cast<bf16*>(smem + SB_GZ2);
  bf16* s_e2 = reinterpret_cast<bf16*>(smem + SB_E2);
  bf16* s_a = reinterpret_cast<bf16*>(smem + SB_A);
  float* s_P = reinterpret_cast<float*>(smem + SB_P);
  float* s_b1 = reinterpret_cast<float*>(smem + SB_B1);     // replay: b1
  float* s_b2 = reinterpret_cast<float*>(smem + SB_B2);     // replay: b2
  float* s_gb1 = reinterpret_cast<float*>(smem + SB_GB1);   // running gradient wrt b1
  float* s_gb2 = reinterpret_cast<float*>(smem + SB_GB2);   // running gradient wrt b2
  float* s_gam = reinterpret_cast<float*>(smem + SB_GAM);
  float* s_bet = reinterpret_cast<float*>(smem + SB_BET);
  float* s_eta = reinterpret_cast<float*>(smem + SB_ETA);
  bf16* s_etah = reinterpret_cast<bf16*>(smem + SB_ETA);     // the replay's view: eta as it sits in HBM
  float* s_deta = reinterpret_cast<float*>(smem + SB_DETA);
  float* s_red = reinterpret_cast<float*>(smem + SB_RED);

  const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5, c = lane & 31;
  const int v = __builtin_amdgcn_readfirstlane(tid >> 6);        // wave index, in a scalar register
  const int pp = v & 3, r = v >> 2;                              // pair, index inside the pair
  const int tb[2] = {r, 1 - r};                                  // token block held in column block 0 / 1 of a Q tile
  const int q8 = lane >> 3, tok = 8 * v + q8, f0 = 8 * (lane & 7);   // LayerNorm ownership (token block r)
  const int head = bh % p.NH;
  const int hid0 = BW_NS * v;
  float* s_own = s_P + (pp * 2 + r) * RGN;
  float* s_partner = s_P + (pp * 2 + (1 - r)) * RGN;
  // the pair sums of token block r sit in region 1-r of every pair
  const float* s_lnrow = s_P + (1 - r) * RGN + (tok & 31) * LDR + f0;
  bf16* const T0 = reinterpret_cast<bf16*>(smem + SB_BNC) + v * (64 * LDH);   // wave-private tiles: T0 = the bounce
  bf16* const T1 = reinterpret_cast<bf16*>(s_own);                            // tile; T1, T2 = the two halves of
  bf16* const T2 = T1 + 64 * LDH;                                             // this wave's pair-sum region
  float* s_b1w = s_b1 + hid0;
  float* s_gb1w = s_gb1 + hid0;
  const int cgs = p.cgs;
  // a segment that is not the first to run continues where the one before it stopped; one that is not the last leaves
  // what the next one needs instead of the norm gradients
  const bool seg_first = k_hi == p.K - 1, seg_last = k_lo == 0;

  if (tid < FD) {
    s_gam[tid] = p.ttt_norm_weight[head * FD + tid];
    s_bet[tid] = p.ttt_norm_bias[head * FD + tid];
    s_gb2[tid] = (seg_first ? p.grad_L_b2_last : p.grad_L_b2_init)[(size_t)bh * FD + tid];
  }
  if (tid < HID) s_gb1[tid] = (seg_first ? p.grad_L_b1_last : p.grad_L_b1_init)[(size_t)bh * HID + tid];
  // Norm-weight / norm-bias gradients accumulate per wave in LDS (summed over the wave's 8 tokens
  // with cross-lane adds in a fixed order); summed over the waves at the end.  The replay and the
  // reverse walk each contribute, and their sums are kept apart (so that the result does not depend on
  // whether one workgroup does both): with one workgroup the sum that is not being added to waits in HBM.
  float* s_dgw = s_red + (v * 2 + 0) * FD;
  float* s_dbw = s_red + (v * 2 + 1) * FD;
  if (lane < FD) { s_dgw[lane] = 0.f; s_dbw[lane] = 0.f; }
  const unsigned np_off = (v * 2 * FD + lane) * 4;   // this lane's two words of the wave's accumulators: +0, +FD*4
  float* s_gy = reinterpret_cast<float*>(smem + SB_XQ) + tok * FD + f0;   // this lane's part of the g_y park
  bf16x8 ones;
#pragma unroll
  for (int j = 0; j < 8; j++) ones[j] = (bf16)1.0f;

  // Buffers: base = this (batch, head)'s part of each tensor; offsets inside stay below 2 GiB (checked
  // by the launcher).  Per-lane offsets: t16 = chunk / tile staging, vln = this LayerNorm lane's 8
  // features of its token in a [tok][F] bf16 tile, vtok = its token in a [tok] fp32 vector.
  // Element offsets of this (batch, head) inside each class of tensor.  A buffer descriptor is built
  // where it is used, from the kernel argument and one of these offsets; the offsets are made opaque
  // to the optimiser once per mini-batch (REFRESH_OFFSETS) so that the thirty descriptors are not all
  // hoisted out of the loops and kept in scalar registers at once.
  size_t ox = uni64((size_t)bh * p.NC * (CS * FD));     // [NC][64][64] inputs / outputs
  size_t oe = uni64((size_t)bh * p.NC * CS);            // [NC][64] eta, d eta
  size_t of = uni64((size_t)bh * cgs * (CS * FD));      // [cgs][64][64] scratch tiles
  size_t oh = uni64((size_t)bh * cgs * (CS * HID));     // [cgs][64][256] scratch tiles (register images)
  size_t ot = uni64((size_t)bh * cgs * CS);             // [cgs][64] scratch vectors
  size_t opk = uni64((size_t)bh * cgs * (FD * HID));    // W1_init_group / W2_init_group
  size_t ock = uni64((size_t)bh * p.K * (FD * HID));    // W1 / W2 checkpoints
  // The tensor pointers are read from the kernel-argument segment (scalar loads) where they are used,
  // through a pointer that is refreshed with the offsets, instead of all fifty living in scalar registers.
  typedef const __attribute__((address_space(4))) BwdParams* KernArgs;
  KernArgs ka = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
#define REFRESH_OFFSETS() asm volatile("" : "+s"(ka), "+s"(ox), "+s"(oe), "+s"(of), "+s"(oh), "+s"(ot), "+s"(opk), "+s"(ock))
  // per-group tensors: the caller's (set 0) or, in two-workgroup mode, the alternate set
#define GRP(name) (set ? ka->alt_##name[set - 1] : ka->name)
#define bXQ gbuf(ka->XQ + ox)
#define bXK gbuf(ka->XK + ox)
#define bXV gbuf(ka->XV + ox)
#define bGO gbuf(ka->grad_L_XQW + ox)
#define bETA gbuf(ka->last_eta + oe)
#define bZ1 gbuf(GRP(Z1_group) + oh)
#define bGZ1B gbuf(GRP(Z1_bar_group) + oh)              // operand image of gZ1_bar = dL/dZ1_bar
#define bX2B gbuf(GRP(X2_bar_group) + oh)               // operand image of X2_bar
#define bGZB gbuf(GRP(grad_x_hat_fused_group) + of)     // gZ2_bar = dL/dZ2_bar, [tok][F] tiles
#define bIMG1 gbuf(GRP(X2_group) + oh)
#define bIMG2 gbuf(GRP(grad_l_wrt_Z1_group) + oh)
#define bXHF gbuf(GRP(x_hat_fused_group) + of)
#define bGOF gbuf(GRP(grad_output_fused_group) + of)
#define bGZ2 gbuf(GRP(grad_l_wrt_Z2_group) + of)
#define bSDF gbuf(GRP(std_fused_group) + ot)
  // While a group is replayed the running gradients are parked in W*_init_group; during the reverse
  // walk the same two 64 KiB slots park what must survive the LayerNorm stage (three 32 KiB images).
  // Several workgroups per (batch, head): slot j of W1_init_group (of the set) carries gelu'(Z1) and gelu''(Z1)
  // of mini-batch j as two register images, and Z1_group carries gelu(Z1) instead of Z1.
#define bDD gbuf(GRP(W1_init_group) + opk)
  // the walk's fourth parked image (-eta * (XK gW1 + gb1) * gelu'(Z1)): second half of slot 0 of W1_init_group,
  // or - where that tensor carries GELU images - the workspace
#define bPUH (ROLE == 0 ? gbuf(ka->W1_init_group + opk) + IMG_BYTES : gbuf(ka->walk_park + (size_t)bh * (CS * HID)))
#define bPW1 gbuf(ka->W1_init_group + opk)
#define bPW2 gbuf(ka->W2_init_group + opk)
  constexpr unsigned PARK_D1 = 0, PARK_T2 = IMG_BYTES, PARK_G1 = 0;   // d1 in bPW1 (one workgroup only); g1, t2 in bPW2
#define bCW1 gbuf(ka->W1_ck + ock)
#define bCW2 gbuf(ka->W2_ck + ock)
#define bDXQ gbuf(ka->grad_L_XQ + ox)
#define bDXK gbuf(ka->grad_L_XK + ox)
#define bDXV gbuf(ka->grad_L_XV + ox)
#define bDETA gbuf(ka->grad_L_last_eta + oe)
// what an accumulating output held before: the tile itself, or zeros when the outputs are overwritten
#define OLD_VALUE(buf, off) (ka->overwrite ? gbuf(zero_tile) : (buf)), vln, (ka->overwrite ? 0u : (off))
  const unsigned t16 = 16 * tid, vln = (tok * FD + f0) * 2, vtok = 4 * tok;
  // Everything derived from the lane index is cheap to recompute and expensive to keep: a value
  // computed once before the loops is held in a register (or spilled and reloaded) for the whole
  // kernel.  LANE_VARS re-derives the lot from a lane index the optimiser cannot see through, so
  // each stage that opens with it gets fresh, short-lived copies.
  int lane_v = lane;
#define LANE_VARS                                                                                       \
  asm volatile("" : "+v"(lane_v));                                                                      \
  const int lane = lane_v, h = lane >> 5, c = lane & 31, tid = (v << 6) | lane;                         \
  const int q8 = lane >> 3, tok = 8 * v + q8, f0 = 8 * (lane & 7);                                      \
  const unsigned t16 = 16 * tid, vln = (tok * FD + f0) * 2, vtok = 4 * tok;                             \
  const float* s_lnrow = s_P + (1 - r) * RGN + (tok & 31) * LDR + f0;                            \
  float* s_gy = reinterpret_cast<float*>(smem + SB_XQ) + tok * FD + f0;                                 \
  (void)h; (void)c; (void)tid; (void)q8; (void)t16; (void)vln; (void)vtok; (void)s_lnrow; (void)s_gy

  // running gradients wrt the state after the last mini-batch
  AccT<2, 1> gW1s;
  AccT<1, 2> gW2s;
  if constexpr (ROLE != 1) {
    acc_load_rows(gW1s, gbuf((seg_first ? p.grad_L_W1_last : p.grad_L_W1_init) + (size_t)bh * FD * HID), 0, HID, 0, hid0, c, h);
    acc_load_rows(gW2s, gbuf((seg_first ? p.grad_L_W2_last : p.grad_L_W2_init) + (size_t)bh * HID * FD), 0, FD, hid0, 0, c, h);
  }
  int* const w_sync = p.sync + (size_t)bh * BWD_SYNC_STRIDE;   // + 0, + 8: groups replayed by workgroup 0 / 1
  int* const w_walked = w_sync + 16;
  int* const w_finished = w_sync + 24;
  const int n_replay = ROLE == 0 ? 1 : p.n_replay, n_sets = 2 * n_replay;
  int* const w_status = p.status;
  int* const s_flag = reinterpret_cast<int*>(smem + SB_FLAG);

  // The replay's share of the norm gradients is kept as two sums, of the even and of the odd groups (counted
  // from the end of the sequence), whoever replays them; the walk's share is a third.  A workgroup that adds
  // to more than one of them keeps the others parked in HBM, 4 KiB each: one workgroup per (batch, head) in
  // two slots of the caller's x_hat_ln_group, a single replaying workgroup in the workspace.
  const gptr_t gPark = ROLE == 0 ? gbuf(p.x_hat_ln_group + (size_t)bh * cgs * (CS * FD))
                                 : gbuf(p.norm_park + (size_t)bh * (BW_NWAVE * 2 * FD));
  constexpr unsigned PARK_BYTES = BW_NWAVE * 2 * FD * 4;
  if (ROLE == 0 ? seg_first : (ROLE == 1 && n_replay == 1)) {   // parked sums start at zero
    g_stf(gPark, np_off, 0, 0.f);
    g_stf(gPark, np_off, FD * 4, 0.f);
    if constexpr (ROLE == 0) {
      g_stf(gPark, np_off, PARK_BYTES, 0.f);
      g_stf(gPark, np_off, PARK_BYTES + FD * 4, 0.f);
    }
  }
  if (ROLE == 0 && !seg_first) {   // the walk's sum as the segment before this one left it (a third slot of the park)
    s_dgw[lane] = g_ldf(gPark, np_off, 2 * PARK_BYTES);
    s_dbw[lane] = g_ldf(gPark, np_off, 2 * PARK_BYTES + FD * 4);
  }
  // Exchanges the wave's LDS accumulators with a parked sum (every lane owns two words of both).
  auto norm_swap = [&](unsigned slot) {
    WAVE_SYNC();
    const float a0 = s_dgw[lane], a1 = s_dbw[lane];
    const float p0 = g_ldf(gPark, np_off, slot * PARK_BYTES), p1 = g_ldf(gPark, np_off, slot * PARK_BYTES + FD * 4);
    s_dgw[lane] = p0;
    s_dbw[lane] = p1;
    g_stf(gPark, np_off, slot * PARK_BYTES, a0);
    g_stf(gPark, np_off, slot * PARK_BYTES + FD * 4, a1);
    WAVE_SYNC();
  };

  TTT_STAGES_BEGIN();
  for (int k = k_hi; k >= k_lo; k--) {
    const int n_mb = min(cgs, p.NC - k * cgs);
    const int done = p.K - 1 - k;                    // number of this group, counted from the end of the sequence
    if (ROLE == 1 && done % n_replay != turn) continue;
    const int set = ROLE == 0 ? 0 : done % n_sets;
    int* const w_replayed = w_sync + 8 * (done % n_replay);
    REFRESH_OFFSETS();
    const size_t slot = (size_t)bh * p.K + k;
    const unsigned ckW = static_cast<unsigned>(k) * (FD * HID * 4u);   // byte offset of this group's checkpoint in bCW1 / bCW2
    // ================================================================= replay
    if constexpr (ROLE != 2) {
      if constexpr (ROLE == 1) {   // the set is free once the reverse walk is done with the group that used it last
        if (done >= n_sets && !wait_at_least(w_walked, done - n_sets + 1, w_status, s_flag, p.wait_limit)) return;
        if constexpr (FIN) {   // ... and so is the workgroup that reads the before-state images for grad_L_XK
          if (done >= n_sets && !wait_at_least(w_finished, done - n_sets + 1, w_status, s_flag, p.wait_limit)) return;
        }
        // a single replaying workgroup adds to the sum of this group's parity: the groups alternate, so from
        // the second group on the live sum and the parked one change places
        if (n_replay == 1 && done > 0) norm_swap(0);
      }
      // park the running gradients while the forward state needs the registers
      if constexpr (ROLE == 0) {
        acc_store_rows(gW1s, bPW1, 0, HID, 0, hid0, c, h);
        acc_store_rows(gW2s, bPW2, 0, FD, hid0, 0, c, h);
        norm_swap(done & 1);   // the walk's sum out, the replay's sum of this parity in
      }
      AccT<2, 1> W1s;
      AccT<1, 2> W2s;
      acc_load_rows(W1s, bCW1, ckW, HID, 0, hid0, c, h);
      acc_load_rows(W2s, bCW2, ckW, FD, hid0, 0, c, h);
      __syncthreads();  // previous group's readers of the bias vectors are done
      if (tid < HID) s_b1[tid] = p.b1_ck[slot * HID + tid];
      if (tid < FD) s_b2[tid] = p.b2_ck[slot * FD + tid];

      {
        Staged3 st;
        stage3_load(st, bXQ, bXK, bXV, bETA, k * cgs, tid, t16);
        stage3_store(st, s_xq, s_xk, s_e2, s_etah, tid);
      }
      TTT_STAGE(BS_GROUP);
      for (int j = 0; j < n_mb; j++) {
        const int mb = k * cgs + j;
        REFRESH_OFFSETS();
        LANE_VARS;
        __syncthreads();   // the staged inputs (and, for j = 0, the biases) are visible
        TTT_STAGE(BS_R_TOP);

        // Z1^T = W1s^T XK^T + b1  (rows hid, lane = tok); X2 rows [tok][hid] -> T0; gelu'(Z1) (fp32) and the
        // low-order term of X2 stay in registers.  The products that carry the state to the next mini-batch
        // take their fp32 operands in two bf16 terms (see split8).
        float d1f[2][16];
        bf16x8 x2lo[2][2];
        {
          LANE_VARS;
          AccT<1, 2> x2;
          acc_init_rows_lds(x2, s_b1w, h);
#pragma unroll
          for (int s = 0; s < 4; s++) {
            bf16x8 wh, wl, xk[2];
            split8(W1s.b[s >> 1][0], s & 1, wh, wl);
#pragma unroll
            for (int i = 0; i < 2; i++) xk[i] = xpiece_rows(s_xk, tb[i], s, c, h);
#pragma unroll
            for (int i = 0; i < 2; i++) {
              x2.b[0][i] = MFMA(wl, xk[i], x2.b[0][i]);
              x2.b[0][i] = MFMA(wh, xk[i], x2.b[0][i]);
            }
          }
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
              const bf16x8 zr = pack8(x2.b[0][i], t);
              if constexpr (!IMG) {
                image_store<ROLE != 0>(bZ1, j * IMG_BYTES, 2 * tb[i] + t, t16, zr);
              } else {
                // The walk needs gelu, gelu' and gelu'' of the ROUNDED Z1 (what it would compute from the image
                // of Z1); a replaying workgroup has the time to do that for it.
                bf16x8 gv, av, bv;
#pragma unroll
                for (int jj = 0; jj < 8; jj++) {
                  float g, a, b;
                  gelu_fdd((float)zr[jj], g, a, b);
                  gv[jj] = (bf16)g;
                  av[jj] = (bf16)a;
                  bv[jj] = (bf16)b;
                }
                image_store<ROLE != 0>(bZ1, j * IMG_BYTES, 2 * tb[i] + t, t16, gv);
                image_store<ROLE != 0>(bDD, j * (2 * IMG_BYTES), 2 * tb[i] + t, t16, av);
                image_store<ROLE != 0>(bDD, j * (2 * IMG_BYTES) + IMG_BYTES, 2 * tb[i] + t, t16, bv);
              }
              bf16x8 xv;
#pragma unroll
              for (int jj = 0; jj < 8; jj++) {
                float g, d;
                gelu_fd(x2.b[0][i][8 * t + jj], g, d);
                const bf16 gh = (bf16)g;
                xv[jj] = gh;
                x2lo[i][t][jj] = (bf16)(g - (float)gh);
                d1f[i][8 * t + jj] = d;
                // pinned: left to itself the compiler finishes gelu' only where it is used, two stages on, and keeps
                // three values per element alive until then instead of one (a dozen of them in scratch memory)
                asm volatile("" : "+v"(d1f[i][8 * t + jj]));
              }
              store_piece_rows<LDH>(T0, tb[i], t, c, h, xv);
            }
        }
        TTT_STAGE(BS_R_F1_GELU);
        WAVE_SYNC();
        {
          LANE_VARS;
          AccT<2, 2> z2;
          acc_zero(z2);
#pragma unroll
          for (int s = 0; s < 2; s++) {                      // W2s: lane = F, contraction = hid, two terms; X2: lane = tok
            bf16x8 wh[2], wl[2], xb[2];
#pragma unroll
            for (int rb = 0; rb < 2; rb++) split8(W2s.b[0][rb], s, wh[rb], wl[rb]);
#pragma unroll
            for (int i = 0; i < 2; i++) xb[i] = piece_rows<LDH>(T0, tb[i], s, c, h);
#pragma unroll
            for (int rb = 0; rb < 2; rb++)
#pragma unroll
              for (int i = 0; i < 2; i++) {
                z2.b[rb][i] = MFMA(wl[rb], xb[i], z2.b[rb][i]);
                z2.b[rb][i] = MFMA(wh[rb], xb[i], z2.b[rb][i]);
              }
          }
          pair_sum(s_own, s_partner, z2, c, h);
        }
        TTT_STAGE(BS_R_F2_PAIRSUM);
        // fused LayerNorm + reconstruction-loss gradient; saves for the reverse walk
        {
          LANE_VARS;
          float z[8], gam[8];
          {
            float b2v[8];
            ln_gather(z, s_lnrow);
            ln_load_f32(b2v, s_b2 + f0);
#pragma unroll
            for (int e = 0; e < 8; e++) z[e] += b2v[e];
          }
          ln_load_f32(gam, s_gam + f0);
          float sd;
          const float rstd = ln_normalize(z, &sd);
          float go[8], gx[8];
          {
            float kv[8], vv[8], bet[8];
            ln_load(kv, s_xk + xrow(tok) + f0);
            ln_load(vv, s_e2 + xrow(tok) + f0);
            ln_load_f32(bet, s_bet + f0);
#pragma unroll
            for (int e = 0; e < 8; e++) {
              go[e] = __builtin_fmaf(gam[e], z[e], bet[e]) - (vv[e] - kv[e]);
              gx[e] = go[e] * gam[e];
            }
          }
          ln_store_g<ROLE != 0>(bXHF, vln, j * TILE_BYTES, z);
          ln_store_g<ROLE != 0>(bGOF, vln, j * TILE_BYTES, go);
          const float s1 = oct_sum(sum8(gx)), s2 = oct_sum(dot8(gx, z));
          const float sc = rstd * (1.f / FD), neg_eta = -bf2f(s_etah[tok]);
#pragma unroll
          for (int e = 0; e < 8; e++) gx[e] = (FD * gx[e] - s1 - z[e] * s2) * sc;   // dl/dZ2
          ln_store_g<ROLE != 0>(bGZ2, vln, j * TILE_BYTES, gx);
#pragma unroll
          for (int e = 0; e < 8; e++) gx[e] *= neg_eta;                             // G2, in two terms (the second in
          ln_token_sum_store(s_deta + v * CS, gx, lane, f0);   // b2's step: this wave's share (s_deta is the walk's otherwise)
          {                                                                          // the tile gZ2_bar takes later)
            bf16x8 gh, gl;
            split8(gx, gh, gl);
            ln_store_h(s_gz2 + tok * LDX + f0, gh);
            ln_store_h(s_a + tok * LDX + f0, gl);
          }
          if ((lane & 7) == 0) g_stf(bSDF, vtok, j * (CS * 4), sd);
        }
        __syncthreads();
        if (v == 0) {   // b2 += sum over the tokens of G2: the eight waves' fp32 shares in a fixed order (next read: the output LayerNorm)
          LANE_VARS;
          float b = s_b2[lane];
#pragma unroll
          for (int u = 0; u < BW_NWAVE; u++) b += s_deta[u * CS + lane];
          s_b2[lane] = b;
        }
        TTT_STAGE(BS_R_LN);
        // G1 = (W2 G2^T) * gelu'(Z1)  (rows hid, lane = tok) -> T1 rows [tok][hid]; weight step
        {
          LANE_VARS;
          AccT<1, 2> g1;
          acc_zero(g1);
          // W2[shard, :] with F contracted (lane = hid): the two terms of W2s, written as rows [F][hid] into T1 / T2
          // and read back transposed
#pragma unroll
          for (int fb = 0; fb < 2; fb++)
#pragma unroll
            for (int s = 0; s < 2; s++) {
              bf16x8 ph, pl;
              split8(W2s.b[0][fb], s, ph, pl);
              store_piece_rows<LDH>(T1, fb, s, c, h, ph);
              store_piece_rows<LDH>(T2, fb, s, c, h, pl);
            }
          WAVE_SYNC();
#pragma unroll
          for (int s = 0; s < 4; s++) {                      // W2: lane = hid, contraction = F; G2: lane = tok; two terms each
            const bf16x8 wh = piece_tr<LDH>(T1, 0, s, lane), wl = piece_tr<LDH>(T2, 0, s, lane);
            bf16x8 gh[2], gl[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
              gh[i] = piece_rows<LDX>(s_gz2, tb[i], s, c, h);
              gl[i] = piece_rows<LDX>(s_a, tb[i], s, c, h);
            }
#pragma unroll
            for (int i = 0; i < 2; i++) {
              g1.b[0][i] = MFMA(wh, gl[i], g1.b[0][i]);
              g1.b[0][i] = MFMA(wl, gh[i], g1.b[0][i]);
              g1.b[0][i] = MFMA(wh, gh[i], g1.b[0][i]);
            }
          }
          WAVE_SYNC();   // W2's terms are read before G1 takes their place
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
              bf16x8 gv, gvl;
#pragma unroll
              for (int jj = 0; jj < 8; jj++) {
                const float g = g1.b[0][i][8 * t + jj] * d1f[i][8 * t + jj];
                const bf16 gh = (bf16)g;
                gv[jj] = gh;
                gvl[jj] = (bf16)(g - (float)gh);
              }
              store_piece_rows<LDH>(T1, tb[i], t, c, h, gv);      // G1 rows [tok][hid], two terms
              store_piece_rows<LDH>(T2, tb[i], t, c, h, gvl);
            }
        }
        WAVE_SYNC();
        TTT_STAGE(BS_R_F3);
        {   // weight step
          LANE_VARS;
#pragma unroll
          for (int s = 0; s < 4; s++) {                        // W1[:, shard] += XK^T G1
            bf16x8 xk[2];
#pragma unroll
            for (int fb = 0; fb < 2; fb++) xk[fb] = xpiece_tr(s_xk, fb, s, lane);               // XK^T: lane = F
            const bf16x8 gh = piece_tr<LDH>(T1, 0, s, lane), gl = piece_tr<LDH>(T2, 0, s, lane);   // G1: lane = hid
#pragma unroll
            for (int fb = 0; fb < 2; fb++) {
              W1s.b[fb][0] = MFMA(xk[fb], gl, W1s.b[fb][0]);
              W1s.b[fb][0] = MFMA(xk[fb], gh, W1s.b[fb][0]);
            }
          }
          lds_rowsum_add_jit(s_b1w, [&](int s) { return piece_tr<LDH>(T2, 0, s, lane); }, ones, c, h);
          lds_rowsum_add_jit(s_b1w, [&](int s) { return piece_tr<LDH>(T1, 0, s, lane); }, ones, c, h);
          // the low-order term of X2 takes G1's place in T1 (rows [tok][hid])
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int t = 0; t < 2; t++) store_piece_rows<LDH>(T1, tb[i], t, c, h, x2lo[i][t]);
          WAVE_SYNC();
#pragma unroll
          for (int s = 0; s < 4; s++) {                        // W2[shard, :] += X2^T G2
            const bf16x8 xh = piece_tr<LDH>(T0, 0, s, lane), xl = piece_tr<LDH>(T1, 0, s, lane);   // X2^T: lane = hid
            bf16x8 gh[2], gl[2];
#pragma unroll
            for (int fb = 0; fb < 2; fb++) {
              gh[fb] = piece_tr<LDX>(s_gz2, fb, s, lane);                                        // G2: lane = F
              gl[fb] = piece_tr<LDX>(s_a, fb, s, lane);
            }
#pragma unroll
            for (int fb = 0; fb < 2; fb++) {
              W2s.b[0][fb] = MFMA(xl, gh[fb], W2s.b[0][fb]);
              W2s.b[0][fb] = MFMA(xh, gl[fb], W2s.b[0][fb]);
              W2s.b[0][fb] = MFMA(xh, gh[fb], W2s.b[0][fb]);
            }
          }
          WAVE_SYNC();   // this wave's readers of T1 / T2 are done
        }
        TTT_STAGE(BS_R_WSTEP);
        // operand images of the state after this step, for the reverse walk; the image of W2 (lane = hid,
        // contraction = F) also serves the output branch below
        bf16x8 w2a[4];
        {
          LANE_VARS;
          // bIMG2: W2, lane = hid, contraction = F;  bIMG1: W1^T, lane = F, contraction = hid
          store_state_rows<LDF>(T2, W1s, c, h);                                 // rows [hid][F]
          store_state_rows<LDH>(T1, W2s, c, h);                                 // rows [F][hid]
          WAVE_SYNC();
#pragma unroll
          for (int s = 0; s < 4; s++) {
            w2a[s] = piece_tr<LDH>(T1, 0, s, lane);
            image_store<ROLE != 0>(bIMG2, j * IMG_BYTES, s, t16, w2a[s]);
          }
#pragma unroll
          for (int fb = 0; fb < 2; fb++)
#pragma unroll
            for (int s = 0; s < 2; s++) image_store<ROLE != 0>(bIMG1, j * IMG_BYTES, 2 * fb + s, t16, piece_tr<LDF>(T2, fb, s, lane));
        }
        TTT_STAGE(BS_R_IMAGES);
        // post-update forward on XQ; X2_bar rows [tok][hid] -> T0, gelu'(Z1_bar) packed
        bf16x8 d1b[2][2];
        bf16x8 gO_n;   // LayerNorm lanes: the upstream gradient of their 8 features, asked for a stage ahead
        {
          LANE_VARS;
          AccT<1, 2> z1b;
          acc_init_rows_lds(z1b, s_b1w, h);
          // W1 after the step in two terms: its rounding pattern persists over many mini-batches, so the error it
          // leaves in Z1_bar - and through it in every gradient the output branch feeds - does not average out
#pragma unroll
          for (int s = 0; s < 4; s++) {
            bf16x8 wh, wl, xq[2];
            split8(W1s.b[s >> 1][0], s & 1, wh, wl);
#pragma unroll
            for (int i = 0; i < 2; i++) xq[i] = xpiece_rows(s_xq, tb[i], s, c, h);
#pragma unroll
            for (int i = 0; i < 2; i++) {
              z1b.b[0][i] = MFMA(wl, xq[i], z1b.b[0][i]);
              z1b.b[0][i] = MFMA(wh, xq[i], z1b.b[0][i]);
            }
          }
          bf16x8 x2bQ[2][2];
          WAVE_SYNC();   // the weight step's readers of T0 are done
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
#pragma unroll
              for (int jj = 0; jj < 8; jj++) {
                float g, d;
                gelu_fd(z1b.b[0][i][8 * t + jj], g, d);
                x2bQ[i][t][jj] = (bf16)g;
                d1b[i][t][jj] = (bf16)d;
              }
              asm volatile("" : "+v"(d1b[i][t]));   // finished here, not where it is used (see gelu'(Z1) above)
              store_piece_rows<LDH>(T0, tb[i], t, c, h, x2bQ[i][t]);
            }
          AccT<2, 2> z2;
          acc_zero(z2);
          mma_jit<2>(z2, [&](int rb, int s) { return piece_state(W2s, rb, s); },
                     [&](int i, int s) { return x2bQ[i][s]; });
          WAVE_SYNC();   // this wave's readers of T1 / T2 are done
          {
            LANE_VARS;
            gO_n = g_ld_stream<bf16x8>(bGO, vln, mb * TILE_BYTES);   // under way during the pair sum
          }
          pair_sum(s_own, s_partner, z2, c, h);
        }
        TTT_STAGE(BS_R_OUT_FORWARD);
        // ---- the output branch, backwards: it needs the state after this step, which is in registers
        //      right now, and nothing of the running gradients.  Output LayerNorm forward and backward:
        float gO[8];
        bf16x8 dxq_old;
        {
          LANE_VARS;
          // The upstream gradient is taken out of its load registers before the loads below are issued: they are
          // issued under a condition, so a wait for an older load placed after them has to be a wait for all of them.
          ln_cvt8(gO, gO_n);
#pragma unroll
          for (int e = 0; e < 8; e++) asm volatile("" : "+v"(gO[e]));
          // Every reader of this mini-batch's XQ / XK / XV / eta is past the barriers of the pair sum: the next
          // mini-batch's leave HBM now - straight to LDS, no registers involved - and have the rest of this
          // mini-batch to arrive.
          if (j + 1 < n_mb) {
            tile_to_lds<CPOL_NT>(bXQ, (mb + 1) * TILE_BYTES, smem + SB_XQ, v, lane);
            tile_to_lds<CPOL_NT>(bXK, (mb + 1) * TILE_BYTES, smem + SB_XK, v, lane);
            tile_to_lds<CPOL_NT>(bXV, (mb + 1) * TILE_BYTES, smem + SB_E2, v, lane);
            eta_to_lds(bETA, (mb + 1) * (CS * 2), smem + SB_ETA, v, lane);
          }
          float z[8], gx[8], gam[8];
          {
            float b2v[8];
            ln_gather(z, s_lnrow);
            ln_load_f32(b2v, s_b2 + f0);
#pragma unroll
            for (int e = 0; e < 8; e++) z[e] += b2v[e];
          }
          float sd;
          ln_normalize(z, &sd);   // z = x_hat
          ln_load_f32(gam, s_gam + f0);
#pragma unroll
          for (int e = 0; e < 8; e++) gx[e] = gO[e] * z[e];
          ln_token_sum_add(s_dbw, gO, lane, f0);
          ln_token_sum_add(s_dgw, gx, lane, f0);
#pragma unroll
          for (int e = 0; e < 8; e++) gx[e] = gO[e] * gam[e];
          const float s1 = oct_sum(sum8(gx)), s2 = oct_sum(dot8(gx, z));
          const float sc = 1.f / (FD * sd);
#pragma unroll
          for (int e = 0; e < 8; e++) gx[e] = (FD * gx[e] - s1 - z[e] * s2) * sc;
          ln_store(s_a + tok * LDX + f0, gx);            // gZ2_bar
          ln_store_g<ROLE != 0>(bGZB, vln, j * TILE_BYTES, gx);
        }
        __syncthreads();
        TTT_STAGE(BS_R_OUT_LN);
        {
          LANE_VARS;
          bf16x8 w1a[2][2];   // W1 after the step (lane = F, contraction = hid): the image stored above, fetched ahead of its use
#pragma unroll
          for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int s = 0; s < 2; s++) w1a[rb][s] = chunk_load(bIMG1, j * IMG_BYTES, 2 * rb + s, t16);
          {
            LANE_VARS;
            AccT<1, 2> gz1b;   // (gZ2_bar W2^T) * gelu'(Z1_bar): rows hid, lane = tok
            acc_zero(gz1b);
            // W2 after the step in two terms here as well (see W1 above): the low-order term goes through T2 like the
            // high-order one went through T1 for the image
#pragma unroll
            for (int fb = 0; fb < 2; fb++)
#pragma unroll
              for (int s = 0; s < 2; s++) {
                bf16x8 ph, pl;
                split8(W2s.b[0][fb], s, ph, pl);
                store_piece_rows<LDH>(T2, fb, s, c, h, pl);
              }
            WAVE_SYNC();
#pragma unroll
            for (int s = 0; s < 4; s++) {
              const bf16x8 wl = piece_tr<LDH>(T2, 0, s, lane);
              bf16x8 gb[2];
#pragma unroll
              for (int i = 0; i < 2; i++) gb[i] = piece_rows<LDX>(s_a, tb[i], s, c, h);
#pragma unroll
              for (int i = 0; i < 2; i++) {
                gz1b.b[0][i] = MFMA(wl, gb[i], gz1b.b[0][i]);
                gz1b.b[0][i] = MFMA(w2a[s], gb[i], gz1b.b[0][i]);
              }
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
              for (int t = 0; t < 2; t++) {
                bf16x8 gzb;
#pragma unroll
                for (int jj = 0; jj < 8; jj++) gzb[jj] = (bf16)(gz1b.b[0][i][8 * t + jj] * (float)d1b[i][t][jj]);
                store_piece_rows<LDH>(T1, tb[i], t, c, h, gzb);    // gZ1_bar rows [tok][hid]
              }
          }
          WAVE_SYNC();
          AccT<2, 2> dq;
          acc_zero(dq);
          mma_jit<2>(dq, [&](int rb, int s) { return w1a[rb][s]; },                                // W1 after: lane = F
                     [&](int i, int s) { return piece_rows<LDH>(T1, tb[i], s, c, h); });                   // gZ1_bar: lane = tok
          // what the reverse walk adds to the running gradients, as ready-made operands (lane = hid, contraction = tok)
#pragma unroll
          for (int s = 0; s < 4; s++) {
            image_store<ROLE != 0>(bX2B, j * IMG_BYTES, s, t16, piece_tr<LDH>(T0, 0, s, lane));
            image_store<ROLE != 0>(bGZ1B, j * IMG_BYTES, s, t16, piece_tr<LDH>(T1, 0, s, lane));
          }
          WAVE_SYNC();   // every reader of T1 / T2 is done before the pair sum takes their place
          {
            LANE_VARS;
            dxq_old = g_ld_stream<bf16x8>(OLD_VALUE(bDXQ, mb * TILE_BYTES));   // under way during the pair sum
          }
          pair_sum(s_own, s_partner, dq, c, h);
        }
        {
          LANE_VARS;
          float z[8];
          ln_gather(z, s_lnrow);
#pragma unroll
          for (int e = 0; e < 8; e++) dxq_old[e] = (bf16)((float)dxq_old[e] + (z[e] + gO[e]));
          g_st_stream<bf16x8>(bDXQ, vln, mb * TILE_BYTES, dxq_old);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the next mini-batch's inputs are in LDS before the barrier at the loop's top
        TTT_STAGE(BS_R_OUT_BACKWARD);
      }
      if constexpr (ROLE == 1) {
        if (done + n_replay >= p.K) {   // this workgroup's last group: hand its norm-gradient sums to the walk
          WAVE_SYNC();
          float* np = p.norm_partial + ((size_t)bh * 2 + (done & 1)) * (BW_NWAVE * 2 * FD) + v * 2 * FD;
          np[lane] = s_dgw[lane];
          np[FD + lane] = s_dbw[lane];
          if (n_replay == 1) {   // and the sum of the other parity (zero if there was one group only)
            float* no = p.norm_partial + ((size_t)bh * 2 + (1 - (done & 1))) * (BW_NWAVE * 2 * FD) + v * 2 * FD;
            no[lane] = g_ldf(gPark, np_off, 0);
            no[FD + lane] = g_ldf(gPark, np_off, FD * 4);
          }
        }
      }
      // running gradients back into registers
      if constexpr (ROLE == 0) {
        acc_load_rows(gW1s, bPW1, 0, HID, 0, hid0, c, h);
        acc_load_rows(gW2s, bPW2, 0, FD, hid0, 0, c, h);
        norm_swap(done & 1);
      }
      if constexpr (ROLE == 1) publish(w_replayed, done / n_replay + 1);
      TTT_STAGE(BS_PUBLISH);
    }

    // ================================================================= reverse walk
    // Operands are fetched from HBM right where they are consumed: with two waves per SIMD the other
    // wave covers the latency, while holding requests in registers across stages costs more in spills
    // than it gains (measured).
    if constexpr (ROLE == 2) {
      if (!wait_at_least(w_replayed, done / n_replay + 1, w_status, s_flag, p.wait_limit)) return;
      if constexpr (FIN) {   // the hand-over set of this group's parity is free once the group before last is finished
        if (done >= 2 && !wait_at_least(w_finished, done - 1, w_status, s_flag, p.wait_limit)) return;
      }
    }
    // hand-over buffers of this group for the grad_L_XK workgroup (set = parity of the group)
    const size_t ofin = uni64(((size_t)bh * 2 + (done & 1)) * cgs);
#define bFDZ gbuf(ka->fin_dz + ofin * (CS * HID))
#define bFGY gbuf(ka->fin_gy + ofin * (2 * CS * FD))
    TTT_STAGE(BS_GROUP);
    // What a mini-batch of the walk needs first - its two input tiles, the two tiles the replay left for it (gZ2 and
    // gZ2_bar) and eta - is requested during the updates of the mini-batch walked before it and held in registers
    // until the barrier that opens the mini-batch (the very first one of a group is requested here).  The walk is the
    // longest chain of the backward pass; with the lines in the L2 already, a request a stage earlier hides the rest.
    u32x4 n_xq, n_xk, n_gz, n_gzb;
    bf16 n_eta, n_etai[2];
    // What the output branch adds to the running gradients: the replay has taken that branch backwards already
    // and left gZ2_bar (a tile) and X2_bar^T, gZ1_bar^T as operand images.
    bf16x8 x2b[4], g1b[4];   // lane = hid, contraction = tok
#define WALK_FETCH(jn)                                                                                   \
    {                                                                                                    \
      LANE_VARS;                                                                                         \
      constexpr bool ST = ROLE != 0;   /* tiles another workgroup left here are read once */             \
      const int jf = __builtin_amdgcn_readfirstlane(jn), mbf = k * cgs + jf;                             \
      const unsigned xo = mbf * TILE_BYTES, so = jf * TILE_BYTES;                                        \
      n_etai[0] = g_ldh(bETA, 2 * c, mbf * (CS * 2) + 64 * tb[0]);                                       \
      n_etai[1] = g_ldh(bETA, 2 * c, mbf * (CS * 2) + 64 * tb[1]);                                       \
      n_xq = ST ? g_ld_stream<u32x4>(bXQ, t16, xo) : g_ld16(bXQ, t16, xo);                               \
      n_xk = ST ? g_ld_stream<u32x4>(bXK, t16, xo) : g_ld16(bXK, t16, xo);                               \
      n_gz = ST ? g_ld_stream<u32x4>(bGZ2, t16, so) : g_ld16(bGZ2, t16, so);                             \
      n_gzb = ST ? g_ld_stream<u32x4>(bGZB, t16, so) : g_ld16(bGZB, t16, so);                            \
      n_eta = g_ldh(bETA, 2 * (tid & (CS - 1)), mbf * (CS * 2));                                         \
    }
    if constexpr (ROLE != 1) WALK_FETCH(n_mb - 1);
    if constexpr (ROLE != 1)
    for (int j = n_mb - 1; j >= 0; j--) {
      const int mb = k * cgs + j;
      REFRESH_OFFSETS();
      LANE_VARS;
      const unsigned xo = mb * TILE_BYTES;       // this mini-batch in the input / output tensors
      const unsigned so = j * TILE_BYTES;        // its slot in the [cgs][64][64] scratch tensors
      const unsigned ho = j * IMG_BYTES;         // its slot in the [cgs][64][256] scratch tensors
      // eta of the token this lane holds in column block i of a Q-orientation tile
      const float eta_i[2] = {bf2f(n_etai[0]), bf2f(n_etai[1])};
      {
        LANE_VARS;
        // the two operand images of the next stage are asked for here: on their way across both barriers
#pragma unroll
        for (int s = 0; s < 4; s++) {
          x2b[s] = image_load<ROLE != 0>(bX2B, ho, s, t16);
          g1b[s] = image_load<ROLE != 0>(bGZ1B, ho, s, t16);
        }
        __syncthreads();   // the previous mini-batch's readers of these tiles are done
        lds_put16x(s_xq, tid, n_xq);
        lds_put16x(s_xk, tid, n_xk);
        lds_put16(s_gz2, tid, n_gz);
        lds_put16(s_a, tid, n_gzb);
        if (tid < CS) s_eta[tid] = bf2f(n_eta);
      }
      __syncthreads();

      TTT_STAGE(BS_W_TOP);
      bf16x8 w2bf[4];   // W2 before this step (lane = hid, contraction = F): fetched now, needed by the next stage
      bf16x8 gq[2][2], aq[2][2], bq[2][2];
      {
        LANE_VARS;
#pragma unroll
        for (int s = 0; s < 4; s++) w2bf[s] = w2_before(bIMG2, bCW2, ckW, j, s, hid0, c, h, t16);
        if constexpr (IMG) {   // the three GELU images of the next stage, under way during this one
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
              gq[i][t] = image_load<true>(bZ1, ho, 2 * tb[i] + t, t16);
              aq[i][t] = chunk_load(bDD, j * (2 * IMG_BYTES), 2 * tb[i] + t, t16);   // read again two stages on
              bq[i][t] = image_load<true>(bDD, j * (2 * IMG_BYTES) + IMG_BYTES, 2 * tb[i] + t, t16);
            }
        } else {               // the image of Z1 (gq takes it), from which the next stage evaluates the three
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int t = 0; t < 2; t++) gq[i][t] = image_load<ROLE != 0>(bZ1, ho, 2 * tb[i] + t, t16);
        }
        mma_jit<4>(gW2s, [&](int, int s) { return x2b[s]; },                                   // X2_bar^T: lane = hid
                   [&](int fb, int s) { return piece_tr<LDX>(s_a, fb, s, lane); });            // gZ2_bar: lane = F
        if (v < 2) lds_rowsum_add_jit(s_gb2 + 32 * v, [&](int s) { return piece_tr<LDX>(s_a, v, s, lane); }, ones, c, h);
        mma_jit<4>(gW1s, [&](int fb, int s) { return xpiece_tr(s_xq, fb, s, lane); },         // XQ^T: lane = F
                   [&](int, int s) { return g1b[s]; });                                        // gZ1_bar: lane = hid
        lds_rowsum_add_jit(s_gb1w, [&](int s) { return g1b[s]; }, ones, c, h);
      }
      // gb2 holds its value after the first update

      TTT_STAGE(BS_W_BAR_TERMS);
      // How far the walk is, for the workgroup that fetches ahead of it: said here, a quarter into the mini-batch, so
      // that the next mini-batch's lines reach the L2 in time for the first of them (requested during this
      // mini-batch's updates) and stay there no longer than needed (said at the top: c4 backward +0.3 ms; two stages
      // further on: +1.9 ms, the lines come too late).
      if constexpr (ROLE == 2 && FIN) {
        if (threadIdx.x == 0) __hip_atomic_store(w_sync + 20, p.NC - mb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      // ---- the weight step, backwards (uses the state BEFORE this mini-batch).
      //      Parked across the LayerNorm stage: X2 in T0; packed d1 = gelu'(Z1), g1 = -eta * dl/dZ1 and
      //      t2 = -eta * (gZ2 W2^T) * (XK gW1 + gb1) * gelu''(Z1).
      bf16x8 dxv_old;            // LayerNorm lanes: the two outputs the stage accumulates into
      bf16 deta_old;
      bf16x8 xhf_n, gof_n;       // and the saved x_hat, grad_output, std of the fused LayerNorm
      float sdf_n;
      {
        LANE_VARS;
        // T1 = W2 before the step, rows [hid][F]; T2 = gW1, rows [hid][F]
#pragma unroll
        for (int s = 0; s < 4; s++)
          store_piece_rows<LDF>(T1, 0, s, c, h, w2bf[s]);
        store_state_rows<LDF>(T2, gW1s, c, h);
        WAVE_SYNC();
        AccT<2, 2> pz;
        acc_zero(pz);
        float de[2] = {0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 2; i++) {
          AccT<1, 1> R, S;   // R = gZ2 W2^T, S = XK gW1 + gb1   (rows hid, lane = tok)
          acc_zero(R);
          acc_init_rows_lds(S, s_gb1w, h);
          mma_jit<4>(R, [&](int, int s) { return piece_rows<LDF>(T1, 0, s, c, h); },
                     [&](int, int s) { return piece_rows<LDX>(s_gz2, tb[i], s, c, h); });
          mma_jit<4>(S, [&](int, int s) { return piece_rows<LDF>(T2, 0, s, c, h); },
                     [&](int, int s) { return xpiece_rows(s_xk, tb[i], s, c, h); });
          bf16x8 x2c[2], uc[2];
          // gelu(Z1), gelu'(Z1), gelu''(Z1), each rounded to bf16: computed here from the image of Z1, or
          // fetched as three images that a replaying workgroup computed the same way
          bf16x8 ac[2], bc[2];
          if constexpr (!IMG) {
            const bf16x8 zc[2] = {gq[i][0], gq[i][1]};
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
              for (int jj = 0; jj < 8; jj++) {
                float g, a, b;
                gelu_fdd((float)zc[t][jj], g, a, b);
                x2c[t][jj] = (bf16)g;
                ac[t][jj] = (bf16)a;
                bc[t][jj] = (bf16)b;
              }
          } else {
#pragma unroll
            for (int t = 0; t < 2; t++) {
              x2c[t] = gq[i][t];
              ac[t] = aq[i][t];
              bc[t] = bq[i][t];
            }
          }
#pragma unroll
          for (int t = 0; t < 2; t++) {
            bf16x8 t2c, g1c, uhc;
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
              const float a = (float)ac[t][jj], b = (float)bc[t][jj];
              const float r0 = R.b[0][0][8 * t + jj], sv = S.b[0][0][8 * t + jj];
              const float gz1 = r0 * a;                                   // dl/dZ1
              de[i] = __builtin_fmaf(gz1, sv, de[i]);
              uc[t][jj] = (bf16)(sv * a);
              uhc[jj] = (bf16)(-eta_i[i] * sv * a);
              g1c[jj] = (bf16)(-eta_i[i] * gz1);
              t2c[jj] = (bf16)(-eta_i[i] * r0 * sv * b);
            }
            chunk_store(bPUH, 0, 2 * tb[i] + t, t16, uhc);
            // nothing stays in registers across the LayerNorm stage: g1 and t2 (and, without the images,
            // gelu'(Z1)) go to their parks at once (L2-resident, rewritten every mini-batch)
            if constexpr (!IMG) chunk_store(bPW1, PARK_D1, 2 * tb[i] + t, t16, ac[t]);
            chunk_store(bPW2, PARK_T2, 2 * tb[i] + t, t16, t2c);
            // only grad_L_XK needs G1: its workgroup, where there is one, forms G1 itself
            if constexpr (!FIN) chunk_store(bPW2, PARK_G1, 2 * tb[i] + t, t16, g1c);
            store_piece_rows<LDH>(T0, tb[i], t, c, h, x2c[t]);             // X2 rows [tok][hid]
          }
          // pz[:, i] = gW2^T X2^T ; dEta partial ; + W2^T u^T
#pragma unroll
          for (int t = 0; t < 2; t++)
#pragma unroll
            for (int rb = 0; rb < 2; rb++) pz.b[rb][i] = MFMA(piece_state(gW2s, rb, t), x2c[t], pz.b[rb][i]);
#pragma unroll
          for (int s = 0; s < 4; s++) {
            const bf16x8 gzv = piece_rows<LDX>(s_gz2, tb[i], s, c, h);
#pragma unroll
            for (int jj = 0; jj < 8; jj++) de[i] = __builtin_fmaf((float)gzv[jj], pz.b[s >> 1][i][8 * (s & 1) + jj], de[i]);
          }
#pragma unroll
          for (int t = 0; t < 2; t++)
#pragma unroll
            for (int rb = 0; rb < 2; rb++) pz.b[rb][i] = MFMA(piece_tr<LDF>(T1, rb, t, lane), uc[t], pz.b[rb][i]);
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
          const float a = half_sum(de[i]);
          if (h == 0) s_deta[v * CS + 32 * tb[i] + c] = a;
        }
        WAVE_SYNC();   // this wave's readers of T1 / T2 are done
        TTT_STAGE(BS_W_STEP_BACK);
        {   // what the LayerNorm stage reads from HBM is under way during the pair sum
          LANE_VARS;
          if constexpr (!FIN) dxv_old = g_ld_stream<bf16x8>(OLD_VALUE(bDXV, xo));
          deta_old = g_ldh(ka->overwrite ? gbuf(zero_tile) : bDETA, 2 * tok, ka->overwrite ? 0u : mb * (CS * 2));
          xhf_n = ROLE != 0 ? g_ld_stream<bf16x8>(bXHF, vln, so) : g_ld8h(bXHF, vln, so);
          gof_n = ROLE != 0 ? g_ld_stream<bf16x8>(bGOF, vln, so) : g_ld8h(bGOF, vln, so);
          sdf_n = g_ldf(bSDF, vtok, j * (CS * 4));
        }
        pair_sum(s_own, s_partner, pz, c, h);
      }
      TTT_STAGE(BS_W_PAIRSUM);
      // all pair sums of ggZ2 and the dEta partial sums are in LDS

      // ---- second-order pass through the fused LayerNorm loss (LayerNorm lanes)
      {
        LANE_VARS;
        float gy[8];
        float gg[8], xh[8], go[8], gz[8], gam[8], gb[8];
        const bf16x8 xhf = xhf_n, gof = gof_n;
        const float sdf = sdf_n;
        ln_gather(gg, s_lnrow);
        ln_load_f32(gb, s_gb2 + f0);
        const float neg_eta = -s_eta[tok];
#pragma unroll
        for (int e = 0; e < 8; e++) gg[e] = (gg[e] + gb[e]) * neg_eta;   // grad wrt dl/dZ2
        ln_cvt8(xh, xhf);
        ln_cvt8(go, gof);
        ln_load(gz, s_gz2 + tok * LDX + f0);
        ln_load_f32(gam, s_gam + f0);
        const float rsd = 1.f / sdf;
        // dEta: -(sum_F gZ2*(X2 gW2 + gb2) + sum_H gZ1*(XK gW1 + gb1))
        {
          LANE_VARS;
          float tot = oct_sum(dot8(gz, gb));
#pragma unroll
          for (int u = 0; u < BW_NWAVE; u++) tot += s_deta[u * CS + tok];
          if ((lane & 7) == 0) g_sth(bDETA, 2 * tok, mb * (CS * 2), (bf16)((float)deta_old - tot));
        }
        const float s0 = oct_sum(sum8(gg)), a = oct_sum(dot8(gg, xh));
        float bb = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) bb = __builtin_fmaf(go[e] * gam[e], xh[e], bb);
        bb = oct_sum(bb);
        float gx[8], dg[8];
        const float inv = rsd * (1.f / FD);
        float sg = 0.f, sx = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float ggx = (gg[e] - (s0 + xh[e] * a) * (1.f / FD)) * rsd;
          gy[e] = gam[e] * ggx;
          dg[e] = go[e] * ggx + gy[e] * xh[e];
          gx[e] = gy[e] * gam[e] - (go[e] * gam[e] * a + gg[e] * bb) * inv;
          sg += (-gx[e] * xh[e] - gg[e] * gz[e]) * rsd;
          sx += gx[e];
        }
        sg = oct_sum(sg);
        sx = oct_sum(sx);
        if constexpr (!FIN) {   // with a grad_L_XK workgroup these token sums and grad_L_XV are formed there, from g_y and dg
          ln_token_sum_add(s_dgw, dg, lane, f0);
          ln_token_sum_add(s_dbw, gy, lane, f0);
        }
#pragma unroll
        for (int e = 0; e < 8; e++) {
          gx[e] = gx[e] * rsd + (sg * xh[e] - sx * rsd) * (1.f / FD);   // dZ2
          if constexpr (!FIN) dxv_old[e] = (bf16)((float)dxv_old[e] - gy[e]);   // dXV accumulates -g_y
        }
        // g_y is needed again for dXK: park it (the XQ / E2 tiles are dead by now), or hand it over
        {
          LANE_VARS;
          f32x4 lo = {gy[0], gy[1], gy[2], gy[3]}, hi = {gy[4], gy[5], gy[6], gy[7]};
          if constexpr (FIN) {
            g_st_stream<f32x4>(bFGY, 2 * vln, 4 * so, lo);
            g_st_stream<f32x4>(bFGY, 2 * vln + 16, 4 * so, hi);
            f32x4 dlo = {dg[0], dg[1], dg[2], dg[3]}, dhi = {dg[4], dg[5], dg[6], dg[7]};
            g_st_stream<f32x4>(bFGY, 2 * vln, 4 * so + 2 * TILE_BYTES, dlo);
            g_st_stream<f32x4>(bFGY, 2 * vln + 16, 4 * so + 2 * TILE_BYTES, dhi);
          } else {
            *reinterpret_cast<f32x4*>(s_gy) = lo;
            *reinterpret_cast<f32x4*>(s_gy + 4) = hi;
          }
        }
        ln_store(s_a + tok * LDX + f0, gx);
        if constexpr (!FIN) g_st_stream<bf16x8>(bDXV, vln, xo, dxv_old);
      }
      TTT_STAGE(BS_W_LN);
      __syncthreads();  // dZ2 tile complete; regions (T1 / T2) free again
      TTT_STAGE(BS_W_LN_BARRIER);

      // ---- inner MLP, backwards (uses the state BEFORE this mini-batch)
      bf16x8 dxk_old;
      {
        LANE_VARS;
        bf16x8 w2b[4];   // W2 before the step: lane = hid, contraction = F
#pragma unroll
        for (int s = 0; s < 4; s++) w2b[s] = w2_before<ROLE == 2>(bIMG2, bCW2, ckW, j, s, hid0, c, h, t16);   // second and last read
        // T2 = gW1 rows [hid][F] (for gW1 G1^T), T1 = gW2 rows [F][hid] (transposed read gives lane = hid)
        if constexpr (!FIN) store_state_rows<LDF>(T2, gW1s, c, h);
        store_state_rows<LDH>(T1, gW2s, c, h);
        WAVE_SYNC();
        AccT<2, 2> dk;
        acc_zero(dk);
        bf16x8 dzp[2][2], uhp[2][2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
          AccT<1, 1> dx2;
          acc_zero(dx2);
          mma_jit<4>(dx2, [&](int, int s) { return piece_tr<LDH>(T1, 0, s, lane); },           // gW2: lane = hid, contraction = F
                     [&](int, int s) { return piece_rows<LDX>(s_gz2, tb[i], s, c, h); });      // P2 = gZ2 gW2^T
#pragma unroll
          for (int e = 0; e < 16; e++) dx2.b[0][0][e] *= -eta_i[i];
          mma_jit<4>(dx2, [&](int, int s) { return w2b[s]; },                                  // + dZ2 W2^T
                     [&](int, int s) { return piece_rows<LDX>(s_a, tb[i], s, c, h); });
          // dk[:, i] = gW1 G1^T  (gW1: lane = F, contraction = hid)
          bf16x8 g1c[2];
          if constexpr (!FIN) {
            g1c[0] = chunk_load(bPW2, PARK_G1, 2 * tb[i], t16);
            g1c[1] = chunk_load(bPW2, PARK_G1, 2 * tb[i] + 1, t16);
          }
          bf16x8 d1c[2];
          if constexpr (!IMG) {
            d1c[0] = chunk_load(bPW1, PARK_D1, 2 * tb[i], t16);
            d1c[1] = chunk_load(bPW1, PARK_D1, 2 * tb[i] + 1, t16);
          } else {
            d1c[0] = image_load<true>(bDD, j * (2 * IMG_BYTES), 2 * tb[i], t16);   // its last reader on this XCD
            d1c[1] = image_load<true>(bDD, j * (2 * IMG_BYTES), 2 * tb[i] + 1, t16);
          }
          const bf16x8 t2c[2] = {chunk_load(bPW2, PARK_T2, 2 * tb[i], t16), chunk_load(bPW2, PARK_T2, 2 * tb[i] + 1, t16)};
          if constexpr (!FIN) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
              for (int rb = 0; rb < 2; rb++) dk.b[rb][i] = MFMA(piece_tr<LDF>(T2, rb, t, lane), g1c[t], dk.b[rb][i]);
          }
          // dZ1 = dX2*gelu' + t2 ;  -eta * S * gelu'   (kept as pieces until T1 / T2 may be overwritten)
#pragma unroll
          for (int t = 0; t < 2; t++)
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
              const float d1v = (float)d1c[t][jj];
              dzp[i][t][jj] = (bf16)__builtin_fmaf(dx2.b[0][0][8 * t + jj], d1v, (float)t2c[t][jj]);
            }
          uhp[i][0] = chunk_load(bPUH, 0, 2 * tb[i], t16);       // -eta * S * gelu', formed with S two stages back
          uhp[i][1] = chunk_load(bPUH, 0, 2 * tb[i] + 1, t16);
        }
        bf16x8 w1bf[2][2];   // W1^T before the step (lane = F, contraction = hid), for the product after the next fence
        if constexpr (!FIN) {
#pragma unroll
          for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int s = 0; s < 2; s++) w1bf[rb][s] = w1_before(bIMG1, bCW1, ckW, j, rb, s, hid0, c, h, t16);
        } else {   // dZ1 leaves for the other workgroup (which keeps its own copy of gW1: it sees every term added to it)
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int t = 0; t < 2; t++) image_store<true>(bFDZ, ho, 2 * tb[i] + t, t16, dzp[i][t]);
        }
        TTT_STAGE(BS_W_MLP_BACK);
        WAVE_SYNC();   // S, P2 and gW1 G1^T have consumed T2 / T1
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int t = 0; t < 2; t++) {
            store_piece_rows<LDH>(T1, tb[i], t, c, h, dzp[i][t]);   // dZ1 rows [tok][hid]
            store_piece_rows<LDH>(T2, tb[i], t, c, h, uhp[i][t]);   // -eta u rows [tok][hid]
          }
        WAVE_SYNC();
        WALK_FETCH(j > 0 ? j - 1 : 0);   // the next mini-batch's tiles (the last step of a group asks for its own again)
        if constexpr (!FIN)
          mma_jit<2>(dk, [&](int rb, int s) { return w1bf[rb][s]; },                           // + W1 dZ1^T, W1 before the step
                     [&](int i, int s) { return dzp[i][s]; });
        mma_jit<4>(gW2s, [&](int, int s) { return piece_tr<LDH>(T2, 0, s, lane); },            // (-eta u)^T: lane = hid
                   [&](int fb, int s) { return piece_tr<LDX>(s_gz2, fb, s, lane); });          // gZ2: lane = F
        mma_jit<4>(gW2s, [&](int, int s) { return piece_tr<LDH>(T0, 0, s, lane); },            // X2^T: lane = hid
                   [&](int fb, int s) { return piece_tr<LDX>(s_a, fb, s, lane); });            // dZ2: lane = F
        if (v < 2) lds_rowsum_add_jit(s_gb2 + 32 * v, [&](int s) { return piece_tr<LDX>(s_a, v, s, lane); }, ones, c, h);
        mma_jit<4>(gW1s, [&](int fb, int s) { return xpiece_tr(s_xk, fb, s, lane); },         // XK^T: lane = F
                   [&](int, int s) { return piece_tr<LDH>(T1, 0, s, lane); });                 // dZ1: lane = hid
        lds_rowsum_add_jit(s_gb1w, [&](int s) { return piece_tr<LDH>(T1, 0, s, lane); }, ones, c, h);
        TTT_STAGE(BS_W_UPDATES);
        WAVE_SYNC();   // this wave's readers of T1 / T2 are done
        if constexpr (!FIN) {
          {
            LANE_VARS;
            dxk_old = g_ld_stream<bf16x8>(OLD_VALUE(bDXK, xo));   // under way during the pair sum
          }
          pair_sum(s_own, s_partner, dk, c, h);
        }
      }
      // pair sums of dXK complete
      if constexpr (!FIN) {
        LANE_VARS;
        float z[8], gyv[8];
        ln_gather(z, s_lnrow);
        ln_load_f32(gyv, s_gy);
#pragma unroll
        for (int e = 0; e < 8; e++) dxk_old[e] = (bf16)((float)dxk_old[e] + (z[e] + gyv[e]));
        g_st_stream<bf16x8>(bDXK, vln, xo, dxk_old);
      }
      TTT_STAGE(BS_W_DXK);
      if constexpr (ROLE == 2 && FIN) {
        // The last group to be walked is handed to the grad_L_XK workgroup in chunks, so that that workgroup follows
        // FIN_CHUNK mini-batches behind instead of ending a whole group after the walk.
        if (k == 0 && (j & (FIN_CHUNK - 1)) == 0) {
          publish(w_sync + 12, n_mb - j);
          TTT_STAGE(BS_PUBLISH);
        }
      }
    }
    if constexpr (ROLE == 2) publish(w_walked, done + 1);
    TTT_STAGE(BS_PUBLISH);
#undef bFDZ
#undef bFGY
#undef WALK_FETCH
  }
  TTT_STAGES_END(p.stage_clocks == nullptr ? nullptr : p.stage_clocks + ((size_t)bh * 4 + (ROLE == 1 ? turn : 2)) * (BW_NWAVE * STAGE_SLOTS));
  if constexpr (ROLE == 1) return;

  // ---- outputs that are written once
  acc_store_rows(gW1s, gbuf(p.grad_L_W1_init + (size_t)bh * FD * HID), 0, HID, 0, hid0, c, h);
  acc_store_rows(gW2s, gbuf(p.grad_L_W2_init + (size_t)bh * HID * FD), 0, FD, hid0, 0, c, h);
  __syncthreads();
  if (tid < HID) p.grad_L_b1_init[(size_t)bh * HID + tid] = s_gb1[tid];
  if (tid < FD) p.grad_L_b2_init[(size_t)bh * FD + tid] = s_gb2[tid];
  // norm-weight / norm-bias gradients: sum the per-wave LDS accumulators
  // The replay's two sums: parked in HBM by this workgroup, or handed over by the replaying workgroups, whose
  // last counts this workgroup has acquired (a second replaying workgroup has nothing to hand over if there is
  // one group only).
  if constexpr (FIN) return;   // with a grad_L_XK workgroup the walk holds no share of these sums: they are written there
  if (ROLE == 0 && !seg_last) {   // the next segment goes on with the walk's sum (the replay's two are parked already)
    g_stf(gPark, np_off, 2 * PARK_BYTES, s_dgw[lane]);
    g_stf(gPark, np_off, 2 * PARK_BYTES + FD * 4, s_dbw[lane]);
    return;
  }
  if (tid < 2 * FD) {
    const int which = tid / FD, f = tid % FD;
    const float* rp = ROLE == 0 ? reinterpret_cast<const float*>(p.x_hat_ln_group + (size_t)bh * cgs * (CS * FD))
                                : p.norm_partial + (size_t)bh * 2 * (BW_NWAVE * 2 * FD);
    const bool have_odd = ROLE == 0 || p.K > 1 || n_replay == 1;
    float s = 0.f, sr0 = 0.f, sr1 = 0.f;
#pragma unroll
    for (int u = 0; u < BW_NWAVE; u++) {
      s += s_red[(u * 2 + which) * FD + f];
      sr0 += rp[(u * 2 + which) * FD + f];
      if (have_odd) sr1 += rp[BW_NWAVE * 2 * FD + (u * 2 + which) * FD + f];
    }
    (which == 0 ? p.grad_L_ttt_norm_weight : p.grad_L_ttt_norm_bias)[(size_t)bh * FD + f] = (sr0 + sr1) + s;
  }
}
#undef REFRESH_OFFSETS
#undef LANE_VARS
#undef GRP
#undef bXQ
#undef bXK
#undef bXV
#undef bGO
#undef bETA
#undef bZ1
#undef bGZ1B
#undef bX2B
#undef bGZB
#undef bIMG1
#undef bIMG2
#undef bXHF
#undef bGOF
#undef bGZ2
#undef bSDF
#undef bDD
#undef bPUH
#undef bPW1
#undef bPW2
#undef bCW1
#undef bCW2
#undef bDXQ
#undef bDXK
#undef bDXV
#undef bDETA

__global__ __launch_bounds__(BW_THREADS) void ttt_mlp_bwd_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  int bh = p.bh0 + blockIdx.x, k_hi = p.K - 1, k_lo = 0;
  if (p.seg_groups > 0) {
    const int pairs = p.B * p.NH, job = p.job0 + blockIdx.x, seg = job / pairs;
    bh = job - seg * pairs;
    k_hi = p.K - 1 - seg * p.seg_groups;
    k_lo = k_hi - p.seg_groups + 1 > 0 ? k_hi - p.seg_groups + 1 : 0;
  }
  bwd_body<0, false, false>(p, smem, bh, 0, k_hi, k_lo);
}

// grad_L_XK on a workgroup of its own: for every mini-batch of every group, as soon as the walk is done with the
// group, dk = gW1 G1^T + W1 dZ1^T (W1 before the step: from the replay's image, or the checkpoint), its sum over
// the hidden dimension, + g_y, accumulated into grad_L_XK.  Same wave / lane roles and the same order of every
// sum as in the walk, so the result is the same to the bit.
TTT_DEV void bwd_finish_dxk(const BwdParams& p, unsigned char* smem, const int bh) {
  float* s_P = reinterpret_cast<float*>(smem + SB_P);
  const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5, c = lane & 31;
  const int v = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pp = v & 3, r = v >> 2;
  const int tb[2] = {r, 1 - r};
  const int q8 = lane >> 3, tok = 8 * v + q8, f0 = 8 * (lane & 7);
  const int hid0 = BW_NS * v;
  float* s_own = s_P + (pp * 2 + r) * RGN;
  float* s_partner = s_P + (pp * 2 + (1 - r)) * RGN;
  const float* s_lnrow = s_P + (1 - r) * RGN + (tok & 31) * LDR + f0;
  const int cgs = p.cgs, n_sets = 2 * p.n_replay;
  const unsigned t16 = 16 * tid, vln = (tok * FD + f0) * 2;
  int* const w_sync = p.sync + (size_t)bh * BWD_SYNC_STRIDE;
  int* const w_walked = w_sync + 16;
  int* const w_finished = w_sync + 24;
  int* const s_flag = reinterpret_cast<int*>(smem + SB_FLAG);
  const gptr_t gDXK = gbuf(p.grad_L_XK + uni64((size_t)bh * p.NC * (CS * FD)));
  const gptr_t gDXV = gbuf(p.grad_L_XV + uni64((size_t)bh * p.NC * (CS * FD)));
  const gptr_t gCW1 = gbuf(p.W1_ck + uni64((size_t)bh * p.K * (FD * HID)));
  const gptr_t gXQ = gbuf(p.XQ + uni64((size_t)bh * p.NC * (CS * FD))), gXK = gbuf(p.XK + uni64((size_t)bh * p.NC * (CS * FD)));
  bf16* const s_xq = reinterpret_cast<bf16*>(smem + SB_XQ);
  bf16* const s_xk = reinterpret_cast<bf16*>(smem + SB_XK);
  bf16* const s_gz2 = reinterpret_cast<bf16*>(smem + SB_GZ2);
  const gptr_t gETA = gbuf(p.last_eta + uni64((size_t)bh * p.NC * CS));
  const gptr_t gCW2 = gbuf(p.W2_ck + uni64((size_t)bh * p.K * (FD * HID)));
  bf16* const T1 = reinterpret_cast<bf16*>(s_own);   // wave-private tiles in this wave's pair-sum region, as in the walk
  bf16* const T2 = T1 + 64 * LDH;
  // This workgroup keeps its own copy of the running gradient wrt W1: both terms the walk adds to it per
  // mini-batch (XQ^T gZ1_bar and XK^T dZ1) are formed from data that reaches this workgroup anyway, in the walk's order.
  AccT<2, 1> gW1s;
  acc_load_rows(gW1s, gbuf(p.grad_L_W1_last + (size_t)bh * FD * HID), 0, HID, 0, hid0, c, h);
  // the walk's share of the norm-weight / norm-bias gradients: per wave, summed in the walk's order
  float* s_red = reinterpret_cast<float*>(smem + SB_RED);
  float* s_dgw = s_red + (v * 2 + 0) * FD;
  float* s_dbw = s_red + (v * 2 + 1) * FD;
  if (lane < FD) { s_dgw[lane] = 0.f; s_dbw[lane] = 0.f; }
  TTT_STAGES_BEGIN();
  for (int k = p.K - 1; k >= 0; k--) {
    const int n_mb = min(cgs, p.NC - k * cgs);
    const int done = p.K - 1 - k, set = done % n_sets;
    // the walk hands over whole groups, except the last one it walks (k = 0): that one in chunks of FIN_CHUNK mini-batches
    if (k > 0 && !wait_at_least(w_walked, done + 1, p.status, s_flag, p.wait_limit)) return;
    TTT_STAGE(BS_X_GROUP);
    const size_t ofin = uni64(((size_t)bh * 2 + (done & 1)) * cgs);
    const size_t o_img = uni64((size_t)bh * cgs * (CS * HID)), o_tile = uni64((size_t)bh * cgs * (CS * FD));
    const gptr_t gIMG2 = gbuf((set ? p.alt_grad_l_wrt_Z1_group[set - 1] : p.grad_l_wrt_Z1_group) + o_img);   // W2 after each step
    const gptr_t gGZ2 = gbuf((set ? p.alt_grad_l_wrt_Z2_group[set - 1] : p.grad_l_wrt_Z2_group) + o_tile);   // dl/dZ2
    const gptr_t gDD = gbuf((set ? p.alt_W1_init_group[set - 1] : p.W1_init_group) + uni64((size_t)bh * cgs * (FD * HID)));   // gelu'(Z1) images
    const gptr_t gGZ1B = gbuf((set ? p.alt_Z1_bar_group[set - 1] : p.Z1_bar_group) + uni64((size_t)bh * cgs * (CS * HID)));
    const gptr_t gDZ = gbuf(p.fin_dz + ofin * (CS * HID)), gGY = gbuf(p.fin_gy + ofin * (2 * CS * FD));
    const gptr_t gIMG1 = gbuf((set ? p.alt_X2_group[set - 1] : p.X2_group) + uni64((size_t)bh * cgs * (CS * HID)));
    const unsigned ckW = static_cast<unsigned>(k) * (FD * HID * 4u);
    for (int j = n_mb - 1; j >= 0; j--) {
      if (k == 0 && (j == n_mb - 1 || (j & (FIN_CHUNK - 1)) == FIN_CHUNK - 1)) {
        if (!wait_at_least(w_sync + 12, n_mb - (j & ~(FIN_CHUNK - 1)), p.status, s_flag, p.wait_limit)) return;
        TTT_STAGE(BS_X_GROUP);
      }
      const unsigned xo = (k * cgs + j) * TILE_BYTES, so = j * TILE_BYTES, ho = j * IMG_BYTES;
      const bf16x8 dxk_ld = g_ld_stream<bf16x8>(p.overwrite ? gbuf(zero_tile) : gDXK, vln, p.overwrite ? 0u : xo);
      const bf16x8 dxv_ld = g_ld_stream<bf16x8>(p.overwrite ? gbuf(zero_tile) : gDXV, vln, p.overwrite ? 0u : xo);
      const f32x4 gy_lo = g_ld_stream<f32x4>(gGY, 2 * vln, 4 * so), gy_hi = g_ld_stream<f32x4>(gGY, 2 * vln + 16, 4 * so);
      const f32x4 dg_lo = g_ld_stream<f32x4>(gGY, 2 * vln, 4 * so + 2 * TILE_BYTES);
      const f32x4 dg_hi = g_ld_stream<f32x4>(gGY, 2 * vln + 16, 4 * so + 2 * TILE_BYTES);
      // everything this workgroup reads it reads once: streaming loads, so that the lines fetched ahead of the walk
      // on the same XCD stay in the L2 (c4 backward -0.35 ms)
      const u32x4 xq = g_ld_stream<u32x4>(gXQ, t16, xo), xk = g_ld_stream<u32x4>(gXK, t16, xo);
      const u32x4 gz = g_ld_stream<u32x4>(gGZ2, t16, so);
      const float eta_i[2] = {bf2f(g_ldh(gETA, 2 * c, (k * cgs + j) * (CS * 2) + 64 * tb[0])),
                              bf2f(g_ldh(gETA, 2 * c, (k * cgs + j) * (CS * 2) + 64 * tb[1]))};
      bf16x8 g1b[4];   // gZ1_bar^T of the output branch: lane = hid, contraction = tok
      bf16x8 w2bf[4];  // W2 before the step: lane = hid, contraction = F
#pragma unroll
      for (int s = 0; s < 4; s++) {
        g1b[s] = image_load<true>(gGZ1B, ho, s, t16);
        w2bf[s] = w2_before<true>(gIMG2, gCW2, ckW, j, s, hid0, c, h, t16);
      }
      bf16x8 g1[2][2], dz[2][2], w1b[2][2], d1[2][2];
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int t = 0; t < 2; t++) {
          d1[a][t] = image_load<true>(gDD, j * (2 * IMG_BYTES), 2 * tb[a] + t, t16);   // gelu'(Z1)
          dz[a][t] = image_load<true>(gDZ, ho, 2 * tb[a] + t, t16);
          w1b[a][t] = w1_before<true>(gIMG1, gCW1, ckW, j, a, t, hid0, c, h, t16);
        }
      lds_put16x(s_xq, tid, xq);
      lds_put16x(s_xk, tid, xk);
      lds_put16(s_gz2, tid, gz);
      __syncthreads();
      mma_jit<4>(gW1s, [&](int fb, int s) { return xpiece_tr(s_xq, fb, s, lane); },         // + XQ^T gZ1_bar
                 [&](int, int s) { return g1b[s]; });
      store_state_rows<LDF>(T2, gW1s, c, h);                                                  // gW1 rows [hid][F]
#pragma unroll
      for (int s = 0; s < 4; s++) store_piece_rows<LDF>(T1, 0, s, c, h, w2bf[s]);            // W2 before the step, rows [hid][F]
      WAVE_SYNC();
      AccT<2, 2> dk;
      acc_zero(dk);
#pragma unroll
      for (int i = 0; i < 2; i++) {
        // G1 = -eta * dl/dZ1 with dl/dZ1 = (gZ2 W2^T) * gelu'(Z1), as the walk forms it
        AccT<1, 1> R;
        acc_zero(R);
        mma_jit<4>(R, [&](int, int s) { return piece_rows<LDF>(T1, 0, s, c, h); },
                   [&](int, int s) { return piece_rows<LDX>(s_gz2, tb[i], s, c, h); });
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
          for (int jj = 0; jj < 8; jj++) {
            const float a = (float)d1[i][t][jj];
            const float gz1 = R.b[0][0][8 * t + jj] * a;
            g1[i][t][jj] = (bf16)(-eta_i[i] * gz1);
          }
#pragma unroll
          for (int rb = 0; rb < 2; rb++) dk.b[rb][i] = MFMA(piece_tr<LDF>(T2, rb, t, lane), g1[i][t], dk.b[rb][i]);
        }
      }
      WAVE_SYNC();   // the readers of T1 (W2 rows) are done
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int t = 0; t < 2; t++) store_piece_rows<LDH>(T1, tb[i], t, c, h, dz[i][t]);     // dZ1 rows [tok][hid]
      WAVE_SYNC();
      mma_jit<2>(dk, [&](int rb, int s) { return w1b[rb][s]; }, [&](int i, int s) { return dz[i][s]; });
      mma_jit<4>(gW1s, [&](int fb, int s) { return xpiece_tr(s_xk, fb, s, lane); },         // + XK^T dZ1
                 [&](int, int s) { return piece_tr<LDH>(T1, 0, s, lane); });
      WAVE_SYNC();   // this wave's readers of T1 / T2 are done
      TTT_STAGE(BS_X_PRODUCTS);
      pair_sum(s_own, s_partner, dk, c, h);
      float z[8];
      ln_gather(z, s_lnrow);
      const float gyv[8] = {gy_lo[0], gy_lo[1], gy_lo[2], gy_lo[3], gy_hi[0], gy_hi[1], gy_hi[2], gy_hi[3]};
      const float dgv[8] = {dg_lo[0], dg_lo[1], dg_lo[2], dg_lo[3], dg_hi[0], dg_hi[1], dg_hi[2], dg_hi[3]};
      bf16x8 dxk_new, dxv_new;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        dxk_new[e] = (bf16)((float)dxk_ld[e] + (z[e] + gyv[e]));
        dxv_new[e] = (bf16)((float)dxv_ld[e] - gyv[e]);                 // dXV accumulates -g_y
      }
      g_st_stream<bf16x8>(gDXK, vln, xo, dxk_new);
      g_st_stream<bf16x8>(gDXV, vln, xo, dxv_new);
      ln_token_sum_add(s_dgw, dgv, lane, f0);
      ln_token_sum_add(s_dbw, gyv, lane, f0);
      __syncthreads();   // the readers of the pair sums are done before the next mini-batch's take their place
      TTT_STAGE(BS_X_SUMS);
    }
    publish(w_finished, done + 1);
    TTT_STAGE(BS_PUBLISH);
  }
  TTT_STAGES_END(p.stage_clocks == nullptr ? nullptr : p.stage_clocks + ((size_t)bh * 4 + 3) * (BW_NWAVE * STAGE_SLOTS));
  // norm-weight / norm-bias gradients: the replaying workgroups' two sums (handed over before their last counts,
  // which the walk had acquired before its own last count) + the walk's, in the order of the other launch shapes
  __syncthreads();
  if (tid < 2 * FD) {
    const int which = tid / FD, f = tid % FD;
    const float* rp = p.norm_partial + (size_t)bh * 2 * (BW_NWAVE * 2 * FD);
    const bool have_odd = p.K > 1 || p.n_replay == 1;
    float s = 0.f, sr0 = 0.f, sr1 = 0.f;
#pragma unroll
    for (int u = 0; u < BW_NWAVE; u++) {
      s += s_red[(u * 2 + which) * FD + f];
      sr0 += rp[(u * 2 + which) * FD + f];
      if (have_odd) sr1 += rp[BW_NWAVE * 2 * FD + (u * 2 + which) * FD + f];
    }
    (which == 0 ? p.grad_L_ttt_norm_weight : p.grad_L_ttt_norm_bias)[(size_t)bh * FD + f] = (sr0 + sr1) + s;
  }
}

// ------------------------------------------------------------------ the workgroup that fetches ahead of the walk
// The walk asks per mini-batch for 240 KiB that a replaying workgroup wrote a checkpoint group earlier (six register
// images, four tiles) or that the caller passed in (two tiles): none of it is in the L2 by then, and one CU cannot
// keep enough requests in flight to hide the way to HBM.  This workgroup computes nothing: it goes through the walk's
// mini-batches in the walk's order, PREFETCH_AHEAD of them ahead of it, and reads one dword of every 128-byte line
// the walk will ask for.  Placed on the walk's XCD, it leaves the lines in the L2 that the walk's requests go to.
// Purely a hint: the values are dropped, nothing is written except the status word of a wait that gives up, and
// the walk's results do not depend on whether, when or where this workgroup runs.
constexpr int PREFETCH_AHEAD = 1;
TTT_DEV void bwd_prefetch(const BwdParams& p, unsigned char* smem, const int bh) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int v = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cgs = p.cgs, n_replay = p.n_replay, n_sets = 2 * n_replay;
  int* const w_sync = p.sync + (size_t)bh * BWD_SYNC_STRIDE;
  int* const w_step = w_sync + 20;
  int* const s_flag = reinterpret_cast<int*>(smem + SB_FLAG);
  const size_t ox = uni64((size_t)bh * p.NC * (CS * FD)), of = uni64((size_t)bh * cgs * (CS * FD));
  const size_t oh = uni64((size_t)bh * cgs * (CS * HID)), opk = uni64((size_t)bh * cgs * (FD * HID));
  const unsigned line_t = 128u * lane, line_i = 128u * (tid & 255);   // this thread's line of a tile / of an image
  int n = 0;   // mini-batches the walk has before the one at hand
  for (int k = p.K - 1; k >= 0; k--) {
    const int n_mb = min(cgs, p.NC - k * cgs);
    const int done = p.K - 1 - k, set = done % n_sets;
    // the group has been replayed: what is fetched is what the walk will read
    if (!wait_at_least(w_sync + 8 * (done % n_replay), done / n_replay + 1, p.status, s_flag, p.wait_limit)) return;
#define PGRP(name) (set ? p.alt_##name[set - 1] : p.name)
    // wave v fetches tile v (v < 6): the two inputs (indexed by the mini-batch's place in the sequence), then four of the set
    gptr_t tile = gbuf(p.XQ + ox);
    unsigned tile0 = k * cgs * TILE_BYTES;
    if (v == 1) tile = gbuf(p.XK + ox);
    if (v >= 2) tile0 = 0;
    if (v == 2) tile = gbuf(PGRP(grad_l_wrt_Z2_group) + of);
    if (v == 3) tile = gbuf(PGRP(grad_x_hat_fused_group) + of);
    if (v == 4) tile = gbuf(PGRP(x_hat_fused_group) + of);
    if (v >= 5) tile = gbuf(PGRP(grad_output_fused_group) + of);
    // and half of three of the six images: waves 0-3 X2_bar, GELU, GELU''; waves 4-7 gZ1_bar, GELU', W2 before the step
    const bool up = v >= 4;
    const gptr_t img0 = up ? gbuf(PGRP(Z1_bar_group) + oh) : gbuf(PGRP(X2_bar_group) + oh);
    const gptr_t img1 = up ? gbuf(PGRP(W1_init_group) + opk) : gbuf(PGRP(Z1_group) + oh);
    const gptr_t img2 = up ? gbuf(PGRP(grad_l_wrt_Z1_group) + oh) : gbuf(PGRP(W1_init_group) + opk);
#undef PGRP
    for (int j = n_mb - 1; j >= 0; j--, n++) {
      const int seen = wait_for_pace(w_step, n + 1 - PREFETCH_AHEAD, p.status, s_flag, p.wait_limit);
      if (seen == 0) return;
      if (seen - 1 > n + 1) continue;   // the walk is past this mini-batch already
      const unsigned ho = j * IMG_BYTES;
      unsigned got[4] = {0, 0, 0, 0};
      if (v < 6) got[0] = g_ld<unsigned>(tile, line_t, tile0 + j * TILE_BYTES);
      got[1] = g_ld<unsigned>(img0, line_i, ho);
      got[2] = g_ld<unsigned>(img1, line_i, up ? 2 * ho : ho);
      if (!up) got[3] = g_ld<unsigned>(img2, line_i, 2 * ho + IMG_BYTES);
      else if (j > 0) got[3] = g_ld<unsigned>(img2, line_i, ho - IMG_BYTES);
#pragma unroll
      for (int i = 0; i < 4; i++) asm volatile("" ::"v"(got[i]));   // landed; nothing is done with them
    }
  }
}

// n_replay + 1 (+ 1) workgroups per (batch, head).  Workgroups are dealt to the 8 XCDs in turn, so with a
// multiple of 8 (batch, head) pairs the workgroups of a pair are placed 8 apart: same XCD, same L2.
// One kernel per combination, so that each holds only the code (and the register allocation) of its own roles.
template <int NREPLAY, bool FINISH>
__global__ __launch_bounds__(BW_THREADS) void ttt_mlp_bwd_split_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int b = blockIdx.x, per = NREPLAY + 1 + (FINISH ? 1 + p.n_prefetch : 0);
  int bh, role;
  if (p.nbh % 8 == 0) {
    bh = (b / (8 * per)) * 8 + (b & 7);
    role = (b >> 3) % per;
  } else {
    bh = b / per;
    role = b % per;
  }
  bh += p.bh0;
  constexpr bool IMG = NREPLAY == 2;   // two replaying workgroups also evaluate the GELU family for the walk
  if (role < NREPLAY) bwd_body<1, IMG, FINISH>(p, smem, bh, role, p.K - 1, 0);
  else if (role == NREPLAY) bwd_body<2, IMG, FINISH>(p, smem, bh, 0, p.K - 1, 0);
  else if constexpr (FINISH) {
    if (role == NREPLAY + 1) bwd_finish_dxk(p, smem, bh);
    else bwd_prefetch(p, smem, bh);
  }
}

__global__ void ttt_mlp_zero_words(int* w, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) w[i] = 0;
}

}  // namespace ttt

extern "C" int ttt_mlp_bwd_threads() { return ttt::BW_THREADS; }
extern "C" int ttt_mlp_bwd_lds_bytes() { return ttt::SM_BWD_BYTES; }

hipError_t ttt_mlp_bwd_enqueue(const ttt::BwdParams& p, hipStream_t stream) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(ttt::ttt_mlp_bwd_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, ttt::SM_BWD_BYTES);
  if (e != hipSuccess) return e;
  if (p.sync == nullptr) {
    hipLaunchKernelGGL(ttt::ttt_mlp_bwd_kernel, dim3(p.nbh), dim3(ttt::BW_THREADS), ttt::SM_BWD_BYTES, stream, p);
    return hipGetLastError();
  }
  const int n = static_cast<int>(ttt::bwd_sync_ints(p.nbh));
  int* const words = p.status - (size_t)p.nbh * ttt::BWD_SYNC_STRIDE;   // p.sync itself is moved back by bh0 entries
  hipLaunchKernelGGL(ttt::ttt_mlp_zero_words, dim3((n + 255) / 256), dim3(256), 0, stream, words, n);
  const dim3 grid((p.n_replay + 1 + p.n_finish + p.n_prefetch) * p.nbh), block(ttt::BW_THREADS);
  auto launch = [&](auto kernel) -> hipError_t {
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, ttt::SM_BWD_BYTES);
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(kernel, grid, block, ttt::SM_BWD_BYTES, stream, p);
    return hipGetLastError();
  };
  if (p.n_finish) return launch(ttt::ttt_mlp_bwd_split_kernel<2, true>);
  if (p.n_replay == 2) return launch(ttt::ttt_mlp_bwd_split_kernel<2, false>);
  return launch(ttt::ttt_mlp_bwd_split_kernel<1, false>);
}
