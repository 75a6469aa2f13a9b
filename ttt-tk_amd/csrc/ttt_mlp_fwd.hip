// Forward scan of the non-causal TTT-MLP layer for gfx950 (MI355X).
//
// Behaviour follows the upstream operator `ttt_forward` (kernels/ttt/ttt.cu:85-586 for the kernel,
// kernels/ttt/matching.py:30-125 for the mathematics): for every (batch, head) the fp32 state
// (W1,b1,W2,b2) is carried through NC mini-batches of 64 tokens; before mini-batch i with
// i % checkpoint_group_size == 0 the state is stored at checkpoint slot i / checkpoint_group_size.
//
// Mapping: workgroups of 8 wavefronts (two per SIMD, at most 256 registers each); one per (batch,
// head), or two where the device has CUs to spare - then one carries the state and the other computes
// Out from the states it leaves behind.  Wave v owns hidden columns [32v, 32v+32).  The state lives in registers for the whole scan
// as MFMA accumulator tiles:
//   W1s = W1[:, shard]      (rows F,   columns hid)  -> chained operand of XK*W1 and of (XQ*W1)^T
//   W2s = W2[shard, :]      (rows hid, columns F)    -> chained operand of (X2*W2)^T
// and the eta-scaled updates are MFMA accumulations into them.  Only gZ2*W2^T needs W2 with the other index
// contracted: for it the two bf16 terms of W2s are transposed through a wave-private LDS tile once per mini-batch
// (a second resident copy W2^T, kept up to date by a second set of update products, cost 32 registers and a
// third more MFMA work, and the registers are what this kernel is short of).
// Operand precision: the products that carry the state from one mini-batch to the next (XK W1, X2 W2,
// G2 W2^T and the two weight steps) take their fp32 operands - the weights, G2 = -eta dl/dZ2, G1 and, in
// the W2 step, X2 - as two bf16 terms (hi + lo, one MFMA product per term; XK is bf16 already), because
// a single bf16 rounding of them, repeated over thousands of mini-batches, moves the gradients of the
// remat backward further from the fp32 mathematics than cosine 0.9999.  The output branch uses one term.
// Sums over the hidden dimension (Z2) are formed in two steps: waves v and v+4 exchange halves of
// their partial tiles through LDS and each finishes one half, then every wave LayerNorms 8 of the
// 64 tokens (8 lanes per token) from the four pair sums.  All sums have a fixed order.
#include "ttt_mlp_common.hpp"
#include "ttt_mlp_kernels.hpp"

namespace ttt {

constexpr int FW_NWAVE = 8;
constexpr int FW_THREADS = 64 * FW_NWAVE;
constexpr int FW_NS = HID / FW_NWAVE;                  // hidden columns per wave: 32
// Row stride (elements) of every bf16 tile in LDS.  136-byte rows put the 32 row-wise 8-byte reads of
// an operand piece on 64 distinct banks (measured: 8.6 clocks per piece against 16 with 144-byte
// rows); rows are 8-byte aligned, so 16-byte accesses are made as two 8-byte ones.
constexpr int FLD = 68;
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16((a), (b), (c), 0, 0, 0)
TTT_DEV OpdT<2, 4> x_rows_kappa(const bf16* tile, int c, int h) {
  OpdT<2, 4> o;
#pragma unroll
  for (int fb = 0; fb < 2; fb++)
#pragma unroll
    for (int s = 0; s < 4; s++) o.v[fb][s] = xpiece_rows(tile, fb, s, c, h);
  return o;
}

// LDS carve-up (bytes)
constexpr int SM_TILE = 64 * FLD * 2;                   // one bf16 tile: 8704
static_assert(32 * 132 * 2 <= SM_TILE, "a tile of row pairs fits a tile slot");
constexpr int SM_XQ = 0;                                // two buffers, alternating per mini-batch
constexpr int SM_XK = SM_XQ + 2 * SM_TILE;
constexpr int SM_XV = SM_XK + SM_TILE;
constexpr int SM_G2 = SM_XV + SM_TILE;
constexpr int SM_G2L = SM_G2 + SM_TILE;                  // low-order bf16 term of G2
constexpr int SM_P = SM_G2L + SM_TILE;                   // 4 fp32 pair-sum tiles [tok][F]
constexpr int SM_PTILE = 64 * LDP * 4;
constexpr int SM_X2T = SM_P + 4 * SM_PTILE;             // per wave: X2 shard stored [hid][tok], bf16
constexpr int SM_X2T_TILE = FW_NS * FLD * 2;
constexpr int SM_B1 = SM_X2T + FW_NWAVE * SM_X2T_TILE;
constexpr int SM_B2 = SM_B1 + HID * 4;
constexpr int SM_ETA = SM_B2 + FD * 4;
constexpr int SM_GAM = SM_ETA + CS * 4;
constexpr int SM_BET = SM_GAM + FD * 4;
constexpr int SM_B2P = SM_BET + FD * 4;                  // per wave: the sum of G2 over its 8 LayerNorm tokens (the step of b2)
constexpr int SM_FLAG = SM_B2P + FW_NWAVE * FD * 4;      // outcome of a wait on the other workgroup
constexpr int SM_FWD_BYTES = SM_FLAG + 16;
static_assert(SM_FWD_BYTES <= 160 * 1024, "forward LDS budget");

// 16 bytes to / from an 8-byte aligned LDS address.
TTT_DEV void lds_put16(void* p, u32x4 v) {
  uint2* d = reinterpret_cast<uint2*>(p);
  d[0] = make_uint2(v[0], v[1]);
  d[1] = make_uint2(v[2], v[3]);
}
TTT_DEV bf16x8 lds_get8h(const bf16* p) { return cat(*reinterpret_cast<const bf16x4*>(p), *reinterpret_cast<const bf16x4*>(p + 4)); }

struct Staged {  // one mini-batch of inputs in flight from HBM: one 16-byte chunk per tile per thread
  u32x4 q, k, v;
  bf16 eta;
};

// gq / gk / gv / ge = this (batch, head)'s XQ, XK, XV, last_eta; thread tid moves 16-byte chunk tid
// (row tid / 8, 8 chunks per row) of each tile of mini-batch mb.
constexpr unsigned TILE_BYTES = CS * FD * 2;
TTT_DEV void stage_load(Staged& s, gptr_t gq, gptr_t gk, gptr_t gv, gptr_t ge, int mb, int tid) {
  s.q = g_ld16(gq, 16 * tid, mb * TILE_BYTES);
  s.k = g_ld16(gk, 16 * tid, mb * TILE_BYTES);
  s.v = g_ld16(gv, 16 * tid, mb * TILE_BYTES);
  s.eta = g_ldh(ge, 2 * (tid & (CS - 1)), mb * (CS * 2));   // threads >= CS drop it
}

TTT_DEV void stage_store(const Staged& s, unsigned char* smem, int xq_buf, int tid) {
  const int off = (xrow(tid >> 3) + (tid & 7) * 8) * 2;
  lds_put16(smem + SM_XQ + xq_buf * SM_TILE + off, s.q);
  lds_put16(smem + SM_XK + off, s.k);
  lds_put16(smem + SM_XV + off, s.v);
  if (tid < CS) reinterpret_cast<bf16*>(smem + SM_ETA)[tid] = s.eta;   // eta stays bf16 in LDS
}

// Two-step sum over the wave pair (v, v ^ 4) of a partial tile z (rows F, columns tok): the wave
// with pair index r gives away row block 1-r, then adds the partner's row block r to its own and
// leaves the pair sum in the pair's LDS tile, stored [tok][F].  Contains two workgroup barriers.
template <int R>
TTT_DEV void pair_give(float* tile, const AccT<2, 2>& z, int c, int h) {
#pragma unroll
  for (int cb = 0; cb < 2; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const f32x16& x = z.b[1 - R][cb];
      f32x4 v = {x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]};
      *reinterpret_cast<f32x4*>(tile + (32 * cb + c) * LDP + 32 * (1 - R) + 8 * g + 4 * h) = v;
    }
}
template <int R>
TTT_DEV void pair_take(float* tile, const AccT<2, 2>& z, int c, int h) {
#pragma unroll
  for (int cb = 0; cb < 2; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      float* q = tile + (32 * cb + c) * LDP + 32 * R + 8 * g + 4 * h;
      const f32x16& x = z.b[R][cb];
      f32x4 v = *reinterpret_cast<const f32x4*>(q);
      v[0] += x[4 * g]; v[1] += x[4 * g + 1]; v[2] += x[4 * g + 2]; v[3] += x[4 * g + 3];
      *reinterpret_cast<f32x4*>(q) = v;
    }
}
TTT_DEV void pair_sum_to_lds(float* tile, const AccT<2, 2>& z, int r, int c, int h) {
  if (r == 0) pair_give<0>(tile, z, c, h); else pair_give<1>(tile, z, c, h);
  __syncthreads();
  if (r == 0) pair_take<0>(tile, z, c, h); else pair_take<1>(tile, z, c, h);
  __syncthreads();
}

// The same sum with the product formed one F block at a time - `half(rb)` returns rows [32 rb, 32 rb + 32) of
// the partial tile - so that 32 accumulator registers are live instead of 64: first the block that is given away,
// then the one that is kept.
template <int R, class HALF>
TTT_DEV void pair_sum_halves_r(float* tile, HALF half, int c, int h) {
  {
    const AccT<1, 2> z = half(1 - R);
#pragma unroll
    for (int cb = 0; cb < 2; cb++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x16& x = z.b[0][cb];
        f32x4 v = {x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]};
        *reinterpret_cast<f32x4*>(tile + (32 * cb + c) * LDP + 32 * (1 - R) + 8 * g + 4 * h) = v;
      }
  }
  const AccT<1, 2> z = half(R);
  __syncthreads();
#pragma unroll
  for (int cb = 0; cb < 2; cb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      float* q = tile + (32 * cb + c) * LDP + 32 * R + 8 * g + 4 * h;
      const f32x16& x = z.b[0][cb];
      f32x4 v = *reinterpret_cast<const f32x4*>(q);
      v[0] += x[4 * g]; v[1] += x[4 * g + 1]; v[2] += x[4 * g + 2]; v[3] += x[4 * g + 3];
      *reinterpret_cast<f32x4*>(q) = v;
    }
  __syncthreads();
}
template <class HALF0, class HALF1>
TTT_DEV void pair_sum_halves(float* tile, HALF0 half0, HALF1 half1, int r, int c, int h) {
  // half0 / half1: the product's F block 0 / 1 (two callables so that each indexes the state registers statically)
  if (r == 0) pair_sum_halves_r<0>(tile, [&](int rb) { return rb == 0 ? half0() : half1(); }, c, h);
  else pair_sum_halves_r<1>(tile, [&](int rb) { return rb == 0 ? half0() : half1(); }, c, h);
}

// Output LayerNorm + residual for the 8 features [f0, f0+8) of token `tok`: Out = XQ + LN(sum of the four
// pair sums + b2).  8 lanes per token, 8 tokens per wave.
TTT_DEV void output_layernorm(const float* s_P, const float* s_b2, const float* s_gam, const float* s_bet,
                              const bf16* s_xq, gptr_t gOut, int mb, int tok, int f0) {
  float z[8];
  {
    f32x4 a0 = *reinterpret_cast<const f32x4*>(s_b2 + f0);
    f32x4 a1 = *reinterpret_cast<const f32x4*>(s_b2 + f0 + 4);
#pragma unroll
    for (int t = 0; t < 4; t++) {
      a0 += *reinterpret_cast<const f32x4*>(s_P + t * 64 * LDP + tok * LDP + f0);
      a1 += *reinterpret_cast<const f32x4*>(s_P + t * 64 * LDP + tok * LDP + f0 + 4);
    }
#pragma unroll
    for (int e = 0; e < 4; e++) { z[e] = a0[e]; z[4 + e] = a1[e]; }
  }
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) sum += z[e];
  const float mu = oct_sum(sum) * (1.f / FD);
  float var = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) { z[e] -= mu; var = __builtin_fmaf(z[e], z[e], var); }
  const float rstd = __builtin_amdgcn_rsqf(oct_sum(var) * (1.f / FD) + LN_EPS);
  const bf16x8 qv = lds_get8h(s_xq + xrow(tok) + f0);
  float gam[8], bet[8];
#pragma unroll
  for (int q = 0; q < 2; q++) {
    const f32x4 gq = *reinterpret_cast<const f32x4*>(s_gam + f0 + 4 * q);
    const f32x4 bq = *reinterpret_cast<const f32x4*>(s_bet + f0 + 4 * q);
#pragma unroll
    for (int e = 0; e < 4; e++) { gam[4 * q + e] = gq[e]; bet[4 * q + e] = bq[e]; }
  }
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 8; e++) o[e] = (bf16)(bf2f(qv[e]) + __builtin_fmaf(gam[e], z[e] * rstd, bet[e]));
  g_st8h(gOut, (tok * FD + f0) * 2, mb * TILE_BYTES, o);
}

// ROLE 0: the whole scan in one workgroup.  ROLE 1: the state recurrence only - after every mini-batch
// the new state is left in HBM as ready-made bf16 operands for the workgroup that runs fwd_output_branch.
// RING: mini-batches per hand-over (ROLE 1).
template <int ROLE, int RING>
// mb0, mb1: the mini-batches [mb0, mb1) of the sequence (ROLE 0: a segment; mb0 is a multiple of the checkpoint group
// size, and so is mb1 unless it is the sequence's end).
TTT_DEV void fwd_body(const FwdParams& p, unsigned char* smem, const int bh, const int mb0, const int mb1) {
  bf16* s_g2 = reinterpret_cast<bf16*>(smem + SM_G2);
  bf16* s_g2l = reinterpret_cast<bf16*>(smem + SM_G2L);
  float* s_P = reinterpret_cast<float*>(smem + SM_P);
  float* s_b1 = reinterpret_cast<float*>(smem + SM_B1);
  float* s_b2 = reinterpret_cast<float*>(smem + SM_B2);
  float* s_gam = reinterpret_cast<float*>(smem + SM_GAM);
  float* s_bet = reinterpret_cast<float*>(smem + SM_BET);

  const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5, c = lane & 31;
  const int v = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave index, in a scalar register
  const int pr = v >> 2;                                    // index inside the wave pair (v & 3)
  const int tok = 8 * v + (lane >> 3), f0 = 8 * (lane & 7); // LayerNorm ownership: 8 lanes per token, 8 features each
  const int head = bh % p.NH;
  const int hid0 = FW_NS * v;
  float* s_Pp = s_P + (v & 3) * 64 * LDP;
  bf16* s_x2t = reinterpret_cast<bf16*>(smem + SM_X2T + v * SM_X2T_TILE);
  // Everything derived from the lane index is cheap to recompute and expensive to keep in a register
  // (or spilled) for the whole scan: LANE_VARS re-derives it from a lane index the optimiser cannot see
  // through, so each stage that opens with it gets fresh, short-lived copies.
  int lane_v = lane;
#define LANE_VARS                                                               \
  asm volatile("" : "+v"(lane_v));                                              \
  const int lane = lane_v, h = lane >> 5, c = lane & 31, tid = (v << 6) | lane; \
  const int tok = 8 * v + (lane >> 3), f0 = 8 * (lane & 7);                     \
  (void)h; (void)c; (void)tid; (void)tok; (void)f0

  // ---- state -> registers: the caller's initial state, or (a later segment) the checkpoint before mini-batch mb0
  AccT<2, 1> W1s;
  AccT<1, 2> W2s;
  float b1L;      // b1 of hidden column hid0 + c; b2 lives in LDS (fp32) and is updated there by wave 0
  {
    const size_t from = mb0 > 0 ? (size_t)bh * p.K + mb0 / p.cgs : (size_t)bh;
    const float* const W1src = (mb0 > 0 ? p.W1_ck : p.W1) + from * FD * HID;
    const float* const W2src = (mb0 > 0 ? p.W2_ck : p.W2) + from * HID * FD;
    const float* const b1src = (mb0 > 0 ? p.b1_ck : p.b1) + from * HID;
    const float* const b2src = (mb0 > 0 ? p.b2_ck : p.b2) + from * FD;
    const gptr_t W1 = gbuf(W1src), W2 = gbuf(W2src);
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int row = 8 * (i >> 2) + (i & 3);   // + 4h in the lane offset
        W1s.b[b][0][i] = g_ldf(W1, (4 * h * HID + c) * 4, ((32 * b + row) * HID + hid0) * 4);
        W2s.b[0][b][i] = g_ldf(W2, (4 * h * FD + c) * 4, ((hid0 + row) * FD + 32 * b) * 4);
      }
    b1L = b1src[hid0 + c];
    if (tid < HID) s_b1[tid] = b1src[tid];
    if (tid < FD) {
      s_b2[tid] = b2src[tid];
      s_gam[tid] = p.ttt_norm_weight[head * FD + tid];
      s_bet[tid] = p.ttt_norm_bias[head * FD + tid];
    }
  }

  // HBM addressing: scalar base of this (batch, head) + scalar offset of the mini-batch + lane offset
  const size_t x_base = uni64((size_t)bh * p.NC * (CS * FD));
  const gptr_t gXQ = gbuf(p.XQ + x_base), gXK = gbuf(p.XK + x_base), gXV = gbuf(p.XV + x_base), gOut = gbuf(p.Out + x_base);
  const gptr_t gEta = gbuf(p.last_eta + uni64((size_t)bh * p.NC * CS));
  const gptr_t gW1ck = gbuf(p.W1_ck + uni64((size_t)bh * p.K * FD * HID)), gW2ck = gbuf(p.W2_ck + uni64((size_t)bh * p.K * HID * FD));
  {
    Staged st;
    stage_load(st, gXQ, gXK, gXV, gEta, mb0, tid);
    stage_store(st, smem, mb0 & 1, tid);
  }
  __syncthreads();

  int* const w_given = p.sync + (size_t)bh * BWD_SYNC_STRIDE;   // groups handed to the output branch
  int* const w_taken = w_given + 16;                             // groups it has finished
  int* const w_status = p.status;
  int* const s_flag = reinterpret_cast<int*>(smem + SM_FLAG);

  // the state as checkpoint number `ck_slot` of this (batch, head)
  auto store_checkpoint = [&](int ck_slot) {
    LANE_VARS;
    const size_t slot = (size_t)bh * p.K + ck_slot;
    const unsigned ck = static_cast<unsigned>(ck_slot) * (FD * HID * 4u);   // byte offset of the slot in gW1ck / gW2ck
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int row = 8 * (i >> 2) + (i & 3);   // + 4h in the lane offset
        g_stf(gW1ck, (4 * h * HID + c) * 4, ck + ((32 * b + row) * HID + hid0) * 4, W1s.b[b][0][i]);
        g_stf(gW2ck, (4 * h * FD + c) * 4, ck + ((hid0 + row) * FD + 32 * b) * 4, W2s.b[0][b][i]);
      }
    if (h == 0) p.b1_ck[slot * HID + hid0 + c] = b1L;
    if (tid < FD) p.b2_ck[slot * FD + tid] = s_b2[tid];
  };

  TTT_STAGES_BEGIN();
  for (int mb = mb0; mb < mb1; mb++) {
    LANE_VARS;
    const bf16* s_xq = reinterpret_cast<const bf16*>(smem + SM_XQ + (mb & 1) * SM_TILE);
    // ROLE 1 has no use for XQ (nor for b1 in LDS): their space holds a second XK / XV / eta buffer, so that
    // the next mini-batch's inputs can be written while this one's are still being read.
    const int alt = ROLE == 1 ? (mb & 1) : 0;
    const bf16* s_xk = reinterpret_cast<const bf16*>(smem + (alt ? SM_XQ : SM_XK));
    const bf16* s_xv = reinterpret_cast<const bf16*>(smem + (alt ? SM_XQ + SM_TILE : SM_XV));
    const bf16* s_eta = reinterpret_cast<const bf16*>(smem + (alt ? SM_B1 : SM_ETA));
    // ROLE 1: where the state after this mini-batch goes (a ring of 2 * ring slots)
    constexpr int ring = RING; const int grp = mb / ring, at = mb % ring, slot = (grp & 1) * ring + at;
    float* const gB = p.bias_img + ((size_t)bh * 2 * FWD_RING_MAX + slot) * FWD_BIAS_FLOATS;
    if constexpr (ROLE == 1) {
      if (at == 0 && grp >= 2) {   // the set is free once the output branch is done with the group before last
        if (!wait_at_least(w_taken, grp - 1, w_status, s_flag, p.wait_limit)) return;
      }
    }

    // ROLE 1 ends a mini-batch without a barrier: this one makes the inputs staged at the end of the last mini-batch
    // visible
    if constexpr (ROLE == 1) {
      if (mb > 0) __syncthreads();
    }
    // ---- checkpoint: the state before this mini-batch
    if (mb % p.cgs == 0) store_checkpoint(mb / p.cgs);

    TTT_STAGE(FS_TOP);
    // ---- Z1 = XK W1 + b1 (rows tok, lane = hid);  X2 = gelu(Z1), D1 = gelu'(Z1)
    AccT<2, 1> x2, d1;
    {
      LANE_VARS;
      OpdT<1, 4> w1h, w1l;
      cvt_chain_split(W1s, w1h, w1l);
      const OpdT<2, 4> xkA = x_rows_kappa(s_xk, c, h);
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int i = 0; i < 16; i++) x2.b[rb][0][i] = b1L;
      mma(x2, xkA, w1l);
      mma(x2, xkA, w1h);
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          float g, d;
          gelu_fd(x2.b[rb][0][i], g, d);
          x2.b[rb][0][i] = g;
          d1.b[rb][0][i] = d;
        }
    }
    TTT_STAGE(FS_F1_GELU);
    OpdT<1, 4> x2lo;                                        // lane = hid, contraction = tok: the low-order term, for the W2 step
    {
      LANE_VARS;
      OpdT<1, 4> x2op;
      cvt_chain_split(x2, x2op, x2lo);
      lds_store_rows_kappa<1, 4>(s_x2t, FLD, x2op, c, h);   // stored [hid][tok], private to the wave; read back as rows by the W2 step
    }
    TTT_WAVE_SYNC();

    TTT_STAGE(FS_X2_SPLIT);
    // ---- Z2^T partial = W2s^T X2^T (rows F, lane = tok), summed over the pair into [tok][F]
    {
      LANE_VARS;
      auto z2_block = [&](const f32x16& w2) {   // one F block of W2s^T X2^T: W2s in two terms, X2^T from the bounce tile
        AccT<1, 2> z;
        acc_zero(z);
#pragma unroll
        for (int s = 0; s < 2; s++) {
          bf16x8 wh, wl, xb[2];
          split8(w2, s, wh, wl);
#pragma unroll
          for (int cb = 0; cb < 2; cb++) xb[cb] = piece_tr<FLD>(s_x2t, cb, s, lane);
#pragma unroll
          for (int cb = 0; cb < 2; cb++) {
            z.b[0][cb] = MFMA(wl, xb[cb], z.b[0][cb]);
            z.b[0][cb] = MFMA(wh, xb[cb], z.b[0][cb]);
          }
        }
        return z;
      };
      pair_sum_halves(s_Pp, [&]() { return z2_block(W2s.b[0][0]); }, [&]() { return z2_block(W2s.b[0][1]); }, pr, c, h);
    }

    TTT_STAGE(FS_F2_PAIRSUM);
    // ---- LayerNorm-fused reconstruction-loss gradient: 8 tokens per wave, 8 lanes per token
    {
      LANE_VARS;
      if constexpr (ROLE == 1) {
        // The next mini-batch's XK / XV / eta leave HBM for the other LDS buffers now (last read a mini-batch ago,
        // two barriers back) without passing through registers: wave v fetches rows 8v .. 8v+7 of both tiles,
        // one pair of rows (256 contiguous bytes) per load, wave 0 also the 128 bytes of eta.
        if (mb + 1 < mb1) {
          tile_to_lds(gXK, (mb + 1) * TILE_BYTES, smem + (alt ? SM_XK : SM_XQ), v, lane);
          tile_to_lds(gXV, (mb + 1) * TILE_BYTES, smem + (alt ? SM_XV : SM_XQ + SM_TILE), v, lane);
          eta_to_lds(gEta, (mb + 1) * (CS * 2), smem + (alt ? SM_ETA : SM_B1), v, lane);
        }
      } else {
        // One workgroup: XQ has two buffers, so the next XQ can leave HBM now; XK / XV / eta follow once their
        // last readers are done (after the pair sum of the output branch).
        if (mb + 1 < mb1) tile_to_lds(gXQ, (mb + 1) * TILE_BYTES, smem + SM_XQ + ((mb + 1) & 1) * SM_TILE, v, lane);
      }
      float z[8];
      {
        f32x4 a0 = *reinterpret_cast<const f32x4*>(s_b2 + f0);
        f32x4 a1 = *reinterpret_cast<const f32x4*>(s_b2 + f0 + 4);
#pragma unroll
        for (int t = 0; t < 4; t++) {
          a0 += *reinterpret_cast<const f32x4*>(s_P + t * 64 * LDP + tok * LDP + f0);
          a1 += *reinterpret_cast<const f32x4*>(s_P + t * 64 * LDP + tok * LDP + f0 + 4);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) { z[e] = a0[e]; z[4 + e] = a1[e]; }
      }
      float sum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) sum += z[e];
      const float mu = oct_sum(sum) * (1.f / FD);
      float var = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) { z[e] -= mu; var = __builtin_fmaf(z[e], z[e], var); }
      const float rstd = __builtin_amdgcn_rsqf(oct_sum(var) * (1.f / FD) + LN_EPS);
      const bf16x8 kv = lds_get8h(s_xk + xrow(tok) + f0);
      const bf16x8 vv = lds_get8h(s_xv + xrow(tok) + f0);
      float gam[8], bet[8];
#pragma unroll
      for (int q = 0; q < 2; q++) {
        const f32x4 gq = *reinterpret_cast<const f32x4*>(s_gam + f0 + 4 * q);
        const f32x4 bq = *reinterpret_cast<const f32x4*>(s_bet + f0 + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; e++) { gam[4 * q + e] = gq[e]; bet[4 * q + e] = bq[e]; }
      }
      float s1 = 0.f, s2 = 0.f;
      float gx[8];
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float xh = z[e] * rstd;
        const float go = __builtin_fmaf(gam[e], xh, bet[e]) - (bf2f(vv[e]) - bf2f(kv[e]));
        z[e] = xh;
        gx[e] = go * gam[e];
        s1 += gx[e];
        s2 = __builtin_fmaf(gx[e], xh, s2);
      }
      s1 = oct_sum(s1);
      s2 = oct_sum(s2);
      const float scale = -bf2f(s_eta[tok]) * rstd * (1.f / FD);  // G2 = -eta * dl/dZ2
      bf16x8 o, ol;
#pragma unroll
      for (int e = 0; e < 8; e++) gx[e] = (FD * gx[e] - s1 - z[e] * s2) * scale;
      ln_token_sum_store(reinterpret_cast<float*>(smem + SM_B2P) + v * FD, gx, lane, f0);   // b2's step, this wave's share
      split8(gx, o, ol);
      lds_put16(s_g2 + tok * FLD + f0, __builtin_bit_cast(u32x4, o));
      lds_put16(s_g2l + tok * FLD + f0, __builtin_bit_cast(u32x4, ol));
    }
    TTT_STAGE(FS_LN);
    __syncthreads();

    TTT_STAGE(FS_LN_BARRIER);
    // b2 += sum over the tokens of G2: the eight waves' fp32 shares, added in a fixed order by wave 0 (read again
    // after the next workgroup barrier at the earliest)
    if (v == 0) {
      LANE_VARS;
      const float* part = reinterpret_cast<const float*>(smem + SM_B2P);
      float b = s_b2[lane];
#pragma unroll
      for (int u = 0; u < FW_NWAVE; u++) b += part[u * FD + lane];
      s_b2[lane] = b;
      if constexpr (ROLE == 1) gB[HID + lane] = b;
    }
    // ---- G1 = (G2 W2^T) * gelu'(Z1);  state += X^T G
    {
      LANE_VARS;
      // g1 = G2 W2^T: G2 rows from LDS (lane = tok, contraction = F); W2 as (lane = hid, contraction = F): the two
      // terms of W2s, written as rows [F][hid] into two wave-private tiles and read back transposed.  The tiles sit in
      // this wave's own part of the pair-sum tile (the part it writes when it gives; dead from the barrier above
      // until this wave's next pair sum).
      AccT<2, 1> g1;
      acc_zero(g1);
      {
        OpdT<1, 4> wh, wl;
        {
          constexpr int LDT = 2 * LDP, LDU = 2 * LDP;       // row stride (bf16 elements): a row of the pair-sum tile
          bf16* const t_hi = reinterpret_cast<bf16*>(s_Pp) + 64 * (1 - pr);   // 64 of the row's elements are this wave's:
          bf16* const t_lo = t_hi + 32;                                       // 32 for each term
#pragma unroll
          for (int fb = 0; fb < 2; fb++)
#pragma unroll
            for (int s = 0; s < 2; s++) {
              bf16x8 ph, pl;
              split8(W2s.b[0][fb], s, ph, pl);
              store_piece_rows<LDT>(t_hi, fb, s, c, h, ph);
              store_piece_rows<LDU>(t_lo, fb, s, c, h, pl);
            }
          TTT_WAVE_SYNC();
#pragma unroll
          for (int s = 0; s < 4; s++) {
            wh.v[0][s] = piece_tr<LDT>(t_hi, 0, s, lane);
            wl.v[0][s] = piece_tr<LDU>(t_lo, 0, s, lane);
          }
        }
#pragma unroll
        for (int s = 0; s < 4; s++) {
          bf16x8 ah[2], al[2];
#pragma unroll
          for (int rb = 0; rb < 2; rb++) {
            ah[rb] = piece_rows<FLD>(s_g2, rb, s, c, h);
            al[rb] = piece_rows<FLD>(s_g2l, rb, s, c, h);
          }
#pragma unroll
          for (int rb = 0; rb < 2; rb++) {
            g1.b[rb][0] = MFMA(al[rb], wh.v[0][s], g1.b[rb][0]);
            g1.b[rb][0] = MFMA(ah[rb], wl.v[0][s], g1.b[rb][0]);
            g1.b[rb][0] = MFMA(ah[rb], wh.v[0][s], g1.b[rb][0]);
          }
        }
      }
      TTT_STAGE(FS_F3);
      float colsum = 0.f;
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          g1.b[rb][0][i] *= d1.b[rb][0][i];
          colsum += g1.b[rb][0][i];
        }
      b1L += half_sum(colsum);
      {   // W1[:,shard] += XK^T G1, G1 chained in two terms (lane = hid, contraction = tok)
        OpdT<1, 4> g1h, g1l;
        cvt_chain_split(g1, g1h, g1l);
#pragma unroll
        for (int s = 0; s < 4; s++) {
          bf16x8 xk[2];
#pragma unroll
          for (int fb = 0; fb < 2; fb++) xk[fb] = xpiece_tr(s_xk, fb, s, lane);      // lane = F, contraction = tok
#pragma unroll
          for (int fb = 0; fb < 2; fb++) {
            W1s.b[fb][0] = MFMA(xk[fb], g1l.v[0][s], W1s.b[fb][0]);
            W1s.b[fb][0] = MFMA(xk[fb], g1h.v[0][s], W1s.b[fb][0]);
          }
        }
      }
      TTT_STAGE(FS_F4);
      // W2[shard,:] += X2^T G2: X2 chained (two terms), G2 through the transposing read
      // (lane = F, contraction = tok; two terms)
#pragma unroll
      for (int s = 0; s < 4; s++) {
        bf16x8 gh[2], gl[2];
#pragma unroll
        for (int fb = 0; fb < 2; fb++) {
          gh[fb] = piece_tr<FLD>(s_g2, fb, s, lane);
          gl[fb] = piece_tr<FLD>(s_g2l, fb, s, lane);
        }
        const bf16x8 xh = piece_rows<FLD>(s_x2t, 0, s, c, h), xl = x2lo.v[0][s];
#pragma unroll
        for (int fb = 0; fb < 2; fb++) {
          W2s.b[0][fb] = MFMA(xl, gh[fb], W2s.b[0][fb]);
          W2s.b[0][fb] = MFMA(xh, gl[fb], W2s.b[0][fb]);
          W2s.b[0][fb] = MFMA(xh, gh[fb], W2s.b[0][fb]);
        }
      }
    }
    TTT_STAGE(FS_F5);
    if constexpr (ROLE != 1) {
      LANE_VARS;
      if (h == 0) s_b1[hid0 + c] = b1L;      // read back below by this wave only
    }
    TTT_WAVE_SYNC();

    if constexpr (ROLE == 1) {
      // ---- hand the state after this mini-batch to the output branch: W1s and W2s exactly as the
      //      post-update forward would convert them, and the two bias vectors
      LANE_VARS;
      // the next mini-batch's inputs, under way to LDS since the LayerNorm stage, have arrived before the barrier
      // that opens the next mini-batch
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      const gptr_t gImg = gbuf(p.state_img + ((size_t)bh * 2 * FWD_RING_MAX + slot) * (FWD_IMG_BYTES / 2));
      const OpdT<1, 4> w1A = cvt_chain(W1s);
      const OpdT<2, 2> w2A = cvt_chain(W2s);
#pragma unroll
      for (int s = 0; s < 4; s++) g_st_stream<bf16x8>(gImg, 16 * tid, s * 8192, w1A.v[0][s]);   // read once, by another CU
#pragma unroll
      for (int fb = 0; fb < 2; fb++)
#pragma unroll
        for (int s = 0; s < 2; s++) g_st_stream<bf16x8>(gImg, 16 * tid, (4 + 2 * fb + s) * 8192, w2A.v[fb][s]);
      if (h == 0) gB[hid0 + c] = b1L;
      TTT_STAGE(FS_HANDOVER);
      if (at == ring - 1 || mb == p.NC - 1) publish(w_given, grp + 1);
      TTT_STAGE(FS_PUBLISH);
      continue;
    }

    // ---- post-update forward on XQ, transposed: Z1b^T = W1s^T XQ^T (rows hid, lane = tok)
    {
      LANE_VARS;
      const OpdT<1, 4> w1A = cvt_chain(W1s);
      const OpdT<2, 4> xqB = x_rows_kappa(s_xq, c, h);
      AccT<1, 2> z1b;
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x4 bv = *reinterpret_cast<const f32x4*>(s_b1 + hid0 + 8 * g + 4 * h);
#pragma unroll
        for (int cb = 0; cb < 2; cb++)
#pragma unroll
          for (int e = 0; e < 4; e++) z1b.b[0][cb][4 * g + e] = bv[e];
      }
      mma(z1b, w1A, xqB);
#pragma unroll
      for (int cb = 0; cb < 2; cb++)
#pragma unroll
        for (int i = 0; i < 16; i++) z1b.b[0][cb][i] = gelu_f(z1b.b[0][cb][i]);
      const OpdT<2, 2> x2bB = cvt_chain(z1b);      // lane = tok, contraction = hid
      auto z2_block = [&](const f32x16& w2) {      // one F block of W2s^T X2b^T: rows F, lane = tok
        AccT<1, 2> z;
        acc_zero(z);
#pragma unroll
        for (int s = 0; s < 2; s++) {
          const bf16x8 wa = pack8(w2, s);
#pragma unroll
          for (int cb = 0; cb < 2; cb++) z.b[0][cb] = MFMA(wa, x2bB.v[cb][s], z.b[0][cb]);
        }
        return z;
      };
      pair_sum_halves(s_Pp, [&]() { return z2_block(W2s.b[0][0]); }, [&]() { return z2_block(W2s.b[0][1]); }, pr, c, h);
    }

    TTT_STAGE(FS_OUT_FORWARD);
    // ---- output LayerNorm + residual, 8 tokens per wave.  XK / XV / eta were last read before the pair sum
    //      above: the next mini-batch's leave HBM for LDS now.
    {
      LANE_VARS;
      if (mb + 1 < mb1) {
        tile_to_lds(gXK, (mb + 1) * TILE_BYTES, smem + SM_XK, v, lane);
        tile_to_lds(gXV, (mb + 1) * TILE_BYTES, smem + SM_XV, v, lane);
        eta_to_lds(gEta, (mb + 1) * (CS * 2), smem + SM_ETA, v, lane);
      }
      output_layernorm(s_P, s_b2, s_gam, s_bet, s_xq, gOut, mb, tok, f0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the next mini-batch's inputs have arrived in LDS
    __syncthreads();
    TTT_STAGE(FS_OUT_LN);
  }
  // a segment that is not the sequence's last leaves the checkpoint the next one starts from (b2 in LDS: every wave is
  // past the barrier that closes the last mini-batch)
  if (mb1 < p.NC) store_checkpoint(mb1 / p.cgs);
  TTT_STAGES_END(p.stage_clocks == nullptr ? nullptr : p.stage_clocks + ((size_t)bh * 2 + 0) * (FW_NWAVE * STAGE_SLOTS));
}

// The output branch of the forward on its own workgroup: Out[mb] = XQ + LN(gelu(XQ W1' + b1') W2' + b2')
// with the state after mini-batch mb, taken from the operand images the recurrence leaves behind.  Nothing
// is carried from one mini-batch to the next here.
template <int RING>
TTT_DEV void fwd_output_branch(const FwdParams& p, unsigned char* smem, const int bh) {
  float* s_P = reinterpret_cast<float*>(smem + SM_P);
  float* s_b1 = reinterpret_cast<float*>(smem + SM_B1);
  float* s_b2 = reinterpret_cast<float*>(smem + SM_B2);   // two buffers: the second takes the place of the eta vector
  static_assert(SM_ETA == SM_B2 + FD * 4, "the second b2 buffer aliases the eta vector");
  float* s_gam = reinterpret_cast<float*>(smem + SM_GAM);
  float* s_bet = reinterpret_cast<float*>(smem + SM_BET);
  const int tid = threadIdx.x, lane = tid & 63;
  const int v = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pr = v >> 2;
  const int head = bh % p.NH;
  const int hid0 = FW_NS * v;
  float* s_Pp = s_P + (v & 3) * 64 * LDP;
  int lane_v = lane;
  if (tid < FD) {
    s_gam[tid] = p.ttt_norm_weight[head * FD + tid];
    s_bet[tid] = p.ttt_norm_bias[head * FD + tid];
  }
  const size_t x_base = uni64((size_t)bh * p.NC * (CS * FD));
  const gptr_t gXQ = gbuf(p.XQ + x_base), gOut = gbuf(p.Out + x_base);
  int* const w_given = p.sync + (size_t)bh * BWD_SYNC_STRIDE;
  int* const w_taken = w_given + 16;
  int* const w_status = p.status;
  int* const s_flag = reinterpret_cast<int*>(smem + SM_FLAG);

  TTT_STAGES_BEGIN();
  for (int mb = 0; mb < p.NC; mb++) {
    LANE_VARS;
    constexpr int ring = RING; const int grp = mb / ring, at = mb % ring, slot = (grp & 1) * ring + at;
    if (at == 0) {
      if (!wait_at_least(w_given, grp + 1, w_status, s_flag, p.wait_limit)) return;
    }
    bf16* s_xq = reinterpret_cast<bf16*>(smem + SM_XQ + (mb & 1) * SM_TILE);
    const gptr_t gImg = gbuf(p.state_img + ((size_t)bh * 2 * FWD_RING_MAX + slot) * (FWD_IMG_BYTES / 2));
    const float* gB = p.bias_img + ((size_t)bh * 2 * FWD_RING_MAX + slot) * FWD_BIAS_FLOATS;
    {
      LANE_VARS;
      // XQ and b2 alternate between two LDS buffers: other waves may still be in the previous mini-batch's
      // LayerNorm, which reads both.  (b1 is read before the pair sum's barriers only.)
      const u32x4 q = g_ld16(gXQ, 16 * tid, mb * TILE_BYTES);
      float bv = 0.f;
      if (tid < FWD_BIAS_FLOATS) bv = gB[tid];
      lds_put16(smem + SM_XQ + (mb & 1) * SM_TILE + (xrow(tid >> 3) + (tid & 7) * 8) * 2, q);
      if (tid < HID) s_b1[tid] = bv;
      else if (tid < FWD_BIAS_FLOATS) s_b2[(mb & 1) * FD + tid - HID] = bv;
    }
    __syncthreads();   // XQ and the biases are visible; the previous mini-batch's readers of s_P are done
    TTT_STAGE(FS_TOP);
    {
      LANE_VARS;
      OpdT<1, 4> w1A;
      OpdT<2, 2> w2A;
#pragma unroll
      for (int s = 0; s < 4; s++) w1A.v[0][s] = g_ld_stream<bf16x8>(gImg, 16 * tid, s * 8192);
#pragma unroll
      for (int fb = 0; fb < 2; fb++)
#pragma unroll
        for (int s = 0; s < 2; s++) w2A.v[fb][s] = g_ld_stream<bf16x8>(gImg, 16 * tid, (4 + 2 * fb + s) * 8192);
      const OpdT<2, 4> xqB = x_rows_kappa(s_xq, c, h);
      AccT<1, 2> z1b;
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x4 bv = *reinterpret_cast<const f32x4*>(s_b1 + hid0 + 8 * g + 4 * h);
#pragma unroll
        for (int cb = 0; cb < 2; cb++)
#pragma unroll
          for (int e = 0; e < 4; e++) z1b.b[0][cb][4 * g + e] = bv[e];
      }
      mma(z1b, w1A, xqB);
#pragma unroll
      for (int cb = 0; cb < 2; cb++)
#pragma unroll
        for (int i = 0; i < 16; i++) z1b.b[0][cb][i] = gelu_f(z1b.b[0][cb][i]);
      const OpdT<2, 2> x2bB = cvt_chain(z1b);      // lane = tok, contraction = hid
      AccT<2, 2> z2;
      acc_zero(z2);
      mma(z2, w2A, x2bB);                          // rows F, lane = tok
      pair_sum_to_lds(s_Pp, z2, pr, c, h);
    }
    TTT_STAGE(FS_OUT_FORWARD);
    {
      LANE_VARS;
      output_layernorm(s_P, s_b2 + (mb & 1) * FD, s_gam, s_bet, s_xq, gOut, mb, tok, f0);
    }
    TTT_STAGE(FS_OUT_LN);
    if (at == ring - 1 || mb == p.NC - 1) publish(w_taken, grp + 1);
    TTT_STAGE(FS_PUBLISH);
  }
  TTT_STAGES_END(p.stage_clocks == nullptr ? nullptr : p.stage_clocks + ((size_t)bh * 2 + 1) * (FW_NWAVE * STAGE_SLOTS));
#undef LANE_VARS
}

__global__ __launch_bounds__(FW_THREADS) void ttt_mlp_fwd_kernel(const FwdParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  int bh = p.bh0 + blockIdx.x, mb0 = 0, mb1 = p.NC;
  if (p.seg_len > 0) {
    const int pairs = p.B * p.NH, job = p.job0 + blockIdx.x, seg = job / pairs;
    bh = job - seg * pairs;
    mb0 = seg * p.seg_len;
    mb1 = mb0 + p.seg_len < p.NC ? mb0 + p.seg_len : p.NC;
  }
  fwd_body<0, 8>(p, smem, bh, mb0, mb1);
}

// Two workgroups per (batch, head), placed like those of the backward (same XCD where the count allows).
// RING = mini-batches per hand-over: each hand-over costs a release (an L2 write-back), and the output branch
// ends that many mini-batches after the recurrence; 32 pays from a few hundred mini-batches on (measured).
template <int RING>
__global__ __launch_bounds__(FW_THREADS) void ttt_mlp_fwd_split_kernel(const FwdParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int b = blockIdx.x;
  int bh, role;
  if (p.nbh % 8 == 0) {
    bh = (b >> 4) * 8 + (b & 7);
    role = (b >> 3) & 1;
  } else {
    bh = b >> 1;
    role = b & 1;
  }
  bh += p.bh0;
  if (role == 0) fwd_body<1, RING>(p, smem, bh, 0, p.NC);
  else fwd_output_branch<RING>(p, smem, bh);
}

__global__ void ttt_mlp_fwd_zero_words(int* w, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) w[i] = 0;
}

}  // namespace ttt

extern "C" int ttt_mlp_fwd_lds_bytes() { return ttt::SM_FWD_BYTES; }
extern "C" int ttt_mlp_fwd_threads() { return ttt::FW_THREADS; }

hipError_t ttt_mlp_fwd_clear_words(int* words, int n, hipStream_t stream) {
  hipLaunchKernelGGL(ttt::ttt_mlp_fwd_zero_words, dim3((n + 255) / 256), dim3(256), 0, stream, words, n);
  return hipGetLastError();
}

hipError_t ttt_mlp_fwd_enqueue(const ttt::FwdParams& p, hipStream_t stream) {
  // Per-device attribute; cheap enough to set on every launch.
  if (p.sync == nullptr) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(ttt::ttt_mlp_fwd_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, ttt::SM_FWD_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(ttt::ttt_mlp_fwd_kernel, dim3(p.nbh), dim3(ttt::FW_THREADS), ttt::SM_FWD_BYTES, stream, p);
    return hipGetLastError();
  }
  const void* kernel = p.ring_log2 == 5 ? reinterpret_cast<const void*>(ttt::ttt_mlp_fwd_split_kernel<32>)
                                        : reinterpret_cast<const void*>(ttt::ttt_mlp_fwd_split_kernel<8>);
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, ttt::SM_FWD_BYTES);
  if (e != hipSuccess) return e;
  const int n = static_cast<int>(ttt::bwd_sync_ints(p.nbh));
  int* const words = p.status - (size_t)p.nbh * ttt::BWD_SYNC_STRIDE;   // p.sync itself is moved back by bh0 entries
  hipLaunchKernelGGL(ttt::ttt_mlp_fwd_zero_words, dim3((n + 255) / 256), dim3(256), 0, stream, words, n);
  if (p.ring_log2 == 5)
    hipLaunchKernelGGL(ttt::ttt_mlp_fwd_split_kernel<32>, dim3(2 * p.nbh), dim3(ttt::FW_THREADS), ttt::SM_FWD_BYTES, stream, p);
  else
    hipLaunchKernelGGL(ttt::ttt_mlp_fwd_split_kernel<8>, dim3(2 * p.nbh), dim3(ttt::FW_THREADS), ttt::SM_FWD_BYTES, stream, p);
  return hipGetLastError();
}
