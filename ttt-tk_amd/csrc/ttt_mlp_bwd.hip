// Remat backward of the non-causal TTT-MLP layer for gfx950 (MI355X).
//
// Behaviour follows the upstream operator `ttt_backward` (kernel kernels/ttt_backward/ttt.cu:179-1443,
// mathematics kernels/ttt_backward/matching.py:57-342, group walk :539-663): for every checkpoint
// group, last to first, the forward is replayed from the checkpoint while the per-mini-batch
// activations are saved, then the group is walked backwards producing the ten output gradients.
//
// Mapping: one workgroup of 4 wavefronts per (batch, head); wave w owns hidden columns [64w, 64w+64).
// All [tokens x hidden] activations live in registers in the "Q" orientation (accumulator rows =
// hidden, lane = token), so per-token scalars (eta, dEta partial sums) are per-lane values and sums
// over the hidden dimension are in-register sums.  An activation that is also needed with tokens as
// the contraction index is bounced once through a wave-private LDS tile (row store + transposing read).
//
// State in registers:
//   replay : W1s [F x hid], W2s [hid x F], W2t [F x hid] (fp32 accumulator tiles); b1, b2 in LDS
//   reverse: gW1s [F x hid], gW2s [hid x F] (running gradients) only; gb1, gb2 in LDS.  The weights
//            enter the reverse walk as ready-made bf16 MFMA operands: after every mini-batch the replay
//            stores the operand images of W1^T[shard] and W2[shard]^T, and the walk reads the image of
//            the state after and before the step (before the first step of a group: converted straight
//            from the fp32 checkpoint).  Half the accumulator file therefore stays free for products.
// While a group is replayed the running gradients are parked in the caller's W*_init_group scratch.
// Saved per mini-batch (caller's *_group scratch): Z1 and Z1_bar as bf16 register images (Z1_group,
// Z1_bar_group); the two weight operand images (X2_group: W1^T[shard], grad_l_wrt_Z1_group:
// W2[shard]^T); x_hat / grad_output of the fused LayerNorm loss, dl/dZ2 and the output LayerNorm's
// x_hat as bf16 [tok][F] tiles; the two std vectors in fp32.
#include "ttt_mlp_common.hpp"
#include "ttt_mlp_kernels.hpp"

namespace ttt {

constexpr int SB_TILE = 64 * LDB * 2;
constexpr int SB_XQ = 0;                  // reverse: XQ until the post-update stage is done, then (with SB_E2)
constexpr int SB_E2 = SB_XQ + SB_TILE;    //          the fp32 park of g_y ; replay: XQ and XV
constexpr int SB_XK = SB_E2 + SB_TILE;
constexpr int SB_GZ2 = SB_XK + SB_TILE;   // replay: G2 = -eta*dl/dZ2 ; reverse: raw dl/dZ2
constexpr int SB_A = SB_GZ2 + SB_TILE;    // reverse: gZ2_bar, later dZ2
static_assert(2 * SB_TILE >= CS * FD * 4, "g_y park does not fit");
constexpr int SB_P = SB_A + SB_TILE;      // 4 fp32 partial tiles
constexpr int SB_PTILE = 64 * LDP * 4;
constexpr int SB_BNC = SB_P + 4 * SB_PTILE;   // 4 wave-private bounce tiles
constexpr int SB_B1 = SB_BNC + 4 * SB_TILE;   // b1 during a replay, 256 floats
constexpr int SB_B2 = SB_B1 + HID * 4;        // b2 during a replay, 64 floats
constexpr int SB_GB1 = SB_B2 + FD * 4;        // running gradient wrt b1
constexpr int SB_GB2 = SB_GB1 + HID * 4;      // running gradient wrt b2
constexpr int SB_GAM = SB_GB2 + FD * 4;       // ttt_norm_weight of this head
constexpr int SB_BET = SB_GAM + FD * 4;       // ttt_norm_bias of this head
constexpr int SB_ETA = SB_BET + FD * 4;
constexpr int SB_DETA = SB_ETA + CS * 4;      // [2][4 waves][64 tokens] partial dEta sums
constexpr int SB_RED = SB_DETA + 2 * 4 * CS * 4;  // [4 waves][2][64] final norm-grad reduction
constexpr int SM_BWD_BYTES = SB_RED + 4 * 2 * FD * 4;
static_assert(SM_BWD_BYTES <= 160 * 1024, "LDS budget of one gfx950 CU exceeded");

// Orders a wave-private LDS store against the transposing read that follows it.  LDS operations of
// one wave execute in issue order, so only the compiler has to be kept from reordering them.
#define WAVE_SYNC()                                        \
  do {                                                     \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); \
    __builtin_amdgcn_wave_barrier();                       \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront"); \
  } while (0)

// ------------------------------------------------------------------ register images in HBM
// A 64x64 tile as 8 chunks of 8 bf16 per lane; chunk n of thread tid sits at (n*256 + tid)*16 bytes,
// so every store/load instruction of a wave moves 1 KiB contiguous.
TTT_DEV void opd_store(bf16* base, const Opd& o, int tid) {
#pragma unroll
  for (int cb = 0; cb < 2; cb++)
#pragma unroll
    for (int s = 0; s < 4; s++) reinterpret_cast<bf16x8*>(base)[(cb * 4 + s) * NTHREADS + tid] = o.v[cb][s];
}
TTT_DEV Opd opd_load(const bf16* base, int tid) {
  Opd o;
#pragma unroll
  for (int cb = 0; cb < 2; cb++)
#pragma unroll
    for (int s = 0; s < 4; s++) o.v[cb][s] = reinterpret_cast<const bf16x8*>(base)[(cb * 4 + s) * NTHREADS + tid];
  return o;
}
TTT_DEV void img_store(bf16* base, const Acc& x, int tid) { opd_store(base, cvt_chain(x), tid); }
// Sign flip of every element (exact).
TTT_DEV Opd opd_neg(const Opd& o) {
  Opd r;
#pragma unroll
  for (int cb = 0; cb < 2; cb++)
#pragma unroll
    for (int s = 0; s < 4; s++) {
      u32x4 u = __builtin_bit_cast(u32x4, o.v[cb][s]);
      u ^= 0x80008000u;
      r.v[cb][s] = __builtin_bit_cast(bf16x8, u);
    }
  return r;
}
TTT_DEV void img_load(const bf16* base, Acc& x, int tid) {
#pragma unroll
  for (int cb = 0; cb < 2; cb++)
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const bf16x8 v = reinterpret_cast<const bf16x8*>(base)[(cb * 4 + s) * NTHREADS + tid];
#pragma unroll
      for (int j = 0; j < 8; j++) x.b[s >> 1][cb][8 * (s & 1) + j] = (float)v[j];
    }
}

// fp32 accumulator tile <-> HBM in the caller's row-major layout.  `ld` = row length, (r0, c0) =
// origin of this wave's 64x64 block; accumulator rows are tensor rows.
TTT_DEV void acc_load_rows(Acc& a, const float* g, int ld, int r0, int c0, int c, int h) {
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int cb = 0; cb < 2; cb++)
#pragma unroll
      for (int i = 0; i < 16; i++)
        a.b[rb][cb][i] = g[(size_t)(r0 + 32 * rb + 8 * (i >> 2) + 4 * h + (i & 3)) * ld + c0 + 32 * cb + c];
}
TTT_DEV void acc_store_rows(const Acc& a, float* g, int ld, int r0, int c0, int c, int h) {
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int cb = 0; cb < 2; cb++)
#pragma unroll
      for (int i = 0; i < 16; i++)
        g[(size_t)(r0 + 32 * rb + 8 * (i >> 2) + 4 * h + (i & 3)) * ld + c0 + 32 * cb + c] = a.b[rb][cb][i];
}
// Same, but accumulator rows are tensor COLUMNS (the tile holds the transpose of the block).
TTT_DEV void acc_load_cols(Acc& a, const float* g, int ld, int r0, int c0, int c, int h) {
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int cb = 0; cb < 2; cb++)
#pragma unroll
      for (int i = 0; i < 16; i++)
        a.b[rb][cb][i] = g[(size_t)(r0 + 32 * cb + c) * ld + c0 + 32 * rb + 8 * (i >> 2) + 4 * h + (i & 3)];
}
// Bias vector in accumulator-row form: element of row r, identical in every lane column.
TTT_DEV void rowvec_load(f32x16 (&v)[2], const float* g, int h) {
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int i = 0; i < 16; i++) v[rb][i] = g[32 * rb + 8 * (i >> 2) + 4 * h + (i & 3)];
}
TTT_DEV void rowvec_store(const f32x16 (&v)[2], float* g, int h) {  // call from lanes with c == 0
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int i = 0; i < 16; i++) g[32 * rb + 8 * (i >> 2) + 4 * h + (i & 3)] = v[rb][i];
}
TTT_DEV void rowvec_store_lds(const f32x16 (&v)[2], float* s, int h) {  // call from lanes with c == 0
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      f32x4 x = {v[rb][4 * g], v[rb][4 * g + 1], v[rb][4 * g + 2], v[rb][4 * g + 3]};
      *reinterpret_cast<f32x4*>(s + 32 * rb + 8 * g + 4 * h) = x;
    }
}
// v[row block] += sum over the 64-long contraction of operand `a` (lane = row index).
TTT_DEV void rowsum_mma(f32x16 (&v)[2], const Opd& a, bf16x8 ones) {
#pragma unroll
  for (int s = 0; s < 4; s++)
#pragma unroll
    for (int rb = 0; rb < 2; rb++) v[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v[rb][s], ones, v[rb], 0, 0, 0);
}
TTT_DEV void acc_init_rowvec(Acc& a, const f32x16 (&v)[2]) {
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int cb = 0; cb < 2; cb++) a.b[rb][cb] = v[rb];
}
// Swap the roles of lane index and contraction index of an operand through a wave-private tile.
TTT_DEV Opd bounce(bf16* tile, const Opd& o, int lane) {
  WAVE_SYNC();  // earlier readers of the tile are done
  lds_store_rows_kappa(tile, o, lane & 31, lane >> 5);
  WAVE_SYNC();
  return lds_tr_kappa(tile, lane);
}
TTT_DEV void acc_scale(Acc& a, float s) {
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int cb = 0; cb < 2; cb++)
#pragma unroll
      for (int i = 0; i < 16; i++) a.b[rb][cb][i] *= s;
}

// Sum over the 16 lanes of a wave that share lane % 4 (the 16 tokens of a LayerNorm stage), result in
// all of them: two row rotations inside each row of 16 lanes, then across the four rows.
TTT_DEV float token_sum16(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x124, 0xF, 0xF, false));  // row_ror:4
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128, 0xF, 0xF, false));  // row_ror:8
  x += __shfl_xor(x, 16, 64);
  x += __shfl_xor(x, 32, 64);
  return x;
}
// acc[16r + 4fq + e] += sum over this wave's tokens of x[r][e]   (wave-private LDS vector)
TTT_DEV void ln_token_sum_add(float* s_acc, const float (&x)[4][4], int q, int fq) {
#pragma unroll
  for (int r = 0; r < 4; r++) {
    f32x4 v;
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = token_sum16(x[r][e]);
    if (q == 0) {
      f32x4* d = reinterpret_cast<f32x4*>(s_acc + 16 * r + 4 * fq);
      *d = *d + v;
    }
  }
}

// ------------------------------------------------------------------ LayerNorm-lane helpers
// A lane of the LayerNorm stage owns token `tok` and features 16r + 4fq + e (r, e in 0..3).
TTT_DEV void ln_load(float (&x)[4][4], const bf16* row, int fq) {
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const bf16x4 v = *reinterpret_cast<const bf16x4*>(row + 16 * r + 4 * fq);
#pragma unroll
    for (int e = 0; e < 4; e++) x[r][e] = (float)v[e];
  }
}
TTT_DEV void ln_store(bf16* row, const float (&x)[4][4], int fq) {
#pragma unroll
  for (int r = 0; r < 4; r++) {
    bf16x4 v;
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = (bf16)x[r][e];
    *reinterpret_cast<bf16x4*>(row + 16 * r + 4 * fq) = v;
  }
}
// dst = bf16(float(dst) + x): the operator accumulates into these outputs.
TTT_DEV void ln_accumulate(bf16* row, const float (&x)[4][4], int fq) {
#pragma unroll
  for (int r = 0; r < 4; r++) {
    bf16x4 v = *reinterpret_cast<const bf16x4*>(row + 16 * r + 4 * fq);
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = (bf16)((float)v[e] + x[r][e]);
    *reinterpret_cast<bf16x4*>(row + 16 * r + 4 * fq) = v;
  }
}
// Sum of the 4 shard partial tiles (plus a bias vector) for this lane's 16 features.
TTT_DEV void ln_gather(float (&z)[4][4], const float* s_P, const float* s_bias, int tok, int fq) {
#pragma unroll
  for (int r = 0; r < 4; r++) {
    f32x4 a = *reinterpret_cast<const f32x4*>(s_bias + 16 * r + 4 * fq);
#pragma unroll
    for (int v = 0; v < 4; v++) a += *reinterpret_cast<const f32x4*>(s_P + v * 64 * LDP + tok * LDP + 16 * r + 4 * fq);
#pragma unroll
    for (int e = 0; e < 4; e++) z[r][e] = a[e];
  }
}
TTT_DEV float sum16(const float (&x)[4][4]) {
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int e = 0; e < 4; e++) s += x[r][e];
  return s;
}
TTT_DEV float dot16(const float (&x)[4][4], const float (&y)[4][4]) {
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int e = 0; e < 4; e++) s = __builtin_fmaf(x[r][e], y[r][e], s);
  return s;
}
// z -> x_hat in place, returns 1/std; *std_out = std.
TTT_DEV float ln_normalize(float (&z)[4][4], float* std_out) {
  const float mu = quad_sum(sum16(z)) * (1.f / FD);
  float var = 0.f;
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int e = 0; e < 4; e++) { z[r][e] -= mu; var = __builtin_fmaf(z[r][e], z[r][e], var); }
  const float v = quad_sum(var) * (1.f / FD) + LN_EPS;
  const float rstd = __builtin_amdgcn_rsqf(v);
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int e = 0; e < 4; e++) z[r][e] *= rstd;
  *std_out = v * rstd;  // sqrt(v)
  return rstd;
}

// 16-byte chunk staging of one [64][64] bf16 tile from HBM into an LDS tile with row stride LDB.
TTT_DEV void stage_tile(bf16* s_tile, const bf16* g_tile, int tid) {
#pragma unroll
  for (int r = 0; r < 2; r++) {
    const int id = tid + 256 * r;
    *reinterpret_cast<u32x4*>(s_tile + (id >> 3) * LDB + (id & 7) * 8) = reinterpret_cast<const u32x4*>(g_tile)[id];
  }
}

// C-init of a Q-orientation tile from an LDS vector indexed by accumulator row (64 floats).
TTT_DEV void acc_init_rows_lds(Acc& a, const float* s_vec, int h) {
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(s_vec + 32 * rb + 8 * g + 4 * h);
#pragma unroll
      for (int cb = 0; cb < 2; cb++)
#pragma unroll
        for (int e = 0; e < 4; e++) a.b[rb][cb][4 * g + e] = v[e];
    }
}
// s_vec[row] += sum over the contraction of operand `a` (lane = row index); the sum is formed on the
// matrix cores, lanes with c == 0 fold it into the LDS vector.
TTT_DEV void lds_rowsum_add(float* s_vec, const Opd& a, bf16x8 ones, int c, int h) {
  f32x16 t[2];
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int i = 0; i < 16; i++) t[rb][i] = 0.f;
  rowsum_mma(t, a, ones);
  if (c == 0) {
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        f32x4* q = reinterpret_cast<f32x4*>(s_vec + 32 * rb + 8 * g + 4 * h);
        f32x4 v = *q;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] += t[rb][4 * g + e];
        *q = v;
      }
  }
  // Other lanes of this wave read the vector next; without a fence the compiler may forward the
  // values each lane saw before the update.
  WAVE_SYNC();
}
TTT_DEV void ln_load_f32(float (&x)[4][4], const float* s_vec, int fq) {
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(s_vec + 16 * r + 4 * fq);
#pragma unroll
    for (int e = 0; e < 4; e++) x[r][e] = v[e];
  }
}
// Sum of the 4 shard partial tiles for this lane's 16 features.
TTT_DEV void ln_gather0(float (&z)[4][4], const float* s_P, int tok, int fq) {
#pragma unroll
  for (int r = 0; r < 4; r++) {
    f32x4 a = *reinterpret_cast<const f32x4*>(s_P + tok * LDP + 16 * r + 4 * fq);
#pragma unroll
    for (int v = 1; v < 4; v++) a += *reinterpret_cast<const f32x4*>(s_P + v * 64 * LDP + tok * LDP + 16 * r + 4 * fq);
#pragma unroll
    for (int e = 0; e < 4; e++) z[r][e] = a[e];
  }
}

// ---------------------------------------------------------------- just-in-time operand pieces
// One MFMA operand piece = 8 bf16 per lane = (free block blk, k-step s).  Loading pieces right
// before the MFMA that consumes them keeps whole 64x64 operands out of the register file.
constexpr int LDT = 68;   // row stride of the two operand tiles that share a wave's partial tile
template <int LD>
TTT_DEV bf16x8 piece_rows(const bf16* tile, int blk, int s, int c, int h) {
  const bf16* q = tile + (32 * blk + c) * LD + 16 * s + 4 * h;
  return cat(*reinterpret_cast<const bf16x4*>(q), *reinterpret_cast<const bf16x4*>(q + 8));
}
template <int LD>
TTT_DEV bf16x8 piece_tr(const bf16* tile, int blk, int s, int lane) {
  const int h = lane >> 5, c = lane & 31, i = lane & 15;
  const bf16* q = tile + (16 * s + 4 * h + (i >> 2)) * LD + 32 * blk + 16 * (c >> 4) + 4 * (i & 3);
  return cat(lds_tr4(q), lds_tr4(q + 8 * LD));
}
template <int LD>
TTT_DEV void store_piece_rows(bf16* tile, int blk, int s, int c, int h, bf16x8 v) {
  bf16* q = tile + (32 * blk + c) * LD + 16 * s + 4 * h;
  *reinterpret_cast<bf16x4*>(q) = __builtin_shufflevector(v, v, 0, 1, 2, 3);
  *reinterpret_cast<bf16x4*>(q + 8) = __builtin_shufflevector(v, v, 4, 5, 6, 7);
}
template <int LD>
TTT_DEV void store_opd_rows(bf16* tile, const Opd& o, int c, int h) {
#pragma unroll
  for (int fb = 0; fb < 2; fb++)
#pragma unroll
    for (int s = 0; s < 4; s++) store_piece_rows<LD>(tile, fb, s, c, h, o.v[fb][s]);
}
// Piece (free block fb, k-step s) of the chained operand of an accumulator tile.
TTT_DEV bf16x8 piece_state(const Acc& x, int fb, int s) { return pack8(x.b[s >> 1][fb], s & 1); }
template <int LD>
TTT_DEV void store_state_rows(bf16* tile, const Acc& x, int c, int h) {
#pragma unroll
  for (int fb = 0; fb < 2; fb++)
#pragma unroll
    for (int s = 0; s < 4; s++) store_piece_rows<LD>(tile, fb, s, c, h, piece_state(x, fb, s));
}
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16((a), (b), (c), 0, 0, 0)
// d += A * B, pieces produced by the callables fa(blk, s) and fb(blk, s).
template <class FA, class FB>
TTT_DEV void mma_jit(Acc& d, FA fa, FB fb) {
#pragma unroll
  for (int s = 0; s < 4; s++) {
    const bf16x8 a0 = fa(0, s), a1 = fa(1, s), b0 = fb(0, s), b1 = fb(1, s);
    d.b[0][0] = MFMA(a0, b0, d.b[0][0]);
    d.b[0][1] = MFMA(a0, b1, d.b[0][1]);
    d.b[1][0] = MFMA(a1, b0, d.b[1][0]);
    d.b[1][1] = MFMA(a1, b1, d.b[1][1]);
  }
}
// s_vec[row] += sum over the contraction of the operand whose pieces fa(rb, s) yields.
template <class FA>
TTT_DEV void lds_rowsum_add_jit(float* s_vec, FA fa, bf16x8 ones, int c, int h) {
  f32x16 t[2];
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int i = 0; i < 16; i++) t[rb][i] = 0.f;
#pragma unroll
  for (int s = 0; s < 4; s++)
#pragma unroll
    for (int rb = 0; rb < 2; rb++) t[rb] = MFMA(fa(rb, s), ones, t[rb]);
  if (c == 0) {
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        f32x4* q = reinterpret_cast<f32x4*>(s_vec + 32 * rb + 8 * g + 4 * h);
        f32x4 v = *q;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] += t[rb][4 * g + e];
        *q = v;
      }
  }
  WAVE_SYNC();
}

TTT_DEV bf16x8 cvt8(const f32x4 lo, const f32x4 hi) {
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 4; e++) { o[e] = (bf16)lo[e]; o[4 + e] = (bf16)hi[e]; }
  return o;
}
// MFMA operand (kappa order) straight from a row-major fp32 matrix: lane = row r0 + 32*fb + c,
// contraction = columns c0 .. c0+63.
TTT_DEV Opd opd_from_f32_rows(const float* g, int ld, int r0, int c0, int c, int h) {
  Opd o;
#pragma unroll
  for (int fb = 0; fb < 2; fb++)
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const float* q = g + (size_t)(r0 + 32 * fb + c) * ld + c0 + 16 * s + 4 * h;
      o.v[fb][s] = cvt8(*reinterpret_cast<const f32x4*>(q), *reinterpret_cast<const f32x4*>(q + 8));
    }
  return o;
}

// Three [64][64] bf16 tiles + the eta vector of one mini-batch in flight from HBM (per thread).
struct Staged3 {
  u32x4 a[2], b[2], c[2];
  float eta;
};
TTT_DEV void stage3_load(Staged3& s, const bf16* ga, const bf16* gb, const bf16* gc, const bf16* geta, size_t tile_off,
                         size_t eta_off, int tid) {
#pragma unroll
  for (int r = 0; r < 2; r++) {
    const int id = tid + 256 * r;
    s.a[r] = reinterpret_cast<const u32x4*>(ga + tile_off)[id];
    s.b[r] = reinterpret_cast<const u32x4*>(gb + tile_off)[id];
    s.c[r] = reinterpret_cast<const u32x4*>(gc + tile_off)[id];
  }
  s.eta = (tid < CS) ? bf2f(geta[eta_off + tid]) : 0.f;
}
TTT_DEV void stage3_store(const Staged3& s, bf16* sa, bf16* sb, bf16* sc, float* s_eta, int tid) {
#pragma unroll
  for (int r = 0; r < 2; r++) {
    const int id = tid + 256 * r;
    const int off = (id >> 3) * LDB + (id & 7) * 8;
    *reinterpret_cast<u32x4*>(sa + off) = s.a[r];
    *reinterpret_cast<u32x4*>(sb + off) = s.b[r];
    *reinterpret_cast<u32x4*>(sc + off) = s.c[r];
  }
  if (tid < CS) s_eta[tid] = s.eta;
}

__global__ __launch_bounds__(NTHREADS) void ttt_mlp_bwd_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
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
  float* s_deta = reinterpret_cast<float*>(smem + SB_DETA);
  float* s_red = reinterpret_cast<float*>(smem + SB_RED);

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, h = lane >> 5, c = lane & 31;
  const int q = lane >> 2, fq = lane & 3, tok = 16 * w + q;
  const int bh = blockIdx.x, head = bh % p.NH;
  float* s_Pw = s_P + w * 64 * LDP;
  bf16* s_bnc = reinterpret_cast<bf16*>(smem + SB_BNC) + w * 64 * LDB;
  float* s_b1w = s_b1 + 64 * w;
  float* s_gb1w = s_gb1 + 64 * w;
  const int cgs = p.cgs;

  if (tid < FD) {
    s_gam[tid] = p.ttt_norm_weight[head * FD + tid];
    s_bet[tid] = p.ttt_norm_bias[head * FD + tid];
    s_gb2[tid] = p.grad_L_b2_last[(size_t)bh * FD + tid];
  }
  s_gb1[tid] = p.grad_L_b1_last[(size_t)bh * HID + tid];
  // Norm-weight / norm-bias gradients accumulate per wave in LDS (summed over the wave's 16 tokens
  // with cross-lane adds in a fixed order); summed over the waves at the end.
  float* s_dgw = s_red + (w * 2 + 0) * FD;
  float* s_dbw = s_red + (w * 2 + 1) * FD;
  if (lane < FD) { s_dgw[lane] = 0.f; s_dbw[lane] = 0.f; }
  float* s_gy = reinterpret_cast<float*>(smem + SB_XQ) + tok * FD;   // this lane's row of the g_y park
  bf16x8 ones;
#pragma unroll
  for (int j = 0; j < 8; j++) ones[j] = (bf16)1.0f;

  const size_t x_base = (size_t)bh * p.NC * (CS * FD);
  const size_t eta_base = (size_t)bh * p.NC * CS;
  // per-(b,h) scratch bases
  const size_t g_TF = (size_t)bh * cgs * (CS * FD);     // [cgs][64][64] tiles
  const size_t g_TH = (size_t)bh * cgs * (CS * HID);    // [cgs][64][256] tiles (register images)
  const size_t g_T = (size_t)bh * cgs * CS;             // [cgs][64] vectors
  float* park_W1 = p.W1_init_group + (size_t)bh * cgs * FD * HID;
  float* park_W2 = p.W2_init_group + (size_t)bh * cgs * HID * FD;
  // During the reverse walk the same two 64 KiB slots park what must survive the LayerNorm stage.
  bf16* park_d1 = reinterpret_cast<bf16*>(park_W1);                  // 32 KiB register image
  bf16* park_t2 = park_d1 + CS * HID;                                // 32 KiB register image
  float* park_dk = park_W2 + (size_t)w * (CS * FD) ;                 // 16 KiB per wave

  // running gradients wrt the state after the last mini-batch
  Acc gW1s, gW2s;
  acc_load_rows(gW1s, p.grad_L_W1_last + (size_t)bh * FD * HID, HID, 0, 64 * w, c, h);
  acc_load_rows(gW2s, p.grad_L_W2_last + (size_t)bh * HID * FD, FD, 64 * w, 0, c, h);

  for (int k = p.K - 1; k >= 0; k--) {
    const int n_mb = min(cgs, p.NC - k * cgs);
    // ================================================================= replay
    {
      // park the running gradients while the forward state needs the registers
      acc_store_rows(gW1s, park_W1, HID, 0, 64 * w, c, h);
      acc_store_rows(gW2s, park_W2, FD, 64 * w, 0, c, h);
      Acc W1s, W2s, W2t;
      const size_t slot = (size_t)bh * p.K + k;
      acc_load_rows(W1s, p.W1_ck + slot * FD * HID, HID, 0, 64 * w, c, h);
      acc_load_rows(W2s, p.W2_ck + slot * HID * FD, FD, 64 * w, 0, c, h);
      acc_load_cols(W2t, p.W2_ck + slot * HID * FD, FD, 64 * w, 0, c, h);
      __syncthreads();  // previous group's readers of the bias vectors are done
      s_b1[tid] = p.b1_ck[slot * HID + tid];
      if (tid < FD) s_b2[tid] = p.b2_ck[slot * FD + tid];

      bf16* const T0 = s_bnc;                                   // wave-private tiles, as in the reverse walk
      bf16* const T1 = reinterpret_cast<bf16*>(s_Pw);
      bf16* const T2 = T1 + 64 * LDT;
      Staged3 st;
      stage3_load(st, p.XQ, p.XK, p.XV, p.last_eta, x_base + (size_t)(k * cgs) * (CS * FD), eta_base + (size_t)(k * cgs) * CS, tid);
      for (int j = 0; j < n_mb; j++) {
        const int mb = k * cgs + j;
        __syncthreads();
        stage3_store(st, s_xq, s_xk, s_e2, s_eta, tid);
        __syncthreads();

        // Z1^T = W1s^T XK^T + b1  (rows hid, lane = tok); X2 rows [tok][hid] -> T0, gelu'(Z1) packed
        Opd d1p;
        {
          Acc x2;
          acc_init_rows_lds(x2, s_b1w, h);
          mma_jit(x2, [&](int blk, int s) { return piece_state(W1s, blk, s); },
                  [&](int blk, int s) { return piece_rows<LDB>(s_xk, blk, s, c, h); });
          bf16* img = p.Z1_group + g_TH + (size_t)j * (CS * HID);
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
#pragma unroll
            for (int s = 0; s < 4; s++) {
              const bf16x8 z = pack8(x2.b[s >> 1][cb], s & 1);
              reinterpret_cast<bf16x8*>(img)[(cb * 4 + s) * NTHREADS + tid] = z;
              bf16x8 xv;
#pragma unroll
              for (int jj = 0; jj < 8; jj++) {
                float g, d;
                gelu_fd(x2.b[s >> 1][cb][8 * (s & 1) + jj], g, d);
                xv[jj] = (bf16)g;
                d1p.v[cb][s][jj] = (bf16)d;
              }
              store_piece_rows<LDB>(T0, cb, s, c, h, xv);
            }
        }
        WAVE_SYNC();
        {
          Acc z2;
          acc_zero(z2);
          mma_jit(z2, [&](int blk, int s) { return piece_state(W2s, blk, s); },                  // lane = F, contraction = hid
                  [&](int blk, int s) { return piece_rows<LDB>(T0, blk, s, c, h); });            // X2: lane = tok
          lds_store_partial(s_Pw, z2, c, h);
        }
        __syncthreads();
        // fused LayerNorm + reconstruction-loss gradient; saves for the reverse walk
        {
          float z[4][4], gam[4][4];
          ln_gather(z, s_P, s_b2, tok, fq);
          ln_load_f32(gam, s_gam, fq);
          float sd;
          const float rstd = ln_normalize(z, &sd);
          float go[4][4], gx[4][4];
          {
            float kv[4][4], vv[4][4], bet[4][4];
            ln_load(kv, s_xk + tok * LDB, fq);
            ln_load(vv, s_e2 + tok * LDB, fq);
            ln_load_f32(bet, s_bet, fq);
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
              for (int e = 0; e < 4; e++) {
                go[r][e] = __builtin_fmaf(gam[r][e], z[r][e], bet[r][e]) - (vv[r][e] - kv[r][e]);
                gx[r][e] = go[r][e] * gam[r][e];
              }
          }
          const size_t so = g_TF + (size_t)j * (CS * FD) + tok * FD;
          ln_store(p.x_hat_fused_group + so, z, fq);
          ln_store(p.grad_output_fused_group + so, go, fq);
          const float s1 = quad_sum(sum16(gx)), s2 = quad_sum(dot16(gx, z));
          const float sc = rstd * (1.f / FD), neg_eta = -s_eta[tok];
#pragma unroll
          for (int r = 0; r < 4; r++)
#pragma unroll
            for (int e = 0; e < 4; e++) gx[r][e] = (FD * gx[r][e] - s1 - z[r][e] * s2) * sc;   // dl/dZ2
          ln_store(p.grad_l_wrt_Z2_group + so, gx, fq);
#pragma unroll
          for (int r = 0; r < 4; r++)
#pragma unroll
            for (int e = 0; e < 4; e++) gx[r][e] *= neg_eta;                                   // G2
          ln_store(s_gz2 + tok * LDB, gx, fq);
          if (fq == 0) p.std_fused_group[g_T + (size_t)j * CS + tok] = sd;
        }
        __syncthreads();
        // G1 = (W2 G2^T) * gelu'(Z1)  (rows hid, lane = tok) -> T1 rows [tok][hid]; weight step
        {
          Acc g1;
          acc_zero(g1);
          mma_jit(g1, [&](int blk, int s) { return piece_state(W2t, blk, s); },                  // lane = hid, contraction = F
                  [&](int blk, int s) { return piece_rows<LDB>(s_gz2, blk, s, c, h); });         // G2: lane = tok
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
#pragma unroll
            for (int s = 0; s < 4; s++) {
              bf16x8 gv;
#pragma unroll
              for (int jj = 0; jj < 8; jj++) gv[jj] = (bf16)(g1.b[s >> 1][cb][8 * (s & 1) + jj] * (float)d1p.v[cb][s][jj]);
              store_piece_rows<LDT>(T1, cb, s, c, h, gv);
            }
        }
        WAVE_SYNC();
        mma_jit(W2s, [&](int blk, int s) { return piece_tr<LDB>(T0, blk, s, lane); },            // X2^T: lane = hid
                [&](int blk, int s) { return piece_tr<LDB>(s_gz2, blk, s, lane); });             // G2: lane = F
        mma_jit(W2t, [&](int blk, int s) { return piece_tr<LDB>(s_gz2, blk, s, lane); },
                [&](int blk, int s) { return piece_tr<LDB>(T0, blk, s, lane); });
        if (w == 0) lds_rowsum_add_jit(s_b2, [&](int blk, int s) { return piece_tr<LDB>(s_gz2, blk, s, lane); }, ones, c, h);
        mma_jit(W1s, [&](int blk, int s) { return piece_tr<LDB>(s_xk, blk, s, lane); },          // XK^T: lane = F
                [&](int blk, int s) { return piece_tr<LDT>(T1, blk, s, lane); });                // G1: lane = hid
        lds_rowsum_add_jit(s_b1w, [&](int blk, int s) { return piece_tr<LDT>(T1, blk, s, lane); }, ones, c, h);
        // operand images of the state after this step, for the reverse walk
        {
          bf16* img2 = p.grad_l_wrt_Z1_group + g_TH + (size_t)j * (CS * HID);   // W2: lane = hid, contraction = F
          bf16* img1 = p.X2_group + g_TH + (size_t)j * (CS * HID);              // W1^T: lane = F, contraction = hid
          store_state_rows<LDT>(T2, W1s, c, h);                                 // rows [hid][F]
#pragma unroll
          for (int fb = 0; fb < 2; fb++)
#pragma unroll
            for (int s = 0; s < 4; s++) reinterpret_cast<bf16x8*>(img2)[(fb * 4 + s) * NTHREADS + tid] = piece_state(W2t, fb, s);
          WAVE_SYNC();
#pragma unroll
          for (int fb = 0; fb < 2; fb++)
#pragma unroll
            for (int s = 0; s < 4; s++) reinterpret_cast<bf16x8*>(img1)[(fb * 4 + s) * NTHREADS + tid] = piece_tr<LDT>(T2, fb, s, lane);
        }
        // post-update forward on XQ
        {
          Acc z1b;
          acc_init_rows_lds(z1b, s_b1w, h);
          mma_jit(z1b, [&](int blk, int s) { return piece_state(W1s, blk, s); },
                  [&](int blk, int s) { return piece_rows<LDB>(s_xq, blk, s, c, h); });
          bf16* img = p.Z1_bar_group + g_TH + (size_t)j * (CS * HID);
          Opd x2bQ;
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
#pragma unroll
            for (int s = 0; s < 4; s++) {
              reinterpret_cast<bf16x8*>(img)[(cb * 4 + s) * NTHREADS + tid] = pack8(z1b.b[s >> 1][cb], s & 1);
#pragma unroll
              for (int jj = 0; jj < 8; jj++) x2bQ.v[cb][s][jj] = (bf16)gelu_f(z1b.b[s >> 1][cb][8 * (s & 1) + jj]);
            }
          Acc z2;
          acc_zero(z2);
          mma_jit(z2, [&](int blk, int s) { return piece_state(W2s, blk, s); },
                  [&](int blk, int s) { return x2bQ.v[blk][s]; });
          WAVE_SYNC();   // readers of T1 / T2 are done
          lds_store_partial(s_Pw, z2, c, h);
        }
        // inputs of the next mini-batch travel while the last LayerNorm stage runs
        if (j + 1 < n_mb)
          stage3_load(st, p.XQ, p.XK, p.XV, p.last_eta, x_base + (size_t)(mb + 1) * (CS * FD), eta_base + (size_t)(mb + 1) * CS, tid);
        __syncthreads();
        {
          float z[4][4];
          ln_gather(z, s_P, s_b2, tok, fq);
          float sd;
          ln_normalize(z, &sd);
          ln_store(p.x_hat_ln_group + g_TF + (size_t)j * (CS * FD) + tok * FD, z, fq);
          if (fq == 0) p.std_ln_group[g_T + (size_t)j * CS + tok] = sd;
        }
      }
      // running gradients back into registers
      acc_load_rows(gW1s, park_W1, HID, 0, 64 * w, c, h);
      acc_load_rows(gW2s, park_W2, FD, 64 * w, 0, c, h);
    }

    // ================================================================= reverse walk
    // Wave-private LDS tiles of the walk: T0 = the bounce tile (row stride LDB); T1, T2 = the two
    // halves of this wave's fp32 partial tile (row stride LDT), free whenever no partial sum is in it.
    const size_t slot = (size_t)bh * p.K + k;
    bf16* const T0 = s_bnc;
    bf16* const T1 = reinterpret_cast<bf16*>(s_Pw);
    bf16* const T2 = T1 + 64 * LDT;
    for (int j = n_mb - 1; j >= 0; j--) {
      const int mb = k * cgs + j;
      const size_t xo = x_base + (size_t)mb * (CS * FD);
      const size_t so = g_TF + (size_t)j * (CS * FD);
      const size_t ho = g_TH + (size_t)j * (CS * HID);
      // eta of the token this lane holds in column block cb of a Q-orientation tile
      const float eta_cb[2] = {bf2f(p.last_eta[eta_base + (size_t)mb * CS + c]),
                               bf2f(p.last_eta[eta_base + (size_t)mb * CS + 32 + c])};
      __syncthreads();
      stage_tile(s_xq, p.XQ + xo, tid);
      stage_tile(s_xk, p.XK + xo, tid);
      stage_tile(s_gz2, p.grad_l_wrt_Z2_group + so, tid);
      if (tid < CS) s_eta[tid] = bf2f(p.last_eta[eta_base + (size_t)mb * CS + tid]);
      // operand tiles of the state after this step: T1 = W2 rows [hid][F], T2 = W1^T rows [F][hid]
      store_opd_rows<LDT>(T1, opd_load(p.grad_l_wrt_Z1_group + ho, tid), c, h);
      store_opd_rows<LDT>(T2, opd_load(p.X2_group + ho, tid), c, h);

      // ---- output LayerNorm backward (LayerNorm lanes)
      {
        float gO[4][4], xh[4][4], gx[4][4], gam[4][4];
        ln_load(gO, p.grad_L_XQW + xo + tok * FD, fq);
        ln_load(xh, p.x_hat_ln_group + so + tok * FD, fq);
        ln_load_f32(gam, s_gam, fq);
        const float sd = p.std_ln_group[g_T + (size_t)j * CS + tok];
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int e = 0; e < 4; e++) gx[r][e] = gO[r][e] * xh[r][e];
        ln_token_sum_add(s_dbw, gO, q, fq);
        ln_token_sum_add(s_dgw, gx, q, fq);
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int e = 0; e < 4; e++) gx[r][e] = gO[r][e] * gam[r][e];
        const float s1 = quad_sum(sum16(gx)), s2 = quad_sum(dot16(gx, xh));
        const float sc = 1.f / (FD * sd);
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int e = 0; e < 4; e++) gx[r][e] = (FD * gx[r][e] - s1 - xh[r][e] * s2) * sc;
        ln_store(s_a + tok * LDB, gx, fq);  // gZ2_bar
      }
      __syncthreads();

      // ---- post-update forward, backwards (uses the state AFTER this mini-batch)
      {
        Acc dq;
        {
          Acc gz1b;   // (gZ2_bar W2^T) * gelu'(Z1_bar): rows hid, lane = tok
          acc_zero(gz1b);
          mma_jit(gz1b, [&](int blk, int s) { return piece_rows<LDT>(T1, blk, s, c, h); },
                  [&](int blk, int s) { return piece_rows<LDB>(s_a, blk, s, c, h); });
          WAVE_SYNC();   // T1 is overwritten below
          const Opd zimg = opd_load(p.Z1_bar_group + ho, tid);
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
#pragma unroll
            for (int s = 0; s < 4; s++) {
              bf16x8 x2b, gzb;
#pragma unroll
              for (int jj = 0; jj < 8; jj++) {
                float g, d;
                gelu_fd((float)zimg.v[cb][s][jj], g, d);
                x2b[jj] = (bf16)g;
                gzb[jj] = (bf16)(gz1b.b[s >> 1][cb][8 * (s & 1) + jj] * d);
              }
              store_piece_rows<LDB>(T0, cb, s, c, h, x2b);    // X2_bar  rows [tok][hid]
              store_piece_rows<LDT>(T1, cb, s, c, h, gzb);    // gZ1_bar rows [tok][hid]
            }
        }
        WAVE_SYNC();
        acc_zero(dq);
        mma_jit(dq, [&](int blk, int s) { return piece_rows<LDT>(T2, blk, s, c, h); },      // W1 after: lane = F
                [&](int blk, int s) { return piece_rows<LDT>(T1, blk, s, c, h); });         // gZ1_bar: lane = tok
        mma_jit(gW2s, [&](int blk, int s) { return piece_tr<LDB>(T0, blk, s, lane); },      // X2_bar^T: lane = hid
                [&](int blk, int s) { return piece_tr<LDB>(s_a, blk, s, lane); });          // gZ2_bar: lane = F
        if (w == 0) lds_rowsum_add_jit(s_gb2, [&](int blk, int s) { return piece_tr<LDB>(s_a, blk, s, lane); }, ones, c, h);
        mma_jit(gW1s, [&](int blk, int s) { return piece_tr<LDB>(s_xq, blk, s, lane); },    // XQ^T: lane = F
                [&](int blk, int s) { return piece_tr<LDT>(T1, blk, s, lane); });           // gZ1_bar: lane = hid
        lds_rowsum_add_jit(s_gb1w, [&](int blk, int s) { return piece_tr<LDT>(T1, blk, s, lane); }, ones, c, h);
        WAVE_SYNC();   // every reader of T1 / T2 is done before the partial tile takes their place
        lds_store_partial(s_Pw, dq, c, h);
      }
      __syncthreads();  // partial dXQ tiles complete; gb2 holds its value after the first update
      {
        float z[4][4], gO[4][4];
        ln_gather0(z, s_P, tok, fq);
        ln_load(gO, p.grad_L_XQW + xo + tok * FD, fq);
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int e = 0; e < 4; e++) z[r][e] += gO[r][e];
        ln_accumulate(p.grad_L_XQ + xo + tok * FD, z, fq);
      }
      __syncthreads();  // dXQ readers of the partial tiles are done: T1 / T2 are free again

      // ---- the weight step, backwards (uses the state BEFORE this mini-batch).
      //      Survive the LayerNorm stage: X2 in T0; packed d1p = gelu'(Z1) and
      //      t2p = -eta * (gZ2 W2^T) * (XK gW1 + gb1) * gelu''(Z1); the accumulator dk.
      {
        Acc dk;
        // T1 = W2 before the step, rows [hid][F]; T2 = gW1, rows [hid][F]
        store_opd_rows<LDT>(T1, (j > 0) ? opd_load(p.grad_l_wrt_Z1_group + ho - CS * HID, tid)
                                        : opd_from_f32_rows(p.W2_ck + slot * HID * FD, FD, 64 * w, 0, c, h), c, h);
        store_state_rows<LDT>(T2, gW1s, c, h);
        WAVE_SYNC();
        Acc R, S;   // R = gZ2 W2^T, S = XK gW1 + gb1   (rows hid, lane = tok)
        acc_zero(R);
        acc_init_rows_lds(S, s_gb1w, h);
        mma_jit(R, [&](int blk, int s) { return piece_rows<LDT>(T1, blk, s, c, h); },
                [&](int blk, int s) { return piece_rows<LDB>(s_gz2, blk, s, c, h); });
        mma_jit(S, [&](int blk, int s) { return piece_rows<LDT>(T2, blk, s, c, h); },
                [&](int blk, int s) { return piece_rows<LDB>(s_xk, blk, s, c, h); });
        const Opd zimg = opd_load(p.Z1_group + ho, tid);
        Acc pz;
        acc_zero(pz);
        acc_zero(dk);
        float de1[2] = {0.f, 0.f}, de3[2] = {0.f, 0.f};
#pragma unroll
        for (int cb = 0; cb < 2; cb++) {
          bf16x8 x2c[4], uc[4], g1c[4];
#pragma unroll
          for (int s = 0; s < 4; s++) {
            bf16x8 d1c, t2c;
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
              float g, a, b;
              gelu_fdd((float)zimg.v[cb][s][jj], g, a, b);
              const float r0 = R.b[s >> 1][cb][8 * (s & 1) + jj], sv = S.b[s >> 1][cb][8 * (s & 1) + jj];
              const float gz1 = r0 * a;                                   // dl/dZ1
              de3[cb] = __builtin_fmaf(gz1, sv, de3[cb]);
              x2c[s][jj] = (bf16)g;
              uc[s][jj] = (bf16)(sv * a);
              g1c[s][jj] = (bf16)(-eta_cb[cb] * gz1);
              d1c[jj] = (bf16)a;
              t2c[jj] = (bf16)(-eta_cb[cb] * r0 * sv * b);
            }
            // nothing stays in registers across the LayerNorm stage: d1 and t2 go to their park at once
            // (L2-resident, rewritten every mini-batch; 1 KiB per wave instruction)
            reinterpret_cast<bf16x8*>(park_d1)[(cb * 4 + s) * NTHREADS + tid] = d1c;
            reinterpret_cast<bf16x8*>(park_t2)[(cb * 4 + s) * NTHREADS + tid] = t2c;
          }
#pragma unroll
          for (int s = 0; s < 4; s++) store_piece_rows<LDB>(T0, cb, s, c, h, x2c[s]);   // X2 rows [tok][hid]
          // pz[:, cb] = gW2^T X2^T ; dEta partial ; + W2^T u^T.   dk[:, cb] = gW1 G1^T
#pragma unroll
          for (int s = 0; s < 4; s++)
#pragma unroll
            for (int rb = 0; rb < 2; rb++) pz.b[rb][cb] = MFMA(piece_state(gW2s, rb, s), x2c[s], pz.b[rb][cb]);
#pragma unroll
          for (int s = 0; s < 4; s++) {
            const bf16x8 gzv = piece_rows<LDB>(s_gz2, cb, s, c, h);
#pragma unroll
            for (int jj = 0; jj < 8; jj++)
              de1[cb] = __builtin_fmaf((float)gzv[jj], pz.b[s >> 1][cb][8 * (s & 1) + jj], de1[cb]);
          }
#pragma unroll
          for (int s = 0; s < 4; s++)
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
              pz.b[rb][cb] = MFMA(piece_tr<LDT>(T1, rb, s, lane), uc[s], pz.b[rb][cb]);
              dk.b[rb][cb] = MFMA(piece_tr<LDT>(T2, rb, s, lane), g1c[s], dk.b[rb][cb]);
            }
        }
        WAVE_SYNC();   // readers of T1 / T2 done
        lds_store_partial(s_Pw, pz, c, h);
        // the accumulator dk is parked too
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
              f32x4 v = {dk.b[rb][cb][4 * g], dk.b[rb][cb][4 * g + 1], dk.b[rb][cb][4 * g + 2], dk.b[rb][cb][4 * g + 3]};
              reinterpret_cast<f32x4*>(park_dk)[((rb * 2 + cb) * 4 + g) * 64 + lane] = v;
            }
#pragma unroll
        for (int cb = 0; cb < 2; cb++) {
          const float a = half_sum(de1[cb]), b = half_sum(de3[cb]);
          if (h == 0) {
            s_deta[(0 * 4 + w) * CS + 32 * cb + c] = a;
            s_deta[(1 * 4 + w) * CS + 32 * cb + c] = b;
          }
        }
      }
      __syncthreads();  // all partial ggZ2 tiles and dEta partial sums are in LDS

      // ---- second-order pass through the fused LayerNorm loss (LayerNorm lanes)
      {
        float gy[4][4];
        float gg[4][4], xh[4][4], go[4][4], gz[4][4], gam[4][4];
        ln_gather(gg, s_P, s_gb2, tok, fq);
        const float neg_eta = -s_eta[tok];
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int e = 0; e < 4; e++) gg[r][e] *= neg_eta;                 // grad wrt dl/dZ2
        ln_load(xh, p.x_hat_fused_group + so + tok * FD, fq);
        ln_load(go, p.grad_output_fused_group + so + tok * FD, fq);
        ln_load(gz, s_gz2 + tok * LDB, fq);
        ln_load_f32(gam, s_gam, fq);
        const float sd = p.std_fused_group[g_T + (size_t)j * CS + tok];
        const float rsd = 1.f / sd;
        // dEta: -(sum_F gZ2*(X2 gW2 + gb2) + sum_H gZ1*(XK gW1 + gb1))
        {
          float gb[4][4];
          ln_load_f32(gb, s_gb2, fq);
          float tot = quad_sum(dot16(gz, gb));
#pragma unroll
          for (int v = 0; v < 8; v++) tot += s_deta[v * CS + tok];
          if (fq == 0) {
            bf16* dst = p.grad_L_last_eta + eta_base + (size_t)mb * CS + tok;
            *dst = (bf16)((float)*dst - tot);
          }
        }
        const float s0 = quad_sum(sum16(gg)), a = quad_sum(dot16(gg, xh));
        float bb = 0.f;
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int e = 0; e < 4; e++) bb = __builtin_fmaf(go[r][e] * gam[r][e], xh[r][e], bb);
        bb = quad_sum(bb);
        float gx[4][4], dg[4][4];
        const float inv = rsd * (1.f / FD);
        float sg = 0.f, sx = 0.f;
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float ggx = (gg[r][e] - (s0 + xh[r][e] * a) * (1.f / FD)) * rsd;
            gy[r][e] = gam[r][e] * ggx;
            dg[r][e] = go[r][e] * ggx + gy[r][e] * xh[r][e];
            gx[r][e] = gy[r][e] * gam[r][e] - (go[r][e] * gam[r][e] * a + gg[r][e] * bb) * inv;
            sg += (-gx[r][e] * xh[r][e] - gg[r][e] * gz[r][e]) * rsd;
            sx += gx[r][e];
          }
        sg = quad_sum(sg);
        sx = quad_sum(sx);
        ln_token_sum_add(s_dgw, dg, q, fq);
        ln_token_sum_add(s_dbw, gy, q, fq);
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int e = 0; e < 4; e++) {
            gx[r][e] = gx[r][e] * rsd + (sg * xh[r][e] - sx * rsd) * (1.f / FD);   // dZ2
            xh[r][e] = -gy[r][e];                                                   // dXV
          }
#pragma unroll
        for (int r = 0; r < 4; r++) {   // g_y is needed again for dXK: park it (XQ / E2 tiles are dead by now)
          f32x4 v = {gy[r][0], gy[r][1], gy[r][2], gy[r][3]};
          *reinterpret_cast<f32x4*>(s_gy + 16 * r + 4 * fq) = v;
        }
        ln_store(s_a + tok * LDB, gx, fq);
        ln_accumulate(p.grad_L_XV + xo + tok * FD, xh, fq);
      }
      __syncthreads();  // dZ2 tile complete; partial tiles (T1 / T2) free again

      // ---- inner MLP, backwards (uses the state BEFORE this mini-batch)
      {
        // T2 = gW1 rows [hid][F] (for S again), T1 = gW2 rows [F][hid] (transposed read gives lane = hid)
        store_state_rows<LDT>(T2, gW1s, c, h);
        store_state_rows<LDT>(T1, gW2s, c, h);
        WAVE_SYNC();
        Acc S, dx2;
        acc_init_rows_lds(S, s_gb1w, h);
        acc_zero(dx2);
        mma_jit(S, [&](int blk, int s) { return piece_rows<LDT>(T2, blk, s, c, h); },
                [&](int blk, int s) { return piece_rows<LDB>(s_xk, blk, s, c, h); });
        mma_jit(dx2, [&](int blk, int s) { return piece_tr<LDT>(T1, blk, s, lane); },       // gW2: lane = hid, contraction = F
                [&](int blk, int s) { return piece_rows<LDB>(s_gz2, blk, s, c, h); });      // P2 = gZ2 gW2^T
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
#pragma unroll
            for (int i = 0; i < 16; i++) dx2.b[rb][cb][i] *= -eta_cb[cb];
        {
          // W2 before the step: lane = hid, contraction = F
          const Opd w2tA = (j > 0) ? opd_load(p.grad_l_wrt_Z1_group + ho - CS * HID, tid)
                                   : opd_from_f32_rows(p.W2_ck + slot * HID * FD, FD, 64 * w, 0, c, h);
          mma_jit(dx2, [&](int blk, int s) { return w2tA.v[blk][s]; },
                  [&](int blk, int s) { return piece_rows<LDB>(s_a, blk, s, c, h); });      // + dZ2 W2^T
        }
        WAVE_SYNC();   // S and P2 have consumed T2 / T1
        const Opd d1p = opd_load(park_d1, tid);
        const Opd t2p = opd_load(park_t2, tid);
        // dZ1 = dX2*gelu' + t2  -> T1 rows [tok][hid];   -eta * S * gelu' -> T2 rows [tok][hid]
#pragma unroll
        for (int cb = 0; cb < 2; cb++)
#pragma unroll
          for (int s = 0; s < 4; s++) {
            bf16x8 dz, uh;
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
              const float d1v = (float)d1p.v[cb][s][jj];
              dz[jj] = (bf16)__builtin_fmaf(dx2.b[s >> 1][cb][8 * (s & 1) + jj], d1v, (float)t2p.v[cb][s][jj]);
              uh[jj] = (bf16)(-eta_cb[cb] * S.b[s >> 1][cb][8 * (s & 1) + jj] * d1v);
            }
            store_piece_rows<LDT>(T1, cb, s, c, h, dz);
            store_piece_rows<LDT>(T2, cb, s, c, h, uh);
          }
        WAVE_SYNC();
        Acc dk;
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
              const f32x4 v = reinterpret_cast<const f32x4*>(park_dk)[((rb * 2 + cb) * 4 + g) * 64 + lane];
#pragma unroll
              for (int e = 0; e < 4; e++) dk.b[rb][cb][4 * g + e] = v[e];
            }
        {
          // W1 before the step: lane = F, contraction = hid
          const Opd w1tA = (j > 0) ? opd_load(p.X2_group + ho - CS * HID, tid)
                                   : opd_from_f32_rows(p.W1_ck + slot * FD * HID, HID, 0, 64 * w, c, h);
          mma_jit(dk, [&](int blk, int s) { return w1tA.v[blk][s]; },
                  [&](int blk, int s) { return piece_rows<LDT>(T1, blk, s, c, h); });       // + dZ1 W1^T
        }
        mma_jit(gW2s, [&](int blk, int s) { return piece_tr<LDT>(T2, blk, s, lane); },      // (-eta u)^T: lane = hid
                [&](int blk, int s) { return piece_tr<LDB>(s_gz2, blk, s, lane); });        // gZ2: lane = F
        mma_jit(gW2s, [&](int blk, int s) { return piece_tr<LDB>(T0, blk, s, lane); },      // X2^T: lane = hid
                [&](int blk, int s) { return piece_tr<LDB>(s_a, blk, s, lane); });          // dZ2: lane = F
        if (w == 0) lds_rowsum_add_jit(s_gb2, [&](int blk, int s) { return piece_tr<LDB>(s_a, blk, s, lane); }, ones, c, h);
        mma_jit(gW1s, [&](int blk, int s) { return piece_tr<LDB>(s_xk, blk, s, lane); },    // XK^T: lane = F
                [&](int blk, int s) { return piece_tr<LDT>(T1, blk, s, lane); });           // dZ1: lane = hid
        lds_rowsum_add_jit(s_gb1w, [&](int blk, int s) { return piece_tr<LDT>(T1, blk, s, lane); }, ones, c, h);
        WAVE_SYNC();   // readers of T1 / T2 done
        lds_store_partial(s_Pw, dk, c, h);
      }
      __syncthreads();  // partial dXK tiles complete
      {
        float z[4][4];
        ln_gather0(z, s_P, tok, fq);
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(s_gy + 16 * r + 4 * fq);
#pragma unroll
          for (int e = 0; e < 4; e++) z[r][e] += v[e];
        }
        ln_accumulate(p.grad_L_XK + xo + tok * FD, z, fq);
      }
    }
  }

  // ---- outputs that are written once
  acc_store_rows(gW1s, p.grad_L_W1_init + (size_t)bh * FD * HID, HID, 0, 64 * w, c, h);
  acc_store_rows(gW2s, p.grad_L_W2_init + (size_t)bh * HID * FD, FD, 64 * w, 0, c, h);
  __syncthreads();
  p.grad_L_b1_init[(size_t)bh * HID + tid] = s_gb1[tid];
  if (tid < FD) p.grad_L_b2_init[(size_t)bh * FD + tid] = s_gb2[tid];
  // norm-weight / norm-bias gradients: sum the per-wave LDS accumulators
  __syncthreads();
  if (tid < 2 * FD) {
    const int which = tid / FD, f = tid % FD;
    float s = 0.f;
#pragma unroll
    for (int v = 0; v < 4; v++) s += s_red[(v * 2 + which) * FD + f];
    (which == 0 ? p.grad_L_ttt_norm_weight : p.grad_L_ttt_norm_bias)[(size_t)bh * FD + f] = s;
  }
}

}  // namespace ttt

extern "C" int ttt_mlp_bwd_threads() { return ttt::NTHREADS; }
extern "C" int ttt_mlp_bwd_lds_bytes() { return ttt::SM_BWD_BYTES; }

hipError_t ttt_mlp_bwd_enqueue(const ttt::BwdParams& p, hipStream_t stream) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(ttt::ttt_mlp_bwd_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, ttt::SM_BWD_BYTES);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ttt::ttt_mlp_bwd_kernel, dim3(p.B * p.NH), dim3(ttt::NTHREADS), ttt::SM_BWD_BYTES, stream, p);
  return hipGetLastError();
}
