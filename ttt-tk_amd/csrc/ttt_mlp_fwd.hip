// Forward scan of the non-causal TTT-MLP layer for gfx950 (MI355X).
//
// Behaviour follows the upstream operator `ttt_forward` (kernels/ttt/ttt.cu:85-586 for the kernel,
// kernels/ttt/matching.py:30-125 for the mathematics): for every (batch, head) the fp32 state
// (W1,b1,W2,b2) is carried through NC mini-batches of 64 tokens; before mini-batch i with
// i % checkpoint_group_size == 0 the state is stored at checkpoint slot i / checkpoint_group_size.
//
// Mapping: one workgroup of 4 wavefronts per (batch, head); wave w owns hidden columns
// [64w, 64w+64).  The state lives in registers for the whole scan as MFMA accumulator tiles:
//   W1s = W1[:, shard]      (rows F,   columns hid)  -> chained operand of XK*W1 and of (XQ*W1)^T
//   W2s = W2[shard, :]      (rows hid, columns F)    -> chained operand of (X2*W2)^T
//   W2t = W2[shard, :]^T    (rows F,   columns hid)  -> chained operand of gZ2*W2^T
// so no weight ever goes through LDS; the eta-scaled updates are MFMA accumulations into them.
// Cross-shard sums of Z2 go through fp32 LDS tiles; each wave then LayerNorms 16 of the 64 tokens
// with 4 lanes per token.
#include "ttt_mlp_common.hpp"
#include "ttt_mlp_kernels.hpp"

namespace ttt {

// LDS carve-up (bytes)
constexpr int SM_TILE = 64 * LDB * 2;                   // one bf16 tile: 9216
constexpr int SM_XQ = 0;
constexpr int SM_XK = SM_XQ + SM_TILE;
constexpr int SM_XV = SM_XK + SM_TILE;
constexpr int SM_G2 = SM_XV + SM_TILE;
constexpr int SM_P = SM_G2 + SM_TILE;                    // 4 fp32 partial tiles; wave w's tile doubles
constexpr int SM_PTILE = 64 * LDP * 4;                   // as its bf16 X2 transposition buffer
constexpr int SM_B1 = SM_P + 4 * SM_PTILE;
constexpr int SM_B2 = SM_B1 + HID * 4;
constexpr int SM_ETA = SM_B2 + FD * 4;
constexpr int SM_FWD_BYTES = SM_ETA + CS * 4;

struct Staged {  // one mini-batch of inputs in flight from HBM (per thread)
  u32x4 q[2], k[2], v[2];
  float eta;
};

TTT_DEV void stage_load(Staged& s, const FwdParams& p, size_t tile_off, size_t eta_off, int tid) {
#pragma unroll
  for (int r = 0; r < 2; r++) {
    const int id = tid + 256 * r;  // 16-byte chunk id: row = id / 8, 8 chunks per 128-byte row
    s.q[r] = reinterpret_cast<const u32x4*>(p.XQ + tile_off)[id];
    s.k[r] = reinterpret_cast<const u32x4*>(p.XK + tile_off)[id];
    s.v[r] = reinterpret_cast<const u32x4*>(p.XV + tile_off)[id];
  }
  s.eta = (tid < CS) ? bf2f(p.last_eta[eta_off + tid]) : 0.f;
}

TTT_DEV void stage_store(const Staged& s, unsigned char* smem, int tid) {
#pragma unroll
  for (int r = 0; r < 2; r++) {
    const int id = tid + 256 * r;
    const int off = ((id >> 3) * LDB + (id & 7) * 8) * 2;
    *reinterpret_cast<u32x4*>(smem + SM_XQ + off) = s.q[r];
    *reinterpret_cast<u32x4*>(smem + SM_XK + off) = s.k[r];
    *reinterpret_cast<u32x4*>(smem + SM_XV + off) = s.v[r];
  }
  if (tid < CS) reinterpret_cast<float*>(smem + SM_ETA)[tid] = s.eta;
}

__global__ __launch_bounds__(NTHREADS) void ttt_mlp_fwd_kernel(const FwdParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* s_xq = reinterpret_cast<bf16*>(smem + SM_XQ);
  bf16* s_xk = reinterpret_cast<bf16*>(smem + SM_XK);
  bf16* s_xv = reinterpret_cast<bf16*>(smem + SM_XV);
  bf16* s_g2 = reinterpret_cast<bf16*>(smem + SM_G2);
  float* s_P = reinterpret_cast<float*>(smem + SM_P);
  float* s_b1 = reinterpret_cast<float*>(smem + SM_B1);
  float* s_b2 = reinterpret_cast<float*>(smem + SM_B2);
  const float* s_eta = reinterpret_cast<const float*>(smem + SM_ETA);

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, h = lane >> 5, c = lane & 31;
  const int q = lane >> 2, fq = lane & 3, tok = 16 * w + q;  // LayerNorm ownership: 4 lanes per token
  const int bh = blockIdx.x, head = bh % p.NH;
  float* s_Pw = s_P + w * 64 * LDP;
  bf16* s_x2t = reinterpret_cast<bf16*>(s_Pw);

  // ---- state -> registers
  Acc W1s, W2s, W2t;
  float b1L[2];
  f32x16 b2acc[2];
  {
    const float* W1 = p.W1 + (size_t)bh * FD * HID;
    const float* W2 = p.W2 + (size_t)bh * HID * FD;
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
      for (int cb = 0; cb < 2; cb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int row = 32 * rb + 8 * (i >> 2) + 4 * h + (i & 3), col = 32 * cb + c;
          W1s.b[rb][cb][i] = W1[row * HID + 64 * w + col];
          W2s.b[rb][cb][i] = W2[(64 * w + row) * FD + col];
          W2t.b[rb][cb][i] = W2[(64 * w + col) * FD + row];
        }
#pragma unroll
    for (int cb = 0; cb < 2; cb++) b1L[cb] = p.b1[(size_t)bh * HID + 64 * w + 32 * cb + c];
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
      for (int i = 0; i < 16; i++) b2acc[rb][i] = p.b2[(size_t)bh * FD + 32 * rb + 8 * (i >> 2) + 4 * h + (i & 3)];
    s_b1[tid] = p.b1[(size_t)bh * HID + tid];
    if (tid < FD) s_b2[tid] = p.b2[(size_t)bh * FD + tid];
  }
  float gam[4][4], bet[4][4];
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      gam[r][e] = p.ttt_norm_weight[head * FD + 16 * r + 4 * fq + e];
      bet[r][e] = p.ttt_norm_bias[head * FD + 16 * r + 4 * fq + e];
    }
  bf16x8 ones;
#pragma unroll
  for (int j = 0; j < 8; j++) ones[j] = (bf16)1.0f;

  const size_t x_base = (size_t)bh * p.NC * (CS * FD);
  const size_t eta_base = (size_t)bh * p.NC * CS;
  Staged st;
  stage_load(st, p, x_base, eta_base, tid);
  stage_store(st, smem, tid);
  __syncthreads();

  for (int mb = 0; mb < p.NC; mb++) {
    if (mb + 1 < p.NC) stage_load(st, p, x_base + (size_t)(mb + 1) * (CS * FD), eta_base + (size_t)(mb + 1) * CS, tid);

    // ---- checkpoint: the state before this mini-batch
    if (mb % p.cgs == 0) {
      const size_t slot = (size_t)bh * p.K + mb / p.cgs;
      float* cW1 = p.W1_ck + slot * FD * HID;
      float* cW2 = p.W2_ck + slot * HID * FD;
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int cb = 0; cb < 2; cb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int row = 32 * rb + 8 * (i >> 2) + 4 * h + (i & 3), col = 32 * cb + c;
            cW1[row * HID + 64 * w + col] = W1s.b[rb][cb][i];
            cW2[(64 * w + row) * FD + col] = W2s.b[rb][cb][i];
          }
      if (h == 0) {
#pragma unroll
        for (int cb = 0; cb < 2; cb++) p.b1_ck[slot * HID + 64 * w + 32 * cb + c] = b1L[cb];
      }
      if (w == 0 && c == 0) {
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
          for (int i = 0; i < 16; i++) p.b2_ck[slot * FD + 32 * rb + 8 * (i >> 2) + 4 * h + (i & 3)] = b2acc[rb][i];
      }
    }

    // ---- Z1 = XK W1 + b1 (rows tok, lane = hid);  X2 = gelu(Z1), D1 = gelu'(Z1)
    Acc x2, d1;
    {
      const Opd w1op = cvt_chain(W1s);
      const Opd xkA = lds_rows_kappa(s_xk, c, h);
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int cb = 0; cb < 2; cb++)
#pragma unroll
          for (int i = 0; i < 16; i++) x2.b[rb][cb][i] = b1L[cb];
      mma(x2, xkA, w1op);
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int cb = 0; cb < 2; cb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            float g, d;
            gelu_fd(x2.b[rb][cb][i], g, d);
            x2.b[rb][cb][i] = g;
            d1.b[rb][cb][i] = d;
          }
    }
    const Opd x2op = cvt_chain(x2);  // lane = hid, contraction = tok
    lds_store_rows_kappa(s_x2t, x2op, c, h);  // stored [hid][tok]
    __syncthreads();

    // ---- Z2^T partial = W2s^T X2^T (rows F, lane = tok) -> fp32 partial tile [tok][F]
    {
      const Opd w2A = cvt_chain(W2s);
      const Opd x2B = lds_tr_kappa(s_x2t, lane);
      Acc z2;
      acc_zero(z2);
      mma(z2, w2A, x2B);
      lds_store_partial(s_Pw, z2, c, h);
    }
    __syncthreads();

    // ---- LayerNorm-fused reconstruction-loss gradient for 16 tokens per wave, 4 lanes per token
    {
      float z[4][4];
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        f32x4 a = *reinterpret_cast<const f32x4*>(s_b2 + 16 * r + 4 * fq);
#pragma unroll
        for (int v = 0; v < 4; v++) a += *reinterpret_cast<const f32x4*>(s_P + v * 64 * LDP + tok * LDP + 16 * r + 4 * fq);
#pragma unroll
        for (int e = 0; e < 4; e++) { z[r][e] = a[e]; sum += a[e]; }
      }
      const float mu = quad_sum(sum) * (1.f / FD);
      float var = 0.f;
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int e = 0; e < 4; e++) { z[r][e] -= mu; var = __builtin_fmaf(z[r][e], z[r][e], var); }
      const float rstd = __builtin_amdgcn_rsqf(quad_sum(var) * (1.f / FD) + LN_EPS);
      float s1 = 0.f, s2 = 0.f;
      float gx[4][4];
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const bf16x4 kv = *reinterpret_cast<const bf16x4*>(s_xk + tok * LDB + 16 * r + 4 * fq);
        const bf16x4 vv = *reinterpret_cast<const bf16x4*>(s_xv + tok * LDB + 16 * r + 4 * fq);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float xh = z[r][e] * rstd;
          const float go = __builtin_fmaf(gam[r][e], xh, bet[r][e]) - (bf2f(vv[e]) - bf2f(kv[e]));
          z[r][e] = xh;
          gx[r][e] = go * gam[r][e];
          s1 += gx[r][e];
          s2 = __builtin_fmaf(gx[r][e], xh, s2);
        }
      }
      s1 = quad_sum(s1);
      s2 = quad_sum(s2);
      const float scale = -s_eta[tok] * rstd * (1.f / FD);  // G2 = -eta * dl/dZ2
#pragma unroll
      for (int r = 0; r < 4; r++) {
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (bf16)((FD * gx[r][e] - s1 - z[r][e] * s2) * scale);
        *reinterpret_cast<bf16x4*>(s_g2 + tok * LDB + 16 * r + 4 * fq) = o;
      }
    }
    __syncthreads();

    // ---- G1 = (G2 W2^T) * gelu'(Z1);  state += X^T G
    {
      const Opd g2A = lds_rows_kappa(s_g2, c, h);   // lane = tok, contraction = F
      const Opd w2tB = cvt_chain(W2t);              // lane = hid, contraction = F
      Acc g1;
      acc_zero(g1);
      mma(g1, g2A, w2tB);                           // rows tok, lane = hid
      float colsum[2] = {0.f, 0.f};
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int cb = 0; cb < 2; cb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            g1.b[rb][cb][i] *= d1.b[rb][cb][i];
            colsum[cb] += g1.b[rb][cb][i];
          }
      const Opd g1op = cvt_chain(g1);               // lane = hid, contraction = tok
#pragma unroll
      for (int cb = 0; cb < 2; cb++) b1L[cb] += half_sum(colsum[cb]);
      const Opd g2T = lds_tr_kappa(s_g2, lane);     // lane = F, contraction = tok
      mma(W2s, x2op, g2T);                          // W2[shard,:]   += X2^T G2
      mma(W2t, g2T, x2op);                          // W2[shard,:]^T += G2^T X2
#pragma unroll
      for (int s = 0; s < 4; s++)
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
          b2acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(g2T.v[rb][s], ones, b2acc[rb], 0, 0, 0);
      const Opd xkT = lds_tr_kappa(s_xk, lane);     // lane = F, contraction = tok
      mma(W1s, xkT, g1op);                          // W1[:,shard]   += XK^T G1
    }
    if (h == 0) {
#pragma unroll
      for (int cb = 0; cb < 2; cb++) s_b1[64 * w + 32 * cb + c] = b1L[cb];
    }
    if (w == 0 && c == 0) {
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          f32x4 v = {b2acc[rb][4 * g], b2acc[rb][4 * g + 1], b2acc[rb][4 * g + 2], b2acc[rb][4 * g + 3]};
          *reinterpret_cast<f32x4*>(s_b2 + 32 * rb + 8 * g + 4 * h) = v;
        }
    }
    __syncthreads();

    // ---- post-update forward on XQ, transposed: Z1b^T = W1s^T XQ^T (rows hid, lane = tok)
    {
      const Opd w1A = cvt_chain(W1s);
      const Opd xqB = lds_rows_kappa(s_xq, c, h);
      Acc z1b;
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const f32x4 bv = *reinterpret_cast<const f32x4*>(s_b1 + 64 * w + 32 * rb + 8 * g + 4 * h);
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
#pragma unroll
            for (int e = 0; e < 4; e++) z1b.b[rb][cb][4 * g + e] = bv[e];
        }
      mma(z1b, w1A, xqB);
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int cb = 0; cb < 2; cb++)
#pragma unroll
          for (int i = 0; i < 16; i++) z1b.b[rb][cb][i] = gelu_f(z1b.b[rb][cb][i]);
      const Opd x2bB = cvt_chain(z1b);              // lane = tok, contraction = hid
      const Opd w2A = cvt_chain(W2s);
      Acc z2;
      acc_zero(z2);
      mma(z2, w2A, x2bB);                           // rows F, lane = tok
      lds_store_partial(s_Pw, z2, c, h);
    }
    __syncthreads();

    // ---- output LayerNorm + residual, 16 tokens per wave
    {
      float z[4][4];
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        f32x4 a = *reinterpret_cast<const f32x4*>(s_b2 + 16 * r + 4 * fq);
#pragma unroll
        for (int v = 0; v < 4; v++) a += *reinterpret_cast<const f32x4*>(s_P + v * 64 * LDP + tok * LDP + 16 * r + 4 * fq);
#pragma unroll
        for (int e = 0; e < 4; e++) { z[r][e] = a[e]; sum += a[e]; }
      }
      const float mu = quad_sum(sum) * (1.f / FD);
      float var = 0.f;
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int e = 0; e < 4; e++) { z[r][e] -= mu; var = __builtin_fmaf(z[r][e], z[r][e], var); }
      const float rstd = __builtin_amdgcn_rsqf(quad_sum(var) * (1.f / FD) + LN_EPS);
      bf16* out = p.Out + x_base + (size_t)mb * (CS * FD) + tok * FD;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const bf16x4 qv = *reinterpret_cast<const bf16x4*>(s_xq + tok * LDB + 16 * r + 4 * fq);
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (bf16)(bf2f(qv[e]) + __builtin_fmaf(gam[r][e], z[r][e] * rstd, bet[r][e]));
        *reinterpret_cast<bf16x4*>(out + 16 * r + 4 * fq) = o;
      }
    }
    __syncthreads();
    if (mb + 1 < p.NC) stage_store(st, smem, tid);
    __syncthreads();
  }
}

}  // namespace ttt

extern "C" int ttt_mlp_fwd_lds_bytes() { return ttt::SM_FWD_BYTES; }

hipError_t ttt_mlp_fwd_enqueue(const ttt::FwdParams& p, hipStream_t stream) {
  // Per-device attribute; cheap enough to set on every launch.
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(ttt::ttt_mlp_fwd_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, ttt::SM_FWD_BYTES);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ttt::ttt_mlp_fwd_kernel, dim3(p.B * p.NH), dim3(ttt::NTHREADS), ttt::SM_FWD_BYTES, stream, p);
  return hipGetLastError();
}
