// The sixteen per-group tensors of `ttt_backward`, filled for checkpoint group 0 in the layouts and with
// the meaning the reference's kernel leaves in them (kernels/ttt_backward/ttt.cu:518-521, 551-552, 607-610,
// 636-637, 669, 699, 744-745, 798-800; compared by kernels/ttt_backward/matching.py:667-690).
//
// The backward kernels of this library use those tensors as their own workspace, in their own formats.
// A caller that wants to look at the group-0 values afterwards enqueues this kernel behind the backward:
// it replays the mini-batches of group 0 from checkpoint 0 once more and writes every intermediate
// row-major.  It is a side path, not part of the timed operator: plain fp32 arithmetic on the vector
// units, one workgroup of 256 threads per (batch, head), nothing rounded before it is stored.
//
// Ownership inside the workgroup (t = thread, 0..255):
//   * thread t holds column t of W1 (64 registers) and b1[t] for the whole replay;
//   * W2 (256 x 64) and b2 live in LDS, row t of W2 is updated by thread t only;
//   * [64 x 256] activations (Z1, X2, grad_l_wrt_Z1, Z1_bar, X2_bar): thread t holds column t;
//   * [64 x 64] tiles (Z2, the LayerNorm values): wave w holds rows 16w..16w+15, lane = column, so a
//     LayerNorm row statistic is a sum over the lanes of one wave.
#include <hip/hip_runtime.h>

#include "ttt_mlp_common.hpp"
#include "ttt_mlp_kernels.hpp"

namespace ttt {

constexpr int EX_THREADS = 256;
constexpr int EX_W2_LD = 65;                       // padded row of W2 in LDS: row-wise and column-wise reads both spread over the banks
constexpr int EX_W2S = 0;                          // [256][65] W2
constexpr int EX_XK = EX_W2S + 256 * EX_W2_LD;     // [64][64] XK
constexpr int EX_XQ = EX_XK + 64 * 64;             // [64][64] XQ
constexpr int EX_GZ = EX_XQ + 64 * 64;             // [64][64] grad_l_wrt_Z2
constexpr int EX_XS = EX_GZ + 64 * 64;             // [64][128] half of a [64 x 256] activation, to contract over its columns
constexpr int EX_ETA = EX_XS + 64 * 128;           // [64] step size of each token
constexpr int EX_B2 = EX_ETA + 64;                 // [64] b2
constexpr int EX_FLOATS = EX_B2 + 64;
constexpr int SM_EX_BYTES = EX_FLOATS * (int)sizeof(float);
static_assert(SM_EX_BYTES <= 160 * 1024, "LDS of one CU");

constexpr float EX_LN_EPS = 1e-8f;

TTT_DEV float lanes_sum(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
  return x;
}

// acc[j] = sum over the 256 columns u of act[row 16*wave + j][u] * W2[u][lane]; every thread passes its own column of act.
TTT_DEV void contract_columns(const float (&act)[64], float (&acc)[16], float* sm, int t) {
  const int wave = t >> 6, lane = t & 63;
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = 0.f;
  for (int half = 0; half < 2; ++half) {
    __syncthreads();  // the staging tile is free
    if ((t >> 7) == half) {
#pragma unroll
      for (int r = 0; r < 64; ++r) sm[EX_XS + r * 128 + (t & 127)] = act[r];
    }
    __syncthreads();
    const float* w2 = sm + EX_W2S + half * 128 * EX_W2_LD + lane;
    const float* xs = sm + EX_XS + 16 * wave * 128;
    for (int u = 0; u < 128; u += 4) {
      const float w0 = w2[(u + 0) * EX_W2_LD], w1 = w2[(u + 1) * EX_W2_LD];
      const float w2v = w2[(u + 2) * EX_W2_LD], w3 = w2[(u + 3) * EX_W2_LD];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float4 x = *reinterpret_cast<const float4*>(xs + j * 128 + u);
        acc[j] = __builtin_fmaf(x.x, w0, acc[j]);
        acc[j] = __builtin_fmaf(x.y, w1, acc[j]);
        acc[j] = __builtin_fmaf(x.z, w2v, acc[j]);
        acc[j] = __builtin_fmaf(x.w, w3, acc[j]);
      }
    }
  }
}

// out[r] = bias + sum_k x[r][k] * wcol[k], x a [64][64] tile in LDS
TTT_DEV void times_w1(const float* x, const float (&wcol)[64], float bias, float (&out)[64]) {
#pragma unroll
  for (int r = 0; r < 64; ++r) {
    float s = bias;
#pragma unroll
    for (int k = 0; k < 64; k += 4) {
      const float4 v = *reinterpret_cast<const float4*>(x + r * 64 + k);
      s = __builtin_fmaf(v.x, wcol[k], s);
      s = __builtin_fmaf(v.y, wcol[k + 1], s);
      s = __builtin_fmaf(v.z, wcol[k + 2], s);
      s = __builtin_fmaf(v.w, wcol[k + 3], s);
    }
    out[r] = s;
  }
}

TTT_DEV void store_column(bf16* dst, const float (&col)[64], int t) {
#pragma unroll
  for (int r = 0; r < 64; ++r) dst[r * 256 + t] = (bf16)col[r];
}

__global__ __launch_bounds__(EX_THREADS) void ttt_mlp_export_group0_kernel(BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) float sm_ex[];
  float* sm = sm_ex;
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  const size_t bh = blockIdx.x;
  const int head = (int)(bh % (size_t)p.NH);
  const int n = p.cgs < p.NC ? p.cgs : p.NC;   // mini-batches of group 0

  // state at the start of group 0 = checkpoint 0
  float w1[64];
  {
    const float* W1c = p.W1_ck + bh * (size_t)p.K * (64 * 256);
#pragma unroll
    for (int k = 0; k < 64; ++k) w1[k] = W1c[k * 256 + t];
  }
  float b1 = p.b1_ck[bh * (size_t)p.K * 256 + t];
  {
    const float* W2c = p.W2_ck + bh * (size_t)p.K * (256 * 64);
    for (int idx = t; idx < 256 * 64; idx += EX_THREADS) sm[EX_W2S + (idx >> 6) * EX_W2_LD + (idx & 63)] = W2c[idx];
    if (t < 64) sm[EX_B2 + t] = p.b2_ck[bh * (size_t)p.K * 64 + t];
  }
  const float gamma = p.ttt_norm_weight[head * 64 + lane], beta = p.ttt_norm_bias[head * 64 + lane];
  __syncthreads();

  for (int i = 0; i < n; ++i) {
    const size_t slot = bh * (size_t)p.cgs + i;   // index of the mini-batch in the per-group tensors
    const size_t mb = bh * (size_t)p.NC + i;      // index of the mini-batch in the sequence tensors

    // the state before the mini-batch
    {
      float* W1g = p.W1_init_group + slot * (64 * 256);
#pragma unroll
      for (int k = 0; k < 64; ++k) W1g[k * 256 + t] = w1[k];
      p.b1_init_group[slot * 256 + t] = b1;
      float* W2g = p.W2_init_group + slot * (256 * 64);
      for (int idx = t; idx < 256 * 64; idx += EX_THREADS) W2g[idx] = sm[EX_W2S + (idx >> 6) * EX_W2_LD + (idx & 63)];
      if (t < 64) p.b2_init_group[slot * 64 + t] = sm[EX_B2 + t];
    }
    // inputs of the mini-batch
    const bf16* xkg = p.XK + mb * 4096;
    const bf16* xqg = p.XQ + mb * 4096;
    const bf16* xvg = p.XV + mb * 4096;
    for (int idx = t; idx < 4096; idx += EX_THREADS) {
      sm[EX_XK + idx] = (float)xkg[idx];
      sm[EX_XQ + idx] = (float)xqg[idx];
    }
    if (t < 64) sm[EX_ETA + t] = (float)p.last_eta[mb * 64 + t];
    float target[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int e = (16 * wave + j) * 64 + lane;
      target[j] = (float)xvg[e] - (float)xkg[e];
    }
    __syncthreads();

    // Z1 = XK W1 + b1, X2 = gelu(Z1)
    float a[64], x2[64];
    times_w1(sm + EX_XK, w1, b1, a);
    store_column(p.Z1_group + slot * 16384, a, t);
#pragma unroll
    for (int r = 0; r < 64; ++r) gelu_fd(a[r], x2[r], a[r]);   // a = gelu'(Z1) from here on
    store_column(p.X2_group + slot * 16384, x2, t);

    // Z2 = X2 W2 + b2; gradient of the reconstruction loss through the LayerNorm
    float z2[16];
    contract_columns(x2, z2, sm, t);
    {
      const float b2 = sm[EX_B2 + lane];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int row = 16 * wave + j;
        const float z = z2[j] + b2;
        const float mu = lanes_sum(z) * (1.f / 64.f);
        const float d = z - mu;
        const float sd = sqrtf(lanes_sum(d * d) * (1.f / 64.f) + EX_LN_EPS);
        const float xh = d / sd;
        const float go = __builtin_fmaf(gamma, xh, beta) - target[j];
        const float gx = go * gamma;
        const float s1 = lanes_sum(gx), s2 = lanes_sum(gx * xh);
        const float gz = (64.f * gx - s1 - xh * s2) / (64.f * sd);
        const size_t e = slot * 4096 + row * 64 + lane;
        p.x_hat_fused_group[e] = (bf16)xh;
        p.grad_output_fused_group[e] = (bf16)go;
        p.grad_x_hat_fused_group[e] = (bf16)gx;
        p.grad_l_wrt_Z2_group[e] = (bf16)gz;
        if (lane == 0) p.std_fused_group[slot * 64 + row] = sd;
        sm[EX_GZ + row * 64 + lane] = gz;
      }
    }
    __syncthreads();

    // grad_l_wrt_Z1 = (grad_l_wrt_Z2 W2^T) * gelu'(Z1); thread t needs row t of W2
    float wrow[64];
#pragma unroll
    for (int c = 0; c < 64; ++c) wrow[c] = sm[EX_W2S + t * EX_W2_LD + c];
#pragma unroll
    for (int r = 0; r < 64; ++r) {
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < 64; c += 4) {
        const float4 g = *reinterpret_cast<const float4*>(sm + EX_GZ + r * 64 + c);
        s = __builtin_fmaf(g.x, wrow[c], s);
        s = __builtin_fmaf(g.y, wrow[c + 1], s);
        s = __builtin_fmaf(g.z, wrow[c + 2], s);
        s = __builtin_fmaf(g.w, wrow[c + 3], s);
      }
      a[r] *= s;   // a = grad_l_wrt_Z1 from here on
    }
    store_column(p.grad_l_wrt_Z1_group + slot * 16384, a, t);

    // the step: W1 -= (eta XK)^T gZ1, b1 -= sum eta gZ1, W2 -= (eta X2)^T gZ2, b2 -= sum eta gZ2
#pragma unroll
    for (int r = 0; r < 64; ++r) {
      const float eta = sm[EX_ETA + r];
      const float ea = eta * a[r], ex = eta * x2[r];
      b1 -= ea;
#pragma unroll
      for (int k = 0; k < 64; k += 4) {
        const float4 v = *reinterpret_cast<const float4*>(sm + EX_XK + r * 64 + k);
        const float4 g = *reinterpret_cast<const float4*>(sm + EX_GZ + r * 64 + k);
        w1[k] = __builtin_fmaf(-v.x, ea, w1[k]);
        w1[k + 1] = __builtin_fmaf(-v.y, ea, w1[k + 1]);
        w1[k + 2] = __builtin_fmaf(-v.z, ea, w1[k + 2]);
        w1[k + 3] = __builtin_fmaf(-v.w, ea, w1[k + 3]);
        wrow[k] = __builtin_fmaf(-g.x, ex, wrow[k]);
        wrow[k + 1] = __builtin_fmaf(-g.y, ex, wrow[k + 1]);
        wrow[k + 2] = __builtin_fmaf(-g.z, ex, wrow[k + 2]);
        wrow[k + 3] = __builtin_fmaf(-g.w, ex, wrow[k + 3]);
      }
    }
#pragma unroll
    for (int c = 0; c < 64; ++c) sm[EX_W2S + t * EX_W2_LD + c] = wrow[c];
    if (t < 64) {
      float s = sm[EX_B2 + t];
      for (int r = 0; r < 64; ++r) s = __builtin_fmaf(-sm[EX_ETA + r], sm[EX_GZ + r * 64 + t], s);
      sm[EX_B2 + t] = s;
    }
    __syncthreads();

    // output branch with the state after the step: Z1_bar = XQ W1 + b1, X2_bar = gelu, Z2_bar = X2_bar W2 + b2, LayerNorm
    times_w1(sm + EX_XQ, w1, b1, a);
    store_column(p.Z1_bar_group + slot * 16384, a, t);
#pragma unroll
    for (int r = 0; r < 64; ++r) x2[r] = gelu_f(a[r]);
    store_column(p.X2_bar_group + slot * 16384, x2, t);
    contract_columns(x2, z2, sm, t);
    {
      const float b2 = sm[EX_B2 + lane];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int row = 16 * wave + j;
        const float z = z2[j] + b2;
        const float mu = lanes_sum(z) * (1.f / 64.f);
        const float d = z - mu;
        const float sd = sqrtf(lanes_sum(d * d) * (1.f / 64.f) + EX_LN_EPS);
        p.x_hat_ln_group[slot * 4096 + row * 64 + lane] = (bf16)(d / sd);
        if (lane == 0) p.std_ln_group[slot * 64 + row] = sd;
      }
    }
    __syncthreads();   // the input tiles and the staging tile are free for the next mini-batch
  }
}

}  // namespace ttt

hipError_t ttt_mlp_export_group0_enqueue(const ttt::BwdParams& p, hipStream_t stream) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(ttt::ttt_mlp_export_group0_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, ttt::SM_EX_BYTES);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ttt::ttt_mlp_export_group0_kernel, dim3(p.B * p.NH), dim3(ttt::EX_THREADS), ttt::SM_EX_BYTES, stream, p);
  return hipGetLastError();
}
