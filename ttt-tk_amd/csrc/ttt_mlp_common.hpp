// Shared device-side building blocks of the gfx950 TTT-MLP kernels.
//
// One workgroup of 8 wavefronts (512 threads, two per SIMD) owns one (batch, head) recurrence, or one
// role of it.  Wave v owns hidden columns [32v, 32v+32) of the inner MLP, so every per-wave contraction
// is a 64x64x32 (or 64x32x64) bf16 MFMA product with fp32 accumulate, built from 32x32x16 tiles.
//
// Register tile conventions (lane = 32*h + c, h in {0,1}, c in 0..31), verified on hardware:
//   accumulator block (32x32 fp32, 16 regs): reg i holds row 8*(i/4) + 4*h + (i%4), column c
//   operand block     (32x16 bf16,  8 slots): lane holds free index c, contraction index 8*h + slot
// A 64x64 accumulator tile whose ROWS are the contraction index of the next product can be fed
// to that product straight from registers ("chained"): packing regs 8t..8t+7 of a block gives the
// operand of k-step (2*rowblock + t) with the contraction index permuted to
//   kappa(s, h, slot) = 16*s + 8*(slot/4) + 4*h + (slot%4).
// Every operand that meets a chained operand is therefore loaded in the same kappa order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ttt {

typedef __bf16 bf16;
typedef bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int CS = 64;         // tokens per mini-batch
constexpr int FD = 64;         // head dimension
constexpr int HID = 256;       // hidden dimension of the inner MLP
constexpr int LDP = 68;        // row stride (floats) of a 64x64 fp32 partial tile in LDS: 272 B
constexpr float LN_EPS = 1e-8f;

#define TTT_DEV __device__ __forceinline__

TTT_DEV bf16x8 pack8(const f32x16& x, int t) {
  bf16x8 o;
#pragma unroll
  for (int j = 0; j < 8; j++) o[j] = (bf16)x[8 * t + j];
  return o;
}

// Two-term bf16 representation of fp32 values: hi = bf16(x), lo = bf16(x - hi), so that hi + lo carries
// about 16 significant bits.  A matrix product whose operand is split this way is the sum of one MFMA
// product per term (fp32 accumulate), which keeps the operand rounding of the products that carry the
// recurrence's state from one mini-batch to the next near 2^-17 instead of 2^-9.
// Two values at a time: one packed conversion for the high-order terms, a shift and a mask to read them back as
// fp32, two subtractions, one packed conversion for the low-order terms (6 instructions per pair).
typedef float f32x2 __attribute__((ext_vector_type(2)));
TTT_DEV void split2(float a, float b, bf16x2& hi, bf16x2& lo) {
  const f32x2 ab = {a, b};
  hi = __builtin_convertvector(ab, bf16x2);
  const uint32_t hp = __builtin_bit_cast(uint32_t, hi);
  const f32x2 r = {a - __builtin_bit_cast(float, hp << 16), b - __builtin_bit_cast(float, hp & 0xffff0000u)};
  lo = __builtin_convertvector(r, bf16x2);
}
TTT_DEV void split8(const f32x16& x, int t, bf16x8& hi, bf16x8& lo) {
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    bf16x2 h2, l2;
    split2(x[8 * t + j], x[8 * t + j + 1], h2, l2);
    hi[j] = h2[0]; hi[j + 1] = h2[1];
    lo[j] = l2[0]; lo[j + 1] = l2[1];
  }
}
TTT_DEV void split8(const float (&x)[8], bf16x8& hi, bf16x8& lo) {
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    bf16x2 h2, l2;
    split2(x[j], x[j + 1], h2, l2);
    hi[j] = h2[0]; hi[j + 1] = h2[1];
    lo[j] = l2[0]; lo[j + 1] = l2[1];
  }
}

TTT_DEV bf16x8 cat(bf16x4 lo, bf16x4 hi) { return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7); }

// Transposing LDS read: within each group of 16 lanes, lane i points at row k0 + i/4, columns m0 + 4*(i%4) .. +3,
// and receives rows k0..k0+3 of column m0 + i.
TTT_DEV bf16x4 lds_tr4(const bf16* p) {
  typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
  s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  return __builtin_bit_cast(bf16x4, t);
}

// ---------------------------------------------------------------------------- cross-lane
TTT_DEV float dpp_quad_xor1(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false));
}
TTT_DEV float dpp_quad_xor2(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false));
}
// Sum over the 4 lanes of a quad, result in all 4.
TTT_DEV float quad_sum(float x) {
  x += dpp_quad_xor1(x);
  x += dpp_quad_xor2(x);
  return x;
}
// Sum of lane l and lane l^32, result in both.
TTT_DEV float half_sum(float x) { return x + __shfl_xor(x, 32, 64); }
// The same sum without the LDS pipe, for stages that form many of them.  v_permlane32_swap exchanges the upper half of its
// first register with the lower half of its second: starting from two copies of x, one register then
// holds x[l % 32] and the other x[l % 32 + 32] in every lane.  (Written as asm: the builtin of this compiler adds the
// first result to itself.)
TTT_DEV float half_sum_valu(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
// Sum of lane l and lane l^16, result in both: v_permlane16_swap exchanges the odd rows of 16 lanes of
// its first register with the even rows of its second.
TTT_DEV float row_pair_sum(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}

// The same two sums for two values at once.  After v_permlane16_swap of (x0, x1) one register holds rows
// (x0.r0, x1.r0, x0.r2, x1.r2) and the other (x0.r1, x1.r1, x0.r3, x1.r3), so their sum carries x0's row-pair sums in
// the even rows and x1's in the odd rows; v_permlane32_swap of two such sums leaves, after the add, the totals over
// the four rows: of the first sum's two values in rows 0 and 1, of the second's in rows 2 and 3.
TTT_DEV float row_pair_sum2(float x0, float x1) {
  float a = x0, b = x1;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
TTT_DEV float half_sum2(float s01, float s23) {
  float a = s01, b = s23;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}

// vec[f0 + e] = sum over this wave's 8 LayerNorm tokens of x[e], for a wave whose lane l holds token l / 8 and the 8
// features f0 = 8 (l % 8) ... of it.  The tokens sit in the lanes that share lane % 8: lanes 8 apart inside a row of
// 16 (one rotation), then the four rows, two values per swap: in the end row r of one register holds the total of
// x[r], of the other that of x[4 + r], and lanes 0..7 of every row store their two totals.  Fixed order, fp32.
TTT_DEV void ln_token_sum_store(float* vec, const float (&x)[8], int lane, int f0) {
  float y[8];
#pragma unroll
  for (int e = 0; e < 8; e++)
    y[e] = x[e] + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x[e]), 0x128, 0xF, 0xF, false));  // row_ror:8
  const float lo = half_sum2(row_pair_sum2(y[0], y[1]), row_pair_sum2(y[2], y[3]));
  const float hi = half_sum2(row_pair_sum2(y[4], y[5]), row_pair_sum2(y[6], y[7]));
  if ((lane & 8) == 0) {
    float* d = vec + f0 + (lane >> 4);
    d[0] = lo;
    d[4] = hi;
  }
}

// ---------------------------------------------------------------------------- shape-generic tiles
// Tiles whose extent along the hidden dimension is one 32-wide block (a wave that owns 32 hidden
// columns) mix with 64-wide token / feature extents, so blocks and k-steps are template parameters.
template <int RB, int CB> struct AccT { f32x16 b[RB][CB]; };   // (32 RB) x (32 CB) fp32 tile
template <int FB, int KS> struct OpdT { bf16x8 v[FB][KS]; };   // free index 32 FB, contraction 16 KS

template <int RB, int CB>
TTT_DEV void acc_zero(AccT<RB, CB>& a) {
#pragma unroll
  for (int r = 0; r < RB; r++)
#pragma unroll
    for (int c = 0; c < CB; c++)
#pragma unroll
      for (int i = 0; i < 16; i++) a.b[r][c][i] = 0.f;
}

template <int RB, int CB, int KS>
TTT_DEV void mma(AccT<RB, CB>& d, const OpdT<RB, KS>& a, const OpdT<CB, KS>& b) {
#pragma unroll
  for (int s = 0; s < KS; s++)
#pragma unroll
    for (int r = 0; r < RB; r++)
#pragma unroll
      for (int c = 0; c < CB; c++)
        d.b[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v[r][s], b.v[c][s], d.b[r][c], 0, 0, 0);
}

// Accumulator tile (rows = contraction index) -> chained operand, contraction in kappa order.
template <int RB, int CB>
TTT_DEV OpdT<CB, 2 * RB> cvt_chain(const AccT<RB, CB>& x) {
  OpdT<CB, 2 * RB> o;
#pragma unroll
  for (int cb = 0; cb < CB; cb++)
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
      for (int t = 0; t < 2; t++) o.v[cb][2 * rb + t] = pack8(x.b[rb][cb], t);
  return o;
}

// The same with the operand split into two bf16 terms.
template <int RB, int CB>
TTT_DEV void cvt_chain_split(const AccT<RB, CB>& x, OpdT<CB, 2 * RB>& hi, OpdT<CB, 2 * RB>& lo) {
#pragma unroll
  for (int cb = 0; cb < CB; cb++)
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
      for (int t = 0; t < 2; t++) split8(x.b[rb][cb], t, hi.v[cb][2 * rb + t], lo.v[cb][2 * rb + t]);
}

// d += A * B over KS k-steps, operand pieces produced by the callables fa(row block, s) and fb(column block, s)
// right before the MFMAs that consume them, so that no whole operand is resident in registers.
template <int KS, int RB, int CB, class FA, class FB>
TTT_DEV void mma_jit(AccT<RB, CB>& d, FA fa, FB fb) {
#pragma unroll
  for (int s = 0; s < KS; s++) {
    bf16x8 a[RB], b[CB];
#pragma unroll
    for (int r = 0; r < RB; r++) a[r] = fa(r, s);
#pragma unroll
    for (int c = 0; c < CB; c++) b[c] = fb(c, s);
#pragma unroll
    for (int r = 0; r < RB; r++)
#pragma unroll
      for (int c = 0; c < CB; c++) d.b[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b[c], d.b[r][c], 0, 0, 0);
  }
}

// ---------------------------------------------------------------------------- just-in-time operand pieces
// One MFMA operand piece = 8 bf16 per lane = (free block blk, k-step s).  Loading pieces right
// before the MFMA that consumes them keeps whole operands out of the register file.
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

// Operand from an LDS tile stored [free index][contraction index], row stride ld elements.
template <int FB, int KS>
TTT_DEV OpdT<FB, KS> lds_rows_kappa(const bf16* base, int ld, int c, int h) {
  OpdT<FB, KS> o;
#pragma unroll
  for (int fb = 0; fb < FB; fb++)
#pragma unroll
    for (int s = 0; s < KS; s++) {
      const bf16* p = base + (32 * fb + c) * ld + 16 * s + 4 * h;
      o.v[fb][s] = cat(*reinterpret_cast<const bf16x4*>(p), *reinterpret_cast<const bf16x4*>(p + 8));
    }
  return o;
}

// Operand from an LDS tile stored [contraction index][free index] through the transposing read.
template <int FB, int KS>
TTT_DEV OpdT<FB, KS> lds_tr_kappa(const bf16* base, int ld, int lane) {
  OpdT<FB, KS> o;
  const int h = lane >> 5, c = lane & 31, i = lane & 15;
#pragma unroll
  for (int fb = 0; fb < FB; fb++)
#pragma unroll
    for (int s = 0; s < KS; s++) {
      const bf16* p = base + (16 * s + 4 * h + (i >> 2)) * ld + 32 * fb + 16 * (c >> 4) + 4 * (i & 3);
      o.v[fb][s] = cat(lds_tr4(p), lds_tr4(p + 8 * ld));
    }
  return o;
}

// Inverse of lds_rows_kappa: writes an operand as an LDS tile stored [free index][contraction index].
template <int FB, int KS>
TTT_DEV void lds_store_rows_kappa(bf16* base, int ld, const OpdT<FB, KS>& o, int c, int h) {
#pragma unroll
  for (int fb = 0; fb < FB; fb++)
#pragma unroll
    for (int s = 0; s < KS; s++) {
      bf16* p = base + (32 * fb + c) * ld + 16 * s + 4 * h;
      *reinterpret_cast<bf16x4*>(p) = __builtin_shufflevector(o.v[fb][s], o.v[fb][s], 0, 1, 2, 3);
      *reinterpret_cast<bf16x4*>(p + 8) = __builtin_shufflevector(o.v[fb][s], o.v[fb][s], 4, 5, 6, 7);
    }
}

// Sum over an aligned group of 8 lanes, result in all 8.
TTT_DEV float oct_sum(float x) {
  x = quad_sum(x);
  return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false));
}

// Orders this wave's LDS traffic: everything issued before is complete and nothing after is hoisted.
#define TTT_WAVE_SYNC()                                     \
  do {                                                      \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); \
    __builtin_amdgcn_wave_barrier();                        \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront"); \
  } while (0)

// ---------------------------------------------------------------------------- HBM addressing
// Every HBM access of the kernels is "wave-uniform 64-bit base + wave-uniform 32-bit offset + 32-bit
// per-lane offset".  Written this way the uniform parts stay in scalar registers (global_load /
// global_store with a scalar base and a 32-bit vector offset), so a lane needs one offset register
// per access pattern instead of one 64-bit address per access.  Buffer (MUBUF) instructions would
// give the same economy but must not be mixed with scratch traffic: the two kinds of load do not
// return in issue order on this hardware while the compiler counts them as one in-order stream.
typedef const __attribute__((address_space(1))) char* gptr_t;   // global address space: global_load / global_store
TTT_DEV unsigned uni(unsigned x) { return __builtin_amdgcn_readfirstlane(x); }   // pins a wave-uniform value to a scalar register
TTT_DEV uint64_t uni64(uint64_t a) {
  return (static_cast<uint64_t>(uni(static_cast<unsigned>(a >> 32))) << 32) | uni(static_cast<unsigned>(a));
}
TTT_DEV gptr_t gbuf(const void* base) { return (gptr_t)uni64(reinterpret_cast<uint64_t>(base)); }
template <class T>
TTT_DEV T g_ld(gptr_t b, unsigned voff, unsigned soff) {
  typedef const __attribute__((address_space(1))) T* ptr_t;
  gptr_t q = b + static_cast<uint64_t>(uni(soff));
  // The empty statements keep the scalar sum in scalar registers and the zero-extension of the lane
  // offset next to the access, which is what lets the instruction selector use the
  // "scalar base + 32-bit vector offset" form.
  asm("" : "+s"(q), "+v"(voff));
  return *(ptr_t)(q + static_cast<uint64_t>(voff));
}
template <class T>
TTT_DEV void g_st(gptr_t b, unsigned voff, unsigned soff, T v) {
  typedef __attribute__((address_space(1))) T* ptr_t;
  gptr_t q = b + static_cast<uint64_t>(uni(soff));
  asm("" : "+s"(q), "+v"(voff));
  *(ptr_t)(q + static_cast<uint64_t>(voff)) = v;
}
// Streaming variants (`nt`): data written once and read once much later, by this or another workgroup,
// should not push re-used lines out of the L2.
template <class T>
TTT_DEV void g_st_stream(gptr_t b, unsigned voff, unsigned soff, T v) {
  typedef __attribute__((address_space(1))) T* ptr_t;
  gptr_t q = b + static_cast<uint64_t>(uni(soff));
  asm("" : "+s"(q), "+v"(voff));
  __builtin_nontemporal_store(v, (ptr_t)(q + static_cast<uint64_t>(voff)));
}
template <class T>
TTT_DEV T g_ld_stream(gptr_t b, unsigned voff, unsigned soff) {
  typedef const __attribute__((address_space(1))) T* ptr_t;
  gptr_t q = b + static_cast<uint64_t>(uni(soff));
  asm("" : "+s"(q), "+v"(voff));
  return __builtin_nontemporal_load((ptr_t)(q + static_cast<uint64_t>(voff)));
}
TTT_DEV u32x4 g_ld16(gptr_t b, unsigned voff, unsigned soff) { return g_ld<u32x4>(b, voff, soff); }
TTT_DEV void g_st16(gptr_t b, unsigned voff, unsigned soff, u32x4 v) { g_st<u32x4>(b, voff, soff, v); }
TTT_DEV bf16x8 g_ld8h(gptr_t b, unsigned voff, unsigned soff) { return g_ld<bf16x8>(b, voff, soff); }
TTT_DEV void g_st8h(gptr_t b, unsigned voff, unsigned soff, bf16x8 v) { g_st<bf16x8>(b, voff, soff, v); }
TTT_DEV f32x4 g_ld4f(gptr_t b, unsigned voff, unsigned soff) { return g_ld<f32x4>(b, voff, soff); }
TTT_DEV void g_st4f(gptr_t b, unsigned voff, unsigned soff, f32x4 v) { g_st<f32x4>(b, voff, soff, v); }
TTT_DEV float g_ldf(gptr_t b, unsigned voff, unsigned soff) { return g_ld<float>(b, voff, soff); }
TTT_DEV void g_stf(gptr_t b, unsigned voff, unsigned soff, float v) { g_st<float>(b, voff, soff, v); }
TTT_DEV bf16 g_ldh(gptr_t b, unsigned voff, unsigned soff) { return g_ld<bf16>(b, voff, soff); }
TTT_DEV void g_sth(gptr_t b, unsigned voff, unsigned soff, bf16 v) { g_st<bf16>(b, voff, soff, v); }

// ---------------------------------------------------------------------------- bf16 helpers
TTT_DEV float bf_lo(uint32_t u) { return __builtin_bit_cast(float, u << 16); }
TTT_DEV float bf_hi(uint32_t u) { return __builtin_bit_cast(float, u & 0xffff0000u); }
TTT_DEV float bf2f(bf16 x) { return (float)x; }

// ---------------------------------------------------------------------------- stage clocks (instrumented builds only)
#ifdef TTT_STAGE_CLOCKS
#define TTT_STAGES_BEGIN() unsigned stage_acc[STAGE_SLOTS] = {}; unsigned stage_last = (unsigned)clock64()
#define TTT_STAGE(i) do { const unsigned t_ = (unsigned)clock64(); stage_acc[i] += t_ - stage_last; stage_last = t_; } while (0)
// `buf` = this workgroup's [8 waves][STAGE_SLOTS] part of the buffer
#define TTT_STAGES_END(buf)                                                                                \
  do {                                                                                                     \
    if ((buf) != nullptr && (threadIdx.x & 63) == 0)                                                       \
      for (int i_ = 0; i_ < STAGE_SLOTS; i_++) (buf)[(threadIdx.x >> 6) * STAGE_SLOTS + i_] = stage_acc[i_]; \
  } while (0)
#else
#define TTT_STAGES_BEGIN() ((void)0)
#define TTT_STAGE(i) ((void)0)
#define TTT_STAGES_END(buf) ((void)0)
#endif

// ---------------------------------------------------------------------------- tanh-GELU family
// gelu(x) = x * r with r = sigmoid(2c), c = K0 * x * (1 + K1 x^2); 1 - tanh(c)^2 = 4 r (1 - r).
constexpr float GK0 = 0.79788456f;
constexpr float GK1 = 0.044715f;
constexpr float GK2 = 0.1070322243f;
constexpr float LOG2E = 1.4426950408889634f;

TTT_DEV float gelu_sigmoid(float x, float u) {
  const float a = x * __builtin_fmaf(u, -2.f * GK0 * GK1 * LOG2E, -2.f * GK0 * LOG2E);  // -2c*log2(e)
  const float e = __builtin_amdgcn_exp2f(a);
  return __builtin_amdgcn_rcpf(1.f + e);
}
TTT_DEV float gelu_f(float x) { return x * gelu_sigmoid(x, x * x); }
// value and first derivative
TTT_DEV void gelu_fd(float x, float& g, float& d1) {
  const float u = x * x;
  const float r = gelu_sigmoid(x, u);
  g = x * r;
  d1 = __builtin_fmaf(g * (1.f - r), __builtin_fmaf(u, 2.f * GK2, 2.f * GK0), r);
}
// value, first and second derivative
TTT_DEV void gelu_fdd(float x, float& g, float& d1, float& d2) {
  const float u = x * x;
  const float r = gelu_sigmoid(x, u);
  const float t = __builtin_fmaf(2.f, r, -1.f);
  const float s = 4.f * r * (1.f - r);  // 1 - t^2
  g = x * r;
  const float q = __builtin_fmaf(u, GK2, GK0);  // K0 + 3 K0 K1 x^2
  d1 = __builtin_fmaf(0.5f * x * s, q, r);
  d2 = s * (__builtin_fmaf(u, 2.f * GK2, GK0) - x * t * q * q);
}

// ---------------------------------------------------------------------------- input tiles in LDS
// The input tiles (XQ, XK, XV) sit in LDS as pairs of rows: two rows of 128 bytes back to back, pairs 264 bytes
// apart.  A pair is what one wave-wide 4-byte LDS-direct load (global_load_lds_dword: lane l writes base + 4 l)
// delivers, so a tile can travel from HBM to LDS without passing through registers, and the 8 bytes between
// pairs put the 32 row-wise 8-byte reads of an operand piece on 64 distinct banks.
constexpr int XPAIR = 132;   // elements from one pair of rows to the next
TTT_DEV int xrow(int r) { return (r >> 1) * XPAIR + (r & 1) * 64; }
TTT_DEV bf16x8 xpiece_rows(const bf16* tile, int blk, int s, int c, int h) {
  const bf16* q = tile + xrow(32 * blk + c) + 16 * s + 4 * h;
  return cat(*reinterpret_cast<const bf16x4*>(q), *reinterpret_cast<const bf16x4*>(q + 8));
}
TTT_DEV bf16x8 xpiece_tr(const bf16* tile, int blk, int s, int lane) {
  const int h = lane >> 5, c = lane & 31, i = lane & 15;
  const bf16* q = tile + xrow(16 * s + 4 * h + (i >> 2)) + 32 * blk + 16 * (c >> 4) + 4 * (i & 3);
  return cat(lds_tr4(q), lds_tr4(q + 4 * XPAIR));   // 8 rows on = 4 pairs on
}
// One [64][64] bf16 tile (8 KiB at byte offset `off` of g) from HBM straight into an LDS tile of row pairs, without
// passing through registers: wave v fetches rows 8v .. 8v+7, one pair of rows (256 contiguous bytes) per load.
// Asynchronous: the data is in LDS once the wave's vmcnt has drained (and visible to other waves after a barrier).
typedef const __attribute__((address_space(1))) unsigned* gword_t;
typedef __attribute__((address_space(3))) unsigned* lword_t;
// AUX = cache policy bits of the load; CPOL_NT marks a tile that is read once (streaming), so that it does not push
// re-used lines out of the L2.
constexpr int CPOL_NT = 2;
template <int AUX = 0>
TTT_DEV void tile_to_lds(gptr_t g, unsigned off, unsigned char* tile, int v, int lane) {
  const gptr_t src = g + static_cast<uint64_t>(uni(off + v * 1024)) + static_cast<uint64_t>(4u * lane);
#pragma unroll
  for (int j = 0; j < 4; j++)
    __builtin_amdgcn_global_load_lds((gword_t)(src + 256 * j), (lword_t)(tile + (4 * v + j) * (XPAIR * 2)), 4, 0, AUX);
}
// The 64 bf16 step sizes of a mini-batch (128 bytes), by wave 0.
TTT_DEV void eta_to_lds(gptr_t g, unsigned off, unsigned char* dst, int v, int lane) {
  if (v == 0 && lane < 32)
    __builtin_amdgcn_global_load_lds((gword_t)(g + static_cast<uint64_t>(uni(off)) + static_cast<uint64_t>(4u * lane)), (lword_t)dst, 4, 0, 0);
}

// ---------------------------------------------------------------------------- workgroups that wait for each other
// Two workgroups of one (batch, head) hand work over through counters in HBM (agent scope).  Both are
// resident at once because the launchers use such a mode only when the grid fits the CUs of the device.
// A wait that sees no progress for `limit` ticks of the 100 MHz clock (20 s unless the host says otherwise)
// raises the status word and makes all workgroups of the launch leave, so every wave always exits.
TTT_DEV bool wait_at_least(int* word, int target, int* status, int* s_flag, uint64_t limit) {
  __syncthreads();   // every wave has read the flag's last value (waits follow one another, here and in wait_for_pace)
  if (threadIdx.x == 0) {
    int ok = 1;
    const uint64_t t0 = wall_clock64();
    // polled without acquire semantics (an acquire at agent scope invalidates caches on every poll);
    // one acquire fence once the value is there
    while (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0 || wall_clock64() - t0 > limit) {
        __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok = 0;
        break;
      }
      __builtin_amdgcn_s_sleep(32);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    *s_flag = ok;
  }
  // The other waves share this CU's caches with thread 0 and are ordered after its fence by the barrier.
  __syncthreads();
  return *s_flag != 0;
}
// Pacing only: waits until `word` has reached `target` without ordering any data after it (no fence, so nothing in
// the caches is invalidated).  Returns 0 if the wait gave up (as above), otherwise the value seen + 1.
TTT_DEV int wait_for_pace(int* word, int target, int* status, int* s_flag, uint64_t limit) {
  __syncthreads();   // the last value of the flag has been read by every wave
  if (threadIdx.x == 0) {
    int seen;
    const uint64_t t0 = wall_clock64();
    while ((seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) < target) {
      if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0 || wall_clock64() - t0 > limit) {
        __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        seen = -1;
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
    *s_flag = seen + 1;
  }
  __syncthreads();
  return *s_flag;
}
// Everything this workgroup has written (or read) so far is ordered before the new value of `word`: every
// wave drains its own outstanding memory operations (a workgroup-scope release alone does not wait for
// stores that are still in flight), the barrier collects the waves, then one thread writes the L2 back at
// agent scope (a release by every wave would write it back eight times over) and stores the counter.
TTT_DEV void publish(int* word, int value) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __hip_atomic_store(word, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace ttt
