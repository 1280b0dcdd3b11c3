// MFMA fragment helpers and in-register score functors for the fused kernels.
//
// Register layouts on gfx950 (wave64), with i = lane % 32 and g = lane / 32:
//   v_mfma_f32_32x32x16_{f16,bf16}:  A[m = i][k = 8g .. 8g+7],  B[k = 8g .. 8g+7][n = i],
//   C[m = 8*(r/4) + 4g + r%4][n = i] for accumulator register r = 0..15.
// The kernels compute transposed products (S^T = K.Q^T, O^T = V^T.P^T, ...) so
// that the *column* index n -- one query row per lane -- is what a lane owns:
// row statistics (max, sum, lse, delta) are per-lane scalars and the
// accumulator of one product is already laid out as the B operand of the next.
#pragma once
#include "flex_common.cuh"

namespace flex {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));

template <typename T> struct Frag;
template <> struct Frag<f16> {
  typedef half8_t vec8;
  static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Frag<bf16> {
  typedef bf16x8_t vec8;
  static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// kv (or row) offset of accumulator register r inside a 32-row block, minus 4g
__device__ __forceinline__ constexpr int acc_row(int r) { return 8 * (r / 4) + (r % 4); }

// exchange with lane ^ 32 and combine
__device__ __forceinline__ float xhalf_max(float x) {
  unsigned u = __float_as_uint(x);
  uint2_t r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
  unsigned u = __float_as_uint(x);
  uint2_t r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Transposing LDS read (ds_read_b64_tr_b16).  Within each group of 16 lanes,
// lane s supplies the address of 4 consecutive 16-bit elements; lane i receives
// element (i % 4) of lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4.  With lane s
// pointing at M[row0 + s/4][col0 + 4*(s%4) ..], lane i ends up with
// M[row0 + 0..3][col0 + i]: a column of a row-major tile, which is what an
// MFMA operand needs when the contraction runs over rows.
template <typename T>
__device__ __forceinline__ short4_t lds_read_tr(const T* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(p));
}

template <typename V> __device__ __forceinline__ V join8(short4_t lo, short4_t hi) {
  short8_t x = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(V, x);
}

// ---------------------------------------------------------------------------
// Score functors in the base-2 domain.  x2 = log2(e) * score_mod(scale * s).
// `off` is the compile-time part of the key index (kv = kvb + off) once the
// register loops are unrolled; tile() receives the lane's query index and kvb.
// grad() is d score_mod / d(scaled score) at the same point.
// ---------------------------------------------------------------------------
template <int KIND> struct Score2;

template <> struct Score2<FLEX_SCORE_IDENTITY> {
  static constexpr bool kGradOne = true;  // d score_mod / d score == 1 everywhere
  float c;
  __device__ __forceinline__ void init(const FlexScoreMod&, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) { c = scale * kLog2e; }
  __device__ __forceinline__ void tile(int q, int kvb) {}
  __device__ __forceinline__ void tileT(int qb, int kv) {}
  __device__ __forceinline__ float apply(float s, int off) const { return s * c; }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const { return fmaf(s, c, -m); }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

template <> struct Score2<FLEX_SCORE_CHECKERBOARD> {
  static constexpr bool kGradOne = false;  // d score_mod / d score == 1 everywhere
  float c0, c1, f0, f1;  // factor (x scale x log2e) for even / odd parity
  float ce, co, fe, fo;  // the same, resolved for even / odd `off` of this lane
  int by_kv;
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) {
    f0 = m.p0; f1 = m.p1; c0 = m.p0 * scale * kLog2e; c1 = m.p1 * scale * kLog2e; by_kv = m.i0;
  }
  // Every caller passes an even kvb (tiles start at multiples of 32, lane halves at multiples of 4), so the parity
  // at off = 0 is that of the lane's query row alone: nothing here depends on the key tile, and the compiler moves
  // the four selects out of the tile loops (they were 8 % of a forward block's vector instructions).
  __device__ __forceinline__ void tile(int q, int kvb) {
    int par = by_kv ? 0 : (q & 1);  // parity of kvb (- q) at off = 0
    ce = par ? c1 : c0; co = par ? c0 : c1;
    fe = par ? f1 : f0; fo = par ? f0 : f1;
  }
  // off runs along the query index instead (q = qb + off, fixed kv); qb is even in every caller (query tiles start at
  // multiples of 32, lane halves at multiples of 4): the parity at off = 0 is that of the lane's key
  __device__ __forceinline__ void tileT(int qb, int kv) {
    int par = kv & 1;
    ce = par ? c1 : c0; fe = par ? f1 : f0;
    if (by_kv) { co = ce; fo = fe; } else { co = par ? c0 : c1; fo = par ? f0 : f1; }
  }
  __device__ __forceinline__ float apply(float s, int off) const { return s * ((off & 1) ? co : ce); }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const { return fmaf(s, (off & 1) ? co : ce, -m); }
  __device__ __forceinline__ float grad(float s, int off) const { return (off & 1) ? fo : fe; }
};

// Checkerboard keyed on the key index alone, for kernels in which a lane owns one key
// (dK/dV): factor and derivative are per-lane constants, so the derivative leaves the
// inner loop and scales the lane's dK row once at the end (key_grad).
constexpr int kScoreCheckerboardKv = 100;
template <> struct Score2<kScoreCheckerboardKv> {
  static constexpr bool kGradOne = true;  // inside the loop; see key_grad
  float c0, c1, f0, f1, ck, key_grad;
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) {
    f0 = m.p0; f1 = m.p1; c0 = m.p0 * scale * kLog2e; c1 = m.p1 * scale * kLog2e;
  }
  __device__ __forceinline__ void tileT(int qb, int kv) {
    ck = (kv & 1) ? c1 : c0;
    key_grad = (kv & 1) ? f1 : f0;
  }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const { return fmaf(s, ck, -m); }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

// Checkerboard with positive factors, for a kernel that only needs dS = P o (dP - delta) o g
// (dQ): the derivative g is the factor itself, and P.g = 2^(x + log2 g), so log2 g joins the
// constant subtracted in the exponent and the derivative costs nothing per element.
constexpr int kScoreCheckerboardFold = 101;
template <> struct Score2<kScoreCheckerboardFold> {
  static constexpr bool kGradOne = true;  // folded into the exponent
  float c0, c1, l0, l1;
  float ce, co, le, lo;
  int by_kv;
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) {
    c0 = m.p0 * scale * kLog2e; c1 = m.p1 * scale * kLog2e; l0 = log2f(m.p0); l1 = log2f(m.p1); by_kv = m.i0;
  }
  __device__ __forceinline__ void tile(int q, int kvb) {
    int par = by_kv ? 0 : (q & 1);  // parity of kvb (- q) at off = 0: kvb is even in every caller, see above
    ce = par ? c1 : c0; co = par ? c0 : c1;
    le = par ? l1 : l0; lo = par ? l0 : l1;
  }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const {
    return (off & 1) ? fmaf(s, co, lo - m) : fmaf(s, ce, le - m);
  }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

template <> struct Score2<FLEX_SCORE_ALIBI> {
  static constexpr bool kGradOne = true;  // d score_mod / d score == 1 everywhere
  float c, slope2, base, step;
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) {
    c = scale * kLog2e;
    slope2 = m.p0 * exp2f(-((float)(h + 1) * 8.0f / (float)m.i0)) * kLog2e;
  }
  __device__ __forceinline__ void tile(int q, int kvb) { base = (float)(q - kvb) * slope2; step = -slope2; }
  __device__ __forceinline__ void tileT(int qb, int kv) { base = (float)(qb - kv) * slope2; step = slope2; }
  __device__ __forceinline__ float apply(float s, int off) const { return fmaf(s, c, fmaf((float)off, step, base)); }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const { return fmaf(s, c, fmaf((float)off, step, base - m)); }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

template <> struct Score2<FLEX_SCORE_REL_BIAS> {
  static constexpr bool kGradOne = true;  // d score_mod / d score == 1 everywhere
  float c, slope2, base, step;
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) {
    c = scale * kLog2e;
    slope2 = m.p0 * kLog2e;
  }
  __device__ __forceinline__ void tile(int q, int kvb) { base = (float)(kvb - q) * slope2; step = slope2; }
  __device__ __forceinline__ void tileT(int qb, int kv) { base = (float)(kv - qb) * slope2; step = -slope2; }
  __device__ __forceinline__ float apply(float s, int off) const { return fmaf(s, c, fmaf((float)off, step, base)); }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const { return fmaf(s, c, fmaf((float)off, step, base - m)); }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

template <> struct Score2<FLEX_SCORE_TANH_SOFTCAP> {
  static constexpr bool kGradOne = false;  // d score_mod / d score == 1 everywhere
  float a, cap2, sc;  // a = 2*log2e*scale/cap, cap2 = cap*log2e
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) {
    a = 2.f * kLog2e * scale * m.p1; cap2 = m.p0 * kLog2e; sc = scale;
  }
  __device__ __forceinline__ void tile(int q, int kvb) {}
  __device__ __forceinline__ void tileT(int qb, int kv) {}
  __device__ __forceinline__ float tanh_(float s) const {
    // no clamp: for a large argument v_exp_f32 gives +inf, v_rcp_f32 of that 0, and the result is exactly 1
    float t = fast_exp2(s * a);
    return 1.f - 2.f * fast_rcp(t + 1.f);
  }
  // r = 1 / (2^(a s) + 1), tanh = 1 - 2 r: cap2 * tanh - m = (cap2 - m) - 2 cap2 r, one fused multiply-add per entry
  // (cap2 - m is common to the entries of a block)
  __device__ __forceinline__ float half_gap(float s) const { return fast_rcp(fast_exp2(s * a) + 1.f); }
  __device__ __forceinline__ float apply(float s, int off) const { return fmaf(-2.f * cap2, half_gap(s), cap2); }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const { return fmaf(-2.f * cap2, half_gap(s), cap2 - m); }
  __device__ __forceinline__ float grad(float s, int off) const { float t = tanh_(s); return 1.f - t * t; }
};

// score + add[b,h,q,kv] from a dense fp32 table (FLEX_SCORE_AFFINE without a multiplicative table:
// what a score_mod that adds a captured bias is lowered to).  The 16 table entries of a lane's
// block are fetched when the block is entered; indices are clamped to the table (entries past the
// ends of the sequences are masked out by the caller whatever they hold).
template <> struct Score2<FLEX_SCORE_AFFINE> {
  static constexpr bool kGradOne = true;  // d score_mod / d score == 1 everywhere
  float c;
  const float* add_bh;
  int64_t sq;
  int q_last, kv_last;
  float bias[16];  // log2(e) * add for accumulator register r (key / query offset acc_row(r))
  static __device__ __forceinline__ constexpr int reg_of(int off) { return 4 * (off / 8) + (off % 4); }
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) {
    c = scale * kLog2e;
    add_bh = m.add + b * m.stride_b + h * m.stride_h;
    sq = m.stride_q;
    q_last = Lq - 1;
    kv_last = Lkv - 1;
  }
  __device__ __forceinline__ void tile(int q, int kvb) {
    const float* row = add_bh + (int64_t)min(q, q_last) * sq;
#pragma unroll
    for (int r = 0; r < 16; r++) bias[r] = row[min(kvb + acc_row(r), kv_last)] * kLog2e;
  }
  __device__ __forceinline__ void tileT(int qb, int kv) {
    const float* col = add_bh + min(kv, kv_last);
#pragma unroll
    for (int r = 0; r < 16; r++) bias[r] = col[(int64_t)min(qb + acc_row(r), q_last) * sq] * kLog2e;
  }
  __device__ __forceinline__ float apply(float s, int off) const { return fmaf(s, c, bias[reg_of(off)]); }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const { return fmaf(s, c, bias[reg_of(off)] - m); }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

// mul[b,h,q,kv] * score + add[b,h,q,kv] from dense fp32 tables (FLEX_SCORE_AFFINE with a multiplicative table: what
// a score_mod that scales the score by a captured or position-dependent factor is lowered to, and what an arbitrary
// differentiable score_mod becomes once it is linearised at the scores of the call).  Both tables' entries of a lane's
// block are fetched when the block is entered; the derivative is the multiplicative entry itself.
constexpr int kScoreAffineMul = 102;
template <> struct Score2<kScoreAffineMul> {
  static constexpr bool kGradOne = false;
  float c;
  const float* add_bh;
  const float* mul_bh;
  int64_t sq;
  int q_last, kv_last;
  float bias[16], fac[16];  // log2(e) * add and mul for accumulator register r
  static __device__ __forceinline__ constexpr int reg_of(int off) { return 4 * (off / 8) + (off % 4); }
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h, int b = 0, int Lq = 0, int Lkv = 0) {
    c = scale * kLog2e;
    const int64_t off = b * m.stride_b + h * m.stride_h;
    add_bh = m.add ? m.add + off : nullptr;
    mul_bh = m.mul + off;
    sq = m.stride_q;
    q_last = Lq - 1;
    kv_last = Lkv - 1;
  }
  __device__ __forceinline__ void tile(int q, int kvb) {
    const int64_t row = (int64_t)min(q, q_last) * sq;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int64_t at = row + min(kvb + acc_row(r), kv_last);
      fac[r] = mul_bh[at];
      bias[r] = add_bh ? add_bh[at] * kLog2e : 0.f;
    }
  }
  __device__ __forceinline__ void tileT(int qb, int kv) {
    const int col = min(kv, kv_last);
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int64_t at = (int64_t)min(qb + acc_row(r), q_last) * sq + col;
      fac[r] = mul_bh[at];
      bias[r] = add_bh ? add_bh[at] * kLog2e : 0.f;
    }
  }
  __device__ __forceinline__ float apply(float s, int off) const { return fmaf(s * fac[reg_of(off)], c, bias[reg_of(off)]); }
  __device__ __forceinline__ float apply_sub(float s, int off, float m) const {
    return fmaf(s * fac[reg_of(off)], c, bias[reg_of(off)] - m);
  }
  __device__ __forceinline__ float grad(float s, int off) const { return fac[reg_of(off)]; }
};

// band / bitmap mask evaluated at (q, kv)
struct Mask2 {
  MaskEval ev;
  int Lkv;
  __device__ __forceinline__ Mask2(const FlexMask& m, int b, int h, int Lkv_) : ev(m, b, h), Lkv(Lkv_) {}
  __device__ __forceinline__ bool operator()(int q, int kv) const { return kv < Lkv && ev(q, kv); }
};

// ---------------------------------------------------------------------------
// Tile-level mask application, hoisted out of the per-element code so that the
// unmasked path stays one straight-line block.
//
// Band masks: with d = q + q_offset - kv, a key is visible iff
//     d >= lo  &&  (d <= hi || kv <= sink)  &&  kv < Lkv.
// Inside a 32-key block a register's key is kvb + off with `off` a compile-time
// constant, so every condition becomes a comparison of `off` with a per-lane
// bound:  off <= up  &&  (off >= wlo || off <= snk).  Bounds are clamped to
// +-2^30 so that no subtraction overflows (sequence positions are far smaller).
// ---------------------------------------------------------------------------
// a mask that hides nothing: without tile lists every tile then counts as fully visible, otherwise as partial
__host__ __device__ __forceinline__ bool mask_hides_nothing(const FlexMask& m) {
  return m.kind == FLEX_MASK_BAND && m.lo == INT32_MIN && m.hi == INT32_MAX;
}
constexpr int kBig = 1 << 30;
__device__ __forceinline__ int clamp_big(int x) { return min(max(x, -kBig), kBig); }

// Wave-uniform classification of one 32-query x 32-key block under a band mask:
// kBlockAll = every entry visible (no mask evaluation needed), kBlockNone = nothing visible,
// kBlockMixed = evaluate per element.  q_first / kv_first are the block's first query row and
// key (wave-uniform values).  Bitmap masks are always kBlockMixed.
enum { kBlockMixed = 0, kBlockAll = 1, kBlockNone = 2 };
__device__ __forceinline__ int band_block_class(const FlexMask& m, int q_first, int kv_first, int Lq, int Lkv) {
  if (m.kind != FLEX_MASK_BAND) return kBlockMixed;
  const int lo = clamp_big(m.lo), hi = clamp_big(m.hi), snk = clamp_big(m.sink);
  const int q_last = q_first + 31, kv_last = kv_first + 31;
  const int dmin = q_first + m.q_offset - kv_last, dmax = q_last + m.q_offset - kv_first;
  if (dmin >= lo && (dmax <= hi || kv_last <= snk) && kv_last < Lkv && q_last < Lq) return kBlockAll;
  if (dmax < lo || (dmin > hi && kv_first > snk) || kv_first >= Lkv || q_first >= Lq) return kBlockNone;
  return kBlockMixed;
}
// The same for any mask: a bitmap answers from its table of block classes when it carries one.
// q_first and kv_first are multiples of 32.  The table describes the padded index range, so a
// block that reaches past the real lengths is never reported as entirely visible.
// KNOWN_BITS: the caller knows that the mask is a bitmap (no band arithmetic is compiled in).
template <bool KNOWN_BITS = false>
__device__ __forceinline__ int block_class(const FlexMask& m, const Mask2& visible, int q_first, int kv_first, int Lq,
                                           int Lkv) {
  if (!KNOWN_BITS && m.kind == FLEX_MASK_BAND) return band_block_class(m, q_first, kv_first, Lq, Lkv);
  if (!visible.ev.blk_bh) return kBlockMixed;
  if (kv_first >= Lkv || q_first >= Lq) return kBlockNone;
  const int c = visible.ev.blk_bh[(int64_t)(q_first >> 5) * visible.ev.blk_stride_q + (kv_first >> 5)];
  if (c == kBlockAll && (kv_first + 31 >= Lkv || (Lq - 31 <= q_first))) return kBlockMixed;
  return c;
}
__device__ __forceinline__ void fill_masked(float16_t& x) {
#pragma unroll
  for (int r = 0; r < 16; r++) x[r] = -INFINITY;
}

// one 32-key block: register r holds key kv0 + 4*g + acc_row(r); lane owns query q
// BITS = false: the caller knows that the mask is a band mask.
template <bool BITS = true, bool KNOWN_BITS = false>
__device__ __forceinline__ void mask_block_q(float16_t& x, const FlexMask& m, const Mask2& visible, int q, int kv0, int g,
                                             int Lkv) {
  const int kvb = kv0 + 4 * g;
  if (!KNOWN_BITS && (!BITS || m.kind == FLEX_MASK_BAND)) {
    const int dq = q + m.q_offset - kvb;                           // d at off = 0; d = dq - off
    const int up = min(dq - clamp_big(m.lo), Lkv - 1 - kvb);       // off <= up  <=>  d >= lo && kv < Lkv
    if (m.hi >= kBig) {
#pragma unroll
      for (int r = 0; r < 16; r++) x[r] = (acc_row(r) <= up) ? x[r] : -INFINITY;
    } else {
      const int wlo = dq - m.hi;                                    // off >= wlo <=> d <= hi
      const int snk = clamp_big(m.sink) - kvb;                      // off <= snk <=> kv <= sink
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int off = acc_row(r);
        const bool vis = (off <= up) & ((off >= wlo) | (off <= snk));
        x[r] = vis ? x[r] : -INFINITY;
      }
    }
  } else {
    const uint32_t w = visible.ev.bits_bh[(int64_t)q * visible.ev.stride_q + (kv0 >> 5)] >> (4 * g);
    const int up = Lkv - 1 - kvb;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int off = acc_row(r);
      const bool vis = ((w >> off) & 1u) & (off <= up);
      x[r] = vis ? x[r] : -INFINITY;
    }
  }
}
// a 64-key tile = two blocks
__device__ __forceinline__ void mask_tile_q(float16_t (&x)[2], const FlexMask& m, const Mask2& visible, int q, int kv0,
                                            int g, int Lkv) {
  mask_block_q(x[0], m, visible, q, kv0, g, Lkv);
  mask_block_q(x[1], m, visible, q, kv0 + 32, g, Lkv);
}

// Lane owns key kv; register r holds query qb + acc_row(r) (qb already includes 4*g).
// BITS = false: the caller knows that the mask is a band mask.
template <bool BITS, bool KNOWN_BITS = false>
__device__ __forceinline__ void mask_block_kv(float16_t& x, const FlexMask& m, const Mask2& visible, int qb, int kv,
                                              int Lq, int Lkv) {
  if (!KNOWN_BITS && (!BITS || m.kind == FLEX_MASK_BAND)) {
    const int dq = qb + m.q_offset - kv;                          // d = dq + off
    const int lo_off = clamp_big(m.lo) - dq;                      // off >= lo_off <=> d >= lo
    const int up = (kv < Lkv) ? (Lq - 1 - qb) : -1;               // off <= up <=> q < Lq (and the key exists)
    const int whi = (kv <= m.sink) ? kBig : (clamp_big(m.hi) - dq);  // off <= whi <=> d <= hi || kv <= sink
    const int hi_off = min(up, whi);
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int off = acc_row(r);
      const bool vis = (off >= lo_off) & (off <= hi_off);
      x[r] = vis ? x[r] : -INFINITY;
    }
  } else if (visible.ev.bits_t_bh) {
    // query-packed copy: the 32 query rows of this block (qb = 32-aligned row + 4*g) are one word of key kv
    const uint32_t w = kv < Lkv ? visible.ev.bits_t_bh[(int64_t)kv * visible.ev.stride_kv + (qb >> 5)] >> (qb & 31) : 0u;
    const int up = Lq - 1 - qb;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int off = acc_row(r);
      const bool vis = ((w >> off) & 1u) & (off <= up);
      x[r] = vis ? x[r] : -INFINITY;
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int qi = qb + acc_row(r);
      const bool vis = qi < Lq && visible(qi, kv);
      x[r] = vis ? x[r] : -INFINITY;
    }
  }
}

// Pairs of 16-bit values: packed conversion and a fused row-sum.
template <typename T> struct Pair;
template <> struct Pair<f16> {
  typedef _Float16 v2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ v2 pack(float a, float b) { v2 h = {(_Float16)a, (_Float16)b}; return h; }
  static __device__ __forceinline__ float add_sum(v2 h, float acc) {
    const v2 one = {(_Float16)1.f, (_Float16)1.f};
    return __builtin_amdgcn_fdot2(h, one, acc, false);
  }
};
template <> struct Pair<bf16> {
  typedef __bf16 v2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ v2 pack(float a, float b) { v2 h = {(__bf16)a, (__bf16)b}; return h; }
  static __device__ __forceinline__ float add_sum(v2 h, float acc) {
    const v2 one = {(__bf16)1.f, (__bf16)1.f};
    return __builtin_amdgcn_fdot2_f32_bf16(h, one, acc, false);
  }
};
// Round two fp32 values through T with ONE packed conversion.  The empty asm
// keeps the pair opaque so that the compiler does not split it back into two
// scalar conversions; widening back to fp32 then fuses into the consumer
// (v_fma_mix_f32 reads either half of an f16 pair as an operand).  No real
// instruction is hidden inside asm here: MFMA results must only ever be read by
// instructions the compiler's hazard handling can see.
template <typename T> __device__ __forceinline__ typename Pair<T>::v2 round_pack(float a, float b) {
  typedef float f2 __attribute__((ext_vector_type(2)));
  const f2 ab = {a, b};
  typename Pair<T>::v2 h = __builtin_convertvector(ab, typename Pair<T>::v2);
  unsigned u = __builtin_bit_cast(unsigned, h);
  asm("" : "+v"(u));
  return __builtin_bit_cast(typename Pair<T>::v2, u);
}
// Split two fp32 values into a high and a low pair of T: hi = T(x), lo = T(x - hi).  A matrix product that is
// issued once with each pair sees x with twice T's mantissa (16 bits for bf16, 22 for fp16): how the "unrounded"
// numerics carry P and dS, which the dense path would hold in fp32 if its internal round trips are optimised away.
template <typename T>
__device__ __forceinline__ void split_pack(float a, float b, typename Pair<T>::v2& hi, typename Pair<T>::v2& lo) {
  hi = round_pack<T>(a, b);
  lo = Pair<T>::pack(a - (float)hi[0], b - (float)hi[1]);
}
template <typename T> __device__ __forceinline__ void round_pair(float& a, float& b) {
  typename Pair<T>::v2 h = round_pack<T>(a, b);
  a = (float)h[0];
  b = (float)h[1];
}
// three-input max without the NaN-quieting canonicalisation the compiler adds to fmaxf
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
template <typename T> __device__ __forceinline__ typename Frag<T>::vec8 join_pairs(typename Pair<T>::v2 a, typename Pair<T>::v2 b,
                                                                                    typename Pair<T>::v2 c, typename Pair<T>::v2 d) {
  auto ab = __builtin_shufflevector(a, b, 0, 1, 2, 3);
  auto cd = __builtin_shufflevector(c, d, 0, 1, 2, 3);
  return __builtin_shufflevector(ab, cd, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ float block_max(const float16_t& x) {
  float a = max3(x[0], x[1], x[2]), b = max3(x[3], x[4], x[5]);
#pragma unroll
  for (int r = 6; r < 14; r += 4) {
    a = max3(a, x[r], x[r + 1]);
    b = max3(b, x[r + 2], x[r + 3]);
  }
  return max3(max3(a, b, x[14]), x[15], x[15]);
}

// maximum of the 32 accumulator values of a lane: two independent chains of v_max3
__device__ __forceinline__ float tile_max(const float16_t (&x)[2]) {
  float a = max3(x[0][0], x[0][1], x[0][2]), b = max3(x[1][0], x[1][1], x[1][2]);
#pragma unroll
  for (int r = 3; r < 15; r += 2) {
    a = max3(a, x[0][r], x[0][r + 1]);
    b = max3(b, x[1][r], x[1][r + 1]);
  }
  return max3(max3(a, b, x[0][15]), x[1][15], x[1][15]);
}

// LDS stages as separate variables, selected at compile time: the compiler tracks a direct global -> LDS fetch per
// variable, so a read of one stage does not wait for a fetch into another only if every access names its
// variable statically.
template <int S> struct StageC { static constexpr int value = S; };
template <int S, typename P> __device__ __forceinline__ P* stage_ptr(StageC<S>, P* s0, P* s1) { return S == 0 ? s0 : s1; }
template <int S, typename P> __device__ __forceinline__ P* stage_ptr(StageC<S>, P* s0, P* s1, P* s2) {
  return S == 0 ? s0 : (S == 1 ? s1 : s2);
}

// Tile-list entries (written by an earlier launch, never by these kernels) are read through the constant
// address space: the entry lands in a scalar register, the addresses derived from it stay wave-uniform, and
// waiting for it does not wait for the vector loads in flight.
__device__ __forceinline__ int uniform_ld(const int32_t* ptr) {
  return *(const __attribute__((address_space(4))) int32_t*)ptr;
}

// Unpadded LDS tiles (rows of 2D bytes, so that a wave-wide direct global -> LDS load can fill 1 KB
// of consecutive rows): the 16-byte chunk c of row r is kept at chunk position c ^ lds_swz<D>(r),
// a function of r & 15 chosen so that both kinds of operand reads are free of bank conflicts
// (64 banks of 4 bytes; measured: 2.1 ns per ds_read_b128 and 1.7 ns per ds_read_b64_tr_b16 per
// compute unit, the same as for linear addresses, where rows padded by 16 bytes take 1.9 ns (D = 64)
// and 3.6 ns (D = 128) per transposing read and c ^ (r & 7) at D = 64 3.8 ns per ds_read_b128):
//   row-fragment reads: 16 lanes read one chunk column of 16 consecutive rows -> the 16 rows must
//     land in 16 different 16-byte slots of the 256-byte bank period;
//   transposing reads: 16 lanes read 2 chunks of 4 consecutive rows, 32 lanes 4 chunks -> the 4 rows
//     must land in different 64-byte quarters of the period.
// D = 64 (128-byte rows, two per period): bit 2 of the chunk follows bit 1 of r, bits 0-1 follow
// bits 2-3.  D = 128 (one row per period): bits 2-3 follow bits 0-1 of r, bits 0-1 follow bits 2-3.
// D = 192 (384-byte rows, one and a half periods: odd rows start half a period in, which supplies bit 3 of the
// slot): only the low three bits may move, or a chunk would leave its row of 24; bit 2 follows bit 1 of r, bits 0-1
// follow bits 2-3.  D = 256 (two periods per row) takes the D = 128 rule.
template <int D> __device__ __forceinline__ constexpr int lds_swz(int r) {
  return (D == 64 || D == 192) ? (((r & 2) << 1) | ((r >> 2) & 3)) : (((r & 3) << 2) | ((r >> 2) & 3));
}

// XCD-aware, heavy-first workgroup map.  Hardware deals consecutive workgroup ids
// round-robin to the 8 XCDs (each has its own L2) and starts them in id order as
// slots free up.  Every XCD gets a contiguous share of the (batch, head) pairs, so
// workgroups that read the same K/V meet in one L2; inside an XCD the ids run
// tile-major -- all heads' heaviest tile first, then the next heaviest -- so that
// under causal-like masks the long workgroups start first and the short ones fill
// the tail.  `rank` counts tiles from the heaviest (0) to the lightest (ntile-1).
__device__ __forceinline__ void xcd_tile_map(int wid, int ntile, int nbh, int& rank, int& bh) {
  constexpr int kXcd = 8;
  if (nbh % kXcd == 0) {
    const int per = nbh / kXcd;           // heads per XCD
    const int xcd = wid % kXcd, local = wid / kXcd;
    rank = local / per;
    bh = xcd * per + local % per;
  } else {
    rank = wid / nbh;
    bh = wid % nbh;
  }
}

}  // namespace flex
