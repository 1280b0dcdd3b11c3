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
  float c;
  __device__ __forceinline__ void init(const FlexScoreMod&, float scale, int h) { c = scale * kLog2e; }
  __device__ __forceinline__ void tile(int q, int kvb) {}
  __device__ __forceinline__ void tileT(int qb, int kv) {}
  __device__ __forceinline__ float apply(float s, int off) const { return s * c; }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

template <> struct Score2<FLEX_SCORE_CHECKERBOARD> {
  float c0, c1, f0, f1;  // factor (x scale x log2e) for even / odd parity
  float ce, co, fe, fo;  // the same, resolved for even / odd `off` of this lane
  int by_kv;
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h) {
    f0 = m.p0; f1 = m.p1; c0 = m.p0 * scale * kLog2e; c1 = m.p1 * scale * kLog2e; by_kv = m.i0;
  }
  __device__ __forceinline__ void tile(int q, int kvb) {
    int par = (by_kv ? kvb : (kvb - q)) & 1;  // parity at off = 0
    ce = par ? c1 : c0; co = par ? c0 : c1;
    fe = par ? f1 : f0; fo = par ? f0 : f1;
  }
  // off runs along the query index instead (q = qb + off, fixed kv)
  __device__ __forceinline__ void tileT(int qb, int kv) {
    int par = (by_kv ? kv : (kv - qb)) & 1;
    ce = par ? c1 : c0; fe = par ? f1 : f0;
    if (by_kv) { co = ce; fo = fe; } else { co = par ? c0 : c1; fo = par ? f0 : f1; }
  }
  __device__ __forceinline__ float apply(float s, int off) const { return s * ((off & 1) ? co : ce); }
  __device__ __forceinline__ float grad(float s, int off) const { return (off & 1) ? fo : fe; }
};

template <> struct Score2<FLEX_SCORE_ALIBI> {
  float c, slope2, base, step;
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h) {
    c = scale * kLog2e;
    slope2 = m.p0 * exp2f(-((float)(h + 1) * 8.0f / (float)m.i0)) * kLog2e;
  }
  __device__ __forceinline__ void tile(int q, int kvb) { base = (float)(q - kvb) * slope2; step = -slope2; }
  __device__ __forceinline__ void tileT(int qb, int kv) { base = (float)(qb - kv) * slope2; step = slope2; }
  __device__ __forceinline__ float apply(float s, int off) const { return fmaf(s, c, fmaf((float)off, step, base)); }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

template <> struct Score2<FLEX_SCORE_REL_BIAS> {
  float c, slope2, base, step;
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h) {
    c = scale * kLog2e;
    slope2 = m.p0 * kLog2e;
  }
  __device__ __forceinline__ void tile(int q, int kvb) { base = (float)(kvb - q) * slope2; step = slope2; }
  __device__ __forceinline__ void tileT(int qb, int kv) { base = (float)(kv - qb) * slope2; step = -slope2; }
  __device__ __forceinline__ float apply(float s, int off) const { return fmaf(s, c, fmaf((float)off, step, base)); }
  __device__ __forceinline__ float grad(float s, int off) const { return 1.f; }
};

template <> struct Score2<FLEX_SCORE_TANH_SOFTCAP> {
  float a, cap2, sc;  // a = 2*log2e*scale/cap, cap2 = cap*log2e
  __device__ __forceinline__ void init(const FlexScoreMod& m, float scale, int h) {
    a = 2.f * kLog2e * scale * m.p1; cap2 = m.p0 * kLog2e; sc = scale;
  }
  __device__ __forceinline__ void tile(int q, int kvb) {}
  __device__ __forceinline__ void tileT(int qb, int kv) {}
  __device__ __forceinline__ float tanh_(float s) const {
    float t = fast_exp2(fminf(s * a, 60.f));
    return 1.f - 2.f * fast_rcp(t + 1.f);
  }
  __device__ __forceinline__ float apply(float s, int off) const { return cap2 * tanh_(s); }
  __device__ __forceinline__ float grad(float s, int off) const { float t = tanh_(s); return 1.f - t * t; }
};

// band / bitmap mask evaluated at (q, kv)
struct Mask2 {
  MaskEval ev;
  int Lkv;
  __device__ __forceinline__ Mask2(const FlexMask& m, int b, int h, int Lkv_) : ev(m, b, h), Lkv(Lkv_) {}
  __device__ __forceinline__ bool operator()(int q, int kv) const { return kv < Lkv && ev(q, kv); }
};

// XCD-aware workgroup remap: hardware deals consecutive workgroup ids round-robin
// to the 8 XCDs, each with its own L2.  Give every XCD a contiguous range of
// logical ids so that workgroups sharing K/V (same batch and head) share an L2.
__device__ __forceinline__ int xcd_remap(int wid, int total) {
  constexpr int kXcd = 8;
  if (total % kXcd != 0) return wid;
  return (wid % kXcd) * (total / kXcd) + wid / kXcd;
}

}  // namespace flex
