// Shared device helpers: dtype conversion, score_mod / mask_mod functors.
// gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/flexattn.h"

namespace flex {

typedef _Float16 f16;
typedef __bf16 bf16;
typedef float f32;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <typename T> struct DTypeOf;
template <> struct DTypeOf<float> { static constexpr int value = FLEX_F32; };
template <> struct DTypeOf<f16> { static constexpr int value = FLEX_F16; };
template <> struct DTypeOf<bf16> { static constexpr int value = FLEX_BF16; };

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x) { return (T)x; }
// round an fp32 value through T (round-to-nearest-even) and back
template <typename T> __device__ __forceinline__ float round_through(float x) { return (float)((T)x); }
template <> __device__ __forceinline__ float round_through<float>(float x) { return x; }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// ---------------------------------------------------------------------------
// score_mod functors.  `s` is the scaled score (attention.py:55 scales before
// the mod is applied, attention.py:59-63).  Each functor also gives
// d(mod)/d(score), which the backward multiplies in
// (kernel/attention.py:459-468 evaluates jax.grad(score_mod) at the pre-mod
// scaled score).
// ---------------------------------------------------------------------------
struct ScoreArgs {
  float p0, p1;
  int32_t i0;
  float slope;  // ALiBi: exp2(-(h+1)*8/H) of the current head
  const float* mul_bh;  // affine tables of the current (b, h), or null
  const float* add_bh;
  int64_t stride_q;
  int32_t q_last, kv_last;  // table bounds: kernels evaluate functors on padded indices too
};

__device__ __forceinline__ ScoreArgs make_score_args(const FlexScoreMod& m, int b, int h, int Lq, int Lkv) {
  ScoreArgs a;
  a.p0 = m.p0; a.p1 = m.p1; a.i0 = m.i0; a.slope = 0.f;
  a.mul_bh = nullptr; a.add_bh = nullptr; a.stride_q = 0;
  a.q_last = Lq - 1; a.kv_last = Lkv - 1;
  if (m.kind == FLEX_SCORE_ALIBI) a.slope = exp2f(-((float)(h + 1) * 8.0f / (float)m.i0));
  if (m.kind == FLEX_SCORE_AFFINE) {
    const int64_t off = b * m.stride_b + h * m.stride_h;
    a.mul_bh = m.mul ? m.mul + off : nullptr;
    a.add_bh = m.add ? m.add + off : nullptr;
    a.stride_q = m.stride_q;
  }
  return a;
}

template <int KIND> struct ScoreMod;

template <> struct ScoreMod<FLEX_SCORE_IDENTITY> {
  static __device__ __forceinline__ float apply(float s, int q, int kv, const ScoreArgs&) { return s; }
  static __device__ __forceinline__ float grad(float s, int q, int kv, const ScoreArgs&) { return 1.f; }
};
template <> struct ScoreMod<FLEX_SCORE_CHECKERBOARD> {
  static __device__ __forceinline__ float factor(int q, int kv, const ScoreArgs& a) {
    int par = (a.i0 == 0 ? (kv - q) : kv) & 1;  // two's complement == floor-mod 2
    return par ? a.p1 : a.p0;
  }
  static __device__ __forceinline__ float apply(float s, int q, int kv, const ScoreArgs& a) { return s * factor(q, kv, a); }
  static __device__ __forceinline__ float grad(float s, int q, int kv, const ScoreArgs& a) { return factor(q, kv, a); }
};
template <> struct ScoreMod<FLEX_SCORE_ALIBI> {
  static __device__ __forceinline__ float apply(float s, int q, int kv, const ScoreArgs& a) {
    return s + (float)(q - kv) * (a.p0 * a.slope);
  }
  static __device__ __forceinline__ float grad(float s, int q, int kv, const ScoreArgs&) { return 1.f; }
};
template <> struct ScoreMod<FLEX_SCORE_TANH_SOFTCAP> {
  static __device__ __forceinline__ float tanh_(float x) {
    // tanh(x) = 1 - 2/(exp(2x)+1); exp2 argument clamped so the result
    // saturates to +-1 without overflow
    float t = fast_exp2(fminf(2.f * kLog2e * x, 60.f));
    return 1.f - 2.f * fast_rcp(t + 1.f);
  }
  static __device__ __forceinline__ float apply(float s, int q, int kv, const ScoreArgs& a) {
    return a.p0 * tanh_(s * a.p1);  // p1 = 1/cap
  }
  static __device__ __forceinline__ float grad(float s, int q, int kv, const ScoreArgs& a) {
    float t = tanh_(s * a.p1);
    return 1.f - t * t;
  }
};
template <> struct ScoreMod<FLEX_SCORE_REL_BIAS> {
  static __device__ __forceinline__ float apply(float s, int q, int kv, const ScoreArgs& a) {
    return s + (float)(kv - q) * a.p0;
  }
  static __device__ __forceinline__ float grad(float s, int q, int kv, const ScoreArgs&) { return 1.f; }
};

template <> struct ScoreMod<FLEX_SCORE_AFFINE> {
  // indices past the end (padding rows / columns of a chunk, masked out by the caller) are clamped
  static __device__ __forceinline__ int64_t at(int q, int kv, const ScoreArgs& a) {
    return (int64_t)min(max(q, 0), a.q_last) * a.stride_q + min(max(kv, 0), a.kv_last);
  }
  static __device__ __forceinline__ float mul(int q, int kv, const ScoreArgs& a) {
    return a.mul_bh ? a.mul_bh[at(q, kv, a)] : 1.f;
  }
  static __device__ __forceinline__ float apply(float s, int q, int kv, const ScoreArgs& a) {
    const float c = a.add_bh ? a.add_bh[at(q, kv, a)] : 0.f;
    return fmaf(s, mul(q, kv, a), c);
  }
  static __device__ __forceinline__ float grad(float s, int q, int kv, const ScoreArgs& a) { return mul(q, kv, a); }
};

// runtime dispatch for the kernels that are not templated on the functor
__device__ __forceinline__ float score_apply(int kind, float s, int q, int kv, const ScoreArgs& a) {
  switch (kind) {
    case FLEX_SCORE_CHECKERBOARD: return ScoreMod<FLEX_SCORE_CHECKERBOARD>::apply(s, q, kv, a);
    case FLEX_SCORE_ALIBI: return ScoreMod<FLEX_SCORE_ALIBI>::apply(s, q, kv, a);
    case FLEX_SCORE_TANH_SOFTCAP: return ScoreMod<FLEX_SCORE_TANH_SOFTCAP>::apply(s, q, kv, a);
    case FLEX_SCORE_REL_BIAS: return ScoreMod<FLEX_SCORE_REL_BIAS>::apply(s, q, kv, a);
    case FLEX_SCORE_AFFINE: return ScoreMod<FLEX_SCORE_AFFINE>::apply(s, q, kv, a);
    default: return s;
  }
}
__device__ __forceinline__ float score_grad(int kind, float s, int q, int kv, const ScoreArgs& a) {
  switch (kind) {
    case FLEX_SCORE_CHECKERBOARD: return ScoreMod<FLEX_SCORE_CHECKERBOARD>::grad(s, q, kv, a);
    case FLEX_SCORE_TANH_SOFTCAP: return ScoreMod<FLEX_SCORE_TANH_SOFTCAP>::grad(s, q, kv, a);
    case FLEX_SCORE_AFFINE: return ScoreMod<FLEX_SCORE_AFFINE>::grad(s, q, kv, a);
    default: return 1.f;
  }
}

// ---------------------------------------------------------------------------
// mask_mod functor
// ---------------------------------------------------------------------------
struct MaskEval {
  int32_t kind, lo, hi, sink, q_offset;
  const uint32_t* bits_bh;  // bitmap row base of the current (b, h)
  int64_t stride_q;
  const uint32_t* bits_t_bh;  // the same bitmap packed along the query axis (may be null)
  int64_t stride_kv;
  const int8_t* blk_bh;  // class of every aligned 32x32 block of the bitmap (may be null)
  int64_t blk_stride_q;

  __device__ __forceinline__ MaskEval(const FlexMask& m, int b, int h) {
    kind = m.kind; lo = m.lo; hi = m.hi; sink = m.sink; q_offset = m.q_offset;
    bits_bh = m.bits ? m.bits + b * m.bits_stride_b + h * m.bits_stride_h : nullptr;
    stride_q = m.bits_stride_q;
    bits_t_bh = m.bits_t ? m.bits_t + b * m.bits_t_stride_b + h * m.bits_t_stride_h : nullptr;
    stride_kv = m.bits_t_stride_kv;
    blk_bh = m.blk ? m.blk + b * m.blk_stride_b + h * m.blk_stride_h : nullptr;
    blk_stride_q = m.blk_stride_q;
  }
  __device__ __forceinline__ bool operator()(int q, int kv) const {
    if (kind == FLEX_MASK_BAND) {
      int d = q + q_offset - kv;
      return (d >= lo) && ((d <= hi) || (kv <= sink));
    }
    uint32_t w = bits_bh[(int64_t)q * stride_q + (kv >> 5)];
    return (w >> (kv & 31)) & 1u;
  }
};

}  // namespace flex
