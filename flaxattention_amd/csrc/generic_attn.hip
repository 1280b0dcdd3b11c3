// Generic (any dtype / head size / length) attention kernels for gfx950.
//
// These are the "faithful" kernels: fp32 arithmetic on the vector ALU with the
// same operation order and, when FLEX_STRICT is set, the same dtype round trips
// as the reference's dense path (flaxattention/core/attention.py:27 rounds
// Q.K^T to the input dtype, :104-105 normalises P in fp32 and rounds it before
// P.V; the transposes of those casts round dP and dS in the backward).  They
// serve fp32 inputs, odd shapes (Dv != D, D not 64/128) and the parity mode
// for fp16/bf16.  One wave owns one row (a query row in the forward and dQ
// kernels, a key row in the dK/dV kernel) and sweeps the other sequence in
// chunks of 64 rows staged through LDS; lane j owns row j of the chunk for the
// dot products and feature j (j+64, ...) for the accumulations.
#include "flex_common.cuh"

namespace flex {

constexpr int kWaves = 4;     // waves (rows) per workgroup
constexpr int kChunk = 64;    // staged rows per step
constexpr int kMaxAcc = 4;    // features per lane: Dv, D <= 64*kMaxAcc

__host__ __device__ inline int padded_row(int d, int elt) {
  // smallest row length (elements) >= d whose size in dwords is odd
  int dw = (d * elt + 3) / 4;
  if ((dw & 1) == 0) dw += 1;
  return dw * 4 / elt;
}

__device__ __forceinline__ float wave_max(float x) {
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}
__device__ __forceinline__ float wave_sum(float x) {
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}

// stage rows [r0, r0+64) of a [L, d] matrix (row stride `stride`) into LDS
template <typename T>
__device__ __forceinline__ void stage_rows(T* dst, int dp, const T* src, int64_t stride, int r0, int L, int d) {
  constexpr int per = 4 / sizeof(T);  // elements per dword
  const int wpr = d / per;
  for (int t = threadIdx.x; t < kChunk * wpr; t += kWaves * 64) {
    int r = t / wpr, w = t % wpr;
    uint32_t val = 0;
    if (r0 + r < L) val = *reinterpret_cast<const uint32_t*>(src + (int64_t)(r0 + r) * stride + w * per);
    *reinterpret_cast<uint32_t*>(dst + r * dp + w * per) = val;
  }
}

// dot( a[0..d) fp32 (LDS, same for all lanes), row[0..d) T (LDS, per lane) )
template <typename T>
__device__ __forceinline__ float dot_row(const float* a, const T* row, int d) {
  float acc = 0.f;
  if constexpr (sizeof(T) == 4) {
    for (int x = 0; x < d; x++) acc = fmaf(a[x], (float)row[x], acc);
  } else {
    for (int x = 0; x < d; x += 2) {
      acc = fmaf(a[x], (float)row[x], acc);
      acc = fmaf(a[x + 1], (float)row[x + 1], acc);
    }
  }
  return acc;
}

struct RowCtx {
  int kind;       // score kind
  ScoreArgs sa;
  float scale;
  bool round_s;
};

// post-mod score in the base-2 domain, before masking
template <typename T>
__device__ __forceinline__ float mod_score2(float s_raw, int qi, int kv, const RowCtx& c, float* pre_mod) {
  float s = c.round_s ? round_through<T>(s_raw) : s_raw;
  s *= c.scale;
  *pre_mod = s;
  return score_apply(c.kind, s, qi, kv, c.sa) * kLog2e;
}

extern __shared__ __align__(16) unsigned char generic_smem[];

// ---------------------------------------------------------------------------
// forward: grid (ceil(Lq/kWaves), Hq, B)
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kWaves * 64) void generic_fwd_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                                  const T* __restrict__ k,
                                                                  const T* __restrict__ v, T* __restrict__ o,
                                                                  float* __restrict__ lse2) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int b = blockIdx.z, h = blockIdx.y, hk = h / (p.Hq / p.Hkv);
  const int qi = blockIdx.x * kWaves + w;
  const bool row_ok = qi < p.Lq;
  const int D = p.D, Dv = p.Dv;
  const int dpk = padded_row(D, sizeof(T)), dpv = padded_row(Dv, sizeof(T));
  T* Ks = reinterpret_cast<T*>(generic_smem);
  T* Vs = Ks + kChunk * dpk;
  float* qf = reinterpret_cast<float*>(Vs + kChunk * dpv) + w * D;
  float* pbuf = reinterpret_cast<float*>(Vs + kChunk * dpv) + kWaves * D + w * kChunk;

  const T* qrow = q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)qi * p.q_stride[2];
  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  if (row_ok) for (int x = lane; x < D; x += 64) qf[x] = (float)qrow[x];

  RowCtx c;
  c.kind = p.score.kind; c.sa = make_score_args(p.score, b, h, p.Lq, p.Lkv); c.scale = p.scale;
  c.round_s = (p.flags & (FLEX_ROUND_S | FLEX_STRICT)) != 0;
  const bool strict = (p.flags & FLEX_STRICT) != 0;
  MaskEval visible(p.mask, b, h);
  const int nchunks = (p.Lkv + kChunk - 1) / kChunk;

  // pass 1: running max and sum
  float m = -INFINITY, l = 0.f;
  for (int ch = 0; ch < nchunks; ch++) {
    __syncthreads();
    stage_rows(Ks, dpk, kbase, p.k_stride[2], ch * kChunk, p.Lkv, D);
    __syncthreads();
    const int kv = ch * kChunk + lane;
    bool vis = row_ok && kv < p.Lkv && visible(qi, kv);
    if (!__any(vis)) continue;
    float pre, x2 = mod_score2<T>(dot_row(qf, Ks + lane * dpk, D), qi, kv, c, &pre);
    x2 = vis ? x2 : -INFINITY;
    float mn = fmaxf(m, wave_max(x2));
    if (mn > -INFINITY) {
      float e = vis ? exp2f(x2 - mn) : 0.f;
      l = l * exp2f(m - mn) + wave_sum(e);
      m = mn;
    }
  }
  const float inv_l = l > 0.f ? 1.f / l : 0.f;

  // pass 2: normalised P, rounded like the reference, times V
  float acc[kMaxAcc];
  for (int a = 0; a < kMaxAcc; a++) acc[a] = 0.f;
  for (int ch = 0; ch < nchunks; ch++) {
    __syncthreads();
    stage_rows(Ks, dpk, kbase, p.k_stride[2], ch * kChunk, p.Lkv, D);
    stage_rows(Vs, dpv, vbase, p.v_stride[2], ch * kChunk, p.Lkv, Dv);
    __syncthreads();
    const int kv = ch * kChunk + lane;
    bool vis = row_ok && kv < p.Lkv && visible(qi, kv) && l > 0.f;
    if (!__any(vis)) continue;
    float pre, x2 = mod_score2<T>(dot_row(qf, Ks + lane * dpk, D), qi, kv, c, &pre);
    float pr = vis ? exp2f(x2 - m) * inv_l : 0.f;
    if (strict) pr = round_through<T>(pr);
    pbuf[lane] = pr;
    __builtin_amdgcn_wave_barrier();
    for (int j = 0; j < kChunk; j++) {
      float pj = pbuf[j];
      for (int a = 0; a < kMaxAcc; a++) {
        int d = lane + 64 * a;
        if (d < Dv) acc[a] = fmaf(pj, (float)Vs[j * dpv + d], acc[a]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (row_ok) {
    T* orow = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)qi * p.o_stride[2];
    for (int a = 0; a < kMaxAcc; a++) {
      int d = lane + 64 * a;
      if (d < Dv) orow[d] = from_f32<T>(acc[a]);
    }
    if (lse2 && lane == 0) lse2[((int64_t)b * p.Hq + h) * p.Lq + qi] = l > 0.f ? m + log2f(l) : -INFINITY;
  }
}

// ---------------------------------------------------------------------------
// dQ (+ delta): grid (ceil(Lq/kWaves), Hq, B)
// delta_i = sum_j P_ij * dP_ij, the quantity softmax' reverse-mode subtracts.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kWaves * 64) void generic_dq_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                                 const T* __restrict__ k,
                                                                 const T* __restrict__ v,
                                                                 const float* __restrict__ lse2,
                                                                 const T* __restrict__ d_o, T* __restrict__ dq,
                                                                 float* __restrict__ delta) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int b = blockIdx.z, h = blockIdx.y, hk = h / (p.Hq / p.Hkv);
  const int qi = blockIdx.x * kWaves + w;
  const bool row_ok = qi < p.Lq;
  const int D = p.D, Dv = p.Dv;
  const int dpk = padded_row(D, sizeof(T)), dpv = padded_row(Dv, sizeof(T));
  T* Ks = reinterpret_cast<T*>(generic_smem);
  T* Vs = Ks + kChunk * dpk;
  float* fbase = reinterpret_cast<float*>(Vs + kChunk * dpv);
  float* qf = fbase + w * D;
  float* dof = fbase + kWaves * D + w * Dv;
  float* pbuf = fbase + kWaves * (D + Dv) + w * kChunk;

  const int64_t row_id = ((int64_t)b * p.Hq + h) * p.Lq + qi;
  const T* qrow = q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)qi * p.q_stride[2];
  const T* dorow = d_o + row_id * Dv;  // dO is contiguous [B,Hq,Lq,Dv]
  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  if (row_ok) {
    for (int x = lane; x < D; x += 64) qf[x] = (float)qrow[x];
    for (int x = lane; x < Dv; x += 64) dof[x] = (float)dorow[x];
  }
  RowCtx c;
  c.kind = p.score.kind; c.sa = make_score_args(p.score, b, h, p.Lq, p.Lkv); c.scale = p.scale;
  c.round_s = (p.flags & (FLEX_ROUND_S | FLEX_STRICT)) != 0;
  const bool strict = (p.flags & FLEX_STRICT) != 0;
  MaskEval visible(p.mask, b, h);
  const int nchunks = (p.Lkv + kChunk - 1) / kChunk;
  const float lse = row_ok ? lse2[row_id] : -INFINITY;
  const bool alive = lse > -INFINITY;

  float dsum = 0.f;
  for (int ch = 0; ch < nchunks; ch++) {
    __syncthreads();
    stage_rows(Ks, dpk, kbase, p.k_stride[2], ch * kChunk, p.Lkv, D);
    stage_rows(Vs, dpv, vbase, p.v_stride[2], ch * kChunk, p.Lkv, Dv);
    __syncthreads();
    const int kv = ch * kChunk + lane;
    bool vis = alive && kv < p.Lkv && visible(qi, kv);
    if (!__any(vis)) continue;
    float pre, x2 = mod_score2<T>(dot_row(qf, Ks + lane * dpk, D), qi, kv, c, &pre);
    float pr = vis ? exp2f(x2 - lse) : 0.f;
    float dp = dot_row(dof, Vs + lane * dpv, Dv);
    if (strict) dp = round_through<T>(dp);
    dsum += pr * dp;
  }
  float dl = wave_sum(dsum);
  // cotangent of the log-sum-exp output: d lse / d X_ij = P_ij joins the row term
  if (p.d_lse2 && row_ok) dl -= kLog2e * p.d_lse2[row_id];
  if (row_ok && lane == 0) delta[row_id] = dl;

  float acc[kMaxAcc];
  for (int a = 0; a < kMaxAcc; a++) acc[a] = 0.f;
  for (int ch = 0; ch < nchunks; ch++) {
    __syncthreads();
    stage_rows(Ks, dpk, kbase, p.k_stride[2], ch * kChunk, p.Lkv, D);
    stage_rows(Vs, dpv, vbase, p.v_stride[2], ch * kChunk, p.Lkv, Dv);
    __syncthreads();
    const int kv = ch * kChunk + lane;
    bool vis = alive && kv < p.Lkv && visible(qi, kv);
    if (!__any(vis)) continue;
    float pre, x2 = mod_score2<T>(dot_row(qf, Ks + lane * dpk, D), qi, kv, c, &pre);
    float pr = vis ? exp2f(x2 - lse) : 0.f;
    float dp = dot_row(dof, Vs + lane * dpv, Dv);
    if (strict) dp = round_through<T>(dp);
    float ds = vis ? pr * (dp - dl) * score_grad(c.kind, pre, qi, kv, c.sa) * c.scale : 0.f;
    if (strict) ds = round_through<T>(ds);
    pbuf[lane] = ds;
    __builtin_amdgcn_wave_barrier();
    for (int j = 0; j < kChunk; j++) {
      float dj = pbuf[j];
      for (int a = 0; a < kMaxAcc; a++) {
        int d = lane + 64 * a;
        if (d < D) acc[a] = fmaf(dj, (float)Ks[j * dpk + d], acc[a]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (row_ok) {
    T* out = dq + row_id * D;
    for (int a = 0; a < kMaxAcc; a++) {
      int d = lane + 64 * a;
      if (d < D) out[d] = from_f32<T>(acc[a]);
    }
  }
}

// ---------------------------------------------------------------------------
// dK, dV: grid (ceil(Lkv/kWaves), Hkv, B); one wave per key row, lanes sweep
// the query rows of every head in the group.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kWaves * 64) void generic_dkv_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                                  const T* __restrict__ k,
                                                                  const T* __restrict__ v,
                                                                  const float* __restrict__ lse2,
                                                                  const float* __restrict__ delta,
                                                                  const T* __restrict__ d_o, T* __restrict__ dk,
                                                                  T* __restrict__ dv) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int b = blockIdx.z, hk = blockIdx.y, G = p.Hq / p.Hkv;
  const int kj = blockIdx.x * kWaves + w;
  const bool row_ok = kj < p.Lkv;
  const int D = p.D, Dv = p.Dv;
  const int dpk = padded_row(D, sizeof(T)), dpv = padded_row(Dv, sizeof(T));
  T* Qs = reinterpret_cast<T*>(generic_smem);
  T* Os = Qs + kChunk * dpk;
  float* fbase = reinterpret_cast<float*>(Os + kChunk * dpv);
  float* kf = fbase + w * D;
  float* vf = fbase + kWaves * D + w * Dv;
  float* pbuf = fbase + kWaves * (D + Dv) + w * 2 * kChunk;
  float* dsbuf = pbuf + kChunk;

  const T* krow = k + b * p.k_stride[0] + hk * p.k_stride[1] + (int64_t)kj * p.k_stride[2];
  const T* vrow = v + b * p.v_stride[0] + hk * p.v_stride[1] + (int64_t)kj * p.v_stride[2];
  if (row_ok) {
    for (int x = lane; x < D; x += 64) kf[x] = (float)krow[x];
    for (int x = lane; x < Dv; x += 64) vf[x] = (float)vrow[x];
  }
  const bool strict = (p.flags & FLEX_STRICT) != 0;
  const int nchunks = (p.Lq + kChunk - 1) / kChunk;
  float acck[kMaxAcc], accv[kMaxAcc];
  for (int a = 0; a < kMaxAcc; a++) acck[a] = accv[a] = 0.f;

  for (int g = 0; g < G; g++) {
    const int h = hk * G + g;
    RowCtx c;
    c.kind = p.score.kind; c.sa = make_score_args(p.score, b, h, p.Lq, p.Lkv); c.scale = p.scale;
    c.round_s = (p.flags & (FLEX_ROUND_S | FLEX_STRICT)) != 0;
    MaskEval visible(p.mask, b, h);
    const T* qbase = q + b * p.q_stride[0] + h * p.q_stride[1];
    const int64_t rows0 = ((int64_t)b * p.Hq + h) * p.Lq;
    const T* dobase = d_o + rows0 * Dv;
    for (int ch = 0; ch < nchunks; ch++) {
      __syncthreads();
      stage_rows(Qs, dpk, qbase, p.q_stride[2], ch * kChunk, p.Lq, D);
      stage_rows(Os, dpv, dobase, (int64_t)Dv, ch * kChunk, p.Lq, Dv);
      __syncthreads();
      const int qi = ch * kChunk + lane;
      float lse = -INFINITY, dl = 0.f;
      if (qi < p.Lq) { lse = lse2[rows0 + qi]; dl = delta[rows0 + qi]; }
      bool vis = row_ok && qi < p.Lq && lse > -INFINITY && visible(qi, kj);
      if (!__any(vis)) continue;
      float pre, x2 = mod_score2<T>(dot_row(kf, Qs + lane * dpk, D), qi, kj, c, &pre);
      float pr = vis ? exp2f(x2 - lse) : 0.f;
      float dp = dot_row(vf, Os + lane * dpv, Dv);
      if (strict) dp = round_through<T>(dp);
      float ds = vis ? pr * (dp - dl) * score_grad(c.kind, pre, qi, kj, c.sa) * c.scale : 0.f;
      if (strict) { ds = round_through<T>(ds); pr = round_through<T>(pr); }
      pbuf[lane] = pr;
      dsbuf[lane] = ds;
      __builtin_amdgcn_wave_barrier();
      for (int j = 0; j < kChunk; j++) {
        float pj = pbuf[j], dj = dsbuf[j];
        for (int a = 0; a < kMaxAcc; a++) {
          int d = lane + 64 * a;
          if (d < Dv) accv[a] = fmaf(pj, (float)Os[j * dpv + d], accv[a]);
          if (d < D) acck[a] = fmaf(dj, (float)Qs[j * dpk + d], acck[a]);
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  if (row_ok) {
    const int64_t row_id = ((int64_t)b * p.Hkv + hk) * p.Lkv + kj;
    for (int a = 0; a < kMaxAcc; a++) {
      int d = lane + 64 * a;
      if (d < D) dk[row_id * D + d] = from_f32<T>(acck[a]);
      if (d < Dv) dv[row_id * Dv + d] = from_f32<T>(accv[a]);
    }
  }
}

template <typename T> size_t generic_smem_bytes(int D, int Dv, int which) {
  size_t tiles = (size_t)kChunk * (padded_row(D, sizeof(T)) + padded_row(Dv, sizeof(T))) * sizeof(T);
  size_t f = 0;
  if (which == 0) f = (size_t)kWaves * (D + kChunk);
  else if (which == 1) f = (size_t)kWaves * (D + Dv + kChunk);
  else f = (size_t)kWaves * (D + Dv + 2 * kChunk);
  return tiles + f * sizeof(float);
}

}  // namespace flex

using namespace flex;
void flex_set_error(const char* fmt, ...);

template <typename K> static int set_smem(K kernel, size_t bytes) {
  if (bytes > 160 * 1024) { flex_set_error("generic kernel: head size needs %zu bytes of LDS (limit 163840)", bytes); return 1; }
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) { flex_set_error("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 2; }
  return 0;
}

static int check_generic(const FlexAttnParams& p) {
  if (p.D > 64 * kMaxAcc || p.Dv > 64 * kMaxAcc) { flex_set_error("generic kernels support D, Dv <= %d (got %d, %d)", 64 * kMaxAcc, p.D, p.Dv); return 1; }
  if (p.dtype != FLEX_F32 && ((p.D & 1) || (p.Dv & 1))) { flex_set_error("16-bit inputs need even D and Dv (got %d, %d)", p.D, p.Dv); return 1; }
  if (p.Hq > 65535 || p.B > 65535) { flex_set_error("B and H must be <= 65535"); return 1; }
  return 0;
}

template <typename T>
static int launch_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, hipStream_t s) {
  size_t sm = generic_smem_bytes<T>(p.D, p.Dv, 0);
  if (int rc = set_smem(generic_fwd_kernel<T>, sm)) return rc;
  dim3 grid((p.Lq + kWaves - 1) / kWaves, p.Hq, p.B);
  hipLaunchKernelGGL(generic_fwd_kernel<T>, grid, dim3(kWaves * 64), sm, s, p, (const T*)q, (const T*)k, (const T*)v, (T*)o, lse2);
  return 0;
}

template <typename T>
static int launch_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const float* lse2, const void* d_o,
                      void* dq, void* dk, void* dv, float* delta, hipStream_t s) {
  size_t sm1 = generic_smem_bytes<T>(p.D, p.Dv, 1), sm2 = generic_smem_bytes<T>(p.D, p.Dv, 2);
  if (int rc = set_smem(generic_dq_kernel<T>, sm1)) return rc;
  if (int rc = set_smem(generic_dkv_kernel<T>, sm2)) return rc;
  dim3 g1((p.Lq + kWaves - 1) / kWaves, p.Hq, p.B), g2((p.Lkv + kWaves - 1) / kWaves, p.Hkv, p.B);
  hipLaunchKernelGGL(generic_dq_kernel<T>, g1, dim3(kWaves * 64), sm1, s, p, (const T*)q, (const T*)k, (const T*)v, lse2, (const T*)d_o, (T*)dq, delta);
  hipLaunchKernelGGL(generic_dkv_kernel<T>, g2, dim3(kWaves * 64), sm2, s, p, (const T*)q, (const T*)k, (const T*)v, lse2, delta, (const T*)d_o, (T*)dk, (T*)dv);
  return 0;
}

int flex_generic_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, hipStream_t s) {
  if (int rc = check_generic(p)) return rc;
  switch (p.dtype) {
    case FLEX_F32: return launch_fwd<float>(p, q, k, v, o, lse2, s);
    case FLEX_F16: return launch_fwd<f16>(p, q, k, v, o, lse2, s);
    case FLEX_BF16: return launch_fwd<bf16>(p, q, k, v, o, lse2, s);
  }
  flex_set_error("unknown dtype %d", p.dtype);
  return 1;
}

// workspace: delta [B,Hq,Lq] fp32
int flex_generic_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const float* lse2, const void* d_o,
                     void* dq, void* dk, void* dv, float* delta, hipStream_t s) {
  if (int rc = check_generic(p)) return rc;
  switch (p.dtype) {
    case FLEX_F32: return launch_bwd<float>(p, q, k, v, lse2, d_o, dq, dk, dv, delta, s);
    case FLEX_F16: return launch_bwd<f16>(p, q, k, v, lse2, d_o, dq, dk, dv, delta, s);
    case FLEX_BF16: return launch_bwd<bf16>(p, q, k, v, lse2, d_o, dq, dk, dv, delta, s);
  }
  flex_set_error("unknown dtype %d", p.dtype);
  return 1;
}
