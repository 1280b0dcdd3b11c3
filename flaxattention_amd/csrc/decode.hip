// Split-KV decode for gfx950: short queries (G * Lq <= 64 columns) against a
// long KV cache, bound by HBM bandwidth.
//
// Serves the decode shapes of examples/benchmark_decoding.py:29-33 (the
// reference pads q to 16 rows and runs its prefill kernel, attention.py:269-273).
//
// Grid: (splits, Hkv, B).  A workgroup owns a contiguous range of 32-row KV
// steps; its four waves take steps round-robin and never synchronise with each
// other until the end, so many independent 8 KB K/V reads are in flight per CU.
// Per step and wave:
//   K rows go straight from global memory into MFMA A-operand registers
//   (lane i holds 16-byte pieces of row kv0 + i%32) -- no LDS round trip;
//   V rows pass through a wave-private LDS strip to be read back transposed.
//   All query heads that share a KV head (GQA) are packed into the N columns of
//   the MFMA, so K and V are read once per group.
// Each workgroup writes an unnormalised partial (O, m, l) per column; a second
// kernel merges the splits:  O = sum_s 2^(m_s-m) O_s / sum_s 2^(m_s-m) l_s.
#include "mfma_common.cuh"

namespace flex {

constexpr int kStep = 32;  // KV rows per wave step

template <typename T, int D, int KIND, bool ROUND_S, int NB>
__global__ __launch_bounds__(256) void decode_split_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                            const T* __restrict__ k, const T* __restrict__ v,
                                                            float* __restrict__ o_part, float* __restrict__ ml_part,
                                                            int splits) {
  typedef typename Frag<T>::vec8 vec8;
  constexpr int DS = D / 16, DB = D / 32, ROWE = D + 8, CPR = D / 8, NV = kStep * CPR / 64;
  __shared__ __align__(16) T Vs[4][kStep * ROWE];
  __shared__ float mbuf[4][NB][32];
  __shared__ __align__(16) float red[4][16][64];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5, i16 = lane & 15;
  const int split = blockIdx.x, hk = blockIdx.y, b = blockIdx.z;
  const int G = p.Hq / p.Hkv;
  const int ncols = G * p.Lq;

  // this lane's columns
  int col_h[NB], col_q[NB];
  bool col_ok[NB];
  vec8 qf[NB][DS];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const int c = nb * 32 + i32;
    col_ok[nb] = c < ncols;
    const int cc = col_ok[nb] ? c : 0;
    col_h[nb] = hk * G + cc / p.Lq;
    col_q[nb] = cc % p.Lq;
    const T* qp = q + b * p.q_stride[0] + col_h[nb] * p.q_stride[1] + (int64_t)col_q[nb] * p.q_stride[2] + 8 * g;
#pragma unroll
    for (int s = 0; s < DS; s++) qf[nb][s] = *reinterpret_cast<const vec8*>(qp + 16 * s);
  }

  // schedule: list entries (64-row tiles of query block 0) when given and G == 1, else every step
  const FlexTileLists& tl = p.tiles;
  const int32_t* full_idx = nullptr;
  const int32_t* part_idx = nullptr;
  int n_full = 0, steps_total;
  if (tl.kv_num && G == 1) {
    const int64_t row = (b * tl.stride_b + hk * tl.stride_h) * tl.n_q_blocks;
    n_full = tl.full_kv_num[row];
    const int n_part = tl.kv_num[row];
    full_idx = tl.full_kv_idx + row * tl.n_kv_blocks;
    part_idx = tl.kv_idx + row * tl.n_kv_blocks;
    steps_total = 2 * (n_full + n_part);
  } else {
    steps_total = (p.Lkv + kStep - 1) / kStep;
  }
  auto step_kv0 = [&](int st) -> int {
    if (!full_idx) return st * kStep;
    const int item = st >> 1;
    const int tile = item < n_full ? full_idx[item] : part_idx[item - n_full];
    return tile * 64 + (st & 1) * kStep;
  };
  const int per = (steps_total + splits - 1) / splits;
  const int st_begin = split * per, st_end = min(st_begin + per, steps_total);

  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  const int64_t ks2 = p.k_stride[2], vs2 = p.v_stride[2];

  vec8 kfr[DS];
  uint4 vreg[NV];
  auto load_step = [&](int kv0) {
    const int kr = kv0 + i32;
    if (kr < p.Lkv) {
      const T* kp = kbase + (int64_t)kr * ks2 + 8 * g;
#pragma unroll
      for (int s = 0; s < DS; s++) kfr[s] = *reinterpret_cast<const vec8*>(kp + 16 * s);
    } else {
#pragma unroll
      for (int s = 0; s < DS; s++)
#pragma unroll
        for (int e = 0; e < 8; e++) kfr[s][e] = (T)0.f;
    }
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int c = lane + 64 * j, r = c / CPR, cc = c % CPR;
      vreg[j] = (kv0 + r < p.Lkv) ? *reinterpret_cast<const uint4*>(vbase + (int64_t)(kv0 + r) * vs2 + cc * 8)
                                  : make_uint4(0, 0, 0, 0);
    }
  };

  Score2<KIND> sm[NB];
  float m_run[NB], l_run[NB];
  float16_t oacc[NB][DB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    sm[nb].init(p.score, p.scale, col_h[nb]);
    m_run[nb] = -INFINITY;
    l_run[nb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[nb][db][r] = 0.f;
  }
  const bool trivial_mask = p.mask.kind == FLEX_MASK_BAND && p.mask.lo == INT32_MIN && p.mask.hi == INT32_MAX;
  T* Vw = Vs[w];

  int st = st_begin + w;
  if (st < st_end) load_step(step_kv0(st));
  for (; st < st_end; st += 4) {
    const int kv0 = step_kv0(st);
    vec8 kcur[DS];
#pragma unroll
    for (int s = 0; s < DS; s++) kcur[s] = kfr[s];
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int c = lane + 64 * j, r = c / CPR, cc = c % CPR;
      *reinterpret_cast<uint4*>(Vw + r * ROWE + cc * 8) = vreg[j];
    }
    if (st + 4 < st_end) load_step(step_kv0(st + 4));
    const bool need_mask = !trivial_mask || (kv0 + kStep > p.Lkv);

    vec8 pf[NB][2];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      float16_t sacc;
#pragma unroll
      for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
      for (int s = 0; s < DS; s++) sacc = Frag<T>::mfma(kcur[s], qf[nb][s], sacc);
      const int kvb = kv0 + 4 * g;
      sm[nb].tile(col_q[nb], kvb);
      Mask2 visible(p.mask, b, col_h[nb], p.Lkv);
      float mloc = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float s = sacc[r];
        if (ROUND_S) s = round_through<T>(s);
        float x = sm[nb].apply(s, acc_row(r));
        if (need_mask) x = visible(col_q[nb], kvb + acc_row(r)) ? x : -INFINITY;
        sacc[r] = x;
        mloc = fmaxf(mloc, x);
      }
      const float m_new = fmaxf(m_run[nb], xhalf_max(mloc));
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = fast_exp2(m_run[nb] - m_use);
      m_run[nb] = m_new;
      float lsum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float pe = fast_exp2(sacc[r] - m_use);
        lsum += pe;
        pf[nb][r / 8][r % 8] = (T)pe;
      }
      l_run[nb] = l_run[nb] * alpha + lsum;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[nb][db][r] *= alpha;
    }
    // V strip was written by this wave only: wait for its LDS writes, no workgroup barrier
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < 2; t++) {
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const T* vp = Vw + (16 * t + 4 * g + (i16 >> 2)) * ROWE + 32 * db + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
        vec8 a = join8<vec8>(lds_read_tr(vp), lds_read_tr(vp + 8 * ROWE));
#pragma unroll
        for (int nb = 0; nb < NB; nb++) oacc[nb][db] = Frag<T>::mfma(a, pf[nb][t], oacc[nb][db]);
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
  }

  // ---- merge the four waves ----
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    l_run[nb] = xhalf_sum(l_run[nb]);
    if (g == 0) mbuf[w][nb][i32] = m_run[nb];
  }
  __syncthreads();
  float m_all[NB], l_scaled[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    float mm = fmaxf(fmaxf(mbuf[0][nb][i32], mbuf[1][nb][i32]), fmaxf(mbuf[2][nb][i32], mbuf[3][nb][i32]));
    m_all[nb] = mm;
    const float sc = (m_run[nb] == -INFINITY) ? 0.f : fast_exp2(m_run[nb] - mm);
    l_scaled[nb] = l_run[nb] * sc;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[nb][db][r] *= sc;
  }
  __syncthreads();
  // l: reuse mbuf
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
    if (g == 0) mbuf[w][nb][i32] = l_scaled[nb];
  __syncthreads();
  const int64_t part_rows = (int64_t)p.B * p.Hq * p.Lq;
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const int64_t row_id = ((int64_t)b * p.Hq + col_h[nb]) * p.Lq + col_q[nb];
    if (w == 0 && g == 0 && col_ok[nb]) {
      float lt = mbuf[0][nb][i32] + mbuf[1][nb][i32] + mbuf[2][nb][i32] + mbuf[3][nb][i32];
      float* ml = ml_part + ((int64_t)split * part_rows + row_id) * 2;
      ml[0] = m_all[nb];
      ml[1] = lt;
    }
#pragma unroll
    for (int db = 0; db < DB; db++) {
      const int blk = nb * DB + db;
      __syncthreads();
#pragma unroll
      for (int r = 0; r < 16; r++) red[w][r][lane] = oacc[nb][db][r];
      __syncthreads();
      if (w == (blk & 3) && col_ok[nb]) {
        float* op = o_part + ((int64_t)split * part_rows + row_id) * D + 32 * db + 4 * g;
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
          float4_t acc4;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const int r = 4 * rr + e;
            acc4[e] = red[0][r][lane] + red[1][r][lane] + red[2][r][lane] + red[3][r][lane];
          }
          *reinterpret_cast<float4_t*>(op + 8 * rr) = acc4;
        }
      }
    }
  }
}

// one wave per output row: merge the splits, normalise, write O and lse2
template <typename T, int D>
__global__ __launch_bounds__(256) void decode_combine_kernel(FlexAttnParams p, const float* __restrict__ o_part,
                                                              const float* __restrict__ ml_part, int splits,
                                                              T* __restrict__ o, float* __restrict__ lse2) {
  const int lane = threadIdx.x & 63;
  const int64_t rows = (int64_t)p.B * p.Hq * p.Lq;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float m = -INFINITY;
  for (int s = 0; s < splits; s++) m = fmaxf(m, ml_part[(s * rows + row) * 2]);
  float l = 0.f, acc[D / 64];
#pragma unroll
  for (int a = 0; a < D / 64; a++) acc[a] = 0.f;
  for (int s = 0; s < splits; s++) {
    const float ms = ml_part[(s * rows + row) * 2];
    const float sc = (ms == -INFINITY) ? 0.f : fast_exp2(ms - m);
    l += sc * ml_part[(s * rows + row) * 2 + 1];
#pragma unroll
    for (int a = 0; a < D / 64; a++) acc[a] += sc * o_part[(s * rows + row) * D + lane + 64 * a];
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  const int qi = (int)(row % p.Lq);
  const int h = (int)((row / p.Lq) % p.Hq), b = (int)(row / ((int64_t)p.Lq * p.Hq));
  T* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)qi * p.o_stride[2];
#pragma unroll
  for (int a = 0; a < D / 64; a++) op[lane + 64 * a] = (T)(acc[a] * inv);
  if (lse2 && lane == 0) lse2[row] = l > 0.f ? m + log2f(l) : -INFINITY;
}

template <typename T, int D, int KIND, bool RS>
static void launch_nb(const FlexAttnParams& p, const void* q, const void* k, const void* v, float* o_part, float* ml_part,
                      int splits, hipStream_t s) {
  dim3 grid(splits, p.Hkv, p.B);
  const int ncols = (p.Hq / p.Hkv) * p.Lq;
  if (ncols <= 32)
    hipLaunchKernelGGL((decode_split_kernel<T, D, KIND, RS, 1>), grid, dim3(256), 0, s, p, (const T*)q, (const T*)k, (const T*)v, o_part, ml_part, splits);
  else
    hipLaunchKernelGGL((decode_split_kernel<T, D, KIND, RS, 2>), grid, dim3(256), 0, s, p, (const T*)q, (const T*)k, (const T*)v, o_part, ml_part, splits);
}

template <typename T, int D, int KIND>
static void launch_rs(const FlexAttnParams& p, const void* q, const void* k, const void* v, float* o_part, float* ml_part,
                      int splits, hipStream_t s) {
  if (p.flags & FLEX_ROUND_S) launch_nb<T, D, KIND, true>(p, q, k, v, o_part, ml_part, splits, s);
  else launch_nb<T, D, KIND, false>(p, q, k, v, o_part, ml_part, splits, s);
}

template <typename T, int D>
static int launch_all(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                      float* o_part, float* ml_part, hipStream_t s) {
  switch (p.score.kind) {
    case FLEX_SCORE_IDENTITY: launch_rs<T, D, FLEX_SCORE_IDENTITY>(p, q, k, v, o_part, ml_part, splits, s); break;
    case FLEX_SCORE_CHECKERBOARD: launch_rs<T, D, FLEX_SCORE_CHECKERBOARD>(p, q, k, v, o_part, ml_part, splits, s); break;
    case FLEX_SCORE_ALIBI: launch_rs<T, D, FLEX_SCORE_ALIBI>(p, q, k, v, o_part, ml_part, splits, s); break;
    case FLEX_SCORE_TANH_SOFTCAP: launch_rs<T, D, FLEX_SCORE_TANH_SOFTCAP>(p, q, k, v, o_part, ml_part, splits, s); break;
    case FLEX_SCORE_REL_BIAS: launch_rs<T, D, FLEX_SCORE_REL_BIAS>(p, q, k, v, o_part, ml_part, splits, s); break;
    default: return 1;
  }
  const int64_t rows = (int64_t)p.B * p.Hq * p.Lq;
  hipLaunchKernelGGL((decode_combine_kernel<T, D>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, p, o_part, ml_part, splits, (T*)o, lse2);
  return 0;
}

}  // namespace flex

using namespace flex;
void flex_set_error(const char* fmt, ...);
bool flex_mfma_shape_ok(const FlexAttnParams& p);

bool flex_decode_supported(const FlexAttnParams& p) {
  if (!flex_mfma_shape_ok(p)) return false;
  return (int64_t)(p.Hq / p.Hkv) * p.Lq <= 64 && p.Hkv <= 65535 && p.B <= 65535;
}

int flex_decode_default_splits(const FlexAttnParams& p) {
  // aim for about four workgroups per CU (256 CUs), at least 8 steps per workgroup
  const int steps = (p.Lkv + kStep - 1) / kStep;
  int64_t heads = (int64_t)p.B * p.Hkv;
  int s = (int)((1024 + heads - 1) / heads);
  if (s > steps / 8) s = steps / 8;
  if (s < 1) s = 1;
  if (s > 64) s = 64;
  return s;
}

size_t flex_decode_workspace(const FlexAttnParams& p, int splits) {
  const size_t rows = (size_t)p.B * p.Hq * p.Lq;
  return (rows * splits * (p.D + 2) * sizeof(float) + 255) / 256 * 256;
}

int flex_decode_launch(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                       void* workspace, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)workspace) & 15) {
    flex_set_error("decode needs 16-byte aligned tensors");
    return 1;
  }
  if (splits > 65535) { flex_set_error("decode: too many splits (%d)", splits); return 1; }
  const size_t rows = (size_t)p.B * p.Hq * p.Lq;
  float* o_part = (float*)workspace;
  float* ml_part = o_part + rows * splits * p.D;
  int rc;
  if (p.dtype == FLEX_F16) rc = p.D == 64 ? launch_all<f16, 64>(p, q, k, v, o, lse2, splits, o_part, ml_part, s)
                                          : launch_all<f16, 128>(p, q, k, v, o, lse2, splits, o_part, ml_part, s);
  else rc = p.D == 64 ? launch_all<bf16, 64>(p, q, k, v, o, lse2, splits, o_part, ml_part, s)
                      : launch_all<bf16, 128>(p, q, k, v, o, lse2, splits, o_part, ml_part, s);
  if (rc) flex_set_error("decode: unsupported score_mod kind %d", p.score.kind);
  return rc;
}
