// Fused flash-attention forward for gfx950 (fp16 / bf16, D = Dv in {64, 128}).
//
// Takes the place of mha_forward_kernel (flaxattention/kernel/attention.py:
// 34-149) and of the dense math path (flaxattention/core/attention.py:14-106)
// for 16-bit inputs, with a real online softmax and with skipping of masked-out
// KV tiles, which the reference computes but never uses.
//
// Work decomposition: one workgroup (4 waves) per 128 query rows of one
// (batch, head); each wave owns 32 query rows.  KV tiles of 64 rows are staged
// through LDS (register-prefetched one tile ahead).  Per tile and wave:
//   S^T[kv, q]  = K_tile . Q^T          8 x v_mfma_f32_32x32x16 (D = 64)
//   online softmax in the accumulator layout: a lane holds 32 of the 64 scores
//   of ONE query row, the other 32 sit in lane ^ 32 -> row max/sum are
//   in-register reductions plus one permlane32 swap
//   O^T[d, q] += V_tile^T . P^T         8 x v_mfma (P^T is already in B-operand
//   layout; V^T fragments come from transposing LDS reads)
#include "mfma_common.cuh"

namespace flex {

constexpr int kFwdBM = 128;
constexpr int kFwdBN = 64;

template <typename T, int D, int KIND, bool ROUND_S>
__global__ __launch_bounds__(256, D == 64 ? 3 : 2) void fwd_mfma_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                           const T* __restrict__ k, const T* __restrict__ v,
                                                           T* __restrict__ o, float* __restrict__ lse2) {
  typedef typename Frag<T>::vec8 vec8;
  constexpr int BM = kFwdBM, BN = kFwdBN;
  constexpr int DS = D / 16;     // k-steps of the Q.K^T product
  constexpr int DB = D / 32;     // 32-row blocks of O^T
  constexpr int ROWE = D + 8;    // LDS row length in elements (16 B of padding)
  constexpr int CPR = D / 8;     // 16-byte chunks per row
  constexpr int NLD = BN * CPR / 256;  // chunks per thread per tile
  __shared__ __align__(16) T Ks[BN * ROWE];
  __shared__ __align__(16) T Vs[BN * ROWE];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5, i16 = lane & 15;
  const int nqt = (p.Lq + BM - 1) / BM;
  const int total = nqt * p.Hq * p.B;
  int rank, bh;
  xcd_tile_map(blockIdx.x, nqt, p.Hq * p.B, rank, bh);
  const int qt = nqt - 1 - rank;  // late query tiles see the most keys under causal masks
  const int h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);

  const int q_row = qt * BM + w * 32 + i32;
  const int q_ld = min(q_row, p.Lq - 1);

  // Q fragments (B operand of S^T = K.Q^T), resident for the whole kernel
  vec8 qf[DS];
  {
    const T* qp = q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)q_ld * p.q_stride[2] + 8 * g;
#pragma unroll
    for (int s = 0; s < DS; s++) qf[s] = *reinterpret_cast<const vec8*>(qp + 16 * s);
  }

  // tile schedule
  const FlexTileLists& tl = p.tiles;
  const int32_t* full_idx = nullptr;
  const int32_t* part_idx = nullptr;
  int n_full, n_part = 0;
  if (tl.kv_num) {
    const int64_t row = (b * tl.stride_b + h * tl.stride_h) * tl.n_q_blocks + qt;
    n_full = tl.full_kv_num[row];
    n_part = tl.kv_num[row];
    full_idx = tl.full_kv_idx + row * tl.n_kv_blocks;
    part_idx = tl.kv_idx + row * tl.n_kv_blocks;
  } else {
    n_full = (p.Lkv + BN - 1) / BN;
  }
  const int nt = n_full + n_part;
  auto tile_at = [&](int it) -> int {
    if (!full_idx) return it;
    return it < n_full ? full_idx[it] : part_idx[it - n_full];
  };

  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  const int64_t ks2 = p.k_stride[2], vs2 = p.v_stride[2];

  uint4 kreg[NLD], vreg[NLD];
  auto load_tile = [&](int kv0) {
#pragma unroll
    for (int j = 0; j < NLD; j++) {
      int c = tid + 256 * j, r = c / CPR, cc = c % CPR;
      int kv = kv0 + r;
      if (kv < p.Lkv) {
        kreg[j] = *reinterpret_cast<const uint4*>(kbase + (int64_t)kv * ks2 + cc * 8);
        vreg[j] = *reinterpret_cast<const uint4*>(vbase + (int64_t)kv * vs2 + cc * 8);
      } else {
        kreg[j] = make_uint4(0, 0, 0, 0);
        vreg[j] = make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < NLD; j++) {
      int c = tid + 256 * j, r = c / CPR, cc = c % CPR;
      *reinterpret_cast<uint4*>(Ks + r * ROWE + cc * 8) = kreg[j];
      *reinterpret_cast<uint4*>(Vs + r * ROWE + cc * 8) = vreg[j];
    }
  };

  Score2<KIND> sm;
  sm.init(p.score, p.scale, h);
  Mask2 visible(p.mask, b, h, p.Lkv);

  float16_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[db][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  constexpr float kTau = 8.f;  // lazy rescale: keep the running reference max until it is beaten by 2^8
  int t_cur = nt > 0 ? tile_at(0) : 0;
  int t_nxt = nt > 1 ? tile_at(1) : 0;
  if (nt > 0) load_tile(t_cur * BN);
  for (int it = 0; it < nt; it++) {
    const int kv0 = t_cur * BN;
    const bool masked = (it >= n_full) || (kv0 + BN > p.Lkv);
    store_tile();
    __syncthreads();
    if (it + 1 < nt) load_tile(t_nxt * BN);
    t_cur = t_nxt;
    if (it + 2 < nt) t_nxt = tile_at(it + 2);

    // Each 32-row half of the tile is one online-softmax step (keeps only 16
    // score registers live, which is what lets four waves share a SIMD).
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
      // ---- S^T = K . Q^T ----
      float16_t sacc;
#pragma unroll
      for (int r = 0; r < 16; r++) sacc[r] = 0.f;
      const T* kp = Ks + (nb * 32 + i32) * ROWE + 8 * g;
#pragma unroll
      for (int s = 0; s < DS; s++) {
        vec8 a = *reinterpret_cast<const vec8*>(kp + 16 * s);
        sacc = Frag<T>::mfma(a, qf[s], sacc);
      }

      // ---- score_mod relative to the running reference max, tile mask where needed ----
      const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
      sm.tile(q_row, kv0 + nb * 32 + 4 * g);
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float s0 = sacc[r], s1 = sacc[r + 1];
        if (ROUND_S) round_pair<T>(s0, s1);
        sacc[r] = sm.apply_sub(s0, acc_row(r), m_use);
        sacc[r + 1] = sm.apply_sub(s1, acc_row(r + 1), m_use);
      }
      if (masked) mask_block_q(sacc, p.mask, visible, q_row, kv0 + nb * 32, g, p.Lkv);

      // ---- online softmax; the reference max moves only when it is beaten by 2^kTau ----
      const float m_rel = xhalf_max(block_max(sacc));
      const bool need = (m_rel > kTau) || (m_run == -INFINITY && m_rel > -INFINITY);
      if (__any(need)) {
        const float delta = need ? m_rel : 0.f;
        const float alpha = (m_run == -INFINITY) ? 0.f : fast_exp2(-delta);
        m_run = need ? (m_use + m_rel) : m_run;
        l_run *= alpha;
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] -= delta;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[db][r] *= alpha;
      }
      vec8 pf[2];
#pragma unroll
      for (int tt = 0; tt < 2; tt++) {
        typename Pair<T>::v2 pr[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float p0 = fast_exp2(sacc[8 * tt + 2 * e]);
          const float p1 = fast_exp2(sacc[8 * tt + 2 * e + 1]);
          pr[e] = Pair<T>::pack(p0, p1);
          l_run = Pair<T>::add_sum(pr[e], l_run);
        }
        pf[tt] = join_pairs<T>(pr[0], pr[1], pr[2], pr[3]);
      }

      // ---- O^T += V^T . P^T ----
#pragma unroll
      for (int tt = 0; tt < 2; tt++) {
#pragma unroll
        for (int db = 0; db < DB; db++) {
          const T* vp = Vs + (32 * nb + 16 * tt + 4 * g + (i16 >> 2)) * ROWE + 32 * db + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
          short4_t lo = lds_read_tr(vp);
          short4_t hi = lds_read_tr(vp + 8 * ROWE);
          oacc[db] = Frag<T>::mfma(join8<vec8>(lo, hi), pf[tt], oacc[db]);
        }
      }
    }
    __syncthreads();
  }

  // ---- epilogue ----
  const float l_tot = xhalf_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (q_row < p.Lq) {
    T* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)q_row * p.o_stride[2] + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        union { T e[4]; uint2 u; } pk;
#pragma unroll
        for (int e = 0; e < 4; e++) pk.e[e] = (T)(oacc[db][4 * rr + e] * inv);
        *reinterpret_cast<uint2*>(op + 32 * db + 8 * rr) = pk.u;
      }
    if (lse2 && g == 0) lse2[((int64_t)b * p.Hq + h) * p.Lq + q_row] = l_tot > 0.f ? m_run + log2f(l_tot) : -INFINITY;
  }
}

template <typename T, int D, int KIND>
static void launch_rs(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, hipStream_t s) {
  const int nqt = (p.Lq + kFwdBM - 1) / kFwdBM;
  dim3 grid(nqt * p.Hq * p.B);
  if (p.flags & FLEX_ROUND_S)
    hipLaunchKernelGGL((fwd_mfma_kernel<T, D, KIND, true>), grid, dim3(256), 0, s, p, (const T*)q, (const T*)k, (const T*)v, (T*)o, lse2);
  else
    hipLaunchKernelGGL((fwd_mfma_kernel<T, D, KIND, false>), grid, dim3(256), 0, s, p, (const T*)q, (const T*)k, (const T*)v, (T*)o, lse2);
}

template <typename T, int D>
static int launch_kind(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, hipStream_t s) {
  switch (p.score.kind) {
    case FLEX_SCORE_IDENTITY: launch_rs<T, D, FLEX_SCORE_IDENTITY>(p, q, k, v, o, lse2, s); return 0;
    case FLEX_SCORE_CHECKERBOARD: launch_rs<T, D, FLEX_SCORE_CHECKERBOARD>(p, q, k, v, o, lse2, s); return 0;
    case FLEX_SCORE_ALIBI: launch_rs<T, D, FLEX_SCORE_ALIBI>(p, q, k, v, o, lse2, s); return 0;
    case FLEX_SCORE_TANH_SOFTCAP: launch_rs<T, D, FLEX_SCORE_TANH_SOFTCAP>(p, q, k, v, o, lse2, s); return 0;
    case FLEX_SCORE_REL_BIAS: launch_rs<T, D, FLEX_SCORE_REL_BIAS>(p, q, k, v, o, lse2, s); return 0;
  }
  return 1;
}

}  // namespace flex

using namespace flex;
void flex_set_error(const char* fmt, ...);

static bool strides_ok(const int64_t* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0; }

bool flex_mfma_shape_ok(const FlexAttnParams& p) {
  if (p.dtype != FLEX_F16 && p.dtype != FLEX_BF16) return false;
  if (p.D != p.Dv || (p.D != 64 && p.D != 128)) return false;
  if (!strides_ok(p.q_stride) || !strides_ok(p.k_stride) || !strides_ok(p.v_stride) || !strides_ok(p.o_stride)) return false;
  const FlexTileLists& t = p.tiles;
  if (t.kv_num && (t.q_block != kFwdBM || t.kv_block != kFwdBN)) return false;
  if ((int64_t)((p.Lq + kFwdBM - 1) / kFwdBM) * p.Hq * p.B > 0x7fffffff) return false;
  return true;
}

bool flex_mfma_fwd_supported(const FlexAttnParams& p) { return flex_mfma_shape_ok(p); }

void flex_mfma_tiles(int dtype, int D, int Dv, int* qb, int* kvb) {
  bool ok = (dtype == FLEX_F16 || dtype == FLEX_BF16) && D == Dv && (D == 64 || D == 128);
  *qb = ok ? kFwdBM : 0;
  *kvb = ok ? kFwdBN : 0;
}

int flex_mfma_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15) {
    flex_set_error("fused forward needs 16-byte aligned tensors");
    return 1;
  }
  int rc = 1;
  if (p.dtype == FLEX_F16) rc = p.D == 64 ? launch_kind<f16, 64>(p, q, k, v, o, lse2, s) : launch_kind<f16, 128>(p, q, k, v, o, lse2, s);
  else rc = p.D == 64 ? launch_kind<bf16, 64>(p, q, k, v, o, lse2, s) : launch_kind<bf16, 128>(p, q, k, v, o, lse2, s);
  if (rc) flex_set_error("fused forward: unsupported score_mod kind %d", p.score.kind);
  return rc;
}
