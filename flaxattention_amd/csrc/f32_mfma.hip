// fp32 attention on the matrix cores of gfx950 (v_mfma_f32_32x32x2_f32), D = Dv in {64, 128}: forward, dQ (+ delta)
// and dK/dV kernels.  What the dense path of the reference computes for float32 inputs (core/attention.py:14-106:
// nothing is rounded below fp32 there), as a one-pass online softmax.
//
// Same conventions as the 16-bit kernels: transposed products, so that a lane owns one query row (forward, dQ) or
// one key (dK/dV); the accumulator layout C[m = 8*(r/4) + 4g + r%4][n = i] of the 32x32 instructions is the same,
// so the score functors and the mask helpers of mfma_common.cuh apply unchanged.  v_mfma_f32_32x32x2_f32 contracts
// two values per instruction: A[m = i][k = g], B[k = g][n = i].  A lane keeps the half row g * D/2 .. of its
// operand row; instruction j of a product pairs element j of both halves (any pairing of the contraction index
// that A and B share is a valid order of the sum).
// These kernels favour simplicity over the last factor in speed: 32-key (or 32-row) steps staged through registers
// into one LDS stage, two barriers per step, one wave per SIMD so that the D = 128 backward has its 300+ registers.
#include "mfma_common.cuh"

using namespace flex;
void flex_set_error(const char* fmt, ...);

namespace {

constexpr int kQTile = 128;   // query rows of a forward / dQ workgroup = q granularity of the tile lists
constexpr int kKvTile = 128;  // keys of a dK/dV workgroup = key granularity of the backward lists
constexpr int kStepRows = 32;  // rows staged per step

__device__ __forceinline__ float16_t mfma2(float a, float b, float16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// 32 rows x D floats, global -> registers -> LDS (rows of D + 4 floats)
template <int D> struct RowTile {
  static constexpr int ROWE = D + 4, C4 = D / 4, NL = kStepRows * C4 / 256;
  float4_t reg[NL];
  // rows past last_row are clamped to it (finite filler; the caller masks them out)
  __device__ __forceinline__ void load(const float* base, int64_t stride, int row0, int last_row, int tid) {
#pragma unroll
    for (int j = 0; j < NL; j++) {
      const int c = tid + 256 * j, r = min(row0 + c / C4, last_row), cc = c % C4;
      reg[j] = *reinterpret_cast<const float4_t*>(base + (int64_t)r * stride + cc * 4);
    }
  }
  __device__ __forceinline__ void store(float* lds, int tid) const {
#pragma unroll
    for (int j = 0; j < NL; j++) {
      const int c = tid + 256 * j;
      *reinterpret_cast<float4_t*>(lds + (c / C4) * ROWE + (c % C4) * 4) = reg[j];
    }
  }
};

// C += A.B^T over the feature axis: A rows come from an LDS tile (row i32 of the block), B is the lane's resident half row
template <int D>
__device__ __forceinline__ float16_t row_product(const float* tile_row_half, const float (&resident)[D / 2], float16_t acc) {
#pragma unroll
  for (int c = 0; c < D / 8; c++) {
    const float4_t a = *reinterpret_cast<const float4_t*>(tile_row_half + 4 * c);
#pragma unroll
    for (int e = 0; e < 4; e++) acc = mfma2(a[e], resident[4 * c + e], acc);
  }
  return acc;
}

// acc[db] (32 feature columns x the lane's column) += tile^T . x, contracting over the 32 rows of the tile: register
// r = 4i + e of x belongs to row 8i + 4g + e, which is also the row the A operand is read from
template <int D>
__device__ __forceinline__ void col_product(const float* tile, int i32, int g, const float16_t& x, float16_t (&acc)[D / 32]) {
  constexpr int ROWE = D + 4;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float* row = tile + (8 * i + 4 * g + e) * ROWE + i32;
#pragma unroll
      for (int db = 0; db < D / 32; db++) acc[db] = mfma2(row[32 * db], x[4 * i + e], acc[db]);
    }
}

// tile schedule of a workgroup: list entries (fully visible ones first) expanded into 32-row steps, or every step
struct Steps {
  const int32_t* full_idx = nullptr;
  const int32_t* part_idx = nullptr;
  int n_full = 0, n_part = 0, sub = 1;
  __device__ __forceinline__ int count() const { return (n_full + n_part) * sub; }
  __device__ __forceinline__ int full_steps() const { return n_full * sub; }
  __device__ __forceinline__ int at(int it) const {
    if (!full_idx) return it;
    const int e = it / sub, part = it - e * sub;
    return uniform_ld(e < n_full ? full_idx + e : part_idx + (e - n_full)) * sub + part;
  }
};

template <int D, int KIND>
__global__ __launch_bounds__(256) void f32_fwd_kernel(FlexAttnParams p, const float* __restrict__ q,
                                                      const float* __restrict__ k, const float* __restrict__ v,
                                                      float* __restrict__ o, float* __restrict__ lse2) {
  constexpr int HD = D / 2, DB = D / 32, ROWE = D + 4;
  __shared__ __align__(16) float Ks[kStepRows * ROWE];
  __shared__ __align__(16) float Vs[kStepRows * ROWE];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5;
  const int nqt = (p.Lq + kQTile - 1) / kQTile;
  int rank, bh;
  xcd_tile_map(blockIdx.x, nqt, p.Hq * p.B, rank, bh);
  const int qt = nqt - 1 - rank;  // late query tiles see the most keys under causal masks
  const int h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);
  const int q_row = qt * kQTile + w * 32 + i32;

  float qf[HD];
  {
    const float* qp = q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)min(q_row, p.Lq - 1) * p.q_stride[2] + g * HD;
#pragma unroll
    for (int c = 0; c < HD / 4; c++) {
      const float4_t x = *reinterpret_cast<const float4_t*>(qp + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; e++) qf[4 * c + e] = x[e];
    }
  }

  Steps st;
  const FlexTileLists& tl = p.tiles;
  if (tl.kv_num) {
    const int64_t row = (b * tl.stride_b + h * tl.stride_h) * tl.n_q_blocks + qt;
    st.n_full = uniform_ld(tl.full_kv_num + row);
    st.n_part = uniform_ld(tl.kv_num + row);
    st.full_idx = tl.full_kv_idx + row * tl.n_kv_blocks;
    st.part_idx = tl.kv_idx + row * tl.n_kv_blocks;
    st.sub = tl.kv_block / kStepRows;
  } else {
    // no lists: every step is visited, and evaluated under a mask that can hide something
    st.n_full = (p.Lkv + kStepRows - 1) / kStepRows;
    if (!mask_hides_nothing(p.mask)) { st.n_part = st.n_full; st.n_full = 0; }
  }
  const int nt = st.count(), n_full_t = st.full_steps();

  const float* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const float* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  Score2<KIND> sm;
  sm.init(p.score, p.scale, h, b, p.Lq, p.Lkv);
  const Mask2 visible(p.mask, b, h, p.Lkv);

  float16_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[db][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // l_run: this lane's share of the row sum

  RowTile<D> kt, vt;
  int s_cur = nt > 0 ? st.at(0) : 0;
  if (nt > 0) {
    kt.load(kbase, p.k_stride[2], s_cur * kStepRows, p.Lkv - 1, tid);
    vt.load(vbase, p.v_stride[2], s_cur * kStepRows, p.Lkv - 1, tid);
  }
  for (int it = 0; it < nt; it++) {
    const int kv0 = s_cur * kStepRows;
    __syncthreads();  // the previous step's reads are done
    kt.store(Ks, tid);
    vt.store(Vs, tid);
    __syncthreads();
    if (it + 1 < nt) {
      s_cur = st.at(it + 1);
      kt.load(kbase, p.k_stride[2], s_cur * kStepRows, p.Lkv - 1, tid);
      vt.load(vbase, p.v_stride[2], s_cur * kStepRows, p.Lkv - 1, tid);
    }
    const bool masked = (it >= n_full_t) || (kv0 + kStepRows > p.Lkv);
    int cls = kBlockAll;
    if (masked) {
      cls = block_class(p.mask, visible, __builtin_amdgcn_readfirstlane(q_row - i32), kv0, 0x7fffffff, p.Lkv);
      if (cls == kBlockNone) continue;
    }
    float16_t x;
#pragma unroll
    for (int r = 0; r < 16; r++) x[r] = 0.f;
    x = row_product<D>(Ks + i32 * ROWE + g * HD, qf, x);  // S^T: rows = keys, the lane's column = its query row
    sm.tile(q_row, kv0 + 4 * g);
#pragma unroll
    for (int r = 0; r < 16; r++) x[r] = sm.apply(x[r], acc_row(r));
    if (cls == kBlockMixed) mask_block_q(x, p.mask, visible, q_row, kv0, g, p.Lkv);
    const float m_new = fmaxf(m_run, xhalf_max(block_max(x)));
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // nothing visible so far: P = 0 against any reference
    const float alpha = fast_exp2(m_run - m_use);
    float l_blk = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      x[r] = fast_exp2(x[r] - m_use);
      l_blk += x[r];
    }
    l_run = fmaf(l_run, alpha, l_blk);
    m_run = m_new;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[db][r] *= alpha;
    col_product<D>(Vs, i32, g, x, oacc);  // O^T += V^T.P^T
  }

  const float l_tot = xhalf_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (q_row < p.Lq) {
    float* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)q_row * p.o_stride[2] + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        float4_t y;
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = oacc[db][4 * rr + e] * inv;
        *reinterpret_cast<float4_t*>(op + 32 * db + 8 * rr) = y;
      }
    if (lse2 && g == 0) lse2[((int64_t)b * p.Hq + h) * p.Lq + q_row] = l_tot > 0.f ? m_run + log2f(l_tot) : -INFINITY;
  }
}

// dQ = scale * (P o (dP - delta) o g) . K with delta_i = sum_d O_id dO_id - log2(e) d_lse2_i, written to delta_out for
// the dK/dV kernel that follows on the stream
template <int D, int KIND>
__global__ __launch_bounds__(256) void f32_dq_kernel(FlexAttnParams p, const float* __restrict__ q,
                                                     const float* __restrict__ k, const float* __restrict__ v,
                                                     const float* __restrict__ o, const float* __restrict__ lse2,
                                                     const float* __restrict__ d_o, float* __restrict__ dq,
                                                     float* __restrict__ delta_out) {
  constexpr int HD = D / 2, DB = D / 32, ROWE = D + 4;
  __shared__ __align__(16) float Ks[kStepRows * ROWE];
  __shared__ __align__(16) float Vs[kStepRows * ROWE];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5;
  const int nqt = (p.Lq + kQTile - 1) / kQTile;
  int rank, bh;
  xcd_tile_map(blockIdx.x, nqt, p.Hq * p.B, rank, bh);
  const int qt = nqt - 1 - rank;
  const int h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);
  const int q_row = qt * kQTile + w * 32 + i32;
  const int q_ld = min(q_row, p.Lq - 1);
  const int64_t row_id = ((int64_t)b * p.Hq + h) * p.Lq + q_ld;

  float qf[HD], dof[HD];
  float dpart = 0.f;
  {
    const float* qp = q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)q_ld * p.q_stride[2] + g * HD;
    const float* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)q_ld * p.o_stride[2] + g * HD;
    const float* dop = d_o + row_id * D + g * HD;  // dO is contiguous [B,Hq,Lq,D]
#pragma unroll
    for (int c = 0; c < HD / 4; c++) {
      const float4_t x = *reinterpret_cast<const float4_t*>(qp + 4 * c);
      const float4_t y = *reinterpret_cast<const float4_t*>(dop + 4 * c);
      const float4_t z = *reinterpret_cast<const float4_t*>(op + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        qf[4 * c + e] = x[e];
        dof[4 * c + e] = y[e];
        dpart = fmaf(z[e], y[e], dpart);
      }
    }
  }
  float delta = xhalf_sum(dpart);
  if (p.d_lse2) delta -= kLog2e * p.d_lse2[row_id];
  if (q_row < p.Lq && g == 0) delta_out[row_id] = delta;
  float lse = lse2[row_id];
  if (lse == -INFINITY) lse = INFINITY;  // row without visible keys: P = 0

  Steps st;
  const FlexTileLists& tl = p.tiles_bwd;
  if (tl.kv_num) {
    const int64_t row = (b * tl.stride_b + h * tl.stride_h) * tl.n_q_blocks + qt;
    st.n_full = uniform_ld(tl.full_kv_num + row);
    st.n_part = uniform_ld(tl.kv_num + row);
    st.full_idx = tl.full_kv_idx + row * tl.n_kv_blocks;
    st.part_idx = tl.kv_idx + row * tl.n_kv_blocks;
    st.sub = tl.kv_block / kStepRows;
  } else {
    st.n_full = (p.Lkv + kStepRows - 1) / kStepRows;
    if (!mask_hides_nothing(p.mask)) { st.n_part = st.n_full; st.n_full = 0; }
  }
  const int nt = st.count(), n_full_t = st.full_steps();

  const float* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const float* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  Score2<KIND> sm;
  sm.init(p.score, p.scale, h, b, p.Lq, p.Lkv);
  const Mask2 visible(p.mask, b, h, p.Lkv);

  float16_t dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) dqacc[db][r] = 0.f;

  RowTile<D> kt, vt;
  int s_cur = nt > 0 ? st.at(0) : 0;
  if (nt > 0) {
    kt.load(kbase, p.k_stride[2], s_cur * kStepRows, p.Lkv - 1, tid);
    vt.load(vbase, p.v_stride[2], s_cur * kStepRows, p.Lkv - 1, tid);
  }
  for (int it = 0; it < nt; it++) {
    const int kv0 = s_cur * kStepRows;
    __syncthreads();
    kt.store(Ks, tid);
    vt.store(Vs, tid);
    __syncthreads();
    if (it + 1 < nt) {
      s_cur = st.at(it + 1);
      kt.load(kbase, p.k_stride[2], s_cur * kStepRows, p.Lkv - 1, tid);
      vt.load(vbase, p.v_stride[2], s_cur * kStepRows, p.Lkv - 1, tid);
    }
    const bool masked = (it >= n_full_t) || (kv0 + kStepRows > p.Lkv);
    int cls = kBlockAll;
    if (masked) {
      cls = block_class(p.mask, visible, __builtin_amdgcn_readfirstlane(q_row - i32), kv0, 0x7fffffff, p.Lkv);
      if (cls == kBlockNone) continue;
    }
    float16_t x, dp, gr;
#pragma unroll
    for (int r = 0; r < 16; r++) { x[r] = 0.f; dp[r] = -delta; }
    x = row_product<D>(Ks + i32 * ROWE + g * HD, qf, x);     // S^T
    dp = row_product<D>(Vs + i32 * ROWE + g * HD, dof, dp);  // dP^T - delta
    sm.tile(q_row, kv0 + 4 * g);
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float s = x[r];
      x[r] = sm.apply_sub(s, acc_row(r), lse);
      if (!Score2<KIND>::kGradOne) gr[r] = sm.grad(s, acc_row(r));
    }
    if (cls == kBlockMixed) mask_block_q(x, p.mask, visible, q_row, kv0, g, p.Lkv);
#pragma unroll
    for (int r = 0; r < 16; r++) {
      float ds = fast_exp2(x[r]) * dp[r];
      if (!Score2<KIND>::kGradOne) ds *= gr[r];
      x[r] = ds;
    }
    col_product<D>(Ks, i32, g, x, dqacc);  // dQ^T += K^T.dS^T
  }

  if (q_row < p.Lq) {
    float* op = dq + row_id * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        float4_t y;
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = dqacc[db][4 * rr + e] * p.scale;
        *reinterpret_cast<float4_t*>(op + 32 * db + 8 * rr) = y;
      }
  }
}

// dV = P^T.dO and dK = scale * (P o (dP - delta) o g)^T . Q for the 128 keys of a workgroup (one 32-key block per
// wave, a lane owns one key), summed over the query heads of the key head's group
template <int D, int KIND>
__global__ __launch_bounds__(256) void f32_dkv_kernel(FlexAttnParams p, const float* __restrict__ q,
                                                      const float* __restrict__ k, const float* __restrict__ v,
                                                      const float* __restrict__ lse2, const float* __restrict__ delta,
                                                      const float* __restrict__ d_o, float* __restrict__ dk,
                                                      float* __restrict__ dv) {
  constexpr int HD = D / 2, DB = D / 32, ROWE = D + 4;
  __shared__ __align__(16) float Qs[kStepRows * ROWE];
  __shared__ __align__(16) float Os[kStepRows * ROWE];
  __shared__ __align__(16) float lse_s[kStepRows];
  __shared__ __align__(16) float ndel_s[kStepRows];

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i32 = lane & 31, g = lane >> 5;
  const int nkt = (p.Lkv + kKvTile - 1) / kKvTile;
  int kt, bh;  // early key tiles see the most queries under causal masks
  xcd_tile_map(blockIdx.x, nkt, p.Hkv * p.B, kt, bh);
  const int hk = bh % p.Hkv, b = bh / p.Hkv, G = p.Hq / p.Hkv;
  const int kv_col = kt * kKvTile + w * 32 + i32;
  const int kv_ld = min(kv_col, p.Lkv - 1);

  float kf[HD], vf[HD];
  {
    const float* kp = k + b * p.k_stride[0] + hk * p.k_stride[1] + (int64_t)kv_ld * p.k_stride[2] + g * HD;
    const float* vp = v + b * p.v_stride[0] + hk * p.v_stride[1] + (int64_t)kv_ld * p.v_stride[2] + g * HD;
#pragma unroll
    for (int c = 0; c < HD / 4; c++) {
      const float4_t x = *reinterpret_cast<const float4_t*>(kp + 4 * c);
      const float4_t y = *reinterpret_cast<const float4_t*>(vp + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; e++) { kf[4 * c + e] = x[e]; vf[4 * c + e] = y[e]; }
    }
  }
  float16_t dkacc[DB], dvacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dkacc[db][r] = 0.f; dvacc[db][r] = 0.f; }

  const FlexTileLists& tl = p.tiles_bwd;
  Score2<KIND> sm;
  for (int gi = 0; gi < G; gi++) {
    const int h = hk * G + gi;
    sm.init(p.score, p.scale, h, b, p.Lq, p.Lkv);
    const Mask2 visible(p.mask, b, h, p.Lkv);
    Steps st;
    if (tl.kv_num) {
      const int64_t row = (b * tl.stride_b + h * tl.stride_h) * tl.n_kv_blocks + kt;
      st.n_full = uniform_ld(tl.full_q_num + row);
      st.n_part = uniform_ld(tl.q_num + row);
      st.full_idx = tl.full_q_idx + row * tl.n_q_blocks;
      st.part_idx = tl.q_idx + row * tl.n_q_blocks;
      st.sub = tl.q_block / kStepRows;
    } else {
      st.n_full = (p.Lq + kStepRows - 1) / kStepRows;
      if (!mask_hides_nothing(p.mask)) { st.n_part = st.n_full; st.n_full = 0; }
    }
    const int nt = st.count(), n_full_t = st.full_steps();
    const float* qbase = q + b * p.q_stride[0] + h * p.q_stride[1];
    const int64_t rows0 = ((int64_t)b * p.Hq + h) * p.Lq;
    const float* dobase = d_o + rows0 * D;

    RowTile<D> qt, ot;
    float lreg = INFINITY, dreg = 0.f;
    auto load_step = [&](int q0) {
      qt.load(qbase, p.q_stride[2], q0, p.Lq - 1, tid);
      ot.load(dobase, D, q0, p.Lq - 1, tid);
      lreg = INFINITY;  // rows past Lq: P = 0, whatever the clamped loads hold
      dreg = 0.f;
      if (tid < kStepRows && q0 + tid < p.Lq) {
        lreg = lse2[rows0 + q0 + tid];
        dreg = delta[rows0 + q0 + tid];
      }
    };
    int s_cur = nt > 0 ? st.at(0) : 0;
    if (nt > 0) load_step(s_cur * kStepRows);
    for (int it = 0; it < nt; it++) {
      const int q0 = s_cur * kStepRows;
      __syncthreads();  // the previous step's (or head's) reads are done
      qt.store(Qs, tid);
      ot.store(Os, tid);
      if (tid < kStepRows) {
        lse_s[tid] = lreg == -INFINITY ? INFINITY : lreg;  // row without visible keys: P = 0
        ndel_s[tid] = -dreg;
      }
      __syncthreads();
      if (it + 1 < nt) {
        s_cur = st.at(it + 1);
        load_step(s_cur * kStepRows);
      }
      const bool masked = (it >= n_full_t) || (q0 + kStepRows > p.Lq) || (kt * kKvTile + kKvTile > p.Lkv);
      int cls = kBlockAll;
      if (masked) {
        cls = block_class(p.mask, visible, q0, kt * kKvTile + w * 32, p.Lq, p.Lkv);
        if (cls == kBlockNone) continue;
      }
      const int ql = 4 * g;  // local row of register 0
      float16_t x, dp, gr;
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        const float4_t d4 = *reinterpret_cast<const float4_t*>(ndel_s + ql + 8 * rr);
#pragma unroll
        for (int e = 0; e < 4; e++) { x[4 * rr + e] = 0.f; dp[4 * rr + e] = d4[e]; }
      }
      x = row_product<D>(Qs + i32 * ROWE + g * HD, kf, x);     // S: rows = queries, the lane's column = its key
      dp = row_product<D>(Os + i32 * ROWE + g * HD, vf, dp);   // dP - delta
      sm.tileT(q0 + ql, kv_col);
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        const float4_t l4 = *reinterpret_cast<const float4_t*>(lse_s + ql + 8 * rr);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 4 * rr + e;
          const float s = x[r];
          x[r] = sm.apply_sub(s, acc_row(r), l4[e]);
          if (!Score2<KIND>::kGradOne) gr[r] = sm.grad(s, acc_row(r));
        }
      }
      if (cls == kBlockMixed) mask_block_kv<true>(x, p.mask, visible, q0 + ql, kv_col, p.Lq, p.Lkv);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        x[r] = fast_exp2(x[r]);  // P
        float ds = x[r] * dp[r];
        if (!Score2<KIND>::kGradOne) ds *= gr[r];
        dp[r] = ds;
      }
      col_product<D>(Os, i32, g, x, dvacc);   // dV^T += dO^T.P
      col_product<D>(Qs, i32, g, dp, dkacc);  // dK^T += Q^T.dS
    }
  }

  if (kv_col < p.Lkv) {
    const int64_t row_id = ((int64_t)b * p.Hkv + hk) * p.Lkv + kv_col;
    float* dkp = dk + row_id * D + 4 * g;
    float* dvp = dv + row_id * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        float4_t yk, yv;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          yk[e] = dkacc[db][4 * rr + e] * p.scale;
          yv[e] = dvacc[db][4 * rr + e];
        }
        *reinterpret_cast<float4_t*>(dkp + 32 * db + 8 * rr) = yk;
        *reinterpret_cast<float4_t*>(dvp + 32 * db + 8 * rr) = yv;
      }
  }
}

struct F32Args {
  const float *q, *k, *v, *o, *d_o;
  const float* lse2_in;
  float *out, *lse2_out, *dq, *dk, *dv, *delta;
  hipStream_t s;
};

template <int D, int KIND> void launch_fwd(const FlexAttnParams& p, const F32Args& a) {
  const int nqt = (p.Lq + kQTile - 1) / kQTile;
  hipLaunchKernelGGL((f32_fwd_kernel<D, KIND>), dim3(nqt * p.Hq * p.B), dim3(256), 0, a.s, p, a.q, a.k, a.v, a.out, a.lse2_out);
}
template <int D, int KIND> void launch_bwd(const FlexAttnParams& p, const F32Args& a) {
  const int nqt = (p.Lq + kQTile - 1) / kQTile, nkt = (p.Lkv + kKvTile - 1) / kKvTile;
  hipLaunchKernelGGL((f32_dq_kernel<D, KIND>), dim3(nqt * p.Hq * p.B), dim3(256), 0, a.s, p, a.q, a.k, a.v, a.o, a.lse2_in,
                     a.d_o, a.dq, a.delta);
  hipLaunchKernelGGL((f32_dkv_kernel<D, KIND>), dim3(nkt * p.Hkv * p.B), dim3(256), 0, a.s, p, a.q, a.k, a.v, a.lse2_in,
                     a.delta, a.d_o, a.dk, a.dv);
}
template <int D, int KIND> void launch(const FlexAttnParams& p, const F32Args& a, bool bwd) {
  if (bwd) launch_bwd<D, KIND>(p, a);
  else launch_fwd<D, KIND>(p, a);
}
template <int D> int launch_kind(const FlexAttnParams& p, const F32Args& a, bool bwd) {
  switch (p.score.kind) {
    case FLEX_SCORE_IDENTITY: launch<D, FLEX_SCORE_IDENTITY>(p, a, bwd); return 0;
    case FLEX_SCORE_CHECKERBOARD: launch<D, FLEX_SCORE_CHECKERBOARD>(p, a, bwd); return 0;
    case FLEX_SCORE_ALIBI: launch<D, FLEX_SCORE_ALIBI>(p, a, bwd); return 0;
    case FLEX_SCORE_TANH_SOFTCAP: launch<D, FLEX_SCORE_TANH_SOFTCAP>(p, a, bwd); return 0;
    case FLEX_SCORE_REL_BIAS: launch<D, FLEX_SCORE_REL_BIAS>(p, a, bwd); return 0;
    case FLEX_SCORE_AFFINE:
      if (p.score.mul) launch<D, kScoreAffineMul>(p, a, bwd);
      else launch<D, FLEX_SCORE_AFFINE>(p, a, bwd);
      return 0;
  }
  return 1;
}

bool strides_ok(const int64_t* s) { return s[0] % 4 == 0 && s[1] % 4 == 0 && s[2] % 4 == 0; }
bool lists_ok(const FlexTileLists& t, int kv_block) { return !t.kv_num || (t.q_block == kQTile && t.kv_block == kv_block); }

}  // namespace

// which: 0 = forward, 1 = backward
bool flex_f32_mfma_supported(const FlexAttnParams& p, int which) {
  if (p.dtype != FLEX_F32 || p.D != p.Dv || (p.D != 64 && p.D != 128)) return false;
  if (p.score.kind == FLEX_SCORE_AFFINE && !p.score.mul && !p.score.add) return false;
  if (!strides_ok(p.q_stride) || !strides_ok(p.k_stride) || !strides_ok(p.v_stride) || !strides_ok(p.o_stride)) return false;
  if ((int64_t)((p.Lq + kQTile - 1) / kQTile) * p.Hq * p.B > 0x7fffffff) return false;
  return which == 0 ? lists_ok(p.tiles, 64) : lists_ok(p.tiles_bwd, kKvTile);
}

int flex_f32_mfma_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15) {
    flex_set_error("fp32 matrix-core forward needs 16-byte aligned tensors");
    return 1;
  }
  F32Args a = {};
  a.q = (const float*)q; a.k = (const float*)k; a.v = (const float*)v;
  a.out = (float*)o; a.lse2_out = lse2; a.s = s;
  const int rc = p.D == 64 ? launch_kind<64>(p, a, false) : launch_kind<128>(p, a, false);
  if (rc) flex_set_error("fp32 matrix-core forward: unsupported score_mod kind %d", p.score.kind);
  return rc;
}

int flex_f32_mfma_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const void* o, const float* lse2,
                      const void* d_o, void* dq, void* dk, void* dv, void* workspace, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)d_o | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) & 15) {
    flex_set_error("fp32 matrix-core backward needs 16-byte aligned tensors");
    return 1;
  }
  F32Args a = {};
  a.q = (const float*)q; a.k = (const float*)k; a.v = (const float*)v; a.o = (const float*)o; a.d_o = (const float*)d_o;
  a.lse2_in = lse2; a.dq = (float*)dq; a.dk = (float*)dk; a.dv = (float*)dv; a.delta = (float*)workspace; a.s = s;
  const int rc = p.D == 64 ? launch_kind<64>(p, a, true) : launch_kind<128>(p, a, true);
  if (rc) flex_set_error("fp32 matrix-core backward: unsupported score_mod kind %d", p.score.kind);
  return rc;
}
