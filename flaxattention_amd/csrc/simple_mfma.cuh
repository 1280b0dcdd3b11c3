// Matrix-core attention kernels for the shapes the tuned kernels (fwd_mfma / bwd_mfma) do not take:
//   float32 inputs, D = Dv in {64, 128}      v_mfma_f32_32x32x2_f32
//   fp16 / bf16 inputs, D = Dv in {192, 256}  v_mfma_f32_32x32x16_{f16,bf16}
// Forward, dQ (+ delta) and dK/dV; instantiated per (dtype, head size) by simple_mfma_inst.hip, dispatched from
// simple_mfma.hip.  What they compute is what the tuned kernels compute (core/attention.py:14-106 of the reference
// and its autodiff transposes), in the "fast" and the "parity" numerics; float32 inputs have no rounding points
// below fp32, so for them every mode is the same computation.
//
// Same conventions as the tuned kernels: transposed products, so that a lane owns one query row (forward, dQ) or one
// key (dK/dV), and the accumulator layout C[m = 8*(r/4) + 4g + r%4][n = i] of the 32x32 instructions, so that the
// score functors and the mask helpers of mfma_common.cuh apply unchanged.  These kernels favour simplicity over the
// last factor in speed: 32-row steps staged through registers into one LDS stage, two barriers per step, one wave
// per SIMD (the widest instantiations hold more than 400 registers, accumulators in AGPRs).
#pragma once
#include "mfma_common.cuh"
#include "decode.cuh"  // decode_combine_kernel merges the partials of a forward over split key ranges

namespace flex {

constexpr int kSimpleQTile = 128;   // query rows of a forward / dQ workgroup = q granularity of the tile lists
constexpr int kSimpleKvTile = 128;  // keys of a dK/dV workgroup = key granularity of the backward lists
constexpr int kSimpleStep = 32;     // rows staged per step

// ---- operand handling per element type ----
// A product "over the feature axis" pairs a tile row (A operand, from LDS) with the lane's resident row (B operand);
// a product "over the tile rows" takes the tile transposed as the A operand and accumulator-layout values as B.
template <typename T, int D> struct SimpleOps;

// float32: v_mfma_f32_32x32x2_f32 contracts two values per instruction, A[m = i][k = g], B[k = g][n = i].  A lane
// keeps the half row g * D/2 .. of its operand row; instruction j pairs element j of both halves (any pairing of the
// contraction index that A and B share is a valid order of the sum).
template <int D> struct SimpleOps<float, D> {
  static constexpr int ROWE = D + 4;   // LDS row length in elements
  static constexpr int EPC = 4;        // elements per 16-byte chunk
  static constexpr bool kRounds = false;  // the element type is the accumulation type: nothing to round
  struct Resident { float v[D / 2]; };
  static __device__ __forceinline__ float16_t mfma(float a, float b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ void load_resident(Resident& r, const float* row, int g) {
#pragma unroll
    for (int c = 0; c < D / 8; c++) {
      const float4_t x = *reinterpret_cast<const float4_t*>(row + g * (D / 2) + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; e++) r.v[4 * c + e] = x[e];
    }
  }
  // sum over the row's features of resident[.] * other[.], this lane's half
  static __device__ __forceinline__ float dot_half(const Resident& r, const float* other_row, int g) {
    float acc = 0.f;
#pragma unroll
    for (int c = 0; c < D / 8; c++) {
      const float4_t x = *reinterpret_cast<const float4_t*>(other_row + g * (D / 2) + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; e++) acc = fmaf(x[e], r.v[4 * c + e], acc);
    }
    return acc;
  }
  static __device__ __forceinline__ float16_t row_product(const float* tile, int i32, int g, const Resident& r, float16_t acc) {
    const float* row = tile + i32 * ROWE + g * (D / 2);
#pragma unroll
    for (int c = 0; c < D / 8; c++) {
      const float4_t a = *reinterpret_cast<const float4_t*>(row + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; e++) acc = mfma(a[e], r.v[4 * c + e], acc);
    }
    return acc;
  }
  // register r = 4i + e of x belongs to tile row 8i + 4g + e, which is also the row the A operand is read from
  static __device__ __forceinline__ void col_product(const float* tile, int lane, const float16_t& x, float16_t (&acc)[D / 32]) {
    const int i32 = lane & 31, g = lane >> 5;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const float* row = tile + (8 * i + 4 * g + e) * ROWE + i32;
#pragma unroll
        for (int db = 0; db < D / 32; db++) acc[db] = mfma(row[32 * db], x[4 * i + e], acc[db]);
      }
  }
  static __device__ __forceinline__ void round_block(float16_t&) {}
  static __device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
    const float4_t y = {a, b, c, d};
    *reinterpret_cast<float4_t*>(p) = y;
  }
};

// fp16 / bf16: v_mfma_f32_32x32x16, A[m = i][k = 8g .. 8g+7], B[k = 8g .. 8g+7][n = i]; tiles in LDS rows padded by 16
// bytes, transposed operands through ds_read_b64_tr_b16
template <typename T, int D> struct SimpleOps16 {
  typedef typename Frag<T>::vec8 vec8;
  static constexpr int ROWE = D + 8;
  static constexpr int EPC = 8;
  static constexpr bool kRounds = true;
  struct Resident { vec8 v[D / 16]; };
  static __device__ __forceinline__ void load_resident(Resident& r, const T* row, int g) {
#pragma unroll
    for (int s = 0; s < D / 16; s++) r.v[s] = *reinterpret_cast<const vec8*>(row + 16 * s + 8 * g);
  }
  static __device__ __forceinline__ float dot_half(const Resident& r, const T* other_row, int g) {
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < D / 16; s++) {
      const vec8 x = *reinterpret_cast<const vec8*>(other_row + 16 * s + 8 * g);
#pragma unroll
      for (int e = 0; e < 8; e++) acc = fmaf((float)x[e], (float)r.v[s][e], acc);
    }
    return acc;
  }
  static __device__ __forceinline__ float16_t row_product(const T* tile, int i32, int g, const Resident& r, float16_t acc) {
    const T* row = tile + i32 * ROWE + 8 * g;
#pragma unroll
    for (int s = 0; s < D / 16; s++) acc = Frag<T>::mfma(*reinterpret_cast<const vec8*>(row + 16 * s), r.v[s], acc);
    return acc;
  }
  // x goes into the product rounded to T.  Registers 8t .. 8t+7 of x belong to tile rows 16t + 4g + {0..3} and
  // 16t + 8 + 4g + {0..3}: the transposing reads fetch the same rows (4 elements of row 4g + (i16 >> 2) + 8e,
  // logical column 32db + 16hh + 4(i16 & 3)).
  static __device__ __forceinline__ void col_product(const T* tile, int lane, const float16_t& x, float16_t (&acc)[D / 32]) {
    const int g = lane >> 5, i16 = lane & 15, hh = (lane >> 4) & 1;
    const int rl = 4 * g + (i16 >> 2);
    const int col = (2 * hh + ((i16 & 3) >> 1)) * 8 + 4 * (i16 & 1);
#pragma unroll
    for (int t = 0; t < 2; t++) {
      typename Pair<T>::v2 pr[4];
#pragma unroll
      for (int e = 0; e < 4; e++) pr[e] = Pair<T>::pack(x[8 * t + 2 * e], x[8 * t + 2 * e + 1]);
      const vec8 b = join_pairs<T>(pr[0], pr[1], pr[2], pr[3]);
      const T* base = tile + (16 * t + rl) * ROWE + col;
#pragma unroll
      for (int db = 0; db < D / 32; db++) {
        const vec8 a = join8<vec8>(lds_read_tr(base + 32 * db), lds_read_tr(base + 8 * ROWE + 32 * db));
        acc[db] = Frag<T>::mfma(a, b, acc[db]);
      }
    }
  }
  static __device__ __forceinline__ void round_block(float16_t& x) {
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      float a = x[r], b = x[r + 1];
      round_pair<T>(a, b);
      x[r] = a;
      x[r + 1] = b;
    }
  }
  static __device__ __forceinline__ void store4(T* p, float a, float b, float c, float d) {
    union { T e[4]; uint2 u; } pk;
    pk.e[0] = (T)a; pk.e[1] = (T)b; pk.e[2] = (T)c; pk.e[3] = (T)d;
    *reinterpret_cast<uint2*>(p) = pk.u;
  }
};
template <int D> struct SimpleOps<f16, D> : SimpleOps16<f16, D> {};
template <int D> struct SimpleOps<bf16, D> : SimpleOps16<bf16, D> {};

// 32 rows x D elements, global -> registers -> LDS (rows of Ops::ROWE elements), in 16-byte chunks
template <typename T, int D> struct RowTile {
  typedef SimpleOps<T, D> Ops;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  static constexpr int CPR = D / Ops::EPC, NL = kSimpleStep * CPR / 256;
  static_assert(kSimpleStep * CPR % 256 == 0, "a step is a whole number of 16-byte chunks per thread");
  u32x4 reg[NL];
  // rows past last_row are clamped to it (finite filler; the caller masks them out)
  __device__ __forceinline__ void load(const T* base, int64_t stride, int row0, int last_row, int tid) {
#pragma unroll
    for (int j = 0; j < NL; j++) {
      const int c = tid + 256 * j, r = min(row0 + c / CPR, last_row), cc = c % CPR;
      reg[j] = *reinterpret_cast<const u32x4*>(base + (int64_t)r * stride + cc * Ops::EPC);
    }
  }
  __device__ __forceinline__ void store(T* lds, int tid) const {
#pragma unroll
    for (int j = 0; j < NL; j++) {
      const int c = tid + 256 * j;
      *reinterpret_cast<u32x4*>(lds + (c / CPR) * Ops::ROWE + (c % CPR) * Ops::EPC) = reg[j];
    }
  }
};

// tile schedule of a workgroup: list entries (fully visible ones first) expanded into 32-row steps, or every step
struct SimpleSteps {
  const int32_t* full_idx = nullptr;
  const int32_t* part_idx = nullptr;
  int n_full = 0, n_part = 0, sub = 1;
  // row: the list row; n_idx: index entries per row; block: rows one entry covers; length: the walked axis
  __device__ __forceinline__ void init(const int32_t* part_num, const int32_t* part, const int32_t* full_num,
                                       const int32_t* full, int64_t row, int n_idx, int block, int length,
                                       const FlexMask& mask) {
    if (part_num) {
      n_full = uniform_ld(full_num + row);
      n_part = uniform_ld(part_num + row);
      full_idx = full + row * n_idx;
      part_idx = part + row * n_idx;
      sub = block / kSimpleStep;
    } else {
      // no lists: every step is visited, and evaluated under a mask that can hide something
      n_full = (length + kSimpleStep - 1) / kSimpleStep;
      if (!mask_hides_nothing(mask)) { n_part = n_full; n_full = 0; }
    }
  }
  __device__ __forceinline__ int count() const { return (n_full + n_part) * sub; }
  __device__ __forceinline__ int full_steps() const { return n_full * sub; }
  __device__ __forceinline__ int at(int it) const {
    if (!full_idx) return it;
    const int e = it / sub, part = it - e * sub;
    return uniform_ld(e < n_full ? full_idx + e : part_idx + (e - n_full)) * sub + part;
  }
};

// PASS, as in the tuned forward:
//   kSimpleOnePass  online softmax, O normalised at the end
//   kSimpleLse      first pass of the parity numerics: only lse2 (unrounded exponentials summed in fp32), V is not read
//   kSimpleNorm     second pass: P = 2^(x - lse2) is the normalised probability, rounded to T for the product with V
enum { kSimpleOnePass = 0, kSimpleLse = 1, kSimpleNorm = 2 };
// Split-KV: with gridDim.y > 1 workgroup (x, y) takes share y of its query tile's key steps and leaves an unnormalised
// partial (O, m, l) per row in o_part / ml_part, in the layout decode_combine_kernel merges (kSimpleLse: only (m, l);
// kSimpleNorm: the partial outputs add up, written with m = 0 and l = 1 for share 0, l = 0 for the others).  For calls
// whose query tiles alone would leave most compute units without a workgroup.
template <typename T, int D, int KIND, int PASS>
__global__ __launch_bounds__(256) void simple_fwd_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                         const T* __restrict__ k, const T* __restrict__ v,
                                                         T* __restrict__ o, float* __restrict__ lse2,
                                                         float* __restrict__ o_part, float* __restrict__ ml_part) {
  typedef SimpleOps<T, D> Ops;
  constexpr int DB = D / 32, ROWE = Ops::ROWE;
  __shared__ __align__(16) T Ks[kSimpleStep * ROWE];
  __shared__ __align__(16) T Vs[PASS == kSimpleLse ? 8 : kSimpleStep * ROWE];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5;
  const int nqt = (p.Lq + kSimpleQTile - 1) / kSimpleQTile;
  int rank, bh;
  xcd_tile_map(blockIdx.x, nqt, p.Hq * p.B, rank, bh);
  const int qt = nqt - 1 - rank;  // late query tiles see the most keys under causal masks
  const int h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);
  const int q_row = qt * kSimpleQTile + w * 32 + i32;
  const bool wave_has_rows = __builtin_amdgcn_readfirstlane(q_row - i32) < p.Lq;  // short queries: decode shapes
  const int64_t row_id = ((int64_t)b * p.Hq + h) * p.Lq + min(q_row, p.Lq - 1);
  const bool round_s = Ops::kRounds && (p.flags & FLEX_ROUND_S);

  typename Ops::Resident qf;
  Ops::load_resident(qf, q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)min(q_row, p.Lq - 1) * p.q_stride[2], g);

  SimpleSteps st;
  const FlexTileLists& tl = p.tiles;
  st.init(tl.kv_num, tl.kv_idx, tl.full_kv_num, tl.full_kv_idx,
          (b * tl.stride_b + h * tl.stride_h) * tl.n_q_blocks + qt, tl.n_kv_blocks, tl.kv_block, p.Lkv, p.mask);
  const int nt = st.count(), n_full_t = st.full_steps();
  const int nsplit = gridDim.y, split = blockIdx.y;
  const int per = (nt + nsplit - 1) / nsplit;
  const int it0 = split * per, it1 = min(it0 + per, nt);  // this workgroup's steps

  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  Score2<KIND> sm;
  sm.init(p.score, p.scale, h, b, p.Lq, p.Lkv);
  const Mask2 visible(p.mask, b, h, p.Lkv);

  float16_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[db][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // l_run: this lane's share of the row sum
  if constexpr (PASS == kSimpleNorm) {
    m_run = lse2[row_id];                          // fixed reference: the log-sum-exp of the first pass
    if (m_run == -INFINITY) m_run = INFINITY;      // row without visible keys: P = 0
  }

  RowTile<T, D> kt, vt;
  int s_cur = it0 < it1 ? st.at(it0) : 0;
  if (it0 < it1) {
    kt.load(kbase, p.k_stride[2], s_cur * kSimpleStep, p.Lkv - 1, tid);
    if constexpr (PASS != kSimpleLse) vt.load(vbase, p.v_stride[2], s_cur * kSimpleStep, p.Lkv - 1, tid);
  }
  for (int it = it0; it < it1; it++) {
    const int kv0 = s_cur * kSimpleStep;
    __syncthreads();  // the previous step's reads are done
    kt.store(Ks, tid);
    if constexpr (PASS != kSimpleLse) vt.store(Vs, tid);
    __syncthreads();
    if (it + 1 < it1) {
      s_cur = st.at(it + 1);
      kt.load(kbase, p.k_stride[2], s_cur * kSimpleStep, p.Lkv - 1, tid);
      if constexpr (PASS != kSimpleLse) vt.load(vbase, p.v_stride[2], s_cur * kSimpleStep, p.Lkv - 1, tid);
    }
    if (!wave_has_rows) continue;  // a wave past the last query row only helps to stage the tiles
    const bool masked = (it >= n_full_t) || (kv0 + kSimpleStep > p.Lkv);
    int cls = kBlockAll;
    if (masked) {
      cls = block_class(p.mask, visible, __builtin_amdgcn_readfirstlane(q_row - i32), kv0, 0x7fffffff, p.Lkv);
      if (cls == kBlockNone) continue;
    }
    float16_t x;
#pragma unroll
    for (int r = 0; r < 16; r++) x[r] = 0.f;
    x = Ops::row_product(Ks, i32, g, qf, x);  // S^T: rows = keys, the lane's column = its query row
    if (round_s) Ops::round_block(x);
    sm.tile(q_row, kv0 + 4 * g);
#pragma unroll
    for (int r = 0; r < 16; r++) x[r] = PASS == kSimpleNorm ? sm.apply_sub(x[r], acc_row(r), m_run) : sm.apply(x[r], acc_row(r));
    if (cls == kBlockMixed) mask_block_q(x, p.mask, visible, q_row, kv0, g, p.Lkv);
    if constexpr (PASS == kSimpleNorm) {
#pragma unroll
      for (int r = 0; r < 16; r++) x[r] = fast_exp2(x[r]);
    } else {
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
      if constexpr (PASS == kSimpleOnePass) {
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[db][r] *= alpha;
      }
    }
    if constexpr (PASS != kSimpleLse) Ops::col_product(Vs, lane, x, oacc);  // O^T += V^T.P^T
  }

  const float l_tot = PASS == kSimpleNorm ? 1.f : xhalf_sum(l_run);
  if (nsplit > 1) {
    if (q_row < p.Lq) {
      const int64_t at = (int64_t)split * p.B * p.Hq * p.Lq + row_id;
      if (g == 0) {
        ml_part[at * 2] = PASS == kSimpleNorm ? 0.f : m_run;
        ml_part[at * 2 + 1] = PASS == kSimpleNorm ? (split == 0 ? 1.f : 0.f) : l_tot;
      }
      if constexpr (PASS != kSimpleLse) {
        float* op = o_part + at * D + 4 * g;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int rr = 0; rr < 4; rr++) {
            float4_t acc4;
#pragma unroll
            for (int e = 0; e < 4; e++) acc4[e] = oacc[db][4 * rr + e];
            *reinterpret_cast<float4_t*>(op + 32 * db + 8 * rr) = acc4;
          }
      }
    }
    return;
  }
  const float inv = PASS == kSimpleNorm ? 1.f : (l_tot > 0.f ? 1.f / l_tot : 0.f);
  if (q_row < p.Lq) {
    if constexpr (PASS != kSimpleLse) {
      T* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)q_row * p.o_stride[2] + 4 * g;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int rr = 0; rr < 4; rr++)
          Ops::store4(op + 32 * db + 8 * rr, oacc[db][4 * rr] * inv, oacc[db][4 * rr + 1] * inv, oacc[db][4 * rr + 2] * inv,
                      oacc[db][4 * rr + 3] * inv);
    }
    if (PASS != kSimpleNorm && lse2 && g == 0) lse2[row_id] = l_tot > 0.f ? m_run + log2f(l_tot) : -INFINITY;
  }
}

// MODE, as in the tuned dQ kernel:
//   kSimpleBwdFast    delta_i = sum_d O_id dO_id - log2(e) d_lse2_i (written to delta_out for the dK/dV kernel),
//                     dQ = scale * (P o (dP - delta) o g) . K
//   kSimpleBwdDelta   the row sweep of the parity numerics: delta_i = sum_j P_ij round(dP_ij) - log2(e) d_lse2_i; no dQ
//   kSimpleBwdParity  reads that delta, rounds dP through T before the subtraction and applies the scale before dS
//                     is rounded
enum { kSimpleBwdFast = 0, kSimpleBwdDelta = 1, kSimpleBwdParity = 2 };
template <typename T, int D, int KIND, int MODE>
__global__ __launch_bounds__(256) void simple_dq_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                        const T* __restrict__ k, const T* __restrict__ v,
                                                        const T* __restrict__ o, const float* __restrict__ lse2,
                                                        const T* __restrict__ d_o, T* __restrict__ dq,
                                                        float* __restrict__ delta_out) {
  typedef SimpleOps<T, D> Ops;
  constexpr int DB = D / 32, ROWE = Ops::ROWE;
  __shared__ __align__(16) T Ks[kSimpleStep * ROWE];
  __shared__ __align__(16) T Vs[kSimpleStep * ROWE];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5;
  const int nqt = (p.Lq + kSimpleQTile - 1) / kSimpleQTile;
  int rank, bh;
  xcd_tile_map(blockIdx.x, nqt, p.Hq * p.B, rank, bh);
  const int qt = nqt - 1 - rank;
  const int h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);
  const int q_row = qt * kSimpleQTile + w * 32 + i32;
  const int q_ld = min(q_row, p.Lq - 1);
  const int64_t row_id = ((int64_t)b * p.Hq + h) * p.Lq + q_ld;
  const bool round_s = Ops::kRounds && (p.flags & FLEX_ROUND_S);

  typename Ops::Resident qf, dof;
  Ops::load_resident(qf, q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)q_ld * p.q_stride[2], g);
  Ops::load_resident(dof, d_o + row_id * D, g);  // dO is contiguous [B,Hq,Lq,D]
  float delta = 0.f;
  if constexpr (MODE == kSimpleBwdFast) {
    delta = xhalf_sum(Ops::dot_half(dof, o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)q_ld * p.o_stride[2], g));
    if (p.d_lse2) delta -= kLog2e * p.d_lse2[row_id];
    if (q_row < p.Lq && g == 0) delta_out[row_id] = delta;
  } else if constexpr (MODE == kSimpleBwdParity) {
    delta = delta_out[row_id];  // written by the row-sweep launch that precedes this one on the stream
  }
  float drow = 0.f;  // kSimpleBwdDelta: this lane's share of sum_j P_ij round(dP_ij)
  float lse = lse2[row_id];
  if (lse == -INFINITY) lse = INFINITY;  // row without visible keys: P = 0

  SimpleSteps st;
  const FlexTileLists& tl = p.tiles_bwd;
  st.init(tl.kv_num, tl.kv_idx, tl.full_kv_num, tl.full_kv_idx,
          (b * tl.stride_b + h * tl.stride_h) * tl.n_q_blocks + qt, tl.n_kv_blocks, tl.kv_block, p.Lkv, p.mask);
  const int nt = st.count(), n_full_t = st.full_steps();

  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  Score2<KIND> sm;
  sm.init(p.score, p.scale, h, b, p.Lq, p.Lkv);
  const Mask2 visible(p.mask, b, h, p.Lkv);

  float16_t dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) dqacc[db][r] = 0.f;

  RowTile<T, D> kt, vt;
  int s_cur = nt > 0 ? st.at(0) : 0;
  if (nt > 0) {
    kt.load(kbase, p.k_stride[2], s_cur * kSimpleStep, p.Lkv - 1, tid);
    vt.load(vbase, p.v_stride[2], s_cur * kSimpleStep, p.Lkv - 1, tid);
  }
  for (int it = 0; it < nt; it++) {
    const int kv0 = s_cur * kSimpleStep;
    __syncthreads();
    kt.store(Ks, tid);
    vt.store(Vs, tid);
    __syncthreads();
    if (it + 1 < nt) {
      s_cur = st.at(it + 1);
      kt.load(kbase, p.k_stride[2], s_cur * kSimpleStep, p.Lkv - 1, tid);
      vt.load(vbase, p.v_stride[2], s_cur * kSimpleStep, p.Lkv - 1, tid);
    }
    const bool masked = (it >= n_full_t) || (kv0 + kSimpleStep > p.Lkv);
    int cls = kBlockAll;
    if (masked) {
      cls = block_class(p.mask, visible, __builtin_amdgcn_readfirstlane(q_row - i32), kv0, 0x7fffffff, p.Lkv);
      if (cls == kBlockNone) continue;
    }
    float16_t x, dp, gr;
#pragma unroll
    for (int r = 0; r < 16; r++) { x[r] = 0.f; dp[r] = MODE == kSimpleBwdFast ? -delta : 0.f; }
    x = Ops::row_product(Ks, i32, g, qf, x);     // S^T
    dp = Ops::row_product(Vs, i32, g, dof, dp);  // dP^T (fast numerics: - delta)
    if (round_s) Ops::round_block(x);
    if constexpr (MODE != kSimpleBwdFast) Ops::round_block(dp);
    sm.tile(q_row, kv0 + 4 * g);
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float s = x[r];
      x[r] = sm.apply_sub(s, acc_row(r), lse);
      if (!Score2<KIND>::kGradOne) gr[r] = sm.grad(s, acc_row(r));
    }
    if (cls == kBlockMixed) mask_block_q(x, p.mask, visible, q_row, kv0, g, p.Lkv);
    if constexpr (MODE == kSimpleBwdDelta) {
#pragma unroll
      for (int r = 0; r < 16; r++) drow = fmaf(fast_exp2(x[r]), dp[r], drow);
      continue;
    }
#pragma unroll
    for (int r = 0; r < 16; r++) {
      float ds = fast_exp2(x[r]) * (MODE == kSimpleBwdParity ? dp[r] - delta : dp[r]);
      if (!Score2<KIND>::kGradOne) ds *= gr[r];
      if constexpr (MODE == kSimpleBwdParity) ds *= p.scale;  // before dS is rounded, as the dense path has it
      x[r] = ds;
    }
    Ops::col_product(Ks, lane, x, dqacc);  // dQ^T += K^T.dS^T
  }

  if constexpr (MODE == kSimpleBwdDelta) {
    drow = xhalf_sum(drow);
    if (p.d_lse2) drow -= kLog2e * p.d_lse2[row_id];
    if (q_row < p.Lq && g == 0) delta_out[row_id] = drow;
    return;
  }
  const float out_scale = MODE == kSimpleBwdParity ? 1.f : p.scale;
  if (q_row < p.Lq) {
    T* op = dq + row_id * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int rr = 0; rr < 4; rr++)
        Ops::store4(op + 32 * db + 8 * rr, dqacc[db][4 * rr] * out_scale, dqacc[db][4 * rr + 1] * out_scale,
                    dqacc[db][4 * rr + 2] * out_scale, dqacc[db][4 * rr + 3] * out_scale);
  }
}

// dV = P^T.dO and dK = scale * (P o (dP - delta) o g)^T . Q for the 128 keys of a workgroup (one 32-key block per
// wave, a lane owns one key), summed over the query heads of the key head's group.  PARITY: dP is rounded through T
// before delta is subtracted and the scale is applied before dS is rounded.
template <typename T, int D, int KIND, bool PARITY>
__global__ __launch_bounds__(256) void simple_dkv_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                         const T* __restrict__ k, const T* __restrict__ v,
                                                         const float* __restrict__ lse2, const float* __restrict__ delta,
                                                         const T* __restrict__ d_o, T* __restrict__ dk,
                                                         T* __restrict__ dv) {
  typedef SimpleOps<T, D> Ops;
  constexpr int DB = D / 32, ROWE = Ops::ROWE;
  __shared__ __align__(16) T Qs[kSimpleStep * ROWE];
  __shared__ __align__(16) T Os[kSimpleStep * ROWE];
  __shared__ __align__(16) float lse_s[kSimpleStep];
  __shared__ __align__(16) float ndel_s[kSimpleStep];

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i32 = lane & 31, g = lane >> 5;
  const int nkt = (p.Lkv + kSimpleKvTile - 1) / kSimpleKvTile;
  int kt, bh;  // early key tiles see the most queries under causal masks
  xcd_tile_map(blockIdx.x, nkt, p.Hkv * p.B, kt, bh);
  const int hk = bh % p.Hkv, b = bh / p.Hkv, G = p.Hq / p.Hkv;
  const int kv_col = kt * kSimpleKvTile + w * 32 + i32;
  const int kv_ld = min(kv_col, p.Lkv - 1);
  const bool round_s = Ops::kRounds && (p.flags & FLEX_ROUND_S);

  typename Ops::Resident kf, vf;
  Ops::load_resident(kf, k + b * p.k_stride[0] + hk * p.k_stride[1] + (int64_t)kv_ld * p.k_stride[2], g);
  Ops::load_resident(vf, v + b * p.v_stride[0] + hk * p.v_stride[1] + (int64_t)kv_ld * p.v_stride[2], g);
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
    SimpleSteps st;
    st.init(tl.q_num, tl.q_idx, tl.full_q_num, tl.full_q_idx,
            (b * tl.stride_b + h * tl.stride_h) * tl.n_kv_blocks + kt, tl.n_q_blocks, tl.q_block, p.Lq, p.mask);
    const int nt = st.count(), n_full_t = st.full_steps();
    const T* qbase = q + b * p.q_stride[0] + h * p.q_stride[1];
    const int64_t rows0 = ((int64_t)b * p.Hq + h) * p.Lq;
    const T* dobase = d_o + rows0 * D;

    RowTile<T, D> qt, ot;
    float lreg = INFINITY, dreg = 0.f;
    auto load_step = [&](int q0) {
      qt.load(qbase, p.q_stride[2], q0, p.Lq - 1, tid);
      ot.load(dobase, D, q0, p.Lq - 1, tid);
      lreg = INFINITY;  // rows past Lq: P = 0, whatever the clamped loads hold
      dreg = 0.f;
      if (tid < kSimpleStep && q0 + tid < p.Lq) {
        lreg = lse2[rows0 + q0 + tid];
        dreg = delta[rows0 + q0 + tid];
      }
    };
    int s_cur = nt > 0 ? st.at(0) : 0;
    if (nt > 0) load_step(s_cur * kSimpleStep);
    for (int it = 0; it < nt; it++) {
      const int q0 = s_cur * kSimpleStep;
      __syncthreads();  // the previous step's (or head's) reads are done
      qt.store(Qs, tid);
      ot.store(Os, tid);
      if (tid < kSimpleStep) {
        lse_s[tid] = lreg == -INFINITY ? INFINITY : lreg;  // row without visible keys: P = 0
        ndel_s[tid] = -dreg;
      }
      __syncthreads();
      if (it + 1 < nt) {
        s_cur = st.at(it + 1);
        load_step(s_cur * kSimpleStep);
      }
      const bool masked = (it >= n_full_t) || (q0 + kSimpleStep > p.Lq) || (kt * kSimpleKvTile + kSimpleKvTile > p.Lkv);
      int cls = kBlockAll;
      if (masked) {
        cls = block_class(p.mask, visible, q0, kt * kSimpleKvTile + w * 32, p.Lq, p.Lkv);
        if (cls == kBlockNone) continue;
      }
      const int ql = 4 * g;  // local row of register 0
      float16_t x, dp, gr, ndel;
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        const float4_t d4 = *reinterpret_cast<const float4_t*>(ndel_s + ql + 8 * rr);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          x[4 * rr + e] = 0.f;
          dp[4 * rr + e] = PARITY ? 0.f : d4[e];
          ndel[4 * rr + e] = d4[e];
        }
      }
      x = Ops::row_product(Qs, i32, g, kf, x);    // S: rows = queries, the lane's column = its key
      dp = Ops::row_product(Os, i32, g, vf, dp);  // dP (fast numerics: - delta)
      if (round_s) Ops::round_block(x);
      if constexpr (PARITY) Ops::round_block(dp);
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
        float ds = x[r] * (PARITY ? dp[r] + ndel[r] : dp[r]);
        if (!Score2<KIND>::kGradOne) ds *= gr[r];
        if constexpr (PARITY) ds *= p.scale;
        dp[r] = ds;
      }
      Ops::col_product(Os, lane, x, dvacc);   // dV^T += dO^T.P
      Ops::col_product(Qs, lane, dp, dkacc);  // dK^T += Q^T.dS
    }
  }

  const float out_scale = PARITY ? 1.f : p.scale;
  if (kv_col < p.Lkv) {
    const int64_t row_id = ((int64_t)b * p.Hkv + hk) * p.Lkv + kv_col;
    T* dkp = dk + row_id * D + 4 * g;
    T* dvp = dv + row_id * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        Ops::store4(dkp + 32 * db + 8 * rr, dkacc[db][4 * rr] * out_scale, dkacc[db][4 * rr + 1] * out_scale,
                    dkacc[db][4 * rr + 2] * out_scale, dkacc[db][4 * rr + 3] * out_scale);
        Ops::store4(dvp + 32 * db + 8 * rr, dvacc[db][4 * rr], dvacc[db][4 * rr + 1], dvacc[db][4 * rr + 2],
                    dvacc[db][4 * rr + 3]);
      }
  }
}

// everything a launch needs besides the template choice
struct SimpleArgs {
  const void *q, *k, *v, *o, *d_o;
  const float* lse2_in;
  void *out, *dq, *dk, *dv;
  float *lse2_out, *delta;
  hipStream_t s;
  bool bwd;
  // forward over split key ranges: shares per query tile (1 = none) and where their partial (O, m, l) go
  int splits;
  float *o_part, *ml_part;
};

template <typename T, int D, int KIND> void simple_launch_fwd(const FlexAttnParams& p, const SimpleArgs& a) {
  const int splits = a.splits > 1 ? a.splits : 1;
  const dim3 grid((p.Lq + kSimpleQTile - 1) / kSimpleQTile * p.Hq * p.B, splits), block(256);
  const T *q = (const T*)a.q, *k = (const T*)a.k, *v = (const T*)a.v;
  // split key ranges: every pass is followed by the merge of its partials (one wave per row)
  auto merge = [&](T* o, float* lse2) {
    if (splits == 1) return;
    const int64_t rows = (int64_t)p.B * p.Hq * p.Lq;
    hipLaunchKernelGGL((decode_combine_kernel<T, D>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, a.s, p, a.o_part, a.ml_part,
                       splits, o, lse2);
  };
  if constexpr (SimpleOps<T, D>::kRounds) {  // the parity numerics exist where something is rounded
    if (p.flags & FLEX_PARITY) {
      hipLaunchKernelGGL((simple_fwd_kernel<T, D, KIND, kSimpleLse>), grid, block, 0, a.s, p, q, k, v, (T*)a.out, a.lse2_out,
                         a.o_part, a.ml_part);
      merge(nullptr, a.lse2_out);
      hipLaunchKernelGGL((simple_fwd_kernel<T, D, KIND, kSimpleNorm>), grid, block, 0, a.s, p, q, k, v, (T*)a.out, a.lse2_out,
                         a.o_part, a.ml_part);
      merge((T*)a.out, nullptr);
      return;
    }
  }
  hipLaunchKernelGGL((simple_fwd_kernel<T, D, KIND, kSimpleOnePass>), grid, block, 0, a.s, p, q, k, v, (T*)a.out, a.lse2_out,
                     a.o_part, a.ml_part);
  merge((T*)a.out, a.lse2_out);
}
template <typename T, int D, int KIND> void simple_launch_bwd(const FlexAttnParams& p, const SimpleArgs& a) {
  const dim3 qgrid((p.Lq + kSimpleQTile - 1) / kSimpleQTile * p.Hq * p.B);
  const dim3 kgrid((p.Lkv + kSimpleKvTile - 1) / kSimpleKvTile * p.Hkv * p.B), block(256);
  const T *q = (const T*)a.q, *k = (const T*)a.k, *v = (const T*)a.v, *o = (const T*)a.o, *d_o = (const T*)a.d_o;
  if constexpr (SimpleOps<T, D>::kRounds) {  // the parity numerics exist where something is rounded
    if (p.flags & FLEX_PARITY) {
      if (!(p.flags & FLEX_BWD_ONLY_DKV)) {
        hipLaunchKernelGGL((simple_dq_kernel<T, D, KIND, kSimpleBwdDelta>), qgrid, block, 0, a.s, p, q, k, v, o, a.lse2_in,
                           d_o, (T*)a.dq, a.delta);
        hipLaunchKernelGGL((simple_dq_kernel<T, D, KIND, kSimpleBwdParity>), qgrid, block, 0, a.s, p, q, k, v, o, a.lse2_in,
                           d_o, (T*)a.dq, a.delta);
      }
      if (!(p.flags & FLEX_BWD_ONLY_DQ))
        hipLaunchKernelGGL((simple_dkv_kernel<T, D, KIND, true>), kgrid, block, 0, a.s, p, q, k, v, a.lse2_in, a.delta, d_o,
                           (T*)a.dk, (T*)a.dv);
      return;
    }
  }
  if (!(p.flags & FLEX_BWD_ONLY_DKV))
    hipLaunchKernelGGL((simple_dq_kernel<T, D, KIND, kSimpleBwdFast>), qgrid, block, 0, a.s, p, q, k, v, o, a.lse2_in, d_o,
                       (T*)a.dq, a.delta);
  if (!(p.flags & FLEX_BWD_ONLY_DQ))
    hipLaunchKernelGGL((simple_dkv_kernel<T, D, KIND, false>), kgrid, block, 0, a.s, p, q, k, v, a.lse2_in, a.delta, d_o,
                       (T*)a.dk, (T*)a.dv);
}
template <typename T, int D, int KIND> void simple_launch(const FlexAttnParams& p, const SimpleArgs& a) {
  if (a.bwd) simple_launch_bwd<T, D, KIND>(p, a);
  else simple_launch_fwd<T, D, KIND>(p, a);
}
// rc: 0 launched, 1 unknown score_mod kind
template <typename T, int D> int simple_launch_kind(const FlexAttnParams& p, const SimpleArgs& a) {
  switch (p.score.kind) {
    case FLEX_SCORE_IDENTITY: simple_launch<T, D, FLEX_SCORE_IDENTITY>(p, a); return 0;
    case FLEX_SCORE_CHECKERBOARD: simple_launch<T, D, FLEX_SCORE_CHECKERBOARD>(p, a); return 0;
    case FLEX_SCORE_ALIBI: simple_launch<T, D, FLEX_SCORE_ALIBI>(p, a); return 0;
    case FLEX_SCORE_TANH_SOFTCAP: simple_launch<T, D, FLEX_SCORE_TANH_SOFTCAP>(p, a); return 0;
    case FLEX_SCORE_REL_BIAS: simple_launch<T, D, FLEX_SCORE_REL_BIAS>(p, a); return 0;
    case FLEX_SCORE_AFFINE:
      if (p.score.mul) simple_launch<T, D, kScoreAffineMul>(p, a);
      else simple_launch<T, D, FLEX_SCORE_AFFINE>(p, a);
      return 0;
  }
  return 1;
}

}  // namespace flex
