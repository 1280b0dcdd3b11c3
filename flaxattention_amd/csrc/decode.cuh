// Split-KV decode kernels for gfx950; instantiated per (dtype, head size) by decode_inst.hip, dispatched from
// decode.hip.
#pragma once
#include "mfma_common.cuh"

namespace flex {

constexpr int kStep = 32;  // KV rows per wave step

// PASS selects the numerics, as in the forward kernel:
//   kDecOnePass  online softmax; the unnormalised P is rounded to the input dtype for the P.V product
//   kDecLse      first pass of the parity numerics: per split only (m, l), no V is read
//   kDecNorm     second pass: P = 2^(x - lse2) with the merged log-sum-exp of the first pass is the normalised
//                probability, rounded to the input dtype and multiplied into V; the splits' partial outputs simply
//                add up (written with m = 0 and l = 1 for split 0, l = 0 for the others, so that the same combine
//                kernel sums them)
enum { kDecOnePass = 0, kDecLse = 1, kDecNorm = 2 };
template <typename T, int D, int KIND, bool ROUND_S, int NB, int PASS = kDecOnePass>
__global__ __launch_bounds__(256, D >= 192 ? 1 : NB == 1 ? (D == 64 ? 3 : 2) : (D == 64 ? 2 : 1)) void decode_split_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                            const T* __restrict__ k, const T* __restrict__ v,
                                                            float* __restrict__ o_part, float* __restrict__ ml_part,
                                                            int splits, const float* __restrict__ lse_in) {
  typedef typename Frag<T>::vec8 vec8;
  // D = 256 serves one column block: the two V strips of the four waves are 128 KB of the 160 KB of LDS, which leaves
  // no room for a second block's Q fragments, and its registers (64 for Q, 64 for K, 128 for O) no room to keep them;
  // D = 192 likewise runs one wave per SIMD with one column block
  static_assert(D == 64 || D == 128 || ((D == 192 || D == 256) && NB == 1), "decode_split_kernel: head size / column blocks");
  constexpr int DS = D / 16, DB = D / 32, ROWE = D + 8, CPR = D / 8;
  // a strip is kStep * CPR chunks, 64 per wave-wide fetch instruction, laid down one after the other (at D = 192 an
  // instruction ends in the middle of a row)
  constexpr int NVI = kStep * CPR / 64;  // fetch instructions per step
  static_assert((kStep * CPR) % 64 == 0, "whole fetch instructions per strip");
  // V strips: per wave NSTG stages of 32 unpadded swizzled rows, filled global -> LDS directly (no staging
  // registers).  The same memory serves the cross-wave reduction of the partial outputs at the end.
  // NSTG V strips per wave and DEPTH = NSTG - 1 steps of loads in flight while one is computed.  Three strips and two
  // sets of K registers (two steps ahead) were measured at D = 64 and change nothing (fp16 KV cache [8,8,16384,64], one workgroup per
  // compute unit: 53.2 us against 52.9 us at q_len 1, 57.1 against 55.7 at q_len 64): the bytes in flight are not what
  // limits this kernel, so two strips and one step ahead it stays.
  constexpr int NSTG = 2, DEPTH = NSTG - 1;
  constexpr int kStripElems = kStep * D;
  constexpr int kVsBytes = 4 * NSTG * kStripElems * (int)sizeof(T), kRedBytes = 4 * 16 * 64 * (int)sizeof(float);
  __shared__ __align__(16) unsigned char vs_red[kVsBytes > kRedBytes ? kVsBytes : kRedBytes];
  __shared__ float mbuf[4][NB][32];
  // two column blocks at D = 128: the Q fragments (64 registers) are re-read from LDS every step instead
  constexpr bool kQInLds = NB == 2 && D == 128;
  __shared__ __align__(16) T Qs[kQInLds ? 64 * ROWE : 8];
  float (*red)[16][64] = reinterpret_cast<float (*)[16][64]>(vs_red);

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, provably uniform: step addresses stay scalar
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
    if (kQInLds && w == 0) {
#pragma unroll
      for (int s = 0; s < DS; s++) *reinterpret_cast<vec8*>(Qs + (nb * 32 + i32) * ROWE + 16 * s + 8 * g) = qf[nb][s];
    }
  }
  if (kQInLds) __syncthreads();

  // schedule, in this order of preference:
  //  (1) a band mask whose visible keys form ONE range for the rows of this call (no sink keys, or no window): the
  //      range follows from the mask parameters by scalar arithmetic, so the steps are walked linearly and no list is
  //      read at all (a list lookup is a dependent global load in front of every K / V fetch: 6 us of a 59 us call);
  //  (2) list entries (64-key tiles of the query block the rows sit in) when given at that granularity, with all
  //      rows in one query block, and G == 1;
  //  (3) every step, with the mask evaluated in each.
  const FlexTileLists& tl = p.tiles;
  const int32_t* full_idx = nullptr;
  const int32_t* part_idx = nullptr;
  int n_full = 0, steps_total, step_lo = 0;
  const int q_lo = p.q_index_base, q_hi = p.q_index_base + p.Lq - 1;  // rows of this call
  const bool one_range = p.mask.kind == FLEX_MASK_BAND && (p.mask.hi >= kBig || p.mask.sink < 0);
  // keys every row sees / some row sees, from d = q + q_offset - kv, d >= lo && d <= hi
  const int vis_hi_all = min(clamp_big(q_lo + p.mask.q_offset) - clamp_big(p.mask.lo), kBig);   // kv <= this for the first row
  const int vis_hi_any = min(clamp_big(q_hi + p.mask.q_offset) - clamp_big(p.mask.lo), kBig);
  const int vis_lo_all = p.mask.hi >= kBig ? 0 : max(q_hi + p.mask.q_offset - p.mask.hi, 0);    // kv >= this for the last row
  const int vis_lo_any = p.mask.hi >= kBig ? 0 : max(q_lo + p.mask.q_offset - p.mask.hi, 0);
  if (one_range) {
    const int kv_last = min(vis_hi_any, p.Lkv - 1);
    step_lo = vis_lo_any / kStep;
    steps_total = kv_last >= vis_lo_any ? kv_last / kStep - step_lo + 1 : 0;
  } else if (tl.kv_num && G == 1 && tl.kv_block == 2 * kStep && p.q_index_base % tl.q_block + p.Lq <= tl.q_block) {
    const int64_t row = (b * tl.stride_b + hk * tl.stride_h) * tl.n_q_blocks + p.q_index_base / tl.q_block;
    n_full = uniform_ld(tl.full_kv_num + row);
    const int n_part = uniform_ld(tl.kv_num + row);
    full_idx = tl.full_kv_idx + row * tl.n_kv_blocks;
    part_idx = tl.kv_idx + row * tl.n_kv_blocks;
    steps_total = 2 * (n_full + n_part);
  } else {
    steps_total = (p.Lkv + kStep - 1) / kStep;
  }
  auto step_kv0 = [&](int st) -> int {
    if (!full_idx) return (step_lo + st) * kStep;
    const int item = st >> 1;
    const int tile = uniform_ld(item < n_full ? full_idx + item : part_idx + (item - n_full));
    return tile * (2 * kStep) + (st & 1) * kStep;
  };
  const int per = (steps_total + splits - 1) / splits;
  const int st_begin = split * per, st_end = min(st_begin + per, steps_total);

  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  const int64_t ks2 = p.k_stride[2], vs2 = p.v_stride[2];

  // Loads of a step: scalar base (kbase + kv0 * stride) plus small per-lane
  // offsets.  Rows past the end are clamped to the last row: their scores are
  // masked out and their P is 0, so what they hold does not matter as long as
  // it is finite.
  const int last = p.Lkv - 1;
  vec8 kfA[DS], kfB[DS];  // two sets of K registers, named so that they stay in registers (kfB unused at DEPTH 1)
  T* Vw = reinterpret_cast<T*>(vs_red) + w * NSTG * kStripElems;
  // V first, K last: loads return in order, so once the K registers of a step have arrived (the
  // compiler waits for them before the first MFMA) the V strip of that step has landed too
  auto load_step = [&](vec8 (&kfr)[DS], int kv0, int stage) {
    const int lim = last - kv0;  // last valid row of this step, relative
    const T* vp = vbase + (int64_t)kv0 * vs2;
    if constexpr (PASS != kDecLse) {
#pragma unroll
      for (int j = 0; j < NVI; j++) {
        const int c = 64 * j + lane, r = c / CPR;   // the strip row and position this lane fills
        const T* vg = vp + min(r, lim) * (int)vs2 + (((c % CPR) ^ lds_swz<D>(r)) * 8);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vg,
                                         (__attribute__((address_space(3))) void*)(Vw + stage * kStripElems + 512 * j), 16, 0, 0);
      }
    }
    const T* kp = kbase + (int64_t)kv0 * ks2 + min(i32, lim) * (int)ks2 + 8 * g;
#pragma unroll
    for (int s = 0; s < DS; s++) kfr[s] = *reinterpret_cast<const vec8*>(kp + 16 * s);
  };
  // transposing reads of a strip: 4 elements of row 4g + (i16 >> 2) + 8e (+16t), logical column 32db + 16hh + 4(i16 & 3)
  int voff[2][DB];
  {
    const int rl = 4 * g + (i16 >> 2), hh = (lane >> 4) & 1;
#pragma unroll
    for (int e = 0; e < 2; e++)
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const int chunk = 4 * db + 2 * hh + ((i16 & 3) >> 1);
        voff[e][db] = (rl + 8 * e) * D + ((chunk ^ lds_swz<D>(rl + 8 * e)) * 8) + 4 * (i16 & 1);
      }
  }

  Score2<KIND> sm[NB];
  float m_run[NB], l_run[NB];
  float16_t oacc[NB][DB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    sm[nb].init(p.score, p.scale, col_h[nb]);
    m_run[nb] = -INFINITY;
    l_run[nb] = 0.f;
    if constexpr (PASS == kDecNorm) {
      // the merged log-sum-exp of the first pass is the fixed reference; a column without visible keys gets +inf (P = 0)
      const float l2 = lse_in[((int64_t)b * p.Hq + col_h[nb]) * p.Lq + col_q[nb]];
      m_run[nb] = l2 == -INFINITY ? INFINITY : l2;
    }
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[nb][db][r] = 0.f;
  }
  const bool trivial_mask = p.mask.kind == FLEX_MASK_BAND && p.mask.lo == INT32_MIN && p.mask.hi == INT32_MAX;
  constexpr float kTau = 8.f;

  // KV offsets are looked up four visits ahead so that the (dependent) tile-index load never sits between a wave
  // and its next K/V loads
  int st = st_begin + w;
  int kv_q0 = st < st_end ? step_kv0(st) : 0;
  int kv_q1 = st + 4 < st_end ? step_kv0(st + 4) : 0;
  int kv_q2 = st + 8 < st_end ? step_kv0(st + 8) : 0;
  int kv_q3 = st + 12 < st_end ? step_kv0(st + 12) : 0;
  int stage = 0;
  if (st < st_end) load_step(kfA, kv_q0, 0);
  if (DEPTH == 2 && st + 4 < st_end) load_step(kfB, kv_q1, 1);
  // one step of this wave; kfr holds its K rows and is refilled for the step DEPTH visits later
  auto visit = [&](vec8 (&kfr)[DS]) {
    const int kv0 = kv_q0;
    // scores first: they consume the K registers, which the next step's loads then reuse
    float16_t s_a, s_b;  // named (not an array) so that they stay in registers
#pragma unroll
    for (int r = 0; r < 16; r++) { s_a[r] = 0.f; s_b[r] = 0.f; }
#pragma unroll
    for (int s = 0; s < DS; s++) {
      if (!kQInLds) {
        s_a = Frag<T>::mfma(kfr[s], qf[0][s], s_a);
        if (NB > 1) s_b = Frag<T>::mfma(kfr[s], qf[NB - 1][s], s_b);
      } else {
        const T* qp = Qs + i32 * ROWE + 16 * s + 8 * g;
        s_a = Frag<T>::mfma(kfr[s], *reinterpret_cast<const vec8*>(qp), s_a);
        s_b = Frag<T>::mfma(kfr[s], *reinterpret_cast<const vec8*>(qp + 32 * ROWE), s_b);
      }
    }
    // this step's V strip landed with its K registers (loads return in order); the strip refilled now was last
    // read a step ago
    if (st + 4 * DEPTH < st_end) load_step(kfr, DEPTH == 2 ? kv_q2 : kv_q1, stage + DEPTH >= NSTG ? stage + DEPTH - NSTG : stage + DEPTH);
    kv_q0 = kv_q1;
    kv_q1 = kv_q2;
    kv_q2 = kv_q3;
    if (st + 16 < st_end) kv_q3 = step_kv0(st + 16);
    // steps that every row of the call sees completely need no mask evaluation: those from the list of fully
    // visible tiles, and under a one-range band mask those inside the range common to all rows
    const bool listed_full = full_idx && (st >> 1) < n_full;
    const bool band_full = one_range && kv0 >= vis_lo_all && kv0 + kStep - 1 <= vis_hi_all;
    const bool need_mask = (!trivial_mask && !listed_full && !band_full) || (kv0 + kStep > p.Lkv);

    vec8 pf[NB][2];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      float16_t sacc = nb ? s_b : s_a;
      const float m_use = (PASS != kDecNorm && m_run[nb] == -INFINITY) ? 0.f : m_run[nb];
      sm[nb].tile(col_q[nb] + p.q_index_base, kv0 + 4 * g);
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float s0 = sacc[r], s1 = sacc[r + 1];
        if (ROUND_S) round_pair<T>(s0, s1);
        sacc[r] = sm[nb].apply_sub(s0, acc_row(r), m_use);
        sacc[r + 1] = sm[nb].apply_sub(s1, acc_row(r + 1), m_use);
      }
      if (need_mask) {
        // a real branch whose inputs pass through the asm, so that none of the mask
        // arithmetic can be hoisted into the unmasked path
        int q_opaque = col_q[nb] + p.q_index_base, kv_opaque = kv0;
        asm volatile("" : "+v"(q_opaque), "+v"(kv_opaque));
        Mask2 visible(p.mask, b, col_h[nb], p.Lkv);
        mask_block_q(sacc, p.mask, visible, q_opaque, kv_opaque, g, p.Lkv);
      }
      // online softmax; the reference max moves only when it is beaten by 2^kTau
      if constexpr (PASS != kDecNorm) {
        const float m_rel = xhalf_max(block_max(sacc));
        const bool need = (m_rel > kTau) || (m_run[nb] == -INFINITY && m_rel > -INFINITY);
        if (__any(need)) {
          const float delta = need ? m_rel : 0.f;
          const float alpha = (m_run[nb] == -INFINITY) ? 0.f : fast_exp2(-delta);
          m_run[nb] = need ? (m_use + m_rel) : m_run[nb];
          l_run[nb] *= alpha;
#pragma unroll
          for (int r = 0; r < 16; r++) sacc[r] -= delta;
          if constexpr (PASS == kDecOnePass) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
              for (int r = 0; r < 16; r++) oacc[nb][db][r] *= alpha;
          }
        }
      }
      if constexpr (PASS == kDecLse) {
        // only the row sums, in fp32 (the dense path sums the unrounded exponentials)
#pragma unroll
        for (int r = 0; r < 16; r++) l_run[nb] += fast_exp2(sacc[r]);
      } else {
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
          typename Pair<T>::v2 pr[4];
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float p0 = fast_exp2(sacc[8 * tt + 2 * e]);
            const float p1 = fast_exp2(sacc[8 * tt + 2 * e + 1]);
            pr[e] = Pair<T>::pack(p0, p1);
            if constexpr (PASS == kDecOnePass) l_run[nb] = Pair<T>::add_sum(pr[e], l_run[nb]);
          }
          pf[nb][tt] = join_pairs<T>(pr[0], pr[1], pr[2], pr[3]);
        }
      }
    }
    if constexpr (PASS != kDecLse) {
      // the V strips belong to this wave alone: no workgroup barrier is needed
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < 2; t++) {
#pragma unroll
        for (int db = 0; db < DB; db++) {
          const T* vp = Vw + stage * kStripElems + 16 * t * D;
          vec8 a = join8<vec8>(lds_read_tr(vp + voff[0][db]), lds_read_tr(vp + voff[1][db]));
#pragma unroll
          for (int nb = 0; nb < NB; nb++) oacc[nb][db] = Frag<T>::mfma(a, pf[nb][t], oacc[nb][db]);
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    st += 4;
    stage = stage + 1 == NSTG ? 0 : stage + 1;
  };
  while (st < st_end) {
    visit(kfA);
    if (DEPTH == 2 && st < st_end) visit(kfB);
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
    // kDecNorm: every wave used the same fixed reference (possibly +inf), the partial outputs just add up
    const float sc = PASS == kDecNorm ? 1.f : ((m_run[nb] == -INFINITY) ? 0.f : fast_exp2(m_run[nb] - mm));
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
      ml[0] = PASS == kDecNorm ? 0.f : m_all[nb];
      ml[1] = PASS == kDecNorm ? (split == 0 ? 1.f : 0.f) : lt;
    }
    if constexpr (PASS == kDecLse) continue;  // no partial output in the log-sum-exp pass
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

// one wave per output row: merge the splits, normalise, write O and lse2.
// Lane s first takes split s's (m, l) so that the max and the weights come from
// one round of loads; the partial outputs are then fetched with all loads in
// flight together.
template <typename T, int D>
__global__ __launch_bounds__(256) void decode_combine_kernel(FlexAttnParams p, const float* __restrict__ o_part,
                                                              const float* __restrict__ ml_part, int splits,
                                                              T* __restrict__ o, float* __restrict__ lse2) {
  const int lane = threadIdx.x & 63;
  const int64_t rows = (int64_t)p.B * p.Hq * p.Lq;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float ms = -INFINITY, ls = 0.f;
  if (lane < splits) {
    const float2 ml = *reinterpret_cast<const float2*>(ml_part + (lane * rows + row) * 2);
    ms = ml.x;
    ls = ml.y;
  }
  // the first eight splits' partial outputs are requested together with the (m, l) pairs, before anything waits:
  // the kernel is a chain of memory latencies (its data was written by other XCDs and comes from HBM), and this
  // way there is one of them instead of two
  float v0[8][D / 64];
  if (o) {
#pragma unroll
    for (int u = 0; u < 8; u++)
#pragma unroll
      for (int a = 0; a < D / 64; a++) v0[u][a] = (u < splits) ? o_part[(u * rows + row) * D + lane + 64 * a] : 0.f;
  }
  float m = ms;
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  const float sc = (ms == -INFINITY) ? 0.f : fast_exp2(ms - m);
  float l = sc * ls;
  for (int off = 32; off > 0; off >>= 1) l += __shfl_xor(l, off, 64);
  if (lse2 && lane == 0) lse2[row] = l > 0.f ? m + log2f(l) : -INFINITY;
  if (!o) return;  // first pass of the parity numerics: only the merged log-sum-exp
  float acc[D / 64];
#pragma unroll
  for (int a = 0; a < D / 64; a++) acc[a] = 0.f;
#pragma unroll
  for (int u = 0; u < 8; u++) {
    const float w = __shfl(sc, u, 64);
#pragma unroll
    for (int a = 0; a < D / 64; a++) acc[a] = fmaf(w, v0[u][a], acc[a]);
  }
  for (int s0 = 8; s0 < splits; s0 += 8) {
    float v[8][D / 64];
#pragma unroll
    for (int u = 0; u < 8; u++)
#pragma unroll
      for (int a = 0; a < D / 64; a++)
        v[u][a] = (s0 + u < splits) ? o_part[((s0 + u) * rows + row) * D + lane + 64 * a] : 0.f;
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const float w = __shfl(sc, s0 + u, 64);
#pragma unroll
      for (int a = 0; a < D / 64; a++) acc[a] = fmaf(w, v[u][a], acc[a]);
    }
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  const int qi = (int)(row % p.Lq);
  const int h = (int)((row / p.Lq) % p.Hq), b = (int)(row / ((int64_t)p.Lq * p.Hq));
  T* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)qi * p.o_stride[2];
#pragma unroll
  for (int a = 0; a < D / 64; a++) op[lane + 64 * a] = (T)(acc[a] * inv);
}

struct DecodeArgs {
  const void *q, *k, *v;
  void* o;
  float* lse2;      // output, may be null
  float* lse_pass;  // parity numerics: where the first pass leaves the merged log-sum-exp (lse2 or workspace)
  float *o_part, *ml_part;
  int splits;
  hipStream_t s;
};

template <typename T, int D, int KIND, bool RS, int PASS>
static void launch_nb(const FlexAttnParams& p, const DecodeArgs& a) {
  dim3 grid(a.splits, p.Hkv, p.B);
  const int ncols = (p.Hq / p.Hkv) * p.Lq;
  if (ncols <= 32 || D >= 192) {  // the caller has checked that D = 192 / 256 come with at most 32 columns
    hipLaunchKernelGGL((decode_split_kernel<T, D, KIND, RS, 1, PASS>), grid, dim3(256), 0, a.s, p, (const T*)a.q, (const T*)a.k,
                       (const T*)a.v, a.o_part, a.ml_part, a.splits, a.lse_pass);
  } else if constexpr (D < 192) {
    hipLaunchKernelGGL((decode_split_kernel<T, D, KIND, RS, 2, PASS>), grid, dim3(256), 0, a.s, p, (const T*)a.q, (const T*)a.k,
                       (const T*)a.v, a.o_part, a.ml_part, a.splits, a.lse_pass);
  }
}

template <typename T, int D>
static void launch_combine(const FlexAttnParams& p, const DecodeArgs& a, T* o, float* lse2) {
  const int64_t rows = (int64_t)p.B * p.Hq * p.Lq;
  hipLaunchKernelGGL((decode_combine_kernel<T, D>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, a.s, p, a.o_part, a.ml_part,
                     a.splits, o, lse2);
}

template <typename T, int D, int KIND>
static void launch_rs(const FlexAttnParams& p, const DecodeArgs& a) {
  if (p.flags & FLEX_PARITY) {
    // parity numerics: (m, l) per split and their merge into the log-sum-exp, then the pass that multiplies the
    // normalised, rounded P into V and the sum of the splits' partial outputs
    launch_nb<T, D, KIND, true, kDecLse>(p, a);
    launch_combine<T, D>(p, a, nullptr, a.lse_pass);
    launch_nb<T, D, KIND, true, kDecNorm>(p, a);
    launch_combine<T, D>(p, a, (T*)a.o, nullptr);
    return;
  }
  if (p.flags & FLEX_ROUND_S) launch_nb<T, D, KIND, true, kDecOnePass>(p, a);
  else launch_nb<T, D, KIND, false, kDecOnePass>(p, a);
  launch_combine<T, D>(p, a, (T*)a.o, a.lse2);
}

template <typename T, int D>
static int launch_all(const FlexAttnParams& p, const DecodeArgs& a) {
  switch (p.score.kind) {
    case FLEX_SCORE_IDENTITY: launch_rs<T, D, FLEX_SCORE_IDENTITY>(p, a); break;
    case FLEX_SCORE_CHECKERBOARD: launch_rs<T, D, FLEX_SCORE_CHECKERBOARD>(p, a); break;
    case FLEX_SCORE_ALIBI: launch_rs<T, D, FLEX_SCORE_ALIBI>(p, a); break;
    case FLEX_SCORE_TANH_SOFTCAP: launch_rs<T, D, FLEX_SCORE_TANH_SOFTCAP>(p, a); break;
    case FLEX_SCORE_REL_BIAS: launch_rs<T, D, FLEX_SCORE_REL_BIAS>(p, a); break;
    default: return 1;
  }
  return 0;
}

}  // namespace flex
