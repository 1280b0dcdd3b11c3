// Fused flash-attention forward for gfx950 (fp16 / bf16, D = Dv in {64, 128}; the list-driven kernel also 256).
//
// Takes the place of mha_forward_kernel (flaxattention/kernel/attention.py:
// 34-149) and of the dense math path (flaxattention/core/attention.py:14-106)
// for 16-bit inputs, with a real online softmax and with skipping of masked-out
// KV tiles, which the reference computes but never uses.
//
// Two kernels.  fwd_mfma_kernel (any supported D, tile lists or not): one workgroup
// (4 waves) per 128 query rows of one (batch, head), one 32-row block per wave; KV tiles of
// 64 rows go through two LDS stages (fetched global -> LDS directly one tile ahead, one workgroup
// barrier per tile).  fwd_pipe_kernel (D = 64, no tile lists, a mask that hides nothing): 256 query rows per
// workgroup, two blocks per wave, software-pipelined (see there).
// Per 32-key step and 32-row block:
//   S^T[kv, q]  = K_step . Q^T          D/16 v_mfma_f32_32x32x16
//   online softmax in the accumulator layout: a lane holds 16 of the 32 scores
//   of ONE query row, the other 16 sit in lane ^ 32 -> row max/sum are
//   in-register reductions plus one permlane32 swap; the reference value of the
//   exponents is not a running maximum: it moves only when a block's exponentials
//   leave the safe range, so there is no max tree and the accumulator is rarely rescaled
//   O^T[d, q] += V_step^T . P^T         D/16 v_mfma (P^T is already in B-operand
//   layout; V^T fragments come from transposing LDS reads)
#pragma once
#include "mfma_common.cuh"
#include "decode.cuh"  // decode_combine_kernel merges the partials of a forward over split key ranges

namespace flex {

constexpr int kFwdBN = 64;
constexpr int kFwdBM = 128;   // query rows of a list-driven workgroup = q granularity of the forward lists
constexpr int kPipeBM = 256;  // query rows of a workgroup of the pipelined dense kernel (D = 64, no lists)

// BITS: the mask is a bitmap.  Band masks get an instantiation of their own, without the bitmap code and the scalar
// registers its pointers and strides occupy.
//
// PASS selects the numerics:
//   kFwdOnePass  online softmax; the unnormalised P is rounded to the input dtype for the P.V product
//   kFwdLse      first pass of the parity numerics: only the base-2 log-sum-exp of every row (no V, no P.V)
//   kFwdNorm     second pass: P = 2^(x - lse2) is the normalised probability, rounded to the input dtype and
//                multiplied into V as it is -- what the dense path computes (attention.py:104-105 normalises in
//                fp32, casts P to the input dtype and then multiplies)
//   kFwdHiLo     one pass as kFwdOnePass, but P goes into the P.V product as a high and a low part (two matrix
//                instructions per fragment) and the row sum adds the unrounded exponentials: the "unrounded"
//                numerics, launched with ROUND_S = false
enum { kFwdOnePass = 0, kFwdLse = 1, kFwdNorm = 2, kFwdHiLo = 3 };
// D = 256: one wave per SIMD (Q fragments, K fragments and the accumulator are 64 + 64 + 128 registers, the V
// fragments another 64 that are fetched late) and the two stages are 128 KB.
template <typename T, int D, int KIND, bool ROUND_S, bool BITS, int PASS = kFwdOnePass>
__global__ __launch_bounds__(256, D >= 192 ? 1 : 2) void fwd_mfma_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                           const T* __restrict__ k, const T* __restrict__ v,
                                                           T* __restrict__ o, float* __restrict__ lse2,
                                                           float* __restrict__ o_part, float* __restrict__ ml_part) {
  // Split-KV: with gridDim.y > 1 workgroup (x, y) visits share y of its query tile's key tiles and leaves an
  // unnormalised partial (O, m, l) per row in o_part / ml_part, in the layout decode_combine_kernel merges (kFwdLse:
  // only (m, l); kFwdNorm: the partial outputs add up, written with m = 0 and l = 1 for share 0, l = 0 for the
  // others).  For calls whose query tiles alone would leave most compute units without a workgroup.
  typedef typename Frag<T>::vec8 vec8;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  constexpr int RQ = 1, BM = kFwdBM, BN = kFwdBN;
  constexpr int DS = D / 16;     // k-steps of the Q.K^T product
  constexpr int DB = D / 32;     // 32-row blocks of O^T
  constexpr int CPR = D / 8;     // 16-byte chunks per row
  // a wave fills 16 rows (one swizzle period) of a tile: 16 * CPR chunks, 64 per fetch instruction, laid down one after
  // the other; at D = 192 an instruction ends in the middle of a row
  constexpr int NI = 16 * CPR / 64;    // fetch instructions per wave, tile and tensor
  static_assert((BN / 4) == 16 && (16 * CPR) % 64 == 0, "a wave's share of a tile is one swizzle period");
  // two LDS stages, filled straight from global memory (no staging registers, unpadded swizzled rows): while one
  // tile is consumed the next one lands, one workgroup barrier per tile.  Each stage is a variable of its own and
  // every access names its stage at compile time (the tile loop is unrolled by two): only then can the compiler
  // tell that a read of one stage need not wait for the fetch into the other.
  constexpr int kVElems = PASS == kFwdLse ? 8 : BN * D;
  __shared__ __align__(16) T Ksm0[BN * D];
  __shared__ __align__(16) T Ksm1[BN * D];
  __shared__ __align__(16) T Vsm0[kVElems];
  __shared__ __align__(16) T Vsm1[kVElems];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5, i16 = lane & 15;
  const int nqt = (p.Lq + BM - 1) / BM;
  int rank, bh;
  xcd_tile_map(blockIdx.x, nqt, p.Hq * p.B, rank, bh);
  const int qt = nqt - 1 - rank;  // late query tiles see the most keys under causal masks
  const int h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);

  // this lane's query rows: block a sits at q_row0 + 32 * a
  const int q_row0 = qt * BM + w * (32 * RQ) + i32;

  // Q fragments (B operand of S^T = K.Q^T), resident for the whole kernel
  vec8 qf[RQ][DS];
#pragma unroll
  for (int a = 0; a < RQ; a++) {
    const int q_ld = min(q_row0 + 32 * a, p.Lq - 1);
    const T* qp = q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)q_ld * p.q_stride[2] + 8 * g;
#pragma unroll
    for (int s = 0; s < DS; s++) qf[a][s] = *reinterpret_cast<const vec8*>(qp + 16 * s);
  }

  // tile schedule
  const FlexTileLists& tl = p.tiles;
  const int32_t* full_idx = nullptr;
  const int32_t* part_idx = nullptr;
  int n_full, n_part = 0;
  if (tl.kv_num) {
    const int64_t row = (b * tl.stride_b + h * tl.stride_h) * tl.n_q_blocks + qt;
    n_full = uniform_ld(tl.full_kv_num + row);
    n_part = uniform_ld(tl.kv_num + row);
    full_idx = tl.full_kv_idx + row * tl.n_kv_blocks;
    part_idx = tl.kv_idx + row * tl.n_kv_blocks;
  } else {
    // no lists: every tile is visited, and evaluated under a mask that can hide something
    n_full = (p.Lkv + BN - 1) / BN;
    if (!mask_hides_nothing(p.mask)) { n_part = n_full; n_full = 0; }
  }
  // Visiting order: partial tiles first, then the fully visible ones, each from the last key tile to the first.
  // Under causal-like masks with a score_mod that favours recent keys (ALiBi, relative-position biases) the largest
  // scores of a row are then met first, and the row's exponent reference, once set, never has to move again.
  const int nt = n_full + n_part;
  auto tile_at = [&](int it) -> int {
    if (!full_idx) return nt - 1 - it;
    return uniform_ld(it < n_part ? part_idx + (n_part - 1 - it) : full_idx + (n_full - 1 - (it - n_part)));
  };
  // this workgroup's share of the visits: [it0, it1)
  const int nsplit = gridDim.y, split = blockIdx.y;
  const int per = (nt + nsplit - 1) / nsplit;
  const int it0 = split * per, it1 = min(it0 + per, nt);

  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  const int64_t ks2 = p.k_stride[2], vs2 = p.v_stride[2];

  // tile fetch: wave w fills rows [16w, 16w + 16) of the K and the V tile, RPI rows per instruction; the lane that
  // fills position (r, pos) fetches chunk pos ^ lds_swz(r) of that row.  The per-lane part of a fetch address (row
  // inside the swizzle period, swizzled chunk) is the same for every tile: kept as byte offsets from a wave-uniform
  // row address.
  const int wu = __builtin_amdgcn_readfirstlane(w);
  uint32_t koff[NI], voff[NI];
#pragma unroll
  for (int j = 0; j < NI; j++) {
    const int c = 64 * j + lane, row = c / CPR, chunk = (c % CPR) ^ lds_swz<D>(row);
    koff[j] = (uint32_t)((row * ks2 + chunk * 8) * (int64_t)sizeof(T));
    voff[j] = (uint32_t)((row * vs2 + chunk * 8) * (int64_t)sizeof(T));
  }
  auto issue_tile = [&](auto stage, int kv0_in) {
    T* const Kst = stage_ptr(stage, Ksm0, Ksm1);
    T* const Vst = stage_ptr(stage, Vsm0, Vsm1);
    const int kv0 = __builtin_amdgcn_readfirstlane(kv0_in);
    const int lim = p.Lkv - 1 - kv0;
    const int r0 = 16 * wu;
    if (lim >= BN - 1) {
      const char* kt = reinterpret_cast<const char*>(kbase + (int64_t)(kv0 + r0) * ks2);
      const char* vt = reinterpret_cast<const char*>(vbase + (int64_t)(kv0 + r0) * vs2);
#pragma unroll
      for (int j = 0; j < NI; j++) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kt + koff[j]),
                                         (__attribute__((address_space(3))) void*)(Kst + r0 * D + 512 * j), 16, 0, 0);
        if constexpr (PASS != kFwdLse)
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vt + voff[j]),
                                           (__attribute__((address_space(3))) void*)(Vst + r0 * D + 512 * j), 16, 0, 0);
      }
    } else {
      // the last tile of a ragged length: rows past the end are clamped (finite filler, masked out below)
#pragma unroll
      for (int j = 0; j < NI; j++) {
        const int c = 64 * j + lane, rw = c / CPR, chunk = (c % CPR) ^ lds_swz<D>(rw);
        const int row = min(r0 + rw, lim);
        const T* kg = kbase + (int64_t)(kv0 + row) * ks2 + chunk * 8;
        const T* vg = vbase + (int64_t)(kv0 + row) * vs2 + chunk * 8;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)kg,
                                         (__attribute__((address_space(3))) void*)(Kst + r0 * D + 512 * j), 16, 0, 0);
        if constexpr (PASS != kFwdLse)
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vg,
                                           (__attribute__((address_space(3))) void*)(Vst + r0 * D + 512 * j), 16, 0, 0);
      }
    }
  };
  // element offsets inside a 32-row block: row fragments (row i32, chunk 2s + g sits at (2s) ^ kz) and
  // transposing reads (4 elements of row 4g + (i16 >> 2) + 8e, logical column 32db + 16hh + 4(i16 & 3))
  const int kz = g ^ lds_swz<D>(i32);
  int toff[2][DB];
  {
    const int rl = 4 * g + (i16 >> 2), hh = (lane >> 4) & 1;
#pragma unroll
    for (int e = 0; e < 2; e++)
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const int chunk = 4 * db + 2 * hh + ((i16 & 3) >> 1);
        toff[e][db] = (rl + 8 * e) * D + ((chunk ^ lds_swz<D>(rl + 8 * e)) * 8) + 4 * (i16 & 1);
      }
  }

  Score2<KIND> sm;
  sm.init(p.score, p.scale, h, b, p.Lq, p.Lkv);

  float16_t oacc[RQ][DB];
  float m_run[RQ], l_run[RQ];
#pragma unroll
  for (int a = 0; a < RQ; a++) {
    m_run[a] = 0.f;  // reference value of the row's exponents; moved only by the guard in the loop
    l_run[a] = 0.f;
    if constexpr (PASS == kFwdNorm) {
      // the row's log-sum-exp from the first pass takes the place of the running reference maximum and never
      // moves; a row without visible keys (-inf) gets +inf, so that every P is 0
      const float l2 = lse2[((int64_t)b * p.Hq + h) * p.Lq + min(q_row0 + 32 * a, p.Lq - 1)];
      m_run[a] = l2 == -INFINITY ? INFINITY : l2;
    }
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[a][db][r] = 0.f;
  }

  // the reference value of a row's exponents moves only when a lane's share of a block's row sum exceeds kPGuard
  // (fp16 tops out at 65504; sums are kept in fp32) or when a row that has accumulated nothing sees a block whose
  // exponentials are all below kPTiny
  constexpr float kPGuard = 32768.f, kPTiny = 1.f / 64.f;
  int t_cur = it0 < it1 ? tile_at(it0) : 0;
  int t_nxt = it0 + 1 < it1 ? tile_at(it0 + 1) : 0;
  if (it0 < it1) issue_tile(StageC<0>{}, t_cur * BN);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the Q fragments and this wave's share of the first tile
  __syncthreads();
  // one tile out of the stage named by `stage` (= (it - it0) & 1)
  auto tile_step = [&](auto stage, int it) {
    constexpr int ST = decltype(stage)::value;
    const int kv0 = t_cur * BN;
    const bool masked = (it < n_part) || (kv0 + BN > p.Lkv);
    const T* const Ks = stage_ptr(stage, Ksm0, Ksm1);
    const T* const Vs = stage_ptr(stage, Vsm0, Vsm1);
    if (it + 1 < it1) {
      // the other stage was last read before the previous barrier: the next tile lands there while this one is
      // consumed; the tile index after that is looked up a tile ahead
      issue_tile(StageC<1 - ST>{}, t_nxt * BN);
      t_cur = t_nxt;
      if (it + 2 < it1) t_nxt = tile_at(it + 2);
    }

    // Each 32-row half of the tile is one online-softmax step.
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
      // most 32x32 blocks of a partial tile are entirely visible (no mask evaluation) or
      // entirely hidden (the step is skipped)
      int cls = kBlockAll;
      if (masked) {
        if constexpr (BITS) {
          const Mask2 visible(p.mask, b, h, p.Lkv);
          cls = block_class<true>(p.mask, visible, __builtin_amdgcn_readfirstlane(q_row0 - i32), kv0 + nb * 32, 0x7fffffff, p.Lkv);
        } else {
          cls = band_block_class(p.mask, __builtin_amdgcn_readfirstlane(q_row0 - i32), kv0 + nb * 32, 0x7fffffff, p.Lkv);
        }
      }
      if (cls != kBlockNone) {
      sm.tile(q_row0, kv0 + nb * 32 + 4 * g);  // a table-reading score_mod fetches its entries under the products
      // ---- operand fragments of this step: K rows, and V columns (transposed reads) ----
      vec8 kfr[DS], vfr[2][DB];
      {
        const T* kp = Ks + (nb * 32 + i32) * D;
#pragma unroll
        for (int s = 0; s < DS; s++) kfr[s] = *reinterpret_cast<const vec8*>(kp + (((2 * s) ^ kz) * 8));
        // (D = 256: the 64 registers of V fragments are fetched right before their product instead, or the block
        // would not fit a wave's registers)
        if constexpr (PASS != kFwdLse && D < 192) {
#pragma unroll
          for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int db = 0; db < DB; db++) {
              const T* vp = Vs + (32 * nb + 16 * tt) * D;
              vfr[tt][db] = join8<vec8>(lds_read_tr(vp + toff[0][db]), lds_read_tr(vp + toff[1][db]));
            }
        }
      }
      // ---- S^T = K . Q^T for every query block of the wave ----
      float16_t sacc[RQ];
#pragma unroll
      for (int a = 0; a < RQ; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[a][r] = 0.f;
#pragma unroll
      for (int s = 0; s < DS; s++)
#pragma unroll
        for (int a = 0; a < RQ; a++) sacc[a] = Frag<T>::mfma(kfr[s], qf[a][s], sacc[a]);

      // Exponents are taken relative to a per-row reference value (m_run) that is NOT a running maximum: it stays
      // where it is until the guard below finds that a block's exponentials have left the safe range.  That saves
      // the max tree, the lane-half exchange and a branch per block.
#pragma unroll
      for (int a = 0; a < RQ; a++) {
        const int q_row = q_row0 + 32 * a;
        // ---- score_mod relative to the reference, tile mask where needed ----
        const float m_use = m_run[a];
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          float s0 = sacc[a][r], s1 = sacc[a][r + 1];
          if (ROUND_S) round_pair<T>(s0, s1);
          sacc[a][r] = sm.apply_sub(s0, acc_row(r), m_use);
          sacc[a][r + 1] = sm.apply_sub(s1, acc_row(r + 1), m_use);
        }
        if (cls == kBlockMixed) {
          // a real branch: every input of the mask arithmetic passes through this asm, so that
          // none of it can be hoisted into the unmasked path (it costs as much as the softmax)
          int q_opaque = q_row, kv_opaque = kv0 + nb * 32;
          asm volatile("" : "+v"(q_opaque), "+v"(kv_opaque));
          const Mask2 visible(p.mask, b, h, p.Lkv);
          mask_block_q<BITS, BITS>(sacc[a], p.mask, visible, q_opaque, kv_opaque, g, p.Lkv);
        }
      }
#pragma unroll
      for (int a = 0; a < RQ; a++) {
        // ---- exponentials; P rounded to the input dtype (not in the log-sum-exp pass, which sums in fp32 what
        // the dense path sums: the unrounded exponentials); l_blk = this lane's share of the block's row sum ----
        vec8 pf[2], pf_lo[2];
        float l_blk = 0.f;
        auto exponentials = [&](float shift) {
          l_blk = 0.f;
          if constexpr (PASS == kFwdLse) {
#pragma unroll
            for (int r = 0; r < 16; r++) l_blk += fast_exp2(sacc[a][r] - shift);
          } else if constexpr (PASS == kFwdHiLo) {
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
              typename Pair<T>::v2 hi[4], lo[4];
#pragma unroll
              for (int e = 0; e < 4; e++) {
                const float p0 = fast_exp2(sacc[a][8 * tt + 2 * e] - shift);
                const float p1 = fast_exp2(sacc[a][8 * tt + 2 * e + 1] - shift);
                split_pack<T>(p0, p1, hi[e], lo[e]);
                l_blk += p0 + p1;
              }
              pf[tt] = join_pairs<T>(hi[0], hi[1], hi[2], hi[3]);
              pf_lo[tt] = join_pairs<T>(lo[0], lo[1], lo[2], lo[3]);
            }
          } else {
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
              typename Pair<T>::v2 pr[4];
#pragma unroll
              for (int e = 0; e < 4; e++) {
                const float p0 = fast_exp2(sacc[a][8 * tt + 2 * e] - shift);
                const float p1 = fast_exp2(sacc[a][8 * tt + 2 * e + 1] - shift);
                pr[e] = Pair<T>::pack(p0, p1);
                if constexpr (PASS == kFwdOnePass) l_blk = Pair<T>::add_sum(pr[e], l_blk);
              }
              pf[tt] = join_pairs<T>(pr[0], pr[1], pr[2], pr[3]);
            }
          }
        };
        exponentials(0.f);
        if constexpr (PASS != kFwdNorm) {
          if (__any(l_blk > kPGuard || (l_run[a] == 0.f && l_blk < kPTiny))) {
            // Rare: the exponents of this block lie far from the reference -- so far above that P nears the top of
            // the 16-bit range, or, for a row that has accumulated nothing yet, so far below that P loses its
            // precision (or the block is masked out for the row: then nothing moves).  Move the row's reference to
            // the block's row maximum, rescale what the row has accumulated and redo the block's exponentials.
            float m_rel = xhalf_max(block_max(sacc[a]));
            asm volatile("" : "+v"(m_rel));  // keeps this rare path a real branch (never if-converted)
            const float l_prev = xhalf_sum(l_run[a]), l_row = xhalf_sum(l_blk);  // row values: both lane halves agree
            const bool fresh = l_prev == 0.f;                                      // nothing accumulated: nothing to rescale
            const bool move = m_rel > -INFINITY && ((l_row > kPGuard && m_rel > 0.f) || (fresh && l_row < 2.f * kPTiny));
            const float delta = move ? m_rel : 0.f;
            const float alpha = fresh ? 1.f : fast_exp2(-delta);
            m_run[a] += delta;
            l_run[a] *= alpha;
            if constexpr (PASS == kFwdOnePass || PASS == kFwdHiLo) {
#pragma unroll
              for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[a][db][r] *= alpha;
            }
            exponentials(delta);
          }
          l_run[a] += l_blk;
        }
        if constexpr (PASS != kFwdLse) {
          // ---- O^T += V^T . P^T ----
#pragma unroll
          for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int db = 0; db < DB; db++) {
              if constexpr (D >= 192) {
                const T* vp = Vs + (32 * nb + 16 * tt) * D;
                vfr[tt][db] = join8<vec8>(lds_read_tr(vp + toff[0][db]), lds_read_tr(vp + toff[1][db]));
              }
              oacc[a][db] = Frag<T>::mfma(vfr[tt][db], pf[tt], oacc[a][db]);
              if constexpr (PASS == kFwdHiLo) oacc[a][db] = Frag<T>::mfma(vfr[tt][db], pf_lo[tt], oacc[a][db]);
            }
        }
      }
      }  // block not entirely hidden
    }
    // this wave's share of the next tile has landed; after the barrier everyone's has
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  for (int it = it0; it < it1; it += 2) {
    tile_step(StageC<0>{}, it);
    if (it + 1 < it1) tile_step(StageC<1>{}, it + 1);
  }

  // ---- epilogue ----
#pragma unroll
  for (int a = 0; a < RQ; a++) {
    const int q_row = q_row0 + 32 * a;
    const float l_tot = PASS == kFwdNorm ? 1.f : xhalf_sum(l_run[a]);
    if (nsplit > 1) {
      // partial result of this share; a row that saw nothing here must not hold the merge's reference up: m = -inf
      if (q_row < p.Lq) {
        const int64_t at = ((int64_t)split * p.B * p.Hq + (int64_t)b * p.Hq + h) * p.Lq + q_row;
        if (g == 0) {
          ml_part[at * 2] = PASS == kFwdNorm ? 0.f : (l_tot > 0.f ? m_run[a] : -INFINITY);
          ml_part[at * 2 + 1] = PASS == kFwdNorm ? (split == 0 ? 1.f : 0.f) : l_tot;
        }
        if constexpr (PASS != kFwdLse) {
          float* op = o_part + at * D + 4 * g;
#pragma unroll
          for (int db = 0; db < DB; db++)
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
              float4_t acc4;
#pragma unroll
              for (int e = 0; e < 4; e++) acc4[e] = oacc[a][db][4 * rr + e];
              *reinterpret_cast<float4_t*>(op + 32 * db + 8 * rr) = acc4;
            }
        }
      }
      continue;
    }
    const float inv = PASS == kFwdNorm ? 1.f : (l_tot > 0.f ? 1.f / l_tot : 0.f);  // kFwdNorm: P came normalised
    if (q_row < p.Lq) {
      if constexpr (PASS != kFwdLse) {
        T* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)q_row * p.o_stride[2] + 4 * g;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int rr = 0; rr < 4; rr++) {
            union { T e[4]; uint2 u; } pk;
#pragma unroll
            for (int e = 0; e < 4; e++) pk.e[e] = (T)(oacc[a][db][4 * rr + e] * inv);
            *reinterpret_cast<uint2*>(op + 32 * db + 8 * rr) = pk.u;
          }
      }
      if (PASS != kFwdNorm && lse2 && g == 0)
        lse2[((int64_t)b * p.Hq + h) * p.Lq + q_row] = l_tot > 0.f ? m_run[a] + log2f(l_tot) : -INFINITY;
    }
  }
}

// ---------------------------------------------------------------------------
// D = 64: software-pipelined variant.  A wave owns two blocks of 32 query rows
// and walks "units" (32-key step, query block).  The instruction stream of a
// unit pairs every group of matrix instructions with independent vector work,
// so that the matrix pipe and the vector ALU of a SIMD run at the same time
// even when the waves of a workgroup march in lockstep:
//   region A: scale / score_mod of S(u)            ||  S^T = K.Q^T of unit u+1
//   (tile mask if needed)
//   region B: exponentials, rounding, row sum      ||  O^T += V^T.P^T of unit u-1
//   (guard: rare move of the row's reference value with a rescale of the accumulator)
// Every matrix result is first read at least half a unit after it was issued.
// Unit u-1 and unit u+1 belong to the wave's other query block, so a rescale in
// unit u never touches an accumulator that a matrix instruction is writing.
// KV tiles go through three LDS stages with one workgroup barrier per tile: a
// stage is refilled only after a barrier that follows its last fragment read.
// Tiles are fetched global -> LDS directly (no staging registers, no LDS stores),
// one tile ahead of the one being read.
// ---------------------------------------------------------------------------
// TAIL: the key length is not a multiple of the tile; that instantiation masks the keys past the end in the last
// tile.  The other one contains no mask code at all.
template <typename T, int KIND, bool ROUND_S, bool TAIL>
__global__ __launch_bounds__(256, 2) void fwd_pipe_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                           const T* __restrict__ k, const T* __restrict__ v,
                                                           T* __restrict__ o, float* __restrict__ lse2) {
  typedef typename Frag<T>::vec8 vec8;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  constexpr int D = 64, RQ = 2, BM = kPipeBM, BN = kFwdBN;
  constexpr int DS = D / 16, DB = D / 32;
  // KV tiles land in LDS straight from global memory (global_load_lds, 16 bytes per lane, a wave
  // instruction fills 8 rows of 128 bytes), so rows are unpadded; the 16-byte chunk c of row r is
  // kept at chunk position c ^ lds_swz(r), which makes both the row-fragment reads and the
  // transposing reads conflict-free.  The lane that fills position (r, pos) therefore fetches
  // chunk pos ^ lds_swz(r) of that row.
  constexpr int kTileElems = BN * D;  // 8 KB per tile
  // each stage is a variable of its own and every access names its stage at compile time (the tile loop is
  // unrolled by three): only then can the compiler tell that a read of one stage need not wait for the fetch
  // into another
  __shared__ __align__(16) T Ksm0[kTileElems];
  __shared__ __align__(16) T Ksm1[kTileElems];
  __shared__ __align__(16) T Ksm2[kTileElems];
  __shared__ __align__(16) T Vsm0[kTileElems];
  __shared__ __align__(16) T Vsm1[kTileElems];
  __shared__ __align__(16) T Vsm2[kTileElems];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5, i16 = lane & 15;
  const int nqt = (p.Lq + BM - 1) / BM;
  int rank, bh;
  xcd_tile_map(blockIdx.x, nqt, p.Hq * p.B, rank, bh);
  const int qt = nqt - 1 - rank;
  const int h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);
  const int q_row0 = qt * BM + w * (32 * RQ) + i32;

  vec8 qf[RQ][DS];
#pragma unroll
  for (int a = 0; a < RQ; a++) {
    const int q_ld = min(q_row0 + 32 * a, p.Lq - 1);
    const T* qp = q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)q_ld * p.q_stride[2] + 8 * g;
#pragma unroll
    for (int s = 0; s < DS; s++) qf[a][s] = *reinterpret_cast<const vec8*>(qp + 16 * s);
  }

  // every key tile is visited and nothing is masked but (TAIL) the keys past the end: this kernel is
  // launched for problems without tile lists and with a mask that hides nothing (mask code in the same
  // function costs the unmasked path 3 %, hence the two instantiations)
  const int nt = TAIL ? (p.Lkv + BN - 1) / BN : p.Lkv / BN;
  auto tile_at = [&](int it) -> int { return it; };

  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  const int64_t ks2 = p.k_stride[2], vs2 = p.v_stride[2];

  // ---- tile fetch: wave w fills rows [16w, 16w + 16) of the K and the V tile, 8 rows per instruction ----
  const int fill_row = lane >> 3;                         // row inside the 8-row group
  // the per-lane part of a fetch address (row among the wave's 16, swizzled chunk) is the same for every tile:
  // kept as byte offsets from the wave's first row of the tile, whose address is wave-uniform
  const int wu = __builtin_amdgcn_readfirstlane(w);
  uint32_t kfo[2], vfo[2];
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int row = 8 * j + fill_row;
    const int fill_chunk = (lane & 7) ^ lds_swz<D>(row);  // logical chunk this lane fetches
    kfo[j] = (uint32_t)((row * ks2 + fill_chunk * 8) * (int64_t)sizeof(T));
    vfo[j] = (uint32_t)((row * vs2 + fill_chunk * 8) * (int64_t)sizeof(T));
  }
  auto issue_tile = [&](auto stage, int kv0) {
    T* const Kst = stage_ptr(stage, Ksm0, Ksm1, Ksm2);
    T* const Vst = stage_ptr(stage, Vsm0, Vsm1, Vsm2);
    const int lim = p.Lkv - 1 - kv0;
    if (!TAIL || lim >= BN - 1) {
      const char* kt = reinterpret_cast<const char*>(kbase + (int64_t)(kv0 + 16 * wu) * ks2);
      const char* vt = reinterpret_cast<const char*>(vbase + (int64_t)(kv0 + 16 * wu) * vs2);
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int r0 = 16 * wu + 8 * j;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kt + kfo[j]),
                                         (__attribute__((address_space(3))) void*)(Kst + r0 * D), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vt + vfo[j]),
                                         (__attribute__((address_space(3))) void*)(Vst + r0 * D), 16, 0, 0);
      }
    } else {
      // the last tile of a ragged length: rows past the end are clamped (finite filler, masked out below)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int r0 = 16 * wu + 8 * j;
        const int fill_chunk = (lane & 7) ^ lds_swz<D>(8 * j + fill_row);
        const int row = min(r0 + fill_row, lim);
        const T* kg = kbase + (int64_t)(kv0 + row) * ks2 + fill_chunk * 8;
        const T* vg = vbase + (int64_t)(kv0 + row) * vs2 + fill_chunk * 8;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)kg,
                                         (__attribute__((address_space(3))) void*)(Kst + r0 * D), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vg,
                                         (__attribute__((address_space(3))) void*)(Vst + r0 * D), 16, 0, 0);
      }
    }
  };
  // ---- fragment reads ----
  vec8 kfr[DS], vfr[2][DB], pf[2];
  int koff[DS];  // element offsets of this lane's K row fragments inside a 32-row block
#pragma unroll
  for (int s = 0; s < DS; s++) koff[s] = i32 * D + (((2 * s + g) ^ lds_swz<D>(i32)) * 8);
  auto read_k = [&](const T* Ks, int nb) {
#pragma unroll
    for (int s = 0; s < DS; s++) kfr[s] = *reinterpret_cast<const vec8*>(Ks + nb * 32 * D + koff[s]);
  };
  // transposing reads: lane points at 4 elements of row 4g + (i16 >> 2) + 8e (+16tt), logical column
  // 32db + 16h + 4(i16 & 3)
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
  auto read_v = [&](const T* Vs, int nb) {
#pragma unroll
    for (int tt = 0; tt < 2; tt++)
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const T* vp = Vs + (32 * nb + 16 * tt) * D;
        vfr[tt][db] = join8<vec8>(lds_read_tr(vp + voff[0][db]), lds_read_tr(vp + voff[1][db]));
      }
  };

  Score2<KIND> sm;
  sm.init(p.score, p.scale, h, b, p.Lq, p.Lkv);

  float16_t oacc[RQ][DB], s_cur;
  float m_run[RQ], l_run[RQ];
#pragma unroll
  for (int a = 0; a < RQ; a++) {
    m_run[a] = 0.f;  // reference value of the row's exponents; moved only by the guard below
    l_run[a] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[a][db][r] = 0.f;
  }
  // nothing is pending before the first unit: P = 0 against V = 0
#pragma unroll
  for (int tt = 0; tt < 2; tt++) {
#pragma unroll
    for (int e = 0; e < 8; e++) pf[tt][e] = (T)0.f;
#pragma unroll
    for (int db = 0; db < DB; db++) vfr[tt][db] = pf[tt];
  }

  // the reference value of a row's exponents stays where the row's first visible block put it until a lane's share of
  // a block's row sum exceeds this (fp16 tops out at 65504; sums are kept in fp32)
  constexpr float kPGuard = 32768.f, kPTiny = 1.f / 64.f;
  int t_cur = nt > 0 ? tile_at(0) : 0;
  int t_nxt = nt > 1 ? tile_at(1) : 0;   // tile it + 1
  int t_nx2 = nt > 2 ? tile_at(2) : 0;   // tile it + 2
  if (nt > 0) issue_tile(StageC<0>{}, t_cur * BN);
  if (nt > 1) issue_tile(StageC<1>{}, t_nxt * BN);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  // S of the first unit
  read_k(Ksm0, 0);
#pragma unroll
  for (int r = 0; r < 16; r++) s_cur[r] = 0.f;
#pragma unroll
  for (int s = 0; s < DS; s++) s_cur = Frag<T>::mfma(kfr[s], qf[0][s], s_cur);

  const int slot = blockIdx.x >= (gridDim.x >> 1) ? 1 : 0;  // second half of the grid = second workgroup of a compute unit
  // one tile out of the stage named by `stage` (= it % 3)
  auto tile_step = [&](auto stage, int it) {
    constexpr int ST = decltype(stage)::value;
    // Two workgroups share a compute unit and the instruction arbiter favours the older wave,
    // which leaves the younger one behind until it runs alone at the end.  All workgroups have
    // the same amount of work here, so trading the wave priority between them every tile keeps
    // both advancing at the same pace.
    if ((it ^ slot) & 1) __builtin_amdgcn_s_setprio(2); else __builtin_amdgcn_s_setprio(0);
    const int kv0 = t_cur * BN;
    const T* const Ks = stage_ptr(stage, Ksm0, Ksm1, Ksm2);
    const T* const Vs = stage_ptr(stage, Vsm0, Vsm1, Vsm2);
    const T* const Kn = stage_ptr(StageC<(ST + 1) % 3>{}, Ksm0, Ksm1, Ksm2);
    const StageC<(ST + 2) % 3> st_p;  // stage of the previous tile = stage of tile it + 2
    const int kv_nx2 = t_nx2 * BN;
    t_cur = t_nxt;
    t_nxt = t_nx2;
    if (it + 3 < nt) t_nx2 = tile_at(it + 3);
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
#pragma unroll
      for (int a = 0; a < RQ; a++) {
        const int q_row = q_row0 + 32 * a;
        if (nb == 1 && a == 0) {
          // this wave's share of tile it + 1 has landed; after the barrier everyone's has, and
          // the previous tile's stage (last read before this barrier) can take tile it + 2
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __syncthreads();
          if (it + 2 < nt) issue_tile(st_p, kv_nx2);
        }
        if (a == 1) read_v(Vs, nb);              // V columns of this step, first used in region B

        // ---- region A: S^T of the next unit || score_mod relative to the row's reference value ----
        float16_t s_nxt;
#pragma unroll
        for (int r = 0; r < 16; r++) s_nxt[r] = 0.f;
#pragma unroll
        for (int s = 0; s < DS; s++) s_nxt = Frag<T>::mfma(kfr[s], qf[1 - a][s], s_nxt);
        const float m_use = m_run[a];
        sm.tile(q_row, kv0 + nb * 32 + 4 * g);
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          float s0 = s_cur[r], s1 = s_cur[r + 1];
          if (ROUND_S) round_pair<T>(s0, s1);
          s_cur[r] = sm.apply_sub(s0, acc_row(r), m_use);
          s_cur[r + 1] = sm.apply_sub(s1, acc_row(r + 1), m_use);
        }
#pragma unroll
        for (int i = 0; i < DS; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // one matrix instruction
          if (a == 1) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // two LDS reads (V columns)
          __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);             // six vector instructions
        }
        if constexpr (TAIL) {
          if (kv0 + BN > p.Lkv) {
            // a real branch whose inputs pass through the asm, so that none of the mask
            // arithmetic can be hoisted into the path of the complete tiles
            int q_opaque = q_row, kv_opaque = kv0 + nb * 32;
            asm volatile("" : "+v"(q_opaque), "+v"(kv_opaque));
            const int cls = band_block_class(p.mask, __builtin_amdgcn_readfirstlane(q_opaque - i32),
                                             __builtin_amdgcn_readfirstlane(kv_opaque), 0x7fffffff, p.Lkv);
            if (cls == kBlockNone) fill_masked(s_cur);
            else if (cls == kBlockMixed) {
              const Mask2 visible(p.mask, b, h, p.Lkv);
              mask_block_q<false>(s_cur, p.mask, visible, q_opaque, kv_opaque, g, p.Lkv);
            }
          }
        }
        // ---- region B: O^T += V^T.P^T of the previous unit || exponentials, rounding, row sum ----
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
          for (int db = 0; db < DB; db++) oacc[1 - a][db] = Frag<T>::mfma(vfr[tt][db], pf[tt], oacc[1 - a][db]);
        vec8 pn[2];
        float l_blk = 0.f;  // this lane's share of the block's row sum
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
          typename Pair<T>::v2 pr[4];
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float p0 = fast_exp2(s_cur[8 * tt + 2 * e]);
            const float p1 = fast_exp2(s_cur[8 * tt + 2 * e + 1]);
            pr[e] = Pair<T>::pack(p0, p1);
            l_blk = Pair<T>::add_sum(pr[e], l_blk);
          }
          pn[tt] = join_pairs<T>(pr[0], pr[1], pr[2], pr[3]);
        }
        if (a == 0) read_k(nb == 0 ? Ks : Kn, nb == 0 ? 1 : 0);  // K rows of the next step (kfr is free after region A)
#pragma unroll
        for (int i = 0; i < 2 * DB; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // one matrix instruction
          if (a == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read (K rows)
          __builtin_amdgcn_sched_group_barrier(0x400, 4, 0);             // four exponentials
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);             // rounding and row sum of the previous four
        }
        if (__any(l_blk > kPGuard || (l_run[a] == 0.f && l_blk < kPTiny))) {
          // Rare: the exponents of this block lie far from the reference -- so far above that P nears the top of the
          // 16-bit range, or, for a row that has accumulated nothing yet, so far below that P loses its precision.
          // Move the row's reference to the block's row maximum, rescale what the row has accumulated and redo the
          // block's exponentials (s_cur still holds the exponents; the block's P has not been multiplied into V yet).
          float m_rel = xhalf_max(block_max(s_cur));
          asm volatile("" : "+v"(m_rel));
          const float l_prev = xhalf_sum(l_run[a]), l_row = xhalf_sum(l_blk);   // row values: both lane halves agree
          const bool fresh = l_prev == 0.f;                                       // nothing accumulated: nothing to rescale
          const bool move = m_rel > -INFINITY && ((l_row > kPGuard && m_rel > 0.f) || (fresh && l_row < 2.f * kPTiny));
          const float delta = move ? m_rel : 0.f;
          const float alpha = fresh ? 1.f : fast_exp2(-delta);
          m_run[a] += delta;
          l_run[a] *= alpha;
#pragma unroll
          for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[a][db][r] *= alpha;
          l_blk = 0.f;
#pragma unroll
          for (int tt = 0; tt < 2; tt++) {
            typename Pair<T>::v2 pr[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
              pr[e] = Pair<T>::pack(fast_exp2(s_cur[8 * tt + 2 * e] - delta), fast_exp2(s_cur[8 * tt + 2 * e + 1] - delta));
              l_blk = Pair<T>::add_sum(pr[e], l_blk);
            }
            pn[tt] = join_pairs<T>(pr[0], pr[1], pr[2], pr[3]);
          }
        }
        l_run[a] += l_blk;
        pf[0] = pn[0];
        pf[1] = pn[1];
        s_cur = s_nxt;
      }
    }
  };
  for (int it = 0; it < nt; it += 3) {
    tile_step(StageC<0>{}, it);
    if (it + 1 < nt) {  // nested: no path may reach a stage's step without the step before it
      tile_step(StageC<1>{}, it + 1);
      if (it + 2 < nt) tile_step(StageC<2>{}, it + 2);
    }
  }
  __builtin_amdgcn_s_setprio(0);
  // the last unit's P is still pending
#pragma unroll
  for (int tt = 0; tt < 2; tt++)
#pragma unroll
    for (int db = 0; db < DB; db++) oacc[1][db] = Frag<T>::mfma(vfr[tt][db], pf[tt], oacc[1][db]);

  // ---- epilogue ----
#pragma unroll
  for (int a = 0; a < RQ; a++) {
    const int q_row = q_row0 + 32 * a;
    const float l_tot = xhalf_sum(l_run[a]);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (q_row < p.Lq) {
      T* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)q_row * p.o_stride[2] + 4 * g;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
          union { T e[4]; uint2 u; } pk;
#pragma unroll
          for (int e = 0; e < 4; e++) pk.e[e] = (T)(oacc[a][db][4 * rr + e] * inv);
          *reinterpret_cast<uint2*>(op + 32 * db + 8 * rr) = pk.u;
        }
      if (lse2 && g == 0) lse2[((int64_t)b * p.Hq + h) * p.Lq + q_row] = l_tot > 0.f ? m_run[a] + log2f(l_tot) : -INFINITY;
    }
  }
}

struct FwdArgs {
  const void *q, *k, *v;
  void* o;
  float* lse2;
  hipStream_t s;
  // forward over split key ranges: shares per query tile (1 = none) and where their partial (O, m, l) go
  int splits;
  float *o_part, *ml_part;
};

// one pass of the list-driven kernel; over split key ranges it is followed by the merge of the partials (one wave per
// row), which writes `o` (unless null) and `lse2` (unless null)
template <typename T, int D, int KIND, bool RS, bool BITS, int PASS>
static void launch_list_kernel(const FlexAttnParams& p, const FwdArgs& a) {
  const int splits = a.splits > 1 ? a.splits : 1;
  dim3 grid((p.Lq + kFwdBM - 1) / kFwdBM * p.Hq * p.B, splits);
  hipLaunchKernelGGL((fwd_mfma_kernel<T, D, KIND, RS, BITS, PASS>), grid, dim3(256), 0, a.s, p, (const T*)a.q, (const T*)a.k,
                     (const T*)a.v, (T*)a.o, a.lse2, a.o_part, a.ml_part);
  if (splits > 1) {
    const int64_t rows = (int64_t)p.B * p.Hq * p.Lq;
    hipLaunchKernelGGL((decode_combine_kernel<T, D>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, a.s, p, a.o_part, a.ml_part,
                       splits, PASS == kFwdLse ? (T*)nullptr : (T*)a.o, PASS == kFwdNorm ? (float*)nullptr : a.lse2);
  }
}

template <typename T, int KIND, bool RS, bool TAIL>
static void launch_pipe_kernel(const FlexAttnParams& p, const FwdArgs& a) {
  dim3 grid((p.Lq + kPipeBM - 1) / kPipeBM * p.Hq * p.B);
  hipLaunchKernelGGL((fwd_pipe_kernel<T, KIND, RS, TAIL>), grid, dim3(256), 0, a.s, p, (const T*)a.q, (const T*)a.k, (const T*)a.v,
                     (T*)a.o, a.lse2);
}

template <typename T, int D, int KIND>
static void launch_rs(const FlexAttnParams& p, const FwdArgs& a) {
  const bool bits = p.mask.kind == FLEX_MASK_BITS;
  if (p.flags & FLEX_UNROUNDED) {
    // "unrounded" numerics: no rounding of S, P carried as a high and a low part
    if (bits) launch_list_kernel<T, D, KIND, false, true, kFwdHiLo>(p, a);
    else launch_list_kernel<T, D, KIND, false, false, kFwdHiLo>(p, a);
    return;
  }
  if (p.flags & FLEX_PARITY) {
    // parity numerics: a log-sum-exp pass, then the pass that multiplies the normalised, rounded P into V
    // (a.lse2 is never null here: the caller substitutes workspace); S is always rounded through the input dtype
    if (bits) {
      launch_list_kernel<T, D, KIND, true, true, kFwdLse>(p, a);
      launch_list_kernel<T, D, KIND, true, true, kFwdNorm>(p, a);
    } else {
      launch_list_kernel<T, D, KIND, true, false, kFwdLse>(p, a);
      launch_list_kernel<T, D, KIND, true, false, kFwdNorm>(p, a);
    }
    return;
  }
  // D = 64 without tile lists or anything to mask (every workgroup has the same work): the pipelined
  // kernel with 256-row workgroups.  Otherwise the 128-row kernel: twice the workgroups, half the length of the
  // longest one, which is what bounds a causal-like schedule.
  // (a table-reading score_mod stalls on its loads where the pipelined kernel has no slack: 128-row kernel)
  if constexpr (KIND != FLEX_SCORE_AFFINE && KIND != kScoreAffineMul && D == 64) {
    if (!p.tiles.kv_num && mask_hides_nothing(p.mask) && a.splits <= 1) {
      const bool tail = p.Lkv % kFwdBN != 0, rs = (p.flags & FLEX_ROUND_S) != 0;
      if (rs && !tail) launch_pipe_kernel<T, KIND, true, false>(p, a);
      else if (rs) launch_pipe_kernel<T, KIND, true, true>(p, a);
      else if (!tail) launch_pipe_kernel<T, KIND, false, false>(p, a);
      else launch_pipe_kernel<T, KIND, false, true>(p, a);
      return;
    }
  }
  if (p.flags & FLEX_ROUND_S) {
    if (bits) launch_list_kernel<T, D, KIND, true, true, kFwdOnePass>(p, a);
    else launch_list_kernel<T, D, KIND, true, false, kFwdOnePass>(p, a);
  } else {
    if (bits) launch_list_kernel<T, D, KIND, false, true, kFwdOnePass>(p, a);
    else launch_list_kernel<T, D, KIND, false, false, kFwdOnePass>(p, a);
  }
}

template <typename T, int D>
static int launch_kind(const FlexAttnParams& p, const FwdArgs& a) {
  switch (p.score.kind) {
    case FLEX_SCORE_IDENTITY: launch_rs<T, D, FLEX_SCORE_IDENTITY>(p, a); return 0;
    case FLEX_SCORE_CHECKERBOARD: launch_rs<T, D, FLEX_SCORE_CHECKERBOARD>(p, a); return 0;
    case FLEX_SCORE_ALIBI: launch_rs<T, D, FLEX_SCORE_ALIBI>(p, a); return 0;
    case FLEX_SCORE_TANH_SOFTCAP: launch_rs<T, D, FLEX_SCORE_TANH_SOFTCAP>(p, a); return 0;
    case FLEX_SCORE_REL_BIAS: launch_rs<T, D, FLEX_SCORE_REL_BIAS>(p, a); return 0;
    case FLEX_SCORE_AFFINE:
      if (p.score.mul) launch_rs<T, D, kScoreAffineMul>(p, a);
      else launch_rs<T, D, FLEX_SCORE_AFFINE>(p, a);
      return 0;
  }
  return 1;
}

}  // namespace flex
