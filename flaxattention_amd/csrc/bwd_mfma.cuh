// Fused flash-attention backward for gfx950 (fp16 / bf16, D = Dv in {64, 128}).
//
// Takes the place of _preprocess_backward + mha_backward_kernel
// (flaxattention/kernel/attention.py:338-553) and of jax.grad through the dense
// path.  P is recomputed from the saved base-2 log-sum-exp.  Two kernels:
//
//  bwd_dq_kernel   one workgroup per 128 query rows, sweeping KV tiles of 128 (64 at D = 128;
//                  the entries of the 128-granular backward lists), fetched global -> LDS
//                  directly into two stages.  Transposed products keep one query
//                  row per lane, so lse and delta are per-lane scalars:
//                    S^T = K.Q^T,  dP^T = V.dO^T,  dS^T = P^T o (dP^T - delta) * g,
//                    dQ^T += K^T.dS^T.
//                  Also produces delta_i = sum_d O_id dO_id for the second kernel.
//  bwd_dkv_kernel  one workgroup per 128 key rows, sweeping query tiles of 128
//                  from the transposed tile lists.  Here a lane owns one key
//                  row: S = Q.K^T, dP = dO.V^T, dV^T += dO^T.P, dK^T += Q^T.dS.
//                  Four waves = four key blocks of 32 rows.  With GQA the
//                  workgroup loops over the query heads of its group.
#pragma once
#include "mfma_common.cuh"

namespace flex {

constexpr int kBM = 128;     // query tile (list granularity)
constexpr int kBN = 128;     // key tile staged per step by the dQ kernel at D = 64 (half of it at D = 128)
constexpr int kListBN = 128; // key granularity of the backward tile lists = key rows of a dK/dV workgroup

// MASKED = false: the caller guarantees that there is nothing to mask (no tile lists, a mask that hides nothing,
// key length a multiple of the tile); that instantiation carries no mask code, which is worth 2 % on its own.
//
// MODE selects the numerics:
//   kBwdFast    delta_i = sum_d O_id dO_id (computed here from the rounded O), dP kept in fp32
//   kBwdDelta   the row sweep of the parity numerics: no dQ; writes delta_i = sum_j P_ij round(dP_ij), which is what
//               differentiating the dense path gives (attention.py:104-105: the softmax is differentiated in fp32,
//               its cotangent dP = dO.V^T arrives rounded to the input dtype because that product is computed in it)
//   kBwdParity  dQ of the parity numerics: reads that delta, rounds dP through the input dtype before the
//               subtraction and applies the scale before dS is rounded
// p.d_lse2 (optional): the cotangent of the base-2 log-sum-exp output.  d lse / d X_ij = P_ij, so it joins the row
// term: dX = P o (dP - (delta - log2(e) d_lse2)).
//   kBwdDeltaRaw the row sweep of the "unrounded" numerics: delta_i = sum_j P_ij dP_ij with nothing rounded
//   kBwdHiLo     dQ of the "unrounded" numerics: reads that delta; dP stays in fp32 and dS goes into the product
//                as a high and a low part (two matrix instructions per fragment); launched with ROUND_S = false
enum { kBwdFast = 0, kBwdDelta = 1, kBwdParity = 2, kBwdDeltaRaw = 3, kBwdHiLo = 4 };
// keys the dQ kernel stages per step (the kernel and the launcher that picks its mask-free instantiation agree on it)
template <int D, int MODE> constexpr int dq_tile_keys() { return D >= 192 ? kBN / 2 : (D == 64 || MODE == kBwdFast) ? kBN : kBN / 2; }
// Registers: two waves per SIMD (256 registers each) everywhere but the fast-numerics kernel at D = 128, which then
// spills 31 - 59 registers and reloads them inside the tile loop (every reload is a vector memory load, and a wait for
// one is a wait for the tile fetch in flight as well); with one wave per SIMD and no spill it is 10 - 15 % faster
// ([4,16,4096,128] bf16: 1213 -> 1031 us dense, 603 -> 544 us causal).  The row sweep does not spill; the parity kernel
// (19 - 52 registers spilled) loses 22 % with one wave per SIMD and the high/low kernel gains nothing, so they keep two.
template <typename T, int D, int KIND, bool ROUND_S, bool MASKED, int MODE = kBwdFast>
__global__ __launch_bounds__(256, ((D == 128 && MODE == kBwdFast) || D >= 192) ? 1 : 2) void bwd_dq_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                      const T* __restrict__ k, const T* __restrict__ v,
                                                      const T* __restrict__ o, const float* __restrict__ lse2,
                                                      const T* __restrict__ d_o, T* __restrict__ dq,
                                                      float* __restrict__ delta_out) {
  typedef typename Frag<T>::vec8 vec8;
  // keys staged per step: 128 at D = 64, 64 at D = 128, so that two stages of K and V are 64 KB
  // either way and two workgroups (two waves per SIMD) share a compute unit; the fast-numerics kernel at
  // D = 128 runs one wave per SIMD (see above), has the 128 KB for 128-key tiles and is 3 - 6 % faster with them
  constexpr int BM = kBM, BN = dq_tile_keys<D, MODE>();
  constexpr int DS = D / 16, DB = D / 32, CPR = D / 8;
  // a wave fills BN / 4 rows of a tile: (BN / 4) * CPR chunks, 64 per fetch instruction, laid down one after the
  // other (at D = 192 an instruction ends in the middle of a row); the fetch pattern repeats every 16 rows
  constexpr int NI = (BN / 4) * CPR / 64;   // fetch instructions per wave, tile and tensor
  static_assert(((BN / 4) * CPR) % 64 == 0 && (16 * CPR) % 64 == 0, "whole fetch instructions per swizzle period");
  // two LDS stages, filled straight from global memory (no staging registers, unpadded swizzled
  // rows): while one tile is consumed the next one lands, one workgroup barrier per tile.  Each stage is a
  // variable of its own and every access names its stage at compile time (the tile loop is unrolled by two):
  // only then can the compiler tell that a read of one stage need not wait for the fetch into the other.
  __shared__ __align__(16) T Ksm0[BN * D];
  __shared__ __align__(16) T Ksm1[BN * D];
  __shared__ __align__(16) T Vsm0[BN * D];
  __shared__ __align__(16) T Vsm1[BN * D];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5, i16 = lane & 15;
  const int nqt = (p.Lq + BM - 1) / BM;
  int rank, bh;
  xcd_tile_map(blockIdx.x, nqt, p.Hq * p.B, rank, bh);
  const int qt = nqt - 1 - rank;
  const int h = bh % p.Hq, b = bh / p.Hq, hk = h / (p.Hq / p.Hkv);
  const int q_row = qt * BM + w * 32 + i32;
  const int q_ld = min(q_row, p.Lq - 1);
  const int64_t row_id = ((int64_t)b * p.Hq + h) * p.Lq + q_ld;

  vec8 qf[DS], dof[DS];
  float dpart = 0.f;
  {
    const T* qp = q + b * p.q_stride[0] + h * p.q_stride[1] + (int64_t)q_ld * p.q_stride[2] + 8 * g;
    const T* op = o + b * p.o_stride[0] + h * p.o_stride[1] + (int64_t)q_ld * p.o_stride[2] + 8 * g;
    const T* dop = d_o + row_id * D + 8 * g;  // dO is contiguous [B,Hq,Lq,D]
#pragma unroll
    for (int s = 0; s < DS; s++) {
      qf[s] = *reinterpret_cast<const vec8*>(qp + 16 * s);
      dof[s] = *reinterpret_cast<const vec8*>(dop + 16 * s);
      if constexpr (MODE == kBwdFast) {
        vec8 of = *reinterpret_cast<const vec8*>(op + 16 * s);
#pragma unroll
        for (int e = 0; e < 8; e++) dpart = fmaf((float)of[e], (float)dof[s][e], dpart);
      }
    }
  }
  float delta = 0.f;
  if constexpr (MODE == kBwdFast) {
    delta = xhalf_sum(dpart);
    if (p.d_lse2) delta -= kLog2e * p.d_lse2[row_id];
    if (q_row < p.Lq && g == 0) delta_out[row_id] = delta;
  } else if constexpr (MODE == kBwdParity || MODE == kBwdHiLo) {
    delta = delta_out[row_id];  // written by the row-sweep launch that precedes this one on the stream
  }
  float drow = 0.f;  // kBwdDelta: this lane's share of sum_j P_ij round(dP_ij)
  float lse = lse2[row_id];
  if (lse == -INFINITY) lse = INFINITY;  // row without visible keys: P = 0

  const FlexTileLists& tl = p.tiles_bwd;
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
  // a list entry covers `sub` staged tiles of BN keys (the lists are kListBN-granular);
  // the schedule below runs over (entry, part) pairs flattened into one index
  const int sub = full_idx ? tl.kv_block / BN : 1;
  const int nt = (n_full + n_part) * sub;
  const int n_full_t = n_full * sub;
  auto tile_at = [&](int it) -> int {
    if (!full_idx) return it;
    const int e = sub == 2 ? (it >> 1) : it, part = sub == 2 ? (it & 1) : 0;
    return uniform_ld(e < n_full ? full_idx + e : part_idx + (e - n_full)) * sub + part;
  };

  const T* kbase = k + b * p.k_stride[0] + hk * p.k_stride[1];
  const T* vbase = v + b * p.v_stride[0] + hk * p.v_stride[1];
  const int64_t ks2 = p.k_stride[2], vs2 = p.v_stride[2];
  // tile fetch: wave w fills rows [32w, 32w + 32) of the K and the V tile, RPI rows per instruction;
  // the lane that fills position (r, pos) fetches chunk pos ^ lds_swz(r) of that row
  // the per-lane part of a fetch address (row among the 16 of a swizzle period, swizzled chunk) is the same for
  // every tile: kept as byte offsets from a wave-uniform row address
  const int wu = __builtin_amdgcn_readfirstlane(w);
  constexpr int NP = 16 * CPR / 64;  // fetch instructions per swizzle period
  uint32_t koff[NP], voff[NP];
#pragma unroll
  for (int jp = 0; jp < NP; jp++) {
    const int c = 64 * jp + lane, row = c / CPR;
    const int chunk = (c % CPR) ^ lds_swz<D>(row);  // the wave's first row is a multiple of 16
    koff[jp] = (uint32_t)((row * ks2 + chunk * 8) * (int64_t)sizeof(T));
    voff[jp] = (uint32_t)((row * vs2 + chunk * 8) * (int64_t)sizeof(T));
  }
  auto issue_tile = [&](auto stage, int kv0_in) {
    T* const Kst = stage_ptr(stage, Ksm0, Ksm1);
    T* const Vst = stage_ptr(stage, Vsm0, Vsm1);
    const int kv0 = __builtin_amdgcn_readfirstlane(kv0_in);
    const int lim = p.Lkv - 1 - kv0;
    if (lim >= BN - 1) {
#pragma unroll
      for (int j = 0; j < NI; j++) {
        const int r0 = (BN / 4) * wu + 16 * (j / NP);   // first row of the swizzle period instruction j belongs to
        const char* kt = reinterpret_cast<const char*>(kbase + (int64_t)(kv0 + r0) * ks2);
        const char* vt = reinterpret_cast<const char*>(vbase + (int64_t)(kv0 + r0) * vs2);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kt + koff[j % NP]),
                                         (__attribute__((address_space(3))) void*)(Kst + r0 * D + 512 * (j % NP)), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vt + voff[j % NP]),
                                         (__attribute__((address_space(3))) void*)(Vst + r0 * D + 512 * (j % NP)), 16, 0, 0);
      }
    } else {
      // the last tile of a ragged length: rows past the end are clamped (finite filler, masked out below)
#pragma unroll
      for (int j = 0; j < NI; j++) {
        const int c = 64 * j + lane, rw = c / CPR;      // row inside the wave's share, and its chunk position
        const int chunk = (c % CPR) ^ lds_swz<D>(rw);
        const int row = min((BN / 4) * wu + rw, lim);
        const T* kg = kbase + (int64_t)(kv0 + row) * ks2 + chunk * 8;
        const T* vg = vbase + (int64_t)(kv0 + row) * vs2 + chunk * 8;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)kg,
                                         (__attribute__((address_space(3))) void*)(Kst + (BN / 4) * wu * D + 512 * j), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vg,
                                         (__attribute__((address_space(3))) void*)(Vst + (BN / 4) * wu * D + 512 * j), 16, 0, 0);
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
  Mask2 visible(p.mask, b, h, p.Lkv);
  float16_t dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) dqacc[db][r] = 0.f;

  int t_cur = nt > 0 ? tile_at(0) : 0;
  int t_nxt = nt > 1 ? tile_at(1) : 0;
  if (nt > 0) issue_tile(StageC<0>{}, t_cur * BN);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  // fast numerics: dP starts at -delta, so the accumulator comes out as dP - delta; the parity numerics
  // round dP first
  const float neg_delta = (MODE == kBwdFast || MODE == kBwdHiLo) ? -delta : 0.f;
  // one tile out of the stage named by `stage` (= it & 1)
  auto tile_step = [&](auto stage, int it) {
    constexpr int ST = decltype(stage)::value;
    const int kv0 = t_cur * BN;
    const bool masked = MASKED && ((it >= n_full_t) || (kv0 + BN > p.Lkv));
    const T* const Ks = stage_ptr(stage, Ksm0, Ksm1);
    const T* const Vs = stage_ptr(stage, Vsm0, Vsm1);
    if (it + 1 < nt) {
      // the other stage was last read before the previous barrier: the next tile lands there
      // while this one is consumed; the tile index after that is looked up a tile ahead
      issue_tile(StageC<1 - ST>{}, t_nxt * BN);
      t_cur = t_nxt;
      if (it + 2 < nt) t_nxt = tile_at(it + 2);
    }

    // one 32-key block at a time (S, dP, softmax, dQ): half the accumulator registers of
    // doing both blocks side by side
#pragma unroll
    for (int nb = 0; nb < BN / 32; nb++) {
      // most 32x32 blocks of a partial tile are entirely visible (no mask evaluation) or
      // entirely hidden (nothing to do)
      int cls = kBlockAll;
      if (masked) {
        cls = block_class(p.mask, visible, __builtin_amdgcn_readfirstlane(q_row - i32), kv0 + nb * 32, 0x7fffffff, p.Lkv);
        if (cls == kBlockNone) continue;
      }
      sm.tile(q_row, kv0 + nb * 32 + 4 * g);  // a table-reading score_mod fetches its entries under the products
      float16_t sacc, dpacc, gacc;
#pragma unroll
      for (int r = 0; r < 16; r++) { sacc[r] = 0.f; dpacc[r] = neg_delta; }
      const T* kp = Ks + (nb * 32 + i32) * D;
      const T* vp = Vs + (nb * 32 + i32) * D;
#pragma unroll
      for (int s = 0; s < DS; s++) {
        sacc = Frag<T>::mfma(*reinterpret_cast<const vec8*>(kp + (((2 * s) ^ kz) * 8)), qf[s], sacc);
        dpacc = Frag<T>::mfma(*reinterpret_cast<const vec8*>(vp + (((2 * s) ^ kz) * 8)), dof[s], dpacc);
      }
      // x = log2(e) * score_mod(scale * s) - lse  (P = 2^x); g = d score_mod / d score kept for later
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float s0 = sacc[r], s1 = sacc[r + 1];
        if (ROUND_S) round_pair<T>(s0, s1);
        sacc[r] = sm.apply_sub(s0, acc_row(r), lse);
        sacc[r + 1] = sm.apply_sub(s1, acc_row(r + 1), lse);
        if (!Score2<KIND>::kGradOne) {
          gacc[r] = sm.grad(s0, acc_row(r));
          gacc[r + 1] = sm.grad(s1, acc_row(r + 1));
        }
      }
      if (cls == kBlockMixed) {
        // a real branch whose inputs pass through the asm, so that none of the mask
        // arithmetic can be hoisted into the unmasked path
        int q_opaque = q_row, kv_opaque = kv0 + nb * 32;
        asm volatile("" : "+v"(q_opaque), "+v"(kv_opaque));
        mask_block_q(sacc, p.mask, visible, q_opaque, kv_opaque, g, p.Lkv);
      }
      if constexpr (MODE == kBwdDelta || MODE == kBwdDeltaRaw) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          float a0 = dpacc[r], a1 = dpacc[r + 1];
          if constexpr (MODE == kBwdDelta) round_pair<T>(a0, a1);
          drow = fmaf(fast_exp2(sacc[r]), a0, drow);
          drow = fmaf(fast_exp2(sacc[r + 1]), a1, drow);
        }
        continue;
      }
      vec8 dsf[2], dsf_lo[2];
#pragma unroll
      for (int tt = 0; tt < 2; tt++) {
        typename Pair<T>::v2 pr[4], pl[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 8 * tt + 2 * e;
          float d0, d1;
          if constexpr (MODE == kBwdParity) {
            float a0 = dpacc[r], a1 = dpacc[r + 1];
            round_pair<T>(a0, a1);
            d0 = fast_exp2(sacc[r]) * (a0 - delta);
            d1 = fast_exp2(sacc[r + 1]) * (a1 - delta);
            if (!Score2<KIND>::kGradOne) { d0 *= gacc[r]; d1 *= gacc[r + 1]; }
            d0 *= p.scale;  // before dS is rounded, as the dense path has it
            d1 *= p.scale;
          } else {
            d0 = fast_exp2(sacc[r]) * dpacc[r];
            d1 = fast_exp2(sacc[r + 1]) * dpacc[r + 1];
            if (!Score2<KIND>::kGradOne) { d0 *= gacc[r]; d1 *= gacc[r + 1]; }
          }
          if constexpr (MODE == kBwdHiLo) split_pack<T>(d0, d1, pr[e], pl[e]);
          else pr[e] = Pair<T>::pack(d0, d1);
        }
        dsf[tt] = join_pairs<T>(pr[0], pr[1], pr[2], pr[3]);
        if constexpr (MODE == kBwdHiLo) dsf_lo[tt] = join_pairs<T>(pl[0], pl[1], pl[2], pl[3]);
      }
#pragma unroll
      for (int tt = 0; tt < 2; tt++) {
#pragma unroll
        for (int db = 0; db < DB; db++) {
          const T* ktp = Ks + (32 * nb + 16 * tt) * D;
          short4_t lo = lds_read_tr(ktp + toff[0][db]);
          short4_t hi = lds_read_tr(ktp + toff[1][db]);
          const vec8 kt = join8<vec8>(lo, hi);
          dqacc[db] = Frag<T>::mfma(kt, dsf[tt], dqacc[db]);
          if constexpr (MODE == kBwdHiLo) dqacc[db] = Frag<T>::mfma(kt, dsf_lo[tt], dqacc[db]);
        }
      }
    }
    // this wave's share of the next tile has landed; after the barrier everyone's has
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  for (int it = 0; it < nt; it += 2) {
    tile_step(StageC<0>{}, it);
    if (it + 1 < nt) tile_step(StageC<1>{}, it + 1);
  }

  if constexpr (MODE == kBwdDelta || MODE == kBwdDeltaRaw) {
    drow = xhalf_sum(drow);
    if (p.d_lse2) drow -= kLog2e * p.d_lse2[row_id];
    if (q_row < p.Lq && g == 0) delta_out[row_id] = drow;
    return;
  }
  // fast numerics: the scale factor of dS = P o (dP - delta) o g * scale is applied once here
  const float out_scale = MODE == kBwdParity ? 1.f : p.scale;
  if (q_row < p.Lq) {
    T* op = dq + row_id * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        union { T e[4]; uint2 u; } pk;
#pragma unroll
        for (int e = 0; e < 4; e++) pk.e[e] = (T)(dqacc[db][4 * rr + e] * out_scale);
        *reinterpret_cast<uint2*>(op + 32 * db + 8 * rr) = pk.u;
      }
  }
}

extern __shared__ __align__(16) unsigned char bwd_smem[];

// dK/dV workgroup: 4 waves = 4 key blocks of 32 rows (kListBN keys); every wave takes the
// four 32-row query blocks of a tile in turn, so a Q / dO tile fetched from L2 serves 128 keys
// and nothing has to be summed across waves.  With D = 64 two such workgroups share a
// compute unit (two waves per SIMD); being independent they drift out of phase, so one's
// matrix work overlaps the other's vector work and barrier waits.  With D = 128 a wave holds
// 410 - 430 registers (128 of them dK / dV accumulators), so one workgroup has the compute unit.
template <int D> struct DkvShape {
  static constexpr int kWaves = kListBN / 32;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int kQBlocks = kBM / 32;        // 32-row query blocks per wave and tile
};

// BITS: the mask is a bitmap.  Band masks get an instantiation of their own, without the bitmap code: with it in the
// same function the compiler allocates registers differently and the unmasked path runs 5 % slower.
// PARITY: the numerics of the dense path: dP is rounded through the input dtype before delta (= sum_j P round(dP),
// from the kBwdDelta sweep) is subtracted, and the scale is applied before dS is rounded.
// HILO (the "unrounded" numerics, exclusive with PARITY, launched with ROUND_S = false): P and dS go into their
// products as a high and a low part each (two matrix instructions per fragment); delta comes from the kBwdDeltaRaw sweep.
template <typename T, int D, int KIND, bool ROUND_S, bool BITS, bool PARITY = false, bool HILO = false>
__global__ __launch_bounds__(DkvShape<D>::kThreads, D == 64 ? 2 : 1) void bwd_dkv_kernel(FlexAttnParams p, const T* __restrict__ q,
                                                               const T* __restrict__ k, const T* __restrict__ v,
                                                               const float* __restrict__ lse2,
                                                               const float* __restrict__ delta,
                                                               const T* __restrict__ d_o, T* __restrict__ dk,
                                                               T* __restrict__ dv) {
  typedef typename Frag<T>::vec8 vec8;
  constexpr int BM = kBM, BN = kListBN;
  constexpr int QBW = DkvShape<D>::kQBlocks;
  // The Q and dO tiles land in LDS straight from global memory (unpadded rows, chunk c of row r at position
  // c ^ lds_swz(r): conflict-free for the row-fragment and the transposing reads), one tile ahead of the one being
  // read, into two stages of (Q tile, dO tile, lse, -delta): one workgroup barrier per tile.  (At D = 128 this replaced
  // one stage filled through registers between two barriers: [4,16,4096,128] bf16 1425 -> 1345 us dense, 828 -> 733 us
  // causal in the parity numerics.)
  constexpr int DS = D / 16, DB = D / 32, ROWE = D, CPR = D / 8;
  constexpr int kStageBytes = 2 * BM * ROWE * (int)sizeof(T) + 2 * BM * (int)sizeof(float);
  auto stage_q = [&](int st) { return reinterpret_cast<T*>(bwd_smem + st * kStageBytes); };

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int i32 = lane & 31, g = lane >> 5, i16 = lane & 15;
  const int wk = __builtin_amdgcn_readfirstlane(w);  // key block (32 rows) of this wave (wave-uniform)
  const int nkt = (p.Lkv + BN - 1) / BN;
  int kt, bh;  // early key tiles see the most queries under causal masks
  xcd_tile_map(blockIdx.x, nkt, p.Hkv * p.B, kt, bh);
  const int hk = bh % p.Hkv, b = bh / p.Hkv, G = p.Hq / p.Hkv;
  const int kv_col = kt * BN + wk * 32 + i32;
  const int kv_ld = min(kv_col, p.Lkv - 1);

  vec8 kf[DS], vf[DS];
  {
    const T* kp = k + b * p.k_stride[0] + hk * p.k_stride[1] + (int64_t)kv_ld * p.k_stride[2] + 8 * g;
    const T* vp = v + b * p.v_stride[0] + hk * p.v_stride[1] + (int64_t)kv_ld * p.v_stride[2] + 8 * g;
#pragma unroll
    for (int s = 0; s < DS; s++) {
      kf[s] = *reinterpret_cast<const vec8*>(kp + 16 * s);
      vf[s] = *reinterpret_cast<const vec8*>(vp + 16 * s);
    }
  }
  float16_t dkacc[DB], dvacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dkacc[db][r] = 0.f; dvacc[db][r] = 0.f; }
  // element offsets inside a 32-row block of a tile: row fragments (row i32, chunk 2s + g) and transposing
  // reads (4 elements of row 4g + (i16 >> 2) + 8e, logical column 32db + 16hh + 4(i16 & 3))
  const int kz = g ^ lds_swz<D>(i32);
  int toff[2][DB];
  {
    const int rl = 4 * g + (i16 >> 2), hh = (lane >> 4) & 1;
#pragma unroll
    for (int e = 0; e < 2; e++)
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const int chunk = 4 * db + 2 * hh + ((i16 & 3) >> 1);
        const int pos = chunk ^ lds_swz<D>(rl + 8 * e);
        toff[e][db] = (rl + 8 * e) * ROWE + pos * 8 + 4 * (i16 & 1);
      }
  }

  const FlexTileLists& tl = p.tiles_bwd;
  Score2<KIND> sm;
  float key_grad = 1.f;  // derivative of a score_mod that depends on the key only: applied to dK at the end

  for (int gi = 0; gi < G; gi++) {
    const int h = hk * G + gi;
    sm.init(p.score, p.scale, h, b, p.Lq, p.Lkv);
    const int32_t* full_idx = nullptr;
    const int32_t* part_idx = nullptr;
    int n_full, n_part = 0;
    if (tl.kv_num) {
      const int64_t row = (b * tl.stride_b + h * tl.stride_h) * tl.n_kv_blocks + kt;
      n_full = uniform_ld(tl.full_q_num + row);
      n_part = uniform_ld(tl.q_num + row);
      full_idx = tl.full_q_idx + row * tl.n_q_blocks;
      part_idx = tl.q_idx + row * tl.n_q_blocks;
    } else {
      // no lists: every tile is visited, and evaluated under a mask that can hide something
      n_full = (p.Lq + BM - 1) / BM;
      if (!mask_hides_nothing(p.mask)) { n_part = n_full; n_full = 0; }
    }
    const int nt = n_full + n_part;
    const T* qbase = q + b * p.q_stride[0] + h * p.q_stride[1];
    const int64_t rows0 = ((int64_t)b * p.Hq + h) * p.Lq;
    const T* dobase = d_o + rows0 * D;

    auto tile_at = [&](int it) -> int {
      if (!full_idx) return it;
      return uniform_ld(it < n_full ? full_idx + it : part_idx + (it - n_full));
    };
    float lreg = INFINITY, dreg = 0.f;  // lse and delta of the tile after next, one row per thread
    // tile fetch: wave w fills rows [32w, 32w + 32) of the Q and the dO tile, 64 / CPR rows per instruction; the lane
    // that fills position (r, pos) fetches chunk pos ^ lds_swz(r) of that row
    auto issue_tile = [&](int st, int q0) {
      T* Qw = stage_q(st);
      T* Ow = Qw + BM * ROWE;
      constexpr int RPI = 64 / CPR, NI = 32 / RPI;  // rows per fetch instruction, instructions per wave and tensor
      const int lim = p.Lq - 1 - q0;  // rows past the end: clamped (finite filler; their lse is +inf, so P = 0)
#pragma unroll
      for (int j = 0; j < NI; j++) {
        const int r0 = 32 * w + RPI * j;
        const int chunk = (lane % CPR) ^ lds_swz<D>(RPI * j + lane / CPR);  // the wave's first row is a multiple of 16
        const int row = min(r0 + lane / CPR, lim);
        const T* qg = qbase + (int64_t)(q0 + row) * p.q_stride[2] + chunk * 8;
        const T* og = dobase + (int64_t)(q0 + row) * D + chunk * 8;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)qg,
                                         (__attribute__((address_space(3))) void*)(Qw + r0 * ROWE), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)og,
                                         (__attribute__((address_space(3))) void*)(Ow + r0 * ROWE), 16, 0, 0);
      }
    };
    auto load_tile = [&](int q0) {
      lreg = INFINITY;
      dreg = 0.f;
      if (tid < BM && q0 + tid < p.Lq) {
        lreg = lse2[rows0 + q0 + tid];
        dreg = delta[rows0 + q0 + tid];
        if (lreg == -INFINITY) lreg = INFINITY;  // row without visible keys: P = 0
      }
    };
    int t_cur = nt > 0 ? tile_at(0) : 0;
    int t_nxt = nt > 1 ? tile_at(1) : 0;
    auto store_tile = [&](int st) {
      T* Qw = stage_q(st);
      T* Ow = Qw + BM * ROWE;
      float* lw = reinterpret_cast<float*>(Ow + BM * ROWE);
      if (tid < BM) {
        lw[tid] = lreg;        // rows past Lq carry lse = +inf: P = 0, whatever the clamped loads hold
        lw[BM + tid] = -dreg;  // the dP accumulator starts from -delta
      }
    };
    __syncthreads();  // the stages may still be in use by the previous head of the group
    if (nt > 0) {
      issue_tile(0, t_cur * BM);
      load_tile(t_cur * BM);
      store_tile(0);
    }
    if (nt > 1) load_tile(t_nxt * BM);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (int it = 0; it < nt; it++) {
      const int q0 = t_cur * BM;
      const bool masked = (it >= n_full) || (q0 + BM > p.Lq) || (kt * BN + BN > p.Lkv);
      const T* Qs = stage_q(it & 1);
      const T* Os = Qs + BM * ROWE;
      const float* lse_s = reinterpret_cast<const float*>(Os + BM * ROWE);
      const float* del_s = lse_s + BM;
      if (it + 1 < nt) {
        // the other stage was last read before the previous barrier: refill it (the tile itself is fetched
        // straight into it now and awaited at the end of this tile; lse and delta were prefetched into
        // registers), then start fetching the lse and delta of the one after
        issue_tile((it + 1) & 1, t_nxt * BM);
        store_tile((it + 1) & 1);
        t_cur = t_nxt;
        if (it + 2 < nt) {
          t_nxt = tile_at(it + 2);
          load_tile(t_nxt * BM);
        }
      }

#pragma unroll
      for (int qs = 0; qs < QBW; qs++) {
      // ---- S = Q.K^T and dP = dO.V^T for 32 query rows x 32 keys ----
      const int qrow_w = qs * 32;
      int cls = kBlockAll;
      if (masked) {
        if constexpr (BITS) {
          const Mask2 visible(p.mask, b, h, p.Lkv);
          cls = block_class(p.mask, visible, q0 + qrow_w, kt * BN + wk * 32, p.Lq, p.Lkv);
        } else {
          cls = band_block_class(p.mask, q0 + qrow_w, kt * BN + wk * 32, p.Lq, p.Lkv);
        }
        if (cls == kBlockNone) continue;
      }
      float16_t sacc, dpacc;
      const int ql = qrow_w + 4 * g;  // local row of register 0
      sm.tileT(q0 + ql, kv_col);      // a table-reading score_mod fetches its entries under the products
      float16_t ndel;  // -delta of the block's rows (parity numerics: subtracted after dP is rounded)
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        const float4_t d4 = *reinterpret_cast<const float4_t*>(del_s + ql + 8 * rr);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          sacc[4 * rr + e] = 0.f;
          dpacc[4 * rr + e] = PARITY ? 0.f : d4[e];
          if constexpr (PARITY) ndel[4 * rr + e] = d4[e];
        }
      }
      {
        const T* qp = Qs + (qrow_w + i32) * ROWE;
        const T* op = Os + (qrow_w + i32) * ROWE;
#pragma unroll
        for (int s = 0; s < DS; s++) {
          sacc = Frag<T>::mfma(*reinterpret_cast<const vec8*>(qp + (((2 * s) ^ kz) * 8)), kf[s], sacc);
          dpacc = Frag<T>::mfma(*reinterpret_cast<const vec8*>(op + (((2 * s) ^ kz) * 8)), vf[s], dpacc);
        }
      }
      // the transposed dO and Q fragments of the closing products are fetched now, under the softmax arithmetic,
      // instead of right before their use (D = 64: 1.7 % of the kernel's time)
      vec8 a_do[2][DB], a_q[2][DB];
#pragma unroll
      for (int tt = 0; tt < 2; tt++)
#pragma unroll
        for (int db = 0; db < DB; db++) {
          const int base = (qrow_w + 16 * tt) * ROWE;
          a_do[tt][db] = join8<vec8>(lds_read_tr(Os + base + toff[0][db]), lds_read_tr(Os + base + toff[1][db]));
          a_q[tt][db] = join8<vec8>(lds_read_tr(Qs + base + toff[0][db]), lds_read_tr(Qs + base + toff[1][db]));
        }
      // x = log2(e) * score_mod(scale * s) - lse_q  (P = 2^x), dp <- dP - delta_q
      float16_t gacc;
      if constexpr (KIND == kScoreCheckerboardKv) key_grad = sm.key_grad;
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        const float4_t l4 = *reinterpret_cast<const float4_t*>(lse_s + ql + 8 * rr);
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          const int r = 4 * rr + e;
          float s0 = sacc[r], s1 = sacc[r + 1];
          if (ROUND_S) round_pair<T>(s0, s1);
          sacc[r] = sm.apply_sub(s0, acc_row(r), l4[e]);
          sacc[r + 1] = sm.apply_sub(s1, acc_row(r + 1), l4[e + 1]);
          if (!Score2<KIND>::kGradOne) {
            gacc[r] = sm.grad(s0, acc_row(r));
            gacc[r + 1] = sm.grad(s1, acc_row(r + 1));
          }
        }
      }
      if (cls == kBlockMixed) {
        int q_opaque = q0 + ql, kv_opaque = kv_col;
        asm volatile("" : "+v"(q_opaque), "+v"(kv_opaque));  // keeps the mask arithmetic behind this branch
        const Mask2 visible(p.mask, b, h, p.Lkv);
        mask_block_kv<BITS>(sacc, p.mask, visible, q_opaque, kv_opaque, p.Lq, p.Lkv);
      }
      vec8 pf[2], dsf[2], pf_lo[2], dsf_lo[2];
#pragma unroll
      for (int tt = 0; tt < 2; tt++) {
        typename Pair<T>::v2 pp[4], dd[4], pl[4], dl[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 8 * tt + 2 * e;
          const float p0 = fast_exp2(sacc[r]), p1 = fast_exp2(sacc[r + 1]);
          float d0, d1;
          if constexpr (PARITY) {
            float a0 = dpacc[r], a1 = dpacc[r + 1];
            round_pair<T>(a0, a1);
            d0 = p0 * (a0 + ndel[r]);
            d1 = p1 * (a1 + ndel[r + 1]);
          } else {
            d0 = p0 * dpacc[r];
            d1 = p1 * dpacc[r + 1];
          }
          if (!Score2<KIND>::kGradOne) { d0 *= gacc[r]; d1 *= gacc[r + 1]; }
          if constexpr (PARITY) { d0 *= p.scale; d1 *= p.scale; }
          if constexpr (HILO) {
            split_pack<T>(p0, p1, pp[e], pl[e]);
            split_pack<T>(d0, d1, dd[e], dl[e]);
          } else {
            pp[e] = Pair<T>::pack(p0, p1);
            dd[e] = Pair<T>::pack(d0, d1);
          }
        }
        pf[tt] = join_pairs<T>(pp[0], pp[1], pp[2], pp[3]);
        dsf[tt] = join_pairs<T>(dd[0], dd[1], dd[2], dd[3]);
        if constexpr (HILO) {
          pf_lo[tt] = join_pairs<T>(pl[0], pl[1], pl[2], pl[3]);
          dsf_lo[tt] = join_pairs<T>(dl[0], dl[1], dl[2], dl[3]);
        }
      }
      // ---- dV^T += dO^T.P, dK^T += Q^T.dS (contraction over this wave's 32 query rows) ----
#pragma unroll
      for (int tt = 0; tt < 2; tt++) {
#pragma unroll
        for (int db = 0; db < DB; db++) {
          dvacc[db] = Frag<T>::mfma(a_do[tt][db], pf[tt], dvacc[db]);
          dkacc[db] = Frag<T>::mfma(a_q[tt][db], dsf[tt], dkacc[db]);
          if constexpr (HILO) {
            dvacc[db] = Frag<T>::mfma(a_do[tt][db], pf_lo[tt], dvacc[db]);
            dkacc[db] = Frag<T>::mfma(a_q[tt][db], dsf_lo[tt], dkacc[db]);
          }
        }
      }
      }  // query blocks of this wave
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next tile has landed
      __syncthreads();
    }
  }

  if (kv_col < p.Lkv) {
    const int64_t row_id = ((int64_t)b * p.Hkv + hk) * p.Lkv + kv_col;
    T* dkp = dk + row_id * D + 4 * g;
    T* dvp = dv + row_id * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        union { T e[4]; uint2 u; } pk, pv;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 4 * rr + e;
          pk.e[e] = (T)(dkacc[db][r] * (PARITY ? 1.f : p.scale * key_grad));  // fast numerics: the scale factor of dS is applied once here
          pv.e[e] = (T)dvacc[db][r];
        }
        *reinterpret_cast<uint2*>(dkp + 32 * db + 8 * rr) = pk.u;
        *reinterpret_cast<uint2*>(dvp + 32 * db + 8 * rr) = pv.u;
      }
  }
}

// two stages of (Q tile, dO tile, lse, -delta)
template <int D, typename T> constexpr size_t dkv_smem() {
  return 2 * ((size_t)2 * kBM * D * sizeof(T) + 2 * kBM * sizeof(float));
}

// everything a backward launch needs besides the template choice
struct BwdArgs {
  const void *q, *k, *v, *o, *d_o;
  const float* lse2;
  void *dq, *dk, *dv;
  float* delta;
  hipStream_t s;
};

// (D = 192 and D = 256 have the dQ kernel only: the resident K / V fragments and the two accumulators of a dK/dV workgroup do not
// fit a wave's registers; the caller runs the dK/dV kernel of the simple family)
template <typename T, int D, int KIND, bool RS, bool BITS, bool PARITY, bool HILO = false>
static int launch_dkv_as(const FlexAttnParams& p, const BwdArgs& a) {
  if constexpr (D >= 192) {
    return 3;
  } else {
  constexpr size_t sm = dkv_smem<D, T>();
  // set on every call: the attribute is per device, and a remembered "already set" would be neither
  // per device nor safe between threads (the call is a host-side table update, no device work)
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(bwd_dkv_kernel<T, D, KIND, RS, BITS, PARITY, HILO>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm) != hipSuccess)
    return 2;
  const int nkt = (p.Lkv + kListBN - 1) / kListBN;
  hipLaunchKernelGGL((bwd_dkv_kernel<T, D, KIND, RS, BITS, PARITY, HILO>), dim3(nkt * p.Hkv * p.B), dim3(DkvShape<D>::kThreads), sm, a.s,
                     p, (const T*)a.q, (const T*)a.k, (const T*)a.v, a.lse2, a.delta, (const T*)a.d_o, (T*)a.dk, (T*)a.dv);
  return 0;
  }
}
template <typename T, int D, int KIND, bool RS, bool PARITY>
static int launch_dkv(const FlexAttnParams& p, const BwdArgs& a) {
  if (p.mask.kind == FLEX_MASK_BITS) return launch_dkv_as<T, D, KIND, RS, true, PARITY>(p, a);
  return launch_dkv_as<T, D, KIND, RS, false, PARITY>(p, a);
}

template <typename T, int D, int KIND, bool RS, bool MASKED, int MODE>
static void launch_dq_as(const FlexAttnParams& p, const BwdArgs& a) {
  const int nqt = (p.Lq + kBM - 1) / kBM;
  hipLaunchKernelGGL((bwd_dq_kernel<T, D, KIND, RS, MASKED, MODE>), dim3(nqt * p.Hq * p.B), dim3(256), 0, a.s, p, (const T*)a.q,
                     (const T*)a.k, (const T*)a.v, (const T*)a.o, a.lse2, (const T*)a.d_o, (T*)a.dq, a.delta);
}

template <typename T, int D, int KIND, bool RS>
static void launch_dq(const FlexAttnParams& p, const BwdArgs& a) {
  constexpr int BN = dq_tile_keys<D, kBwdFast>();   // the kernel's key tile
  if constexpr (D < 192) {  // (at D = 192 / 256 the mask-free instantiation is the one that spills: not used)
    if (!p.tiles_bwd.kv_num && mask_hides_nothing(p.mask) && p.Lkv % BN == 0) {
      launch_dq_as<T, D, KIND, RS, false, kBwdFast>(p, a);
      return;
    }
  }
  launch_dq_as<T, D, KIND, RS, true, kBwdFast>(p, a);
}

template <typename T, int D, int KIND, bool RS>
static int launch_one(const FlexAttnParams& p, const BwdArgs& a) {
  if (!(p.flags & FLEX_BWD_ONLY_DKV)) {
    if (KIND == FLEX_SCORE_CHECKERBOARD && p.score.p0 > 0.f && p.score.p1 > 0.f) {
      // positive factors: the derivative folds into the exponent
      constexpr int KF = KIND == FLEX_SCORE_CHECKERBOARD ? kScoreCheckerboardFold : KIND;
      launch_dq<T, D, KF, RS>(p, a);
    } else {
      launch_dq<T, D, KIND, RS>(p, a);
    }
  }
  if (p.flags & FLEX_BWD_ONLY_DQ) return 0;
  if (KIND == FLEX_SCORE_CHECKERBOARD && p.score.i0) {
    // keyed on the key index: the derivative is constant along a lane's dK row
    constexpr int KV = KIND == FLEX_SCORE_CHECKERBOARD ? kScoreCheckerboardKv : KIND;
    return launch_dkv<T, D, KV, RS, false>(p, a);
  }
  return launch_dkv<T, D, KIND, RS, false>(p, a);
}

// parity numerics (FLEX_PARITY): row sweep for delta, then dQ and dK/dV with rounded dP; S is always rounded
// through the input dtype here, and the score_mod derivative stays inside the rounding (no folded variants)
template <typename T, int D, int KIND>
static int launch_parity(const FlexAttnParams& p, const BwdArgs& a) {
  if (!(p.flags & FLEX_BWD_ONLY_DKV)) {
    launch_dq_as<T, D, KIND, true, true, kBwdDelta>(p, a);
    launch_dq_as<T, D, KIND, true, true, kBwdParity>(p, a);
  }
  if (p.flags & FLEX_BWD_ONLY_DQ) return 0;
  return launch_dkv<T, D, KIND, true, true>(p, a);
}

// "unrounded" numerics (FLEX_UNROUNDED): unrounded row sweep for delta, then dQ and dK/dV with P and dS carried as
// high and low parts; S is not rounded
template <typename T, int D, int KIND>
static int launch_unrounded(const FlexAttnParams& p, const BwdArgs& a) {
  if (!(p.flags & FLEX_BWD_ONLY_DKV)) {
    launch_dq_as<T, D, KIND, false, true, kBwdDeltaRaw>(p, a);
    launch_dq_as<T, D, KIND, false, true, kBwdHiLo>(p, a);
  }
  if (p.flags & FLEX_BWD_ONLY_DQ) return 0;
  if (p.mask.kind == FLEX_MASK_BITS) return launch_dkv_as<T, D, KIND, false, true, false, true>(p, a);
  return launch_dkv_as<T, D, KIND, false, false, false, true>(p, a);
}

template <typename T, int D, int KIND>
static int launch_rs(const FlexAttnParams& p, const BwdArgs& a) {
  if (p.flags & FLEX_UNROUNDED) return launch_unrounded<T, D, KIND>(p, a);
  if (p.flags & FLEX_PARITY) return launch_parity<T, D, KIND>(p, a);
  if (p.flags & FLEX_ROUND_S) return launch_one<T, D, KIND, true>(p, a);
  return launch_one<T, D, KIND, false>(p, a);
}

// rc: 0 launched, 1 unknown score_mod kind, 2 the dynamic LDS limit could not be raised
template <typename T, int D>
static int launch_kind(const FlexAttnParams& p, const BwdArgs& a) {
  switch (p.score.kind) {
    case FLEX_SCORE_IDENTITY: return launch_rs<T, D, FLEX_SCORE_IDENTITY>(p, a);
    case FLEX_SCORE_CHECKERBOARD: return launch_rs<T, D, FLEX_SCORE_CHECKERBOARD>(p, a);
    case FLEX_SCORE_ALIBI: return launch_rs<T, D, FLEX_SCORE_ALIBI>(p, a);
    case FLEX_SCORE_TANH_SOFTCAP: return launch_rs<T, D, FLEX_SCORE_TANH_SOFTCAP>(p, a);
    case FLEX_SCORE_REL_BIAS: return launch_rs<T, D, FLEX_SCORE_REL_BIAS>(p, a);
    case FLEX_SCORE_AFFINE:
      return p.score.mul ? launch_rs<T, D, kScoreAffineMul>(p, a) : launch_rs<T, D, FLEX_SCORE_AFFINE>(p, a);
  }
  return 1;
}

}  // namespace flex
