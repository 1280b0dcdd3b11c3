// Block-mask builder for gfx950.
//
// Replaces the dense [B,H,Q,KV] boolean mask + reshape/sum + argsort pipeline of
// flaxattention/core/blockmask.py:277-322, 335-369, 57-64: the mask functor is
// evaluated per tile in registers, each tile is classified empty / partial /
// full, and the per-row ordered index lists are produced by a wave-level
// stable partition (selected ids ascending, then the rest ascending -- the
// order a stable descending argsort of a 0/1 row gives).  The dense mask is
// never materialised.  All outputs are integers and bit-exact.
#include "flex_common.cuh"

namespace flex {

constexpr int kClassifyThreads = 256;

// One workgroup per tile.  flags: [B*H, nq, nkv] int8 for partial and full.
__global__ __launch_bounds__(kClassifyThreads) void classify_tiles_kernel(
    FlexMask mask, int H, int nq, int nkv, int qb, int kvb, int8_t* __restrict__ partial,
    int8_t* __restrict__ full) {
  const int ki = blockIdx.x, qi = blockIdx.y, bh = blockIdx.z;
  const int b = bh / H, h = bh % H;
  MaskEval visible(mask, b, h);
  const int q0 = qi * qb, kv0 = ki * kvb;
  const long long total = (long long)qb * kvb;
  unsigned long long cnt = 0;
  if (mask.kind == FLEX_MASK_BITS && (kvb % 32) == 0) {
    // word-at-a-time: every aligned 32-bit word of a row lies inside the tile
    const int words = kvb / 32;
    const long long nwords = (long long)qb * words;
    for (long long t = threadIdx.x; t < nwords; t += kClassifyThreads) {
      int r = (int)(t / words), w = (int)(t % words);
      uint32_t bits = visible.bits_bh[(int64_t)(q0 + r) * visible.stride_q + (kv0 >> 5) + w];
      cnt += __popc(bits);
    }
  } else if (mask.kind == FLEX_MASK_BAND) {
    // closed form per row: with d = q + q_offset - kv the visible keys of a row are
    //   { kv <= U } minus the gap { S < kv < W },   U = q + q_offset - lo,  W = q + q_offset - hi,  S = sink
    // (d >= lo <=> kv <= U;  d <= hi <=> kv >= W), so the count inside [kv0, kv_end] takes a few
    // integer operations instead of kvb evaluations.  Same count as the element-wise loop below.
    const long long kv_end = (long long)kv0 + kvb - 1;
    for (int r = threadIdx.x; r < qb; r += kClassifyThreads) {
      const long long qo = (long long)q0 + r + mask.q_offset;
      const long long top = min(qo - mask.lo, kv_end);           // last visible candidate in the tile
      const long long seen = max(0LL, top - kv0 + 1);
      const long long gap_lo = max((long long)mask.sink + 1, (long long)kv0);
      const long long gap_hi = min(qo - mask.hi - 1, top);
      cnt += (unsigned long long)(seen - max(0LL, gap_hi - gap_lo + 1));
    }
  } else {
    for (long long t = threadIdx.x; t < total; t += kClassifyThreads) {
      int r = (int)(t / kvb), c = (int)(t % kvb);
      cnt += visible(q0 + r, kv0 + c) ? 1u : 0u;
    }
  }
  // workgroup reduction
  for (int off = 32; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off, 64);
  __shared__ unsigned long long wsum[kClassifyThreads / 64];
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long s = 0;
    for (int w = 0; w < kClassifyThreads / 64; w++) s += wsum[w];
    size_t at = ((size_t)bh * nq + qi) * nkv + ki;
    full[at] = (s == (unsigned long long)total) ? 1 : 0;
    partial[at] = (s > 0 && s < (unsigned long long)total) ? 1 : 0;
  }
}

// The four ordered lists of a block mask (partial / full, by query block / by key block) come from one
// launch: blockIdx.y names the list.
struct OrderJob {
  const int8_t* flags;
  int32_t* num;
  int32_t* idx;
  int nrows, ncols, row_stride, col_stride;
};
struct OrderJobs { OrderJob job[4]; };

// One wave per output row.  Reads flags[bh][r*row_stride + c*col_stride] for
// c in [0, ncols) and writes num[bh][r] and idx[bh][r][0..ncols).
__global__ __launch_bounds__(256) void order_rows_kernel(OrderJobs jobs, long long mat_stride, long long n_bh) {
  const OrderJob& jb = jobs.job[blockIdx.y];
  if (!jb.num && !jb.idx) return;
  const int nrows = jb.nrows, ncols = jb.ncols;
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= n_bh * nrows) return;
  const long long bh = row / nrows;
  const int r = (int)(row % nrows);
  const int8_t* f = jb.flags + bh * mat_stride + (long long)r * jb.row_stride;
  const int col_stride = jb.col_stride;
  int count = 0;
  for (int c0 = 0; c0 < ncols; c0 += 64) {
    int c = c0 + lane;
    bool sel = (c < ncols) && f[(long long)c * col_stride] != 0;
    count += __popcll(__ballot(sel));
  }
  if (jb.num && lane == 0) jb.num[row] = count;
  if (!jb.idx) return;
  int32_t* out = jb.idx + row * ncols;
  int before_sel = 0, before_uns = 0;
  const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int c0 = 0; c0 < ncols; c0 += 64) {
    int c = c0 + lane;
    bool in = c < ncols;
    bool sel = in && f[(long long)c * col_stride] != 0;
    unsigned long long ms = __ballot(sel), mu = __ballot(in && !sel);
    if (sel) out[before_sel + __popcll(ms & lt)] = c;
    else if (in) out[count + before_uns + __popcll(mu & lt)] = c;
    before_sel += __popcll(ms);
    before_uns += __popcll(mu);
  }
}

}  // namespace flex

using namespace flex;

extern "C" size_t flexattn_block_mask_workspace_bytes(int32_t B, int32_t H, int32_t nq, int32_t nkv) {
  size_t n = (size_t)B * H * nq * nkv;
  return 2 * ((n + 255) / 256 * 256);
}

void flex_set_error(const char* fmt, ...);

extern "C" int flexattn_block_mask_build(const FlexMask* mask, int32_t B, int32_t H, int32_t nq,
                                         int32_t nkv, int32_t qb, int32_t kvb, int32_t* kv_num,
                                         int32_t* kv_idx, int32_t* full_kv_num, int32_t* full_kv_idx,
                                         int32_t* q_num, int32_t* q_idx, int32_t* full_q_num,
                                         int32_t* full_q_idx, void* workspace,
                                         flexattn_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!mask || !workspace) { flex_set_error("block_mask_build: null mask or workspace"); return 1; }
  if (B <= 0 || H <= 0 || nq <= 0 || nkv <= 0 || qb <= 0 || kvb <= 0) {
    flex_set_error("block_mask_build: non-positive size B=%d H=%d nq=%d nkv=%d qb=%d kvb=%d", B, H, nq, nkv, qb, kvb);
    return 1;
  }
  if ((long long)B * H > 65535 || nq > 65535) {
    flex_set_error("block_mask_build: grid too large (B*H=%lld, nq=%d; limit 65535)", (long long)B * H, nq);
    return 1;
  }
  if (mask->kind == FLEX_MASK_BITS && !mask->bits) { flex_set_error("block_mask_build: bitmap mask without bits"); return 1; }
  if (mask->kind != FLEX_MASK_BITS && mask->kind != FLEX_MASK_BAND) { flex_set_error("block_mask_build: unknown mask kind %d", mask->kind); return 1; }
  size_t n = (size_t)B * H * nq * nkv;
  int8_t* partial = (int8_t*)workspace;
  int8_t* full = partial + (n + 255) / 256 * 256;
  // a band mask (or a bitmap broadcast over batch and head) does not look at (b, h): its tiles are classified once
  // and every (b, h) orders the same flags
  const bool uniform = mask->kind == FLEX_MASK_BAND || (mask->bits_stride_b == 0 && mask->bits_stride_h == 0);
  dim3 grid(nkv, nq, uniform ? 1 : B * H);
  hipLaunchKernelGGL(classify_tiles_kernel, grid, dim3(kClassifyThreads), 0, stream, *mask, H, nq, nkv, qb, kvb, partial, full);
  const long long mat = uniform ? 0 : (long long)nq * nkv;
  OrderJobs jobs;
  auto job = [&](int at, const int8_t* flags, bool transposed, int32_t* num, int32_t* idx) {
    OrderJob& j = jobs.job[at];
    j.flags = flags; j.num = num; j.idx = idx;
    j.nrows = transposed ? nkv : nq; j.ncols = transposed ? nq : nkv;
    j.row_stride = transposed ? 1 : nkv; j.col_stride = transposed ? nkv : 1;
  };
  job(0, partial, false, kv_num, kv_idx);
  job(1, full, false, full_kv_num, full_kv_idx);
  job(2, partial, true, q_num, q_idx);
  job(3, full, true, full_q_num, full_q_idx);
  const bool by_kv = kv_num || kv_idx || full_kv_num || full_kv_idx, by_q = q_num || q_idx || full_q_num || full_q_idx;
  if (by_kv || by_q) {
    const int waves = 4;
    const long long most_rows = (long long)B * H * (by_q ? (by_kv ? (nq > nkv ? nq : nkv) : nkv) : nq);
    const long long blocks = (most_rows + waves - 1) / waves;
    hipLaunchKernelGGL(order_rows_kernel, dim3((unsigned)blocks, 4), dim3(64 * waves), 0, stream, jobs, mat, (long long)B * H);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { flex_set_error("block_mask_build: launch failed: %s", hipGetErrorString(e)); return 2; }
  return 0;
}
