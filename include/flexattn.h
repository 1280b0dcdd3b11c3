/*
 * flexattn.h -- C ABI of the MI355X (gfx950) FlexAttention engine.
 *
 * The reference (zinccat/flaxattention) has no native boundary: its surface is
 * Python (flax_attention, flax_attention_pallas, create_block_mask) over
 * jax.custom_vjp.  Each entry point below names the reference function whose
 * device work it replaces.  All tensor pointers are DEVICE pointers; every
 * call only enqueues work on `stream` and returns without synchronising.
 * Return value: 0 on success, non-zero on error with a thread-local message
 * available from flexattn_last_error().  No entry point allocates memory:
 * scratch is passed in by the caller and sized by the *_workspace_bytes
 * helpers.  Entry points are re-entrant.
 */
#ifndef FLEXATTN_H_
#define FLEXATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* flexattn_stream_t; /* a hipStream_t */

enum FlexDType { FLEX_F32 = 0, FLEX_F16 = 1, FLEX_BF16 = 2 };

/* score_mod functors: the scalar functions of (score, b, h, q_idx, kv_idx)
 * that flaxattention/core/common.py:7 types as _score_mod_signature. */
enum FlexScoreKind {
  FLEX_SCORE_IDENTITY = 0,     /* flaxattention/core/attention.py:109-116 */
  FLEX_SCORE_CHECKERBOARD = 1, /* examples/benchmark.py:16-22; i0 = 0: parity of
                                  (kv_idx - q_idx), i0 = 1: parity of kv_idx;
                                  p0 multiplies even entries, p1 odd entries */
  FLEX_SCORE_ALIBI = 2,        /* flaxattention/mods/alibi.py:15-18:
                                  score + p0*(q_idx-kv_idx)*exp2(-(h+1)*8/i0) */
  FLEX_SCORE_TANH_SOFTCAP = 3, /* p0 * tanh(score / p0) */
  FLEX_SCORE_REL_BIAS = 4,     /* score + p0 * (kv_idx - q_idx) */
  FLEX_SCORE_AFFINE = 5        /* mul[b,h,q,kv] * score + add[b,h,q,kv] from dense fp32
                                  tables: what a Python score_mod that is affine in the score
                                  (captured bias tables, position-dependent scaling;
                                  attention.py:22-23, 59-63) is lowered to, and what an arbitrary
                                  differentiable score_mod becomes when it is linearised at the
                                  scores of the call.  The fused kernels read both tables
                                  (16 entries per lane and 32x32 block).  */
};

typedef struct FlexScoreMod {
  int32_t kind;
  float p0, p1;
  int32_t i0, i1;
  /* FLEX_SCORE_AFFINE: tables indexed [b*stride_b + h*stride_h + q*stride_q + kv]
   * (strides in elements, 0 broadcasts); a NULL mul means 1, a NULL add means 0 */
  const float* mul;
  const float* add;
  int64_t stride_b, stride_h, stride_q;
} FlexScoreMod;

/* mask_mod functors (flaxattention/core/common.py:8).  FLEX_MASK_BAND is a
 * canonical form that covers noop_mask (blockmask.py:20-27), causal_mask
 * (masks/causal.py:4-5), generate_sliding_window (masks/sliding_window.py:
 * 7-22), generate_attention_sink (masks/attention_sink.py:6-24) and their
 * and_masks combinations:
 *     d = q_idx + q_offset - kv_idx
 *     visible = (d >= lo) && (d <= hi || kv_idx <= sink)
 * FLEX_MASK_BITS reads a packed bitmap produced from an arbitrary Python
 * callable: bit (kv & 31) of word bits[b*sb + h*sh + q*sq + (kv >> 5)].
 * bits_t is an optional second copy of the same bitmap packed along the query
 * axis: bit (q & 31) of word bits_t[b*tb + h*th + kv*tkv + (q >> 5)].  The
 * dK/dV kernel, whose lanes own keys, then reads one word per 32x32 block
 * instead of one per entry; without it (NULL) the result is the same.
 * blk, also optional, classifies every aligned 32x32 block of the bitmap:
 * blk[b*kb + h*kh + (q >> 5)*kq + (kv >> 5)] = 0 (some entries set), 1 (all
 * set) or 2 (none set).  Inside a partial tile the fused kernels then skip
 * hidden blocks and the mask evaluation of fully visible ones, as they do
 * for band masks by arithmetic.  */
enum FlexMaskKind { FLEX_MASK_BAND = 0, FLEX_MASK_BITS = 1 };

typedef struct FlexMask {
  int32_t kind;
  int32_t lo, hi, sink, q_offset;
  int32_t pad_;
  const uint32_t* bits;
  int64_t bits_stride_b, bits_stride_h, bits_stride_q; /* in 32-bit words */
  const uint32_t* bits_t;
  int64_t bits_t_stride_b, bits_t_stride_h, bits_t_stride_kv; /* in 32-bit words */
  const int8_t* blk;
  int64_t blk_stride_b, blk_stride_h, blk_stride_q; /* in bytes */
} FlexMask;

/* numerics switches (OR-ed into FlexAttnParams.flags) */
enum FlexFlags {
  FLEX_ROUND_S = 1,      /* round Q.K^T through the input dtype before scaling
                            (attention.py:27 computes the product in that dtype) */
  FLEX_STRICT = 2,       /* generic kernels only: also round the normalised P,
                            dP and dS through the input dtype (attention.py:105
                            and its transposes) */
  FLEX_FORCE_GENERIC = 4, /* never use the MFMA kernels */
  FLEX_PARITY = 32,      /* fused (MFMA) kernels with the rounding points of the reference's dense
                            path (attention.py:27, 104-105 and their transposes under jax.grad):
                            forward in two passes (log-sum-exp, then the NORMALISED P rounded to
                            the input dtype and multiplied into V); backward with dP rounded to the
                            input dtype, delta_i = sum_j P_ij round(dP_ij) from a row sweep of its
                            own, and the scale applied before dS is rounded.  Implies FLEX_ROUND_S.
                            Costs about 1.5x the time of the default numerics, which round the
                            unnormalised P and use delta = sum_d O dO.  Where only the generic
                            kernels apply the flag means FLEX_STRICT.  */
  FLEX_UNROUNDED = 64,   /* fused (MFMA) kernels WITHOUT the dense path's internal round trips: S is not
                            rounded, P and dS enter their matrix products as a high and a low part of
                            the input dtype (twice its mantissa), dP stays in fp32 and
                            delta_i = sum_j P_ij dP_ij comes from an unrounded row sweep; only O, dQ, dK,
                            dV are rounded.  What the reference computes if XLA's excess-precision
                            simplification removes the round trips of attention.py:27, 104-105.
                            Exclusive with FLEX_PARITY / FLEX_ROUND_S (it wins); the generic kernels
                            do the same when neither FLEX_STRICT nor FLEX_ROUND_S is set.  */
  /* profiling aids for flexattn_bwd: launch only one of the two fused backward
   * kernels.  The dK/dV kernel then reads the delta values a previous complete
   * call left in the same workspace. */
  FLEX_BWD_ONLY_DQ = 8,
  FLEX_BWD_ONLY_DKV = 16
};

/* Ordered tile lists in the layout of BlockMask.kv_num_blocks / kv_indices /
 * full_kv_* (blockmask.py:72-119), at the granularity (q_block, kv_block).
 * A NULL kv_num means "visit every tile and evaluate the mask in each".
 * Counts are [Bm, Hm, n_q_blocks], indices [Bm, Hm, n_q_blocks, n_kv_blocks];
 * Bm/Hm may be 1 (broadcast) -- give stride 0.  The transposed lists
 * (q_num / q_idx, per kv block) drive the dK/dV kernel.  */
typedef struct FlexTileLists {
  const int32_t* kv_num;
  const int32_t* kv_idx;
  const int32_t* full_kv_num;
  const int32_t* full_kv_idx;
  const int32_t* q_num;
  const int32_t* q_idx;
  const int32_t* full_q_num;
  const int32_t* full_q_idx;
  int32_t q_block, kv_block;
  int32_t n_q_blocks, n_kv_blocks;
  int64_t stride_b, stride_h; /* in rows of the count arrays */
} FlexTileLists;

typedef struct FlexAttnParams {
  int32_t dtype; /* FlexDType of q, k, v, o, do, dq, dk, dv */
  int32_t B, Hq, Hkv, Lq, Lkv, D, Dv;
  /* element strides of the (batch, head, position) axes; the feature axis is
   * contiguous.  [B,H,L,D] and [B,L,H,D] (flax_attention_pallas bhln=False,
   * attention.py:243-246) are both expressible. */
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];
  float scale;
  int32_t flags;
  FlexScoreMod score;
  FlexMask mask;
  FlexTileLists tiles;     /* lists for flexattn_fwd / flexattn_decode */
  FlexTileLists tiles_bwd; /* lists for flexattn_bwd (its kernels tile differently) */
  /* flexattn_decode only (0 elsewhere): the query tensor passed in is rows
   * [q_index_base, q_index_base + Lq) of a longer query; score_mod, mask_mod and the tile
   * lists see the full-sequence row index.  Lets a caller run a query of more rows than one
   * call takes against a long KV cache as several decode calls.  Not negative. */
  int32_t q_index_base;
  int32_t pad_;
  /* flexattn_bwd only, optional (NULL = zero): cotangent of the lse2 output, [B,Hq,Lq] fp32.
   * In the reference the log-sum-exp is an ordinary differentiable output of math_attention
   * (attention.py:97-106); d lse / d score_ij = P_ij joins the softmax's row term.  */
  const float* d_lse2;
} FlexAttnParams;

int flexattn_abi_version(void);
const char* flexattn_last_error(void);

/* Which kernel family flexattn_fwd (which = 0) or flexattn_bwd (which = 1) runs for these parameters: a pure
 * function of *p, no device work.  The reference has one dense path and one fused kernel
 * (core/attention.py:14-106, kernel/attention.py:166-653); here the choice depends on dtype, head sizes, strides,
 * flags and list granularity, and a caller (or a test) can ask instead of guessing. */
enum FlexKernelFamily {
  FLEX_FAMILY_GENERIC = 0,    /* vector-ALU kernels: any dtype / head size, FLEX_STRICT numerics */
  FLEX_FAMILY_MFMA_16BIT = 1, /* fused fp16 / bf16 matrix-core kernels */
  FLEX_FAMILY_MFMA_F32 = 2    /* fp32 matrix-core kernels */
};
int flexattn_kernel_family(const FlexAttnParams* p, int32_t which);

/* Tile sizes the fused kernels want their FlexTileLists built at for this
 * problem (0/0 when only the generic kernels apply and lists are ignored).
 * which = 0: FlexAttnParams.tiles (forward, decode); which = 1: tiles_bwd. */
int flexattn_preferred_tiles(int32_t dtype, int32_t D, int32_t Dv, int32_t Lq, int32_t Lkv,
                             int32_t which, int32_t* q_block, int32_t* kv_block);

/* Block-mask builder.  Replaces create_block_mask -> _create_block_mask_inner
 * -> create_mask / _convert_mask_to_block_mask -> _dense_to_ordered
 * (flaxattention/core/blockmask.py:419-455, 400-416, 277-322, 335-369, 57-64)
 * and the transposes of BlockMask.from_kv_blocks (121-164).  q_len / kv_len
 * are the padded lengths n_q_blocks*q_block / n_kv_blocks*kv_block; the mask is
 * evaluated on that whole index range (blockmask.py:440-444).  Outputs are
 * int32: counts [B,H,nq], indices [B,H,nq,nkv]; q_* are [B,H,nkv] and
 * [B,H,nkv,nq].  Any output pointer may be NULL.  `workspace` holds
 * flexattn_block_mask_workspace_bytes() bytes.  */
size_t flexattn_block_mask_workspace_bytes(int32_t B, int32_t H, int32_t n_q_blocks, int32_t n_kv_blocks);
int flexattn_block_mask_build(const FlexMask* mask, int32_t B, int32_t H,
                              int32_t n_q_blocks, int32_t n_kv_blocks,
                              int32_t q_block, int32_t kv_block,
                              int32_t* kv_num, int32_t* kv_idx,
                              int32_t* full_kv_num, int32_t* full_kv_idx,
                              int32_t* q_num, int32_t* q_idx,
                              int32_t* full_q_num, int32_t* full_q_idx,
                              void* workspace, flexattn_stream_t stream);

/* Forward.  With FLEX_PARITY and lse2 == NULL the log-sum-exp that the second pass reads is kept
 * in `workspace` (flexattn_fwd_workspace_bytes); otherwise workspace may be NULL.  A workspace
 * of that size also lets the matrix-core kernels split calls with few query rows against many
 * keys over the keys, so that they fill the GPU; without one such calls run unsplit.
 * Replaces math_attention (flaxattention/core/attention.py:67-106)
 * behind flax_attention (169-218) and mha_forward_kernel / _mha_forward
 * (flaxattention/kernel/attention.py:34-149, 260-335) behind
 * flax_attention_pallas (attention.py:220-312).  o: same layout family as q
 * with Dv features; lse2: [B,Hq,Lq] fp32 base-2 log-sum-exp (-inf on rows with
 * no visible key), may be NULL.  */
size_t flexattn_fwd_workspace_bytes(const FlexAttnParams* p);
int flexattn_fwd(const FlexAttnParams* p, const void* q, const void* k, const void* v,
                 void* o, float* lse2, void* workspace, flexattn_stream_t stream);

/* Backward.  Replaces jax.grad through math_attention (the reference's pure
 * path) and _preprocess_backward / mha_backward_kernel / _mha_backward
 * (flaxattention/kernel/attention.py:338-650).  P is recomputed from lse2.
 * d_o is a contiguous [B,Hq,Lq,Dv] tensor (the strides in `p` describe q, k,
 * v and o only); dq/dk/dv are contiguous [B,H,L,D] tensors of the input dtype.  */
size_t flexattn_bwd_workspace_bytes(const FlexAttnParams* p);
int flexattn_bwd(const FlexAttnParams* p, const void* q, const void* k, const void* v,
                 const void* o, const float* lse2, const void* d_o,
                 void* dq, void* dk, void* dv, void* workspace, flexattn_stream_t stream);

/* Split-KV decode for short queries: fp16 / bf16, D = Dv in {64, 128} with at most 64 query
 * columns (query rows x query heads per KV head) or D = Dv in {192, 256} with at most 32.  Replaces the
 * same reference functions as flexattn_fwd for the decode shapes of
 * examples/benchmark_decoding.py:29-33.  num_splits <= 0 picks a default.  */
size_t flexattn_decode_workspace_bytes(const FlexAttnParams* p, int32_t num_splits);
int flexattn_decode(const FlexAttnParams* p, const void* q, const void* k, const void* v,
                    void* o, float* lse2, int32_t num_splits, void* workspace,
                    flexattn_stream_t stream);

/* flexattn_decode for callers that cannot allocate device memory or hand in a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  The split-KV partials go to a buffer of
 * FLEXATTN_DECODE_STATIC_BYTES that is part of the library image on every GPU it runs on (held
 * until the process ends); the call makes no hipMalloc / hipFree and no other allocating call.
 * Problems whose partials (flexattn_decode_workspace_bytes) exceed that size are refused with
 * an error; use flexattn_decode for those.  All calls on one GPU share the buffer, whose
 * contents do not carry over between calls (every call overwrites what it reads): calls that
 * overlap on one GPU -- two streams, two threads -- race.  Results are bit-identical to
 * flexattn_decode with the same num_splits.  */
#define FLEXATTN_DECODE_STATIC_BYTES ((size_t)16 << 20)
int flexattn_decode_static(const FlexAttnParams* p, const void* q, const void* k, const void* v,
                           void* o, float* lse2, int32_t num_splits, flexattn_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FLEXATTN_H_ */
