// XLA-FFI adapter: the four entry points of include/flexattn.h as typed XLA custom-call handlers, so that the
// reference's JAX front-end can call libflexattn.so through jax.ffi.ffi_call in place of its Pallas kernels
// (flaxattention/kernel/attention.py:243-257 forward, :321-334 forward with residuals, :612-647 backward;
// flaxattention/core/blockmask.py:419-455 block-mask builder).
//
// Build (on a machine that has JAX; the XLA headers ship inside jaxlib):
//     make -C flaxattention_amd/csrc ffi XLA_INCLUDE=$(python -c "import jax.ffi; print(jax.ffi.include_dir())")
// Without the XLA headers this translation unit is empty: everything below is behind __has_include.
//
// Conventions shared by the handlers
//   * buffers are dense row-major [B,H,L,D] device arrays, as XLA hands them over; the stream is XLA's;
//   * an operand that does not apply is passed as a ZERO-ELEMENT buffer (XLA has no optional operands):
//     no tile lists, no bitmap mask, no query-packed copy, no block classes, no score tables, no d_lse2;
//   * tile lists arrive as ONE int32 buffer per granularity holding the eight arrays of a BlockMask back to back
//     (kv_num [lb,lh,nq], kv_idx [lb,lh,nq,nkv], full_kv_num, full_kv_idx, q_num [lb,lh,nkv], q_idx [lb,lh,nkv,nq],
//     full_q_num, full_q_idx), which is what FlexBlockMaskBuild returns; lb / lh are 1 (broadcast) or B / Hq;
//   * scalars (scale, flags, functor parameters, list geometry) are attributes, read from the dictionary;
//   * scratch is declared as an extra result, so XLA allocates it and nothing here does.
#if defined(__has_include)
#if __has_include("xla/ffi/api/ffi.h")
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "../../include/flexattn.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

ffi::Error Fail(const char* who) {
  return ffi::Error(ffi::ErrorCode::kInternal, std::string(who) + ": " + flexattn_last_error());
}

int DTypeOf(ffi::DataType t) {
  switch (t) {
    case ffi::DataType::F16: return FLEX_F16;
    case ffi::DataType::BF16: return FLEX_BF16;
    default: return FLEX_F32;
  }
}

template <typename T> T Get(const ffi::Dictionary& a, const char* name, T fallback) {
  auto v = a.get<T>(name);
  return v.has_value() ? *v : fallback;
}

void Dense(int64_t* s, int64_t H, int64_t L, int64_t D) { s[0] = H * L * D; s[1] = L * D; s[2] = D; }

// One packed list buffer -> FlexTileLists (see the conventions above).  geometry attributes: <prefix>_q_block,
// <prefix>_kv_block, <prefix>_nq, <prefix>_nkv, <prefix>_b, <prefix>_h.
void Lists(FlexTileLists* t, const ffi::AnyBuffer& buf, const ffi::Dictionary& a, const std::string& prefix) {
  *t = FlexTileLists{};
  if (buf.element_count() == 0) return;
  const int32_t nq = Get<int32_t>(a, (prefix + "_nq").c_str(), 0), nkv = Get<int32_t>(a, (prefix + "_nkv").c_str(), 0);
  const int64_t lb = Get<int32_t>(a, (prefix + "_b").c_str(), 1), lh = Get<int32_t>(a, (prefix + "_h").c_str(), 1);
  const int32_t* p = static_cast<const int32_t*>(buf.untyped_data());
  const int64_t rows_q = lb * lh * nq, rows_kv = lb * lh * nkv;
  t->kv_num = p;                p += rows_q;
  t->kv_idx = p;                p += rows_q * nkv;
  t->full_kv_num = p;           p += rows_q;
  t->full_kv_idx = p;           p += rows_q * nkv;
  t->q_num = p;                 p += rows_kv;
  t->q_idx = p;                 p += rows_kv * nq;
  t->full_q_num = p;            p += rows_kv;
  t->full_q_idx = p;
  t->q_block = Get<int32_t>(a, (prefix + "_q_block").c_str(), 0);
  t->kv_block = Get<int32_t>(a, (prefix + "_kv_block").c_str(), 0);
  t->n_q_blocks = nq;
  t->n_kv_blocks = nkv;
  t->stride_b = lb == 1 ? 0 : lh;
  t->stride_h = lh == 1 ? 0 : 1;
}

// mask functor: band parameters from attributes; a non-empty `bits` makes it a bitmap [Bm,Hm,Qp,W] (int32 words),
// with the optional query-packed copy [Bm,Hm,KVp,Wq] and block classes [Bm,Hm,Qp/32,KVp/32] (int8)
void Mask(FlexMask* m, const ffi::Dictionary& a, const ffi::AnyBuffer& bits, const ffi::AnyBuffer* bits_t,
          const ffi::AnyBuffer* blk) {
  *m = FlexMask{};
  m->kind = FLEX_MASK_BAND;
  m->lo = Get<int32_t>(a, "mask_lo", INT32_MIN);
  m->hi = Get<int32_t>(a, "mask_hi", INT32_MAX);
  m->sink = Get<int32_t>(a, "mask_sink", -1);
  m->q_offset = Get<int32_t>(a, "mask_q_offset", 0);
  if (bits.element_count() == 0) return;
  auto d = bits.dimensions();
  m->kind = FLEX_MASK_BITS;
  m->bits = static_cast<const uint32_t*>(bits.untyped_data());
  m->bits_stride_b = d[0] == 1 ? 0 : d[1] * d[2] * d[3];
  m->bits_stride_h = d[1] == 1 ? 0 : d[2] * d[3];
  m->bits_stride_q = d[3];
  if (bits_t && bits_t->element_count() != 0) {
    auto t = bits_t->dimensions();
    m->bits_t = static_cast<const uint32_t*>(bits_t->untyped_data());
    m->bits_t_stride_b = t[0] == 1 ? 0 : t[1] * t[2] * t[3];
    m->bits_t_stride_h = t[1] == 1 ? 0 : t[2] * t[3];
    m->bits_t_stride_kv = t[3];
  }
  if (blk && blk->element_count() != 0) {
    auto c = blk->dimensions();
    m->blk = static_cast<const int8_t*>(blk->untyped_data());
    m->blk_stride_b = c[0] == 1 ? 0 : c[1] * c[2] * c[3];
    m->blk_stride_h = c[1] == 1 ? 0 : c[2] * c[3];
    m->blk_stride_q = c[3];
  }
}

// score functor: closed-form families from attributes; non-empty fp32 tables [b',h',q',Lkv] (extents 1 broadcast)
// make it FLEX_SCORE_AFFINE
void ScoreClosedForm(FlexScoreMod* s, const ffi::Dictionary& a) {
  *s = FlexScoreMod{};
  s->kind = Get<int32_t>(a, "score_kind", FLEX_SCORE_IDENTITY);
  s->p0 = Get<float>(a, "score_p0", 0.f);
  s->p1 = Get<float>(a, "score_p1", 0.f);
  s->i0 = Get<int32_t>(a, "score_i0", 0);
}
void Score(FlexScoreMod* s, const ffi::Dictionary& a, const ffi::AnyBuffer& add, const ffi::AnyBuffer& mul) {
  ScoreClosedForm(s, a);
  const ffi::AnyBuffer* tab = add.element_count() ? &add : (mul.element_count() ? &mul : nullptr);
  if (!tab) return;
  auto d = tab->dimensions();
  s->kind = FLEX_SCORE_AFFINE;
  s->add = add.element_count() ? static_cast<const float*>(add.untyped_data()) : nullptr;
  s->mul = mul.element_count() ? static_cast<const float*>(mul.untyped_data()) : nullptr;
  s->stride_b = d[0] == 1 ? 0 : d[1] * d[2] * d[3];
  s->stride_h = d[1] == 1 ? 0 : d[2] * d[3];
  s->stride_q = d[2] == 1 ? 0 : d[3];
}

void Problem(FlexAttnParams* p, const ffi::AnyBuffer& q, const ffi::AnyBuffer& k, const ffi::AnyBuffer& v,
             const ffi::Dictionary& a) {
  *p = FlexAttnParams{};
  auto qd = q.dimensions(), kd = k.dimensions(), vd = v.dimensions();
  p->dtype = DTypeOf(q.element_type());
  p->B = (int32_t)qd[0]; p->Hq = (int32_t)qd[1]; p->Lq = (int32_t)qd[2]; p->D = (int32_t)qd[3];
  p->Hkv = (int32_t)kd[1]; p->Lkv = (int32_t)kd[2]; p->Dv = (int32_t)vd[3];
  Dense(p->q_stride, p->Hq, p->Lq, p->D);
  Dense(p->k_stride, p->Hkv, p->Lkv, p->D);
  Dense(p->v_stride, p->Hkv, p->Lkv, p->Dv);
  Dense(p->o_stride, p->Hq, p->Lq, p->Dv);
  p->scale = Get<float>(a, "scale", 1.f);
  p->flags = Get<int32_t>(a, "flags", FLEX_ROUND_S);
  p->q_index_base = Get<int32_t>(a, "q_index_base", 0);
}

// ---- flexattn_fwd: (q, k, v, lists, bits, bits_t, blk, score_add, score_mul) -> (o, lse2, workspace) ----
ffi::Error FwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer lists,
                   ffi::AnyBuffer bits, ffi::AnyBuffer bits_t, ffi::AnyBuffer blk, ffi::AnyBuffer score_add,
                   ffi::AnyBuffer score_mul, ffi::Result<ffi::AnyBuffer> o, ffi::Result<ffi::AnyBuffer> lse2,
                   ffi::Result<ffi::AnyBuffer> workspace, ffi::Dictionary attrs) {
  FlexAttnParams p;
  Problem(&p, q, k, v, attrs);
  Score(&p.score, attrs, score_add, score_mul);
  Mask(&p.mask, attrs, bits, &bits_t, &blk);
  Lists(&p.tiles, lists, attrs, "lists");
  if (flexattn_fwd(&p, q.untyped_data(), k.untyped_data(), v.untyped_data(), o->untyped_data(),
                   static_cast<float*>(lse2->untyped_data()), workspace->untyped_data(), stream))
    return Fail("FlexAttnFwd");
  return ffi::Error::Success();
}

// ---- flexattn_bwd: (q, k, v, o, lse2, d_o, d_lse2, lists_bwd, bits, bits_t, blk, score_add, score_mul)
//                    -> (dq, dk, dv, workspace of flexattn_bwd_workspace_bytes) ----
ffi::Error BwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer o,
                   ffi::AnyBuffer lse2, ffi::AnyBuffer d_o, ffi::AnyBuffer d_lse2, ffi::AnyBuffer lists_bwd,
                   ffi::AnyBuffer bits, ffi::AnyBuffer bits_t, ffi::AnyBuffer blk, ffi::AnyBuffer score_add,
                   ffi::AnyBuffer score_mul, ffi::Result<ffi::AnyBuffer> dq, ffi::Result<ffi::AnyBuffer> dk,
                   ffi::Result<ffi::AnyBuffer> dv, ffi::Result<ffi::AnyBuffer> workspace, ffi::Dictionary attrs) {
  FlexAttnParams p;
  Problem(&p, q, k, v, attrs);
  Score(&p.score, attrs, score_add, score_mul);
  Mask(&p.mask, attrs, bits, &bits_t, &blk);
  Lists(&p.tiles_bwd, lists_bwd, attrs, "lists_bwd");
  p.d_lse2 = d_lse2.element_count() ? static_cast<const float*>(d_lse2.untyped_data()) : nullptr;
  if (flexattn_bwd(&p, q.untyped_data(), k.untyped_data(), v.untyped_data(), o.untyped_data(),
                   static_cast<const float*>(lse2.untyped_data()), d_o.untyped_data(), dq->untyped_data(),
                   dk->untyped_data(), dv->untyped_data(), workspace->untyped_data(), stream))
    return Fail("FlexAttnBwd");
  return ffi::Error::Success();
}

// ---- flexattn_decode: (q, k, v, lists, bits, blk) -> (o, lse2, workspace of flexattn_decode_workspace_bytes) ----
ffi::Error DecodeImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer lists,
                      ffi::AnyBuffer bits, ffi::AnyBuffer blk, ffi::Result<ffi::AnyBuffer> o,
                      ffi::Result<ffi::AnyBuffer> lse2, ffi::Result<ffi::AnyBuffer> workspace, ffi::Dictionary attrs) {
  FlexAttnParams p;
  Problem(&p, q, k, v, attrs);
  ScoreClosedForm(&p.score, attrs);   // the decode kernel takes the closed-form functors only
  Mask(&p.mask, attrs, bits, nullptr, &blk);
  Lists(&p.tiles, lists, attrs, "lists");
  if (flexattn_decode(&p, q.untyped_data(), k.untyped_data(), v.untyped_data(), o->untyped_data(),
                      static_cast<float*>(lse2->untyped_data()), Get<int32_t>(attrs, "num_splits", 0),
                      workspace->untyped_data(), stream))
    return Fail("FlexAttnDecode");
  return ffi::Error::Success();
}

// ---- flexattn_block_mask_build: (bits, blk) -> (lists packed as described above, workspace) ----
// attributes: B, H, nq, nkv, q_block, kv_block and the band parameters; `bits` non-empty = a bitmap mask
ffi::Error BlockMaskImpl(hipStream_t stream, ffi::AnyBuffer bits, ffi::AnyBuffer blk, ffi::Result<ffi::AnyBuffer> lists,
                         ffi::Result<ffi::AnyBuffer> workspace, ffi::Dictionary attrs) {
  FlexMask m;
  Mask(&m, attrs, bits, nullptr, &blk);
  const int32_t B = Get<int32_t>(attrs, "B", 1), H = Get<int32_t>(attrs, "H", 1);
  const int32_t nq = Get<int32_t>(attrs, "nq", 0), nkv = Get<int32_t>(attrs, "nkv", 0);
  int32_t* p = static_cast<int32_t*>(lists->untyped_data());
  const int64_t rows_q = (int64_t)B * H * nq, rows_kv = (int64_t)B * H * nkv;
  int32_t* kv_num = p;       p += rows_q;
  int32_t* kv_idx = p;       p += rows_q * nkv;
  int32_t* full_kv_num = p;  p += rows_q;
  int32_t* full_kv_idx = p;  p += rows_q * nkv;
  int32_t* q_num = p;        p += rows_kv;
  int32_t* q_idx = p;        p += rows_kv * nq;
  int32_t* full_q_num = p;   p += rows_kv;
  int32_t* full_q_idx = p;
  if (flexattn_block_mask_build(&m, B, H, nq, nkv, Get<int32_t>(attrs, "q_block", 128), Get<int32_t>(attrs, "kv_block", 128),
                                kv_num, kv_idx, full_kv_num, full_kv_idx, q_num, q_idx, full_q_num, full_q_idx,
                                workspace->untyped_data(), stream))
    return Fail("FlexBlockMaskBuild");
  return ffi::Error::Success();
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(FlexAttnFwd, FwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()   // q
                                  .Arg<ffi::AnyBuffer>()   // k
                                  .Arg<ffi::AnyBuffer>()   // v
                                  .Arg<ffi::AnyBuffer>()   // lists (forward granularity) or empty
                                  .Arg<ffi::AnyBuffer>()   // mask bits or empty
                                  .Arg<ffi::AnyBuffer>()   // mask bits, query-packed, or empty
                                  .Arg<ffi::AnyBuffer>()   // mask block classes or empty
                                  .Arg<ffi::AnyBuffer>()   // additive score table or empty
                                  .Arg<ffi::AnyBuffer>()   // multiplicative score table or empty
                                  .Ret<ffi::AnyBuffer>()   // o
                                  .Ret<ffi::AnyBuffer>()   // lse2
                                  .Ret<ffi::AnyBuffer>()   // workspace (flexattn_fwd_workspace_bytes, at least 1 byte)
                                  .Attrs());

XLA_FFI_DEFINE_HANDLER_SYMBOL(FlexAttnBwd, BwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()   // q
                                  .Arg<ffi::AnyBuffer>()   // k
                                  .Arg<ffi::AnyBuffer>()   // v
                                  .Arg<ffi::AnyBuffer>()   // o
                                  .Arg<ffi::AnyBuffer>()   // lse2
                                  .Arg<ffi::AnyBuffer>()   // d_o
                                  .Arg<ffi::AnyBuffer>()   // d_lse2 or empty
                                  .Arg<ffi::AnyBuffer>()   // lists (backward granularity) or empty
                                  .Arg<ffi::AnyBuffer>()   // mask bits or empty
                                  .Arg<ffi::AnyBuffer>()   // mask bits, query-packed, or empty
                                  .Arg<ffi::AnyBuffer>()   // mask block classes or empty
                                  .Arg<ffi::AnyBuffer>()   // additive score table or empty
                                  .Arg<ffi::AnyBuffer>()   // multiplicative score table or empty
                                  .Ret<ffi::AnyBuffer>()   // dq
                                  .Ret<ffi::AnyBuffer>()   // dk
                                  .Ret<ffi::AnyBuffer>()   // dv
                                  .Ret<ffi::AnyBuffer>()   // workspace (flexattn_bwd_workspace_bytes)
                                  .Attrs());

XLA_FFI_DEFINE_HANDLER_SYMBOL(FlexAttnDecode, DecodeImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()   // q (at most 64 query columns)
                                  .Arg<ffi::AnyBuffer>()   // k
                                  .Arg<ffi::AnyBuffer>()   // v
                                  .Arg<ffi::AnyBuffer>()   // lists (forward granularity) or empty
                                  .Arg<ffi::AnyBuffer>()   // mask bits or empty
                                  .Arg<ffi::AnyBuffer>()   // mask block classes or empty
                                  .Ret<ffi::AnyBuffer>()   // o
                                  .Ret<ffi::AnyBuffer>()   // lse2
                                  .Ret<ffi::AnyBuffer>()   // workspace (flexattn_decode_workspace_bytes)
                                  .Attrs());

XLA_FFI_DEFINE_HANDLER_SYMBOL(FlexBlockMaskBuild, BlockMaskImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()   // mask bits or empty (band mask from attributes)
                                  .Arg<ffi::AnyBuffer>()   // mask block classes or empty
                                  .Ret<ffi::AnyBuffer>()   // the eight list arrays, packed
                                  .Ret<ffi::AnyBuffer>()   // workspace (flexattn_block_mask_workspace_bytes)
                                  .Attrs());

#endif  // __has_include("xla/ffi/api/ffi.h")
#endif  // defined(__has_include)
