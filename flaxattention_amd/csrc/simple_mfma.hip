// Simple matrix-core kernels (float32 at D 64 / 128, fp16 / bf16 at D 192 / 256): checks and dispatch.  The kernels
// are in simple_mfma.cuh, instantiated per (dtype, head size) by simple_mfma_inst.hip.
#include "simple_mfma.cuh"

using namespace flex;
void flex_set_error(const char* fmt, ...);
int flex_cu_count();
int flex_simple_f32_64(const FlexAttnParams& p, const SimpleArgs& a);
int flex_simple_f32_128(const FlexAttnParams& p, const SimpleArgs& a);
int flex_simple_f16_192(const FlexAttnParams& p, const SimpleArgs& a);
int flex_simple_f16_256(const FlexAttnParams& p, const SimpleArgs& a);
int flex_simple_bf16_192(const FlexAttnParams& p, const SimpleArgs& a);
int flex_simple_bf16_256(const FlexAttnParams& p, const SimpleArgs& a);

// the (dtype, head size) pairs these kernels are instantiated for
bool flex_simple_shape(int dtype, int D, int Dv) {
  if (D != Dv) return false;
  if (dtype == FLEX_F32) return D == 64 || D == 128;
  if (dtype == FLEX_F16 || dtype == FLEX_BF16) return D == 192 || D == 256;
  return false;
}

static bool strides_ok(const int64_t* s, int epc) { return s[0] % epc == 0 && s[1] % epc == 0 && s[2] % epc == 0; }
static bool lists_ok(const FlexTileLists& t, int kv_block) {
  return !t.kv_num || (t.q_block == kSimpleQTile && t.kv_block == kv_block);
}

// which: 0 = forward, 1 = backward
bool flex_simple_supported(const FlexAttnParams& p, int which) {
  if (!flex_simple_shape(p.dtype, p.D, p.Dv)) return false;
  if (p.flags & FLEX_UNROUNDED) {
    if (p.dtype != FLEX_F32) return false;  // high / low parts are not built here; float32 rounds nothing anyway
  }
  if (p.score.kind == FLEX_SCORE_AFFINE && !p.score.mul && !p.score.add) return false;
  const int epc = p.dtype == FLEX_F32 ? 4 : 8;  // rows are read in 16-byte chunks
  if (!strides_ok(p.q_stride, epc) || !strides_ok(p.k_stride, epc) || !strides_ok(p.v_stride, epc) || !strides_ok(p.o_stride, epc))
    return false;
  if ((int64_t)((p.Lq + kSimpleQTile - 1) / kSimpleQTile) * p.Hq * p.B > 0x7fffffff) return false;
  return which == 0 ? lists_ok(p.tiles, 64) : lists_ok(p.tiles_bwd, kSimpleKvTile);
}

static int dispatch(const FlexAttnParams& p, const SimpleArgs& a) {
  int rc = 1;
  if (p.dtype == FLEX_F32) rc = p.D == 64 ? flex_simple_f32_64(p, a) : flex_simple_f32_128(p, a);
  else if (p.dtype == FLEX_F16) rc = p.D == 192 ? flex_simple_f16_192(p, a) : flex_simple_f16_256(p, a);
  else rc = p.D == 192 ? flex_simple_bf16_192(p, a) : flex_simple_bf16_256(p, a);
  if (rc) flex_set_error("simple matrix-core kernels: unsupported score_mod kind %d", p.score.kind);
  return rc;
}

// Shares of the key steps a forward call is split into (1 = none): calls whose query tiles alone would leave most
// compute units without a workgroup -- few rows against a long key sequence -- are split until there is about one
// workgroup per compute unit, with at least 16 steps of 32 keys each.
int flex_simple_fwd_splits(const FlexAttnParams& p) {
  const int64_t wgs = (int64_t)((p.Lq + kSimpleQTile - 1) / kSimpleQTile) * p.Hq * p.B;
  const int cus = flex_cu_count();
  if (wgs > cus / 2) return 1;
  const int steps = (p.Lkv + kSimpleStep - 1) / kSimpleStep;
  int s = (int)(cus / wgs);
  if (s > steps / 16) s = steps / 16;
  if (s > 64) s = 64;  // the merge kernel takes one split per lane
  return s < 2 ? 1 : s;
}
// bytes of the partial (O, m, l) of a split forward
size_t flex_simple_fwd_partial_bytes(const FlexAttnParams& p, int splits) {
  if (splits <= 1) return 0;
  return ((size_t)p.B * p.Hq * p.Lq * splits * (p.D + 2) * sizeof(float) + 255) / 256 * 256;
}

// partials: nullptr for one pass over all keys, else flex_simple_fwd_partial_bytes(p, splits) bytes
int flex_simple_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                    void* partials, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15) {
    flex_set_error("matrix-core forward needs 16-byte aligned tensors");
    return 1;
  }
  if ((p.flags & FLEX_PARITY) && p.dtype != FLEX_F32 && !lse2) {
    flex_set_error("matrix-core forward: the parity numerics need a log-sum-exp buffer (lse2 or workspace)");
    return 1;
  }
  SimpleArgs a = {};
  a.q = q; a.k = k; a.v = v; a.out = o; a.lse2_out = lse2; a.s = s; a.bwd = false;
  a.splits = 1;
  if (splits > 1 && partials) {
    if ((uintptr_t)partials & 15) {
      flex_set_error("matrix-core forward needs a 16-byte aligned workspace");
      return 1;
    }
    a.splits = splits;
    a.o_part = (float*)partials;
    a.ml_part = a.o_part + (size_t)p.B * p.Hq * p.Lq * splits * p.D;
  }
  return dispatch(p, a);
}

int flex_simple_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const void* o, const float* lse2,
                    const void* d_o, void* dq, void* dk, void* dv, void* workspace, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)d_o | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) & 15) {
    flex_set_error("matrix-core backward needs 16-byte aligned tensors");
    return 1;
  }
  SimpleArgs a = {};
  a.q = q; a.k = k; a.v = v; a.o = o; a.d_o = d_o; a.lse2_in = lse2;
  a.dq = dq; a.dk = dk; a.dv = dv; a.delta = (float*)workspace; a.s = s; a.bwd = true;
  return dispatch(p, a);
}
