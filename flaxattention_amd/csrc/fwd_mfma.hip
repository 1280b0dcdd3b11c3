// Fused flash-attention forward for gfx950 (fp16 / bf16, D = Dv in {64, 128, 192, 256}): checks and dispatch.  The kernels
// are in fwd_mfma.cuh, instantiated per (dtype, head size) by fwd_mfma_inst.hip.
#include "fwd_mfma.cuh"

using namespace flex;
void flex_set_error(const char* fmt, ...);
int flex_cu_count();
int flex_mfma_fwd_f16_64(const FlexAttnParams& p, const FwdArgs& a);
int flex_mfma_fwd_f16_128(const FlexAttnParams& p, const FwdArgs& a);
int flex_mfma_fwd_bf16_64(const FlexAttnParams& p, const FwdArgs& a);
int flex_mfma_fwd_bf16_128(const FlexAttnParams& p, const FwdArgs& a);
int flex_mfma_fwd_f16_192(const FlexAttnParams& p, const FwdArgs& a);
int flex_mfma_fwd_bf16_192(const FlexAttnParams& p, const FwdArgs& a);
int flex_mfma_fwd_f16_256(const FlexAttnParams& p, const FwdArgs& a);
int flex_mfma_fwd_bf16_256(const FlexAttnParams& p, const FwdArgs& a);

// rows of 16-byte chunks; the kernels keep the offset of a row inside a tile in 32 bits
static bool strides_ok(const int64_t* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0 && s[2] >= 0 && s[2] < (1 << 24); }

// dtype / head size / layout the MFMA kernels can take at all
bool flex_mfma_shape_ok(const FlexAttnParams& p) {
  if (p.dtype != FLEX_F16 && p.dtype != FLEX_BF16) return false;
  // dense tables (additive, multiplicative or both) are read per block by the fused kernels
  if (p.score.kind == FLEX_SCORE_AFFINE && !p.score.mul && !p.score.add) return false;
  if (p.D != p.Dv || (p.D != 64 && p.D != 128)) return false;
  if (!strides_ok(p.q_stride) || !strides_ok(p.k_stride) || !strides_ok(p.v_stride) || !strides_ok(p.o_stride)) return false;
  if ((int64_t)((p.Lq + 127) / 128) * p.Hq * p.B > 0x7fffffff) return false;
  return true;
}

// which: 0 = forward and decode lists, 1 = backward lists
bool flex_simple_shape(int dtype, int D, int Dv);
void flex_mfma_tiles(int dtype, int D, int Dv, int which, int* qb, int* kvb) {
  // the simple matrix-core kernels (float32, 16-bit head sizes above 128) walk lists of the same granularity
  const bool ok = ((dtype == FLEX_F16 || dtype == FLEX_BF16) && D == Dv && (D == 64 || D == 128)) || flex_simple_shape(dtype, D, Dv);
  *qb = !ok ? 0 : 128;
  *kvb = !ok ? 0 : (which == 0 ? kFwdBN : 128);
}

bool flex_mfma_fwd_supported(const FlexAttnParams& p) {
  if (p.D == p.Dv && (p.D == 192 || p.D == 256)) {
    // the list-driven forward is also instantiated for 192- and 256-wide heads (one wave per SIMD); everything but
    // the head size is checked as for 128
    FlexAttnParams as128 = p;
    as128.D = as128.Dv = 128;
    if (!flex_mfma_shape_ok(as128)) return false;
  } else if (!flex_mfma_shape_ok(p)) {
    return false;
  }
  const FlexTileLists& t = p.tiles;
  return !t.kv_num || (t.q_block == kFwdBM && t.kv_block == kFwdBN);
}

// Shares of the key tiles a forward call is split into (1 = none): calls whose query tiles alone would leave most
// compute units without a workgroup, or with one where two fit (at most one per compute unit) -- few rows against a
// long key sequence -- are split until there are about two workgroups per compute unit, with at least 8 tiles of 64
// keys each.
int flex_mfma_fwd_splits(const FlexAttnParams& p) {
  const int64_t wgs = (int64_t)((p.Lq + kFwdBM - 1) / kFwdBM) * p.Hq * p.B;
  const int slots = (p.D >= 192 ? 1 : 2) * flex_cu_count();  // 192- and 256-wide heads run one workgroup per compute unit
  if (wgs > slots / 2) return 1;
  const int tiles = (p.Lkv + kFwdBN - 1) / kFwdBN;
  int s = (int)(slots / wgs);
  if (s > tiles / 8) s = tiles / 8;
  if (s > 64) s = 64;  // the merge kernel takes one split per lane
  return s < 2 ? 1 : s;
}
// bytes of the partial (O, m, l) of a split forward
size_t flex_mfma_fwd_partial_bytes(const FlexAttnParams& p, int splits) {
  if (splits <= 1) return 0;
  return ((size_t)p.B * p.Hq * p.Lq * splits * (p.D + 2) * sizeof(float) + 255) / 256 * 256;
}

// partials: nullptr for one pass over all keys, else flex_mfma_fwd_partial_bytes(p, splits) bytes
int flex_mfma_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                  void* partials, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15) {
    flex_set_error("fused forward needs 16-byte aligned tensors");
    return 1;
  }
  if ((p.flags & FLEX_PARITY) && !lse2) {
    flex_set_error("fused forward: the parity numerics need a log-sum-exp buffer (lse2 or workspace)");
    return 1;
  }
  FwdArgs a = {q, k, v, o, lse2, s, 1, nullptr, nullptr};
  if (splits > 1 && partials) {
    if ((uintptr_t)partials & 15) {
      flex_set_error("fused forward needs a 16-byte aligned workspace");
      return 1;
    }
    a.splits = splits;
    a.o_part = (float*)partials;
    a.ml_part = a.o_part + (size_t)p.B * p.Hq * p.Lq * splits * p.D;
  }
  int rc = 1;
  if (p.dtype == FLEX_F16)
    rc = p.D == 64 ? flex_mfma_fwd_f16_64(p, a) : p.D == 128 ? flex_mfma_fwd_f16_128(p, a) : p.D == 192 ? flex_mfma_fwd_f16_192(p, a) : flex_mfma_fwd_f16_256(p, a);
  else
    rc = p.D == 64 ? flex_mfma_fwd_bf16_64(p, a) : p.D == 128 ? flex_mfma_fwd_bf16_128(p, a) : p.D == 192 ? flex_mfma_fwd_bf16_192(p, a) : flex_mfma_fwd_bf16_256(p, a);
  if (rc) flex_set_error("fused forward: unsupported score_mod kind %d", p.score.kind);
  return rc;
}
