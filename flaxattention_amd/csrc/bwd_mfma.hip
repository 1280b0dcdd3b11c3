// Fused flash-attention backward for gfx950 (fp16 / bf16, D = Dv in {64, 128}; dQ also at 192 / 256): checks and dispatch.  The kernels are
// in bwd_mfma.cuh, instantiated per (dtype, head size) by bwd_mfma_inst.hip.
#include "bwd_mfma.cuh"

using namespace flex;
void flex_set_error(const char* fmt, ...);
bool flex_mfma_shape_ok(const FlexAttnParams& p);
int flex_mfma_bwd_f16_64(const FlexAttnParams& p, const BwdArgs& a);
int flex_mfma_bwd_f16_128(const FlexAttnParams& p, const BwdArgs& a);
int flex_mfma_bwd_bf16_64(const FlexAttnParams& p, const BwdArgs& a);
int flex_mfma_bwd_bf16_128(const FlexAttnParams& p, const BwdArgs& a);
int flex_mfma_bwd_f16_192(const FlexAttnParams& p, const BwdArgs& a);   // dQ kernels only
int flex_mfma_bwd_bf16_192(const FlexAttnParams& p, const BwdArgs& a);  // dQ kernels only
int flex_mfma_bwd_f16_256(const FlexAttnParams& p, const BwdArgs& a);   // dQ kernels only
int flex_mfma_bwd_bf16_256(const FlexAttnParams& p, const BwdArgs& a);  // dQ kernels only

// 192- and 256-wide heads: the dQ kernel (and its row sweep) is instantiated, the dK/dV kernel is not.  A backward call
// at those sizes is served by flex_mfma_bwd with FLEX_BWD_ONLY_DQ set and the dK/dV kernel of the simple family.
bool flex_mfma_dq_wide_supported(const FlexAttnParams& p) {
  if (p.D != p.Dv || (p.D != 192 && p.D != 256) || (p.flags & FLEX_UNROUNDED)) return false;
  FlexAttnParams as128 = p;  // everything but the head size is checked as for 128
  as128.D = as128.Dv = 128;
  if (!flex_mfma_shape_ok(as128)) return false;
  const FlexTileLists& t = p.tiles_bwd;
  return !t.kv_num || (t.q_block == kBM && t.kv_block == kListBN);
}

bool flex_mfma_bwd_supported(const FlexAttnParams& p) {
  if (!flex_mfma_shape_ok(p)) return false;
  // the dK/dV kernel needs the transposed lists whenever lists are given
  const FlexTileLists& t = p.tiles_bwd;
  if (t.kv_num && (t.q_block != kBM || t.kv_block != kListBN)) return false;
  if (t.kv_num && (!t.q_num || !t.q_idx || !t.full_q_num || !t.full_q_idx)) return false;
  return true;
}

size_t flex_mfma_bwd_workspace(const FlexAttnParams& p) { return 0; }  // delta is accounted for by the caller

int flex_mfma_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const void* o, const float* lse2,
                  const void* d_o, void* dq, void* dk, void* dv, void* workspace, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)d_o | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) & 15) {
    flex_set_error("fused backward needs 16-byte aligned tensors");
    return 1;
  }
  const BwdArgs a = {q, k, v, o, d_o, lse2, dq, dk, dv, (float*)workspace, s};
  int rc;
  if (p.D >= 192 && !(p.flags & FLEX_BWD_ONLY_DQ)) {
    flex_set_error("fused backward: only the dQ kernel exists for 192- and 256-wide heads");
    return 1;
  }
  if (p.dtype == FLEX_F16)
    rc = p.D == 64 ? flex_mfma_bwd_f16_64(p, a) : p.D == 128 ? flex_mfma_bwd_f16_128(p, a) : p.D == 192 ? flex_mfma_bwd_f16_192(p, a) : flex_mfma_bwd_f16_256(p, a);
  else
    rc = p.D == 64 ? flex_mfma_bwd_bf16_64(p, a) : p.D == 128 ? flex_mfma_bwd_bf16_128(p, a) : p.D == 192 ? flex_mfma_bwd_bf16_192(p, a) : flex_mfma_bwd_bf16_256(p, a);
  if (rc == 1) flex_set_error("fused backward: unsupported score_mod kind %d", p.score.kind);
  if (rc == 2) flex_set_error("fused backward: could not raise the dynamic LDS limit");
  return rc;
}
