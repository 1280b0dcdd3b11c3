// extern "C" entry points: validation, dispatch, error reporting.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include "flex_common.cuh"

static thread_local char g_err[512] = "";

void flex_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// Compute units of the current device, asked once per device (the split heuristics size their grids by it).  Without
// a usable device -- a size query on a machine that only builds -- the answer is the MI355X's 256.
int flex_cu_count() {
  constexpr int kMaxDev = 64, kDefault = 256;
  static std::mutex mu;
  static int cus_of[kMaxDev] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) {
    (void)hipGetLastError();
    return kDefault;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!cus_of[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = kDefault;
    }
    cus_of[dev] = n;
  }
  return cus_of[dev];
}

// implemented in the kernel translation units
int flex_generic_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, hipStream_t s);
int flex_generic_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const float* lse2, const void* d_o,
                     void* dq, void* dk, void* dv, float* delta, hipStream_t s);
bool flex_mfma_fwd_supported(const FlexAttnParams& p);
int flex_mfma_fwd_splits(const FlexAttnParams& p);
size_t flex_mfma_fwd_partial_bytes(const FlexAttnParams& p, int splits);
int flex_mfma_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                  void* partials, hipStream_t s);
bool flex_mfma_bwd_supported(const FlexAttnParams& p);
bool flex_mfma_dq_wide_supported(const FlexAttnParams& p);
size_t flex_mfma_bwd_workspace(const FlexAttnParams& p);
int flex_mfma_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const void* o, const float* lse2,
                  const void* d_o, void* dq, void* dk, void* dv, void* workspace, hipStream_t s);
bool flex_decode_supported(const FlexAttnParams& p);
int flex_decode_default_splits(const FlexAttnParams& p);
size_t flex_decode_workspace(const FlexAttnParams& p, int splits);
int flex_decode_launch(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                       void* workspace, hipStream_t s);
void* flex_decode_static_scratch(size_t* bytes);
void flex_mfma_tiles(int dtype, int D, int Dv, int which, int* qb, int* kvb);
bool flex_simple_supported(const FlexAttnParams& p, int which);
int flex_simple_fwd_splits(const FlexAttnParams& p);
size_t flex_simple_fwd_partial_bytes(const FlexAttnParams& p, int splits);
int flex_simple_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                    void* partials, hipStream_t s);
int flex_simple_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const void* o, const float* lse2,
                    const void* d_o, void* dq, void* dk, void* dv, void* workspace, hipStream_t s);

static int validate(const FlexAttnParams* p, const char* who) {
  if (!p) { flex_set_error("%s: null params", who); return 1; }
  if (p->dtype < FLEX_F32 || p->dtype > FLEX_BF16) { flex_set_error("%s: unknown dtype %d", who, p->dtype); return 1; }
  if (p->B <= 0 || p->Hq <= 0 || p->Hkv <= 0 || p->Lq <= 0 || p->Lkv <= 0 || p->D <= 0 || p->Dv <= 0) {
    flex_set_error("%s: non-positive size B=%d Hq=%d Hkv=%d Lq=%d Lkv=%d D=%d Dv=%d", who, p->B, p->Hq, p->Hkv, p->Lq, p->Lkv, p->D, p->Dv);
    return 1;
  }
  if (p->Hq % p->Hkv != 0) { flex_set_error("%s: Hq=%d is not a multiple of Hkv=%d", who, p->Hq, p->Hkv); return 1; }
  if (p->Dv > p->D) { flex_set_error("%s: Dv=%d must be <= D=%d", who, p->Dv, p->D); return 1; }
  if (p->score.kind < FLEX_SCORE_IDENTITY || p->score.kind > FLEX_SCORE_AFFINE) { flex_set_error("%s: unknown score_mod kind %d", who, p->score.kind); return 1; }
  if (p->score.kind == FLEX_SCORE_ALIBI && p->score.i0 <= 0) { flex_set_error("%s: ALiBi needs the head count in i0", who); return 1; }
  if (p->score.kind == FLEX_SCORE_TANH_SOFTCAP && !(p->score.p0 > 0.f)) { flex_set_error("%s: tanh soft-cap needs cap > 0", who); return 1; }
  if (p->score.kind == FLEX_SCORE_AFFINE && !p->score.mul && !p->score.add) { flex_set_error("%s: affine score_mod without tables", who); return 1; }
  if (p->mask.kind != FLEX_MASK_BAND && p->mask.kind != FLEX_MASK_BITS) { flex_set_error("%s: unknown mask kind %d", who, p->mask.kind); return 1; }
  if (p->mask.kind == FLEX_MASK_BITS && !p->mask.bits) { flex_set_error("%s: bitmap mask without bits", who); return 1; }
  const FlexTileLists* both[2] = {&p->tiles, &p->tiles_bwd};
  for (int i = 0; i < 2; i++) {
    const FlexTileLists& t = *both[i];
    if (!t.kv_num) continue;
    if (!t.kv_idx || !t.full_kv_num || !t.full_kv_idx) { flex_set_error("%s: tile lists need kv_idx, full_kv_num and full_kv_idx", who); return 1; }
    if (t.q_block <= 0 || t.kv_block <= 0 || (int64_t)t.n_q_blocks * t.q_block < (int64_t)p->Lq + p->q_index_base || (int64_t)t.n_kv_blocks * t.kv_block < p->Lkv) {
      flex_set_error("%s: tile lists (%d x %d blocks of %d x %d) do not cover Lq=%d, Lkv=%d", who, t.n_q_blocks, t.n_kv_blocks, t.q_block, t.kv_block, p->Lq, p->Lkv);
      return 1;
    }
  }
  return 0;
}

static int check_launch(const char* who) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { flex_set_error("%s: kernel launch failed: %s", who, hipGetErrorString(e)); return 2; }
  return 0;
}

extern "C" int flexattn_abi_version(void) { return 4; }
extern "C" const char* flexattn_last_error(void) { return g_err; }

extern "C" int flexattn_preferred_tiles(int32_t dtype, int32_t D, int32_t Dv, int32_t Lq, int32_t Lkv, int32_t which, int32_t* qb, int32_t* kvb) {
  int a = 0, b = 0;
  flex_mfma_tiles(dtype, D, Dv, which, &a, &b);
  if (qb) *qb = a;
  if (kvb) *kvb = b;
  return 0;
}

// FLEX_PARITY asks for the reference's rounding points.  The fused kernels have a mode for it; where only the
// generic kernels apply, FLEX_STRICT is the same numerics.
static FlexAttnParams with_parity_resolved(const FlexAttnParams* p, bool fused) {
  FlexAttnParams r = *p;
  if (r.flags & FLEX_UNROUNDED) {
    r.flags &= ~(FLEX_PARITY | FLEX_ROUND_S | FLEX_STRICT);
    if (!fused) r.flags &= ~FLEX_UNROUNDED;   // the generic kernels round nothing unless told to
    return r;
  }
  if (r.flags & FLEX_PARITY) {
    if (fused) r.flags |= FLEX_ROUND_S;
    else r.flags = (r.flags & ~FLEX_PARITY) | FLEX_STRICT;
  }
  return r;
}
static bool wants_fused(const FlexAttnParams* p) {
  if (p->flags & FLEX_FORCE_GENERIC) return false;
  return (p->flags & FLEX_UNROUNDED) || !(p->flags & FLEX_STRICT);
}

extern "C" int flexattn_kernel_family(const FlexAttnParams* p, int32_t which) {
  if (!p || !wants_fused(p)) return FLEX_FAMILY_GENERIC;
  if (flex_simple_supported(*p, which ? 1 : 0)) return p->dtype == FLEX_F32 ? FLEX_FAMILY_MFMA_F32 : FLEX_FAMILY_MFMA_16BIT;
  if (which ? flex_mfma_bwd_supported(*p) : flex_mfma_fwd_supported(*p)) return FLEX_FAMILY_MFMA_16BIT;
  return FLEX_FAMILY_GENERIC;
}

static size_t lse_bytes(const FlexAttnParams* p) { return ((size_t)p->B * p->Hq * p->Lq * sizeof(float) + 255) / 256 * 256; }

// the two passes of the parity numerics hand the log-sum-exp over in lse2, or in the workspace when the caller wants
// no lse2; the space is reserved whenever the flag is set
static size_t fwd_lse_bytes(const FlexAttnParams* p) {
  return ((p->flags & FLEX_PARITY) && !(p->flags & FLEX_UNROUNDED)) ? lse_bytes(p) : 0;
}

extern "C" size_t flexattn_fwd_workspace_bytes(const FlexAttnParams* p) {
  if (!p) return 0;
  size_t n = fwd_lse_bytes(p);
  // the matrix-core forward kernels split the keys of a call with few query tiles over several workgroups, whose
  // partial results live here
  if (wants_fused(p) && flex_mfma_fwd_supported(*p)) n += flex_mfma_fwd_partial_bytes(*p, flex_mfma_fwd_splits(*p));
  else if (wants_fused(p) && flex_simple_supported(*p, 0)) n += flex_simple_fwd_partial_bytes(*p, flex_simple_fwd_splits(*p));
  return n;
}

extern "C" int flexattn_fwd(const FlexAttnParams* p, const void* q, const void* k, const void* v, void* o, float* lse2,
                            void* workspace, flexattn_stream_t stream) {
  if (int rc = validate(p, "flexattn_fwd")) return rc;
  if (p->q_index_base != 0) { flex_set_error("flexattn_fwd: q_index_base is for flexattn_decode only"); return 1; }
  if (!q || !k || !v || !o) { flex_set_error("flexattn_fwd: null tensor pointer"); return 1; }
  hipStream_t s = (hipStream_t)stream;
  int rc;
  // the simple matrix-core kernels: float32 inputs (the reference rounds nothing below fp32, so every numerics mode
  // but FLEX_STRICT is the same computation) and the 16-bit head sizes above 128
  if (wants_fused(p) && flex_simple_supported(*p, 0) && !flex_mfma_fwd_supported(*p)) {
    const FlexAttnParams ps = with_parity_resolved(p, true);
    if ((ps.flags & FLEX_PARITY) && p->dtype != FLEX_F32 && !lse2) {
      if (!workspace) { flex_set_error("flexattn_fwd: FLEX_PARITY needs lse2 or a workspace of flexattn_fwd_workspace_bytes()"); return 1; }
      lse2 = (float*)workspace;
    }
    // with a workspace, a call with few query tiles is split over the keys (the partials follow the log-sum-exp space)
    const int splits = workspace ? flex_simple_fwd_splits(ps) : 1;
    void* partials = splits > 1 ? (char*)workspace + fwd_lse_bytes(p) : nullptr;
    if (int rcs = flex_simple_fwd(ps, q, k, v, o, lse2, splits, partials, s)) return rcs;
    return check_launch("flexattn_fwd");
  }
  const bool fused = wants_fused(p) && flex_mfma_fwd_supported(*p);
  const FlexAttnParams pr = with_parity_resolved(p, fused);
  if (fused) {
    if ((pr.flags & FLEX_PARITY) && !lse2) {
      if (!workspace) { flex_set_error("flexattn_fwd: FLEX_PARITY needs lse2 or a workspace of flexattn_fwd_workspace_bytes()"); return 1; }
      lse2 = (float*)workspace;
    }
    // with a workspace, a call with few query tiles is split over the keys (the partials follow the log-sum-exp space)
    const int splits = workspace ? flex_mfma_fwd_splits(pr) : 1;
    void* partials = splits > 1 ? (char*)workspace + fwd_lse_bytes(p) : nullptr;
    rc = flex_mfma_fwd(pr, q, k, v, o, lse2, splits, partials, s);
  } else {
    rc = flex_generic_fwd(pr, q, k, v, o, lse2, s);
  }
  if (rc) return rc;
  return check_launch("flexattn_fwd");
}

static size_t delta_bytes(const FlexAttnParams* p) { return ((size_t)p->B * p->Hq * p->Lq * sizeof(float) + 255) / 256 * 256; }

extern "C" size_t flexattn_bwd_workspace_bytes(const FlexAttnParams* p) {
  if (!p) return 0;
  size_t n = delta_bytes(p);
  if (!(p->flags & (FLEX_FORCE_GENERIC | FLEX_STRICT)) && flex_mfma_bwd_supported(*p)) n += flex_mfma_bwd_workspace(*p);
  return n;
}

extern "C" int flexattn_bwd(const FlexAttnParams* p, const void* q, const void* k, const void* v, const void* o,
                            const float* lse2, const void* d_o, void* dq, void* dk, void* dv, void* workspace,
                            flexattn_stream_t stream) {
  if (int rc = validate(p, "flexattn_bwd")) return rc;
  if (p->q_index_base != 0) { flex_set_error("flexattn_bwd: q_index_base is for flexattn_decode only"); return 1; }
  if (!q || !k || !v || !o || !lse2 || !d_o || !dq || !dk || !dv || !workspace) { flex_set_error("flexattn_bwd: null pointer"); return 1; }
  hipStream_t s = (hipStream_t)stream;
  int rc;
  if (wants_fused(p) && flex_simple_supported(*p, 1)) {
    FlexAttnParams ps = with_parity_resolved(p, true);
    if (flex_mfma_dq_wide_supported(ps) && !(ps.flags & (FLEX_BWD_ONLY_DQ | FLEX_BWD_ONLY_DKV))) {
      // 192- and 256-wide heads: dQ (and the row sweep for delta, which the dK/dV kernel reads from the workspace) on the tuned
      // kernel, dK/dV on the simple one
      FlexAttnParams pq = ps;
      pq.flags |= FLEX_BWD_ONLY_DQ;
      if (int rcq = flex_mfma_bwd(pq, q, k, v, o, lse2, d_o, dq, dk, dv, workspace, s)) return rcq;
      ps.flags |= FLEX_BWD_ONLY_DKV;
    }
    if (int rcs = flex_simple_bwd(ps, q, k, v, o, lse2, d_o, dq, dk, dv, workspace, s)) return rcs;
    return check_launch("flexattn_bwd");
  }
  const bool fused = wants_fused(p) && flex_mfma_bwd_supported(*p);
  const FlexAttnParams pr = with_parity_resolved(p, fused);
  if (fused) rc = flex_mfma_bwd(pr, q, k, v, o, lse2, d_o, dq, dk, dv, workspace, s);
  else rc = flex_generic_bwd(pr, q, k, v, lse2, d_o, dq, dk, dv, (float*)workspace, s);
  if (rc) return rc;
  return check_launch("flexattn_bwd");
}

extern "C" size_t flexattn_decode_workspace_bytes(const FlexAttnParams* p, int32_t num_splits) {
  if (!p) return 0;
  if (num_splits <= 0) num_splits = flex_decode_default_splits(*p);
  return flex_decode_workspace(*p, num_splits);
}

static int decode_checked(const FlexAttnParams* p, const void* q, const void* k, const void* v, void* o, float* lse2,
                          int32_t num_splits, void* workspace, flexattn_stream_t stream);

extern "C" int flexattn_decode(const FlexAttnParams* p, const void* q, const void* k, const void* v, void* o, float* lse2,
                               int32_t num_splits, void* workspace, flexattn_stream_t stream) {
  if (int rc = validate(p, "flexattn_decode")) return rc;
  return decode_checked(p, q, k, v, o, lse2, num_splits, workspace, stream);
}

extern "C" int flexattn_decode_static(const FlexAttnParams* p, const void* q, const void* k, const void* v, void* o,
                                      float* lse2, int32_t num_splits, flexattn_stream_t stream) {
  if (int rc = validate(p, "flexattn_decode_static")) return rc;
  if (!flex_decode_supported(*p)) {
    flex_set_error("flexattn_decode_static: needs fp16/bf16 and D == Dv in {64,128} with at most 64 query columns or D == Dv in {192,256} with at most 32 (got dtype=%d D=%d Dv=%d Lq=%d)", p->dtype, p->D, p->Dv, p->Lq);
    return 1;
  }
  if (num_splits <= 0) num_splits = flex_decode_default_splits(*p);
  const size_t need = flex_decode_workspace(*p, num_splits);
  size_t cap = 0;
  void* ws = flex_decode_static_scratch(&cap);
  if (!ws) return 2;
  if (need > cap) {
    flex_set_error("flexattn_decode_static: %zu bytes of split-KV partials (B=%d Hq=%d Lq=%d D=%d, %d splits) exceed the "
                   "built-in scratch of %zu bytes; use flexattn_decode with a caller workspace",
                   need, p->B, p->Hq, p->Lq, p->D, num_splits, cap);
    return 1;
  }
  return decode_checked(p, q, k, v, o, lse2, num_splits, ws, stream);
}

static int decode_checked(const FlexAttnParams* p, const void* q, const void* k, const void* v, void* o, float* lse2,
                          int32_t num_splits, void* workspace, flexattn_stream_t stream) {
  if (p->flags & FLEX_UNROUNDED) { flex_set_error("flexattn_decode: FLEX_UNROUNDED is served by flexattn_fwd (the decode kernel carries P in one part)"); return 1; }
  if (p->q_index_base < 0) { flex_set_error("flexattn_decode: q_index_base must not be negative (got %d)", p->q_index_base); return 1; }
  if (!q || !k || !v || !o || !workspace) { flex_set_error("flexattn_decode: null pointer"); return 1; }
  if (!flex_decode_supported(*p)) {
    flex_set_error("flexattn_decode: needs fp16/bf16 and D == Dv in {64,128} with at most 64 query columns or D == Dv in {192,256} with at most 32 (got dtype=%d D=%d Dv=%d Lq=%d)", p->dtype, p->D, p->Dv, p->Lq);
    return 1;
  }
  if (num_splits <= 0) num_splits = flex_decode_default_splits(*p);
  int rc = flex_decode_launch(*p, q, k, v, o, lse2, num_splits, workspace, (hipStream_t)stream);
  if (rc) return rc;
  return check_launch("flexattn_decode");
}
