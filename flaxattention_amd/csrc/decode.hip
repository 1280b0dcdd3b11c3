// Split-KV decode for gfx950: short queries (G * Lq <= 64 columns; 32 at D = 192 / 256) against a
// long KV cache, bound by HBM bandwidth.
//
// Serves the decode shapes of examples/benchmark_decoding.py:29-33 (the
// reference pads q to 16 rows and runs its prefill kernel, attention.py:269-273).
//
// Grid: (splits, Hkv, B).  A workgroup owns a contiguous range of 32-row KV
// steps; its four waves take steps round-robin and never synchronise with each
// other until the end, so many independent 8 KB K/V reads are in flight per CU.
// Per step and wave:
//   K rows go straight from global memory into MFMA A-operand registers
//   (lane i holds 16-byte pieces of row kv0 + i%32) -- no LDS round trip;
//   V rows are fetched global -> LDS directly into one of two wave-private strips
//   (unpadded, swizzled) and read back transposed; with more than 32 columns at D = 128
//   the Q fragments are re-read from LDS every step.
//   All query heads that share a KV head (GQA) are packed into the N columns of
//   the MFMA, so K and V are read once per group.
// Each workgroup writes an unnormalised partial (O, m, l) per column; a second
// kernel merges the splits:  O = sum_s 2^(m_s-m) O_s / sum_s 2^(m_s-m) l_s.
#include <mutex>
#include "decode.cuh"

// Split-KV partials of flexattn_decode_static: every GPU the library runs on holds its own copy of
// this array, at its own address, until the process ends.  Host code never uses the array's name as
// an address; flex_decode_static_scratch() asks the runtime for the device address once per device.
constexpr size_t kStaticScratchBytes = FLEXATTN_DECODE_STATIC_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

using namespace flex;
int flex_decode_f16_64(const FlexAttnParams& p, const DecodeArgs& a);
int flex_decode_f16_128(const FlexAttnParams& p, const DecodeArgs& a);
int flex_decode_bf16_64(const FlexAttnParams& p, const DecodeArgs& a);
int flex_decode_bf16_128(const FlexAttnParams& p, const DecodeArgs& a);
int flex_decode_f16_192(const FlexAttnParams& p, const DecodeArgs& a);
int flex_decode_bf16_192(const FlexAttnParams& p, const DecodeArgs& a);
int flex_decode_f16_256(const FlexAttnParams& p, const DecodeArgs& a);
int flex_decode_bf16_256(const FlexAttnParams& p, const DecodeArgs& a);
void flex_set_error(const char* fmt, ...);
int flex_cu_count();
bool flex_mfma_shape_ok(const FlexAttnParams& p);

// 16-bit inputs, D = Dv in {64, 128} with up to 64 query columns (rows x heads per KV head) or D = Dv in {192, 256}
// with up to 32
bool flex_decode_supported(const FlexAttnParams& p) {
  if (p.score.kind == FLEX_SCORE_AFFINE) return false;
  int max_cols = 64;
  if (p.D == p.Dv && (p.D == 192 || p.D == 256)) {
    FlexAttnParams as128 = p;  // dtype, stride and grid checks are those of the narrower heads
    as128.D = as128.Dv = 128;
    if (!flex_mfma_shape_ok(as128)) return false;
    max_cols = 32;
  } else if (!flex_mfma_shape_ok(p)) {
    return false;
  }
  return (int64_t)(p.Hq / p.Hkv) * p.Lq <= max_cols && p.Hkv <= 65535 && p.B <= 65535;
}

int flex_decode_default_splits(const FlexAttnParams& p) {
  // ONE workgroup per compute unit: a bandwidth-bound kernel gains nothing from more, and every further split adds
  // partials to write and merge (fp16 KV cache [8,8,16384,64] at q_len 1: 53 us with 4 splits = 256 workgroups, 54 us with 8, 58 us with
  // 16; at q_len 64: 56 us with 4, 60 us with 8).  At least 8 steps each.
  const int steps = (p.Lkv + kStep - 1) / kStep;
  int64_t heads = (int64_t)p.B * p.Hkv;
  const int slots = flex_cu_count();
  int s = (int)((slots + heads - 1) / heads);
  if (s > steps / 8) s = steps / 8;
  if (s < 1) s = 1;
  if (s > 64) s = 64;
  return s;
}

// partial outputs and (m, l) per split; the parity numerics add one float per row for the merged log-sum-exp
// that the second pass reads (used when the caller passes no lse2)
size_t flex_decode_workspace(const FlexAttnParams& p, int splits) {
  const size_t rows = (size_t)p.B * p.Hq * p.Lq;
  const size_t lse = (p.flags & FLEX_PARITY) ? rows : 0;
  return ((rows * splits * (p.D + 2) + lse) * sizeof(float) + 255) / 256 * 256;
}

// Device address of this file's scratch array on the current device, looked up once per device
// (hipGetSymbolAddress neither allocates nor frees).  Returns nullptr with the error set on failure.
void* flex_decode_static_scratch(size_t* bytes) {
  constexpr int kMaxDev = 64;
  static std::mutex mu;
  static void* ptr_of[kMaxDev] = {};
  *bytes = kStaticScratchBytes;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDev) {
    flex_set_error("decode (static scratch): no usable current device (%s)", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr_of[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      flex_set_error("decode (static scratch): hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    ptr_of[dev] = ptr;
  }
  return ptr_of[dev];
}

int flex_decode_launch(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                       void* workspace, hipStream_t s) {
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)workspace) & 15) {
    flex_set_error("decode needs 16-byte aligned tensors");
    return 1;
  }
  if (splits > 64) { flex_set_error("decode: at most 64 splits (got %d)", splits); return 1; }
  const size_t rows = (size_t)p.B * p.Hq * p.Lq;
  float* o_part = (float*)workspace;
  float* ml_part = o_part + rows * splits * p.D;
  float* lse_ws = ml_part + rows * splits * 2;
  const DecodeArgs a = {q, k, v, o, lse2, lse2 ? lse2 : lse_ws, o_part, ml_part, splits, s};
  int rc;
  if (p.dtype == FLEX_F16)
    rc = p.D == 64 ? flex_decode_f16_64(p, a) : p.D == 128 ? flex_decode_f16_128(p, a) : p.D == 192 ? flex_decode_f16_192(p, a) : flex_decode_f16_256(p, a);
  else
    rc = p.D == 64 ? flex_decode_bf16_64(p, a) : p.D == 128 ? flex_decode_bf16_128(p, a) : p.D == 192 ? flex_decode_bf16_192(p, a) : flex_decode_bf16_256(p, a);
  if (rc) flex_set_error("decode: unsupported score_mod kind %d", p.score.kind);
  return rc;
}
