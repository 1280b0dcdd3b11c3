#include "flex_common.cuh"
void flex_set_error(const char* fmt, ...);
bool flex_mfma_bwd_supported(const FlexAttnParams& p) { return false; }
size_t flex_mfma_bwd_workspace(const FlexAttnParams& p) { return 0; }
int flex_mfma_bwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, const void* o, const float* lse2,
                  const void* d_o, void* dq, void* dk, void* dv, void* workspace, hipStream_t s) { flex_set_error("mfma bwd not built"); return 3; }
