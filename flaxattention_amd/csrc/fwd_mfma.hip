#include "flex_common.cuh"
void flex_set_error(const char* fmt, ...);
bool flex_mfma_fwd_supported(const FlexAttnParams& p) { return false; }
int flex_mfma_fwd(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, hipStream_t s) { flex_set_error("mfma fwd not built"); return 3; }
void flex_mfma_tiles(int dtype, int D, int Dv, int* qb, int* kvb) { *qb = 0; *kvb = 0; }
