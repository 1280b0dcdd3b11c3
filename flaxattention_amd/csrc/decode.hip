#include "flex_common.cuh"
void flex_set_error(const char* fmt, ...);
bool flex_decode_supported(const FlexAttnParams& p) { return false; }
int flex_decode_default_splits(const FlexAttnParams& p) { return 1; }
size_t flex_decode_workspace(const FlexAttnParams& p, int splits) { return 256; }
int flex_decode_launch(const FlexAttnParams& p, const void* q, const void* k, const void* v, void* o, float* lse2, int splits,
                       void* workspace, hipStream_t s) { flex_set_error("decode not built"); return 3; }
