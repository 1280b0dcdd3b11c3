// One (dtype, head size) instantiation of the fused forward kernels.  The Makefile compiles this file once per
// combination (FLEX_T = f16 | bf16, FLEX_D = 64 | 128 | 256, FLEX_FN = the exported launcher's name), so that the six sets
// of kernels build in parallel.
#include "fwd_mfma.cuh"

int FLEX_FN(const FlexAttnParams& p, const flex::FwdArgs& a) { return flex::launch_kind<flex::FLEX_T, FLEX_D>(p, a); }
