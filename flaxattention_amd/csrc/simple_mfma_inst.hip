// One (dtype, head size) instantiation of the simple matrix-core kernels.  The Makefile compiles this file once per
// combination (FLEX_T = f32 | f16 | bf16, FLEX_D, FLEX_FN = the exported launcher's name), so that the sets of
// kernels build in parallel.
#include "simple_mfma.cuh"

int FLEX_FN(const FlexAttnParams& p, const flex::SimpleArgs& a) { return flex::simple_launch_kind<flex::FLEX_T, FLEX_D>(p, a); }
