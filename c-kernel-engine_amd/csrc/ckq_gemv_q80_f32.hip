/* ckq_gemv_q80_f32.hip - the weight-streaming kernel instantiated for FmtQ80F32. */
#include "ckq_gemv.hpp"

int ckq_gemv_launch_q80_f32(const GemvArgs &a, const GemvGroup &grp, hipStream_t s) { return launch_fmt<FmtQ80F32>(a, grp, 1, s); }
