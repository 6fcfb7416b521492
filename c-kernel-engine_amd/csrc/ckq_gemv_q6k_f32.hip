/* ckq_gemv_q6k_f32.hip - the weight-streaming kernel instantiated for FmtQ6KF32. */
#include "ckq_gemv.hpp"

int ckq_gemv_launch_q6k_f32(const GemvArgs &a, const GemvGroup &grp, hipStream_t s) { return launch_fmt<FmtQ6KF32>(a, grp, 1, s); }
