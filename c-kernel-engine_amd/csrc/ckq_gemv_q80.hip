/* ckq_gemv_q80.hip - the weight-streaming kernel instantiated for FmtQ80. */
#include "ckq_gemv.hpp"

int ckq_gemv_launch_q80(const GemvArgs &a, const GemvGroup &grp, hipStream_t s) { return launch_fmt<FmtQ80>(a, grp, 8, s); }
