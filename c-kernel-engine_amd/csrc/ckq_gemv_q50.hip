/* ckq_gemv_q50.hip - the weight-streaming kernel instantiated for FmtQ50. */
#include "ckq_gemv.hpp"

int ckq_gemv_launch_q50(const GemvArgs &a, const GemvGroup &grp, hipStream_t s) { return launch_fmt<FmtQ50>(a, grp, 8, s); }
