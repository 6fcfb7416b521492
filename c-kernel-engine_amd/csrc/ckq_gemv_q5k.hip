/* ckq_gemv_q5k.hip - the weight-streaming kernel instantiated for FmtQ5K. */
#include "ckq_gemv.hpp"

int ckq_gemv_launch_q5k(const GemvArgs &a, const GemvGroup &grp, hipStream_t s) { return launch_fmt<FmtQ5K>(a, grp, 8, s); }
