/* ckq_gemv_q6k.hip - the weight-streaming kernel instantiated for FmtQ6K. */
#include "ckq_gemv.hpp"

int ckq_gemv_launch_q6k(const GemvArgs &a, const GemvGroup &grp, hipStream_t s) { return launch_fmt<FmtQ6K>(a, grp, 8, s); }
