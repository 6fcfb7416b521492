/* ckq_gemv_q80p.hip - the weight-streaming kernel instantiated for FmtQ80P. */
#include "ckq_gemv.hpp"

int ckq_gemv_launch_q80p(const GemvArgs &a, const GemvGroup &grp, hipStream_t s) { return launch_fmt<FmtQ80P>(a, grp, 8, s); }
