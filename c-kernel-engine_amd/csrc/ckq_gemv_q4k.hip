/* ckq_gemv_q4k.hip - the weight-streaming kernel instantiated for FmtQ4K. */
#include "ckq_gemv.hpp"

int ckq_gemv_launch_q4k(const GemvArgs &a, const GemvGroup &grp, hipStream_t s) { return launch_fmt<FmtQ4K>(a, grp, 8, s); }
