// gemv_kernel instantiations for Q4_1 (one translation unit per weight type keeps
// the device compile parallel).
#include "gemv_launch.hip.h"

bool cera_gemv_launch_q4_1(const GemvArgs& a, const GemvPlan& p, int epi, bool dbg, hipStream_t s) {
    return gemv_launch_t<Q4_1>(a, p, epi, dbg, s);
}
