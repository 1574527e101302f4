// gemv_kernel instantiations for Q8_0 (one translation unit per weight type keeps
// the device compile parallel).
#include "gemv_launch.hip.h"

bool cera_gemv_launch_q8_0(const GemvArgs& a, const GemvPlan& p, int epi, bool dbg, hipStream_t s) {
    return gemv_launch_t<Q8_0>(a, p, epi, dbg, s);
}
