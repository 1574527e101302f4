// gemv_kernel instantiations for Q6K (one translation unit per weight type keeps
// the device compile parallel).
#include "gemv_launch.hip.h"

bool cera_gemv_launch_q6k(const GemvArgs& a, const GemvPlan& p, int epi, bool dbg, hipStream_t s) {
    return gemv_launch_t<Q6K>(a, p, epi, dbg, s);
}
