// gemv_kernel instantiations for Q4K (one translation unit per weight type keeps
// the device compile parallel).
#include "gemv_launch.hip.h"

bool cera_gemv_launch_q4k(const GemvArgs& a, const GemvPlan& p, int epi, bool dbg, hipStream_t s) {
    return gemv_launch_t<Q4K>(a, p, epi, dbg, s);
}
