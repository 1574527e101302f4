// gemv_pair_kernel instantiations: a Q4_K matrix and a Q6_K matrix whose rows each fit one wavefront
// (k <= 4096) -- Q|K and V of a Q4_K_M-style layer in one launch.
#include "gemv_launch.hip.h"

bool cera_gemv_launch_pair_q4k_q6k(const GemvPairArgs& a, const GemvPlan& pa, const GemvPlan& pb, hipStream_t s) {
    if (pa.U != 1 || pa.KS != 1 || pb.U != 1 || pb.KS != 1) return false;
    const dim3 grid(pa.n_blocks + pb.n_blocks), block(64);
#define PAIR(RA, RB_)                                                                                      \
    if (pa.RB == RA && pb.RB == RB_) {                                                                     \
        hipLaunchKernelGGL((gemv_pair_kernel<Q4K, 1, RA, Q6K, RB_>), grid, block, 0, s, a);                \
        return true;                                                                                       \
    }
    PAIR(1, 1) PAIR(1, 2) PAIR(2, 1) PAIR(2, 2)
#undef PAIR
    return false;
}
