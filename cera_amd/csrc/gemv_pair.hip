// gemv_pair_kernel instantiations: a Q4_K matrix whose K takes two wavefronts (k = 4096) with a
// Q6_K matrix whose K fits one -- Q|K and V of a Q4_K_M-style layer in one launch.
#include "gemv_launch.cuh"

bool cera_gemv_launch_pair_q4k_q6k(const GemvPairArgs& a, const GemvPlan& pa, const GemvPlan& pb, hipStream_t s) {
    if (pa.U != 1 || pa.KS != 2 || pb.U != 1 || pb.KS != 1) return false;
    const uint32_t blocks_b = (pb.n_blocks + 1) / 2;   // two of B's one-wavefront workgroups per real one
    const dim3 grid(pa.n_blocks + blocks_b), block(128);
#define PAIR(RA, RB_)                                                                                      \
    if (pa.RB == RA && pb.RB == RB_) {                                                                     \
        hipLaunchKernelGGL((gemv_pair_kernel<Q4K, 2, RA, Q6K, RB_>), grid, block, 0, s, a);                \
        return true;                                                                                       \
    }
    PAIR(1, 1) PAIR(1, 2) PAIR(2, 1) PAIR(2, 2) PAIR(4, 1) PAIR(4, 2)
#undef PAIR
    return false;
}
