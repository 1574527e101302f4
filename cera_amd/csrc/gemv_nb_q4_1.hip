// gemv_nb_kernel instantiations for Q4_1 (one translation unit per weight type keeps the device
// compile parallel).
#include "gemv_nb.hip.h"
#include "host_common.h"

bool cera_gemv_nb_launch_q4_1(const GemvNbArgs& a, int KS, int RB, int NB, bool add, uint32_t n_blocks, hipStream_t s) {
    return gemv_nb_launch_t<Q4_1>(a, KS, RB, NB, add, n_blocks, s);
}
