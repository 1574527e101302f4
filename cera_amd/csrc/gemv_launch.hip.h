// Host-side dispatch of gemv_kernel<T, U, KS, RB, EPI, DBG> over the run-time
// values of the K split (KS wavefronts per workgroup, U units per lane), RB
// (rows in flight) and the epilogue.
#pragma once
#include "gemv.hip.h"
#include "host_common.h"

struct GemvPlan {
    int U, KS, RB;
    uint32_t rows_per_block, n_blocks;
};

// n_units = K / elements per unit (64 for the K-quants, 32 for the block formats).  One unit per
// lane up to 512 units (KS up to 8 wavefronts), two per lane up to 1024.  KS is rounded up to an instantiated width; surplus
// lanes carry zeroed activations.
static inline bool gemv_pick_split(uint32_t n_units, int* U, int* KS) {
    const int widths[] = {1, 2, 4, 7, 8};
    for (int u = 1; u <= 2; ++u)
        for (int w : widths)
            if (n_units <= static_cast<uint32_t>(64 * w * u)) { *U = u; *KS = w; return true; }
    return false;
}

// Measured on MI355X: ~32 wavefronts per CU in flight; rows in flight per workgroup step are
// capped by the caller (max_rb) by the registers a row of the type takes.
static inline bool gemv_plan(uint32_t m, uint32_t n_units, uint32_t n_cu, bool dbg, int max_rb, GemvPlan* p,
                             bool dual = false) {
    if (!gemv_pick_split(n_units, &p->U, &p->KS)) return false;
    // very tall matrices (the vocabulary head) do better with few long-lived workgroups that
    // stream row groups through the two register buffers; everything else with many short ones
    // (wavefronts per CU the launch aims at; the fused gate+up pair, whose workgroups carry two
    // matrices' rows, likes 32, plain two-wavefront splits 24, the wide K splits of long rows 16:
    // measured 2-3 % apart on the Llama-3-8B shapes)
    const uint32_t per_cu = m >= 65536 ? 4 : (dual ? 32 : (p->KS >= 4 ? 16 : 24));
    const uint32_t target_blocks = std::max(1u, n_cu * per_cu / static_cast<uint32_t>(p->KS));
    uint32_t rpb = (m + target_blocks - 1) / target_blocks;
    p->RB = rpb >= 4 ? 4 : (rpb >= 2 ? 2 : 1);

    if (p->RB > max_rb) p->RB = max_rb;
    if (dbg) p->RB = 1;
    rpb = (rpb + p->RB - 1) / p->RB * p->RB;
    p->rows_per_block = rpb;
    p->n_blocks = (m + rpb - 1) / rpb;
    return true;
}

template <class T, int U, int KS, int RB>
static void gemv_launch_epi(const GemvArgs& a, int epi, bool dbg, dim3 grid, hipStream_t s) {
    const dim3 block(64 * KS);
    if (dbg) {
        if (RB == 1) hipLaunchKernelGGL((gemv_kernel<T, U, KS, 1, EPI_STORE, true>), grid, block, 0, s, a);
        return;
    }
    switch (epi) {
        case EPI_ADD: hipLaunchKernelGGL((gemv_kernel<T, U, KS, RB, EPI_ADD, false>), grid, block, 0, s, a); break;
        case EPI_SILU_MUL: hipLaunchKernelGGL((gemv_kernel<T, U, KS, RB, EPI_SILU_MUL, false>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((gemv_kernel<T, U, KS, RB, EPI_STORE, false>), grid, block, 0, s, a); break;
    }
}

template <class T, int U, int KS>
static void gemv_launch_rb(const GemvArgs& a, int RB, int epi, bool dbg, dim3 grid, hipStream_t s) {
    switch (RB) {
        case 1: gemv_launch_epi<T, U, KS, 1>(a, epi, dbg, grid, s); break;
        case 2: gemv_launch_epi<T, U, KS, 2>(a, epi, dbg, grid, s); break;
        default: gemv_launch_epi<T, U, KS, 4>(a, epi, dbg, grid, s); break;
    }
}

template <class T>
static bool gemv_launch_t(const GemvArgs& a, const GemvPlan& p, int epi, bool dbg, hipStream_t s) {
    dim3 grid(p.n_blocks);
#define CASE(UU, KK) if (p.U == UU && p.KS == KK) { gemv_launch_rb<T, UU, KK>(a, p.RB, epi, dbg, grid, s); return true; }
    CASE(1, 1) CASE(1, 2) CASE(1, 4) CASE(1, 7) CASE(1, 8) CASE(2, 7) CASE(2, 8)
#undef CASE
    return false;
}
