// Host-side dispatch of gemv_kernel<T, U, RB, EPI, DBG> over the run-time
// values of U (units per lane), RB (rows in flight) and the epilogue.
#pragma once
#include "gemv.cuh"
#include "host_common.h"

// U is rounded up to the next instantiated width; the surplus lanes carry
// zeroed activations.
static inline int gemv_pick_u(uint32_t n_units) {
    uint32_t u = (n_units + 63) / 64;
    const int widths[] = {1, 2, 4, 7, 8};
    for (int w : widths)
        if (u <= static_cast<uint32_t>(w)) return w;
    return 0;  // K too large for the register-resident kernel
}

template <class T, int U, int RB>
static void gemv_launch_epi(const GemvArgs& a, int epi, bool dbg, dim3 grid, hipStream_t s) {
    if (dbg) {
        hipLaunchKernelGGL((gemv_kernel<T, U, RB, EPI_STORE, true>), grid, dim3(256), 0, s, a);
        return;
    }
    switch (epi) {
        case EPI_ADD: hipLaunchKernelGGL((gemv_kernel<T, U, RB, EPI_ADD, false>), grid, dim3(256), 0, s, a); break;
        case EPI_SILU_MUL: hipLaunchKernelGGL((gemv_kernel<T, U, RB, EPI_SILU_MUL, false>), grid, dim3(256), 0, s, a); break;
        default: hipLaunchKernelGGL((gemv_kernel<T, U, RB, EPI_STORE, false>), grid, dim3(256), 0, s, a); break;
    }
}

// Wide rows keep two rows in flight, narrow rows four (when a wavefront has
// that many rows at all): enough bytes outstanding per CU without spilling.
template <class T>
static bool gemv_launch_t(const GemvArgs& a, int U, int RB, int epi, bool dbg, dim3 grid, hipStream_t s) {
    switch (U) {
        case 1: if (RB == 4) gemv_launch_epi<T, 1, 4>(a, epi, dbg, grid, s); else gemv_launch_epi<T, 1, 2>(a, epi, dbg, grid, s); return true;
        case 2: if (RB == 4) gemv_launch_epi<T, 2, 4>(a, epi, dbg, grid, s); else gemv_launch_epi<T, 2, 2>(a, epi, dbg, grid, s); return true;
        case 4: gemv_launch_epi<T, 4, 2>(a, epi, dbg, grid, s); return true;
        case 7: gemv_launch_epi<T, 7, 2>(a, epi, dbg, grid, s); return true;
        case 8: gemv_launch_epi<T, 8, 2>(a, epi, dbg, grid, s); return true;
        default: return false;
    }
}

struct GemvPlan {
    int U, RB;
    uint32_t rows_per_wave, n_blocks;
};

static inline GemvPlan gemv_plan(uint32_t m, uint32_t n_units, uint32_t n_cu, bool dbg) {
    GemvPlan p;
    p.U = gemv_pick_u(n_units);
    const uint32_t target_waves = n_cu * 8;
    uint32_t rpw = (m + target_waves - 1) / target_waves;
    p.RB = (p.U <= 2 && rpw >= 4) ? 4 : 2;
    if (dbg) p.RB = 2;
    rpw = (rpw + p.RB - 1) / p.RB * p.RB;
    p.rows_per_wave = rpw;
    uint32_t waves = (m + rpw - 1) / rpw;
    p.n_blocks = (waves + 3) / 4;
    return p;
}
