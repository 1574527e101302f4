// Types shared by the attention kernels and their host-side launchers.
#pragma once
#include <stdint.h>

// The new token's own key and value, when the decode step lets the attention kernel do the
// RoPE and the cache append: q arrives unrotated and is rotated on load; the wavefront whose
// range holds the last position takes that position's K/V rows from the projection outputs
// (rotating K), uses them, and writes them into the cache.  One launch less per layer.
struct AttnNewKV {
    const float* rope_row;   // [64] (cos, sin) pairs of the token's position
    uint32_t rope_type;      // 0 NEOX, 1 NORM
    const float* k_new;      // [n_kv][128], unrotated
    const float* v_new;      // [n_kv][128]
    void* kc_w;              // the caches, writable (f32 or half, as the kernel is instantiated)
    void* vc_w;
};
