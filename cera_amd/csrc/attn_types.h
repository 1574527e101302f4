// Types shared by the attention kernels and their host-side launchers.
#pragma once
#include <stdint.h>

// The new token's own key and value, when the decode step lets the attention kernel do the
// RoPE and the cache append: q arrives unrotated and is rotated on load; the wavefront whose
// range holds the last position takes that position's K/V rows from the projection outputs
// (rotating K), uses them, and writes them into the cache.  One launch less per layer.
// Measured in the model: the fused form wins while a wavefront holds a single 8-key chunk
// (6.1 us against 2.6 + 5.4 us for a RoPE/append launch plus plain attention at 640 keys), is
// level at 2k keys and loses 3 us per layer at 8k, where the per-wavefront q rotation and the
// extra registers cost more than the launch they replace.  The decode step fuses below this
// context length and launches rope_kv_kernel above it; the launcher's chunk size switches at
// the same point.
#define ATTN_FUSED_NEW_KV_MAX_KEYS 1024u

struct AttnNewKV {
    const float* rope_row;   // [64] (cos, sin) pairs of the token's position
    uint32_t rope_type;      // 0 NEOX, 1 NORM
    const float* k_new;      // [n_kv][128], unrotated
    const float* v_new;      // [n_kv][128]
    void* kc_w;              // the caches, writable (f32 or half, as the kernel is instantiated)
    void* vc_w;
};
