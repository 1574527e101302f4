// Device-side helpers shared by the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

// ---- unaligned global loads ------------------------------------------------
// GGUF blocks of 18/34/210 bytes are only 2-byte aligned inside a row, and
// 20-byte blocks 4-byte aligned.  gfx950 global loads accept any alignment;
// these typedefs tell the compiler the true (small) alignment so it still
// emits one wide load instead of byte loads.
typedef uint32_t u32_a2 __attribute__((aligned(2)));
typedef uint2 uint2_a2 __attribute__((aligned(2)));
typedef uint4 uint4_a2 __attribute__((aligned(2)));
typedef uint4 uint4_a4 __attribute__((aligned(4)));
typedef uint2 uint2_a4 __attribute__((aligned(4)));

__device__ __forceinline__ uint32_t ld_u32_a2(const uint8_t* p) { return *reinterpret_cast<const u32_a2*>(p); }
__device__ __forceinline__ uint2 ld_u64_a2(const uint8_t* p) { return *reinterpret_cast<const uint2_a2*>(p); }
__device__ __forceinline__ uint4 ld_u128_a2(const uint8_t* p) { return *reinterpret_cast<const uint4_a2*>(p); }
__device__ __forceinline__ uint4 ld_u128_a4(const uint8_t* p) { return *reinterpret_cast<const uint4_a4*>(p); }
__device__ __forceinline__ uint4 ld_u128(const uint8_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ uint32_t ld_u16(const uint8_t* p) { return *reinterpret_cast<const uint16_t*>(p); }

// IEEE half bits -> float (v_cvt_f32_f16).
__device__ __forceinline__ float h2f(uint32_t bits16) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16)));
}
// float -> IEEE half bits, round to nearest even (v_cvt_f16_f32).
__device__ __forceinline__ uint32_t f2h(float v) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
}

// KV cache element access.  The cache holds f32, or IEEE half when the session asks for an f16
// KV cache (cera/src/kv_cache.rs:93-98): values are narrowed with round-to-nearest-even when a
// row is appended and widened exactly on every read, accumulation stays f32
// (cera/src/model/transformer.rs:1424-1447, 1170-1196).
typedef _Float16 kv_half;
// col4(j, c) is the float4 column (of the 32 in a 128-wide row) that lane j of an 8-lane group
// holds as its c-th register quad in the decode attention kernels: chosen per element type so
// that a lane's loads are 16 bytes wide and the 8 lanes of a load cover whole 128-byte lines.
typedef float cera_f4v __attribute__((ext_vector_type(4)));
typedef unsigned int cera_u4v __attribute__((ext_vector_type(4)));
// 16-byte loads with the non-temporal hint: for data read once by one wavefront, where every load
// instruction of the wavefront covers whole 128-byte lines (a line touched by two instructions is
// fetched twice).  Streaming reads of that shape run at ~7.0 instead of ~6.1 TB/s.
__device__ __forceinline__ float4 ld_f4_nt(const float* p) {
    const cera_f4v t = __builtin_nontemporal_load(reinterpret_cast<const cera_f4v*>(p));
    return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ uint4 ld_u128_nt(const void* p) {
    const cera_u4v t = __builtin_nontemporal_load(reinterpret_cast<const cera_u4v*>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
}
template <typename KV> struct KvOps;
template <> struct KvOps<float> {
    __device__ static __forceinline__ float4 ld4(const float* row, uint32_t i) { return reinterpret_cast<const float4*>(row)[i]; }
    __device__ static __forceinline__ float4 ld4nt(const float* row, uint32_t i) { return ld_f4_nt(row + 4 * i); }
    __device__ static __forceinline__ void st4(float* row, uint32_t i, float4 v) { reinterpret_cast<float4*>(row)[i] = v; }
    __device__ static __forceinline__ float4 rnd4(float4 v) { return v; }
    __device__ static __forceinline__ float ld1(const float* p) { return *p; }
    __device__ static __forceinline__ uint32_t col4(uint32_t j, int c) { return j + 8 * c; }
    __device__ static __forceinline__ void ld16(const float* row, uint32_t j, float4 (&v)[4]) {
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = reinterpret_cast<const float4*>(row)[j + 8 * c];
    }
};
template <> struct KvOps<kv_half> {
    __device__ static __forceinline__ float4 cvt4(uint32_t lo, uint32_t hi) {
        return make_float4(h2f(lo & 0xFFFF), h2f(lo >> 16), h2f(hi & 0xFFFF), h2f(hi >> 16));
    }
    __device__ static __forceinline__ float4 ld4(const kv_half* row, uint32_t i) {
        const uint2 r = reinterpret_cast<const uint2*>(row)[i];
        return cvt4(r.x, r.y);
    }
    __device__ static __forceinline__ float4 ld4nt(const kv_half* row, uint32_t i) { return ld4(row, i); }   // 8-byte pieces: half lines
    __device__ static __forceinline__ void st4(kv_half* row, uint32_t i, float4 v) {
        reinterpret_cast<uint2*>(row)[i] = make_uint2(f2h(v.x) | (f2h(v.y) << 16), f2h(v.z) | (f2h(v.w) << 16));
    }
    __device__ static __forceinline__ float4 rnd4(float4 v) {
        return make_float4(h2f(f2h(v.x)), h2f(f2h(v.y)), h2f(f2h(v.z)), h2f(f2h(v.w)));
    }
    __device__ static __forceinline__ float ld1(const kv_half* p) { return static_cast<float>(*p); }
    // quads 2c', 2c'+1 are the two halves of one 16-byte load: float4 columns 2(j + 8c'), +1
    __device__ static __forceinline__ uint32_t col4(uint32_t j, int c) { return 2 * (j + 8 * (c >> 1)) + (c & 1); }
    __device__ static __forceinline__ void ld16(const kv_half* row, uint32_t j, float4 (&v)[4]) {
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const uint4 r = reinterpret_cast<const uint4*>(row)[j + 8 * cc];
            v[2 * cc] = cvt4(r.x, r.y);
            v[2 * cc + 1] = cvt4(r.z, r.w);
        }
    }
};

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences global memory, which
// on this target means waiting for every outstanding global load of the wavefront -- including
// prefetched weight rows that nothing behind the barrier needs yet.  Use this where the data
// exchanged across the barrier lives in LDS.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// 4 x int8 dot with int32 accumulate (v_dot4_i32_i8).
__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), c, false);
}
// sum of the four signed bytes of a
__device__ __forceinline__ int sum4(uint32_t a, int c) { return dot4(a, 0x01010101u, c); }

// ---- wavefront reductions (DPP; gfx9 row/bank semantics) --------------------
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, true));
}
// Sum over the 64 lanes; the total is returned in every lane.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f<0x141>(v);  // row_half_mirror
    v += dpp_f<0x140>(v);  // row_mirror: every lane of a 16-lane row holds the row sum
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (r0 + r1) + (r2 + r3);
}
// The same for a double: each step moves the two halves of the value with a DPP move apiece
// (a wave shuffle of a 64-bit value is two LDS-pipe permutes, ~10x the latency).
template <int CTRL>
__device__ __forceinline__ double dpp_d(double v) {
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(b)), CTRL, 0xF, 0xF, true));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(b >> 32)), CTRL, 0xF, 0xF, true));
    return __builtin_bit_cast(double, (static_cast<uint64_t>(hi) << 32) | lo);
}
__device__ __forceinline__ double readlane_d(double v, int lane) {
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(b)), lane));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(b >> 32)), lane));
    return __builtin_bit_cast(double, (static_cast<uint64_t>(hi) << 32) | lo);
}
__device__ __forceinline__ double wave_sum_f64(double v) {
    v += dpp_d<0xB1>(v);
    v += dpp_d<0x4E>(v);
    v += dpp_d<0x141>(v);
    v += dpp_d<0x140>(v);
    return (readlane_d(v, 0) + readlane_d(v, 16)) + (readlane_d(v, 32) + readlane_d(v, 48));
}
// sum over each 16-lane row; every lane of a row ends up with its row's sum
__device__ __forceinline__ float wave_row_sum(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    v += dpp_f<0x140>(v);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x141>(v));
    v = fmaxf(v, dpp_f<0x140>(v));
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// ggml's polynomial expf as cera uses it (cera/src/backend/cpu.rs:2504-2544),
// evaluated without FMA contraction so it rounds exactly like the CPU path.
__device__ __forceinline__ float cera_expf(float x) {
    const float R = __builtin_bit_cast(float, 0x4B400000u);
    const float LOG2E = __builtin_bit_cast(float, 0x3FB8AA3Bu);
    const float LN2_HI = __builtin_bit_cast(float, 0x3F317200u);
    const float LN2_LO = __builtin_bit_cast(float, 0x35BFBE8Eu);
    const float C1 = __builtin_bit_cast(float, 0x3F7FFFF6u);
    const float C2 = __builtin_bit_cast(float, 0x3EFFFEDBu);
    const float C3 = __builtin_bit_cast(float, 0x3E2AAF33u);
    const float C4 = __builtin_bit_cast(float, 0x3D2B9F17u);
    const float C5 = __builtin_bit_cast(float, 0x3C072010u);
    float z = __fadd_rn(R, __fmul_rn(x, LOG2E));
    float n = __fsub_rn(z, R);
    float b = __fsub_rn(__fsub_rn(x, __fmul_rn(n, LN2_HI)), __fmul_rn(n, LN2_LO));
    uint32_t e = __builtin_bit_cast(uint32_t, z) << 23;
    float k = __builtin_bit_cast(float, e + 0x3F800000u);
    float u = __fmul_rn(b, b);
    float t45 = __fadd_rn(C4, __fmul_rn(C5, b));
    float t23 = __fadd_rn(C2, __fmul_rn(C3, b));
    float j = __fadd_rn(__fmul_rn(C1, b), __fmul_rn(__fadd_rn(t23, __fmul_rn(t45, u)), u));
    float abs_n = fabsf(n);
    if (abs_n <= 126.0f) return __fadd_rn(k, __fmul_rn(j, k));
    if (abs_n > 192.0f) return n > 0.0f ? __builtin_inff() : 0.0f;
    uint32_t d = n <= 0.0f ? 0x82000000u : 0u;
    float s1 = __builtin_bit_cast(float, d + 0x7f000000u);
    float s2 = __builtin_bit_cast(float, e - d);
    return __fmul_rn(__fadd_rn(s2, __fmul_rn(s2, j)), s1);
}
