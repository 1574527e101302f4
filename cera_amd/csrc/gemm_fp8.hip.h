// Prefill GEMM for Q4_K on the fp8 matrix cores: out[m][n] = W[m, k] . B[k, n], the same contract as
// gemm.hip.h (cera's batched int8 path, cera/src/backend/simd.rs:5693-5878, 5392-5518;
// cera/src/model/transformer.rs:710-788, 865-946): exact integer dots of 4-bit weight codes with
// int8 activations per 32-element block, then per block  acc += dot * (xs * (d*sc))  in f32 and
// the min terms  - dmin*mn * (xs * sum a).
//
// What is different from the int8 kernel is where each piece of work runs:
//   * the block dot leaves the matrix core as a float.  A weight code 0..15 stored in a byte IS an
//     E4M3 number (exponent fields 0 and 1 are linear: byte n = n * 2^-9), and an int8 activation
//     splits exactly as a = 16*a_hi + a_lo, a_lo in 0..15 (again a raw byte), a_hi in -8..7
//     (16*a_hi*2^-9 is an exact E4M3 number).  One v_mfma_f32_32x32x64_f8f6f4 over
//     [q | q] x [a_lo | a_hi] is therefore 2^-18 times the exact integer dot of one block, every
//     partial sum an integer below 2^24: no int->float convert on the vector ALU, one FMA per
//     output and block (the 2^18 rides on the row scale, a power of two, so the product
//     xs * (d*sc) and the FMA round exactly as before);
//   * nothing is unpacked into LDS and nothing staged costs a vector instruction.  A wavefront owns 32
//     rows for the whole K loop; the bytes of its rows and the activations both reach LDS by DMA
//     (global_load_lds_dwordx4, inline assembly with scalar addresses: two scalar instructions and
//     the load per KB).  The weights arrive as 16-byte pieces in row order (consecutive lanes on
//     consecutive pieces of a row: every cache line is fetched once) and a lane picks its row's header
//     and its half of each 32-byte chunk (16 codes of block 2g in the low nibbles, 16 of block 2g+1
//     in the high ones) out of the wavefront's private copy; two AND/shift passes make both A
//     operands.  The activations come from a copy that the split kernel below wrote in exactly the
//     order the MFMA wants them, so fragment reads are lane-contiguous (no bank conflicts);
//   * the min terms run on the bf16 matrix core once per 256-element super-block: dmin*mn (17
//     significant bits) and xs*sum(a) (24) are split exactly into three bf16 pieces each and the
//     six products above 2^-24 of the term take six K slots per block, 48 per super-block, three
//     v_mfma_f32_32x32x16_bf16 accumulating (negated) into the same tile as the dots.
//
// Workgroup: 256 threads = 4 wavefronts stacked along M; tile 128 rows x 64 tokens; a wavefront
// owns 32 rows x 64 tokens (two MFMA tiles, 32 accumulator registers); two workgroups share a CU.
// K advances in stages of 128 elements, double-buffered in LDS with one barrier per stage, and the
// K loop is software-pipelined inside the wavefront (see the kernel).
//
// What bounds it: on this chip the matrix core and the vector ALU of a SIMD do not run at the same
// time in a kernel of this kind (matrix-core busy + vector-ALU busy = 100 % of the dispatch, here as
// in the int8 kernel), so the cost of a 32 x 32 x 32 tile step is the SUM of its MFMA clocks (64 dot +
// 32 scale tile + 12 min terms) and its vector instructions (16 FMAs + about 12 of unpacking and
// scale decoding, ~3 clocks each).  Against the int8 form (32 + 32 + 32 MFMA clocks, 16 converts + 16
// FMAs + staging) that sum is what the fp8 dot lowers.
#pragma once
#include "gemm.hip.h"
#include "gemm_q6k_f16.hip.h"

typedef int v8i __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

#ifndef G8_NW
#define G8_NW 4                   // wavefronts per workgroup
#endif
#define G8_BM (32 * G8_NW)        // rows per workgroup
#define G8_BN 64                  // tokens per workgroup
#define G8_REC 21504              // bytes of the activation copy per (32-token tile, 256-element super-block)
#define G8_REC_XS 16384           //   offset of the activation scales  [8 blocks][32 tokens] f32
#define G8_REC_MIN 17408          //   offset of the min-term operands  [3][64 lanes][16 B] (+ 1 KB unused)

// ---- activation split: Q8_0 rows -> the fragment-ordered fp8 copy ----------------------------
// One workgroup per (32-token tile, super-block).  Record layout:
//   [blk 0..7][piece 0..1][lane 0..63][16 B]   piece 0: a & 15 (raw bytes), piece 1: E4M3 of
//       (a >> 4) * 2^-5; lane = token%32 + 32*half holds elements 16*half .. 16*half+15 of the block
//   [blk 0..7][token%32] f32                    the Q8_0 scales
//   [j 0..2][lane][8 bf16]                      xs*sum(a) of blocks 4*half .. 4*half+3 as three bf16 pieces
//       b0, b1, b2 in slot order (b0, b1, b0, b2, b1, b0) per block, slots 8j .. 8j+7 of the lane's 24
// Tokens at or beyond n are zero.
// halves (nullable): the same quants also as f16 [n][k] in gemm_act_f16_kernel's order, for a Q6_K matrix
// multiplied by the same activations (a layer's V next to its Q4_K Q and K): one launch for both copies.
__device__ __forceinline__ void gemm_act_fp8_body(const int8_t* __restrict__ xq, const float* __restrict__ xs,
                                                                  const float* __restrict__ bsum, uint8_t* __restrict__ rec,
                                                                  uint32_t n, uint32_t k, uint4* __restrict__ halves = nullptr) {
    const uint32_t nsb = k / 256, tile = blockIdx.x / nsb, sb = blockIdx.x % nsb, tid = threadIdx.x;
    uint8_t* const r = rec + static_cast<uint64_t>(blockIdx.x) * G8_REC;
    // quants: thread t handles (blk = t / 32, token = t % 32): 32 bytes in, 2 x 2 x 16 bytes out
    {
        const uint32_t blk = tid >> 5, col = tid & 31, tok = tile * 32 + col;
        uint4 in[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
        if (tok < n) {
            const uint4* src = reinterpret_cast<const uint4*>(xq + static_cast<uint64_t>(tok) * k + sb * 256 + blk * 32);
            in[0] = src[0];
            in[1] = src[1];
            if (halves) {
                uint4* const dst = halves + (static_cast<uint64_t>(tok) * k + sb * 256 + blk * 32) / 8;
                gemm_act_f16_words(in[0], dst[0], dst[1]);
                gemm_act_f16_words(in[1], dst[2], dst[3]);
            }
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const uint32_t w[4] = {in[half].x, in[half].y, in[half].z, in[half].w};
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                lo[i] = w[i] & 0x0F0F0F0Fu;
                uint32_t o = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int a = static_cast<int8_t>(w[i] >> (8 * b));
                    const int h = a >> 4;                       // -8..7
                    const uint32_t mag = static_cast<uint32_t>(h < 0 ? -h : h);
                    // E4M3 of mag * 2^-5, mag = 0..8: 0, 2^-5, 2^-4, 1.5*2^-4, 2^-3, 1.25*2^-3, 1.5*2^-3, 1.75*2^-3, 2^-2
                    const uint32_t code = (0x28262422201C1810ull >> (8 * (mag ? mag - 1 : 0))) & 0xFF;
                    const uint32_t byte = mag == 0 ? 0u : (code | (h < 0 ? 0x80u : 0u));
                    o |= byte << (8 * b);
                }
                hi[i] = o;
            }
            uint8_t* dst = r + blk * 2048 + (col + 32 * half) * 16;
            *reinterpret_cast<uint4*>(dst) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            *reinterpret_cast<uint4*>(dst + 1024) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        }
        reinterpret_cast<float*>(r + G8_REC_XS)[blk * 32 + col] = tok < n ? xs[static_cast<uint64_t>(tok) * (k / 32) + sb * 8 + blk] : 0.0f;
    }
    // min operands: thread t < 64 is lane t: blocks 4*half .. +3 of token col
    if (tid < 64) {
        const uint32_t col = tid & 31, half = tid >> 5, tok = tile * 32 + col;
        uint32_t slot[24];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float v = tok < n ? bsum[static_cast<uint64_t>(tok) * (k / 32) + sb * 8 + 4 * half + i] : 0.0f;
            const uint32_t b0 = __builtin_bit_cast(uint32_t, v) & 0xFFFF0000u;
            const float e1 = v - __builtin_bit_cast(float, b0);
            const uint32_t b1 = __builtin_bit_cast(uint32_t, e1) & 0xFFFF0000u;
            const float e2 = e1 - __builtin_bit_cast(float, b1);
            const uint32_t b2 = __builtin_bit_cast(uint32_t, e2) & 0xFFFF0000u;
            const uint32_t s0 = b0 >> 16, s1 = b1 >> 16, s2 = b2 >> 16;
            slot[6 * i + 0] = s0; slot[6 * i + 1] = s1; slot[6 * i + 2] = s0;
            slot[6 * i + 3] = s2; slot[6 * i + 4] = s1; slot[6 * i + 5] = s0;
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            uint4 o;
            o.x = slot[8 * j + 0] | (slot[8 * j + 1] << 16);
            o.y = slot[8 * j + 2] | (slot[8 * j + 3] << 16);
            o.z = slot[8 * j + 4] | (slot[8 * j + 5] << 16);
            o.w = slot[8 * j + 6] | (slot[8 * j + 7] << 16);
            *reinterpret_cast<uint4*>(r + G8_REC_MIN + j * 1024 + tid * 16) = o;
        }
    }
}
static __global__ __launch_bounds__(256) void gemm_act_fp8_kernel(const int8_t* __restrict__ xq, const float* __restrict__ xs,
                                                                  const float* __restrict__ bsum, uint8_t* __restrict__ rec,
                                                                  uint32_t n, uint32_t k, uint4* __restrict__ halves) {
    gemm_act_fp8_body(xq, xs, bsum, rec, n, k, halves);
}

// global -> LDS copy of 1 KB (64 lanes x 16 B) without passing through registers: lane i's 16 bytes
// at base + off_lane land at LDS address lds + 16 i.  base and lds are wavefront-uniform (scalar
// registers), so a copy costs two scalar instructions and the load itself.  Written as inline
// assembly: the compiler's own form of this load makes it treat every later wait on an LDS read or
// a global load as a wait for everything in flight.
__device__ __forceinline__ void g8_dma_1k(const uint8_t* base, uint32_t off_lane, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off_lane), "s"(base), "s"(lds) : "memory", "m0");
}
// the same for 256 B (64 lanes x 4 B)
__device__ __forceinline__ void g8_dma_256(const uint8_t* base, uint32_t off_lane, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(off_lane), "s"(base), "s"(lds) : "memory", "m0");
}
// LDS byte address of a __shared__ object
__device__ __forceinline__ uint32_t g8_lds_addr(const void* p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)(p)));
}

struct G8Stage {
    uint8_t bf[2][4][2048];   // [token tile][block of the stage][piece][lane][16]
    float xs[2][4][32];       // [token tile][block][token]
};
struct G8Mins {
    uint8_t b[2][4096];       // [token tile][j][lane][16], the last KB unused
};

template <bool SWIGLU = false, bool DBG = false, int NW = G8_NW>
__device__ __forceinline__ void gemm_q4k_fp8_body(GemmArgs p) {
    constexpr uint32_t BM = 32 * NW;   // rows per workgroup
    // the two stage buffers are separate variables so that the compiler can tell the DMA into one
    // from the fragment reads of the other (a shared array would make every LDS read wait for
    // the DMA in flight)
    __shared__ __attribute__((aligned(16))) G8Stage st0;
    __shared__ __attribute__((aligned(16))) G8Stage st1;
    __shared__ __attribute__((aligned(16))) G8Mins mnb_lds;   // min operands of the super-block in progress
    // each wavefront's own rows of the next super-block, 32 x 144 bytes as 16-byte pieces in row order
    // (+ 32 unused pieces: the fifth copy instruction runs with all lanes)
    __shared__ __attribute__((aligned(16))) uint8_t wts[NW][320 * 16];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wavefront-uniform: a scalar register
    const uint32_t col = lane & 31, half = lane >> 5;
    const bool second = !SWIGLU && p.w2 != nullptr && blockIdx.y >= p.tiles1;
    const uint8_t* const wmat = second ? p.w2 : p.w;
    float* const omat = second ? p.out2 : p.out;
    const uint32_t mrows = second ? p.m2 : p.m;
    const uint64_t ldn = second ? p.ld_n2 : p.ld_n;
    const uint32_t m0 = (second ? blockIdx.y - p.tiles1 : blockIdx.y) * (SWIGLU ? BM / 2 : BM);
    const uint32_t n0 = blockIdx.x * G8_BN;
    const uint32_t nsb_all = p.k / 256;
    // this wavefront's 32 rows.  SwiGLU: the first half of the wavefronts take rows of the gate
    // matrix and the second half the same rows of the up matrix.
    const uint32_t row0 = SWIGLU ? m0 + 32 * (wave % (NW / 2)) : m0 + 32 * wave;
    // uniform base + 32-bit lane offset: one address register per lane instead of a pointer
    const uint8_t* const wbase = (SWIGLU ? (wave < NW / 2 ? p.w : p.w2) : wmat) + static_cast<uint64_t>(m0) * p.row_bytes;
    // Weights reach the lanes through LDS as well.  A lane that loaded its own row's bytes from
    // global memory made every load instruction touch 32 rows = 32 cache lines for 16 bytes each, and a
    // row's two lines were fetched again by each of the five loads of a super-block (they do not survive
    // in the 16 KB first-level cache between them): the loads alone took a fifth of the kernel.  Instead
    // five DMA instructions copy the wavefront's 32 x 144 bytes with consecutive lanes on consecutive
    // 16-byte pieces of a row (every line fetched once), and each lane then picks its row's header and
    // its half of the four chunks out of LDS.
    uint32_t wpiece[5];   // global offset (from wbase, without the super-block) of piece 64 j + lane
#pragma unroll
    for (int j = 0; j < 5; ++j) {
        const uint32_t q = min(64u * j + lane, 287u), r = q / 9, part = q - 9 * r;
        wpiece[j] = (min(row0 + r, mrows - 1) - m0) * p.row_bytes + part * 16;
    }
    const uint32_t wts_lds = g8_lds_addr(&wts[0][0]) + wave * (320 * 16);
    const uint8_t* const wts_row = &wts[0][0] + wave * (320 * 16) + col * 144;   // this lane's row in the staged copy
    const uint32_t sb_begin = blockIdx.z * (p.k_chunk / 256), sb_end = sb_begin + p.k_chunk / 256;
    const uint8_t* const rec0 = p.bf8 + static_cast<uint64_t>(blockIdx.x * 2) * nsb_all * G8_REC;   // token tile 2*blockIdx.x
    const uint64_t rec_tile = static_cast<uint64_t>(nsb_all) * G8_REC;
    const uint32_t lane16 = lane * 16, lane4 = lane * 4;

    // stage (sb, s) -> LDS buffer, every wavefront the same share of the 16 KB of fragments; 1 KB of
    // scales in four quarters; with_mins: also the 8 KB of min operands of super-block sb_mins
    auto stage_in = [&](uint32_t sb, uint32_t s, G8Stage& dst, bool with_mins, uint32_t sb_mins) {
        constexpr int CW = 16 / NW;   // fragment chunks of 1 KB per wavefront
        const uint32_t c0 = wave * CW, tn = c0 >> 3;
        const uint8_t* const r = rec0 + tn * rec_tile + static_cast<uint64_t>(sb) * G8_REC + s * 8192 + (c0 & 7) * 1024;
        const uint32_t l = g8_lds_addr(&dst.bf[tn][0][0]) + (c0 & 7) * 1024;
#pragma unroll
        for (int i = 0; i < CW; ++i) g8_dma_1k(r + i * 1024, lane16, l + i * 1024);
        if (wave < 4) {
            const uint8_t* const rx = rec0 + (wave >> 1) * rec_tile + static_cast<uint64_t>(sb) * G8_REC + G8_REC_XS + s * 512 + (wave & 1) * 256;
            g8_dma_256(rx, lane4, g8_lds_addr(&dst.xs[wave >> 1][0][0]) + (wave & 1) * 256);
        }
        if (with_mins) {
            constexpr int MW = 8 / NW;   // min-operand chunks per wavefront
            const uint32_t q0 = wave * MW, tm = q0 >> 2;
            const uint8_t* const rm = rec0 + tm * rec_tile + static_cast<uint64_t>(sb_mins) * G8_REC + G8_REC_MIN + (q0 & 3) * 1024;
            const uint32_t lm = g8_lds_addr(mnb_lds.b[tm]) + (q0 & 3) * 1024;
#pragma unroll
            for (int j = 0; j < MW; ++j) g8_dma_1k(rm + j * 1024, lane16, lm + j * 1024);
        }
    };

    // acc takes the scaled block dots (vector ALU) and, negated, the min terms (matrix core)
    v16f acc[2];
#pragma unroll
    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[tn][e] = 0.0f;

    // The K loop is software-pipelined inside the wavefront.  A step is one (pair g, token tile tn,
    // block jb of the pair): 16 per super-block.  Tick t issues the matrix-core work of step t+1, reads
    // the fragments of step t+3 from LDS and then runs the 16 FMAs of step t while that work
    // executes: on this hardware a SIMD overlaps matrix-core and vector instructions of the SAME
    // wavefront, not those of two different wavefronts.
    //
    // Weight prefetch: a super-block's rows are copied to LDS one super-block ahead (behind the barrier
    // of tick 13) and read into registers at tick 13 of the super-block before theirs.
    uint4 hdr, raw[4];
    // global -> this wavefront's LDS rows, super-block sb
    auto weights_in = [&](uint32_t sb) {
        const uint8_t* const b = wbase + static_cast<uint64_t>(sb) * 144;
#pragma unroll
        for (int j = 0; j < 5; ++j) g8_dma_1k(b, wpiece[j], wts_lds + j * 1024);
    };
    // LDS -> registers: header and this lane's half of the four chunks
    auto weights_read = [&]() {
        hdr = *reinterpret_cast<const uint4*>(wts_row);
#pragma unroll
        for (int g = 0; g < 4; ++g) raw[g] = *reinterpret_cast<const uint4*>(wts_row + 16 + g * 32 + half * 16);
    };

    // per super-block row state (lane = row col), decoded from the header
    float d18 = 0.0f, ndmin = 0.0f;   // d * 2^18, -dmin
    uint32_t scb = 0, mnb = 0;        // 6-bit scales of blocks 2g + half (g = 0..3) / mins of blocks 4*half .. +3, one per byte
    auto decode_hdr = [&]() {
        const uint4 h = hdr;
        d18 = h2f(h.x & 0xFFFF) * 262144.0f;
        ndmin = -h2f(h.x >> 16);
        const uint32_t s0 = h.y, s1 = h.z, s2 = h.w;
        const uint32_t sc_lo = s0 & 0x3F3F3F3Fu, mn_lo = s1 & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
        scb = __builtin_amdgcn_perm(sc_hi, sc_lo, half ? 0x07050301u : 0x06040200u);   // bytes half, 2+half of lo, then of hi
        mnb = half ? mn_hi : mn_lo;
    };

    v8i af[2];          // A operands of the pair being issued: low-nibble block, high-nibble block
    float rsl = 0.0f;   // this lane's row scale for the pair's scale-tile MFMA
    v8i bfr[4];         // B fragments, by step % 4 (read three steps ahead of the FMAs)
    float xsl[2];       // scale operand (token col, block 2pr + half), by (step / 2) parity
    v32f sct[2];        // scale tiles of a (pair, token tile), by (step / 2) parity
    v16f dot[2];        // block dots, by step parity

    // LDS reads of step t (0..15) of a super-block: stage t / 8, pair (t / 4) % 2, token tile (t / 2) % 2, block t % 2
    auto lds_read = [&](int t) {
        const G8Stage& st = (t & 8) ? st1 : st0;
        const int pr = (t >> 2) & 1, tn = (t >> 1) & 1, jb = t & 1;
        const uint8_t* f = &st.bf[tn][2 * pr + jb][0] + lane * 16;
        const v4i lo = *reinterpret_cast<const v4i*>(f), hi = *reinterpret_cast<const v4i*>(f + 1024);
        bfr[t & 3] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        if (jb == 0) xsl[(t >> 1) & 1] = st.xs[tn][2 * pr + half][col];
    };
    // matrix-core work of step t in two parts, so that other work can sit between them (behind the
    // scale-tile MFMA, whose 64 clocks are otherwise spent waiting to issue the dot): at a (pair,
    // token tile)'s first step the scale tile ...
    auto issue_s = [&](int t) {
        const int g = t >> 2;
        if ((t & 3) == 0) rsl = d18 * static_cast<float>((scb >> (8 * g)) & 0xFF);
        if ((t & 1) == 0) {
            v32f z32;
#pragma unroll
            for (int e = 0; e < 32; ++e) z32[e] = 0.0f;
            sct[(t >> 1) & 1] = __builtin_amdgcn_mfma_f32_32x32x1f32(rsl, xsl[(t >> 1) & 1], z32, 0, 0, 0);
        }
    };
    // ... and, after the A operands at a pair's first step, the block dot
    auto issue_d = [&](int t) {
        const int g = t >> 2, jb = t & 1;
        if ((t & 3) == 0) {
            const uint4 q = raw[g];
            const int l0 = q.x & 0x0F0F0F0F, l1 = q.y & 0x0F0F0F0F, l2 = q.z & 0x0F0F0F0F, l3 = q.w & 0x0F0F0F0F;
            const int h0 = (q.x >> 4) & 0x0F0F0F0F, h1 = (q.y >> 4) & 0x0F0F0F0F, h2 = (q.z >> 4) & 0x0F0F0F0F,
                      h3 = (q.w >> 4) & 0x0F0F0F0F;
            af[0] = v8i{l0, l1, l2, l3, l0, l1, l2, l3};
            af[1] = v8i{h0, h1, h2, h3, h0, h1, h2, h3};
        }
        v16f z16;
#pragma unroll
        for (int e = 0; e < 16; ++e) z16[e] = 0.0f;
        dot[t & 1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[jb], bfr[t & 3], z16, 0, 0, 0, 0, 0, 0);
    };
    auto fma_step = [&](int t, uint32_t sb) {
        const int tn = (t >> 1) & 1, jb = t & 1;
        if (DBG) {
            const uint32_t dtok = n0 + tn * 32 + col, dblk = sb * 8 + 2 * (t >> 2) + jb;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t drow = row0 + (e >> 2) * 8 + half * 4 + (e & 3);
                if (drow < mrows && dtok < p.n)
                    p.dbg_dots[(static_cast<uint64_t>(drow) * p.n + dtok) * (p.k / 32) + dblk] = static_cast<int32_t>(dot[t & 1][e] * 262144.0f);
            }
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[tn][e] = fmaf(dot[t & 1][e], sct[(t >> 1) & 1][16 * jb + e], acc[tn][e]);
        // pin the FMAs here: without it instruction selection sinks them to the end of the
        // super-block and every matrix-core result is spilled on the way
        asm volatile("" : "+v"(acc[tn]));
    };
    // min terms of the super-block in progress: acc -= sum_b (dmin*mn)[row][b] * (xs*sum a)[tok][b]
    auto mins = [&]() {
        uint32_t aw[12];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float rm = ndmin * static_cast<float>((mnb >> (8 * i)) & 0xFF);
            const uint32_t r0 = __builtin_bit_cast(uint32_t, rm) & 0xFFFF0000u;
            const float e1 = rm - __builtin_bit_cast(float, r0);
            const uint32_t r1 = __builtin_bit_cast(uint32_t, e1) & 0xFFFF0000u;
            const float e2 = e1 - __builtin_bit_cast(float, r1);
            const uint32_t r2 = __builtin_bit_cast(uint32_t, e2) & 0xFFFF0000u;
            // slots (r0, r0, r1, r0, r1, r2), low half first
            aw[3 * i + 0] = (r0 >> 16) | r0;
            aw[3 * i + 1] = (r1 >> 16) | r0;
            aw[3 * i + 2] = (r1 >> 16) | r2;
        }
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const uint4 b = *reinterpret_cast<const uint4*>(mnb_lds.b[tn] + j * 1024 + lane * 16);
                const uint4 a = make_uint4(aw[4 * j], aw[4 * j + 1], aw[4 * j + 2], aw[4 * j + 3]);
                acc[tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), acc[tn], 0, 0, 0);
            }
    };

    // ---- prologue: stage 0 (with the first super-block's min operands) and the weights of the first
    // super-block, then steps 0 (issued), 1 and 2 (read)
    stage_in(sb_begin, 0, st0, true, sb_begin);
    weights_in(sb_begin);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    __syncthreads();
    stage_in(sb_begin, 1, st1, false, 0);
    weights_read();
    __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the staged rows are in registers, their LDS copy is free
    weights_in(min(sb_begin + 1, sb_end - 1));
    decode_hdr();
    lds_read(0);
    lds_read(1);
    lds_read(2);
    issue_s(0);
    issue_d(0);

    for (uint32_t sb = sb_begin; sb < sb_end; ++sb) {
        const uint32_t sb_next = min(sb + 1, sb_end - 1);   // the last super-block re-requests itself: no branch around the loads
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            // matrix-core work of step t+1 first, everything else behind it.  (While a DMA into LDS is
            // in flight the compiler makes every wait for an LDS read a wait for ALL LDS reads, so the
            // reads of step t+3 are requested behind these instructions, not in front of them.)
            if (t == 15) decode_hdr();   // step 0 of the next super-block: its header
            __builtin_amdgcn_sched_barrier(0);
            issue_s((t + 1) & 15);
            __builtin_amdgcn_sched_barrier(0);
            if (t == 11) {
                // the min terms go here: their operands are read before the barrier of tick 13 lets the
                // next super-block's overwrite them
                mins();
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- the barrier that publishes the stage step t+3 starts, and the DMA of the stage after it
            if (t == 5 || t == 13) {
                __builtin_amdgcn_s_waitcnt(0x0F70);   // this wavefront's DMA of that stage has landed
                __syncthreads();
                if (t == 5) {
                    if (sb + 1 < sb_end) stage_in(sb + 1, 0, st0, false, 0);
                } else {
                    if (sb + 1 < sb_end) stage_in(sb + 1, 1, st1, true, sb + 1);
                    // the next super-block's rows into registers (landed: waited for above; every pair of this
                    // one is unpacked), then their LDS copy is free for the super-block after it
                    weights_read();
                    __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0)
                    weights_in(min(sb + 2, sb_end - 1));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            issue_d((t + 1) & 15);
            __builtin_amdgcn_sched_barrier(0);
            lds_read((t + 3) & 15);
            __builtin_amdgcn_sched_barrier(0);
            fma_step(t, sb);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- store: a lane holds token n0 + 32 tn + col and rows row0 + 8 blk + 4 half + r
    if (SWIGLU) {
        // The up wavefronts hand their tiles to the gate wavefronts through LDS (the stage buffers are
        // free after the last barrier): same lane, same register positions.
        float* const xch = reinterpret_cast<float*>(&st0);   // [wave % (NW/2)][tn][e][lane], 8 KB per wavefront
        static_assert(sizeof(G8Stage) >= (NW / 2) * 8192 || NW == 8, "exchange area");
        float* const xch2 = NW == 8 ? reinterpret_cast<float*>(&st1) : xch;   // waves 2, 3 of four pairs use the second buffer
        const uint32_t xw = wave % (NW / 2);
        float* const myx = (xw >= 2 ? xch2 : xch) + (xw & 1) * 2048;
        if (wave >= NW / 2) {
#pragma unroll
            for (int tn = 0; tn < 2; ++tn)
#pragma unroll
                for (int e = 0; e < 16; ++e) myx[(tn * 16 + e) * 64 + lane] = acc[tn][e];
        }
        __syncthreads();
        if (wave >= NW / 2) return;
        // h = silu(gate) * up (cera/src/backend/cpu.rs:2570-2575), then the Q8_0 block of this token's
        // rows row0 .. row0+31 (cpu.rs:942-958): this lane holds 16 of them, lane ^ 32 the others
#pragma unroll
        for (int tn = 0; tn < 2; ++tn) {
            const uint32_t tok = n0 + tn * 32 + col;
            float hv[16];
            float amax = 0.0f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float g = acc[tn][e], u = myx[(tn * 16 + e) * 64 + lane];
                hv[e] = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, cera_expf(-g))), u);
                amax = fmaxf(amax, fabsf(hv[e]));   // fmaxf drops a NaN operand, as f32::max does
            }
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            const float d = __fdiv_rn(amax, 127.0f), r = __fdiv_rn(1.0f, d);
            const float id = (d != 0.0f && fabsf(r) != __builtin_inff() && r == r) ? r : 0.0f;
            const float scale = h2f(f2h(d));
            uint32_t packed[4];
            uint2 halves[4];   // the same four quants as f16, in gemm_act_f16_kernel's order 0, 2, 1, 3
            int sum = 0;
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                packed[blk] = 0;
                uint32_t hb[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int v = q8_round(hv[4 * blk + q], id);
                    sum += v;
                    packed[blk] |= (static_cast<uint32_t>(v) & 0xFF) << (8 * q);
                    hb[q] = f2h(static_cast<float>(v));   // |v| <= 127: exact
                }
                halves[blk] = make_uint2(hb[0] | (hb[2] << 16), hb[1] | (hb[3] << 16));
            }
            sum += __shfl_xor(sum, 32, 64);
            if (tok < p.n && row0 < mrows) {   // m % 32 == 0: the block is whole or absent
#pragma unroll
                for (int blk = 0; blk < 4; ++blk)
                    *reinterpret_cast<uint32_t*>(p.hq + static_cast<uint64_t>(tok) * mrows + row0 + 8 * blk + 4 * half) = packed[blk];
                if (p.hh) {
#pragma unroll
                    for (int blk = 0; blk < 4; ++blk)
                        *reinterpret_cast<uint2*>(p.hh + static_cast<uint64_t>(tok) * mrows + row0 + 8 * blk + 4 * half) = halves[blk];
                }
                if (half == 0) {
                    const uint64_t b = static_cast<uint64_t>(tok) * (mrows / 32) + row0 / 32;
                    p.hs[b] = scale;
                    p.hbsum[b] = scale * static_cast<float>(sum);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
        const uint32_t tok = n0 + tn * 32 + col;
        if (tok >= p.n) continue;
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            const uint32_t row = row0 + blk * 8 + half * 4;
            if (p.ld_m == 1 && row + 3 < mrows && (ldn & 3) == 0) {
                // token-major output: the lane's four rows are 16 contiguous bytes
                const uint64_t idx = row + tok * ldn;
                float4 v = make_float4(acc[tn][blk * 4], acc[tn][blk * 4 + 1], acc[tn][blk * 4 + 2], acc[tn][blk * 4 + 3]);
                if (p.resid) {
                    const float4 r = *reinterpret_cast<const float4*>(p.resid + idx);
                    if (p.resid_scale != 1.0f) { v.x *= p.resid_scale; v.y *= p.resid_scale; v.z *= p.resid_scale; v.w *= p.resid_scale; }
                    v.x = r.x + v.x; v.y = r.y + v.y; v.z = r.z + v.z; v.w = r.w + v.w;
                }
                *reinterpret_cast<float4*>(omat + idx + blockIdx.z * p.part_stride) = v;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (row + r < mrows) {
                        float v = acc[tn][blk * 4 + r];
                        const uint64_t idx = (row + r) * p.ld_m + tok * ldn;
                        if (p.resid) v = p.resid[idx] + (p.resid_scale != 1.0f ? v * p.resid_scale : v);
                        omat[idx + blockIdx.z * p.part_stride] = v;
                    }
                }
            }
        }
    }
}
template <bool SWIGLU = false, bool DBG = false, int NW = G8_NW>
static __global__ __launch_bounds__(64 * NW, 8 / NW) void gemm_q4k_fp8_kernel(GemmArgs p) {
    gemm_q4k_fp8_body<SWIGLU, DBG, NW>(p);
}
