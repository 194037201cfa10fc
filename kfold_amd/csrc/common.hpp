// Shared device helpers for the gfx950 (CDNA4) kernels of the Pairformer pair-update path.
//
// Conventions used by every kernel in this directory
// --------------------------------------------------
// * Wavefront = 64 lanes.  lane = threadIdx.x & 63, half = lane >> 5, col = lane & 31.
// * MFMA v_mfma_f32_32x32x16_bf16, D[32x32] += A[32x16] * B[16x32]:
//     A operand: lane holds A[row = col][k = 8*half + 0..7]          (8 bf16 = one "fragment")
//     B operand: lane holds B[k = 8*half + 0..7][column = col]
//     D / C    : lane holds D[row = 8*(v/4) + 4*half + (v%4)][column = col], v = 0..15
//   A and B fragments have the same register shape, so one fragment of a
//   [32 rows x 16 k] operand block can be fed to either side.
// * "Fragment order" in memory: a [32 x 16] operand block is stored as 64 lanes x 16 bytes
//   (1 KiB, lane-major), so that a wavefront loads or stores a whole fragment with one
//   fully coalesced 16-byte-per-lane access.
// * Because a contraction is a sum, the k-slots of a fragment may hold any permutation of
//   the true k indices as long as both operands use the same one.  Accumulator registers
//   converted to bf16 are re-used directly as fragments of the next MFMA: register group
//   v = 8*ks + e (e = 0..7) becomes k-step ks, and lane (col, half) then holds the true
//   indices  8*(e/4) + 4*half + (e%4) + 16*ks  (KPERM_ACC below).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kfold_hip.h"   // KFH_BF16 / KFH_F32 and the error codes

namespace kfh {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// round-to-nearest-even pack of two floats into one dword of two bf16 (lo = a, hi = b)
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    bf16x2 v = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, v);
}

// x rounded to the nearest bf16 value, as a float
__device__ __forceinline__ float bf16_round(float x) { return bf16_lo(pack_bf16(x, 0.f)); }

// Three-way split of an fp32 value into bf16-representable parts, x = p[0] + p[1] + p[2] to
// fp32 accuracy (8 + 8 + 8 significant bits; the two subtractions are exact).  A product of two
// split operands summed over the part pairs (i, j) with i + j <= 2, each an exact bf16 x bf16
// product accumulated in fp32, carries fp32 accuracy: this is how the matrix cores run the
// fp32 ("ieee") arithmetic of the diffusion stack.
__device__ __forceinline__ void split3(float x, float (&p)[3]) {
    p[0] = bf16_round(x);
    const float r = x - p[0];
    p[1] = bf16_round(r);
    p[2] = bf16_round(r - p[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float sigmoidf_fast(float x) {
    return fast_rcp(1.0f + fast_exp2(-kLog2e * x));
}

// Exchange between lane l and lane l^32.  r0/r1 hold {own, partner} in the lower half and
// {partner, own} in the upper half, so symmetric reductions need no select.
__device__ __forceinline__ float xhalf_max(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// 16 accumulator values -> two fragments (k-steps) in KPERM_ACC order.
__device__ __forceinline__ void acc_to_frags(const f32x16& c, bf16x8& f0, bf16x8& f1) {
    u32x4 a, b;
    a[0] = pack_bf16(c[0], c[1]);   a[1] = pack_bf16(c[2], c[3]);
    a[2] = pack_bf16(c[4], c[5]);   a[3] = pack_bf16(c[6], c[7]);
    b[0] = pack_bf16(c[8], c[9]);   b[1] = pack_bf16(c[10], c[11]);
    b[2] = pack_bf16(c[12], c[13]); b[3] = pack_bf16(c[14], c[15]);
    f0 = __builtin_bit_cast(bf16x8, a);
    f1 = __builtin_bit_cast(bf16x8, b);
}

// Pair-bias tiles: a [32 queries x 32 keys] tile is stored in bf16 (2 KiB) in the register
// order of the transposed score accumulator S^T[key][query]: [chunk c][lane = query + 32*half][8],
// where element j of chunk c is accumulator register v = 8c + j, i.e. key
// 8*(v/4) + 4*half + v%4.  The attention kernels read a tile with two 16-byte loads per lane
// and widen it to the fp32 C operand of the first score MFMA.
constexpr int kBiasTileElems = 1024;
__host__ __device__ __forceinline__ int bias_tile_elem(int q32, int k32) {
    const int v = 4 * (k32 >> 3) + (k32 & 3), lane = q32 + 32 * ((k32 >> 2) & 1);
    return ((v >> 3) * 64 + lane) * 8 + (v & 7);
}
// the two 16-byte chunks of a tile held by this lane -> fp32 accumulator registers
__device__ __forceinline__ f32x16 bias_tile_acc(const u32x4& c0, const u32x4& c1) {
    f32x16 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        r[2 * i] = __uint_as_float(c0[i] << 16);
        r[2 * i + 1] = __uint_as_float(c0[i] & 0xffff0000u);
        r[8 + 2 * i] = __uint_as_float(c1[i] << 16);
        r[8 + 2 * i + 1] = __uint_as_float(c1[i] & 0xffff0000u);
    }
    return r;
}

// fp32 tiles of the fp32 arithmetic: [chunk c = 0..3][lane][4], element j of chunk c is
// accumulator register v = 4c + j (4 KiB per tile, four 16-byte loads per lane)
constexpr int kBiasTileF32Bytes = 4096;
__host__ __device__ __forceinline__ int bias_tile_f32_elem(int q32, int k32) {
    const int v = 4 * (k32 >> 3) + (k32 & 3), lane = q32 + 32 * ((k32 >> 2) & 1);
    return ((v >> 2) * 64 + lane) * 4 + (v & 3);
}

// row index inside a 32x32 accumulator block for register v of this lane
__device__ __forceinline__ int acc_row(int v, int half) { return 8 * (v >> 2) + 4 * half + (v & 3); }

// ---------------------------------------------------------------------------------------
// Staging tile of LayerNorm-ed rows in LDS: 128 bf16 channels per row, row stride 272 bytes
// (16 bytes of padding keep 16-byte fragment reads of consecutive rows on distinct banks).
// ---------------------------------------------------------------------------------------
constexpr int kC = 128;            // channels of the pair representation handled by the fused kernels
constexpr int kXS = 272;           // bytes per staged row
constexpr int kKS = kC / 16;       // k-steps per 128-channel contraction

// fragment ks (0..7) of staged row `row` for this lane: channels 16*ks + 8*half + 0..7
__device__ __forceinline__ bf16x8 lds_frag(const char* tile, int row, int ks, int half) {
    return *reinterpret_cast<const bf16x8*>(tile + row * kXS + ks * 32 + half * 16);
}

template <int IO> struct IoT;
template <> struct IoT<KFH_BF16> { using type = uint16_t; };
template <> struct IoT<KFH_F32> { using type = float; };

// Load 8 consecutive channels of one row as floats.
template <int IO>
__device__ __forceinline__ void load8(const void* base, size_t elem_off, float (&x)[8]) {
    if constexpr (IO == KFH_BF16) {
        u32x4 w = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + elem_off);
#pragma unroll
        for (int i = 0; i < 4; ++i) { x[2 * i] = bf16_lo(w[i]); x[2 * i + 1] = bf16_hi(w[i]); }
    } else {
        const f32x4* p = reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + elem_off);
        f32x4 a = p[0], b = p[1];
#pragma unroll
        for (int i = 0; i < 4; ++i) { x[i] = a[i]; x[4 + i] = b[i]; }
    }
}

// sum over the 16 lanes that share one row (lanes 16*g .. 16*g+15)
__device__ __forceinline__ float row16_sum(float v) {
    v += __shfl_xor(v, 1);
    v += __shfl_xor(v, 2);
    v += __shfl_xor(v, 4);
    v += __shfl_xor(v, 8);
    return v;
}

// LayerNorm of one 128-channel row held as 8 channels per lane over 16 lanes (two-pass,
// fp32 statistics, biased variance), result rounded to bf16 and packed.
__device__ __forceinline__ u32x4 ln_row16(const float (&x)[8], const float (&gam)[8],
                                          const float (&bet)[8], float eps) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += x[i];
    const float mean = row16_sum(s) * (1.0f / kC);
    float d[8], q = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) { d[i] = x[i] - mean; q += d[i] * d[i]; }
    const float rstd = __builtin_amdgcn_rsqf(row16_sum(q) * (1.0f / kC) + eps);
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float a = d[2 * i] * rstd * gam[2 * i] + bet[2 * i];
        float b = d[2 * i + 1] * rstd * gam[2 * i + 1] + bet[2 * i + 1];
        o[i] = pack_bf16(a, b);
    }
    return o;
}

// Stage ROWS LayerNorm-ed rows of 128 channels into an LDS tile (NTHREADS threads, 16 lanes
// per row).  `row_off(row)` returns the element offset of the row in `src`, or -1 for a row
// outside the tensor (staged as LN(0) = beta, finite).  `lnp` points at gamma[128], beta[128].
template <int IO, int ROWS, class RowOff, int NTHREADS = 256>
__device__ __forceinline__ void stage_ln_rows(char* tile, const void* src, const float* lnp,
                                              float eps, int tid, RowOff row_off) {
    constexpr int RG = NTHREADS / 16;          // rows in flight per iteration
    const int r16 = tid >> 4, ch = tid & 15;
    float gam[8], bet[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { gam[i] = lnp[ch * 8 + i]; bet[i] = lnp[kC + ch * 8 + i]; }
    // all rows of this thread are requested before the first is normalised: one memory latency
    // per tile instead of one per row
    constexpr int NIT = ROWS / RG;
    float x[NIT][8];
    bool valid[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const long long off = row_off(it * RG + r16);
        valid[it] = off >= 0;
        load8<IO>(src, (size_t)(valid[it] ? off : 0) + ch * 8, x[it]);
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const int row = it * RG + r16;
        if (!valid[it]) {
#pragma unroll
            for (int i = 0; i < 8; ++i) x[it][i] = 0.f;
        }
        *reinterpret_cast<u32x4*>(tile + row * kXS + ch * 16) = ln_row16(x[it], gam, bet, eps);
    }
}

// ---------------------------------------------------------------------------------------
// The same staging for a channel count C that is a multiple of 128 (C = 256: the shipping pair
// width): row stride 2*C + 16 bytes; a row is held by 16 lanes, lane ch owning the channels
// 128*j + 8*ch + 0..7 for j < C/128 (16-byte loads, 256 contiguous bytes per 16 lanes).
// ---------------------------------------------------------------------------------------
template <int C> constexpr int xs_bytes() { return 2 * C + 16; }

template <int C>
__device__ __forceinline__ bf16x8 lds_frag_c(const char* tile, int row, int ks, int half) {
    return *reinterpret_cast<const bf16x8*>(tile + row * xs_bytes<C>() + ks * 32 + half * 16);
}

// `src2` (may be null) is a second tensor of the same layout that is added before normalising.
template <int IO, int ROWS, int C, class RowOff, int NTHREADS = 256>
__device__ __forceinline__ void stage_ln_rows_c(char* tile, const void* src, const float* lnp,
                                                float eps, int tid, RowOff row_off,
                                                const void* src2 = nullptr) {
    constexpr int NJ = C / 128;
    constexpr int RG = NTHREADS / 16, NIT = ROWS / RG;
    const int r16 = tid >> 4, ch = tid & 15;
    // rows in groups of at most 4 per thread: all loads of a group are requested before the
    // first row is normalised
    constexpr int GROUP = NIT < 4 ? NIT : 4;
    static_assert(NIT % GROUP == 0, "rows per thread");
#pragma unroll 1
    for (int g0 = 0; g0 < NIT; g0 += GROUP) {
        float x[GROUP][NJ][8];
        bool valid[GROUP];
#pragma unroll
        for (int it = 0; it < GROUP; ++it) {
            const long long off = row_off((g0 + it) * RG + r16);
            valid[it] = off >= 0;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                load8<IO>(src, (size_t)(valid[it] ? off : 0) + 128 * j + ch * 8, x[it][j]);
            if (src2) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    float y[8];
                    load8<IO>(src2, (size_t)(valid[it] ? off : 0) + 128 * j + ch * 8, y);
#pragma unroll
                    for (int i = 0; i < 8; ++i) x[it][j][i] += y[i];
                }
            }
        }
#pragma unroll
        for (int it = 0; it < GROUP; ++it) {
            const int row = (g0 + it) * RG + r16;
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (!valid[it]) x[it][j][i] = 0.f;
                    s += x[it][j][i];
                }
            const float mean = row16_sum(s) * (1.0f / C);
            float q = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    x[it][j][i] -= mean;
                    q += x[it][j][i] * x[it][j][i];
                }
            const float rstd = __builtin_amdgcn_rsqf(row16_sum(q) * (1.0f / C) + eps);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const float* gam = lnp + 128 * j + ch * 8;
                const float* bet = lnp + C + 128 * j + ch * 8;
                u32x4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    o[i] = pack_bf16(x[it][j][2 * i] * rstd * gam[2 * i] + bet[2 * i],
                                     x[it][j][2 * i + 1] * rstd * gam[2 * i + 1] + bet[2 * i + 1]);
                *reinterpret_cast<u32x4*>(tile + row * xs_bytes<C>() + 256 * j + ch * 16) = o;
            }
        }
    }
}

}  // namespace kfh
