// Triangle multiplication, input and output phases (C = D = 128).
//
// Follows the math of the reference's torch path
// (src/kfold/model/primitives/triangle_multiplication.py:212-229 outgoing, :296-313
// incoming):
//     xn  = LN_in(z)
//     ab  = (Wp_in xn) * sigmoid(Wg_in xn) * mask          a = first D channels, b = last D
//     y   = sum_k a[i,k] b[j,k]   (outgoing)   |   sum_k a[k,i] b[k,j]   (incoming)
//     out = (Wp_out LN_out(y)) * sigmoid(Wg_out xn)
//
// trimul_in_kernel   z -> channel-major planes ab[2D][Np][Np] (bf16, zero padded)
// contract_kernel    (contract.hip) per channel d:  Y_d = A_d * B_d^T
// trimul_out_kernel  planes y[D][Np][Np] -> LN_out -> Wp_out -> * sigmoid(Wg_out LN_in(z)) (+ residual)
//                    -> out; the output gate is recomputed from z here (z is read for the residual
//                    anyway) instead of being stored by the input phase and read back
//
// For the incoming direction the input phase walks z down a column and stores the plane
// transposed (plane[d][i][k] = ab[k,i,d]), so the contraction is the same NT product.
#include "kernels.hpp"

namespace kfh {


// TILE positions per workgroup, 32 per wavefront: 32 fragment + 32 accumulator registers per
// lane keep the kernel at 4 wavefronts per SIMD, which the VALU-heavy LayerNorm and gating
// phases need; small tiles put several workgroups in different phases on one CU, so the
// load phase of one overlaps the MFMA phase of another.
template <int IO, int TILE>
__global__ __launch_bounds__(TILE * 2, 4) void trimul_in_kernel(
    const void* __restrict__ z, const uint8_t* __restrict__ mask, const char* __restrict__ blob,
    uint16_t* __restrict__ planes, int N, int Np, int incoming, float eps) {
    // staged LayerNorm rows first, then two 16 KiB weight buffers over the same memory
    constexpr int NT = TILE * 2;
    constexpr int SMEM = TILE * kXS > 32768 ? TILE * kXS : 32768;
    __shared__ __attribute__((aligned(16))) char smem[SMEM];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int line = blockIdx.y, t0 = blockIdx.x * TILE;
    const size_t plane_sz = (size_t)Np * Np;

    if (line >= N) {   // padded line: zeros in every plane
        const int t = t0 + 2 * (tid % (TILE / 2));
        if (t < Np) {
            for (int ch = tid / (TILE / 2); ch < 2 * kC; ch += 4)
                *reinterpret_cast<uint32_t*>(planes + ch * plane_sz + (size_t)line * Np + t) = 0u;
        }
        return;
    }

    // ---- phase A: load 256 rows, LayerNorm, stage as bf16 ---------------------------------
    auto row_off = [&](int row) -> long long {
        const int t = t0 + row;
        if (t >= N) return -1;
        const size_t pos = incoming ? (size_t)t * N + line : (size_t)line * N + t;
        return (long long)(pos * kC);
    };
    const u32x4* wsrc = reinterpret_cast<const u32x4*>(blob + kTmAbOff);
    constexpr int NPRE = 1024 / NT;
    u32x4 pre[NPRE];
    auto prefetch = [&](int s) {
#pragma unroll
        for (int i = 0; i < NPRE; ++i) pre[i] = wsrc[s * 1024 + i * NT + tid];
    };
    prefetch(0);        // the first weight step travels while the rows are loaded and normalised
    stage_ln_rows<IO, TILE, decltype(row_off), NT>(
        smem, z, reinterpret_cast<const float*>(blob + kTmLnOff), eps, tid, row_off);
    __syncthreads();

    // ---- phase B: fragments of this wavefront's 32 positions; lane col <-> position 32*wave + col
    const int tpos = t0 + wave * 32 + col;
    bf16x8 xf[kKS];
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) xf[ks] = lds_frag(smem, wave * 32 + col, ks, half);
    bool valid = false;
    if (tpos < N) {
        const size_t pos = incoming ? (size_t)tpos * N + line : (size_t)line * N + tpos;
        valid = mask[pos] != 0;
    }
    __syncthreads();

    // ---- phase C: 8 steps of two 32-column weight blocks (16 KiB), double-buffered in LDS:
    //   step s: a|b channels 32s .. 32s+31: { p_in block, g_in block } (weights = A operand)
    // Gate weights are packed pre-multiplied by -log2(e): sigmoid(g) = 1 / (1 + exp2(acc)).
    // The fragments of masked positions are zeroed first, which makes
    // ab = p * sigmoid(g) * mask come out as exact zeros without a multiply (no bias terms).
    constexpr int NSTEP = 8;
    auto commit = [&](int s) {
#pragma unroll
        for (int i = 0; i < NPRE; ++i)
            reinterpret_cast<u32x4*>(smem + (s & 1) * 16384)[i * NT + tid] = pre[i];
    };
    auto wfrag = [&](int s, int blk, int ks) {
        return *reinterpret_cast<const bf16x8*>(smem + (s & 1) * 16384 + blk * 8192 + ks * 1024 + lane * 16);
    };
    commit(0);
    __syncthreads();

#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) {
        u32x4 w = __builtin_bit_cast(u32x4, xf[ks]);
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = valid ? w[i] : 0u;
        xf[ks] = __builtin_bit_cast(bf16x8, w);
    }

    for (int s = 0; s < NSTEP; ++s) {
        if (s + 1 < NSTEP) prefetch(s + 1);
        f32x16 acc[2];
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) {
            acc[0] = mfma32(wfrag(s, 0, ks), xf[ks], acc[0]);
            acc[1] = mfma32(wfrag(s, 1, ks), xf[ks], acc[1]);
        }
        if (tpos < Np) {
            uint16_t* dst = planes + (size_t)(s * 32) * plane_sz + (size_t)line * Np + tpos;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float a0 = acc[0][v] * fast_rcp(1.0f + fast_exp2(acc[1][v]));
                dst[(size_t)acc_row(v, half) * plane_sz] = (uint16_t)(pack_bf16(a0, 0.f) & 0xffffu);
            }
        }
        if (s + 1 < NSTEP) commit(s + 1);
        __syncthreads();
    }
}

void launch_trimul_in(const void* z, int io_dtype, const uint8_t* mask, const char* blob,
                      uint16_t* planes, int N, int Np, int incoming, float eps, hipStream_t stream) {
    constexpr int TILE = 256;
    dim3 grid((Np + TILE - 1) / TILE, Np), block(TILE * 2);
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL((trimul_in_kernel<KFH_F32, TILE>), grid, block, 0, stream, z, mask, blob, planes,
                           N, Np, incoming, eps);
    else
        hipLaunchKernelGGL((trimul_in_kernel<KFH_BF16, TILE>), grid, block, 0, stream, z, mask, blob,
                           planes, N, Np, incoming, eps);
}

// -----------------------------------------------------------------------------------------
// output phase: 128 positions of one row i per workgroup, 32 per wavefront
// -----------------------------------------------------------------------------------------
template <int IO>
__global__ __launch_bounds__(256, 3) void trimul_out_kernel(
    const uint16_t* __restrict__ planes_y, const void* z, const char* __restrict__ blob,
    const void* residual, void* out, int N, int Np, float eps) {
    // first the LN_in(z) rows of the 128 positions [position][128 ch], then y [d][128 positions]
    __shared__ __attribute__((aligned(16))) char yt[kC * kXS];
    __shared__ float lnw[2 * kC];                                // LN_out gamma, beta
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int i = blockIdx.y, j0 = blockIdx.x * 128;
    // the y values of this tile travel while the z rows are loaded and normalised
    u32x4 yv[8];
    {
        const int r16 = tid >> 4, ch = tid & 15;
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int d = it * 16 + r16;
            yv[it] = *reinterpret_cast<const u32x4*>(planes_y + ((size_t)d * Np + i) * Np + j0 + ch * 8);
        }
        lnw[tid] = reinterpret_cast<const float*>(blob + kTmLnOff)[2 * kC + tid];
    }
    auto row_off = [&](int row) -> long long {
        const int j = j0 + row;
        if (j >= N) return -1;
        return (long long)(((size_t)i * N + j) * kC);
    };
    stage_ln_rows<IO, 128, decltype(row_off), 256>(yt, z, reinterpret_cast<const float*>(blob + kTmLnOff),
                                                   eps, tid, row_off);
    __syncthreads();
    // LN_in(z) fragments of this wavefront's 32 positions (A operand of the gate product)
    bf16x8 xf[kKS];
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) xf[ks] = lds_frag(yt, 32 * wave + col, ks, half);
    __syncthreads();
    {
        const int r16 = tid >> 4, ch = tid & 15;
#pragma unroll
        for (int it = 0; it < 8; ++it)
            *reinterpret_cast<u32x4*>(yt + (it * 16 + r16) * kXS + ch * 16) = yv[it];
    }
    __syncthreads();

    // lane (col, half) owns position 32*wave + col and channels d = 64*half + 0..63 (K_HALF)
    const int p = 32 * wave + col;
    float y[64];
    float s = 0.f;
#pragma unroll
    for (int dd = 0; dd < 64; ++dd) {
        const uint16_t w = *reinterpret_cast<const uint16_t*>(yt + (64 * half + dd) * kXS + p * 2);
        y[dd] = __uint_as_float((uint32_t)w << 16);
        s += y[dd];
    }
    const float mean = xhalf_sum(s) * (1.0f / kC);
    float q = 0.f;
#pragma unroll
    for (int dd = 0; dd < 64; ++dd) { y[dd] -= mean; q += y[dd] * y[dd]; }
    const float rstd = __builtin_amdgcn_rsqf(xhalf_sum(q) * (1.0f / kC) + eps);
    bf16x8 yf[kKS];
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) {
        u32x4 w;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int d0 = 64 * half + 8 * ks + 2 * e;
            const float a = y[8 * ks + 2 * e] * rstd * lnw[d0] + lnw[kC + d0];
            const float b = y[8 * ks + 2 * e + 1] * rstd * lnw[d0 + 1] + lnw[kC + d0 + 1];
            w[e] = pack_bf16(a, b);
        }
        yf[ks] = __builtin_bit_cast(bf16x8, w);
    }

    f32x16 acc[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[nb][v] = 0.f;
    const bf16x8* wo = reinterpret_cast<const bf16x8*>(blob + kTmOutOff);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks)
            acc[nb] = mfma32(yf[ks], wo[(nb * kKS + ks) * 64 + lane], acc[nb]);
        __builtin_amdgcn_sched_barrier(0);      // keep the weight loads of later blocks out of flight
    }

    // output gate sigmoid(Wg_out LN_in(z)): same block / lane <-> channel mapping as the projection
    // (ROW_INTERLEAVE4); the weights are packed times -log2(e), so sigmoid = 1 / (1 + exp2(acc))
    const bf16x8* wg = reinterpret_cast<const bf16x8*>(blob + kTmGateOff);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
        f32x16 g;
#pragma unroll
        for (int v = 0; v < 16; ++v) g[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) g = mfma32(xf[ks], wg[(nb * kKS + ks) * 64 + lane], g);
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[nb][v] *= fast_rcp(1.0f + fast_exp2(g[v]));
        __builtin_amdgcn_sched_barrier(0);
    }

    // block nb, lane col <-> channel 4*col + nb (ROW_INTERLEAVE4): 8 or 16 contiguous bytes per
    // lane.  Rows in two groups of 8: all residual values of a group are requested before its
    // first store, so one memory latency is paid per group and, with out aliasing residual, a
    // row is read before it is written.
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        u32x2 rb[8];
        f32x4 rf[8];
        if (residual) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = j0 + 32 * wave + acc_row(8 * g + u, half);
                const size_t e0 = ((size_t)i * N + min(j, N - 1)) * kC + 4 * col;
                if constexpr (IO == KFH_BF16)
                    rb[u] = *reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(residual) + e0);
                else
                    rf[u] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(residual) + e0);
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int v = 8 * g + u;
            const int j = j0 + 32 * wave + acc_row(v, half);
            if (j < N) {
                const size_t e0 = ((size_t)i * N + j) * kC + 4 * col;
                float o0 = acc[0][v], o1 = acc[1][v], o2 = acc[2][v], o3 = acc[3][v];
                if constexpr (IO == KFH_BF16) {
                    if (residual) {
                        o0 += bf16_lo(rb[u][0]); o1 += bf16_hi(rb[u][0]);
                        o2 += bf16_lo(rb[u][1]); o3 += bf16_hi(rb[u][1]);
                    }
                    u32x2 o = {pack_bf16(o0, o1), pack_bf16(o2, o3)};
                    *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + e0) = o;
                } else {
                    if (residual) {
                        o0 += rf[u][0]; o1 += rf[u][1]; o2 += rf[u][2]; o3 += rf[u][3];
                    }
                    f32x4 o = {o0, o1, o2, o3};
                    *reinterpret_cast<f32x4*>(static_cast<float*>(out) + e0) = o;
                }
            }
        }
    }
}

void launch_trimul_out(const uint16_t* planes_y, const void* z, const char* blob,
                       const void* residual, void* out, int io_dtype, int N, int Np, float eps,
                       hipStream_t stream, int row0, int nrows) {
    // rows [row0, row0 + nrows) of the result: the kernel's row index is blockIdx.y, so the range is
    // the same kernel entered row0 rows down every operand
    if (nrows < 0) { row0 = 0; nrows = N; }
    if (nrows == 0) return;
    const size_t esz = io_dtype == KFH_F32 ? 4 : 2, shift = (size_t)row0 * N * kC * esz;
    planes_y += (size_t)row0 * Np;
    z = static_cast<const char*>(z) + shift;
    if (residual) residual = static_cast<const char*>(residual) + shift;
    out = static_cast<char*>(out) + shift;
    dim3 grid((N + 127) / 128, nrows), block(256);
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL(trimul_out_kernel<KFH_F32>, grid, block, 0, stream, planes_y, z, blob,
                           residual, out, N, Np, eps);
    else
        hipLaunchKernelGGL(trimul_out_kernel<KFH_BF16>, grid, block, 0, stream, planes_y, z, blob,
                           residual, out, N, Np, eps);
}

}  // namespace kfh
