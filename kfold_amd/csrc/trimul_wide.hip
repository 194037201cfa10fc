// Triangle multiplication, input and output phases for a pair width C = D other than 128
// (C = 256: the shipping trunk, configs/kfold.yaml:3, model/modules/tri_stack.py:119-125).
// Same math and the same three-kernel structure as trimul.hip (which is tuned for C = 128):
//     trimul_in_wide_kernel   z -> planes ab[2C][Np][Np]
//     contract_kernel         (contract.hip, one product per channel)
//     trimul_out_wide_kernel  planes y[C][Np][Np] -> LN_out -> Wp_out -> * sigmoid(Wg_out LN_in(z))
// Reference: src/kfold/model/primitives/triangle_multiplication.py:212-229, :296-313.
//
// Packed blob for width C (block = 32 rows x C channels = 64*C bytes):
//   g_out   C/32 blocks (ROW_INTERLEAVE4)          gate weights are pre-multiplied by -log2(e)
//   a|b     C/16 steps x { p_in block, g_in block }
//   p_out   C/32 blocks (ROW_INTERLEAVE4, K_HALF)
//   fp32    ln_in gamma, beta, ln_out gamma, beta (C each)
#include "kernels.hpp"

namespace kfh {

template <int C> struct TmWide {
    static constexpr size_t blk = 64 * (size_t)C;
    static constexpr size_t gate = 0;
    static constexpr size_t ab = (C / 32) * blk;
    static constexpr size_t out = ab + (C / 8) * blk;
    static constexpr size_t ln = out + (C / 32) * blk;
    static constexpr size_t total = ln + 4 * (size_t)C * sizeof(float);
};

size_t trimul_wide_blob_bytes(int C) { return C == 256 ? TmWide<256>::total : 0; }
void trimul_wide_offsets(int C, size_t* gate, size_t* ab, size_t* out, size_t* ln, size_t* blk) {
    *gate = TmWide<256>::gate; *ab = TmWide<256>::ab; *out = TmWide<256>::out; *ln = TmWide<256>::ln;
    *blk = TmWide<256>::blk;
    (void)C;
}

// ------------------------------------------------------------------------------------------
// input phase: TILE positions of one line per workgroup, 32 per wavefront
// ------------------------------------------------------------------------------------------
template <int IO, int TILE, int C>
__global__ __launch_bounds__(TILE * 2) void trimul_in_wide_kernel(
    const void* __restrict__ z, const uint8_t* __restrict__ mask, const char* __restrict__ blob,
    uint16_t* __restrict__ planes, int N, int Np, int incoming, float eps) {
    constexpr int NT = TILE * 2, KS = C / 16;
    constexpr int STEP = 2 * (int)TmWide<C>::blk;                 // bytes of one weight step
    constexpr int SMEM = TILE * xs_bytes<C>() > 2 * STEP ? TILE * xs_bytes<C>() : 2 * STEP;
    __shared__ __attribute__((aligned(16))) char smem[SMEM];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int line = blockIdx.y, t0 = blockIdx.x * TILE;
    const size_t plane_sz = (size_t)Np * Np;

    if (line >= N) {   // padded line: zeros in every plane
        const int t = t0 + 2 * (tid % (TILE / 2));
        if (t < Np) {
            for (int ch = tid / (TILE / 2); ch < 2 * C; ch += 4)
                *reinterpret_cast<uint32_t*>(planes + ch * plane_sz + (size_t)line * Np + t) = 0u;
        }
        return;
    }
    auto row_off = [&](int row) -> long long {
        const int t = t0 + row;
        if (t >= N) return -1;
        const size_t pos = incoming ? (size_t)t * N + line : (size_t)line * N + t;
        return (long long)(pos * C);
    };
    const u32x4* wsrc = reinterpret_cast<const u32x4*>(blob + TmWide<C>::ab);
    constexpr int NPRE = STEP / 16 / NT;
    u32x4 pre[NPRE];
    auto prefetch = [&](int s) {
#pragma unroll
        for (int i = 0; i < NPRE; ++i) pre[i] = wsrc[(size_t)s * (STEP / 16) + i * NT + tid];
    };
    stage_ln_rows_c<IO, TILE, C, decltype(row_off), NT>(
        smem, z, reinterpret_cast<const float*>(blob + TmWide<C>::ln), eps, tid, row_off);
    prefetch(0);
    __syncthreads();

    const int tpos = t0 + wave * 32 + col;
    bf16x8 xf[KS];
    bool valid = false;
    if (tpos < N) {
        const size_t pos = incoming ? (size_t)tpos * N + line : (size_t)line * N + tpos;
        valid = mask[pos] != 0;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        // fragments of masked positions are zero: ab = p * sigmoid(g) * mask without a multiply
        u32x4 w = __builtin_bit_cast(u32x4, lds_frag_c<C>(smem, wave * 32 + col, ks, half));
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = valid ? w[i] : 0u;
        xf[ks] = __builtin_bit_cast(bf16x8, w);
    }
    __syncthreads();

    constexpr int NSTEP = C / 16;      // 32 channels of a|b per step
    auto commit = [&](int s) {
#pragma unroll
        for (int i = 0; i < NPRE; ++i)
            reinterpret_cast<u32x4*>(smem + (s & 1) * STEP)[i * NT + tid] = pre[i];
    };
    auto wfrag = [&](int s, int blk, int ks) {
        return *reinterpret_cast<const bf16x8*>(smem + (s & 1) * STEP + blk * (STEP / 2) + ks * 1024 + lane * 16);
    };
    commit(0);
    __syncthreads();
#pragma unroll 1
    for (int s = 0; s < NSTEP; ++s) {
        if (s + 1 < NSTEP) prefetch(s + 1);
        f32x16 acc[2];
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
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

// ------------------------------------------------------------------------------------------
// output phase: 64 positions of one row i per workgroup (4 wavefronts: 2 position blocks x 2
// halves of the output channels).  Both operand tiles live in LDS as bf16 rows [position][C]:
// LN_in(z) and LN_out(y) (the y planes are transposed through registers).
// ------------------------------------------------------------------------------------------
template <int IO, int C>
__global__ __launch_bounds__(256) void trimul_out_wide_kernel(
    const uint16_t* __restrict__ planes_y, const void* z, const char* __restrict__ blob,
    const void* residual, void* out, int N, int Np, float eps) {
    constexpr int P = 64, KS = C / 16;
    constexpr int XS = xs_bytes<C>();
    __shared__ __attribute__((aligned(16))) char xt[P * XS];     // LN_in(z)  [position][C]
    __shared__ __attribute__((aligned(16))) char yt[P * XS];     // LN_out(y) [position][C]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int i = blockIdx.y, j0 = blockIdx.x * P;
    const float* lnp = reinterpret_cast<const float*>(blob + TmWide<C>::ln);

    auto row_off = [&](int row) -> long long {
        const int j = j0 + row;
        if (j >= N) return -1;
        return (long long)(((size_t)i * N + j) * C);
    };
    stage_ln_rows_c<IO, P, C, decltype(row_off), 256>(xt, z, lnp, eps, tid, row_off);

    // y: thread (position p = tid & 63, channel quarter cq = tid >> 6) reads C/4 channels of its
    // position from the planes (64 consecutive positions per channel: 128-byte segments), the
    // four quarters of a position meet through LDS for the LayerNorm statistics
    {
        __shared__ float red[2][4][P];
        const int p = tid & 63, cq = tid >> 6;
        constexpr int CQ = C / 4;
        float y[CQ];
        float s = 0.f;
#pragma unroll
        for (int d = 0; d < CQ; ++d) {
            const uint16_t w = planes_y[((size_t)(cq * CQ + d) * Np + i) * Np + j0 + p];
            y[d] = __uint_as_float((uint32_t)w << 16);
            s += y[d];
        }
        red[0][cq][p] = s;
        __syncthreads();
        const float mean = (red[0][0][p] + red[0][1][p] + red[0][2][p] + red[0][3][p]) * (1.0f / C);
        float q = 0.f;
#pragma unroll
        for (int d = 0; d < CQ; ++d) { y[d] -= mean; q += y[d] * y[d]; }
        red[1][cq][p] = q;
        __syncthreads();
        const float rstd = __builtin_amdgcn_rsqf((red[1][0][p] + red[1][1][p] + red[1][2][p] + red[1][3][p]) * (1.0f / C) + eps);
        const float* gam = lnp + 2 * C + cq * CQ;
        const float* bet = lnp + 3 * C + cq * CQ;
#pragma unroll
        for (int d = 0; d < CQ; d += 2)
            *reinterpret_cast<uint32_t*>(yt + p * XS + (cq * CQ + d) * 2) =
                pack_bf16(y[d] * rstd * gam[d] + bet[d], y[d + 1] * rstd * gam[d + 1] + bet[d + 1]);
    }
    __syncthreads();

    // wavefront = (position block pb, channel group cg of 128 output channels)
    const int pb = wave & 1, cg = wave >> 1;
    static_assert(C == 256, "two channel groups of 128");
    f32x16 acc[4];
    const bf16x8* wo = reinterpret_cast<const bf16x8*>(blob + TmWide<C>::out);
    const bf16x8* wg = reinterpret_cast<const bf16x8*>(blob + TmWide<C>::gate);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[nb][v] = 0.f;
        // the p_out blocks use the K_HALF channel order: k-step ks of lane half h holds the
        // channels (C/2)*h + 8*ks + e, i.e. 16 bytes at that offset of the staged row
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 yf = *reinterpret_cast<const bf16x8*>(yt + (32 * pb + col) * XS + ((C / 2) * half + 8 * ks) * 2);
            acc[nb] = mfma32(yf, wo[((size_t)(4 * cg + nb) * KS + ks) * 64 + lane], acc[nb]);
        }
        f32x16 g;
#pragma unroll
        for (int v = 0; v < 16; ++v) g[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            g = mfma32(lds_frag_c<C>(xt, 32 * pb + col, ks, half), wg[((size_t)(4 * cg + nb) * KS + ks) * 64 + lane], g);
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[nb][v] *= fast_rcp(1.0f + fast_exp2(g[v]));
        __builtin_amdgcn_sched_barrier(0);
    }
    // block nb, lane col <-> channel 128*cg + 4*col + nb
    const int c0 = 128 * cg + 4 * col;
#pragma unroll
    for (int h8 = 0; h8 < 2; ++h8) {
        u32x2 rb[8];
        f32x4 rf[8];
        if (residual) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = j0 + 32 * pb + acc_row(8 * h8 + u, half);
                const size_t e0 = ((size_t)i * N + min(j, N - 1)) * C + c0;
                if constexpr (IO == KFH_BF16)
                    rb[u] = *reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(residual) + e0);
                else
                    rf[u] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(residual) + e0);
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int v = 8 * h8 + u;
            const int j = j0 + 32 * pb + acc_row(v, half);
            if (j < N) {
                const size_t e0 = ((size_t)i * N + j) * C + c0;
                float o0 = acc[0][v], o1 = acc[1][v], o2 = acc[2][v], o3 = acc[3][v];
                if constexpr (IO == KFH_BF16) {
                    if (residual) {
                        o0 += bf16_lo(rb[u][0]); o1 += bf16_hi(rb[u][0]);
                        o2 += bf16_lo(rb[u][1]); o3 += bf16_hi(rb[u][1]);
                    }
                    u32x2 o = {pack_bf16(o0, o1), pack_bf16(o2, o3)};
                    *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + e0) = o;
                } else {
                    if (residual) { o0 += rf[u][0]; o1 += rf[u][1]; o2 += rf[u][2]; o3 += rf[u][3]; }
                    f32x4 o = {o0, o1, o2, o3};
                    *reinterpret_cast<f32x4*>(static_cast<float*>(out) + e0) = o;
                }
            }
        }
    }
}

int launch_trimul_in_wide(const void* z, int io_dtype, const uint8_t* mask, const char* blob, uint16_t* planes,
                          int N, int Np, int C, int incoming, float eps, hipStream_t stream) {
    if (C != 256) return -1;
    constexpr int TILE = 128;
    dim3 grid((Np + TILE - 1) / TILE, Np), block(TILE * 2);
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL((trimul_in_wide_kernel<KFH_F32, TILE, 256>), grid, block, 0, stream, z, mask, blob,
                           planes, N, Np, incoming, eps);
    else
        hipLaunchKernelGGL((trimul_in_wide_kernel<KFH_BF16, TILE, 256>), grid, block, 0, stream, z, mask, blob,
                           planes, N, Np, incoming, eps);
    return 0;
}

int launch_trimul_out_wide(const uint16_t* planes_y, const void* z, const char* blob, const void* residual,
                           void* out, int io_dtype, int N, int Np, int C, float eps, hipStream_t stream,
                           int row0, int nrows) {
    if (C != 256) return -1;
    if (nrows < 0) { row0 = 0; nrows = N; }
    if (nrows == 0) return 0;
    // rows [row0, row0 + nrows): blockIdx.y is the row, so every operand is entered row0 rows down
    const size_t esz = io_dtype == KFH_F32 ? 4 : 2, shift = (size_t)row0 * N * C * esz;
    planes_y += (size_t)row0 * Np;
    z = static_cast<const char*>(z) + shift;
    if (residual) residual = static_cast<const char*>(residual) + shift;
    out = static_cast<char*>(out) + shift;
    dim3 grid((N + 63) / 64, nrows), block(256);
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL((trimul_out_wide_kernel<KFH_F32, 256>), grid, block, 0, stream, planes_y, z, blob,
                           residual, out, N, Np, eps);
    else
        hipLaunchKernelGGL((trimul_out_wide_kernel<KFH_BF16, 256>), grid, block, 0, stream, planes_y, z, blob,
                           residual, out, N, Np, eps);
    return 0;
}

}  // namespace kfh
