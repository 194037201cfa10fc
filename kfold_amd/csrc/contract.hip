// Triangle-multiplication contraction: for every channel d an NT product on bf16 planes,
//     Y_d[i][j] = sum_k A_d[i][k] * B_d[j][k],      fp32 accumulation, bf16 result.
// (the einsum of src/kfold/model/primitives/triangle_multiplication.py:224 / :308 after the
// input phase has laid a and b out channel-major; planes are Np x Np, zero padded).
//
// Workgroup = 4 wavefronts in a 2x2 grid, each owning WM x WN accumulator blocks of 32x32.
// K is walked in tiles of 32 through double-buffered LDS; the next tile's global loads are
// issued before the current tile's MFMAs.  Rows of the B tile are stored to LDS permuted
// (row WN*c + n of a wavefront's range goes to block n, column c) so that after the MFMA a
// lane owns WN adjacent output columns and writes them with one store.
//
// Workgroups are numbered so that all tiles of one channel run on the same XCD (workgroup
// ids are dealt round-robin over the 8 XCDs): the two planes of a channel are then read
// from HBM once and served from that XCD's L2 afterwards.
#include "kernels.hpp"

namespace kfh {

template <int WM, int WN>
__global__ __launch_bounds__(256) void contract_kernel(const uint16_t* __restrict__ A,
                                                       const uint16_t* __restrict__ B,
                                                       uint16_t* __restrict__ Y, int Np,
                                                       int tiles_m, int tiles_n) {
    constexpr int BM = 64 * WM, BN = 64 * WN, BK = 32;
    constexpr int RS = 80;                  // bytes per LDS row: 32 bf16 + 16 B padding
    constexpr int SKEW = 64;                // extra bytes per 32-row group of the B tile
    constexpr int A_BYTES = BM * RS;
    constexpr int B_BYTES = BN * RS + (BN / 32) * SKEW;
    __shared__ __attribute__((aligned(16))) char lds[2 * (A_BYTES + B_BYTES)];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    const int tiles = tiles_m * tiles_n;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int d = (local / tiles) * 8 + xcd;
    const int tile = local % tiles;
    const int tm = tile / tiles_n, tn = tile % tiles_n;

    const uint16_t* Ad = A + (size_t)d * Np * Np + (size_t)tm * BM * Np;
    const uint16_t* Bd = B + (size_t)d * Np * Np + (size_t)tn * BN * Np;

    constexpr int ITA = BM / 64, ITB = BN / 64;
    const int lrow = tid >> 2, lchunk = tid & 3;
    u32x4 ra[ITA], rb[ITB];
    // LDS byte offset of B-tile row g (0..BN-1) after the column permutation
    int boff[ITB];
#pragma unroll
    for (int it = 0; it < ITB; ++it) {
        const int g = lrow + 64 * it;
        const int w = g / (32 * WN), gl = g % (32 * WN);
        const int blk = w * WN + gl % WN;             // 32-row group in LDS
        boff[it] = (blk * 32 + gl / WN) * RS + blk * SKEW + lchunk * 16;
    }

    auto gload = [&](int kt) {
#pragma unroll
        for (int it = 0; it < ITA; ++it)
            ra[it] = *reinterpret_cast<const u32x4*>(Ad + (size_t)(lrow + 64 * it) * Np + kt * BK + lchunk * 8);
#pragma unroll
        for (int it = 0; it < ITB; ++it)
            rb[it] = *reinterpret_cast<const u32x4*>(Bd + (size_t)(lrow + 64 * it) * Np + kt * BK + lchunk * 8);
    };
    auto lstore = [&](int buf) {
        char* as = lds + buf * (A_BYTES + B_BYTES);
        char* bs = as + A_BYTES;
#pragma unroll
        for (int it = 0; it < ITA; ++it)
            *reinterpret_cast<u32x4*>(as + (lrow + 64 * it) * RS + lchunk * 16) = ra[it];
#pragma unroll
        for (int it = 0; it < ITB; ++it) *reinterpret_cast<u32x4*>(bs + boff[it]) = rb[it];
    };

    f32x16 acc[WM][WN];
#pragma unroll
    for (int m = 0; m < WM; ++m)
#pragma unroll
        for (int n = 0; n < WN; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[m][n][v] = 0.f;

    const int KT = Np / BK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) gload(kt + 1);
        const char* as = lds + cur * (A_BYTES + B_BYTES);
        const char* bs = as + A_BYTES;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 af[WM], bf[WN];
#pragma unroll
            for (int m = 0; m < WM; ++m)
                af[m] = *reinterpret_cast<const bf16x8*>(as + ((wm * WM + m) * 32 + col) * RS + ks * 32 + half * 16);
#pragma unroll
            for (int n = 0; n < WN; ++n) {
                const int blk = wn * WN + n;
                bf[n] = *reinterpret_cast<const bf16x8*>(bs + (blk * 32 + col) * RS + blk * SKEW + ks * 32 + half * 16);
            }
#pragma unroll
            for (int m = 0; m < WM; ++m)
#pragma unroll
                for (int n = 0; n < WN; ++n) acc[m][n] = mfma32(af[m], bf[n], acc[m][n]);
        }
        if (kt + 1 < KT) lstore(cur ^ 1);
        __syncthreads();
    }

    // lane (col, half) owns rows acc_row(v, half) and the WN adjacent columns WN*col + n
    uint16_t* Yd = Y + (size_t)d * Np * Np;
    const int jbase = tn * BN + wn * 32 * WN + WN * col;
#pragma unroll
    for (int m = 0; m < WM; ++m) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int i = tm * BM + (wm * WM + m) * 32 + acc_row(v, half);
            uint16_t* dst = Yd + (size_t)i * Np + jbase;
            if constexpr (WN == 4) {
                u32x2 o = {pack_bf16(acc[m][0][v], acc[m][1][v]), pack_bf16(acc[m][2][v], acc[m][3][v])};
                *reinterpret_cast<u32x2*>(dst) = o;
            } else {
                static_assert(WN == 2, "WN must be 2 or 4");
                *reinterpret_cast<uint32_t*>(dst) = pack_bf16(acc[m][0][v], acc[m][1][v]);
            }
        }
    }
}

void launch_contract(const uint16_t* planes_a, const uint16_t* planes_b, uint16_t* planes_y,
                     int Np, int D, hipStream_t stream) {
    // Np is a multiple of 128; use 256x256 tiles when they divide it, else 128x128
    if (Np % 256 == 0) {
        const int t = Np / 256;
        hipLaunchKernelGGL((contract_kernel<4, 4>), dim3(D * t * t), dim3(256), 0, stream, planes_a,
                           planes_b, planes_y, Np, t, t);
    } else {
        const int t = Np / 128;
        hipLaunchKernelGGL((contract_kernel<2, 2>), dim3(D * t * t), dim3(256), 0, stream, planes_a,
                           planes_b, planes_y, Np, t, t);
    }
}

}  // namespace kfh
