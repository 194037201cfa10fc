// Triangle-multiplication contraction: for every channel d an NT product on bf16 planes,
//     Y_d[i][j] = sum_k A_d[i][k] * B_d[j][k],      fp32 accumulation, bf16 result.
// (the einsum of src/kfold/model/primitives/triangle_multiplication.py:224 / :308 after the
// input phase has laid a and b out channel-major; planes are Np x Np, zero padded).
//
// Workgroup = 4 wavefronts in a 2x2 grid, each owning WM x WN accumulator blocks of 32x32.
// K is walked in tiles of BK through double-buffered LDS with a third tile in flight in
// registers.  Rows of the B tile are stored to LDS permuted
// (row WN*c + n of a wavefront's range goes to block n, column c) so that after the MFMA a
// lane owns WN adjacent output columns and writes them with one store.
//
// Workgroups are numbered so that all tiles of one channel run on the same XCD (workgroup
// ids are dealt round-robin over the 8 XCDs): the two planes of a channel are then read
// from HBM once and served from that XCD's L2 afterwards.
#include "kernels.hpp"

namespace kfh {

template <int MASK, int N, int SYNC>
__device__ __forceinline__ void sched_group() {
    if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(MASK, N, SYNC);
}

// Instruction order of one k-step: NM MFMAs (mask 0x008) with the NFR fragment reads (0x100)
// and NLD operations of kind EXTRA (0x200 LDS stores, 0x020 global loads, 0 none) spread
// evenly between them.
template <int I, int NM, int NFR, int NLD, int EXTRA, int SYNC>
__device__ __forceinline__ void schedule_kstep() {
    if constexpr (I < NM) {
        sched_group<0x100, ((I + 1) * NFR) / NM - (I * NFR) / NM, SYNC>();
        if constexpr (EXTRA != 0) sched_group<EXTRA, ((I + 1) * NLD) / NM - (I * NLD) / NM, SYNC>();
        sched_group<0x008, 1, SYNC>();
        schedule_kstep<I + 1, NM, NFR, NLD, EXTRA, SYNC>();
    }
}

template <int WM, int WN, int BK, int OCC>
__global__ __launch_bounds__(256, OCC) void contract_kernel(const uint16_t* __restrict__ A,
                                                       const uint16_t* __restrict__ B,
                                                       uint16_t* __restrict__ Y, int Np,
                                                       int tiles_m, int tiles_n) {
    constexpr int BM = 64 * WM, BN = 64 * WN;
    constexpr int RS = BK * 2 + 16;         // bytes per LDS row: BK bf16 + 16 B padding
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

    constexpr int CPR = BK / 8;             // 16-byte chunks per tile row
    constexpr int RPP = 256 / CPR;          // rows per pass of the 256 threads
    constexpr int ITA = BM / RPP, ITB = BN / RPP;
    const int lrow = tid / CPR, lchunk = tid % CPR;
    u32x4 ra[ITA], rb[ITB];
    // LDS byte offset of B-tile row g (0..BN-1) after the column permutation
    int boff[ITB];
#pragma unroll
    for (int it = 0; it < ITB; ++it) {
        const int g = lrow + RPP * it;
        const int w = g / (32 * WN), gl = g % (32 * WN);
        const int blk = w * WN + gl % WN;             // 32-row group in LDS
        boff[it] = (blk * 32 + gl / WN) * RS + blk * SKEW + lchunk * 16;
    }

    auto gload = [&](int kt) {
#pragma unroll
        for (int it = 0; it < ITA; ++it)
            ra[it] = *reinterpret_cast<const u32x4*>(Ad + (size_t)(lrow + RPP * it) * Np + kt * BK + lchunk * 8);
#pragma unroll
        for (int it = 0; it < ITB; ++it)
            rb[it] = *reinterpret_cast<const u32x4*>(Bd + (size_t)(lrow + RPP * it) * Np + kt * BK + lchunk * 8);
    };
    auto lstore = [&](int buf) {
        char* as = lds + buf * (A_BYTES + B_BYTES);
        char* bs = as + A_BYTES;
#pragma unroll
        for (int it = 0; it < ITA; ++it)
            *reinterpret_cast<u32x4*>(as + (lrow + RPP * it) * RS + lchunk * 16) = ra[it];
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

    constexpr int KS = BK / 16;             // MFMA k-steps per tile
    constexpr int NFR = WM + WN;            // fragment reads per k-step
    constexpr int NM = WM * WN;             // MFMAs per k-step
    constexpr int NLD = ITA + ITB;          // tile loads (and LDS stores) per thread
    static_assert(KS == 2 || KS == 4, "schedule shape");

    bf16x8 af[2][WM], bf[2][WN];
    auto load_frags = [&](int buf, int ks, int slot) {
        const char* as = lds + buf * (A_BYTES + B_BYTES);
        const char* bs = as + A_BYTES;
#pragma unroll
        for (int m = 0; m < WM; ++m)
            af[slot][m] = *reinterpret_cast<const bf16x8*>(as + ((wm * WM + m) * 32 + col) * RS + ks * 32 + half * 16);
#pragma unroll
        for (int n = 0; n < WN; ++n) {
            const int blk = wn * WN + n;
            bf[slot][n] = *reinterpret_cast<const bf16x8*>(bs + (blk * 32 + col) * RS + blk * SKEW + ks * 32 + half * 16);
        }
    };
    auto mfmas = [&](int slot) {
#pragma unroll
        for (int m = 0; m < WM; ++m)
#pragma unroll
            for (int n = 0; n < WN; ++n) acc[m][n] = mfma32(af[slot][m], bf[slot][n], acc[m][n]);
    };

    // Software pipeline, one branch-free body per tile kt:
    //   registers -> LDS for tile kt+1, global -> registers for tile kt+2, and the fragments of
    //   k-step ks+1 are read from LDS while the MFMAs of k-step ks run.  The single barrier sits
    //   before the last k-step, whose MFMAs cover the first fragment reads of tile kt+1.
    // Tile indices past the end are clamped: the surplus loads and stores touch valid memory
    // that nothing reads afterwards.
    const int KT = Np / BK;
    gload(0);
    lstore(0);
    gload(KT > 1 ? 1 : 0);
    __syncthreads();
    load_frags(0, 0, 0);
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        lstore(cur ^ 1);
        gload(kt + 2 < KT ? kt + 2 : KT - 1);
        if constexpr (KS == 4) {
            load_frags(cur, 1, 1);
            mfmas(0);
            load_frags(cur, 2, 0);
            mfmas(1);
            load_frags(cur, 3, 1);
            mfmas(0);
            schedule_kstep<0, NM, NFR, NLD, 0x200, 0>();      // + LDS tile stores
            schedule_kstep<0, NM, NFR, NLD, 0x020, 0>();      // + global tile loads
            schedule_kstep<0, NM, NFR, NLD, 0, 0>();
        } else {
            load_frags(cur, 1, 1);
            mfmas(0);
            schedule_kstep<0, NM, NFR, NLD, 0x200, 0>();
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        load_frags(cur ^ 1, 0, 0);
        mfmas(1);
        if constexpr (KS == 4) schedule_kstep<0, NM, NFR, NLD, 0, 1>();
        else schedule_kstep<0, NM, NFR, NLD, 0x020, 1>();
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
                     int Np, int D, hipStream_t stream, int row0, int nrows) {
    // Np is a multiple of 128; use 256x256 tiles when they divide it, else 128x128.
    // (192x256 tiles fill the CUs evenly at Np = 768, 6 rounds instead of 4.5, but measured
    // slower: 189 against 161-177 us.)
    // a range of result rows = the tile rows that hold it: the A and Y planes are entered row0 rows
    // down (the plane stride stays Np * Np), B is used whole
    const int bm = contract_tile_rows(Np);
    if (nrows < 0) { row0 = 0; nrows = Np; }
    const int tm0 = row0 / bm, tm1 = (row0 + nrows + bm - 1) / bm;
    if (tm1 <= tm0) return;
    planes_a += (size_t)tm0 * bm * Np;
    planes_y += (size_t)tm0 * bm * Np;
    const int tn = Np / bm;
    if (bm == 256)
        hipLaunchKernelGGL((contract_kernel<4, 4, 64, 1>), dim3(D * (tm1 - tm0) * tn), dim3(256), 0, stream, planes_a,
                           planes_b, planes_y, Np, tm1 - tm0, tn);
    else
        hipLaunchKernelGGL((contract_kernel<2, 2, 64, 2>), dim3(D * (tm1 - tm0) * tn), dim3(256), 0, stream, planes_a,
                           planes_b, planes_y, Np, tm1 - tm0, tn);
}

}  // namespace kfh
