// Triangle attention (C = 128, H = 4 heads of 32), starting and ending node.
//
// Math of the reference's torch path (src/kfold/model/primitives/triangle_attention.py
// :375-434 with :246-335 and :132-152), written for x' = x (starting) or x' = x^T (ending,
// :400-402; the result is transposed back, :431-432):
//     xn         = LN(x')
//     beta[h,j,k] = (W_b xn[j,k])[h]
//     q,k,v,g    = W_{q,k,v,g} xn ,  q /= sqrt(32)
//     L[i,h,j,k] = q[i,j,h] . k[i,k,h] + beta[h,j,k] - 1e9 * (1 - mask'[i,k])
//     o[i,j,h]   = softmax_k(L) v[i,k,h] ;  out'[i,j] = W_o (o[i,j] * sigmoid(g[i,j]))
//
// triattn_proj_kernel  x' rows -> LN -> q,k,v in MFMA fragment order + bias tiles + key codes
// flash_kernel         (flash.hip) per (row, head, 32 queries): online-softmax attention
// triattn_out_kernel   o fragments * sigmoid(W_g LN(x')) -> W_o -> (+ residual) -> out (transposed
//                      back); the gate is recomputed from x' here (its rows are read for the
//                      residual anyway) instead of being stored by the projection kernel
//
// Fragment buffers: [row a][head h][position block of 32][k-step 0..1][lane][8 bf16], the
// accumulator-to-fragment order of common.hpp, so the three kernels exchange MFMA operands
// with fully coalesced 16-byte accesses and no layout conversion.  The logits are kept in
// the exp2 domain: W_q and W_b are packed pre-multiplied by log2(e).
//
// Masking follows the reference's finite -1e9 semantics: for a row with at least one valid
// key a masked key gets probability exactly 0; for a row with no valid key every real key
// gets the same logit (q.k + beta is absorbed by -1e9 in fp32), i.e. uniform attention.
#include "kernels.hpp"

namespace kfh {

constexpr int kH = 4;          // heads
constexpr int kTileA = 256;    // positions per workgroup in proj/out kernels (32 per wavefront)

__device__ __forceinline__ size_t frag_index(int a, int h, int blk, int ks, int nb, int lane) {
    return ((((size_t)a * kH + h) * nb + blk) * 2 + ks) * 64 + lane;
}

// key codes: 0 = beyond N (padding of the last block), 1 = masked, 2 = valid
// PB = position blocks of 32 per wavefront: the workgroup has 8 / PB wavefronts.  PB = 1 keeps
// the register count low enough for 4 wavefronts per SIMD.
template <int IO, int PB>
__global__ __launch_bounds__(512 / PB, (PB == 1 ? 4 : 2)) void triattn_proj_kernel(
    const void* __restrict__ x, const uint8_t* __restrict__ mask, const char* __restrict__ blob,
    bf16x8* __restrict__ qf, bf16x8* __restrict__ kf, bf16x8* __restrict__ vf,
    uint16_t* __restrict__ biast, uint8_t* __restrict__ codes, int N, int nb, int ending, float eps) {
    __shared__ __attribute__((aligned(16))) char smem[kTileA * kXS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int a = blockIdx.y, t0 = blockIdx.x * kTileA;

    constexpr int NT = 512 / PB;
    auto row_off = [&](int row) -> long long {
        const int b = t0 + row;
        if (b >= N) return -1;
        const size_t pos = ending ? (size_t)b * N + a : (size_t)a * N + b;
        return (long long)(pos * kC);
    };
    const u32x4* wsrc = reinterpret_cast<const u32x4*>(blob + kTaProjOff);
    constexpr int NPRE = 1024 / NT;
    u32x4 pre[NPRE];
    auto prefetch = [&](int s) {
#pragma unroll
        for (int i = 0; i < NPRE; ++i) pre[i] = wsrc[s * 1024 + i * NT + tid];
    };
    prefetch(0);        // the first weight step travels while the rows are loaded and normalised
    stage_ln_rows<IO, kTileA, decltype(row_off), NT>(
        smem, x, reinterpret_cast<const float*>(blob + kTaLnOff), eps, tid, row_off);
    __syncthreads();

    // wavefront = PB blocks of 32 positions starting at blk0; lane col <-> position 32*pb + col
    const int blk0 = (t0 + wave * 32 * PB) >> 5;
    bf16x8 xf[PB][kKS];
#pragma unroll
    for (int pb = 0; pb < PB; ++pb) {
        const int row = wave * 32 * PB + 32 * pb + col;
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) xf[pb][ks] = lds_frag(smem, row, ks, half);
        const int b = t0 + row;
        if (half == 0 && blk0 + pb < nb) {
            uint8_t code = 0;
            if (b < N) {
                const size_t pos = ending ? (size_t)b * N + a : (size_t)a * N + b;
                code = mask[pos] ? 2 : 1;
            }
            codes[(size_t)a * nb * 32 + b] = code;
        }
    }
    __syncthreads();

    // 7 steps of two 32-column weight blocks (16 KiB), double-buffered in LDS:
    //   0..3  { q_h , k_h }      channels as accumulator rows (weights = A operand)
    //   4, 5  { v_2s , v_2s+1 }  positions as rows (activations = A operand)
    //   6     { pair bias, - }   rows 0..3 of the block are the 4 heads
    auto commit = [&](int s) {
#pragma unroll
        for (int i = 0; i < NPRE; ++i)
            reinterpret_cast<u32x4*>(smem + (s & 1) * 16384)[i * NT + tid] = pre[i];
    };
    auto wfrag = [&](int s, int blk, int ks) {
        return *reinterpret_cast<const bf16x8*>(smem + (s & 1) * 16384 + blk * 8192 + ks * 1024 + lane * 16);
    };
    auto store_frags = [&](bf16x8* dst, int h, int pb, const f32x16& c) {
        bf16x8 f0, f1;
        acc_to_frags(c, f0, f1);
        dst[frag_index(a, h, blk0 + pb, 0, nb, lane)] = f0;
        dst[frag_index(a, h, blk0 + pb, 1, nb, lane)] = f1;
    };
    commit(0);
    __syncthreads();

    for (int s = 0; s < 6; ++s) {
        prefetch(s + 1);
        const bool vv = s >= 4;
        f32x16 acc[2][PB];
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int pb = 0; pb < PB; ++pb)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[b][pb][v] = 0.f;
        if (!vv) {
#pragma unroll
            for (int ks = 0; ks < kKS; ++ks) {
                const bf16x8 w0 = wfrag(s, 0, ks), w1 = wfrag(s, 1, ks);
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) {
                    acc[0][pb] = mfma32(w0, xf[pb][ks], acc[0][pb]);
                    acc[1][pb] = mfma32(w1, xf[pb][ks], acc[1][pb]);
                }
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < kKS; ++ks) {
                const bf16x8 w0 = wfrag(s, 0, ks), w1 = wfrag(s, 1, ks);
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) {
                    acc[0][pb] = mfma32(xf[pb][ks], w0, acc[0][pb]);
                    acc[1][pb] = mfma32(xf[pb][ks], w1, acc[1][pb]);
                }
            }
        }
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            if (blk0 + pb < nb) {
                if (!vv) {
                    store_frags(qf, s, pb, acc[0][pb]);
                    store_frags(kf, s, pb, acc[1][pb]);
                } else {
                    store_frags(vf, 2 * (s - 4), pb, acc[0][pb]);
                    store_frags(vf, 2 * (s - 4) + 1, pb, acc[1][pb]);
                }
            }
        }
        commit(s + 1);
        __syncthreads();
    }

    {
        // pair bias: x' position (a, b) is (query a, key b).  The heads are accumulator rows
        // 0..3, i.e. registers v = 0..3 of the lanes with half == 0.  Scatter into the bf16 tile
        // of (a/32, b/32) (layout: bias_tile_elem in common.hpp).
        f32x16 acc[PB];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[pb][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) {
            const bf16x8 w0 = wfrag(6, 0, ks);
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) acc[pb] = mfma32(w0, xf[pb][ks], acc[pb]);
        }
        if (half == 0) {
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                const int kblk = blk0 + pb;
                if (kblk < nb) {
                    const int e = bias_tile_elem(a & 31, col);   // lane col = key inside its block
#pragma unroll
                    for (int h = 0; h < kH; ++h) {
                        const size_t tile = ((size_t)h * nb + (a >> 5)) * nb + kblk;
                        biast[tile * kBiasTileElems + e] = (uint16_t)(pack_bf16(acc[pb][h], 0.f) & 0xffffu);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// output projection: out'[a][b] = W_o (o * sigmoid(W_g LN(x'[a][b]))), 32 positions per wavefront,
// 8 wavefronts (model/primitives/triangle_attention.py:269-283)
// ------------------------------------------------------------------------------------------
template <int IO>
__global__ __launch_bounds__(512, 2) void triattn_out_kernel(
    const bf16x8* __restrict__ of, const void* x, const char* __restrict__ blob, const void* residual,
    void* out, int N, int nb, int ending, float eps) {
    __shared__ __attribute__((aligned(16))) char smem[kTileA * kXS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int a = blockIdx.y, t0 = blockIdx.x * kTileA;
    const int blk = (t0 >> 5) + wave;

    // LN(x') rows of the tile -> LDS (every wavefront takes part, also one past the last block)
    auto row_off = [&](int row) -> long long {
        const int b = t0 + row;
        if (b >= N) return -1;
        const size_t pos = ending ? (size_t)b * N + a : (size_t)a * N + b;
        return (long long)(pos * kC);
    };
    stage_ln_rows<IO, kTileA, decltype(row_off), 512>(
        smem, x, reinterpret_cast<const float*>(blob + kTaLnOff), eps, tid, row_off);
    __syncthreads();
    if (blk >= nb) return;

    // (requesting the o fragments before the staging costs 6 more registers, which drops the
    // kernel to one workgroup per CU: 172 instead of 122 us at N = 768)
    bf16x8 xf[kKS];
#pragma unroll
    for (int h = 0; h < kH; ++h) {
        xf[2 * h] = of[frag_index(a, h, blk, 0, nb, lane)];
        xf[2 * h + 1] = of[frag_index(a, h, blk, 1, nb, lane)];
    }
    // gate of head h: channels as accumulator rows, so that the accumulator has the layout of
    // the o fragments (k-step = register group of 8, see acc_to_frags); the weights are packed
    // times -log2(e): sigmoid = 1 / (1 + exp2(acc))
    {
        bf16x8 zf[kKS];
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) zf[ks] = lds_frag(smem, wave * 32 + col, ks, half);
        const bf16x8* wg = reinterpret_cast<const bf16x8*>(blob + kTaGateOff);
#pragma unroll
        for (int h = 0; h < kH; ++h) {
            f32x16 g;
#pragma unroll
            for (int v = 0; v < 16; ++v) g[v] = 0.f;
#pragma unroll
            for (int ks = 0; ks < kKS; ++ks) g = mfma32(wg[(h * kKS + ks) * 64 + lane], zf[ks], g);
            const u32x4 o0 = __builtin_bit_cast(u32x4, xf[2 * h]), o1 = __builtin_bit_cast(u32x4, xf[2 * h + 1]);
            f32x16 og;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                og[2 * e] = bf16_lo(o0[e]) * fast_rcp(1.0f + fast_exp2(g[2 * e]));
                og[2 * e + 1] = bf16_hi(o0[e]) * fast_rcp(1.0f + fast_exp2(g[2 * e + 1]));
                og[8 + 2 * e] = bf16_lo(o1[e]) * fast_rcp(1.0f + fast_exp2(g[8 + 2 * e]));
                og[8 + 2 * e + 1] = bf16_hi(o1[e]) * fast_rcp(1.0f + fast_exp2(g[8 + 2 * e + 1]));
            }
            acc_to_frags(og, xf[2 * h], xf[2 * h + 1]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    auto elem0 = [&](int v) -> size_t {
        const int b = min(blk * 32 + acc_row(v, half), N - 1);
        const size_t pos = ending ? (size_t)b * N + a : (size_t)a * N + b;
        return pos * kC + 4 * col;
    };

    f32x16 acc[4];
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[n][v] = 0.f;
    const bf16x8* wo = reinterpret_cast<const bf16x8*>(blob + kTaOutOff);
#pragma unroll
    for (int n = 0; n < 4; ++n) {
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) acc[n] = mfma32(xf[ks], wo[(n * kKS + ks) * 64 + lane], acc[n]);
        __builtin_amdgcn_sched_barrier(0);      // keep the weight loads of later blocks out of flight
    }
    // Rows in two groups of 8: all residual values of a group are requested before its first
    // store, so one memory latency is paid per group and, with out aliasing residual, a row is
    // read before it is written.
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        u32x2 rb[8];
        f32x4 rf[8];
        if (residual) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if constexpr (IO == KFH_BF16)
                    rb[u] = *reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(residual) + elem0(8 * g + u));
                else
                    rf[u] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(residual) + elem0(8 * g + u));
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int v = 8 * g + u;
            const int b = blk * 32 + acc_row(v, half);
            if (b < N) {
                const size_t e0 = elem0(v);
                float o0 = acc[0][v], o1 = acc[1][v], o2 = acc[2][v], o3 = acc[3][v];
                if constexpr (IO == KFH_BF16) {
                    if (residual) {
                        const u32x2 r = rb[u];
                        o0 += bf16_lo(r[0]); o1 += bf16_hi(r[0]); o2 += bf16_lo(r[1]); o3 += bf16_hi(r[1]);
                    }
                    u32x2 o = {pack_bf16(o0, o1), pack_bf16(o2, o3)};
                    *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + e0) = o;
                } else {
                    if (residual) {
                        const f32x4 r = rf[u];
                        o0 += r[0]; o1 += r[1]; o2 += r[2]; o3 += r[3];
                    }
                    f32x4 o = {o0, o1, o2, o3};
                    *reinterpret_cast<f32x4*>(static_cast<float*>(out) + e0) = o;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
int launch_triattn(const void* x, int io_dtype, const uint8_t* mask, const char* blob,
                    const TriattnWorkspace& ws, const void* residual, void* out, int N, int ending,
                    float eps, int stages, hipStream_t stream, int row0, int nrows) {
    // The input phase always covers all rows (the pair bias of a row is made from every row).  The
    // attention and the output phase take the rows [row0, row0 + nrows) of x' (the transposed view
    // for the ending node): a row is blockIdx.y / an entry of the row loop in every kernel, so a
    // range is the same kernel entered row0 rows down its operands.
    if (nrows < 0) { row0 = 0; nrows = N; }
    const int nb = (N + 31) / 32;
    bf16x8* qf = static_cast<bf16x8*>(ws.qf);
    bf16x8* kf = static_cast<bf16x8*>(ws.kf);
    bf16x8* vf = static_cast<bf16x8*>(ws.vf);
    bf16x8* of = static_cast<bf16x8*>(ws.of);
    dim3 grid_rows((N + kTileA - 1) / kTileA, N), block(256);
    if (stages & KFH_STAGE_IN) {
        if (io_dtype == KFH_F32)
            hipLaunchKernelGGL((triattn_proj_kernel<KFH_F32, 1>), grid_rows, dim3(512), 0, stream, x, mask,
                               blob, qf, kf, vf, ws.biast, ws.codes, N, nb, ending, eps);
        else
            hipLaunchKernelGGL((triattn_proj_kernel<KFH_BF16, 1>), grid_rows, dim3(512), 0, stream, x, mask,
                               blob, qf, kf, vf, ws.biast, ws.codes, N, nb, ending, eps);
    }

    if (nrows == 0) return 0;
    const size_t row_frags = (size_t)kH * nb * 128;      // bf16x8 units of one row in q, k, v and o
    FlashArgs fa{};
    fa.qf = qf + row0 * row_frags; fa.kf = kf + row0 * row_frags; fa.vf = vf + row0 * row_frags;
    fa.gf = nullptr; fa.of = of + row0 * row_frags;
    fa.biast = ws.biast; fa.codes = ws.codes + (size_t)row0 * nb * 32;
    fa.nrows = nrows; fa.nb = nb; fa.H = kH; fa.bias_per_row = 0;
    if (stages & KFH_STAGE_CORE) {
        const int rc = launch_flash(fa, 32, stream, N);
        if (rc) return rc;
    }
    if (!(stages & KFH_STAGE_OUT)) return 0;

    // position (row a, b) of x' is element (a * N + b) * C of x, or (b * N + a) * C for the ending node
    const size_t esz = io_dtype == KFH_F32 ? 4 : 2;
    const size_t shift = (ending ? (size_t)row0 : (size_t)row0 * N) * kC * esz;
    const void* xr = static_cast<const char*>(x) + shift;
    const void* rr = residual ? static_cast<const char*>(residual) + shift : nullptr;
    void* outr = static_cast<char*>(out) + shift;
    const dim3 grid_out((N + kTileA - 1) / kTileA, nrows);
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL(triattn_out_kernel<KFH_F32>, grid_out, dim3(512), 0, stream, of + row0 * row_frags, xr, blob,
                           rr, outr, N, nb, ending, eps);
    else
        hipLaunchKernelGGL(triattn_out_kernel<KFH_BF16>, grid_out, dim3(512), 0, stream, of + row0 * row_frags, xr, blob,
                           rr, outr, N, nb, ending, eps);
    return 0;
}

}  // namespace kfh
