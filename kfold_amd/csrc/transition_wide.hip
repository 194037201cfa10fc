// Pair transition at C = 256 (expansion E = 2 or 4), fully fused — the kernel of transition.hip
// (C = 128) with the channel count as a template parameter:
//     out = [residual +] W_out ( silu(u) * v ),   [u, v] = W_sw LN(x)        (then * mask)
// Reference: src/kfold/model/layers/folding/transition.py:48-68 with
// primitives/activation.py:27-29; the optional mask multiply is the final `z * pair_mask` of
// modules/apo_module.py:172.
//
// Workgroup = 128 positions, 32 per wavefront.  The hidden activations never leave
// registers: each step computes 32 hidden channels of u and of v (channels as accumulator
// rows), and silu(u)*v rounded to bf16 is directly the A operand of the second GEMM, whose
// [32 positions x C channels] accumulators stay resident across the steps.  Weights of a
// step (u block, v block, the matching 32-column slice of W_out: 24 KiB at C = 128, 48 KiB at
// C = 256) are double-buffered in LDS.  C = 256 with expansion 4 is the transition of the
// shipping trunk block (model/modules/tri_stack.py:119-125), applied to all N^2 positions.
#include "kernels.hpp"

namespace kfh {

// TILE positions per workgroup, 32 per wavefront.
template <int IO, int E, int TILE, int C>
__global__ __launch_bounds__(TILE * 2, 1) void transition_wide_kernel(
    const void* __restrict__ x, const char* __restrict__ blob, const void* residual,
    const uint8_t* __restrict__ mask, void* out, long long M, float eps) {
    // staged LayerNorm rows first, then two weight-step buffers over the same memory
    constexpr int NT = TILE * 2;
    constexpr int KS = C / 16;                    // k-steps of the first GEMM
    constexpr int NB = C / 32;                    // 32-channel output blocks of the second GEMM
    constexpr int XS = xs_bytes<C>();             // bytes per staged row
    constexpr int kStepBytes = 3 * 32 * C * 2;    // u block, v block, W_out slice
    constexpr int SMEM = TILE * XS > 2 * kStepBytes ? TILE * XS : 2 * kStepBytes;
    __shared__ __attribute__((aligned(16))) char smem[SMEM];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const long long p0 = (long long)blockIdx.x * TILE;
    constexpr int NSTEP = C * E / 32;             // 32 hidden channels per step
    const size_t ln_off = (size_t)NSTEP * kStepBytes;

    auto row_off = [&](int row) -> long long {
        const long long p = p0 + row;
        return p < M ? p * C : -1;
    };
    const u32x4* wsrc = reinterpret_cast<const u32x4*>(blob);
    constexpr int NPRE = (kStepBytes / 16 + NT - 1) / NT;
    u32x4 pre[NPRE];
    auto prefetch = [&](int s) {
#pragma unroll
        for (int i = 0; i < NPRE; ++i)
            if (i * NT + tid < kStepBytes / 16) pre[i] = wsrc[(size_t)s * (kStepBytes / 16) + i * NT + tid];
    };
    prefetch(0);        // the first weight step travels while the rows are loaded and normalised
    stage_ln_rows_c<IO, TILE, C, decltype(row_off), NT>(
        smem, x, reinterpret_cast<const float*>(blob + ln_off), eps, tid, row_off);
    __syncthreads();
    bf16x8 xf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) xf[ks] = lds_frag_c<C>(smem, wave * 32 + col, ks, half);
    __syncthreads();

    auto commit = [&](int s) {
#pragma unroll
        for (int i = 0; i < NPRE; ++i)
            if (i * NT + tid < kStepBytes / 16)
                reinterpret_cast<u32x4*>(smem + (s & 1) * kStepBytes)[i * NT + tid] = pre[i];
    };
    commit(0);
    __syncthreads();

    f32x16 oacc[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[n][v] = 0.f;

    for (int s = 0; s < NSTEP; ++s) {
        if (s + 1 < NSTEP) prefetch(s + 1);
        const char* wcur = smem + (s & 1) * kStepBytes;
        f32x16 u, g;
#pragma unroll
        for (int v = 0; v < 16; ++v) { u[v] = 0.f; g[v] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 w0 = *reinterpret_cast<const bf16x8*>(wcur + ks * 1024 + lane * 16);
            const bf16x8 w1 = *reinterpret_cast<const bf16x8*>(wcur + 64 * C + ks * 1024 + lane * 16);
            u = mfma32(w0, xf[ks], u);
            g = mfma32(w1, xf[ks], g);
        }
        // hidden = silu(u) * v ; lane = position, registers = 16 of the step's hidden channels.
        // The packed u rows carry a factor -log2(e) and W_out its inverse, so with
        // u' = -log2(e) u:  silu(u) v = (-ln 2) u' v / (1 + exp2(u')).
#pragma unroll
        for (int v = 0; v < 16; ++v) u[v] = u[v] * g[v] * fast_rcp(1.0f + fast_exp2(u[v]));
        bf16x8 hf0, hf1;
        acc_to_frags(u, hf0, hf1);
        // second GEMM: out[pos][c] += hidden[pos][32 of this step] * W_out[c][those 32]
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            oacc[n] = mfma32(hf0, *reinterpret_cast<const bf16x8*>(wcur + 128 * C + (n * 2) * 1024 + lane * 16), oacc[n]);
            oacc[n] = mfma32(hf1, *reinterpret_cast<const bf16x8*>(wcur + 128 * C + (n * 2 + 1) * 1024 + lane * 16), oacc[n]);
        }
        if (s + 1 < NSTEP) commit(s + 1);
        __syncthreads();
    }

    // block n of channel group G, lane col <-> channel 128*G + 4*col + n (ROW_INTERLEAVE4).  Rows in
    // two groups of 8: all residual values of a group are requested before its first store, so
    // one memory latency is paid per group and, with out aliasing residual, a row is read before
    // it is written.
#pragma unroll
    for (int G = 0; G < NB / 4; ++G) {
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            u32x2 rb[8];
            f32x4 rf[8];
            if (residual) {
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const long long p = min(p0 + wave * 32 + acc_row(8 * g + u, half), M - 1);
                    const size_t e0 = (size_t)p * C + 128 * G + 4 * col;
                    if constexpr (IO == KFH_BF16)
                        rb[u] = *reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(residual) + e0);
                    else
                        rf[u] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(residual) + e0);
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int v = 8 * g + u;
                const long long p = p0 + wave * 32 + acc_row(v, half);
                if (p < M) {
                    const size_t e0 = (size_t)p * C + 128 * G + 4 * col;
                    float o0 = oacc[4 * G][v], o1 = oacc[4 * G + 1][v], o2 = oacc[4 * G + 2][v], o3 = oacc[4 * G + 3][v];
                    const float mk = mask ? (mask[p] ? 1.f : 0.f) : 1.f;
                    if constexpr (IO == KFH_BF16) {
                        if (residual) {
                            o0 += bf16_lo(rb[u][0]); o1 += bf16_hi(rb[u][0]);
                            o2 += bf16_lo(rb[u][1]); o3 += bf16_hi(rb[u][1]);
                        }
                        u32x2 o = {pack_bf16(o0 * mk, o1 * mk), pack_bf16(o2 * mk, o3 * mk)};
                        *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + e0) = o;
                    } else {
                        if (residual) {
                            o0 += rf[u][0]; o1 += rf[u][1]; o2 += rf[u][2]; o3 += rf[u][3];
                        }
                        f32x4 o = {o0 * mk, o1 * mk, o2 * mk, o3 * mk};
                        *reinterpret_cast<f32x4*>(static_cast<float*>(out) + e0) = o;
                    }
                }
            }
        }
    }
}

int launch_pair_transition_wide(const void* x, int io_dtype, const char* blob, int expansion,
                                const void* residual, const uint8_t* mask, void* out, long long M,
                                float eps, hipStream_t stream, int C) {
    constexpr int TILE = 128;
    if (C != 256) return -1;
    dim3 grid((unsigned)((M + TILE - 1) / TILE)), block(TILE * 2);
#define KFH_LAUNCH_TRW(IO, E)                                                                                  \
    hipLaunchKernelGGL((transition_wide_kernel<IO, E, TILE, 256>), grid, block, 0, stream, x, blob, residual, mask, \
                       out, M, eps)
    if (expansion == 2) {
        if (io_dtype == KFH_F32) KFH_LAUNCH_TRW(KFH_F32, 2); else KFH_LAUNCH_TRW(KFH_BF16, 2);
    } else if (expansion == 4) {
        if (io_dtype == KFH_F32) KFH_LAUNCH_TRW(KFH_F32, 4); else KFH_LAUNCH_TRW(KFH_BF16, 4);
    } else {
        return -1;
    }
#undef KFH_LAUNCH_TRW
    return 0;
}

}  // namespace kfh
