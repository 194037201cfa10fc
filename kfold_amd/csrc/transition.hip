// Pair transition (C = 128, expansion E = 2 or 4), fully fused:
//     out = [residual +] W_out ( silu(u) * v ),   [u, v] = W_sw LN(x)        (then * mask)
// Reference: src/kfold/model/layers/folding/transition.py:48-68 with
// primitives/activation.py:27-29; the optional mask multiply is the final `z * pair_mask` of
// modules/apo_module.py:172.
//
// Workgroup = 256 positions, 64 per wavefront.  The hidden activations never leave
// registers: each step computes 32 hidden channels of u and of v (channels as accumulator
// rows), and silu(u)*v rounded to bf16 is directly the A operand of the second GEMM, whose
// [64 positions x 128 channels] accumulators stay resident across the steps.  Weights of a
// step (u block, v block, the matching 32-column slice of W_out: 24 KiB) are
// double-buffered in LDS.
#include "kernels.hpp"

namespace kfh {

constexpr int kTileT = 256;
constexpr int kStepBytes = 3 * (int)kBlockBytes;   // 24 KiB

template <int IO, int E>
__global__ __launch_bounds__(256) void transition_kernel(
    const void* __restrict__ x, const char* __restrict__ blob, const void* residual,
    const uint8_t* __restrict__ mask, void* out, long long M, float eps) {
    // staged LayerNorm rows (69632 B) first, then two 24 KiB weight buffers
    __shared__ __attribute__((aligned(16))) char smem[kTileT * kXS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const long long p0 = (long long)blockIdx.x * kTileT;
    constexpr int NSTEP = 4 * E;                  // 32 hidden channels per step
    const size_t ln_off = (size_t)NSTEP * kStepBytes;

    stage_ln_rows<IO, kTileT>(smem, x, reinterpret_cast<const float*>(blob + ln_off), eps, tid,
                              [&](int row) -> long long {
                                  const long long p = p0 + row;
                                  return p < M ? p * kC : -1;
                              });
    __syncthreads();
    bf16x8 xf[2][kKS];
#pragma unroll
    for (int pb = 0; pb < 2; ++pb)
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) xf[pb][ks] = lds_frag(smem, wave * 64 + 32 * pb + col, ks, half);
    __syncthreads();

    const u32x4* wsrc = reinterpret_cast<const u32x4*>(blob);
    u32x4 pre[6];
    auto prefetch = [&](int s) {
#pragma unroll
        for (int i = 0; i < 6; ++i) pre[i] = wsrc[(size_t)s * (kStepBytes / 16) + i * 256 + tid];
    };
    auto commit = [&](int s) {
#pragma unroll
        for (int i = 0; i < 6; ++i)
            reinterpret_cast<u32x4*>(smem + (s & 1) * kStepBytes)[i * 256 + tid] = pre[i];
    };
    prefetch(0);
    commit(0);
    __syncthreads();

    f32x16 oacc[2][4];
#pragma unroll
    for (int pb = 0; pb < 2; ++pb)
#pragma unroll
        for (int n = 0; n < 4; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[pb][n][v] = 0.f;

    for (int s = 0; s < NSTEP; ++s) {
        if (s + 1 < NSTEP) prefetch(s + 1);
        const char* wcur = smem + (s & 1) * kStepBytes;
        f32x16 u[2], g[2];
#pragma unroll
        for (int pb = 0; pb < 2; ++pb)
#pragma unroll
            for (int v = 0; v < 16; ++v) { u[pb][v] = 0.f; g[pb][v] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) {
            const bf16x8 w0 = *reinterpret_cast<const bf16x8*>(wcur + ks * 1024 + lane * 16);
            const bf16x8 w1 = *reinterpret_cast<const bf16x8*>(wcur + 8192 + ks * 1024 + lane * 16);
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) {
                u[pb] = mfma32(w0, xf[pb][ks], u[pb]);
                g[pb] = mfma32(w1, xf[pb][ks], g[pb]);
            }
        }
        // hidden = silu(u) * v ; lane = position, registers = 16 of the step's hidden channels
        bf16x8 hf[2][2];
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) u[pb][v] = u[pb][v] * sigmoidf_fast(u[pb][v]) * g[pb][v];
            acc_to_frags(u[pb], hf[pb][0], hf[pb][1]);
        }
        // second GEMM: out[pos][c] += hidden[pos][32 of this step] * W_out[c][those 32]
#pragma unroll
        for (int n = 0; n < 4; ++n)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const bf16x8 w = *reinterpret_cast<const bf16x8*>(wcur + 16384 + (n * 2 + ks) * 1024 + lane * 16);
                oacc[0][n] = mfma32(hf[0][ks], w, oacc[0][n]);
                oacc[1][n] = mfma32(hf[1][ks], w, oacc[1][n]);
            }
        if (s + 1 < NSTEP) commit(s + 1);
        __syncthreads();
    }

    // block n, lane col <-> channel 4*col + n (ROW_INTERLEAVE4)
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const long long p = p0 + wave * 64 + 32 * pb + acc_row(v, half);
            if (p < M) {
                const size_t e0 = (size_t)p * kC + 4 * col;
                float o0 = oacc[pb][0][v], o1 = oacc[pb][1][v], o2 = oacc[pb][2][v], o3 = oacc[pb][3][v];
                const float mk = mask ? (mask[p] ? 1.f : 0.f) : 1.f;
                if constexpr (IO == KFH_BF16) {
                    if (residual) {
                        const u32x2 r = *reinterpret_cast<const u32x2*>(
                            static_cast<const uint16_t*>(residual) + e0);
                        o0 += bf16_lo(r[0]); o1 += bf16_hi(r[0]); o2 += bf16_lo(r[1]); o3 += bf16_hi(r[1]);
                    }
                    u32x2 o = {pack_bf16(o0 * mk, o1 * mk), pack_bf16(o2 * mk, o3 * mk)};
                    *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + e0) = o;
                } else {
                    if (residual) {
                        const f32x4 r = *reinterpret_cast<const f32x4*>(static_cast<const float*>(residual) + e0);
                        o0 += r[0]; o1 += r[1]; o2 += r[2]; o3 += r[3];
                    }
                    f32x4 o = {o0 * mk, o1 * mk, o2 * mk, o3 * mk};
                    *reinterpret_cast<f32x4*>(static_cast<float*>(out) + e0) = o;
                }
            }
        }
    }
}

int launch_pair_transition(const void* x, int io_dtype, const char* blob, int expansion,
                           const void* residual, const uint8_t* mask, void* out, long long M,
                           float eps, hipStream_t stream) {
    dim3 grid((unsigned)((M + kTileT - 1) / kTileT)), block(256);
#define KFH_LAUNCH_TR(IO, E)                                                                   \
    hipLaunchKernelGGL((transition_kernel<IO, E>), grid, block, 0, stream, x, blob, residual, mask, \
                       out, M, eps)
    if (expansion == 2) {
        if (io_dtype == KFH_F32) KFH_LAUNCH_TR(KFH_F32, 2); else KFH_LAUNCH_TR(KFH_BF16, 2);
    } else if (expansion == 4) {
        if (io_dtype == KFH_F32) KFH_LAUNCH_TR(KFH_F32, 4); else KFH_LAUNCH_TR(KFH_BF16, 4);
    } else {
        return -1;
    }
#undef KFH_LAUNCH_TR
    return 0;
}

}  // namespace kfh
