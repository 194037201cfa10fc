// Weight packing: row-major [out, in] projection weights -> MFMA fragment order.
//
// A packed "block" is 32 output rows x K input channels, stored as K/16 fragments of
// 1 KiB (64 lanes x 8 bf16).  Lane (col = lane & 31, half = lane >> 5) of fragment ks holds
// the weights of output row `rowmap(block, col)` at the 8 input channels
// `kmap(ks, half, e)`, e = 0..7.  The maps are chosen per consumer so that its global
// stores come out contiguous (row maps) or so that the k-slots agree with the layout of
// the activation fragments it multiplies with (k maps).
#include "kernels.hpp"

namespace kfh {

__device__ __forceinline__ int pack_row(int mode, int b, int col) {
    switch (mode) {
        case ROW_NATURAL: return 32 * b + col;
        case ROW_INTERLEAVE2: return 64 * (b >> 1) + 2 * col + (b & 1);
        case ROW_INTERLEAVE4: return 128 * (b >> 2) + 4 * col + (b & 3);
        default: return 32 * b + col;
    }
}

// source column of k-slot (ks, half, e), or -1 for a zero (padding) slot
__device__ __forceinline__ int pack_k(int mode, int K, int ks, int half, int e, int kparam) {
    switch (mode) {
        case K_NATURAL: return 16 * ks + 8 * half + e;
        case K_ACC: return 16 * ks + 8 * (e >> 2) + 4 * half + (e & 3);
        case K_HALF: return (K >> 1) * half + 8 * ks + e;
        case K_ACC_HEADPAD: {
            // k-steps are grouped per head: kparam = (real head dim) | (k-steps per padded head) << 16
            const int dh = kparam & 0xffff, dks = kparam >> 16;
            const int h = ks / dks, d = 16 * (ks % dks) + 8 * (e >> 2) + 4 * half + (e & 3);
            return d < dh ? h * dh + d : -1;
        }
        default: return 16 * ks + 8 * half + e;
    }
}

template <int WT>
__global__ void pack_blocks_kernel(const void* __restrict__ src, int src_rows, int K, int ld,
                                   int row0, int nblk, int row_mode, int k_mode, int kparam,
                                   float scale, uint16_t* __restrict__ dst, int part) {
    const int ksteps = K / 16;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;      // (block, ks, lane)
    if (idx >= nblk * ksteps * 64) return;
    const int lane = idx & 63;
    const int ks = (idx >> 6) % ksteps;
    const int b = (idx >> 6) / ksteps;
    const int col = lane & 31, half = lane >> 5;
    const int r = pack_row(row_mode, b, col);
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
        float v[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int k = pack_k(k_mode, K, ks, half, e + u, kparam);
            float x = 0.f;
            if (r < src_rows && k >= 0) {
                const size_t off = (size_t)(row0 + r) * ld + k;
                if constexpr (WT == KFH_F32) x = static_cast<const float*>(src)[off];
                else x = bf16_lo(static_cast<const uint16_t*>(src)[off]);
            }
            v[u] = x * scale;
            if (part >= 0) {
                float sp[3];
                split3(v[u], sp);
                v[u] = sp[part];
            }
        }
        w[e >> 1] = pack_bf16(v[0], v[1]);
    }
    u32x4 o = {w[0], w[1], w[2], w[3]};
    reinterpret_cast<u32x4*>(dst)[idx] = o;
}

template <int WT>
__global__ void copy_f32_kernel(const void* __restrict__ src, float* __restrict__ dst, int n,
                                float fill) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float x = fill;
    if (src) {
        if constexpr (WT == KFH_F32) x = static_cast<const float*>(src)[i];
        else x = bf16_lo(static_cast<const uint16_t*>(src)[i]);
    }
    dst[i] = x;
}

__global__ void fill_zero_kernel(u32x4* __restrict__ dst, size_t n16) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) dst[i] = u32x4{0u, 0u, 0u, 0u};
}

// zero `bytes` (a multiple of 16) at a 16-byte aligned address with a plain kernel, so that
// callers may record the call sequence into a HIP graph
void launch_fill_zero(void* dst, size_t bytes, hipStream_t stream) {
    const size_t n16 = bytes / 16;
    if (n16 == 0) return;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, stream,
                       static_cast<u32x4*>(dst), n16);
}

void launch_pack_blocks(const void* src, int wdtype, int src_rows, int K, int ld, int row0,
                        int nblk, int row_mode, int k_mode, float scale, void* dst,
                        hipStream_t stream, int kparam, int part) {
    const int total = nblk * (K / 16) * 64;
    const int threads = 256, blocks = (total + threads - 1) / threads;
    if (wdtype == KFH_F32)
        hipLaunchKernelGGL(pack_blocks_kernel<KFH_F32>, dim3(blocks), dim3(threads), 0, stream, src,
                           src_rows, K, ld, row0, nblk, row_mode, k_mode, kparam, scale,
                           static_cast<uint16_t*>(dst), part);
    else
        hipLaunchKernelGGL(pack_blocks_kernel<KFH_BF16>, dim3(blocks), dim3(threads), 0, stream, src,
                           src_rows, K, ld, row0, nblk, row_mode, k_mode, kparam, scale,
                           static_cast<uint16_t*>(dst), part);
}

void launch_copy_f32(const void* src, int wdtype, float* dst, int n, float fill,
                     hipStream_t stream) {
    const int threads = 256, blocks = (n + threads - 1) / threads;
    if (wdtype == KFH_F32)
        hipLaunchKernelGGL(copy_f32_kernel<KFH_F32>, dim3(blocks), dim3(threads), 0, stream, src, dst,
                           n, fill);
    else
        hipLaunchKernelGGL(copy_f32_kernel<KFH_BF16>, dim3(blocks), dim3(threads), 0, stream, src, dst,
                           n, fill);
}

}  // namespace kfh
