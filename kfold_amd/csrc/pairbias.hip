// Pair bias of the single-track attention:  bias[h, q, k] = (W LN(z[q, k]))[h]
// (reference: model/modules/confidence_head.py:162-163, `linear_pair_bias(layernorm_z(z))`
// moved to [B, H, L, L]).  One pass over z, HBM-bound on the z read; the result is written
// directly as the log2(e)-scaled bf16 bias tiles the attention kernels consume (flash.hip).
#include "kernels.hpp"

namespace kfh {

// 256 keys of one query per workgroup, 32 per wavefront (8 wavefronts, 4 per SIMD)
template <int IO>
__global__ __launch_bounds__(512, 4) void pair_bias_kernel(const void* __restrict__ z,
                                                           const char* __restrict__ blob,
                                                           uint16_t* __restrict__ tiles, int N, int nb,
                                                           int H, float eps) {
    __shared__ __attribute__((aligned(16))) char smem[256 * kXS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int a = blockIdx.y, t0 = blockIdx.x * 256;      // query a, keys t0 .. t0+255
    auto row_off = [&](int row) -> long long {
        const int b = t0 + row;
        return b < N ? (long long)(((size_t)a * N + b) * kC) : -1;
    };
    stage_ln_rows<IO, 256, decltype(row_off), 512>(smem, z, reinterpret_cast<const float*>(blob + kBlockBytes),
                                                    eps, tid, row_off);
    __syncthreads();
    const int kblk = (t0 >> 5) + wave;
    if (kblk >= nb) return;
    const bf16x8* w = reinterpret_cast<const bf16x8*>(blob) + lane;
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) acc = mfma32(w[ks * 64], lds_frag(smem, wave * 32 + col, ks, half), acc);
    // accumulator rows are heads; lane col is the key inside its block
    const int e = bias_tile_elem(a & 31, col);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int h = acc_row(v, half);
        if (h < H) {
            const size_t tile = ((size_t)h * nb + (a >> 5)) * nb + kblk;
            tiles[tile * kBiasTileElems + e] = (uint16_t)(pack_bf16(acc[v], 0.f) & 0xffffu);
        }
    }
}

void launch_pair_bias(const void* z, int io_dtype, const char* blob, uint16_t* tiles, int N, int H,
                      float eps, hipStream_t stream) {
    const int nb = (N + 31) / 32;
    dim3 grid((N + 255) / 256, N), block(512);
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL(pair_bias_kernel<KFH_F32>, grid, block, 0, stream, z, blob, tiles, N, nb, H, eps);
    else
        hipLaunchKernelGGL(pair_bias_kernel<KFH_BF16>, grid, block, 0, stream, z, blob, tiles, N, nb, H, eps);
}

}  // namespace kfh
