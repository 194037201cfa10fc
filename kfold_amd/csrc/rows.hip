// Small row-wise kernels of the single (token) track: LayerNorm / cast of [rows, C] tensors,
// key-code construction and dense pair bias -> bias tiles.  These tensors are tiny next to
// the pair representation; the kernels are plain, coalesced and wavefront-reduced.
#include "kernels.hpp"

namespace kfh {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) v += __shfl_xor(v, off);
    return v;
}

// out[r', :] = bf16( normalize ? LN(x[r, :]) * gamma + beta : x[r, :] ), one wavefront per row.
// gamma / beta may be null (1 / 0).  C is even, at most 2048.  With tn > 0 the rows are the
// positions (i, j) of one or more [tn, tn] grids (a batch) and are written transposed inside their
// grid: r = g * tn^2 + i * tn + j -> r' = g * tn^2 + j * tn + i.
// (reference: model/primitives/normalization.py:61-91 — fp32 statistics, biased variance)
// PARTS = 3: the fp32 result is written as its three split3 planes, plane q at out + q * M * C.
template <int IO, int PARTS = 1>
__global__ __launch_bounds__(256) void rows_norm_kernel(const void* __restrict__ x,
                                                        const float* __restrict__ gamma,
                                                        const float* __restrict__ beta,
                                                        uint16_t* __restrict__ out, long long M, int C,
                                                        int normalize, float eps, int tn) {
    const int lane = threadIdx.x & 63;
    const long long r = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= M) return;
    long long ro = r;
    if (tn > 0) {
        const long long grid = (long long)tn * tn, q = r % grid;
        ro = r - q + (q % tn) * tn + q / tn;
    }
    const int npair = (C + 127) / 128;
    float a[16], b[16];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        if (i >= npair) break;
        const int c = 128 * i + 2 * lane;
        a[i] = 0.f; b[i] = 0.f;
        if (c < C) {
            const size_t e = (size_t)r * C + c;
            if constexpr (IO == KFH_BF16) {
                const uint32_t w = *reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(x) + e);
                a[i] = bf16_lo(w); b[i] = bf16_hi(w);
            } else {
                const f32x2 w = *reinterpret_cast<const f32x2*>(static_cast<const float*>(x) + e);
                a[i] = w[0]; b[i] = w[1];
            }
        }
        s += a[i] + b[i];
    }
    float mean = 0.f, rstd = 1.f;
    if (normalize) {
        mean = wave_sum(s) / C;
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if (i >= npair) break;
            if (128 * i + 2 * lane < C) { a[i] -= mean; b[i] -= mean; q += a[i] * a[i] + b[i] * b[i]; }
        }
        rstd = __builtin_amdgcn_rsqf(wave_sum(q) / C + eps);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        if (i >= npair) break;
        const int c = 128 * i + 2 * lane;
        if (c >= C) continue;
        float u = a[i] * rstd, v = b[i] * rstd;
        if (normalize) {
            if (gamma) { u *= gamma[c]; v *= gamma[c + 1]; }
            if (beta) { u += beta[c]; v += beta[c + 1]; }
        }
        if constexpr (PARTS == 1) {
            *reinterpret_cast<uint32_t*>(out + (size_t)ro * C + c) = pack_bf16(u, v);
        } else {
            float pu[3], pv[3];
            split3(u, pu);
            split3(v, pv);
#pragma unroll
            for (int q = 0; q < PARTS; ++q)
                *reinterpret_cast<uint32_t*>(out + (size_t)q * M * C + (size_t)ro * C + c) = pack_bf16(pu[q], pv[q]);
        }
    }
}

int launch_rows_norm(const void* x, int io_dtype, const float* gamma, const float* beta, uint16_t* out,
                     long long M, int C, int normalize, float eps, hipStream_t stream, int transpose_n,
                     int parts) {
    if (C % 2 || C > 2048 || C <= 0) return -1;
    if (transpose_n > 0 && M % ((long long)transpose_n * transpose_n) != 0) return -1;
    if (parts != 1 && parts != 3) return -1;
    dim3 grid((unsigned)((M + 3) / 4)), block(256);
    if (parts == 3) {
        if (io_dtype == KFH_F32)
            hipLaunchKernelGGL((rows_norm_kernel<KFH_F32, 3>), grid, block, 0, stream, x, gamma, beta, out, M, C,
                               normalize, eps, transpose_n);
        else
            hipLaunchKernelGGL((rows_norm_kernel<KFH_BF16, 3>), grid, block, 0, stream, x, gamma, beta, out, M, C,
                               normalize, eps, transpose_n);
        return 0;
    }
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL(rows_norm_kernel<KFH_F32>, grid, block, 0, stream, x, gamma, beta, out, M, C,
                           normalize, eps, transpose_n);
    else
        hipLaunchKernelGGL(rows_norm_kernel<KFH_BF16>, grid, block, 0, stream, x, gamma, beta, out, M, C,
                           normalize, eps, transpose_n);
    return 0;
}

// codes[a][k] = k < L ? (mask[b * batch_stride + i * row_stride + k * key_stride] ? 2 : 1) : 0  for k < Lp = nb * 32,
// where row a = b * rows_per_batch + i (rows_per_batch = 0: one batch, i = a)
__global__ void key_codes_kernel(const uint8_t* __restrict__ mask, uint8_t* __restrict__ codes,
                                 int rows, int L, int Lp, long long row_stride, long long key_stride,
                                 int rows_per_batch, long long batch_stride) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long long)rows * Lp) return;
    const int a = (int)(i / Lp), k = (int)(i % Lp);
    const int b = rows_per_batch > 0 ? a / rows_per_batch : 0, ai = rows_per_batch > 0 ? a % rows_per_batch : a;
    codes[i] = k < L ? (mask[b * batch_stride + ai * row_stride + k * key_stride] ? 2 : 1) : 0;
}

void launch_key_codes(const uint8_t* mask, uint8_t* codes, int rows, int L, int Lp,
                      long long mask_stride, hipStream_t stream, long long key_stride, int rows_per_batch,
                      long long batch_stride) {
    const long long n = (long long)rows * Lp;
    hipLaunchKernelGGL(key_codes_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, mask,
                       codes, rows, L, Lp, mask_stride, key_stride, rows_per_batch, batch_stride);
}

// Dense pair bias [nbatch][H][L][L] -> log2(e)-scaled bf16 tiles (bias_tile_elem layout);
// one thread writes the 8 keys of one (tile, chunk, lane) slot.
// element (t, q, k) of the source is at t * st + q * sq + k * sk (t = batch * H + head), or with
// hdiv > 0 at (t / hdiv) * sb + (t % hdiv) * st + q * sq + k * sk (a batch stride of its own);
// Lq x Lk logits in nbq x nbk tiles
template <int IO>
__global__ void bias_tiles_kernel(const void* __restrict__ dense, uint16_t* __restrict__ tiles,
                                  long long total, int Lq, int Lk, int nbq, int nbk, long long st,
                                  long long sq, long long sk, int hdiv, long long sb) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;      // 16-byte slot
    if (i >= total) return;
    const int lane = (int)(i & 63), c = (int)((i >> 6) & 1);
    long long t = i >> 7;
    const int kb = (int)(t % nbk); t /= nbk;
    const int qb = (int)(t % nbq); t /= nbq;        // t = batch * H + h
    const int q = qb * 32 + (lane & 31);
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
        float v[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int k = kb * 32 + acc_row(8 * c + e + u, lane >> 5);
            float x = 0.f;
            if (q < Lq && k < Lk) {
                const long long tb = hdiv > 0 ? (t / hdiv) * sb + (t % hdiv) * st : t * st;
                const size_t off = (size_t)(tb + q * sq + k * sk);
                if constexpr (IO == KFH_F32) x = static_cast<const float*>(dense)[off];
                else x = bf16_lo(static_cast<const uint16_t*>(dense)[off]);
            }
            v[u] = x * kLog2e;
        }
        w[e >> 1] = pack_bf16(v[0], v[1]);
    }
    reinterpret_cast<u32x4*>(tiles)[i] = u32x4{w[0], w[1], w[2], w[3]};
}

void launch_bias_tiles(const void* dense, int io_dtype, uint16_t* tiles, int nbatch, int H, int L, int nb,
                       hipStream_t stream, long long st, long long sq, long long sk, int Lk, long long sb) {
    const int Lq = L, nbq = nb;
    if (Lk <= 0) Lk = L;
    const int nbk = (Lk + 31) / 32;
    if (st == 0 && sq == 0 && sk == 0) { st = (long long)Lq * Lk; sq = Lk; sk = 1; }    // dense [.., H, Lq, Lk]
    const long long total = (long long)nbatch * H * nbq * nbk * 128;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL(bias_tiles_kernel<KFH_F32>, grid, block, 0, stream, dense, tiles, total, Lq, Lk, nbq,
                           nbk, st, sq, sk, sb != 0 ? H : 0, sb);
    else
        hipLaunchKernelGGL(bias_tiles_kernel<KFH_BF16>, grid, block, 0, stream, dense, tiles, total, Lq, Lk, nbq,
                           nbk, st, sq, sk, sb != 0 ? H : 0, sb);
}

// Dense pair bias -> log2(e)-scaled fp32 tiles (bias_tile_f32_elem layout): one thread writes the
// 4 keys of one (tile, chunk, lane) slot.  Source [nbatch][H][Lq][Lk] contiguous.
template <int IO>
__global__ void bias_tiles_f32_kernel(const void* __restrict__ dense, float* __restrict__ tiles,
                                      long long total, int Lq, int Lk, int nbq, int nbk) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;      // 16-byte slot
    if (i >= total) return;
    const int lane = (int)(i & 63), c = (int)((i >> 6) & 3);
    long long t = i >> 8;
    const int kb = (int)(t % nbk); t /= nbk;
    const int qb = (int)(t % nbq); t /= nbq;        // t = batch * H + h
    const int q = qb * 32 + (lane & 31);
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int k = kb * 32 + acc_row(4 * c + e, lane >> 5);
        float x = 0.f;
        if (q < Lq && k < Lk) {
            const size_t off = ((size_t)t * Lq + q) * Lk + k;
            if constexpr (IO == KFH_F32) x = static_cast<const float*>(dense)[off];
            else x = bf16_lo(static_cast<const uint16_t*>(dense)[off]);
        }
        o[e] = x * kLog2e;
    }
    reinterpret_cast<f32x4*>(tiles)[i] = o;
}

void launch_bias_tiles_f32(const void* dense, int io_dtype, float* tiles, int nbatch, int H, int L, int nb,
                           hipStream_t stream, int Lk) {
    if (Lk <= 0) Lk = L;
    const int nbk = (Lk + 31) / 32;
    const long long total = (long long)nbatch * H * nb * nbk * 256;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (io_dtype == KFH_F32)
        hipLaunchKernelGGL(bias_tiles_f32_kernel<KFH_F32>, grid, block, 0, stream, dense, tiles, total, L, Lk, nb, nbk);
    else
        hipLaunchKernelGGL(bias_tiles_f32_kernel<KFH_BF16>, grid, block, 0, stream, dense, tiles, total, L, Lk, nb, nbk);
}

}  // namespace kfh
