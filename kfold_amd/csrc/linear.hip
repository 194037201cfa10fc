// Generic bf16 MFMA linear layers for the single (token) track and the pair-bias attention
// projections:  Y = X W^T (+ bias) followed by a small epilogue.  X is either row-major bf16
// or already in MFMA fragment order; W is a packed weight (pack.hip).  One workgroup computes
// one 32 x 32 output tile, its 4 wavefronts splitting K, with operands read straight from
// global memory / L2: these problems are a few hundred rows, so no LDS staging is used.
//
// Epilogues (reference lines in src/kfold/model):
//   EPI_STORE    y = acc + bias
//   EPI_SIGMOID  y = sigmoid(acc + bias)
//   EPI_SWIGLU   y = silu(acc) * acc2                                    primitives/activation.py:27-29
//   EPI_ADALN    y = sigmoid(acc + bias) * aux + acc2                    primitives/normalization.py:117-125
//   EPI_RESID    y = (aux + gate * (acc + bias)) * row mask   (aux, gate, mask optional)
//                layers/folding/attention_pair_bias.py:155-157, modules/apo_module.py:172
//   EPI_FRAG_CH  fragments with channels as accumulator rows (q, k, gate of attention)
//   EPI_FRAG_POS fragments with positions as accumulator rows (v of attention)
//   EPI_PLANES   (acc * sigmoid(acc2)) * mask as bf16 channel-major planes   primitives/triangle_multiplication.py:216-221
#include <cstdlib>

#include "kernels.hpp"

namespace kfh {

// Epilogue of one 32 x 32 accumulator block: `a` = row group, `blk` = position block inside it,
// `wb` = 32-channel block of the packed weight.  Shared by the two kernels below.
template <int EPI, int PARTS>
__device__ __forceinline__ void linear_epilogue(const LinearArgs& p, f32x16& acc, f32x16& acc2, int a, int blk,
                                                int wb, int lane) {
    const int col = lane & 31, half = lane >> 5;
    if constexpr (EPI == EPI_PLANES) {
        // lane col <-> position, registers <-> 16 of the block's 32 channels: for one register the
        // 32 lanes of a half write 32 consecutive positions of one plane
        const int ps = blk * 32 + col;
        if (ps >= p.L) return;
        const int br = p.batch_rows > 0 ? p.batch_rows : p.rows_a;      // row groups per batch element
        const int bq = a / br, ai = a % br;
        const size_t mi = p.mask_transposed ? ((size_t)bq * br * p.L + (size_t)ps * br + ai) : (size_t)a * p.L + ps;
        const bool valid = p.mask[mi] != 0;
        const size_t plane_sz = (size_t)p.ldo * p.ldo;
        uint16_t* dst = static_cast<uint16_t*>(p.out) + (size_t)ai * p.ldo + ps;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int c = 32 * wb + acc_row(v, half);
            if (c >= p.Nout) continue;
            const size_t plane = p.nbatch > 1 ? (size_t)(c / p.plane_side) * p.nbatch * p.plane_side +
                                                    (size_t)bq * p.plane_side + c % p.plane_side
                                              : (size_t)c;
            const float y = valid ? acc[v] * sigmoidf_fast(acc2[v]) : 0.f;
            dst[plane * plane_sz] = (uint16_t)(pack_bf16(y, 0.f) & 0xffffu);
        }
    } else if constexpr (EPI == EPI_FRAG_CH || EPI == EPI_FRAG_POS) {
        const int h = wb / p.PB, pp = wb % p.PB;
        if constexpr (EPI == EPI_FRAG_CH) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int d = 32 * pp + acc_row(v, half);
                float y = acc[v];
                if (p.bias && d < p.Dh) y += p.bias[h * p.Dh + d] * p.bias_scale;
                if (p.sigmoid) y = PARTS == 3 ? 1.0f / (1.0f + exp2f(-kLog2e * y)) : sigmoidf_fast(y);
                acc[v] = y;
            }
        }
        const size_t u0 = (((((size_t)a * p.H + h) * p.nb + blk) * p.PB + pp) * 2 * 64 + lane) * 16;
        if constexpr (PARTS == 1) {
            bf16x8 f0, f1;
            acc_to_frags(acc, f0, f1);
            bf16x8* dst = reinterpret_cast<bf16x8*>(static_cast<char*>(p.out) + u0);
            dst[0] = f0;
            dst[64] = f1;
        } else {
            f32x16 part[PARTS];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float sp[3];
                split3(acc[v], sp);
#pragma unroll
                for (int q = 0; q < PARTS; ++q) part[q][v] = sp[q];
            }
#pragma unroll
            for (int q = 0; q < PARTS; ++q) {
                bf16x8 f0, f1;
                acc_to_frags(part[q], f0, f1);
                bf16x8* dst = reinterpret_cast<bf16x8*>(static_cast<char*>(p.out) + (size_t)q * p.out_part + u0);
                dst[0] = f0;
                dst[64] = f1;
            }
        }
    } else {
        const int c = 32 * wb + col;
        if (c >= p.Nout) return;
        const float bc = p.bias ? p.bias[c] : 0.f;
        auto sig = [&](float x) { return PARTS == 3 ? 1.0f / (1.0f + exp2f(-kLog2e * x)) : sigmoidf_fast(x); };
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int ps = blk * 32 + acc_row(v, half);
            if (ps >= p.L) continue;
            size_t r = (size_t)a * p.L + ps;
            size_t r_aux = (size_t)(p.aux_shared ? 0 : a) * p.L + ps;
            if constexpr (EPI == EPI_RESID) {
                if (p.out_transposed) {
                    const int br = p.batch_rows > 0 ? p.batch_rows : p.rows_a;
                    r = (size_t)(a / br) * br * p.L + (size_t)ps * br + a % br;
                    r_aux = r;
                }
            }
            const size_t r_gate = (size_t)(p.gate_shared ? 0 : a) * p.L + ps;
            float y = acc[v] + bc;
            if constexpr (EPI == EPI_SIGMOID) y = sig(y);
            if constexpr (EPI == EPI_SWIGLU) y = acc[v] * sig(acc[v]) * acc2[v];
            if constexpr (EPI == EPI_ADALN) {
                const char* ap = static_cast<const char*>(p.aux) + (r_aux * p.ld_aux + c) * 2;
                float ax = bf16_lo(*reinterpret_cast<const uint16_t*>(ap));
                if constexpr (PARTS == 3)
                    ax = (bf16_lo(*reinterpret_cast<const uint16_t*>(ap + 2 * p.aux_part)) +
                          bf16_lo(*reinterpret_cast<const uint16_t*>(ap + p.aux_part))) + ax;
                y = sig(y) * ax + acc2[v];
            }
            if constexpr (EPI == EPI_RESID) {
                if (p.gate) {
                    y *= p.gate_dtype == KFH_F32 ? reinterpret_cast<const float*>(p.gate)[r_gate * p.ld_gate + c]
                                                 : bf16_lo(p.gate[r_gate * p.ld_gate + c]);
                }
                if (p.aux) {
                    y += p.aux_dtype == KFH_F32 ? static_cast<const float*>(p.aux)[r_aux * p.ld_aux + c]
                                                : bf16_lo(static_cast<const uint16_t*>(p.aux)[r_aux * p.ld_aux + c]);
                }
                if (p.mask && p.mask[r] == 0) y = 0.f;       // row mask of the output (the block's final z * mask)
            }
            if (p.out_dtype == KFH_F32) {
                static_cast<float*>(p.out)[r * p.ldo + c] = y;
            } else if constexpr (PARTS == 1) {
                static_cast<uint16_t*>(p.out)[r * p.ldo + c] = (uint16_t)(pack_bf16(y, 0.f) & 0xffffu);
            } else {
                float sp[3];
                split3(y, sp);
#pragma unroll
                for (int q = 0; q < PARTS; ++q)
                    *reinterpret_cast<uint16_t*>(static_cast<char*>(p.out) + (size_t)q * p.out_part + (r * p.ldo + c) * 2) =
                        (uint16_t)(pack_bf16(sp[q], 0.f) & 0xffffu);
            }
        }
    }
}

// PARTS = 3 is the fp32 arithmetic: A, W (and W2) arrive as their three split3 planes and every
// k-step runs the six part products (i, j), i + j <= 2; bf16 outputs leave as three planes too.
template <int EPI, bool AFRAG, int PARTS>
__global__ __launch_bounds__(256) void linear_kernel(LinearArgs p) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    // The 4 wavefronts of a workgroup share one 32 x 32 output tile and split K between them in
    // chunks of CH k-steps (wavefront w takes chunks w, w+4, ...): these problems have few tiles
    // and long K, so the serial chain of dependent operand loads is what costs.
    __shared__ float red[3][2][64 * 16];
    const int wb = blockIdx.y;
    const int a = blockIdx.x / p.nb, blk = blockIdx.x % p.nb;
    const int ksteps = p.K / 16;
    const char* Wb = static_cast<const char*>(p.W) + ((size_t)wb * ksteps * 64 + lane) * 16;
    const char* W2b = p.W2 ? static_cast<const char*>(p.W2) + ((size_t)wb * ksteps * 64 + lane) * 16 : nullptr;
    auto wfrag = [&](const char* base, int ks, int q) -> bf16x8 {
        return *reinterpret_cast<const bf16x8*>(base + (size_t)q * p.w_part + (size_t)ks * 1024);
    };

    const int pos = min(blk * 32 + col, p.L - 1);
    const char* arow = AFRAG ? nullptr
                             : static_cast<const char*>(p.A) +
                                   (((size_t)(p.a_shared ? 0 : a) * p.L + pos) * p.lda + 8 * half) * 2;
    const int dks = 2 * p.PB;
    auto afrag = [&](int ks, int q) -> bf16x8 {
        if constexpr (AFRAG) {
            const int h = ks / dks, kk = ks % dks;
            const size_t u = ((((size_t)a * p.H + h) * p.nb + blk) * dks + kk) * 64 + lane;
            return *reinterpret_cast<const bf16x8*>(static_cast<const char*>(p.A) + (size_t)q * p.a_part + u * 16);
        } else {
            return *reinterpret_cast<const bf16x8*>(arow + (size_t)q * p.a_part + 32 * ks);
        }
    };

    f32x16 acc, acc2;
#pragma unroll
    for (int v = 0; v < 16; ++v) { acc[v] = 0.f; acc2[v] = 0.f; }
    constexpr bool W_IS_A = (EPI == EPI_FRAG_CH || EPI == EPI_PLANES);     // channels as accumulator rows
    constexpr bool TWO = (EPI == EPI_SWIGLU || EPI == EPI_ADALN || EPI == EPI_PLANES);
    // part pairs (A part, W part) of one k-step, smallest terms first
    constexpr int NPROD = PARTS == 3 ? 6 : 1;
    constexpr int PA[6] = {PARTS == 3 ? 2 : 0, PARTS == 3 ? 1 : 0, 0, PARTS == 3 ? 1 : 0, 0, 0};
    constexpr int PW[6] = {0, PARTS == 3 ? 1 : 0, PARTS == 3 ? 2 : 0, 0, PARTS == 3 ? 1 : 0, 0};
    // K is walked in chunks of CH k-steps; the operands of chunk c+1 are requested before the
    // MFMAs of chunk c, so one memory latency is paid per chunk at most
    constexpr int CH = PARTS == 3 ? 2 : 8;
    bf16x8 xa[CH][PARTS], wa[CH][PARTS], va[CH][PARTS], xb[CH][PARTS], wb2[CH][PARTS], vb[CH][PARTS];
    auto load = [&](int c, bf16x8 (&x)[CH][PARTS], bf16x8 (&w)[CH][PARTS], bf16x8 (&v)[CH][PARTS]) {
#pragma unroll
        for (int i = 0; i < CH; ++i)
#pragma unroll
            for (int q = 0; q < PARTS; ++q) {
                x[i][q] = afrag(c * CH + i, q);
                w[i][q] = wfrag(Wb, c * CH + i, q);
                if constexpr (TWO) v[i][q] = wfrag(W2b, c * CH + i, q);
            }
    };
    auto compute = [&](const bf16x8 (&x)[CH][PARTS], const bf16x8 (&w)[CH][PARTS], const bf16x8 (&v)[CH][PARTS]) {
#pragma unroll
        for (int i = 0; i < CH; ++i)
#pragma unroll
            for (int pr = 0; pr < NPROD; ++pr) {
                const bf16x8 xq = x[i][PA[pr]], wq = w[i][PW[pr]];
                acc = W_IS_A ? mfma32(wq, xq, acc) : mfma32(xq, wq, acc);
                if constexpr (TWO) acc2 = W_IS_A ? mfma32(v[i][PW[pr]], xq, acc2) : mfma32(xq, v[i][PW[pr]], acc2);
            }
    };
    const int nch = ksteps / CH;
    const int mine = nch > wave ? (nch - wave + 3) / 4 : 0;          // chunks of this wavefront
    auto chunk = [&](int i) { return wave + 4 * i; };
    if (mine > 0) load(chunk(0), xa, wa, va);
    for (int i = 0; i < mine; i += 2) {
        if (i + 1 < mine) load(chunk(i + 1), xb, wb2, vb);
        compute(xa, wa, va);
        if (i + 1 < mine) {
            if (i + 2 < mine) load(chunk(i + 2), xa, wa, va);
            compute(xb, wb2, vb);
        }
    }
    if (wave == 0) {
        for (int ks = nch * CH; ks < ksteps; ++ks) {      // K not a multiple of 16 * CH
#pragma unroll
            for (int pr = 0; pr < NPROD; ++pr) {
                const bf16x8 x = afrag(ks, PA[pr]);
                const bf16x8 w = wfrag(Wb, ks, PW[pr]);
                acc = W_IS_A ? mfma32(w, x, acc) : mfma32(x, w, acc);
                if constexpr (TWO) {
                    const bf16x8 w2 = wfrag(W2b, ks, PW[pr]);
                    acc2 = W_IS_A ? mfma32(w2, x, acc2) : mfma32(x, w2, acc2);
                }
            }
        }
    }
    // partial sums of wavefronts 1..3 -> LDS -> wavefront 0, which runs the epilogue
    if (wave > 0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            red[wave - 1][0][v * 64 + lane] = acc[v];
            if constexpr (TWO) red[wave - 1][1][v * 64 + lane] = acc2[v];
        }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            acc[v] += red[w][0][v * 64 + lane];
            if constexpr (TWO) acc2[v] += red[w][1][v * 64 + lane];
        }

    linear_epilogue<EPI, PARTS>(p, acc, acc2, a, blk, wb, lane);
}

// The same products for problems with many rows (the diffusion attention's 5 x 768 tokens, the
// N^2 positions of the generic pair-track paths): one workgroup computes 128 positions x 128 output
// channels, its 4 wavefronts in a 2 x 2 grid of 64 x 64 (2 position blocks x 2 weight blocks, every
// fragment feeds two MFMAs), the whole K per wavefront in register-prefetched chunks, no partial sums.
template <int EPI, bool AFRAG>
__global__ __launch_bounds__(256) void linear_tile_kernel(LinearArgs p) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    const int groups = (p.nb + 3) / 4;                       // groups of 4 position blocks per row group
    const int a = blockIdx.x / groups, blk0 = (blockIdx.x % groups) * 4 + 2 * wm;
    const int wb0 = blockIdx.y * 4 + 2 * wn;
    const int ksteps = p.K / 16;
    constexpr bool W_IS_A = (EPI == EPI_FRAG_CH || EPI == EPI_PLANES);
    constexpr bool TWO = (EPI == EPI_SWIGLU || EPI == EPI_ADALN || EPI == EPI_PLANES);
    constexpr int CH = TWO ? 2 : 4;                          // k-steps per prefetched chunk

    // blocks past the end are clamped for the loads and skipped in the epilogue
    int blk[2], wb[2];
    const char* arow[2];
    const char* Wb[2];
    const char* W2b[2];
    const int dks = 2 * p.PB;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        blk[i] = min(blk0 + i, p.nb - 1);
        wb[i] = min(wb0 + i, p.nblk - 1);
        const int pos = min(blk[i] * 32 + col, p.L - 1);
        arow[i] = AFRAG ? nullptr
                        : static_cast<const char*>(p.A) +
                              (((size_t)(p.a_shared ? 0 : a) * p.L + pos) * p.lda + 8 * half) * 2;
        Wb[i] = static_cast<const char*>(p.W) + ((size_t)wb[i] * ksteps * 64 + lane) * 16;
        W2b[i] = p.W2 ? static_cast<const char*>(p.W2) + ((size_t)wb[i] * ksteps * 64 + lane) * 16 : nullptr;
    }
    auto afrag = [&](int i, int ks) -> bf16x8 {
        if constexpr (AFRAG) {
            const int h = ks / dks, kk = ks % dks;
            const size_t u = ((((size_t)a * p.H + h) * p.nb + blk[i]) * dks + kk) * 64 + lane;
            return *reinterpret_cast<const bf16x8*>(static_cast<const char*>(p.A) + u * 16);
        } else {
            return *reinterpret_cast<const bf16x8*>(arow[i] + 32 * ks);
        }
    };
    auto wfrag = [&](const char* base, int ks) -> bf16x8 {
        return *reinterpret_cast<const bf16x8*>(base + (size_t)ks * 1024);
    };

    f32x16 acc[2][2], acc2[2][2];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) { acc[m][n][v] = 0.f; acc2[m][n][v] = 0.f; }

    bf16x8 xa[CH][2], wa[CH][2], va[CH][2], xb[CH][2], wb2[CH][2], vb[CH][2];
    auto load = [&](int c, bf16x8 (&x)[CH][2], bf16x8 (&w)[CH][2], bf16x8 (&v)[CH][2]) {
#pragma unroll
        for (int i = 0; i < CH; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int ks = min(c * CH + i, ksteps - 1);        // the last chunk may be short
                x[i][j] = afrag(j, ks);
                w[i][j] = wfrag(Wb[j], ks);
                if constexpr (TWO) v[i][j] = wfrag(W2b[j], ks);
            }
    };
    auto compute = [&](int c, const bf16x8 (&x)[CH][2], const bf16x8 (&w)[CH][2], const bf16x8 (&v)[CH][2]) {
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            if (c * CH + i >= ksteps) break;
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int n = 0; n < 2; ++n) {
                    acc[m][n] = W_IS_A ? mfma32(w[i][n], x[i][m], acc[m][n]) : mfma32(x[i][m], w[i][n], acc[m][n]);
                    if constexpr (TWO)
                        acc2[m][n] = W_IS_A ? mfma32(v[i][n], x[i][m], acc2[m][n]) : mfma32(x[i][m], v[i][n], acc2[m][n]);
                }
        }
    };
    const int nch = (ksteps + CH - 1) / CH;
    load(0, xa, wa, va);
    for (int c = 0; c < nch; c += 2) {
        if (c + 1 < nch) load(c + 1, xb, wb2, vb);
        compute(c, xa, wa, va);
        if (c + 1 < nch) {
            if (c + 2 < nch) load(c + 2, xa, wa, va);
            compute(c + 1, xb, wb2, vb);
        }
    }
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            if (blk0 + m >= p.nb || wb0 + n >= p.nblk) continue;
            linear_epilogue<EPI, 1>(p, acc[m][n], acc2[m][n], a, blk0 + m, wb0 + n, lane);
        }
}

int launch_linear(const LinearArgs& p, hipStream_t stream) {
    if (p.K % 16 || p.nb <= 0 || p.rows_a <= 0) return -1;
    dim3 grid((unsigned)(p.rows_a * p.nb), (unsigned)p.nblk), block(256);
#define KFH_LIN(E, F, P) hipLaunchKernelGGL((linear_kernel<E, F, P>), grid, block, 0, stream, p)
    if (p.parts == 3) {          // fp32 arithmetic on split operands (pair-bias attention only)
        switch (p.epi) {
            case EPI_SIGMOID: KFH_LIN(EPI_SIGMOID, false, 3); break;
            case EPI_ADALN: KFH_LIN(EPI_ADALN, false, 3); break;
            case EPI_RESID: if (p.a_frag) KFH_LIN(EPI_RESID, true, 3); else return -1; break;
            case EPI_FRAG_CH: KFH_LIN(EPI_FRAG_CH, false, 3); break;
            case EPI_FRAG_POS: KFH_LIN(EPI_FRAG_POS, false, 3); break;
            default: return -1;
        }
        return 0;
    }
    if (p.parts != 0 && p.parts != 1) return -1;
    // many rows and more than one weight block: the 128 x 128 tile kernel, once its grid has enough
    // workgroups for the chip (default 128; the environment variable KFH_LINEAR_TILE_MIN_WORKGROUPS
    // overrides it, e.g. 1 to use the tile kernel wherever it applies)
    const char* tile_env = std::getenv("KFH_LINEAR_TILE_MIN_WORKGROUPS");
    const long long tile_req = tile_env ? std::atoll(tile_env) : 0;
    const long long tile_min = tile_req > 0 ? tile_req : 128LL;
    const long long tile_groups = (long long)p.rows_a * ((p.nb + 3) / 4);
    const int tile_cols = (p.nblk + 3) / 4;
    if (p.nblk >= 2 && tile_groups * tile_cols >= tile_min && tile_groups <= 0x7fffffffLL) {
        dim3 tgrid((unsigned)tile_groups, (unsigned)tile_cols);
#define KFH_TILE(E, F) hipLaunchKernelGGL((linear_tile_kernel<E, F>), tgrid, block, 0, stream, p)
        switch (p.epi) {
            case EPI_STORE: if (p.a_frag) KFH_TILE(EPI_STORE, true); else KFH_TILE(EPI_STORE, false); return 0;
            case EPI_SIGMOID: KFH_TILE(EPI_SIGMOID, false); return 0;
            case EPI_SWIGLU: KFH_TILE(EPI_SWIGLU, false); return 0;
            case EPI_ADALN: KFH_TILE(EPI_ADALN, false); return 0;
            case EPI_RESID: if (p.a_frag) KFH_TILE(EPI_RESID, true); else KFH_TILE(EPI_RESID, false); return 0;
            case EPI_FRAG_CH: KFH_TILE(EPI_FRAG_CH, false); return 0;
            case EPI_FRAG_POS: KFH_TILE(EPI_FRAG_POS, false); return 0;
            case EPI_PLANES: if (!p.mask || !p.W2) return -1; KFH_TILE(EPI_PLANES, false); return 0;
            default: return -1;
        }
#undef KFH_TILE
    }
    switch (p.epi) {
        case EPI_STORE: if (p.a_frag) KFH_LIN(EPI_STORE, true, 1); else KFH_LIN(EPI_STORE, false, 1); break;
        case EPI_SIGMOID: KFH_LIN(EPI_SIGMOID, false, 1); break;
        case EPI_SWIGLU: KFH_LIN(EPI_SWIGLU, false, 1); break;
        case EPI_ADALN: KFH_LIN(EPI_ADALN, false, 1); break;
        case EPI_RESID: if (p.a_frag) KFH_LIN(EPI_RESID, true, 1); else KFH_LIN(EPI_RESID, false, 1); break;
        case EPI_FRAG_CH: KFH_LIN(EPI_FRAG_CH, false, 1); break;
        case EPI_FRAG_POS: KFH_LIN(EPI_FRAG_POS, false, 1); break;
        case EPI_PLANES: if (!p.mask || !p.W2) return -1; KFH_LIN(EPI_PLANES, false, 1); break;
        default: return -1;
    }
#undef KFH_LIN
    return 0;
}

}  // namespace kfh
