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
//   EPI_RESID    y = aux + gate * (acc + bias)      (aux, gate optional) layers/folding/attention_pair_bias.py:155-157
//   EPI_FRAG_CH  fragments with channels as accumulator rows (q, k, gate of attention)
//   EPI_FRAG_POS fragments with positions as accumulator rows (v of attention)
#include "kernels.hpp"

namespace kfh {

template <int EPI, bool AFRAG>
__global__ __launch_bounds__(256) void linear_kernel(LinearArgs p) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    // The 4 wavefronts of a workgroup share one 32 x 32 output tile and split K between them in
    // chunks of 8 k-steps (wavefront w takes chunks w, w+4, ...): these problems have few tiles
    // and long K, so the serial chain of dependent operand loads is what costs.
    __shared__ float red[3][2][64 * 16];
    const int wb = blockIdx.y;
    const int a = blockIdx.x / p.nb, blk = blockIdx.x % p.nb;
    const int ksteps = p.K / 16;
    const bf16x8* __restrict__ W = static_cast<const bf16x8*>(p.W) + (size_t)wb * ksteps * 64 + lane;
    const bf16x8* __restrict__ W2 = p.W2 ? static_cast<const bf16x8*>(p.W2) + (size_t)wb * ksteps * 64 + lane : nullptr;

    const int pos = min(blk * 32 + col, p.L - 1);
    const uint16_t* arow = AFRAG ? nullptr
                                 : static_cast<const uint16_t*>(p.A) + ((size_t)(p.a_shared ? 0 : a) * p.L + pos) * p.lda + 8 * half;
    const int dks = 2 * p.PB;
    auto afrag = [&](int ks) -> bf16x8 {
        if constexpr (AFRAG) {
            const int h = ks / dks, kk = ks % dks;
            return static_cast<const bf16x8*>(p.A)[((((size_t)a * p.H + h) * p.nb + blk) * dks + kk) * 64 + lane];
        } else {
            return *reinterpret_cast<const bf16x8*>(arow + 16 * ks);
        }
    };

    f32x16 acc, acc2;
#pragma unroll
    for (int v = 0; v < 16; ++v) { acc[v] = 0.f; acc2[v] = 0.f; }
    constexpr bool W_IS_A = (EPI == EPI_FRAG_CH);
    constexpr bool TWO = (EPI == EPI_SWIGLU || EPI == EPI_ADALN);
    // K is walked in chunks of 8 k-steps; the operands of chunk c+1 are
    // requested before the MFMAs of chunk c, so one memory latency is paid per 8 k-steps at most
    constexpr int CH = 8;
    bf16x8 xa[CH], wa[CH], va[CH], xb[CH], wb2[CH], vb[CH];
    auto load = [&](int c, bf16x8 (&x)[CH], bf16x8 (&w)[CH], bf16x8 (&v)[CH]) {
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            x[i] = afrag(c * CH + i);
            w[i] = W[(size_t)(c * CH + i) * 64];
            if constexpr (TWO) v[i] = W2[(size_t)(c * CH + i) * 64];
        }
    };
    auto compute = [&](const bf16x8 (&x)[CH], const bf16x8 (&w)[CH], const bf16x8 (&v)[CH]) {
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            acc = W_IS_A ? mfma32(w[i], x[i], acc) : mfma32(x[i], w[i], acc);
            if constexpr (TWO) acc2 = mfma32(x[i], v[i], acc2);
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
        for (int ks = nch * CH; ks < ksteps; ++ks) {      // K not a multiple of 128
            const bf16x8 x = afrag(ks);
            const bf16x8 w = W[(size_t)ks * 64];
            acc = W_IS_A ? mfma32(w, x, acc) : mfma32(x, w, acc);
            if constexpr (TWO) acc2 = mfma32(x, W2[(size_t)ks * 64], acc2);
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

    if constexpr (EPI == EPI_FRAG_CH || EPI == EPI_FRAG_POS) {
        const int h = wb / p.PB, pp = wb % p.PB;
        if constexpr (EPI == EPI_FRAG_CH) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int d = 32 * pp + acc_row(v, half);
                float y = acc[v];
                if (p.bias && d < p.Dh) y += p.bias[h * p.Dh + d] * p.bias_scale;
                if (p.sigmoid) y = sigmoidf_fast(y);
                acc[v] = y;
            }
        }
        bf16x8 f0, f1;
        acc_to_frags(acc, f0, f1);
        bf16x8* dst = static_cast<bf16x8*>(p.out) +
                      ((((size_t)a * p.H + h) * p.nb + blk) * p.PB + pp) * 2 * 64 + lane;
        dst[0] = f0;
        dst[64] = f1;
    } else {
        const int c = 32 * wb + col;
        if (c >= p.Nout) return;
        const float bc = p.bias ? p.bias[c] : 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int ps = blk * 32 + acc_row(v, half);
            if (ps >= p.L) continue;
            size_t r = (size_t)a * p.L + ps;
            size_t r_aux = (size_t)(p.aux_shared ? 0 : a) * p.L + ps;
            if constexpr (EPI == EPI_RESID) {
                if (p.out_transposed) { r = (size_t)ps * p.rows_a + a; r_aux = r; }
            }
            const size_t r_gate = (size_t)(p.gate_shared ? 0 : a) * p.L + ps;
            float y = acc[v] + bc;
            if constexpr (EPI == EPI_SIGMOID) y = sigmoidf_fast(y);
            if constexpr (EPI == EPI_SWIGLU) y = acc[v] * sigmoidf_fast(acc[v]) * acc2[v];
            if constexpr (EPI == EPI_ADALN) {
                const float ax = bf16_lo(static_cast<const uint16_t*>(p.aux)[r_aux * p.ld_aux + c]);
                y = sigmoidf_fast(y) * ax + acc2[v];
            }
            if constexpr (EPI == EPI_RESID) {
                if (p.gate) y *= bf16_lo(p.gate[r_gate * p.ld_gate + c]);
                if (p.aux) {
                    y += p.aux_dtype == KFH_F32 ? static_cast<const float*>(p.aux)[r_aux * p.ld_aux + c]
                                                : bf16_lo(static_cast<const uint16_t*>(p.aux)[r_aux * p.ld_aux + c]);
                }
            }
            if (p.out_dtype == KFH_F32) static_cast<float*>(p.out)[r * p.ldo + c] = y;
            else static_cast<uint16_t*>(p.out)[r * p.ldo + c] = (uint16_t)(pack_bf16(y, 0.f) & 0xffffu);
        }
    }
}

int launch_linear(const LinearArgs& p, hipStream_t stream) {
    if (p.K % 16 || p.nb <= 0 || p.rows_a <= 0) return -1;
    dim3 grid((unsigned)(p.rows_a * p.nb), (unsigned)p.nblk), block(256);
#define KFH_LIN(E, F) hipLaunchKernelGGL((linear_kernel<E, F>), grid, block, 0, stream, p)
    switch (p.epi) {
        case EPI_STORE: if (p.a_frag) KFH_LIN(EPI_STORE, true); else KFH_LIN(EPI_STORE, false); break;
        case EPI_SIGMOID: KFH_LIN(EPI_SIGMOID, false); break;
        case EPI_SWIGLU: KFH_LIN(EPI_SWIGLU, false); break;
        case EPI_ADALN: KFH_LIN(EPI_ADALN, false); break;
        case EPI_RESID: if (p.a_frag) KFH_LIN(EPI_RESID, true); else KFH_LIN(EPI_RESID, false); break;
        case EPI_FRAG_CH: KFH_LIN(EPI_FRAG_CH, false); break;
        case EPI_FRAG_POS: KFH_LIN(EPI_FRAG_POS, false); break;
        default: return -1;
    }
#undef KFH_LIN
    return 0;
}

}  // namespace kfh
