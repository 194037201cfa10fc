// Attention with an additive pair bias in fp32 arithmetic on the bf16 matrix cores.
//
// The diffusion stack of the reference runs outside autocast (model/model.py:419) and its kernels
// with full fp32 dot products (kernels/triton/attention_pair_bias/dispatch.py:439,453).  Here every
// fp32 operand of a product — q, k, v, and the probabilities — is carried as the three bf16 parts
// of split3() (common.hpp), and a product is the sum of the six part pairs (i, j), i + j <= 2,
// each an exact bf16 x bf16 MFMA product accumulated in fp32.  The pair bias enters as fp32 tiles
// (the C operand of the first score MFMA), softmax statistics and the gate are plain fp32.
//
// Same math and masking rules as flash.hip (model/primitives/attention.py:151-166, 255-257):
//   L[a,h,q,k] = q . k + bias[h,q,k],  masked keys get probability 0,  o = softmax_k(L) v * gate
// and a row without any valid key attends uniformly over its real keys (finite -1e9 semantics).
//
// Operand layouts are those of flash.hip with a leading part index:
//   q, k, g, of : [part][row a][head h][block of 32][k-step 0..DKS-1][lane][8 bf16]
//   v           : [part][row a][head h][block of 32 keys][d-block][k-step 0..1][lane][8 bf16]
//   bias        : [bias batch][head][query block][key block] fp32 tiles of 4 KiB, times log2(e)
//
// One wavefront owns one (row, head, query block) and walks the key blocks with the exact online
// softmax (running maximum, rescale per block).  These problems are small (a few samples or
// windows), so operands are read straight from L2 and nothing is staged in LDS.
#include "kernels.hpp"

namespace kfh {

namespace {

__device__ __forceinline__ bf16x8 frag_at(const void* base, size_t part_bytes, int q, size_t unit) {
    return *reinterpret_cast<const bf16x8*>(static_cast<const char*>(base) + (size_t)q * part_bytes + unit * 16);
}

// the six part pairs of a split product, smallest terms first
__device__ constexpr int kPairA[6] = {2, 1, 0, 1, 0, 0};
__device__ constexpr int kPairB[6] = {0, 1, 2, 0, 1, 0};

}  // namespace

template <int DKS, int DV>
__global__ __launch_bounds__(256) void flash_split_kernel(FlashArgs p) {
    static_assert(DKS == 2 * DV, "head dim = 16*DKS = 32*DV");
    constexpr int KV_UNITS = DKS * 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int nb = p.nb, nbq = p.nbq, H = p.H;
    const int qb = blockIdx.x * 4 + wave, h = blockIdx.y, a = blockIdx.z;
    if (qb >= nbq) return;                               // no workgroup barrier below

    const size_t qunit = (((size_t)a * H + h) * nbq + qb) * KV_UNITS + lane;
    bf16x8 q[3][DKS];
#pragma unroll
    for (int s = 0; s < 3; ++s)
#pragma unroll
        for (int ks = 0; ks < DKS; ++ks) q[s][ks] = frag_at(p.qf, p.q_part, s, qunit + ks * 64);

    // does the row have a valid key at all?
    const uint8_t* crow = p.codes + (size_t)a * nb * 32;
    bool mine_valid = false;
    for (int k = lane; k < nb * 32; k += 64) mine_valid = mine_valid || crow[k] == 2;
    const bool row_valid = __any(mine_valid);

    const size_t batch = p.bias_per_row ? (size_t)a : 0;
    const f32x4* bt = reinterpret_cast<const f32x4*>(
        static_cast<const char*>(p.biast) + (((batch * H + h) * nbq + qb) * nb) * (size_t)kBiasTileF32Bytes);

    f32x16 o[DV];
#pragma unroll
    for (int d = 0; d < DV; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[d][v] = 0.f;
    float m = 0.f, l = 0.f;
    bool first = true;

    for (int kb = 0; kb < nb; ++kb) {
        // codes of this lane's 16 keys: key = 32 kb + acc_row(v, half)
        uint32_t cw[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) cw[g] = *reinterpret_cast<const uint32_t*>(crow + kb * 32 + 8 * g + 4 * half);
        bool take[16];
        bool any_mine = false;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t code = (cw[v >> 2] >> (8 * (v & 3))) & 0xffu;
            take[v] = row_valid ? code == 2 : code >= 1;
            any_mine = any_mine || take[v];
        }
        if (!__any(any_mine)) continue;                  // nothing of this block takes part

        // S^T[key][query] = bias + K Q^T over the six part pairs
        const size_t kunit = (((size_t)a * H + h) * nb + kb) * KV_UNITS + lane;
        f32x16 s;
        {
            const f32x4* t = bt + (size_t)kb * (kBiasTileF32Bytes / 16) + lane;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const f32x4 w = t[c * 64];
#pragma unroll
                for (int e = 0; e < 4; ++e) s[4 * c + e] = w[e];
            }
        }
#pragma unroll
        for (int ks = 0; ks < DKS; ++ks) {
            bf16x8 kf[3];
#pragma unroll
            for (int i = 0; i < 3; ++i) kf[i] = frag_at(p.kf, p.k_part, i, kunit + ks * 64);
#pragma unroll
            for (int pr = 0; pr < 6; ++pr) s = mfma32(kf[kPairA[pr]], q[kPairB[pr]][ks], s);
        }
        // masking; a row without valid keys weighs all its real keys equally
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            s[v] = take[v] ? (row_valid ? s[v] : 0.f) : -INFINITY;
            mx = fmaxf(mx, s[v]);
        }
        mx = xhalf_max(mx);                              // finite: every query sees the same keys
        const float m_new = first ? mx : fmaxf(m, mx);
        const float alpha = first ? 0.f : exp2f(m - m_new);
        m = m_new;
        first = false;
        float e[16], ls = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            e[v] = exp2f(s[v] - m_new);
            ls += e[v];
        }
        l = l * alpha + ls;
#pragma unroll
        for (int d = 0; d < DV; ++d)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[d][v] *= alpha;
        // probabilities as split B operands: two k-steps (registers 0..7, 8..15) per part
        bf16x8 pf[3][2];
        {
            f32x16 part[3];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float sp[3];
                split3(e[v], sp);
#pragma unroll
                for (int i = 0; i < 3; ++i) part[i][v] = sp[i];
            }
#pragma unroll
            for (int i = 0; i < 3; ++i) acc_to_frags(part[i], pf[i][0], pf[i][1]);
        }
        // O^T[d][query] += V^T[d][key] P^T[key][query]
#pragma unroll
        for (int d = 0; d < DV; ++d) {
            bf16x8 vf[3][2];
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                vf[i][0] = frag_at(p.vf, p.v_part, i, kunit + (2 * d) * 64);
                vf[i][1] = frag_at(p.vf, p.v_part, i, kunit + (2 * d + 1) * 64);
            }
#pragma unroll
            for (int pr = 0; pr < 6; ++pr) {
                o[d] = mfma32(vf[kPairA[pr]][0], pf[kPairB[pr]][0], o[d]);
                o[d] = mfma32(vf[kPairA[pr]][1], pf[kPairB[pr]][1], o[d]);
            }
        }
    }

    const float inv = 1.0f / xhalf_sum(l);
#pragma unroll
    for (int d = 0; d < DV; ++d) {
        const size_t u0 = qunit + (2 * d) * 64;
        f32x16 og;
#pragma unroll
        for (int v = 0; v < 16; ++v) og[v] = o[d][v] * inv;
        if (p.gf != nullptr) {
            // gate = sum of its three parts, in the register order of the accumulator
            float g[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) g[v] = 0.f;
#pragma unroll
            for (int i = 2; i >= 0; --i) {
                const u32x4 g0 = __builtin_bit_cast(u32x4, frag_at(p.gf, p.g_part, i, u0));
                const u32x4 g1 = __builtin_bit_cast(u32x4, frag_at(p.gf, p.g_part, i, u0 + 64));
#pragma unroll
                for (int e2 = 0; e2 < 4; ++e2) {
                    g[2 * e2] += bf16_lo(g0[e2]);
                    g[2 * e2 + 1] += bf16_hi(g0[e2]);
                    g[8 + 2 * e2] += bf16_lo(g1[e2]);
                    g[8 + 2 * e2 + 1] += bf16_hi(g1[e2]);
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) og[v] *= g[v];
        }
        f32x16 part[3];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float sp[3];
            split3(og[v], sp);
#pragma unroll
            for (int i = 0; i < 3; ++i) part[i][v] = sp[i];
        }
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            bf16x8 f0, f1;
            acc_to_frags(part[i], f0, f1);
            bf16x8* dst = reinterpret_cast<bf16x8*>(static_cast<char*>(p.of) + (size_t)i * p.o_part + u0 * 16);
            dst[0] = f0;
            dst[64] = f1;
        }
    }
}

int launch_flash_split(const FlashArgs& args_in, int head_dim_pad, hipStream_t stream) {
    FlashArgs p = args_in;
    if (p.nbq <= 0) p.nbq = p.nb;
    if (p.nb <= 0 || p.nb > 256 || p.nbq > 256 || p.nrows <= 0 || p.nrows > 65535 || p.H <= 0 || p.H > 65535)
        return -1;
    const dim3 grid((unsigned)((p.nbq + 3) / 4), (unsigned)p.H, (unsigned)p.nrows), block(256);
    if (head_dim_pad == 32) hipLaunchKernelGGL((flash_split_kernel<2, 1>), grid, block, 0, stream, p);
    else if (head_dim_pad == 64) hipLaunchKernelGGL((flash_split_kernel<4, 2>), grid, block, 0, stream, p);
    else return -1;
    return 0;
}

}  // namespace kfh
