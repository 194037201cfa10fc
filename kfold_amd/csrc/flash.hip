// Attention with an additive pair bias shared by all rows of a batch, online softmax.
// Used by triangle attention (rows = the N rows of x', H = 4, head dim 32) and by pair-bias
// attention (rows = samples, H = 16, head dim 24 or 48 zero-padded to 32 or 64).
//
//   L[a,h,q,k] = q[a,h,q] . k[a,h,k] + bias[h,q,k]  (+ mask term),  o = softmax_k(L) v
//   of[a,h,q]  = o * g[a,h,q]                                   (g = sigmoid gate)
// Reference math: model/primitives/triangle_attention.py:132-152,328-330 and
// model/primitives/attention.py:151-166,255-257.  Logits are in the exp2 domain (q and the
// bias arrive pre-multiplied by log2 e).
//
// All operands are in MFMA fragment order (see common.hpp):
//   q, k, g, of : [row a][head h][block of 32 positions][k-step 0..DKS-1][lane][8 bf16]
//   v           : [row a][head h][block of 32 keys][d-block 0..DV-1][k-step 0..1][lane][8 bf16]
//   bias        : [bias batch][head h][query block][key block][4][lane][4 floats]
//   codes       : [row a][nb*32] bytes, 0 = beyond the sequence, 1 = masked key, 2 = valid key
//
// Wavefront = 32 queries of up to R rows for one head; workgroup = 4 adjacent query blocks.
// S^T[key][query] = K Q^T + bias comes out of the MFMA with the bias tile as its C operand,
// so a lane owns 16 keys of one query: the row max and row sum need one cross-half
// exchange, and exp2(S - m) rounded to bf16 is already the B operand of
// O^T[d][query] += V^T[d][key] P^T[key][query].  The R rows share the bias tile registers.
//
// Masking follows the reference's finite -1e9 semantics: in a row with a valid key, masked
// keys get probability exactly 0; in a row with no valid key all real keys get the same
// logit (q.k + bias is absorbed by -1e9 in fp32), i.e. uniform attention.
#include "kernels.hpp"

namespace kfh {

template <int R, int DKS, int DV>
__global__ __launch_bounds__(256, (DKS == 2 ? 2 : 1)) void flash_kernel(FlashArgs p) {
    static_assert(DKS == 2 * DV, "head dim = 16*DKS = 32*DV");
    __shared__ uint8_t cls_s[4][R][256];      // per wavefront: class of each key block per row
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int half = lane >> 5;
    const int nb = p.nb, H = p.H;
    const bf16x8* __restrict__ qf = static_cast<const bf16x8*>(p.qf);
    const bf16x8* __restrict__ kf = static_cast<const bf16x8*>(p.kf);
    const bf16x8* __restrict__ vf = static_cast<const bf16x8*>(p.vf);
    const bf16x8* __restrict__ gf = static_cast<const bf16x8*>(p.gf);
    bf16x8* __restrict__ of = static_cast<bf16x8*>(p.of);

    // chunk = (head, row set); all query groups of a chunk run on one XCD (workgroup ids are
    // dealt round-robin over 8 XCDs); heads are the slowest index
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int chunk = (slot / p.qgroups) * 8 + xcd;
    if (chunk >= p.nchunks) return;
    const int qb = (slot % p.qgroups) * 4 + wave;
    const int rowsets = (p.nrows + R - 1) / R;
    const int h = chunk / rowsets, a0 = (chunk % rowsets) * R;
    if (qb >= nb) return;
    const int nr = min(R, p.nrows - a0);      // rows of this set that exist

    auto qidx = [&](int a, int blk, int ks) -> size_t {
        return ((((size_t)a * H + h) * nb + blk) * DKS + ks) * 64 + lane;
    };
    auto vidx = [&](int a, int blk, int d, int ks) -> size_t {
        return (((((size_t)a * H + h) * nb + blk) * DV + d) * 2 + ks) * 64 + lane;
    };

    // ---- per row: classify key blocks: 2 all valid, 1 some valid, 0x81 real keys but none
    // valid, 0x80 nothing --------------------------------------------------------------------
    bool uniform_row[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        uniform_row[r] = false;
        if (r >= nr) continue;
        const uint8_t* crow = p.codes + (size_t)(a0 + r) * nb * 32;
        bool any_valid = false;
        for (int base = 0; base < nb; base += 64) {
            const int blk = base + lane;
            int nvalid = 0, nreal = 0;
            if (blk < nb) {
                const u32x4* c = reinterpret_cast<const u32x4*>(crow + blk * 32);
                const u32x4 c0 = c[0], c1 = c[1];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    nvalid += __popc(c0[i] & 0x02020202u) + __popc(c1[i] & 0x02020202u);
                    nreal += __popc(c0[i] & 0x03030303u) + __popc(c1[i] & 0x03030303u);
                }
                cls_s[wave][r][blk] = nvalid == 32 ? 2 : (nvalid > 0 ? 1 : (nreal > 0 ? 0x81 : 0x80));
            }
            const bool v = __ballot(nvalid > 0) != 0ull;
            any_valid = any_valid || v;
        }
        uniform_row[r] = !any_valid;
    }
    __builtin_amdgcn_s_waitcnt(0);   // the LDS bytes above are read back by this wavefront only
    __builtin_amdgcn_wave_barrier();

    bf16x8 q[R][DKS];
    f32x16 o[R][DV];
    float m[R], l[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int a = a0 + min(r, nr - 1);
#pragma unroll
        for (int ks = 0; ks < DKS; ++ks) q[r][ks] = qf[qidx(a, qb, ks)];
#pragma unroll
        for (int d = 0; d < DV; ++d)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[r][d][v] = 0.f;
        m[r] = -1e30f;
        l[r] = 0.f;
    }

    const size_t bias_stride = (size_t)H * nb * nb * 256;     // f32x4 units per bias batch
    for (int kb = 0; kb < nb; ++kb) {
        f32x16 bias;
        bool have_bias = false;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r >= nr) continue;
            const int a = a0 + r;
            int cls = __builtin_amdgcn_readfirstlane((int)cls_s[wave][r][kb]);
            const bool uni = uniform_row[r];
            if (cls & 0x80) {                    // no valid key in this block
                if (!(uni && (cls & 1))) continue;
                cls = 1;                         // uniform row: masked real keys take part
            }
            if (!have_bias || p.bias_per_row) {
                const f32x4* bt = static_cast<const f32x4*>(p.biasf) +
                                  (p.bias_per_row ? (size_t)a * bias_stride : 0) +
                                  (((size_t)h * nb + qb) * nb + kb) * 256 + lane;
                const f32x4 b0 = bt[0], b1 = bt[64], b2 = bt[128], b3 = bt[192];
#pragma unroll
                for (int e = 0; e < 4; ++e) { bias[e] = b0[e]; bias[4 + e] = b1[e]; bias[8 + e] = b2[e]; bias[12 + e] = b3[e]; }
                have_bias = true;
            }
            bf16x8 kk[DKS], vv[DV][2];
#pragma unroll
            for (int ks = 0; ks < DKS; ++ks) kk[ks] = kf[qidx(a, kb, ks)];
#pragma unroll
            for (int d = 0; d < DV; ++d) { vv[d][0] = vf[vidx(a, kb, d, 0)]; vv[d][1] = vf[vidx(a, kb, d, 1)]; }
            f32x16 s = bias;
#pragma unroll
            for (int ks = 0; ks < DKS; ++ks) s = mfma32(kk[ks], q[r][ks], s);
            if (cls != 2) {
                // this lane's keys: 8*(v/4) + 4*half + (v%4) -> one dword of codes per 4 keys
                const uint32_t* cw = reinterpret_cast<const uint32_t*>(
                    p.codes + (size_t)a * nb * 32 + kb * 32 + 4 * half);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t w = cw[2 * g];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t code = (w >> (8 * e)) & 0xffu;
                        const int v = 4 * g + e;
                        if (uni) s[v] = code == 1 ? 0.f : -INFINITY;
                        else if (code != 2) s[v] = -INFINITY;
                    }
                }
            }
            float mx = s[0];
#pragma unroll
            for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[v]);
            mx = xhalf_max(mx);
            const float m_new = fmaxf(m[r], mx);
            const float alpha = fast_exp2(m[r] - m_new);
            m[r] = m_new;
            float ls = 0.f;
#pragma unroll
            for (int v = 0; v < 16; ++v) { s[v] = fast_exp2(s[v] - m_new); ls += s[v]; }
            l[r] = l[r] * alpha + ls;
            bf16x8 p0, p1;
            acc_to_frags(s, p0, p1);
#pragma unroll
            for (int d = 0; d < DV; ++d) {
#pragma unroll
                for (int v = 0; v < 16; ++v) o[r][d][v] *= alpha;
                o[r][d] = mfma32(vv[d][0], p0, o[r][d]);
                o[r][d] = mfma32(vv[d][1], p1, o[r][d]);
            }
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (r >= nr) continue;
        const int a = a0 + r;
        const float inv = fast_rcp(xhalf_sum(l[r]));
#pragma unroll
        for (int d = 0; d < DV; ++d) {
            const u32x4 g0 = __builtin_bit_cast(u32x4, gf[qidx(a, qb, 2 * d)]);
            const u32x4 g1 = __builtin_bit_cast(u32x4, gf[qidx(a, qb, 2 * d + 1)]);
            f32x16 og;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                og[2 * e] = o[r][d][2 * e] * inv * bf16_lo(g0[e]);
                og[2 * e + 1] = o[r][d][2 * e + 1] * inv * bf16_hi(g0[e]);
                og[8 + 2 * e] = o[r][d][8 + 2 * e] * inv * bf16_lo(g1[e]);
                og[8 + 2 * e + 1] = o[r][d][8 + 2 * e + 1] * inv * bf16_hi(g1[e]);
            }
            bf16x8 f0, f1;
            acc_to_frags(og, f0, f1);
            of[qidx(a, qb, 2 * d)] = f0;
            of[qidx(a, qb, 2 * d + 1)] = f1;
        }
    }
}

int launch_flash(const FlashArgs& args, int head_dim_pad, hipStream_t stream) {
    constexpr int R = 4;
    FlashArgs p = args;
    p.qgroups = (p.nb + 3) / 4;
    p.nchunks = p.H * ((p.nrows + R - 1) / R);
    const int nslots = ((p.nchunks + 7) / 8) * p.qgroups;
    if (p.nb > 256) return -1;
    if (head_dim_pad == 32)
        hipLaunchKernelGGL((flash_kernel<R, 2, 1>), dim3(nslots * 8), dim3(256), 0, stream, p);
    else if (head_dim_pad == 64)
        hipLaunchKernelGGL((flash_kernel<R, 4, 2>), dim3(nslots * 8), dim3(256), 0, stream, p);
    else
        return -1;
    return 0;
}

}  // namespace kfh
