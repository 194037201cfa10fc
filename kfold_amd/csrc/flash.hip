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
//   bias        : [bias batch][head h][query block][key block] bf16 tiles of 2 KiB
//   codes       : [row a][nb*32] bytes, 0 = beyond the sequence, 1 = masked key, 2 = valid key
//
// A wavefront computes S^T[key][query] for 32 keys x 32 queries with keys as accumulator rows:
//   S^T = bias^T + 1 (-m)^T + K Q^T
// the bias tile (stored in accumulator register order, widened from bf16) is the C operand, a
// constant-one column against the running maximum m makes the accumulator S - m (so the
// exponent needs no subtraction), then the scores.  A lane then owns 16 keys of one query: the
// row max and row sum need one cross-half exchange, and exp2(S - m) rounded to bf16 is
// already the B operand of O^T[d][query] += V^T[d][key] P^T[key][query].  m only moves when
// a logit exceeds it by 2^8 (lazy rescale, exact path) or a lane's partial row sum exceeds
// 2^40 (max-free path); it is kept bf16-representable so the MFMA subtracts it exactly.
//
// Two kernels share that tile code:
//   flash_strip_kernel  (triangle attention, N <= 1216): a workgroup owns one head, two query
//       blocks and a range of rows; the bias strip of its query blocks (all key blocks) is
//       loaded into LDS once, then each wavefront walks its rows with K/V fragments read
//       straight from L2 — no barrier in the main loop, two score tiles in flight per step.
//   flash_staged_kernel (any size / head dim): 8 wavefronts = 4 query blocks x 2 row groups;
//       per key block K, V and bias tiles are staged in double-buffered LDS.
//
// Masking follows the reference's finite -1e9 semantics: in a row with a valid key, masked
// keys get probability exactly 0; in a row with no valid key all real keys get the same
// logit (q.k + bias is absorbed by -1e9 in fp32), i.e. uniform attention.
#include <atomic>

#include "kernels.hpp"

namespace kfh {

constexpr float kLazyMax = 8.0f;   // rescale only when a logit exceeds the running max by 2^8

// bf16 fragment with one non-zero k-slot: slot 0 of the lanes with half == 0
__device__ __forceinline__ bf16x8 slot0_frag(float v, int half) {
    u32x4 w = {0u, 0u, 0u, 0u};
    w[0] = half == 0 ? (pack_bf16(v, 0.f) & 0xffffu) : 0u;
    return __builtin_bit_cast(bf16x8, w);
}

__device__ __forceinline__ bf16x8 as_frag(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// Classify the key blocks of one row from its codes: 2 all valid, 1 some valid; with no valid
// key: 0x82 all 32 keys real (masked), 0x81 some real, 0x80 none.  One wavefront; returns
// true if the row has a valid key.
__device__ __forceinline__ int classify_block(const u32x4& c0, const u32x4& c1, int& nvalid) {
    int nreal = 0;
    nvalid = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        nvalid += __popc(c0[i] & 0x02020202u) + __popc(c1[i] & 0x02020202u);
        nreal += __popc(c0[i] & 0x03030303u) + __popc(c1[i] & 0x03030303u);
    }
    return nvalid == 32 ? 2 : (nvalid > 0 ? 1 : (nreal == 32 ? 0x82 : (nreal > 0 ? 0x81 : 0x80)));
}

__device__ __forceinline__ bool classify_row(const uint8_t* crow, int nb, int lane, uint8_t* cls,
                                             unsigned long long& act, unsigned long long& full) {
    bool any_valid = false;
    for (int base = 0; base < nb; base += 64) {
        const int blk = base + lane;
        int nvalid = 0;
        if (blk < nb) {
            const u32x4* c = reinterpret_cast<const u32x4*>(crow + blk * 32);
            cls[blk] = classify_block(c[0], c[1], nvalid);
        }
        // bit masks of the blocks with a valid key / with only valid keys (first 64 blocks)
        const unsigned long long va = __ballot(nvalid > 0), vf = __ballot(nvalid == 32);
        if (base == 0) { act = va; full = vf; }
        any_valid = any_valid || va != 0ull;
    }
    return any_valid;
}

// mixed block: per-key select.  s holds S - m; this lane's keys are 8*(v/4) + 4*half + (v%4)
__device__ __forceinline__ void mask_scores(f32x16& s, const uint8_t* codes_blk, int half, bool uni,
                                            float m) {
    const uint32_t* cw = reinterpret_cast<const uint32_t*>(codes_blk + 4 * half);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t w = cw[2 * g];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t code = (w >> (8 * e)) & 0xffu;
            const int v = 4 * g + e;
            const float masked = (uni && code == 1) ? -m : -INFINITY;
            s[v] = (!uni && code == 2) ? s[v] : masked;
        }
    }
}

__device__ __forceinline__ float tile_max(const f32x16& s) {
    float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
    for (int v = 3; v < 15; v += 2) mx = fmaxf(fmaxf(mx, s[v]), s[v + 1]);
    mx = fmaxf(mx, s[15]);
    return xhalf_max(mx);
}

// move the running maximum by (bf16-rounded) mx and rescale the partial results
template <int DV>
__device__ __forceinline__ void rescale(f32x16& s, float mx, float& m, float& l, f32x16 (&o)[DV],
                                        bf16x8& qx, int half, bool fresh) {
    // `fresh`: nothing accumulated yet (m = 0, l = 0, o = 0): the maximum may start anywhere,
    // and nothing needs scaling.  Afterwards the maximum only rises, so alpha <= 1 (a large
    // downward move would scale by exp2(+big) = inf).
    const float m_new = bf16_lo(pack_bf16(fresh ? mx : m + fmaxf(mx, 0.f), 0.f));
    const float delta = m_new - m;
    const float alpha = fresh ? 1.0f : fast_exp2(-delta);
    m = m_new;
    qx = slot0_frag(-m_new, half);
    l *= alpha;
#pragma unroll
    for (int d = 0; d < DV; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[d][v] *= alpha;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] -= delta;
}

// p = bf16(exp2(s)) as the two B-operand fragments of the PV product; returns this lane's
// partial row sum, taken over the fp32 exponentials with plain adds.  (A v_dot2c chain over the
// rounded bf16 values needs half the instructions, but DOT instructions do not overlap with
// MFMAs of other wavefronts: measured, 14 MFMAs + 32 v_dot2c take the sum of their times.  The
// rounding of p is unbiased, so numerator and normaliser still agree to well below bf16.)
__device__ __forceinline__ float exp_pack_sum(const f32x16& s, bf16x8& p0, bf16x8& p1) {
    f32x16 e;
#pragma unroll
    for (int v = 0; v < 16; ++v) e[v] = fast_exp2(s[v]);
    u32x4 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = pack_bf16(e[2 * i], e[2 * i + 1]);
        b[i] = pack_bf16(e[8 + 2 * i], e[8 + 2 * i + 1]);
    }
    p0 = __builtin_bit_cast(bf16x8, a);
    p1 = __builtin_bit_cast(bf16x8, b);
    const float t0 = (e[0] + e[1]) + (e[2] + e[3]), t1 = (e[4] + e[5]) + (e[6] + e[7]);
    const float t2 = (e[8] + e[9]) + (e[10] + e[11]), t3 = (e[12] + e[13]) + (e[14] + e[15]);
    return (t0 + t1) + (t2 + t3);
}

// Instruction order for a block of NM independent MFMAs and VALU work: one MFMA, then NV VALU
// instructions, repeated.
template <int NM, int NV>
__device__ __forceinline__ void interleave_mfma() {
    if constexpr (NM > 0) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);
        interleave_mfma<NM - 1, NV>();
    }
}

// A lane's partial row sum above this (or inf / NaN from an overflowed exponent) sends the
// tile through the exact max-and-rescale path instead.
constexpr float kSumLimit = 1.0995116e12f;   // 2^40

// ------------------------------------------------------------------------------------------
// strip kernel (head dim 32)
// ------------------------------------------------------------------------------------------
constexpr int kStripWaves = 12;          // 768 threads, 3 wavefronts per SIMD, one workgroup per CU
constexpr int kStripMaxBlocks = 38;      // 38 * 4 KiB strip + scratch <= 160 KiB LDS

__global__ __launch_bounds__(kStripWaves * 64, 3) void flash_strip_kernel(FlashArgs p) {
    HIP_DYNAMIC_SHARED(__attribute__((aligned(16))) char, lds)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int nb = p.nb, H = p.H;
    u32x4* strip = reinterpret_cast<u32x4*>(lds);                       // [kb][qbl][c][lane]
    uint8_t* cls = reinterpret_cast<uint8_t*>(lds) + (size_t)nb * 4096 + wave * 64;
    const u32x4* __restrict__ qf = static_cast<const u32x4*>(p.qf);
    const u32x4* __restrict__ kf = static_cast<const u32x4*>(p.kf);
    const u32x4* __restrict__ vf = static_cast<const u32x4*>(p.vf);
    const u32x4* __restrict__ gf = static_cast<const u32x4*>(p.gf);
    const u32x4* __restrict__ bt = static_cast<const u32x4*>(p.biast);
    u32x4* __restrict__ of = static_cast<u32x4*>(p.of);

    // chunk = (head, row range); the query-block pairs of a chunk share an XCD, heads slowest
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int chunk = (slot / p.qgroups) * 8 + xcd;
    if (chunk >= p.nchunks) return;
    const int pair = slot % p.qgroups;
    const int h = chunk / p.rowranges, rr = chunk % p.rowranges;
    const int qb[2] = {2 * pair, min(2 * pair + 1, nb - 1)};
    const bool have_b = 2 * pair + 1 < nb;

    // ---- bias strip of the two query blocks -> LDS -------------------------------------------
    for (int u = tid; u < nb * 256; u += kStripWaves * 64) {
        const int kb = u >> 8, qbl = (u >> 7) & 1, off = u & 127;
        strip[u] = bt[(((size_t)h * nb + qb[qbl]) * nb + kb) * 128 + off];
    }
    __syncthreads();

    const bf16x8 kx = slot0_frag(1.0f, half);
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // rows are dealt round-robin over the row ranges so that every workgroup gets the same mix
    // of padded and valid rows
    // The q fragments and key codes of a row are requested while the previous row of this
    // wavefront is being finished.
    u32x4 nq[4], nc[2];
    auto request_row = [&](int a) {
        const size_t ru = ((size_t)a * H + h) * nb * 128;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            nq[2 * t] = qf[ru + qb[t] * 128 + lane];
            nq[2 * t + 1] = qf[ru + qb[t] * 128 + 64 + lane];
        }
        const u32x4* c = reinterpret_cast<const u32x4*>(p.codes + (size_t)a * nb * 32 + min(lane, nb - 1) * 32);
        nc[0] = c[0];
        nc[1] = c[1];
    };
    const int a_first = rr + p.rowranges * wave, a_step = p.rowranges * kStripWaves;
    if (a_first < p.nrows) request_row(a_first);
    for (int a = a_first; a < p.nrows; a += a_step) {
        const size_t row_units = ((size_t)a * H + h) * nb * 128;        // fragment units of (a, h)
        const uint8_t* crow = p.codes + (size_t)a * nb * 32;
        int nvalid = 0;
        const int c_lane = classify_block(nc[0], nc[1], nvalid);
        if (lane < nb) cls[lane] = (uint8_t)c_lane; else nvalid = 0;
        const unsigned long long act = __ballot(nvalid > 0), full = __ballot(nvalid == 32);
        const bool uni = act == 0ull;
        bf16x8 q[2][2], qx[2];
        f32x16 o[2][1];
        float m[2] = {0.f, 0.f}, l[2] = {0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            q[t][0] = as_frag(nq[2 * t]);
            q[t][1] = as_frag(nq[2 * t + 1]);
            qx[t] = slot0_frag(0.f, half);
            o[t][0] = zero;
        }
        __builtin_amdgcn_s_waitcnt(0);   // cls bytes written above are read by this wavefront
        __builtin_amdgcn_wave_barrier();

        // scores of query block t against key block kb: bias + (1)(-m) + K Q^T
        auto score = [&](int t, int kb, const bf16x8& k0, const bf16x8& k1) -> f32x16 {
            const u32x4* sb = strip + kb * 256 + t * 128 + lane;
            f32x16 r = bias_tile_acc(sb[0], sb[64]);
            r = mfma32(kx, qx[t], r);
            r = mfma32(k0, q[t][0], r);
            return mfma32(k1, q[t][1], r);
        };
        // true maximum of the tile, running maximum moved, partial results rescaled
        auto renorm = [&](int t, f32x16& st) {
            rescale<1>(st, tile_max(st), m[t], l[t], o[t], qx[t], half, false);
        };

        if (uni) {
            // No valid key: every real key gets the same weight (see the masking note on top),
            // whatever the query, so both query blocks get the plain sum of V over real keys.
            // The V fragments of four blocks are requested before the first is used.
            const bf16x8 ones = as_frag(u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});
            for (int kb0 = 0; kb0 < nb; kb0 += 4) {
                u32x4 vv[4][2];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const u32x4* vp = vf + row_units + min(kb0 + i, nb - 1) * 128 + lane;
                    vv[i][0] = vp[0];
                    vv[i][1] = vp[64];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int kb = kb0 + i;
                    if (kb >= nb) break;
                    const int c = __builtin_amdgcn_readfirstlane((int)cls[kb]);
                    if (c == 0x80) continue;
                    bf16x8 p0 = ones, p1 = ones;
                    float cnt = 16.f;
                    if (c != 0x82) {
                        f32x16 sc = zero;
                        mask_scores(sc, crow + kb * 32, half, true, 0.f);
                        cnt = exp_pack_sum(sc, p0, p1);
                    }
                    l[0] += cnt;
                    o[0][0] = mfma32(as_frag(vv[i][0]), p0, o[0][0]);
                    o[0][0] = mfma32(as_frag(vv[i][1]), p1, o[0][0]);
                }
            }
            l[1] = l[0];
            o[1][0] = o[0][0];
        } else {
            // ---- Max-free pass over every block with a valid key.  The running maximum starts
            // at 0 (exp2 domain: logits are a few units wide in practice) and only moves when a
            // lane's partial row sum exceeds 2^40: then the tile is recomputed through the true
            // maximum (renorm).  First the blocks whose keys are all valid: the two query blocks
            // are two independent streams, run half a step apart so that the MFMAs of one are
            // issued between the exponentials of the other.
            unsigned long long fm = full;
            if (fm) {
                int kb = __builtin_ctzll(fm);
                fm &= fm - 1;
                const u32x4* kp = kf + row_units + kb * 128 + lane;
                const u32x4* vp = vf + row_units + kb * 128 + lane;
                bf16x8 k0 = as_frag(kp[0]), k1 = as_frag(kp[64]);
                bf16x8 v0 = as_frag(vp[0]), v1 = as_frag(vp[64]);
                f32x16 s0 = score(0, kb, k0, k1), s1;
                while (true) {
                    const bool more = fm != 0;
                    const int kn = more ? __builtin_ctzll(fm) : kb;
                    fm &= fm - 1;
                    // -- scores of stream 1 and the next K among the exponentials of stream 0
                    s1 = score(1, kb, k0, k1);
                    const u32x4* kpn = kf + row_units + kn * 128 + lane;
                    const bf16x8 kn0 = as_frag(kpn[0]), kn1 = as_frag(kpn[64]);
                    bf16x8 p0, p1;
                    float ls = exp_pack_sum(s0, p0, p1);
                    interleave_mfma<3, 12>();
                    if (__any(!(ls < kSumLimit))) {
                        s0 = score(0, kb, k0, k1);
                        renorm(0, s0);
                        ls = exp_pack_sum(s0, p0, p1);
                    }
                    l[0] += ls;
                    // -- PV of stream 0 and its next scores among the exponentials of stream 1
                    o[0][0] = mfma32(v0, p0, o[0][0]);
                    o[0][0] = mfma32(v1, p1, o[0][0]);
                    s0 = score(0, kn, kn0, kn1);
                    ls = exp_pack_sum(s1, p0, p1);
                    interleave_mfma<5, 8>();
                    if (__any(!(ls < kSumLimit))) {
                        s1 = score(1, kb, k0, k1);
                        renorm(1, s1);
                        ls = exp_pack_sum(s1, p0, p1);
                    }
                    l[1] += ls;
                    o[1][0] = mfma32(v0, p0, o[1][0]);
                    o[1][0] = mfma32(v1, p1, o[1][0]);
                    if (!more) break;
                    const u32x4* vpn = vf + row_units + kn * 128 + lane;
                    v0 = as_frag(vpn[0]);
                    v1 = as_frag(vpn[64]);
                    k0 = kn0;
                    k1 = kn1;
                    kb = kn;
                }
            }
            // blocks with masked keys, same max-free rule, one block at a time
            unsigned long long mixed = act & ~full;
            while (mixed) {
                const int kb = __builtin_ctzll(mixed);
                mixed &= mixed - 1;
                const u32x4* kp = kf + row_units + kb * 128 + lane;
                const u32x4* vp = vf + row_units + kb * 128 + lane;
                const bf16x8 k0 = as_frag(kp[0]), k1 = as_frag(kp[64]);
                const bf16x8 v0 = as_frag(vp[0]), v1 = as_frag(vp[64]);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    f32x16 st = score(t, kb, k0, k1);
                    mask_scores(st, crow + kb * 32, half, false, 0.f);
                    bf16x8 p0, p1;
                    float ls = exp_pack_sum(st, p0, p1);
                    if (__any(!(ls < kSumLimit))) {
                        st = score(t, kb, k0, k1);
                        mask_scores(st, crow + kb * 32, half, false, 0.f);
                        renorm(t, st);
                        ls = exp_pack_sum(st, p0, p1);
                    }
                    l[t] += ls;
                    o[t][0] = mfma32(v0, p0, o[t][0]);
                    o[t][0] = mfma32(v1, p1, o[t][0]);
                }
            }
            // ---- Every exponential underflowed (all logits of a query below -100 or so) or
            // something overflowed to NaN: redo the row with the true running maximum, block by
            // block (mask, maximum, rescale when it moved by more than 2^8).
            const float lt0 = xhalf_sum(l[0]), lt1 = xhalf_sum(l[1]);
            if (__any(!(fminf(lt0, lt1) > 1e-30f))) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    qx[t] = slot0_frag(0.f, half);
                    o[t][0] = zero;
                    m[t] = 0.f;
                    l[t] = 0.f;
                }
                unsigned long long todo = act;
                bool first = true;
                while (todo) {
                    const int kb = __builtin_ctzll(todo);
                    todo &= todo - 1;
                    const bool mixed = !((full >> kb) & 1ull);
                    const u32x4* kp = kf + row_units + kb * 128 + lane;
                    const u32x4* vp = vf + row_units + kb * 128 + lane;
                    const bf16x8 k0 = as_frag(kp[0]), k1 = as_frag(kp[64]);
                    const bf16x8 v0 = as_frag(vp[0]), v1 = as_frag(vp[64]);
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        f32x16 st = score(t, kb, k0, k1);
                        if (mixed) mask_scores(st, crow + kb * 32, half, false, m[t]);
                        const float mx = tile_max(st);
                        if (first || __any(mx > kLazyMax)) rescale<1>(st, mx, m[t], l[t], o[t], qx[t], half, first);
                        bf16x8 p0, p1;
                        l[t] += exp_pack_sum(st, p0, p1);
                        o[t][0] = mfma32(v0, p0, o[t][0]);
                        o[t][0] = mfma32(v1, p1, o[t][0]);
                    }
                    first = false;
                }
            }
        }

        const bool gated = p.gf != nullptr;     // triangle attention gates in its output kernel
        u32x4 gg[2][2];
        if (gated) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                gg[t][0] = gf[row_units + qb[t] * 128 + lane];
                gg[t][1] = gf[row_units + qb[t] * 128 + 64 + lane];
            }
        }
        if (a + a_step < p.nrows) request_row(a + a_step);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (t == 1 && !have_b) break;
            const float inv = fast_rcp(xhalf_sum(l[t]));
            const size_t u0 = row_units + qb[t] * 128 + lane;
            f32x16 og;
            if (gated) {
                const u32x4 g0 = gg[t][0], g1 = gg[t][1];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    og[2 * e] = o[t][0][2 * e] * inv * bf16_lo(g0[e]);
                    og[2 * e + 1] = o[t][0][2 * e + 1] * inv * bf16_hi(g0[e]);
                    og[8 + 2 * e] = o[t][0][8 + 2 * e] * inv * bf16_lo(g1[e]);
                    og[8 + 2 * e + 1] = o[t][0][8 + 2 * e + 1] * inv * bf16_hi(g1[e]);
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v) og[v] = o[t][0][v] * inv;
            }
            bf16x8 f0, f1;
            acc_to_frags(og, f0, f1);
            of[u0] = __builtin_bit_cast(u32x4, f0);
            of[u0 + 64] = __builtin_bit_cast(u32x4, f1);
        }
    }
}

// ------------------------------------------------------------------------------------------
// staged kernel (any sequence length, head dim 32 or 64)
// ------------------------------------------------------------------------------------------
// PERROW: every row has its own bias batch (pair-bias attention with a bias per sample, local
// attention windows); otherwise all rows share bias batch 0.  Queries come in p.nbq blocks of 32
// per row, keys in p.nb blocks (equal for self attention).
template <int R, int DKS, int DV, bool PERROW>
__global__ __launch_bounds__(512, (DKS == 2 ? (PERROW ? 3 : 4) : 2)) void flash_staged_kernel(FlashArgs p) {
    static_assert(DKS == 2 * DV, "head dim = 16*DKS = 32*DV");
    constexpr int A = 2 * R;                       // rows per workgroup
    constexpr int KV_UNITS = DKS * 64;             // 16-byte units of one row's K (or V) block
    constexpr int BIAS_OFF = 2 * A * KV_UNITS;     // unit offset of the bias tiles in a stage
    constexpr int BIAS_SETS = PERROW ? A : 1;      // bias tiles of the 4 query blocks, per row or shared
    constexpr int STAGE_UNITS = BIAS_OFF + BIAS_SETS * 4 * 128;
    constexpr int NLOAD = (STAGE_UNITS + 511) / 512;
    __shared__ __attribute__((aligned(16))) u32x4 stage[2][STAGE_UNITS];
    __shared__ uint8_t cls_s[A][256];              // class of each key block per row
    __shared__ int uniform_s[A];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int nb = p.nb, nbq = p.nbq, H = p.H;
    const u32x4* __restrict__ qf = static_cast<const u32x4*>(p.qf);
    const u32x4* __restrict__ kf = static_cast<const u32x4*>(p.kf);
    const u32x4* __restrict__ vf = static_cast<const u32x4*>(p.vf);
    const u32x4* __restrict__ gf = static_cast<const u32x4*>(p.gf);
    const u32x4* __restrict__ bt = static_cast<const u32x4*>(p.biast);
    u32x4* __restrict__ of = static_cast<u32x4*>(p.of);

    // chunk = (head, row set of A rows); the query groups of a chunk share an XCD
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int chunk = (slot / p.qgroups) * 8 + xcd;
    if (chunk >= p.nchunks) return;
    const int qb0 = (slot % p.qgroups) * 4;
    const int rowsets = (p.nrows + A - 1) / A;
    const int h = chunk / rowsets, a0 = (chunk % rowsets) * A;
    const int qbl = wave & 3, rg = wave >> 2;      // this wavefront: query block, row group
    const int qb = qb0 + qbl;
    const bool wave_active = qb < nbq;
    const int qbc = min(qb, nbq - 1);
    const int nr = max(0, min(R, p.nrows - (a0 + rg * R)));   // rows of this wavefront that exist

    auto rowc = [&](int ra) { return min(a0 + ra, p.nrows - 1); };                  // clamped row
    auto blk_units = [&](int a, int blk) -> size_t {          // key-side fragments (K, V)
        return (((size_t)a * H + h) * nb + blk) * KV_UNITS;
    };
    auto qblk_units = [&](int a, int blk) -> size_t {         // query-side fragments (Q, gate, output)
        return (((size_t)a * H + h) * nbq + blk) * KV_UNITS;
    };

    if (wave < A) {
        unsigned long long act_unused, full_unused;
        const bool any_valid = classify_row(p.codes + (size_t)rowc(wave) * nb * 32, nb, lane, cls_s[wave],
                                            act_unused, full_unused);
        if (lane == 0) uniform_s[wave] = any_valid ? 0 : 1;
    }

    u32x4 pre[NLOAD];
    auto prefetch = [&](int kb) {
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) {
            const int u = i * 512 + tid;
            if (u < BIAS_OFF) {
                const int region = u / KV_UNITS, off = u % KV_UNITS;      // K rows, then V rows
                const u32x4* src = region < A ? kf : vf;
                pre[i] = src[blk_units(rowc(region % A), kb) + off];
            } else if (u < STAGE_UNITS) {
                const int t = u - BIAS_OFF, set = t >> 9, q = (t >> 7) & 3, off = t & 127;
                const size_t batch = PERROW ? (size_t)rowc(set) : 0;
                pre[i] = bt[(((batch * H + h) * nbq + min(qb0 + q, nbq - 1)) * nb + kb) * 128 + off];
            }
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) {
            const int u = i * 512 + tid;
            if (u < STAGE_UNITS) stage[buf][u] = pre[i];
        }
    };

    const bf16x8 kx = slot0_frag(1.0f, half);
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    bf16x8 q[R][DKS], qx[R];
    f32x16 o[R][DV];
    float m[R], l[R];
    bool first[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int a = rowc(rg * R + r);
#pragma unroll
        for (int ks = 0; ks < DKS; ++ks) q[r][ks] = as_frag(qf[qblk_units(a, qbc) + ks * 64 + lane]);
        qx[r] = slot0_frag(0.f, half);
#pragma unroll
        for (int d = 0; d < DV; ++d) o[r][d] = zero;
        m[r] = 0.f;
        l[r] = 0.f;
        first[r] = true;
    }

    prefetch(0);
    commit(0);
    __syncthreads();
    bool uniform_row[R];
#pragma unroll
    for (int r = 0; r < R; ++r) uniform_row[r] = uniform_s[rg * R + r] != 0;

    for (int kb = 0; kb < nb; ++kb) {
        if (kb + 1 < nb) prefetch(kb + 1);
        const u32x4* st = stage[kb & 1];
        if (wave_active) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r >= nr) continue;
                const int ra = rg * R + r;
                const int bset = PERROW ? ra : 0;
                const u32x4 b0 = st[BIAS_OFF + (bset * 4 + qbl) * 128 + lane];
                const u32x4 b1 = st[BIAS_OFF + (bset * 4 + qbl) * 128 + 64 + lane];
                int cls = __builtin_amdgcn_readfirstlane((int)cls_s[ra][kb]);
                const bool uni = uniform_row[r];
                if (cls & 0x80) {                    // no valid key in this block
                    if (!uni || cls == 0x80) continue;
                    cls = 1;                         // uniform row: masked real keys take part
                }
                f32x16 s;
                auto scores = [&]() {
                    s = bias_tile_acc(b0, b1);
                    s = mfma32(kx, qx[r], s);
#pragma unroll
                    for (int ks = 0; ks < DKS; ++ks)
                        s = mfma32(as_frag(st[(ra * DKS + ks) * 64 + lane]), q[r][ks], s);
                };
                auto exact = [&](bool force, bool fresh) {
                    if (cls != 2)
                        mask_scores(s, p.codes + (size_t)(a0 + ra) * nb * 32 + kb * 32, half, uni, m[r]);
                    const float mx = tile_max(s);
                    if (force || __any(mx > kLazyMax)) rescale<DV>(s, mx, m[r], l[r], o[r], qx[r], half, fresh);
                };
                scores();
                if (first[r] || cls != 2) exact(first[r], first[r]);
                first[r] = false;
                bf16x8 p0, p1;
                float ls = exp_pack_sum(s, p0, p1);
                if (__any(!(ls < kSumLimit))) {      // a block towering over the running maximum
                    scores();
                    exact(true, false);
                    ls = exp_pack_sum(s, p0, p1);
                }
                l[r] += ls;
#pragma unroll
                for (int d = 0; d < DV; ++d) {
                    const u32x4* vt = st + A * KV_UNITS + (ra * DKS + 2 * d) * 64 + lane;
                    o[r][d] = mfma32(as_frag(vt[0]), p0, o[r][d]);
                    o[r][d] = mfma32(as_frag(vt[64]), p1, o[r][d]);
                }
            }
        }
        if (kb + 1 < nb) commit((kb + 1) & 1);
        __syncthreads();
    }

    if (!wave_active) return;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (r >= nr) continue;
        const int a = a0 + rg * R + r;
        const float inv = fast_rcp(xhalf_sum(l[r]));
#pragma unroll
        for (int d = 0; d < DV; ++d) {
            const size_t u0 = qblk_units(a, qb) + (2 * d) * 64 + lane;
            f32x16 og;
            if (p.gf != nullptr) {
                const u32x4 g0 = gf[u0], g1 = gf[u0 + 64];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    og[2 * e] = o[r][d][2 * e] * inv * bf16_lo(g0[e]);
                    og[2 * e + 1] = o[r][d][2 * e + 1] * inv * bf16_hi(g0[e]);
                    og[8 + 2 * e] = o[r][d][8 + 2 * e] * inv * bf16_lo(g1[e]);
                    og[8 + 2 * e + 1] = o[r][d][8 + 2 * e + 1] * inv * bf16_hi(g1[e]);
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v) og[v] = o[r][d][v] * inv;
            }
            bf16x8 f0, f1;
            acc_to_frags(og, f0, f1);
            of[u0] = __builtin_bit_cast(u32x4, f0);
            of[u0 + 64] = __builtin_bit_cast(u32x4, f1);
        }
    }
}

static int launch_staged(FlashArgs p, int head_dim_pad, hipStream_t stream) {
    constexpr int R = 1, A = 2 * R;
    p.qgroups = (p.nbq + 3) / 4;
    p.nchunks = p.H * ((p.nrows + A - 1) / A);
    const int nslots = ((p.nchunks + 7) / 8) * p.qgroups;
    const dim3 grid(nslots * 8), block(512);
    if (head_dim_pad == 32) {
        if (p.bias_per_row) hipLaunchKernelGGL((flash_staged_kernel<R, 2, 1, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((flash_staged_kernel<R, 2, 1, false>), grid, block, 0, stream, p);
    } else if (head_dim_pad == 64) {
        if (p.bias_per_row) hipLaunchKernelGGL((flash_staged_kernel<R, 4, 2, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((flash_staged_kernel<R, 4, 2, false>), grid, block, 0, stream, p);
    } else {
        return -1;
    }
    return 0;
}

static int launch_strip(FlashArgs p, hipStream_t stream) {
    const size_t lds_bytes = (size_t)p.nb * 4096 + kStripWaves * 64;
    // per-device launch state (a process may drive several GPUs; the writes are idempotent, so
    // concurrent first calls are harmless)
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cu_count[kMaxDevices];      // 0 = not queried yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -2;
    int n_cu = cu_count[dev].load(std::memory_order_relaxed);
    if (n_cu == 0) {
        // the strip needs more dynamic LDS than the default limit: raise it once per device
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(flash_strip_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                kStripMaxBlocks * 4096 + kStripWaves * 64) != hipSuccess)
            return -2;
        if (hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0)
            n_cu = 256;
        cu_count[dev].store(n_cu, std::memory_order_relaxed);
    }
    p.qgroups = (p.nb + 1) / 2;                                    // query-block pairs
    // rows per workgroup: a multiple of the wavefront count; one workgroup per CU is resident,
    // so pick the split whose number of full-chip rounds times rows per round is smallest
    int per = kStripWaves;
    long long best = -1;
    for (int cand = kStripWaves; cand <= kStripWaves * 8; cand += kStripWaves) {
        const long long wgs = (long long)p.H * p.qgroups * ((p.nrows + cand - 1) / cand);
        const long long cost = ((wgs + n_cu - 1) / n_cu) * cand;
        if (best < 0 || cost <= best) { best = cost; per = cand; }
    }
    p.rows_per_range = per;
    p.rowranges = (p.nrows + per - 1) / per;
    p.nchunks = p.H * p.rowranges;
    const int nslots = ((p.nchunks + 7) / 8) * p.qgroups;
    hipLaunchKernelGGL(flash_strip_kernel, dim3(nslots * 8), dim3(kStripWaves * 64), lds_bytes, stream, p);
    return 0;
}

int launch_flash(const FlashArgs& args_in, int head_dim_pad, hipStream_t stream, int full_rows) {
    FlashArgs args = args_in;
    if (args.nbq <= 0) args.nbq = args.nb;            // self attention
    if (args.nb > 256 || args.nbq > 256) return -1;
    const bool strip_shape = !args.bias_per_row && args.nbq == args.nb && head_dim_pad == 32 &&
                             args.nb <= kStripMaxBlocks;
    if (strip_shape && (full_rows > 0 ? full_rows : args.nrows) >= 4 * kStripWaves) {
        // a range of rows runs on the kernel the whole problem runs on (the two kernels visit the
        // key blocks in different orders and do not give the same bits)
        if (args.nrows < 4 * kStripWaves) return -3;
        return launch_strip(args, stream);
    }
    return launch_staged(args, head_dim_pad, stream);
}

}  // namespace kfh
