// C ABI, single (token) track: pair bias, pair-bias attention, generic transition.
#include "../../include/kfold_hip.h"

#include <atomic>
#include <cmath>

#include "api_util.hpp"
#include "kernels.hpp"

using namespace kfh;

// run a launch_* helper that reports an unsupported shape with a non-zero code
#define KFH_TRY(call, what)                                                             \
    do {                                                                                \
        const int rc_ = (call);                                                         \
        if (rc_ != 0) return fail(KFH_EUNSUPPORTED, "%s: shape not built (%d)", what, rc_); \
    } while (0)

namespace {

// ---- blob / workspace layouts -------------------------------------------------------------
// parts = 1: bf16 arithmetic; parts = 3 (KFH_ARITH_F32): every packed matrix and every bf16
// intermediate is stored as its three split3 planes, one after the other
struct ApbLayout {
    int C, H, Dh, PB, Cs, kq, nhb, ko, parts;
    size_t wq, wk, wv, wg, wo, w_adag, w_adab, w_adaout, f_bq, f_ln_g, f_ln_b, f_lns_g, f_adag_b,
        f_adaout_b, total;
    size_t wh, wo_bytes, wa;          // bytes of one part of a head projection / the output projection / an AdaLN matrix
    bool ok;
    ApbLayout(int C_, int H_, int Cs_, int arith = KFH_ARITH_BF16) : C(C_), H(H_), Cs(Cs_) {
        parts = arith == KFH_ARITH_F32 ? 3 : 1;
        ok = (arith == KFH_ARITH_BF16 || arith == KFH_ARITH_F32) && C > 0 && H > 0 && C % H == 0 && C % 128 == 0 &&
             C <= 2048 && (Cs == 0 || (Cs % 128 == 0 && Cs <= 2048));
        if (!ok) { total = 0; return; }
        Dh = C / H;
        PB = (Dh + 31) / 32;
        ok = PB <= 2;
        if (!ok) { total = 0; return; }
        kq = C / 16;
        nhb = H * PB;
        ko = nhb * 2;
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        wh = (size_t)nhb * kq * 1024;
        wq = take(parts * wh); wk = take(parts * wh); wv = take(parts * wh); wg = take(parts * wh);
        wo_bytes = (size_t)(C / 32) * ko * 1024;
        wo = take(parts * wo_bytes);
        wa = Cs ? (size_t)(C / 32) * (Cs / 16) * 1024 : 0;
        w_adag = take(parts * wa); w_adab = take(parts * wa); w_adaout = take(parts * wa);
        f_bq = take(C * 4); f_ln_g = take(C * 4); f_ln_b = take(C * 4);
        f_lns_g = take(Cs * 4); f_adag_b = take(C * 4); f_adaout_b = take(C * 4);
        total = off;
    }
};

struct ApbWs {
    size_t xn, an, sn, sraw, gate_out, qf, kf, vf, gf, of, codes, total;
    size_t rows_c, rows_cs, frag;     // bytes of one part of a [rows, C] / [rows, Cs] bf16 tensor / a fragment buffer
    int nb;
    ApbWs(const ApbLayout& l, int S, int L) {
        nb = (L + 31) / 32;
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        const size_t rows = (size_t)S * L;
        const size_t P = l.parts;
        rows_c = rows * l.C * 2;
        rows_cs = rows * l.Cs * 2;
        xn = take(P * rows_c);
        an = take(l.Cs ? P * rows_c : 0);
        sn = take(l.Cs ? P * rows_cs : 0);
        sraw = take(l.Cs ? P * rows_cs : 0);
        gate_out = take(l.Cs ? rows * l.C * (P == 3 ? 4 : 2) : 0);      // fp32 gate in fp32 arithmetic
        frag = (size_t)S * l.H * nb * l.PB * 2048;
        qf = take(P * frag); kf = take(P * frag); vf = take(P * frag); gf = take(P * frag); of = take(P * frag);
        codes = take((size_t)S * nb * 32);
        total = off;
    }
};

struct GtLayout {   // generic transition
    size_t wu, wv, wo, f_ln, total;
    int hid;
    GtLayout(int C, int E) {
        hid = C * E;
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        wu = take((size_t)(hid / 32) * (C / 16) * 1024);
        wv = take((size_t)(hid / 32) * (C / 16) * 1024);
        wo = take((size_t)(C / 32) * (hid / 16) * 1024);
        f_ln = take(2 * C * 4);
        total = off;
    }
};

LinearArgs plain(const void* A, long long lda, long long M, int K, const void* W, int Nout) {
    LinearArgs p{};
    p.A = A; p.lda = lda; p.rows_a = 1; p.L = (int)M; p.nb = (int)((M + 31) / 32); p.K = K;
    p.W = W; p.nblk = (Nout + 31) / 32; p.Nout = Nout; p.bias_scale = 1.f;
    p.H = 1; p.PB = 1; p.Dh = 32;
    return p;
}

}  // namespace

extern "C" {

// ------------------------------------------------------------------------------------------
// pair bias tiles
// ------------------------------------------------------------------------------------------
size_t kfh_bias_tiles_bytes(int nbatch, int H, int L, int arith) {
    if (nbatch <= 0 || H <= 0 || L <= 0 || (arith != KFH_ARITH_BF16 && arith != KFH_ARITH_F32)) return 0;
    const size_t nb = (L + 31) / 32;
    return align_up((size_t)nbatch * H * nb * nb * (arith == KFH_ARITH_F32 ? kBiasTileF32Bytes : 2048));
}

int kfh_bias_tiles_from_dense(const void* dense, int io_dtype, void* tiles, int nbatch, int H, int L,
                              int arith, void* stream) {
    if (!dense || !tiles || nbatch <= 0 || H <= 0 || L <= 0)
        return fail(KFH_EINVAL, "bias_tiles_from_dense: bad argument");
    if (!dtype_ok(io_dtype)) return fail(KFH_EINVAL, "bias_tiles_from_dense: bad io_dtype %d", io_dtype);
    if (arith != KFH_ARITH_BF16 && arith != KFH_ARITH_F32)
        return fail(KFH_EINVAL, "bias_tiles_from_dense: bad arith %d", arith);
    if (arith == KFH_ARITH_F32)
        launch_bias_tiles_f32(dense, io_dtype, static_cast<float*>(tiles), nbatch, H, L, (L + 31) / 32,
                              static_cast<hipStream_t>(stream));
    else
        launch_bias_tiles(dense, io_dtype, static_cast<uint16_t*>(tiles), nbatch, H, L, (L + 31) / 32,
                          static_cast<hipStream_t>(stream));
    return check_launch("bias_tiles_from_dense");
}

size_t kfh_pair_bias_packed_bytes(int C, int H) {
    return (C == kC && H >= 1 && H <= 32) ? align_up(kPbBlobBytes) : 0;
}

int kfh_pair_bias_pack(const void* ln_w, const void* ln_b, const void* w, int w_dtype, int C, int H,
                       void* blob, void* stream_) {
    if (C != kC || H < 1 || H > 32)
        return fail(KFH_EUNSUPPORTED, "pair_bias_pack: C=%d H=%d, built for C=128, H<=32", C, H);
    if (!dtype_ok(w_dtype) || !w || !blob) return fail(KFH_EINVAL, "pair_bias_pack: bad argument");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    char* b = static_cast<char*>(blob);
    launch_pack_blocks(w, w_dtype, H, C, C, 0, 1, ROW_NATURAL, K_NATURAL, kLog2e, b, stream);
    float* ln = reinterpret_cast<float*>(b + kBlockBytes);
    launch_copy_f32(ln_w, w_dtype, ln, C, 1.f, stream);
    launch_copy_f32(ln_b, w_dtype, ln + C, C, 0.f, stream);
    return check_launch("pair_bias_pack");
}

int kfh_pair_bias_project(const void* z, const void* blob, void* tiles, int B, int N, int C, int H,
                          float eps, int io_dtype, void* stream_) {
    if (C != kC || H < 1 || H > 32)
        return fail(KFH_EUNSUPPORTED, "pair_bias_project: C=%d H=%d, built for C=128, H<=32", C, H);
    if (!z || !blob || !tiles || B <= 0 || N <= 0 || !dtype_ok(io_dtype))
        return fail(KFH_EINVAL, "pair_bias_project: bad argument");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const size_t nb = (N + 31) / 32, esz = io_dtype == KFH_F32 ? 4 : 2;
    for (int b = 0; b < B; ++b) {
        uint16_t* t = static_cast<uint16_t*>(tiles) + (size_t)b * H * nb * nb * kBiasTileElems;
        if (N % 32) {   // queries beyond N in the last query block: keep their tiles finite
            for (int h = 0; h < H; ++h)
                launch_fill_zero(t + (((size_t)h * nb + (nb - 1)) * nb) * kBiasTileElems, nb * 2048, stream);
        }
        launch_pair_bias(static_cast<const char*>(z) + (size_t)b * N * N * C * esz, io_dtype,
                         static_cast<const char*>(blob), t, N, H, eps, stream);
    }
    return check_launch("pair_bias_project");
}

// ------------------------------------------------------------------------------------------
// pair-bias attention
// ------------------------------------------------------------------------------------------
size_t kfh_apb_packed_bytes(int C, int H, int Cs, int arith) { return ApbLayout(C, H, Cs, arith).total; }

int kfh_apb_pack(const void* ln_w, const void* ln_b, const void* q_w, const void* q_b, const void* k_w,
                 const void* v_w, const void* g_w, const void* o_w, const void* adaln_s_w,
                 const void* adaln_g_w, const void* adaln_g_b, const void* adaln_bias_w,
                 const void* ada_out_w, const void* ada_out_b, int w_dtype, int C, int H, int Cs,
                 int arith, void* blob, void* stream_) {
    const ApbLayout l(C, H, Cs, arith);
    if (!l.ok) return fail(KFH_EUNSUPPORTED, "apb_pack: C=%d H=%d Cs=%d arith=%d not supported (C,Cs multiples of 128 up to 2048, head dim <= 64)", C, H, Cs, arith);
    if (!dtype_ok(w_dtype)) return fail(KFH_EINVAL, "apb_pack: bad w_dtype %d", w_dtype);
    if (!q_w || !k_w || !v_w || !g_w || !o_w || !blob) return fail(KFH_EINVAL, "apb_pack: null pointer");
    if (Cs && (!adaln_g_w || !adaln_bias_w || !ada_out_w))
        return fail(KFH_EINVAL, "apb_pack: conditioned module needs the AdaLN / ada_out weights");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    char* b = static_cast<char*>(blob);
    const float qscale = kLog2e / sqrtf((float)l.Dh);
    const size_t blk = (size_t)l.kq * 1024;
    for (int q = 0; q < l.parts; ++q) {
        const int part = l.parts == 3 ? q : -1;
        for (int h = 0; h < H; ++h)
            for (int pp = 0; pp < l.PB; ++pp) {
                const int rows = l.Dh - 32 * pp < 32 ? l.Dh - 32 * pp : 32;
                const int row0 = h * l.Dh + 32 * pp;
                const size_t o = (size_t)q * l.wh + (size_t)(h * l.PB + pp) * blk;
                launch_pack_blocks(q_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, qscale, b + l.wq + o, stream, 0, part);
                launch_pack_blocks(k_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wk + o, stream, 0, part);
                launch_pack_blocks(v_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wv + o, stream, 0, part);
                launch_pack_blocks(g_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wg + o, stream, 0, part);
            }
        launch_pack_blocks(o_w, w_dtype, C, l.ko * 16, C, 0, C / 32, ROW_NATURAL, K_ACC_HEADPAD, 1.f,
                           b + l.wo + (size_t)q * l.wo_bytes, stream, l.Dh | ((2 * l.PB) << 16), part);
        if (Cs) {
            const size_t oa = (size_t)q * l.wa;
            launch_pack_blocks(adaln_g_w, w_dtype, C, Cs, Cs, 0, C / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.w_adag + oa, stream, 0, part);
            launch_pack_blocks(adaln_bias_w, w_dtype, C, Cs, Cs, 0, C / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.w_adab + oa, stream, 0, part);
            launch_pack_blocks(ada_out_w, w_dtype, C, Cs, Cs, 0, C / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.w_adaout + oa, stream, 0, part);
        }
    }
    launch_copy_f32(q_b, w_dtype, reinterpret_cast<float*>(b + l.f_bq), C, 0.f, stream);
    launch_copy_f32(ln_w, w_dtype, reinterpret_cast<float*>(b + l.f_ln_g), C, 1.f, stream);
    launch_copy_f32(ln_b, w_dtype, reinterpret_cast<float*>(b + l.f_ln_b), C, 0.f, stream);
    if (Cs) {
        launch_copy_f32(adaln_s_w, w_dtype, reinterpret_cast<float*>(b + l.f_lns_g), Cs, 1.f, stream);
        launch_copy_f32(adaln_g_b, w_dtype, reinterpret_cast<float*>(b + l.f_adag_b), C, 0.f, stream);
        launch_copy_f32(ada_out_b, w_dtype, reinterpret_cast<float*>(b + l.f_adaout_b), C, 0.f, stream);
    }
    return check_launch("apb_pack");
}

size_t kfh_apb_workspace_bytes(int S, int L, int C, int H, int Cs, int arith) {
    const ApbLayout l(C, H, Cs, arith);
    if (!l.ok || S <= 0 || L <= 0 || L > 8192) return 0;
    return ApbWs(l, S, L).total;
}

int kfh_apb_forward(const void* a, const void* s_cond, const void* bias_tiles, const uint8_t* mask,
                    const void* blob, const void* residual, void* out, void* workspace,
                    size_t workspace_bytes, int S, int L, int C, int H, int Cs, int apply_norm,
                    int bias_per_sample, int mask_per_sample, int s_per_sample, float eps,
                    int io_dtype, int arith, void* stream_) {
    const ApbLayout l(C, H, Cs, arith);
    if (!l.ok) return fail(KFH_EUNSUPPORTED, "apb_forward: C=%d H=%d Cs=%d arith=%d not supported", C, H, Cs, arith);
    if (S <= 0 || L <= 0) return fail(KFH_EINVAL, "apb_forward: bad shape S=%d L=%d", S, L);
    if (L > 8192) return fail(KFH_EUNSUPPORTED, "apb_forward: L=%d > 8192", L);
    if (!dtype_ok(io_dtype)) return fail(KFH_EINVAL, "apb_forward: bad io_dtype %d", io_dtype);
    if (!a || !bias_tiles || !mask || !blob || !out || !workspace)
        return fail(KFH_EINVAL, "apb_forward: null pointer argument");
    const bool cond = Cs > 0 && apply_norm;
    if (cond && !s_cond) return fail(KFH_EINVAL, "apb_forward: conditioned module needs s_cond");
    const ApbWs w(l, S, L);
    if (workspace_bytes < w.total)
        return fail(KFH_EINVAL, "apb_forward: workspace %zu < %zu bytes", workspace_bytes, w.total);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* b = static_cast<const char*>(blob);
    char* ws = static_cast<char*>(workspace);
    const long long rows = (long long)S * L;
    auto f32p = [&](size_t off) { return reinterpret_cast<const float*>(b + off); };
    uint16_t* xn = reinterpret_cast<uint16_t*>(ws + w.xn);

    const int P = l.parts;
    // with P = 3 a [rows, C] bf16 tensor is three planes `rows * C * 2` bytes apart (split3)
    auto plane = [&](long long r, int ch) { return P == 3 ? (size_t)r * ch * 2 : (size_t)0; };

    // 1. normalised input rows (bf16, or split fp32)
    if (!apply_norm) {
        KFH_TRY(launch_rows_norm(a, io_dtype, nullptr, nullptr, xn, rows, C, 0, eps, stream, 0, P), "rows_norm");
    } else if (!Cs) {
        KFH_TRY(launch_rows_norm(a, io_dtype, f32p(l.f_ln_g), f32p(l.f_ln_b), xn, rows, C, 1, eps, stream, 0, P), "rows_norm");
    } else {
        // AdaLN: sigmoid(W_g LN_s(s) + b_g) * LN(a) + W_b LN_s(s)
        const long long srows = s_per_sample ? rows : L;
        uint16_t* an = reinterpret_cast<uint16_t*>(ws + w.an);
        uint16_t* sn = reinterpret_cast<uint16_t*>(ws + w.sn);
        uint16_t* sraw = reinterpret_cast<uint16_t*>(ws + w.sraw);
        KFH_TRY(launch_rows_norm(a, io_dtype, nullptr, nullptr, an, rows, C, 1, eps, stream, 0, P), "rows_norm");
        KFH_TRY(launch_rows_norm(s_cond, io_dtype, f32p(l.f_lns_g), nullptr, sn, srows, Cs, 1, eps, stream, 0, P), "rows_norm");
        KFH_TRY(launch_rows_norm(s_cond, io_dtype, nullptr, nullptr, sraw, srows, Cs, 0, eps, stream, 0, P), "rows_norm");
        LinearArgs p = plain(sn, Cs, L, Cs, b + l.w_adag, C);
        p.rows_a = S; p.a_shared = !s_per_sample;
        p.W2 = b + l.w_adab; p.bias = f32p(l.f_adag_b);
        p.aux = an; p.aux_dtype = KFH_BF16; p.ld_aux = C;
        p.out = xn; p.out_dtype = KFH_BF16; p.ldo = C; p.epi = EPI_ADALN;
        p.parts = P; p.a_part = plane(srows, Cs); p.w_part = l.wa; p.aux_part = plane(rows, C); p.out_part = plane(rows, C);
        KFH_TRY(launch_linear(p, stream), "linear");
        // output gate sigmoid(W_ada s + b_ada) on the raw conditioning (kept in fp32 in fp32 arithmetic)
        LinearArgs g = plain(sraw, Cs, srows, Cs, b + l.w_adaout, C);
        g.bias = f32p(l.f_adaout_b);
        g.out = ws + w.gate_out; g.out_dtype = P == 3 ? KFH_F32 : KFH_BF16; g.ldo = C; g.epi = EPI_SIGMOID;
        g.parts = P; g.a_part = plane(srows, Cs); g.w_part = l.wa;
        KFH_TRY(launch_linear(g, stream), "linear");
    }

    // 2. q (with bias, pre-scaled), k, gate, v projections into fragment order
    {
        LinearArgs p = plain(xn, C, L, C, nullptr, C);
        p.rows_a = S; p.nblk = l.nhb; p.H = H; p.PB = l.PB; p.Dh = l.Dh;
        p.parts = P; p.a_part = plane(rows, C); p.w_part = l.wh; p.out_part = w.frag;
        p.epi = EPI_FRAG_CH;
        p.W = b + l.wq; p.bias = f32p(l.f_bq); p.bias_scale = kLog2e / sqrtf((float)l.Dh);
        p.out = ws + w.qf;
        KFH_TRY(launch_linear(p, stream), "linear");
        p.bias = nullptr;
        p.W = b + l.wk; p.out = ws + w.kf;
        KFH_TRY(launch_linear(p, stream), "linear");
        p.W = b + l.wg; p.out = ws + w.gf; p.sigmoid = 1;
        KFH_TRY(launch_linear(p, stream), "linear");
        p.sigmoid = 0; p.epi = EPI_FRAG_POS;
        p.W = b + l.wv; p.out = ws + w.vf;
        KFH_TRY(launch_linear(p, stream), "linear");
    }

    // 3. key codes, attention
    uint8_t* codes = reinterpret_cast<uint8_t*>(ws + w.codes);
    launch_key_codes(mask, codes, S, L, w.nb * 32, mask_per_sample ? L : 0, stream);
    FlashArgs fa{};
    fa.qf = ws + w.qf; fa.kf = ws + w.kf; fa.vf = ws + w.vf; fa.gf = ws + w.gf; fa.of = ws + w.of;
    fa.biast = bias_tiles; fa.codes = codes;
    fa.nrows = S; fa.nb = w.nb; fa.H = H; fa.bias_per_row = bias_per_sample ? 1 : 0;
    if (P == 3) {
        fa.q_part = fa.k_part = fa.v_part = fa.g_part = fa.o_part = w.frag;
        if (launch_flash_split(fa, 32 * l.PB, stream) != 0) return fail(KFH_EUNSUPPORTED, "apb_forward: attention shape");
    } else if (launch_flash(fa, 32 * l.PB, stream) != 0) {
        return fail(KFH_EUNSUPPORTED, "apb_forward: attention shape");
    }

    // 4. output projection (+ conditioning gate, + residual)
    {
        LinearArgs p{};
        p.A = ws + w.of; p.a_frag = 1; p.rows_a = S; p.L = L; p.nb = w.nb; p.K = l.ko * 16;
        p.W = b + l.wo; p.nblk = C / 32; p.Nout = C; p.bias_scale = 1.f;
        p.H = H; p.PB = l.PB; p.Dh = l.Dh;
        p.parts = P; p.a_part = w.frag; p.w_part = l.wo_bytes;
        p.epi = EPI_RESID;
        if (cond) {
            p.gate = reinterpret_cast<const uint16_t*>(ws + w.gate_out); p.ld_gate = C; p.gate_shared = !s_per_sample;
            p.gate_dtype = P == 3 ? KFH_F32 : KFH_BF16;
        }
        if (residual) { p.aux = residual; p.aux_dtype = io_dtype; p.ld_aux = C; }
        p.out = out; p.out_dtype = io_dtype; p.ldo = C;
        KFH_TRY(launch_linear(p, stream), "linear");
    }
    return check_launch("apb_forward");
}

// ------------------------------------------------------------------------------------------
// transition for any channel count (token track); C = 128 uses the fused pair kernel
// ------------------------------------------------------------------------------------------
size_t kfh_transition_packed_bytes(int C, int expansion) {
    if (transition_fused(C, expansion)) return align_up(transition_blob_bytes(expansion, C));
    if (C <= 0 || C % 32 || C > 2048 || expansion < 1 || expansion > 8) return 0;
    return GtLayout(C, expansion).total;
}

int kfh_transition_pack(const void* ln_w, const void* ln_b, const void* swiglu_w, const void* out_w,
                        int w_dtype, int C, int expansion, void* blob, void* stream_) {
    if (kfh_transition_packed_bytes(C, expansion) == 0)
        return fail(KFH_EUNSUPPORTED, "transition_pack: C=%d E=%d not supported", C, expansion);
    if (!dtype_ok(w_dtype)) return fail(KFH_EINVAL, "transition_pack: bad w_dtype %d", w_dtype);
    if (!swiglu_w || !out_w || !blob) return fail(KFH_EINVAL, "transition_pack: null pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    char* b = static_cast<char*>(blob);
    const int hid = C * expansion;
    const size_t wsz = w_dtype == KFH_F32 ? 4 : 2;
    if (transition_fused(C, expansion)) {
        const int nstep = hid / 32;
        const size_t blk = (size_t)32 * C * 2;          // one 32-row block of C channels
        for (int s = 0; s < nstep; ++s) {
            char* step = b + (size_t)s * 3 * blk;
            // u rows are packed times -log2(e) and W_out times -ln(2): the kernel then needs
            // u' v / (1 + exp2(u')) with u' = -log2(e) u, one multiply less per element
            launch_pack_blocks(swiglu_w, w_dtype, 32, C, C, 32 * s, 1, ROW_NATURAL, K_NATURAL, -kLog2e, step, stream);
            launch_pack_blocks(swiglu_w, w_dtype, 32, C, C, hid + 32 * s, 1, ROW_NATURAL, K_NATURAL, 1.f,
                               step + blk, stream);
            // W_out[:, 32s .. 32s+31]: a 32-wide column slice of the [C, hid] matrix
            launch_pack_blocks(static_cast<const char*>(out_w) + (size_t)32 * s * wsz, w_dtype, C, 32, hid,
                               0, C / 32, ROW_INTERLEAVE4, K_ACC, -1.0f / kLog2e, step + 2 * blk, stream);
        }
        float* ln = reinterpret_cast<float*>(b + (size_t)nstep * 3 * blk);
        launch_copy_f32(ln_w, w_dtype, ln, C, 1.f, stream);
        launch_copy_f32(ln_b, w_dtype, ln + C, C, 0.f, stream);
    } else {
        const GtLayout l(C, expansion);
        launch_pack_blocks(swiglu_w, w_dtype, hid, C, C, 0, hid / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.wu, stream);
        launch_pack_blocks(swiglu_w, w_dtype, hid, C, C, hid, hid / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.wv, stream);
        launch_pack_blocks(out_w, w_dtype, C, hid, hid, 0, C / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.wo, stream);
        float* ln = reinterpret_cast<float*>(b + l.f_ln);
        launch_copy_f32(ln_w, w_dtype, ln, C, 1.f, stream);
        launch_copy_f32(ln_b, w_dtype, ln + C, C, 0.f, stream);
    }
    return check_launch("transition_pack");
}

size_t kfh_transition_workspace_bytes(long long rows, int C, int expansion) {
    if (transition_fused(C, expansion)) return 0;
    if (rows <= 0 || kfh_transition_packed_bytes(C, expansion) == 0) return 0;
    return align_up((size_t)rows * C * 2) + align_up((size_t)rows * C * expansion * 2);
}

}  // extern "C"

namespace {
int transition_forward_impl(const void* x, const void* blob, const void* residual, const uint8_t* mask,
                            void* out, void* workspace, size_t workspace_bytes, long long rows, int C,
                            int expansion, float eps, int io_dtype, void* stream_) {
    if (kfh_transition_packed_bytes(C, expansion) == 0)
        return fail(KFH_EUNSUPPORTED, "transition_forward: C=%d E=%d not supported", C, expansion);
    if (rows < 0) return fail(KFH_EINVAL, "transition_forward: rows=%lld", rows);
    if (!dtype_ok(io_dtype)) return fail(KFH_EINVAL, "transition_forward: bad io_dtype %d", io_dtype);
    if (!x || !blob || !out) return fail(KFH_EINVAL, "transition_forward: null pointer argument");
    if (rows == 0) return KFH_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* b = static_cast<const char*>(blob);
    if (transition_fused(C, expansion)) {
        KFH_TRY(C == kC ? launch_pair_transition(x, io_dtype, b, expansion, residual, mask, out, rows, eps, stream)
                        : launch_pair_transition_wide(x, io_dtype, b, expansion, residual, mask, out, rows, eps, stream, C),
                "pair transition");
        return check_launch("transition_forward");
    }
    if (rows > 0x7fffffffLL) return fail(KFH_EUNSUPPORTED, "transition_forward: too many rows");
    const size_t need = kfh_transition_workspace_bytes(rows, C, expansion);
    if (!workspace || workspace_bytes < need)
        return fail(KFH_EINVAL, "transition_forward: workspace %zu < %zu bytes", workspace_bytes, need);
    const GtLayout l(C, expansion);
    char* ws = static_cast<char*>(workspace);
    uint16_t* xn = reinterpret_cast<uint16_t*>(ws);
    uint16_t* hid = reinterpret_cast<uint16_t*>(ws + align_up((size_t)rows * C * 2));
    const float* ln = reinterpret_cast<const float*>(b + l.f_ln);
    KFH_TRY(launch_rows_norm(x, io_dtype, ln, ln + C, xn, rows, C, 1, eps, stream), "rows_norm");
    LinearArgs p = plain(xn, C, rows, C, b + l.wu, l.hid);
    p.W2 = b + l.wv; p.out = hid; p.out_dtype = KFH_BF16; p.ldo = l.hid; p.epi = EPI_SWIGLU;
    KFH_TRY(launch_linear(p, stream), "linear");
    LinearArgs q = plain(hid, l.hid, rows, l.hid, b + l.wo, C);
    q.epi = EPI_RESID;
    if (residual) { q.aux = residual; q.aux_dtype = io_dtype; q.ld_aux = C; }
    q.mask = mask;
    q.out = out; q.out_dtype = io_dtype; q.ldo = C;
    KFH_TRY(launch_linear(q, stream), "linear");
    return check_launch("transition_forward");
}

// ---- static scratch of kfh_transition_forward_static ---------------------------------------
// Device memory beyond inputs and outputs for callers that cannot allocate: the LayerNorm-ed
// rows and the SwiGLU hidden activations of the token-track transition.  Each GPU the library
// runs on holds its own copy of the array until the process ends.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device, looked up once per device.  (In host code
// the array's name is only a handle for this lookup, never a device address.)
int static_scratch_ptr(void** ptr) {
    constexpr int kMaxDevices = 64;
    static std::atomic<void*> table[kMaxDevices];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(KFH_EHIP, "transition_forward_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(KFH_EUNSUPPORTED, "transition_forward_static: device %d", dev);
    void* p = table[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(KFH_EHIP, "transition_forward_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        table[dev].store(p, std::memory_order_release);     // same value from every thread
    }
    *ptr = p;
    return KFH_OK;
}
}  // namespace

extern "C" {

int kfh_transition_forward(const void* x, const void* blob, const void* residual, const uint8_t* mask,
                           void* out, void* workspace, size_t workspace_bytes, long long rows, int C,
                           int expansion, float eps, int io_dtype, void* stream) {
    return transition_forward_impl(x, blob, residual, mask, out, workspace, workspace_bytes, rows, C,
                                   expansion, eps, io_dtype, stream);
}

// Also the set-up call: it looks up (and keeps) the scratch array's address on the current device, so
// that a later kfh_transition_forward_static on this device does no symbol lookup — callers that
// capture a graph or run a tight loop call this once per device beforehand.  The size is returned
// whether or not a device is present.
size_t kfh_transition_static_scratch_bytes(void) {
    void* p = nullptr;
    (void)static_scratch_ptr(&p);
    return kStaticScratchBytes;
}

int kfh_transition_forward_static(const void* x, const void* blob, const void* residual,
                                  const uint8_t* mask, void* out, long long rows, int C, int expansion,
                                  float eps, int io_dtype, void* stream) {
    if (kfh_transition_packed_bytes(C, expansion) == 0)
        return fail(KFH_EUNSUPPORTED, "transition_forward_static: C=%d E=%d not supported", C, expansion);
    if (rows < 0) return fail(KFH_EINVAL, "transition_forward_static: rows=%lld", rows);
    const size_t need = kfh_transition_workspace_bytes(rows, C, expansion);
    if (need > kStaticScratchBytes)
        return fail(KFH_EINVAL,
                    "transition_forward_static: rows=%lld C=%d E=%d needs %zu bytes of scratch, the static "
                    "buffer holds %zu (use kfh_transition_forward with a workspace)",
                    rows, C, expansion, need, kStaticScratchBytes);
    void* ws = nullptr;
    if (need) {                      // the fused C = 128 kernel keeps everything in registers
        const int rc = static_scratch_ptr(&ws);
        if (rc) return rc;
    }
    return transition_forward_impl(x, blob, residual, mask, out, ws, need, rows, C, expansion, eps,
                                   io_dtype, stream);
}

size_t kfh_single_track_workspace_bytes(int B, int N, int Cz, int Cs, int H, int expansion) {
    const size_t tiles = kfh_bias_tiles_bytes(B, H, N, KFH_ARITH_BF16);
    const size_t att = kfh_apb_workspace_bytes(B, N, Cs, H, 0, KFH_ARITH_BF16);
    if (Cz != kC || tiles == 0 || att == 0 || kfh_transition_packed_bytes(Cs, expansion) == 0) return 0;
    const size_t tr = kfh_transition_workspace_bytes((long long)B * N, Cs, expansion);
    return tiles + (att > tr ? att : tr);
}

int kfh_single_track_forward(const void* z, void* s, const uint8_t* token_mask, const void* pair_bias_blob,
                             const void* apb_blob, const void* transition_blob, void* workspace,
                             size_t workspace_bytes, int B, int N, int Cz, int Cs, int H, int expansion,
                             float eps, int io_dtype, void* stream) {
    if (B <= 0 || N <= 0) return fail(KFH_EINVAL, "single_track_forward: bad shape B=%d N=%d", B, N);
    const size_t need = kfh_single_track_workspace_bytes(B, N, Cz, Cs, H, expansion);
    if (need == 0)
        return fail(KFH_EUNSUPPORTED, "single_track_forward: Cz=%d Cs=%d H=%d expansion=%d N=%d not supported", Cz, Cs,
                    H, expansion, N);
    if (!z || !s || !token_mask || !pair_bias_blob || !apb_blob || !transition_blob || !workspace)
        return fail(KFH_EINVAL, "single_track_forward: null pointer argument");
    if (workspace_bytes < need)
        return fail(KFH_EINVAL, "single_track_forward: workspace %zu < %zu bytes", workspace_bytes, need);
    char* ws = static_cast<char*>(workspace);
    const size_t tiles = kfh_bias_tiles_bytes(B, H, N, KFH_ARITH_BF16);
    // pair bias of every batch element from z, attention with it (s += ...), transition (s += ...)
    int rc = kfh_pair_bias_project(z, pair_bias_blob, ws, B, N, Cz, H, eps, io_dtype, stream);
    if (rc) return rc;
    rc = kfh_apb_forward(s, nullptr, ws, token_mask, apb_blob, s, s, ws + tiles, workspace_bytes - tiles, B, N, Cs, H, 0,
                         1, B > 1, B > 1, 0, eps, io_dtype, KFH_ARITH_BF16, stream);
    if (rc) return rc;
    return kfh_transition_forward(s, transition_blob, s, nullptr, s, ws + tiles, workspace_bytes - tiles,
                                  (long long)B * N, Cs, expansion, eps, io_dtype, stream);
}

}  // extern "C"
